"""Pins the attention oracle (oracle/attn_oracle.py) independently of its own formula: torch's
scaled_dot_product_attention per segment (a library routine), closed forms, the reference wrapper's explicit
K/V head repeat (reference gpu_process_worker.py:154-161), segment independence and gradients."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import attn_oracle as A


def _rand(T, Hq, Hkv, D, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(T, Hq, D, generator=g, dtype=dtype)
    k = torch.randn(T, Hkv, D, generator=g, dtype=dtype)
    v = torch.randn(T, Hkv, D, generator=g, dtype=dtype)
    return q, k, v


def _sdpa(q, k, v, cu, causal, scale=None):
    """Library routine, one segment at a time, with the K/V heads repeated the way the reference wrapper does."""
    rep = q.shape[1] // k.shape[1]
    outs = []
    for a, b in zip(cu[:-1].tolist(), cu[1:].tolist()):
        def rk(x):
            x = x[a:b].unsqueeze(0)                                    # [1, n, Hkv, D]
            B, L, H, D = x.shape
            x = x.unsqueeze(3).expand(B, L, H, rep, D).reshape(B, L, H * rep, D)
            return x.transpose(1, 2)                                   # [1, Hq, n, D]
        o = F.scaled_dot_product_attention(q[a:b].unsqueeze(0).transpose(1, 2), rk(k), rk(v), is_causal=causal, scale=scale)
        outs.append(o.transpose(1, 2)[0])
    return torch.cat(outs, 0)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("heads", [(4, 4), (6, 2), (8, 1)])
def test_matches_sdpa_per_segment(causal, heads):
    Hq, Hkv = heads
    cu = torch.tensor([0, 5, 6, 23, 40], dtype=torch.int32)
    q, k, v = _rand(40, Hq, Hkv, 16, seed=1)
    out = A.varlen_attention(q, k, v, cu, causal=causal)
    ref = _sdpa(q, k, v, cu, causal)
    assert torch.allclose(out, ref, atol=1e-12, rtol=1e-10)
    out2 = A.varlen_attention(q, k, v, cu, softmax_scale=0.37, causal=causal)
    assert torch.allclose(out2, _sdpa(q, k, v, cu, causal, scale=0.37), atol=1e-12, rtol=1e-10)
    assert not torch.allclose(out, out2)


def test_closed_forms():
    q, k, v = _rand(12, 2, 2, 8, seed=2)
    # one-token segments: every token attends to itself only -> out = v
    cu1 = torch.arange(13, dtype=torch.int32)
    assert torch.allclose(A.varlen_attention(q, k, v, cu1, causal=True), v, atol=1e-14)
    assert torch.allclose(A.varlen_attention(q, k, v, cu1, causal=False), v, atol=1e-14)
    # equal keys: uniform weights -> causal running mean / segment mean of v
    cu = torch.tensor([0, 5, 12], dtype=torch.int32)
    k0 = torch.zeros_like(k)
    out, lse = A.varlen_attention(q, k0, v, cu, causal=True, return_lse=True)
    for a, b in ((0, 5), (5, 12)):
        run = torch.cumsum(v[a:b], 0) / torch.arange(1, b - a + 1, dtype=v.dtype).view(-1, 1, 1)
        assert torch.allclose(out[a:b], run, atol=1e-13)
        assert torch.allclose(lse[:, a:b], torch.log(torch.arange(1, b - a + 1, dtype=v.dtype)).expand(2, -1), atol=1e-13)
    outn = A.varlen_attention(q, k0, v, cu, causal=False)
    assert torch.allclose(outn[0:5], v[0:5].mean(0, keepdim=True).expand(5, -1, -1), atol=1e-13)


def test_segments_do_not_see_each_other():
    cu = torch.tensor([0, 7, 19], dtype=torch.int32)
    q, k, v = _rand(19, 4, 2, 8, seed=3)
    base = A.varlen_attention(q, k, v, cu, causal=False)
    k2, v2 = k.clone(), v.clone()
    k2[7:] += 3.0
    v2[7:] -= 2.0
    pert = A.varlen_attention(q, k2, v2, cu, causal=False)
    assert torch.equal(base[:7], pert[:7]) and not torch.allclose(base[7:], pert[7:])
    # causal: a token does not see later tokens of its own segment
    k3, v3 = k.clone(), v.clone()
    k3[5] += 1.0
    v3[5] += 1.0
    c0 = A.varlen_attention(q, k, v, cu, causal=True)
    c1 = A.varlen_attention(q, k3, v3, cu, causal=True)
    assert torch.equal(c0[:5], c1[:5]) and not torch.allclose(c0[5:7], c1[5:7]) and torch.equal(c0[7:], c1[7:])


def test_lse_is_the_log_denominator():
    cu = torch.tensor([0, 4, 9], dtype=torch.int32)
    q, k, v = _rand(9, 2, 1, 4, seed=4)
    _, lse = A.varlen_attention(q, k, v, cu, causal=True, return_lse=True)
    # brute force for token 6 (segment [4, 9), sees keys 4..6), head 1
    s = torch.stack([(q[6, 1] * k[j, 0]).sum() * 4 ** -0.5 for j in (4, 5, 6)])
    assert math.isclose(float(lse[1, 6]), float(torch.log(torch.exp(s).sum())), rel_tol=1e-12)


def test_gradients():
    cu = torch.tensor([0, 3, 8], dtype=torch.int32)
    q, k, v = _rand(8, 4, 2, 4, seed=5)
    q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
    assert torch.autograd.gradcheck(lambda a, b, c: A.varlen_attention(a, b, c, cu, causal=True), (q, k, v), atol=1e-7)
    w = torch.randn(8, 4, 4, dtype=torch.float64, generator=torch.Generator().manual_seed(6))
    g1 = torch.autograd.grad((A.varlen_attention(q, k, v, cu, causal=True) * w).sum(), (q, k, v))
    g2 = torch.autograd.grad((_sdpa(q, k, v, cu, True) * w).sum(), (q, k, v))
    for a, b in zip(g1, g2):
        assert torch.allclose(a, b, atol=1e-12, rtol=1e-10)


def test_segment_bounds_brute_force():
    cu = torch.tensor([0, 3, 3, 8, 9], dtype=torch.int32)
    s, e = A.segment_bounds(cu, 9)
    want_s = [0, 0, 0, 3, 3, 3, 3, 3, 8]
    want_e = [3, 3, 3, 8, 8, 8, 8, 8, 9]
    assert s.tolist() == want_s and e.tolist() == want_e
