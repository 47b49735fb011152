"""CPU oracle for packed variable-length attention.  TEST INFRASTRUCTURE ONLY.

Only ``tests/`` and ``__graft_entry__.smoke()`` may import this module; nothing in
the shipped package does.

What it restates: the call the reference makes for packed micro-batches,
``flash_attn_varlen_func(q, k, v, cu_seqlens_q=cu, cu_seqlens_k=cu, max_seqlen_q,
max_seqlen_k, dropout_p, softmax_scale, causal)`` (reference
``gpu_process_worker.py:265-276``), after the wrapper has derived ``cu_seqlens``
from the resets of ``position_ids`` (``gpu_process_worker.py:239-252``) and repeated
the K/V heads for grouped-query attention (``gpu_process_worker.py:154-161, 209-214``:
``x.unsqueeze(3).expand(B, L, H, repeats, D).reshape(B, L, H * repeats, D)``, i.e.
query head ``j`` reads K/V head ``j // repeats``).

The arithmetic itself lives in flash-attn 2.7.4.post1 (``requirements_fsdp.txt:11``),
which is not under the reference tree and is not installed here.  Its published
algorithm (Dao, "FlashAttention-2", 2023) computes, per segment and head,
``softmax(scale * Q K^T + mask) V`` with ``scale = D ** -0.5`` by default and, for
``causal=True`` with equal query and key lengths, the lower-triangular mask; the
tiling and online softmax change the rounding, not the function.  The reference
holds no tests or golden vectors for this call -> **parity unpinned by the
reference**; the restatement below is pinned independently of its own formula by
``tests/test_attn_oracle_pins.py``:

* ``varlen_attention``  pinned (``torch.nn.functional.scaled_dot_product_attention``
                        per segment in fp64; one-token segment -> V itself; equal
                        keys -> running mean of V; explicit K/V head repeat as in
                        the reference wrapper; segments do not see each other;
                        gradients by ``torch.autograd.gradcheck`` and against SDPA's
                        autograd)
* ``segment_bounds``    pinned (brute force over tokens)
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch


def segment_bounds(cu_seqlens: torch.Tensor, total: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """For every packed token t: first token of its segment and one past its last token.
    ``cu_seqlens`` is the int32 ``[n+1]`` vector of reference ``gpu_process_worker.py:239-252``."""
    cu = cu_seqlens.to(torch.int64).cpu()
    start = torch.zeros(total, dtype=torch.int64)
    end = torch.zeros(total, dtype=torch.int64)
    for i in range(cu.numel() - 1):
        a, b = int(cu[i]), int(cu[i + 1])
        start[a:b] = a
        end[a:b] = b
    return start, end


def varlen_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens: torch.Tensor,
                     softmax_scale: Optional[float] = None, causal: bool = True,
                     return_lse: bool = False):
    """``q`` [T, Hq, D], ``k``/``v`` [T, Hkv, D] (packed tokens), math in the dtype of the inputs
    (use fp32/fp64 tensors).  Returns ``out`` [T, Hq, D] (and ``lse`` [Hq, T], natural log of the
    softmax denominator of ``scale * q k^T``).  Differentiable: autograd of this function is the
    gradient oracle.  Follows the call at reference ``gpu_process_worker.py:265-276``."""
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    assert Hq % Hkv == 0
    rep = Hq // Hkv
    scale = float(D) ** -0.5 if softmax_scale is None else float(softmax_scale)
    cu = [int(x) for x in cu_seqlens.cpu().tolist()]
    assert cu[0] == 0 and cu[-1] == T, "cu_seqlens must cover the packed tokens exactly"
    lse = torch.full((Hq, T), float("-inf"), dtype=q.dtype)
    outs = []
    for i in range(len(cu) - 1):
        a, b = cu[i], cu[i + 1]
        n = b - a
        if n == 0:
            continue
        qs = q[a:b].transpose(0, 1)                                  # [Hq, n, D]
        ks = k[a:b].transpose(0, 1).repeat_interleave(rep, dim=0)    # head j -> K/V head j // rep
        vs = v[a:b].transpose(0, 1).repeat_interleave(rep, dim=0)
        s = torch.matmul(qs, ks.transpose(1, 2)) * scale             # [Hq, n, n]
        if causal:
            keep = torch.ones(n, n, dtype=torch.bool).tril()
            s = s.masked_fill(~keep, float("-inf"))
        l = torch.logsumexp(s, dim=-1)                               # [Hq, n]
        p = torch.exp(s - l.unsqueeze(-1))
        outs.append(torch.matmul(p, vs).transpose(0, 1))             # [n, Hq, D]
        lse[:, a:b] = l.detach()
    out = torch.cat(outs, dim=0) if outs else torch.zeros_like(q)
    return (out, lse) if return_lse else out
