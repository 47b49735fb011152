"""The training step walked in token chunks inside the forward call (``fgrpo_grpo_step_chunked``): forward with kept
soft-max numerators on one chunk, the objective on that chunk, its rows of dH and its share of dW, then the next
chunk - what the reference's chunk loop is for (grpo_loss.py:280-316), with gradients instead of a retained graph.

Checked against the CPU oracle at sizes it finishes in seconds, against the other two ways to the same gradients
(whole-batch kept numerators, recomputation), for invariance under the chunk size, for the bound on transient
memory, and for being capturable in a HIP graph (no host synchronisation anywhere)."""
import pytest
import torch

from test_gpu_kept_logits import filling_workload
from test_gpu_parity import check, run_case

pytestmark = pytest.mark.gpu


def cos(a, b):
    """Cosine in float64 (a float32 sum over millions of like-signed products is itself only good to 1e-4)."""
    a, b = a.detach().double().flatten(), b.detach().double().flatten()
    return float((a @ b) / (a.norm() * b.norm()))


@pytest.mark.parametrize("mode", ["reference", "north_star"])
@pytest.mark.parametrize("chunk", [1024, 2560, 8192])
def test_chunked_step_against_oracle(dev, mode, chunk):
    """8155 tokens under a chunk bound of 2 * loss_chunksize: four chunks of 2048 (the last one ragged), two of 4096
    (dealt evenly under the bound of 5120), or a single chunk."""
    from fgrpo import ops
    w = filling_workload(31)
    assert ops.chunked_supported(w.T, w.H, w.V, torch.bfloat16, 2 * chunk)
    want, got, o, g, _, _ = run_case(w, dev, mode, chunk=chunk, keep_logits="chunked")
    check(want, got, o, g, f32=False)


def test_chunked_step_with_bias_temperature_and_compaction(dev):
    from fgrpo import ops
    w = filling_workload(32)
    bias = (torch.randn(w.V, generator=torch.Generator().manual_seed(9)) * 0.3).to(w.dtype)
    want, got, o, g, _, _ = run_case(w, dev, "north_star", temperature=0.7, bias=bias, chunk=1024, keep_logits="chunked")
    check(want, got, o, g, f32=False)
    # prompts make up a third of the batch: the projection runs on the scored rows only
    w = filling_workload(33)
    lab = w.labels.clone()
    cu = w.cu_seqlens.tolist()
    for a, b in zip(cu[:-1], cu[1:]):
        lab[0, a:a + (b - a) // 3] = -100
    w.labels = lab
    want, got, o, g, _, _ = run_case(w, dev, "north_star", chunk=1024, keep_logits="chunked", compact_masked_tokens=True)
    check(want, got, o, g, f32=False)


def _step(w, dev, keep_logits, chunk_tokens=0, scale=1.0, mode="north_star", seed=3):
    from fgrpo import ops
    hs = w.hidden.reshape(w.T, w.H).to(dev).clone().requires_grad_(True)
    W = w.weight.to(dev).clone().requires_grad_(True)
    y = ops.shift_labels(w.labels.to(dev)).reshape(-1)
    gen = torch.Generator().manual_seed(seed)
    adv = torch.randn(w.T, generator=gen).to(dev)
    with torch.no_grad():
        lp0 = ops.lmhead_logprob_fwd(hs.detach(), W.detach(), None, y)[0]
    old = lp0 + 0.05 * torch.randn(w.T, generator=gen).to(dev)
    ref = lp0 + 0.1 * torch.randn(w.T, generator=gen).to(dev)
    kw = dict(ref_lp=ref, kl_beta=0.02, loss_agg_mode="sample_mean", cu_seqlens=w.cu_seqlens.to(dev)) if mode == "north_star" else {}
    out = ops.fused_grpo_loss(hs, W, None, y, old, adv, clip_low=0.2, clip_high=0.28, clip_ratio_c=3.0,
                              keep_logits=keep_logits, chunk_tokens=chunk_tokens, **kw)
    (out[0] * scale).backward()
    torch.cuda.synchronize()
    return out, hs.grad, W.grad


@pytest.mark.parametrize("mode", ["reference", "north_star"])
def test_results_do_not_depend_on_the_chunk(dev, mode):
    """Loss, logprobs, entropy and the diagnostics agree with the whole-batch paths' to fp32 rounding for every
    chunk size (the vocabulary splits of the forward, hence the order in which a token's partial sums are merged,
    follow the token count of a launch; the normalisers are the same numbers, formed from the labels); dH and dW
    agree to bf16 rounding with the whole-batch kept path and the recomputing one; an upstream scale other than 1
    multiplies the gradients."""
    w = filling_workload(34, tokens=8192 + 300)
    ref_out, ref_dh, ref_dw = _step(w, dev, "whole", mode=mode)
    rec_out, rec_dh, rec_dw = _step(w, dev, "recompute", mode=mode)
    for chunk in (2048, 3072, 4096, 16384):
        out, dh, dw = _step(w, dev, "chunked", chunk, mode=mode)
        assert abs(out[0].item() - ref_out[0].item()) <= 1e-6 * abs(ref_out[0].item()) + 1e-9, f"chunk {chunk}"
        for a, b in zip(out[1:], ref_out[1:]):
            assert (a - b).abs().max().item() <= 2e-5, f"chunk {chunk}"
        assert cos(dh, ref_dh) >= 0.99999 and cos(dw, ref_dw) >= 0.99999
        assert cos(dh, rec_dh) >= 0.99999 and cos(dw, rec_dw) >= 0.99999
    out2, dh2, dw2 = _step(w, dev, "chunked", 2048, scale=-2.5, mode=mode)
    out1, dh1, dw1 = _step(w, dev, "chunked", 2048, mode=mode)
    assert torch.equal(out1[0], out2[0]) and torch.equal(out1[6], out2[6])
    assert cos(dh2, -dh1) >= 0.99999 and cos(dw2, -dw1) >= 0.99999
    assert abs(dw2.float().norm().item() / dw1.float().norm().item() - 2.5) < 2e-2


def test_chunked_runs_are_bit_identical(dev):
    w = filling_workload(35)
    a = _step(w, dev, "chunked", 2048)
    b = _step(w, dev, "chunked", 2048)
    assert torch.equal(a[1], b[1]) and torch.equal(a[2], b[2]) and torch.equal(a[0][0], b[0][0])


def test_auto_is_chunked_and_ignores_what_else_is_resident(dev):
    """"auto" decides from shapes and settings alone: the same step with tens of gigabytes of other tensors resident
    gives bit-identical gradients (and they are the chunked path's)."""
    w = filling_workload(36)
    a = _step(w, dev, "auto", 2048)
    free, _ = torch.cuda.mem_get_info(dev)
    ballast = torch.empty(min(100 << 30, int(free * 0.6)), dtype=torch.uint8, device=dev)
    b = _step(w, dev, "auto", 2048)
    del ballast
    c = _step(w, dev, "chunked", 2048)
    assert torch.equal(a[1], b[1]) and torch.equal(a[2], b[2])
    assert torch.equal(a[1], c[1]) and torch.equal(a[2], c[2])


def test_second_backward_recomputes(dev):
    """The chunked step's gradients are handed out once; a second backward through the same node (retain_graph)
    recomputes them from what the node saved."""
    from fgrpo import ops
    w = filling_workload(37)
    hs = w.hidden.reshape(w.T, w.H).to(dev).clone().requires_grad_(True)
    W = w.weight.to(dev).clone().requires_grad_(True)
    y = ops.shift_labels(w.labels.to(dev)).reshape(-1)
    adv = torch.randn(w.T, generator=torch.Generator().manual_seed(1)).to(dev)
    out = ops.fused_grpo_loss(hs, W, None, y, None, adv, keep_logits="chunked", chunk_tokens=2048)
    out[0].backward(retain_graph=True)
    g1h, g1w = hs.grad.clone(), W.grad.clone()
    hs.grad = None
    W.grad = None
    out[0].backward()
    assert cos(hs.grad, g1h) >= 0.99999 and cos(W.grad, g1w) >= 0.99999


def test_out_of_range_chunk_is_recomputed_on_the_device(dev):
    """One chunk of the batch holds rows whose largest logit lies 256 above the target's and outside the sampled
    vocabulary rows: its kept numerators overflow, the forward raises that chunk's flag, and the library - reading
    the flag on the device - recomputes that chunk's dLogits; the other chunks take the kept values.  Gradients
    agree with the recomputing backward's; nothing waits on the host."""
    from fgrpo import ops
    T, H, V = 8192, 1024, 8192
    gen = torch.Generator().manual_seed(21)
    hs = (torch.randn(T, H, generator=gen) * 0.5).bfloat16()
    hs[2048:4096] = 1.0                                # the second chunk of four
    W = (torch.randn(V, H, generator=gen) * 0.01).bfloat16()
    W[4000] = 0.25                                     # logit 256 for entry 4000 on the rows of ones
    y = torch.randint(8, 3999, (T,), generator=gen)
    adv = torch.randn(T, generator=gen)
    hs_d, W_d, y_d, adv_d = hs.to(dev), W.to(dev), y.to(dev), adv.to(dev)
    kept = ops.lmhead_logprob_fwd(hs_d[2048:4096].contiguous(), W_d, None, y_d[2048:4096], 1.0, keep=True)[3]
    assert ops.keep_overflowed(kept, 2048, V)
    kept = ops.lmhead_logprob_fwd(hs_d[:2048].contiguous(), W_d, None, y_d[:2048], 1.0, keep=True)[3]
    assert not ops.keep_overflowed(kept, 2048, V)
    grads = []
    for keep in ("chunked", "recompute", "whole"):
        h = hs_d.clone().requires_grad_(True)
        w = W_d.clone().requires_grad_(True)
        out = ops.fused_grpo_loss(h, w, None, y_d, None, adv_d, keep_logits=keep, chunk_tokens=2048)
        out[0].backward()
        grads.append((h.grad, w.grad, out[0].detach()))
    torch.cuda.synchronize()
    for k in (0, 2):
        assert torch.isfinite(grads[k][0].float()).all() and torch.isfinite(grads[k][1].float()).all()
        assert torch.equal(grads[k][2], grads[1][2])
        assert cos(grads[k][0], grads[1][0]) >= 0.99999 and cos(grads[k][1], grads[1][1]) >= 0.99999
        # rows of the out-of-range chunk alone, too
        assert cos(grads[k][0][2048:4096], grads[1][0][2048:4096]) >= 0.99999


def test_transient_memory_is_one_chunk(dev):
    """Peak memory beyond the inputs and the outputs (gradients, per-token vectors) is the call's workspace: one
    chunk of kept numerators - 2 * loss_chunksize tokens x V in bf16 - the fp32 dW sum, and per-chunk scratch
    bounded by the device, not by the batch (fp32 pieces of dHidden's split contraction, at most eight 256 x 256
    tiles per CU = 537 MB; the scaled transposed copy of the chunk's hidden rows)."""
    import grpo_loss as G
    from fgrpo import _lib, ops
    w = filling_workload(38, tokens=16384, V=32000)
    T, H, V = w.T, w.H, w.V
    Lc = 1024
    hs = w.hidden.to(dev).clone().requires_grad_(True)
    W = w.weight.to(dev).clone().requires_grad_(True)
    labels = w.labels.to(dev)
    adv = torch.randn(T, generator=torch.Generator().manual_seed(1)).to(dev)
    old = torch.full((T,), -9.0, device=dev)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats(dev)
    base = torch.cuda.memory_allocated(dev)
    out = G.grpo_loss_and_entropy_ce_fn(W, None, hs, labels, 1.0, old, adv, 0.2, 0.2, 1e32, loss_chunksize=Lc,
                                        keep_logits="chunked")
    out[0].backward()
    torch.cuda.synchronize()
    peak = torch.cuda.max_memory_allocated(dev) - base
    outputs = 2 * T * H + 2 * V * H + 16 * 4 * T            # dH, dW, the per-token vectors
    chunk = ops.chunk_tokens_for(T, H, V, Lc)
    assert chunk == 2 * Lc
    chunk_bytes = 2 * Lc * V * 2
    dw_sum = 4 * V * H
    ws = _lib.load().fgrpo_grpo_step_chunked_workspace(T, H, V, _lib.BF16, chunk)
    scratch_max = 8 * 256 * 256 * 256 * 4 + 2 * H * (chunk + 192) + (4 << 20)
    assert ws <= 1.01 * chunk_bytes + dw_sum + scratch_max, (ws, chunk_bytes, dw_sum)
    assert peak - outputs <= ws + (8 << 20), (peak, outputs, ws)
    # and far below what keeping the whole batch takes
    assert peak - outputs < 0.5 * ops.logits_keep_bytes(T, V)


def test_chunked_step_is_capturable_in_a_hip_graph(dev):
    """Forward, objective and gradients of a device-filling shape in one captured graph: the library neither
    synchronises nor allocates, and the out-of-range decision is taken on the device.  Three replays with changed
    inputs, eager work and synchronisations between them, each equal to the eager result bit for bit."""
    from fgrpo import ops
    w = filling_workload(39, tokens=4096)
    hs = w.hidden.reshape(w.T, w.H).to(dev).contiguous()
    W = w.weight.to(dev)
    y = ops.shift_labels(w.labels.to(dev)).reshape(-1)
    adv = torch.randn(w.T, generator=torch.Generator().manual_seed(0)).to(dev)
    old = torch.full((w.T,), -9.0, device=dev)
    cu = w.cu_seqlens.to(dev)

    def step():
        tokw, pre = ops.loss_prepare(y, cu, "sample_mean")
        res = ops.grpo_step_chunked(hs, W, None, y, old, None, adv, tokw, pre, 1.0, 0.2, 0.28, 3.0, 0.0, 1024)
        return res[0], res[1], res[2], res[4], res[10], res[11]

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    torch.cuda.synchronize()
    for k in range(3):
        hs.mul_(1.0 + 0.1 * (k + 1))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        eager = step()
        torch.cuda.synchronize()
        for a, b in zip(captured, eager):
            assert torch.equal(a, b), f"replay {k}"
