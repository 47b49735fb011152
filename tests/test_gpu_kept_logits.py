"""The forward/backward pair that keeps a [T x V] bf16 matrix for the backward (as the reference's autograd keeps
its logits, grpo_loss.py:286-313) instead of recomputing the logits - here the soft-max numerators against a
per-token reference - and the whole path at the full benchmark sizes through the drop-in's own entry point.

Small device-filling shapes are compared with the CPU oracle outright.  At the full sizes the oracle cannot form
[T x V] in seconds: the per-token logprobs (pinned against sampled oracle rows in test_gpu_parity) feed the oracle's
objective on [T] vectors, whose autograd gives the per-token gradient that sampled rows of dH and dW must show."""
import math

import pytest
import torch

from oracle import grpo_oracle as O
from test_gpu_parity import COS_MIN, LOSS_REL, LP_TOL_BF16, check, cos, group_adv, run_case

pytestmark = pytest.mark.gpu


def filling_workload(seed, **over):
    """A shape the kept-logits kernels accept (H % 256 == 0, at least half the device's tiles in both gradient
    products) that the oracle still finishes in seconds."""
    from fgrpo.synthetic import make_workload
    cfg = dict(H=1024, V=8492, tokens=8155, len_lo=40, len_hi=700, h_scale=1.0, w_std=0.05, prompts=4, group=8)
    cfg.update(over)
    return make_workload("cfg1", seed=seed, overrides=cfg)


@pytest.mark.parametrize("mode", ["reference", "north_star"])
def test_kept_logits_against_oracle(dev, mode):
    from fgrpo import ops
    w = filling_workload(11)
    assert ops.keep_supported(w.T, w.H, w.V, torch.bfloat16)
    want, got, o, g, _, _ = run_case(w, dev, mode, keep_logits=True)
    check(want, got, o, g, f32=False)


@pytest.mark.parametrize("keep", [True, False])
def test_hidden_size_that_is_not_a_multiple_of_the_tile(dev, keep):
    """H = 896 (the 0.5B model's width, 3.5 tiles of 256): the gradient products still read W, hidden and the
    [T x V] buffer where they lie; both the kept and the recomputing backward against the oracle."""
    from fgrpo import ops
    w = filling_workload(16, H=896)
    assert ops.keep_supported(w.T, w.H, w.V, torch.bfloat16)
    want, got, o, g, _, _ = run_case(w, dev, "north_star", keep_logits=keep)
    check(want, got, o, g, f32=False)


def test_kept_logits_with_bias_and_temperature(dev):
    w = filling_workload(12)
    bias = (torch.randn(w.V, generator=torch.Generator().manual_seed(9)) * 0.3).to(w.dtype)
    want, got, o, g, _, _ = run_case(w, dev, "north_star", temperature=0.7, bias=bias, keep_logits=True)
    check(want, got, o, g, f32=False)


def test_kept_forward_is_bit_identical_and_backward_close_to_recompute(dev):
    """Keeping the numerators changes nothing in the forward (statistics come from the fp32 accumulators either
    way); the backward differs from the recomputing one only by bf16 rounding (of the kept values there, of
    dLogits here)."""
    from fgrpo import ops
    w = filling_workload(13, tokens=8192 + 64)           # token count past a multiple of 256
    hs, W = w.hidden.reshape(w.T, w.H).to(dev), w.weight.to(dev)
    y = ops.shift_labels(w.labels.to(dev)).reshape(-1)
    a = ops.lmhead_logprob_fwd(hs, W, None, y, 0.9)
    b = ops.lmhead_logprob_fwd(hs, W, None, y, 0.9, keep=True)
    for x, z in zip(a, b[:3]):
        assert torch.equal(x, z)
    g = torch.randn(w.T, generator=torch.Generator().manual_seed(2)).to(dev) / w.T
    g[::5] = 0
    gout = torch.tensor([2.5], device=dev)
    dH0, dW0, _ = ops.lmhead_bwd(hs, W, None, y, a[2], g, gout, 0.9, True, True, False, 0)
    dH1, dW1, _ = ops.lmhead_bwd_kept(hs, W, None, y, a[2], g, gout, 0.9, b[3], True, True, False)
    assert cos(dH0, dH1) >= 0.99999 and cos(dW0, dW1) >= 0.99999
    dead = (g == 0) | (y == -100)
    assert (dH1[dead] == 0).all()                                      # rows without gradient are exact zeros
    # two runs on the same kept logits are bit-identical (no atomics anywhere)
    b2 = ops.lmhead_logprob_fwd(hs, W, None, y, 0.9, keep=True)
    dH2, dW2, _ = ops.lmhead_bwd_kept(hs, W, None, y, a[2], g, gout, 0.9, b2[3], True, True, False)
    assert torch.equal(dH1, dH2) and torch.equal(dW1, dW2)


def test_kept_logits_panel_split_matches_single_launch(dev):
    """The tuning key keep_panels splits the gradient products into vocabulary panels with an fp32 dH accumulator:
    dW is bit-identical (each row block is still written once), dH agrees to bf16 rounding."""
    from fgrpo import _lib, ops
    w = filling_workload(14)
    hs, W = w.hidden.reshape(w.T, w.H).to(dev), w.weight.to(dev)
    y = ops.shift_labels(w.labels.to(dev)).reshape(-1)
    g = torch.randn(w.T, generator=torch.Generator().manual_seed(3)).to(dev) / w.T
    lp, ent, lse, kept = ops.lmhead_logprob_fwd(hs, W, None, y, 1.0, keep=True)
    dH1, dW1, _ = ops.lmhead_bwd_kept(hs, W, None, y, lse, g, None, 1.0, kept, True, True, False)
    _lib.set_tuning(keep_panels=3)
    try:
        dH3, dW3, _ = ops.lmhead_bwd_kept(hs, W, None, y, lse, g, None, 1.0, kept, True, True, False)
    finally:
        _lib.set_tuning(keep_panels=0)
    assert torch.equal(dW1, dW3)
    assert cos(dH1, dH3) >= 0.99999


def test_kept_values_out_of_range_fall_back_to_recomputation(dev):
    """The kept numerators are exp(x_v - ref - 40) in bf16 with ref = max(target logit, largest logit among the first
    512 vocabulary entries): a row whose largest logit exceeds both by more than 128 would overflow them.  The
    forward flags it, and the backward - which reads the flag on the device, no host wait - then overwrites the
    buffer with dLogits recomputed from the operands before its two products: the recomputing backward's gradients
    (the same bf16 dLogits; the fp32 sums run in another order), finite everywhere; the forward's own outputs never
    depend on the kept values.  The same dominant entry INSIDE the sampled rows raises no flag."""
    from fgrpo import ops
    T, H, V = 8192, 1024, 8192
    gen = torch.Generator().manual_seed(21)
    hs = torch.ones(T, H).bfloat16()
    W = (torch.randn(V, H, generator=gen) * 0.01).bfloat16()
    W[4000] = 0.25                                     # logit 256 for entry 4000 on every row; the targets sit near 0
    y = torch.randint(8, 3999, (T,), generator=gen)
    adv = torch.randn(T, generator=gen)
    hs_d, W_d, y_d, adv_d = hs.to(dev), W.to(dev), y.to(dev), adv.to(dev)
    lp, ent, lse, kept = ops.lmhead_logprob_fwd(hs_d, W_d, None, y_d, 1.0, keep=True)
    assert ops.keep_overflowed(kept, T, V)
    assert (lp < -128).all() and torch.isfinite(lp).all() and torch.isfinite(lse).all()
    grads = []
    for keep in (True, False):
        h = hs_d.clone().requires_grad_(True)
        w = W_d.clone().requires_grad_(True)
        out = ops.fused_grpo_loss(h, w, None, y_d, None, adv_d, keep_logits=keep)
        out[0].backward()
        grads.append((h.grad, w.grad, out[0].detach()))
    cos64 = lambda a, b: float((a.double().flatten() @ b.double().flatten()) / (a.double().norm() * b.double().norm()))
    assert cos64(grads[0][0], grads[1][0]) >= 0.99999 and cos64(grads[0][1], grads[1][1]) >= 0.99999
    assert (grads[0][0].float() - grads[1][0].float()).abs().max() <= 2e-2 * grads[1][0].float().abs().max()
    assert torch.equal(grads[0][2], grads[1][2])
    assert torch.isfinite(grads[0][0].float()).all() and torch.isfinite(grads[0][1].float()).all()
    # the dominant entry among the sampled rows: the reference follows it, nothing overflows
    W1 = W.clone()
    W1[4000] = W[4001]
    W1[7] = 0.25
    lp1, _, _, kept1 = ops.lmhead_logprob_fwd(hs_d, W1.to(dev), None, y_d, 1.0, keep=True)
    assert not ops.keep_overflowed(kept1, T, V) and (lp1 < -128).all()
    # and an ordinary batch does not raise the flag
    W2 = (torch.randn(V, H, generator=gen) * 0.05).bfloat16().to(dev)
    kept2 = ops.lmhead_logprob_fwd(torch.randn(T, H, generator=gen).bfloat16().to(dev), W2, None, y_d, 1.0, keep=True)[3]
    assert not ops.keep_overflowed(kept2, T, V)


def test_kept_buffer_survives_the_backward(dev):
    """The backward patches one element per row with a value computed from scratch and otherwise only reads the
    buffer: running it twice on the same buffer gives the same gradients."""
    from fgrpo import ops
    w = filling_workload(15)
    hs, W = w.hidden.reshape(w.T, w.H).to(dev), w.weight.to(dev)
    y = ops.shift_labels(w.labels.to(dev)).reshape(-1)
    g = torch.randn(w.T, generator=torch.Generator().manual_seed(4)).to(dev) / w.T
    lp, ent, lse, kept = ops.lmhead_logprob_fwd(hs, W, None, y, 1.0, keep=True)
    a = ops.lmhead_bwd_kept(hs, W, None, y, lse, g, None, 1.0, kept, True, True, False)
    b = ops.lmhead_bwd_kept(hs, W, None, y, lse, 2 * g, None, 1.0, kept, True, True, False)
    c = ops.lmhead_bwd_kept(hs, W, None, y, lse, g, None, 1.0, kept, True, True, False)
    assert torch.equal(a[0], c[0]) and torch.equal(a[1], c[1])
    assert cos(b[0], a[0]) >= 0.99999 and abs(b[1].float().norm().item() / a[1].float().norm().item() - 2.0) < 1e-2


@pytest.mark.parametrize("pattern", ["groups", "all_dead", "alternating", "tail"])
def test_rows_without_gradient_are_skipped_exactly(dev, pattern):
    """Zero-advantage samples give long stretches of tokens with g_t = 0 (the reference logs their share as
    adv_zero_frac, grpo_loss.py:450).  The kept-path backward skips them - dHidden by 256-row tile, dW by 64-row
    step of its contraction - and must produce the very same gradients as without skipping: leaving out exact
    zeros changes no fp32 sum."""
    from fgrpo import _lib, ops
    w = filling_workload(17, tokens=8192 + 300)
    T = w.T
    hs, W = w.hidden.reshape(T, w.H).to(dev), w.weight.to(dev)
    y = ops.shift_labels(w.labels.to(dev)).reshape(-1)
    g = torch.randn(T, generator=torch.Generator().manual_seed(5)).to(dev) / T
    if pattern == "groups":                       # dead stretches that start and end anywhere
        for a, b in ((0, 700), (1500, 1501), (2048, 4096), (5000, 5063), (6000, 8300)):
            g[a:b] = 0
    elif pattern == "all_dead":
        g.zero_()
    elif pattern == "alternating":                # every other 64-row step dead: many short runs
        g.view(-1)[: (T // 128) * 128].view(-1, 2, 64)[:, 1, :] = 0
    else:                                         # only the very last rows live
        g[: T - 5] = 0
    lp, ent, lse, kept = ops.lmhead_logprob_fwd(hs, W, None, y, 1.0, keep=True)
    res = {}
    for skip in (1, 0):
        _lib.set_tuning(keep_skip_dead=skip)
        try:
            res[skip] = ops.lmhead_bwd_kept(hs, W, None, y, lse, g, None, 1.0, kept, True, True, False)
        finally:
            _lib.set_tuning(keep_skip_dead=1)
    assert torch.equal(res[1][0], res[0][0]) and torch.equal(res[1][1], res[0][1])
    assert (res[1][0][g == 0] == 0).all()
    if pattern == "all_dead":
        assert (res[1][1] == 0).all()
    else:
        dH0, dW0, _ = ops.lmhead_bwd(hs, W, None, y, lse, g, None, 1.0, True, True, False, 0)
        assert cos(res[1][0], dH0) >= 0.9999 and cos(res[1][1], dW0) >= 0.9999


@pytest.mark.parametrize("tokens", [1, 77, 300, 1000])
def test_few_tokens_take_the_kept_path_too(dev, tokens):
    """The kept numerators need the vocabulary side to fill the device, not the token side: with one or a few token
    tiles the forward splits the vocabulary finely and dHidden its contraction.  Forward against the oracle row by
    row, the backward against the oracle's autograd, for token counts down to a single token."""
    from fgrpo import ops
    H, V = 512, 33000              # 129 vocabulary tiles: the large tile for any token count
    assert ops.keep_supported(tokens, H, V, torch.bfloat16)
    g0 = torch.Generator().manual_seed(100 + tokens)
    hidden = torch.randn(tokens, H, generator=g0).to(torch.bfloat16)
    weight = (torch.randn(V, H, generator=g0) * 0.05).to(torch.bfloat16)
    bias = (torch.randn(V, generator=g0) * 0.3).to(torch.bfloat16)
    y = torch.randint(0, V, (tokens,), generator=g0)
    if tokens > 10:
        y[3] = -100
    gt = torch.randn(tokens, generator=g0)
    gt[y == -100] = 0
    hd, wd, bd, yd, gd = (t.to(dev) for t in (hidden, weight, bias, y, gt))
    lp, ent, lse, kept = ops.lmhead_logprob_fwd(hd, wd, bd, yd, 0.8, keep=True)
    assert not ops.keep_overflowed(kept, tokens, V)
    dH, dW, db = ops.lmhead_bwd_kept(hd, wd, bd, yd, lse, gd, None, 0.8, kept, True, True, True)
    hs = hidden.float().requires_grad_(True)
    Wo = weight.float().requires_grad_(True)
    bo = bias.float().requires_grad_(True)
    logits = O.project(Wo, bo, hs, 0.8)
    want_lp = O.logprobs_from_logits(logits, y)
    valid = y != -100
    assert (lp.cpu() - want_lp.detach()).abs().max().item() <= LP_TOL_BF16
    assert ((ent.cpu() - O.entropy_from_logits(logits.detach())) * valid).abs().max().item() <= 5e-3
    (want_lp * gt).sum().backward()
    assert cos(dH, hs.grad) >= COS_MIN and cos(dW, Wo.grad) >= COS_MIN and cos(db, bo.grad) >= COS_MIN
    assert (dH.cpu()[~valid] == 0).all()


@pytest.mark.parametrize("tokens,H", [(64 * 256 + 700, 2048), (9000, 1024), (33 * 256 + 1, 1536)])
def test_split_contraction_of_the_last_row_tiles(dev, tokens, H):
    """dHidden's row tiles beyond whole device rounds (or all of them, when there are few) have their contraction
    over the vocabulary split among several work-groups, whose fp32 tiles are then added in a fixed order: against
    the same backward with the split switched off (equal up to the rounding of bf16 outputs summed in another
    order), bit-identical between two runs, rows without gradient exact zeros, and dW untouched by the switch."""
    from fgrpo import _lib, ops
    V = 4000 if H == 2048 else 8492
    g0 = torch.Generator().manual_seed(tokens)
    hs = torch.randn(tokens, H, generator=g0).to(torch.bfloat16).to(dev)
    W = (torch.randn(V, H, generator=g0) * 0.03).to(torch.bfloat16).to(dev)
    y = torch.randint(0, V, (tokens,), generator=g0).to(dev)
    g = (torch.randn(tokens, generator=g0) / tokens).to(dev)
    g[tokens - 300: tokens - 40] = 0             # a dead stretch inside the last row tiles
    g[100:700] = 0                               # a whole dead tile (rows 256..511) in the first ones
    nt = (tokens + 255) // 256
    g[(nt - 3) * 256: (nt - 2) * 256] = 0        # and one among the last ones
    assert ops.keep_supported(tokens, H, V, torch.bfloat16)
    lp, ent, lse, kept = ops.lmhead_logprob_fwd(hs, W, None, y, 1.0, keep=True)
    res = {}
    for split in (1, 0, 1):
        _lib.set_tuning(tail_split=split)
        try:
            out = ops.lmhead_bwd_kept(hs, W, None, y, lse, g, None, 1.0, kept, True, True, False)
        finally:
            _lib.set_tuning(tail_split=1)
        if split in res:
            assert torch.equal(out[0], res[split][0]) and torch.equal(out[1], res[split][1])
        res[split] = out
    a, b = res[1][0].float(), res[0][0].float()
    assert ((a - b).norm() / b.norm()).item() <= 3e-3 and cos(a, b) >= 0.99999
    assert (res[1][0][g == 0] == 0).all()
    assert torch.equal(res[1][1], res[0][1])
    dH0, _, _ = ops.lmhead_bwd(hs, W, None, y, lse, g, None, 1.0, True, False, False, 0)
    assert cos(res[1][0], dH0) >= 0.9999


@pytest.mark.parametrize("tokens", [4321, 13 * 256 + 17])
def test_wide_hidden_takes_the_patch_rasters(dev, tokens):
    """More than 8 column tiles (H = 2560: 10): the gradient GEMMs walk 4 x 8 tile patches per XCD - the grouped
    raster for dW, the round-robin one for dHidden when dead rows are skipped - with row-tile counts that are no
    multiple of the patch.  Against the oracle, and skipping against not skipping bit for bit."""
    from fgrpo import _lib, ops
    w = filling_workload(18, H=2560, V=4200, tokens=tokens, len_hi=500)
    assert ops.keep_supported(w.T, w.H, w.V, torch.bfloat16)
    want, got, o, g_, _, _ = run_case(w, dev, "north_star", keep_logits=True)
    check(want, got, o, g_, f32=False)
    T = w.T
    hs, W = w.hidden.reshape(T, w.H).to(dev), w.weight.to(dev)
    y = ops.shift_labels(w.labels.to(dev)).reshape(-1)
    g = torch.randn(T, generator=torch.Generator().manual_seed(6)).to(dev) / T
    for a, b in ((0, 300), (1000, 2600), (T - 700, T - 3)):
        g[a:b] = 0
    lp, ent, lse, kept = ops.lmhead_logprob_fwd(hs, W, None, y, 1.0, keep=True)
    res = {}
    for skip in (1, 0):
        _lib.set_tuning(keep_skip_dead=skip)
        try:
            res[skip] = ops.lmhead_bwd_kept(hs, W, None, y, lse, g, None, 1.0, kept, True, True, False)
        finally:
            _lib.set_tuning(keep_skip_dead=1)
    assert torch.equal(res[1][0], res[0][0]) and torch.equal(res[1][1], res[0][1])
    dH0, dW0, _ = ops.lmhead_bwd(hs, W, None, y, lse, g, None, 1.0, True, True, False, 0)
    assert cos(res[1][0], dH0) >= 0.9999 and cos(res[1][1], dW0) >= 0.9999


def test_keep_refuses_what_it_cannot_do(dev):
    from fgrpo import ops
    hs = torch.randn(512, 192, device=dev).bfloat16()
    W = torch.randn(4096, 192, device=dev).bfloat16()
    y = torch.randint(0, 4096, (512,), device=dev)
    assert not ops.keep_supported(512, 192, 4096, torch.bfloat16)
    with pytest.raises(RuntimeError, match="kept-logits"):
        ops.lmhead_logprob_fwd(hs, W, None, y, 1.0, keep=True)
    with pytest.raises(RuntimeError, match="keep_logits=True"):
        ops.fused_grpo_loss(hs.requires_grad_(True), W, None, y, None, torch.randn(512, device=dev), keep_logits=True)
    # "auto" quietly recomputes for such a shape
    out = ops.fused_grpo_loss(hs, W, None, y, None, torch.randn(512, device=dev), keep_logits="auto")
    out[0].backward()
    assert hs.grad is not None and torch.isfinite(hs.grad.float()).all()


# ------------------------------------------------------------------ full benchmark sizes through the drop-in
@pytest.mark.parametrize("name,keep,tokens", [("cfg1", "chunked", None), ("cfg1", True, None), ("cfg1", False, None),
                                              ("cfg2", "chunked", None), ("cfg2", True, None), ("cfg2", False, None),
                                              ("cfg4", "chunked", None), ("cfg4", True, None), ("cfg4", False, None),
                                              ("cfg1", "chunked", 33000), ("cfg1", True, 33000)])
def test_full_size_through_the_drop_in(dev, name, keep, tokens):
    """grpo_loss_and_entropy_ce_fn exactly as bench.py calls it (KL to the reference policy, mean over samples of
    per-sample token means, cu_seqlens, the configuration's chunk hint), then backward with a non-unit upstream
    scale.  Checked: loss and the four per-token diagnostics against the oracle's objective evaluated on the
    kernel's per-token logprobs; sampled rows of dH and of dW against the closed form with the oracle's per-token
    gradient (with every row's soft-max normaliser taken from plain torch, which also pins the kernel's lse on all
    T rows); columns of dW summing to zero.  keep: "chunked" = the default, the whole step in token chunks of twice
    the configuration's chunk size; True = numerators of the whole batch kept; False = logits recomputed."""
    import grpo_loss as G
    from fgrpo import ops
    from fgrpo.synthetic import make_workload
    # tokens: a count off the 256-token tile grid (129 token tiles at 33000: the forward's two token regions and the
    # split contraction of dHidden's last row tile, at the benchmark's H and V)
    w = make_workload(name, seed=0, device=dev, overrides=None if tokens is None else dict(tokens=tokens))
    p = w.params
    T, H, V = w.T, w.H, w.V
    assert ops.keep_supported(T, H, V, torch.bfloat16) and (tokens is None or T == tokens)
    shifted = ops.shift_labels(w.labels).reshape(-1)
    hs2 = w.hidden.reshape(T, H)
    adv = group_adv(w, p["adv_eps"]).to(dev)
    lp0, _, lse = ops.lmhead_logprob_fwd(hs2, w.weight, None, shifted)
    old, ref = lp0 + w.noise_old, lp0 + w.noise_ref

    hidden = w.hidden.clone().requires_grad_(True)
    weight = w.weight.clone().requires_grad_(True)
    out = G.grpo_loss_and_entropy_ce_fn(weight, None, hidden, w.labels, 1.0, old, adv, p["clip_low"], p["clip_high"],
                                        p["clip_ratio_c"], loss_chunksize=p["chunk"], ref_logprobs=ref,
                                        kl_beta=p["kl_beta"], loss_agg_mode="sample_mean", cu_seqlens=w.cu_seqlens,
                                        keep_logits=keep)
    scale = 3.7
    (out[0] * scale).backward()
    torch.cuda.synchronize()

    # the oracle's objective on the kernel's logprobs, on the CPU in fp64
    lp_c = lp0.double().cpu().requires_grad_(True)
    want = O.grpo_objective_from_logprobs(lp_c, shifted.cpu(), old.double().cpu(), adv.double().cpu(), p["clip_low"],
                                          p["clip_high"], p["clip_ratio_c"], ref.double().cpu(), p["kl_beta"],
                                          "sample_mean", w.cu_seqlens.cpu())
    (want[0] * scale).backward()
    assert abs(out[0].item() - want[0].item()) <= LOSS_REL * abs(want[0].item()) + 1e-7
    for k_got, k_want in ((2, 1), (3, 2), (4, 3), (5, 4)):          # log_ratio, clip1, unclipped, clipped
        assert (out[k_got].double().cpu() - want[k_want].detach()).abs().max().item() <= 10 * LP_TOL_BF16
    g = lp_c.grad.float().to(dev)                                    # d (scale * loss) / d lp_t

    gsel = torch.Generator().manual_seed(5)
    rows = torch.randperm(T, generator=gsel)[:128].to(dev)
    x = hs2[rows].float() @ w.weight.float().t()
    prob = torch.softmax(x, -1)
    safe = shifted[rows].clamp(min=0)
    want_dH = g[rows, None] * (w.weight.float()[safe] - prob @ w.weight.float())
    assert cos(hidden.grad.reshape(T, H)[rows], want_dH) >= COS_MIN
    # the soft-max normaliser of EVERY row from plain torch (fp32 matmul + logsumexp, a block of rows at a time):
    # it pins the kernel's lse on all T rows and is what the closed form of the sampled dW rows uses
    w32 = w.weight.float()
    lse_ref = torch.empty(T, dtype=torch.float32, device=dev)
    for a in range(0, T, 2048):
        lse_ref[a:a + 2048] = torch.logsumexp(hs2[a:a + 2048].float() @ w32.t(), dim=-1)
    assert (lse - lse_ref).abs().max().item() <= LP_TOL_BF16
    vs = torch.randperm(V, generator=gsel)[:16].to(dev)
    xv = hs2.float() @ w.weight[vs].float().t()
    coef = g[:, None] * ((shifted[:, None] == vs[None, :]).float() - torch.exp(xv - lse_ref[:, None]))
    want_dW = coef.t() @ hs2.float()
    assert cos(weight.grad[vs], want_dW) >= COS_MIN
    col = weight.grad.float().sum(0)
    assert col.abs().max().item() <= 1e-2 * weight.grad.float().abs().sum(0).max().item()


def test_cfg3_through_the_logprob_harness(dev):
    """The forward-only configuration (T = 131072, H = 5120) through LogProbHarness on a model whose body is an
    embedding: per-sample lists equal the kernel's flat vectors, sampled rows equal the oracle."""
    from types import SimpleNamespace
    import grpo_loss as G
    import workers
    from fgrpo import ops
    from fgrpo.synthetic import make_workload
    w = make_workload("cfg3", seed=0, device=dev)
    T, H, V = w.T, w.H, w.V

    class Body(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.table = w.hidden.reshape(T, H)

        def forward(self, input_ids=None, position_ids=None, **kw):
            # hidden state of packed position t is row t of the workload's hidden matrix
            n = input_ids.shape[1]
            return (self.table[:n].reshape(1, n, H),)

    class Model(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.model = Body()
            self.lm_head = torch.nn.Linear(H, V, bias=False, device="meta")
            self.lm_head.weight = torch.nn.Parameter(w.weight, requires_grad=False)
            self.config = SimpleNamespace(output_attentions=False, output_hidden_states=False, use_return_dict=True)

        def forward(self, *a, **kw):
            raise AssertionError("the patched forward must be used")

    model = G.make_grpo_forward(Model(), temperature=1.0, mode="eval")
    harness = workers.LogProbHarness(model, dev)
    ids, labels = w.input_ids.reshape(-1).cpu(), w.labels.reshape(-1).cpu()
    cu = w.cu_seqlens.cpu().tolist()
    samples = [dict(sample_ids=ids[a:b].tolist(), labels=labels[a:b].tolist()) for a, b in zip(cu[:-1], cu[1:])]
    got = harness.compute_log_probs_from_samples(samples)
    shifted = ops.shift_labels(w.labels).reshape(-1)
    lp, ent, _ = ops.lmhead_logprob_fwd(w.hidden.reshape(T, H), w.weight, None, shifted)
    flat_lp = torch.tensor([v for s in got for v in s["logprobs"]])
    flat_ent = torch.tensor([v for s in got for v in s["entropies"]])
    assert torch.equal(flat_lp, lp.cpu()) and torch.equal(flat_ent, ent.cpu())
    rows = torch.randperm(T, generator=torch.Generator().manual_seed(6))[:96].to(dev)
    x_c = (w.hidden.reshape(T, H)[rows].float() @ w.weight.float().t()).cpu()
    want_lp = O.logprobs_from_logits(x_c, shifted[rows].cpu())
    assert (lp[rows].cpu() - want_lp).abs().max() <= LP_TOL_BF16
    assert (lp <= 1e-6).all() and (ent <= math.log(V) + 1e-3).all()
