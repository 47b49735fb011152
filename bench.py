"""Benchmark of the fused logprob + GRPO forward/backward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config cfg1]

A step is one pass of the hot path (LM-head projection -> log-softmax -> target
gather -> dual-clip GRPO objective -> backward to dHidden and dW) over one packed
micro-batch of synthetic data already resident in HBM.  Prints ONE JSON line:
packed tokens/s, the MFMA roofline fraction of the dominant kernel (measured with
HIP events on the launch stream) and the CPU oracle timed on the host cores."""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (os.path.join(ROOT, "async-grpo-nccl_amd"), ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA, published (256 CUs x 4 SIMDs x 1024 flop/cycle at 2.4 GHz)
PEAK_CLOCK_MHZ = 2400.0

# HBM-side bytes per launch of the forward kernel, from two rocprofv3 --pmc runs of this file (FETCH_SIZE, then
# WRITE_SIZE, KiB per dispatch), each scaled by what the same counter reads for the 1 GiB device copy of
# --copy-probe.  Not measured in the run that prints it: the figure belongs to the binary and workload named in the
# profile summary it cites, and is None for workloads that were not profiled.
PROFILED_TRAFFIC = {
    # (workload, path): (bytes per launch of the forward kernel, summary under profiles/); a launch of the chunked
    # path is one token chunk
    ("cfg1", "chunked"): (8.116e+09, "profiles/lmhead_chunked_step_cfg1_counters_pmc.txt"),
    ("cfg1", "whole"): (3.256e+10, "profiles/lmhead_whole_batch_kept_cfg1_counters_pmc.txt"),
    ("cfg2", "chunked"): (3.121e+10, "profiles/lmhead_chunked_step_cfg2_counters_pmc.txt"),
    ("cfg3", "forward"): (3.387e+11, "profiles/lmhead_fwd_kernel_cfg3_counters_pmc.txt"),
    ("cfg4", "chunked"): (2.172e+10, "profiles/lmhead_chunked_step_cfg4_counters_pmc.txt"),
}


def cpu_baseline(name: str, cfg_chunk, seed: int):
    """The oracle (a port of the reference's eager path) on the host cores, on a
    bounded slice: one chunk of tokens at the full H and V, forward + backward,
    bf16-rounded inputs with fp32 math, one warm-up then the median of three runs.  Work is linear in tokens."""
    import torch
    from oracle import grpo_oracle as O
    from fgrpo.synthetic import CONFIGS
    cfg = CONFIGS[name]
    # every core this process may use: the harness states its share in OMP_NUM_THREADS where the machine has more
    # cores than that share (torch then starts with that many threads); otherwise all of os.cpu_count()
    cores = int(os.environ.get("OMP_NUM_THREADS") or 0) or (os.cpu_count() or 1)
    torch.set_num_threads(cores)
    H, V = cfg["H"], cfg["V"]
    g = torch.Generator().manual_seed(seed)
    W = (torch.randn(V, H, generator=g) * cfg["w_std"]).bfloat16().float()

    def run(n_tok):
        hs = (torch.randn(1, n_tok, H, generator=g) / H ** 0.5).bfloat16().float().requires_grad_(not cfg["forward_only"])
        Wl = W.clone().requires_grad_(not cfg["forward_only"])
        labels = torch.randint(0, V, (1, n_tok), generator=g)
        adv = torch.randn(n_tok, generator=g)
        old = torch.full((n_tok,), -12.0)
        t0 = time.perf_counter()
        if cfg["forward_only"]:
            with torch.no_grad():
                O.fused_log_probs_and_entropy(Wl, None, hs, labels, 1.0)
        else:
            out = O.grpo_loss_and_entropy(Wl, None, hs, labels, 1.0, old, adv, cfg["clip_low"], cfg["clip_high"], cfg["clip_ratio_c"])
            out[0].backward()
        return time.perf_counter() - t0

    probe = 128
    t_probe = run(probe)            # also the warm-up
    # one chunk of the configuration's own size, unless three runs of it would take more than 45 s on this host
    # (then the largest multiple of 128 tokens that stays inside; the line says which)
    want = cfg_chunk or 4096
    fits = probe * (45.0 / 3.0) / max(t_probe, 1e-3)
    n = int(max(probe, min(want, fits)))
    n = max(probe, (n // 128) * 128)
    times = sorted(run(n) for _ in range(3))
    t = times[1]
    what = "one chunk of the configuration's size" if n == want else f"a slice of the configuration's {want}-token chunk: three runs of the whole chunk would exceed the 45 s bound"
    return {"value": n / t, "unit": "tokens/s", "cores": cores, "os_cpu_count": os.cpu_count(), "kind": "port",
            "sample": f"{n} tokens ({what}) at full H={H}, V={V}, fwd{'' if cfg['forward_only'] else '+bwd'}, "
                      f"fp32 math on bf16-rounded inputs, one warm-up, median of 3 ({times[0]:.2f}/{times[1]:.2f}/"
                      f"{times[2]:.2f} s); tokens/s is linear in tokens"}


class ClockSampler:
    """Samples the GPU's shader clock from sysfs (the level pp_dpm_sclk marks with '*') while the timed steps run."""

    def __init__(self, period=0.02):
        import glob
        import threading
        self.paths = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))
        self.samples, self.period = [], period
        self._stop = threading.Event()
        self._thread = threading.Thread(target=self._run, daemon=True)

    def _read(self):
        for path in self.paths:
            try:
                for line in open(path):
                    if "*" in line:
                        return float(line.split(":")[1].lower().replace("mhz", "").replace("*", "").strip())
            except (OSError, ValueError, IndexError):
                continue
        return None

    def _run(self):
        while not self._stop.is_set():
            v = self._read()
            if v is not None:
                self.samples.append(v)
            time.sleep(self.period)

    def __enter__(self):
        if self.paths:
            self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        if self.paths:
            self._thread.join(timeout=1.0)

    def summary(self):
        if not self.samples:
            return None
        xs = sorted(self.samples)
        return {"median_mhz": xs[len(xs) // 2], "min_mhz": xs[0], "max_mhz": xs[-1], "samples": len(xs),
                "source": "pp_dpm_sclk (active level) sampled during the timed steps"}


def parity_gate(w, step_fn, hidden2d, weight, shifted, old, ref, adv, north_star=True, rows_n=64):
    """Before anything is timed: one step of the path on the benchmark's own inputs against the oracle.
    `rows_n` sampled token rows (logprob, entropy, and the dHidden row when the workload has a backward) and the
    loss.  The oracle forms the sampled rows' logits on the host from the same bf16 inputs in fp32; the loss is
    its objective on the [T] logprob vector; its autograd gives the per-token gradient the dHidden rows must
    show.  Returns the errors and whether they are inside the tolerances of the parity tests."""
    import torch
    from oracle import grpo_oracle as O
    p = w.params
    T, V = w.T, w.V
    lp_all, ent_all, loss, dH = step_fn()          # what the timed steps compute, from the timed entry point
    gsel = torch.Generator().manual_seed(17)
    valid = torch.nonzero(shifted != -100).reshape(-1).cpu()
    rows = valid[torch.randperm(valid.numel(), generator=gsel)[:rows_n]]
    W_c = weight.detach().float().cpu()
    hs_rows = hidden2d[rows.to(hidden2d.device)].detach().float().cpu().requires_grad_(not p["forward_only"])
    y_rows = shifted[rows.to(shifted.device)].cpu()
    x = hs_rows @ W_c.t()
    want_lp = O.logprobs_from_logits(x, y_rows)
    want_ent = O.entropy_from_logits(x.detach())
    res = {"rows": int(rows.numel()),
           "max_abs_dlogprob": float((lp_all[rows.to(lp_all.device)].cpu() - want_lp.detach()).abs().max()),
           "max_abs_dentropy": float((ent_all[rows.to(ent_all.device)].cpu() - want_ent).abs().max()),
           "tolerance": {"dlogprob": 2e-3, "dentropy": 5e-3, "loss_rel": 1e-3,
                         "loss_abs_over_mean_abs_token_term": 1e-6, "dH_rows_cosine": 0.999}}
    ok = res["max_abs_dlogprob"] <= 2e-3 and res["max_abs_dentropy"] <= 5e-3
    if not p["forward_only"]:
        lp_c = lp_all.double().cpu().requires_grad_(True)
        if north_star:
            want = O.grpo_objective_from_logprobs(lp_c, shifted.cpu(), old.double().cpu(), adv.double().cpu(),
                                                  p["clip_low"], p["clip_high"], p["clip_ratio_c"], ref.double().cpu(),
                                                  p["kl_beta"], "sample_mean", w.cu_seqlens.cpu())
        else:
            want = O.grpo_objective_from_logprobs(lp_c, shifted.cpu(), old.double().cpu(), adv.double().cpu(),
                                                  p["clip_low"], p["clip_high"], p["clip_ratio_c"])
        want[0].backward()
        res["loss"] = float(loss.detach())
        res["loss_oracle"] = float(want[0].detach())
        res["loss_rel_err"] = abs(float(loss.detach()) - float(want[0].detach())) / max(abs(float(want[0].detach())), 1e-30)
        # The loss is a mean of signed per-token terms (group-normalised advantages sum to zero) and may come out
        # orders of magnitude below the terms themselves; the error is then also judged against the terms' size.
        m = (shifted.cpu() != -100)
        res["mean_abs_token_term"] = float(want[2].detach().abs()[m].mean()) if bool(m.any()) else 0.0
        res["loss_abs_err"] = abs(float(loss.detach()) - float(want[0].detach()))
        g_rows = lp_c.grad[rows].float()
        (want_lp * g_rows).sum().backward()
        got = dH.reshape(T, -1)[rows.to(dH.device)].float().cpu()
        res["dH_rows_cosine"] = float(torch.nn.functional.cosine_similarity(got.flatten(), hs_rows.grad.flatten(), dim=0))
        loss_ok = res["loss_rel_err"] <= 1e-3 or res["loss_abs_err"] <= 1e-6 * res["mean_abs_token_term"]
        ok = ok and loss_ok and res["dH_rows_cosine"] >= 0.999
    res["passed"] = bool(ok)
    return res


def library_yardstick(hidden2d, weight, fwd_only, reps=5):
    """The vendor library's GEMM (torch.matmul -> hipBLASLt) on the products of the path, same shapes and dtype, on
    this device right after the timed steps: logits = hidden . weight^T (written as bf16), and for the backward
    dHidden = logits . weight and dW = logits^T . hidden with the logits standing in for dLogits.  Nothing of the
    soft-max, the objective or the gather is in these times: they are what the matrix products alone cost through
    the library, the yardstick for the fused kernels' fractions of peak."""
    import torch
    T, H = hidden2d.shape
    V = weight.shape[0]
    thv = 2.0 * T * H * V

    def timed(fn):
        fn()
        torch.cuda.synchronize()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(reps + 1)]
        ev[0].record()
        for i in range(reps):
            fn()
            ev[i + 1].record()
        torch.cuda.synchronize()
        ms = sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(reps))[reps // 2]
        return {"ms": ms, "tflops": thv / (ms * 1e-3) / 1e12, "frac": thv / (ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS}
    logits = torch.empty(T, V, dtype=hidden2d.dtype, device=hidden2d.device)
    out = {"what": "torch.matmul (hipBLASLt) on the same shapes, matrix products only, median of %d" % reps,
           "logits": timed(lambda: torch.matmul(hidden2d, weight.t(), out=logits))}
    if not fwd_only:
        dh = torch.empty_like(hidden2d)
        dw = torch.empty_like(weight)
        out["dhidden"] = timed(lambda: torch.matmul(logits, weight, out=dh))
        out["dweight"] = timed(lambda: torch.matmul(logits.t(), hidden2d, out=dw))
        out["sum_ms"] = out["logits"]["ms"] + out["dhidden"]["ms"] + out["dweight"]["ms"]
    return out


def attention_line(args):
    """One layer of packed variable-length attention (forward + backward) at the packing of the benchmark
    micro-batch: T tokens in segments of 128..1024, 12 query heads over 2 K/V heads, head dimension 128
    (the attention shape of the 1.5B model).  Algorithmic flops count the visible (query, key) pairs only:
    forward 4*D per pair and head, backward 10*D (recomputing the scores is not counted)."""
    import torch
    from fgrpo import ops
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    T, D = 32768, 128
    g = torch.Generator().manual_seed(args.seed)
    if args.attention_shape == "long":      # the 7B model's heads on four 8192-token samples
        Hq, Hkv, lens = 28, 4, [8192] * 4
    else:                                   # the 1.5B model's heads on the benchmark packing
        Hq, Hkv, lens = 12, 2, []
        while sum(lens) < T:
            lens.append(int(torch.randint(128, 1025, (1,), generator=g)))
        lens[-1] -= sum(lens) - T
    cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32, device=dev)
    q = torch.randn(T, Hq, D, generator=g).bfloat16().to(dev)
    k = torch.randn(T, Hkv, D, generator=g).bfloat16().to(dev)
    v = torch.randn(T, Hkv, D, generator=g).bfloat16().to(dev)
    do = torch.randn(T, Hq, D, generator=g).bfloat16().to(dev)
    pairs = sum(n * (n + 1) // 2 for n in lens)
    f_fwd = 4.0 * D * Hq * pairs

    # per-token segment bounds and tile launch order: built once per packed batch and shared by every layer's
    # forward and backward, so outside the per-layer timing
    bounds = ops.attention_bounds(cu, T, True)

    def step():
        out, lse = ops.varlen_attn_fwd(q, k, v, cu, bounds=bounds)
        return ops.varlen_attn_bwd(do, q, k, v, out, lse, cu, bounds=bounds)

    # a layer takes under a millisecond: keep the GPU busy for a quarter of a second first, or the timed steps run
    # while the clocks are still ramping up from idle (measured: 0.70 ms/step after 3 warm-up steps, 0.64 after 200)
    n_warm, t_w = 0, time.perf_counter()
    while n_warm < args.warmup or time.perf_counter() - t_w < 0.25:
        step()
        n_warm += 1
        if n_warm % 16 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
    t_f = t_b = 0.0
    t0 = time.perf_counter()
    for _ in range(args.steps):
        ev[0].record()
        out, lse = ops.varlen_attn_fwd(q, k, v, cu, bounds=bounds)
        ev[1].record()
        ops.varlen_attn_bwd(do, q, k, v, out, lse, cu, bounds=bounds)
        ev[2].record()
        torch.cuda.synchronize()
        t_f += ev[0].elapsed_time(ev[1])
        t_b += ev[1].elapsed_time(ev[2])
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    t_f /= args.steps
    t_b /= args.steps
    achieved = f_fwd / (t_f * 1e-3) / 1e12
    print(json.dumps({
        "metric": "packed tokens/sec of one layer's variable-length attention fwd+bwd; MFMA % peak",
        "value": T / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": n_warm,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"attention: T={T} packed tokens in {len(lens)} segments of {min(lens)}..{max(lens)}, Hq={Hq}, Hkv={Hkv}, "
                               f"D={D}, causal, forward + backward", "tokens": T, "segments": len(lens)},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_BF16_TFLOPS, "traffic": None, "kernel": "varlen_attn_fwd_kernel",
                     "kernel_ms": t_f, "algorithmic_flops_per_launch": f_fwd},
        "backward": {"ms": t_b, "algorithmic_flops": 2.5 * f_fwd, "achieved": 2.5 * f_fwd / (t_b * 1e-3) / 1e12,
                     "frac": 2.5 * f_fwd / (t_b * 1e-3) / 1e12 / PEAK_BF16_TFLOPS},
    }), flush=True)


def hbm_line(args):
    """The bandwidth-bound kernels of the path at a size where bandwidth, not launch latency, decides: the
    per-token objective (loss_fwd = token kernel + normaliser), the diagnostics, the segmented reductions and
    broadcasts over cu_seqlens, and the row kernels on materialised logits.  Algorithmic bytes per kernel are the
    arrays it must read and write once; times are HIP-event brackets on the launch stream."""
    import torch
    from fgrpo import ops
    import grpo_loss as G
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    g = torch.Generator().manual_seed(args.seed)
    PEAK = 8000.0

    def timed(fn):
        n_warm, t_w = 0, time.perf_counter()       # short kernels: warm up by time (0.1 s), not by count
        while n_warm < args.warmup or time.perf_counter() - t_w < 0.1:
            fn()
            n_warm += 1
            if n_warm % 16 == 0:
                torch.cuda.synchronize()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps

    rows = []
    for T in (32768, 1 << 20):
        lens = []
        while sum(lens) < T:
            lens.append(int(torch.randint(128, 1025, (1,), generator=g)))
        lens[-1] -= sum(lens) - T
        cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32, device=dev)
        lp = (-torch.rand(T, generator=g) * 3).to(dev)
        old = lp + 0.01 * torch.randn(T, generator=g).to(dev)
        ref = lp + 0.05 * torch.randn(T, generator=g).to(dev)
        adv = torch.randn(T, generator=g).to(dev)
        y = torch.randint(0, 1000, (T,), generator=g).to(dev)
        idx = torch.nonzero(y >= 0).reshape(-1)
        per_seg = torch.randn(len(lens), generator=g).to(dev)
        # loss: reads lp, old, ref, adv (4 B each) and labels (8 B); writes g and four diagnostics; g is read and
        # written once more by the normaliser
        ms = timed(lambda: ops.grpo_loss_fwd(lp, old, ref, adv, y, None, 0.2, 0.2, 3.0, 0.01))
        rows.append((f"objective (token + normaliser kernels), T={T}", T * (4 * 4 + 8 + 5 * 4 + 8), ms))
        out = ops.grpo_loss_fwd(lp, old, ref, adv, y, None, 0.2, 0.2, 3.0, 0.01)
        ms = timed(lambda: ops.grpo_metrics(idx, out[2], lp, None, adv, out[4], out[5], 0.2, 0.2))
        rows.append((f"diagnostics (two-stage sum), T={T}", T * (8 + 5 * 4), ms))
        ms = timed(lambda: ops.segment_reduce(lp, cu, y))
        rows.append((f"segment_reduce over cu_seqlens, T={T}", T * (4 + 8), ms))
        ms = timed(lambda: ops.segment_broadcast(per_seg, cu, T))
        rows.append((f"segment_broadcast (incl. torch zero fill), T={T}", T * 8, ms))
    for dt in (torch.bfloat16, torch.float32):
        N, V = 4096, 151936
        x = torch.randn(N, V, device=dev, dtype=dt)
        yy = torch.randint(0, V, (N,), device=dev)
        nb = x.numel() * x.element_size()
        ms = timed(lambda: G.logprobs_from_logits_flash_attn(x, yy))
        rows.append((f"row logprob forward, {str(dt).split('.')[1]} logits [{N} x {V}]", nb, ms))
        ms = timed(lambda: G.entropy_from_logits(x))
        rows.append((f"row entropy, {str(dt).split('.')[1]} logits [{N} x {V}]", nb, ms))
        lse = ops.logits_logprob_entropy(x, yy, -100)[2]
        gg = torch.randn(N, device=dev)
        ms = timed(lambda: ops.logits_logprob_bwd(x, yy, -100, gg, lse))
        rows.append((f"row logprob backward, {str(dt).split('.')[1]} logits [{N} x {V}]", 2 * nb, ms))
        del x
    kernels = [{"kernel": n, "algorithmic_bytes": b, "ms": ms, "achieved_GBps": b / (ms * 1e-3) / 1e9,
                "frac": b / (ms * 1e-3) / 1e9 / PEAK} for n, b, ms in rows]
    best = max(kernels, key=lambda r: r["achieved_GBps"])
    print(json.dumps({
        "metric": "achieved HBM GB/s of the reduction / elementwise / row kernels of the path",
        "value": best["achieved_GBps"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": best["ms"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic", "config": {"workload": "bandwidth-bound kernels: " + best["kernel"]},
        "roofline": {"bound": "hbm", "achieved": best["achieved_GBps"], "peak": PEAK, "unit": "GB/s",
                     "frac": best["frac"], "traffic": None},
        "kernels": kernels,
    }), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", default="cfg1")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-parity", action="store_true", help="skip the oracle check that precedes the timed steps")
    ap.add_argument("--no-library-yardstick", action="store_true",
                    help="skip timing the vendor GEMM library on the three products of the path (after the timed steps)")
    ap.add_argument("--objective", choices=["north_star", "reference"], default="north_star",
                    help="north_star: KL to the reference policy + mean over samples of per-sample token means (every "
                         "scored token has a gradient); reference: the reference's own objective, token mean without "
                         "KL (grpo_loss.py:318-348) - tokens of zero-advantage groups then have no gradient and the "
                         "backward skips them")
    ap.add_argument("--reward-p", type=float, default=None,
                    help="probability of reward 1 per sample (default: the configuration's); with --objective reference "
                         "it sets the share of zero-advantage groups")
    ap.add_argument("--keep-logits", choices=["auto", "chunked", "whole", "on", "recompute", "off"], default="auto",
                    help="the headline path's way to the gradients: chunked (the default where supported: the whole step in "
                         "token chunks, one chunk of bf16 soft-max numerators as the transient), whole / on (numerators of the "
                         "whole batch kept, [T x V] bf16), recompute / off (logits recomputed in the backward)")
    ap.add_argument("--chunk", type=int, default=None,
                    help="loss_chunksize handed to the drop-in instead of the configuration's (the chunked step walks twice that many tokens at a time)")
    ap.add_argument("--no-alt-paths", action="store_true",
                    help="time the headline path only (by default the other ways to the same gradients are timed after it)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="after the timed steps, run one 1 GiB device copy (reference point for traffic counters)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--tokens", type=int, default=None,
                    help="pack this many tokens instead of the configuration's own count (the reference fills a "
                         "micro-batch up to a budget, 36000 by default: token counts off the 256-token tile grid)")
    ap.add_argument("--attention", action="store_true",
                    help="time the packed attention kernels instead (prints their own JSON line)")
    ap.add_argument("--attention-shape", choices=["cfg1", "long"], default="cfg1")
    ap.add_argument("--hbm-kernels", action="store_true",
                    help="time the bandwidth-bound kernels of the path instead (prints their own JSON line)")
    ap.add_argument("--tuning", action="append", default=[], metavar="KEY=VALUE",
                    help="set a tuning key of the library before anything runs (e.g. attn_dkv=1: the single-wavefront "
                         "dK/dV kernel); may be given several times")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (the path shards by micro-batch, one per GPU); "
              "--gpus must be 1", file=sys.stderr)
        sys.exit(2)

    if args.tuning:
        from fgrpo import _lib
        _lib.set_tuning(**{k: int(v) for k, v in (kv.split("=", 1) for kv in args.tuning)})

    if args.attention:
        return attention_line(args)
    if args.hbm_kernels:
        return hbm_line(args)

    import torch
    import grpo_loss as G
    from fgrpo import ops
    from fgrpo.synthetic import make_workload

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    over = {}
    if args.reward_p is not None:
        over["reward_p"] = args.reward_p
    if args.tokens is not None:
        over["tokens"] = args.tokens
    w = make_workload(args.config, seed=args.seed, device=dev, overrides=over or None)
    p = w.params
    T, H, V = w.T, w.H, w.V
    fwd_only = p["forward_only"]
    labels = w.labels
    shifted = ops.shift_labels(labels).reshape(-1)
    north_star = args.objective == "north_star"
    thv = 2.0 * T * H * V
    chunk_arg = p["chunk"] if args.chunk is None else args.chunk

    # inputs of the objective: advantages from the group kernel, old/ref = current logprob + noise
    adv_s = ops.group_advantages(w.rewards, w.group_offsets, p["adv_eps"])
    adv = ops.segment_broadcast(adv_s, w.cu_seqlens, T)
    with torch.no_grad():
        lp0, _, _ = ops.lmhead_logprob_fwd(w.hidden.reshape(T, H), w.weight, None, shifted)
    old = lp0 + w.noise_old
    ref = lp0 + w.noise_ref

    # Two input sets at different addresses, used in turn: no step finds the previous step's operands in a cache.
    class Inputs:
        def __init__(self):
            self.hidden = w.hidden.clone().requires_grad_(not fwd_only)
            self.weight = w.weight.clone().requires_grad_(not fwd_only)
            self.old, self.ref, self.adv, self.labels = old.clone(), ref.clone(), adv.clone(), labels.clone()
            self.cu = w.cu_seqlens.clone()
    sets = [Inputs(), Inputs()]

    def step(k=0, keep_logits=None):
        s = sets[k % len(sets)]
        if fwd_only:
            with torch.no_grad():
                return G.fused_log_probs_and_entropy_fn(s.weight, None, s.hidden, s.labels)
        s.hidden.grad = None
        s.weight.grad = None
        extra = dict(ref_logprobs=s.ref, kl_beta=p["kl_beta"], loss_agg_mode="sample_mean", cu_seqlens=s.cu) if north_star else {}
        out = G.grpo_loss_and_entropy_ce_fn(s.weight, None, s.hidden, s.labels, 1.0, s.old, s.adv, p["clip_low"],
                                            p["clip_high"], p["clip_ratio_c"], loss_chunksize=chunk_arg,
                                            keep_logits=keep_logits, **extra)
        out[0].backward()
        return out

    # Which way to the gradients each timed path takes (fgrpo.ops.KEEP_LOGITS); the headline is the default.
    chunk_tok = ops.chunk_tokens_for(T, H, V, chunk_arg)
    chunked_ok = (not fwd_only) and ops.chunked_supported(T, H, V, w.dtype, chunk_tok)
    whole_ok = (not fwd_only) and ops.keep_supported(T, H, V, w.dtype)
    headline = {"auto": "chunked" if chunked_ok else "recompute", "chunked": "chunked", "on": "whole", "whole": "whole",
                "off": "recompute", "recompute": "recompute"}[args.keep_logits]
    if fwd_only:
        headline = "forward"
    n_chunks = (T + chunk_tok - 1) // chunk_tok if chunked_ok else 1      # (the library may cut the last two chunks evenly)
    lib = ops._lib.load()
    path_notes = {
        "chunked": {"never_holds_T_x_V": True, "executed_products": 3,
                    "what": f"the whole step in {n_chunks} token chunks of at most {chunk_tok}: forward keeping one chunk of bf16 soft-max "
                            "numerators, objective, dHidden rows, dW summed in fp32 across chunks; backward() scales by the upstream scalar",
                    "transient_bytes": int(lib.fgrpo_grpo_step_chunked_workspace(T, H, V, ops._lib.BF16, chunk_tok)) if chunked_ok else None,
                    "transient_of_which_kept_numerators_bytes": int(ops.logits_keep_bytes(min(T, chunk_tok), V)) if chunked_ok else None,
                    "transient_of_which_fp32_dW_sum_bytes": (4 * V * H if n_chunks > 1 else 0) if chunked_ok else None},
        "whole": {"never_holds_T_x_V": False, "executed_products": 3,
                  "what": "bf16 soft-max numerators of the whole batch kept between forward and backward",
                  "transient_bytes": int(ops.logits_keep_bytes(T, V)) if whole_ok else None},
        "recompute": {"never_holds_T_x_V": True, "executed_products": 4,
                      "what": "logits recomputed in backward(), one vocabulary panel of dLogits at a time",
                      "transient_bytes": None if fwd_only else int(lib.fgrpo_lmhead_bwd_workspace(T, H, V, ops._lib.BF16 if w.dtype == torch.bfloat16 else ops._lib.F32,
                                                                                     ops.panel_elems_bound(T, V, chunk_arg)))},
        "forward": {"never_holds_T_x_V": True, "executed_products": 1, "what": "forward only (logprobs and entropy), no gradient",
                    "transient_bytes": int(lib.fgrpo_logprob_fwd_workspace(T, H, V, ops._lib.BF16 if w.dtype == torch.bfloat16 else ops._lib.F32))},
    }

    # ---- parity on the same inputs, before timing ----
    def gate_step():
        out = step(0, None if fwd_only else headline)
        torch.cuda.synchronize()
        if fwd_only:
            return out[0], out[1], None, None
        return out[2] + old, out[1], out[0], sets[0].hidden.grad        # log_ratio = lp - old
    parity = None
    if not args.no_parity:
        parity = parity_gate(w, gate_step, w.hidden.reshape(T, H), w.weight, shifted, old, ref, adv, north_star)
        if not parity["passed"]:
            print("bench.py: parity check failed, nothing timed: " + json.dumps(parity), file=sys.stderr)
            sys.exit(1)

    def phase(kernel, total_ms, launches, steps, flops, note=None):
        per = total_ms / steps
        d = {"kernel": kernel, "ms": per, "launches_per_step": launches // steps if steps else 0, "flops": flops,
             "frac": (flops / (per * 1e-3) / 1e12 / PEAK_BF16_TFLOPS) if (flops and per > 0) else None}
        if note:
            d["note"] = note
        return d

    def measure(path, steps, warmup, sample_clock=False):
        """`steps` timed steps of one path after `warmup` untimed ones: wall clock around the loop (bracketed by
        synchronisations), HIP events per step, and HIP events on the launch stream around the kernels' launches
        (inside the library for the backward and the chunked step, around the library call for the stand-alone
        forward)."""
        keep = None if fwd_only else path
        for i in range(warmup):
            step(i, keep)
        torch.cuda.synchronize()
        fwd_events = []
        ops.set_fwd_event_sink(fwd_events)
        if not fwd_only:
            ops.phase_timing_begin()
        step_events = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
        clock = ClockSampler()
        with clock:
            t0 = time.perf_counter()
            step_events[0].record()
            for i in range(steps):
                step(i, keep)
                step_events[i + 1].record()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
        ops.set_fwd_event_sink(None)
        phase_ms, phase_n, dropped = ops.phase_timing_end() if not fwd_only else ({}, {}, 0)
        per_step = sorted(step_events[i].elapsed_time(step_events[i + 1]) for i in range(steps))
        ms = dt / steps * 1e3
        if path == "chunked":
            k_total, k_n = phase_ms["fwd"], phase_n["fwd"]
            tok_per_launch = T / max(1, k_n // steps)
        else:
            k_total, k_n = sum(a.elapsed_time(b) for a, b in fwd_events), len(fwd_events)
            tok_per_launch = T
        k_ms = k_total / max(1, k_n)
        flops_launch = 2.0 * tok_per_launch * H * V
        kept = path in ("chunked", "whole")
        fwd_name = "lmhead_fwd_kernel" + (" (keeps the bf16 soft-max numerators" + (" of one token chunk)" if path == "chunked" else ")") if kept else "") + " + combine"
        phases = [phase(fwd_name, k_total, k_n, steps, thv)]
        if not fwd_only:
            if kept:
                phases.append(phase("keep_backward_prep_kernel (+ the gated recompute launch, scaled transposed copy of hidden, live runs)",
                                    phase_ms["dlogits"], phase_n["dlogits"], steps, 0.0,
                                    f"per-token factors, one patched element per row ({4.0 * T * H / 1e6:.0f} MB): no pass over [T x V]"))
            else:
                phases.append(phase("lmhead_ds_kernel (recomputes the logits, one vocabulary panel per launch)",
                                    phase_ms["dlogits"], phase_n["dlogits"], steps, thv, "executed, not algorithmic, work"))
            phases.append(phase("gemm_store_kernel dHidden", phase_ms["dh"], phase_n["dh"], steps, thv))
            phases.append(phase("gemm_store_kernel dW" + (" (fp32 sum across chunks)" if path == "chunked" and n_chunks > 1 else ""),
                                phase_ms["dw"], phase_n["dw"], steps, thv))
            phases.append(phase("everything else inside the library calls (chunked: reference pre-pass of the kept numerators, objective kernels; bias sums)",
                                phase_ms["other"], phase_n["other"], steps, 0.0))
        alg = (1.0 if fwd_only else 3.0) * thv
        res = {"path": path, **path_notes[path], "steps": steps, "warmup": warmup, "ms_per_step": ms,
               "ms_per_step_median": per_step[len(per_step) // 2], "ms_per_step_min": per_step[0],
               "tokens_per_s": T / (ms / 1e3), "path_mfma_frac": alg / (ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
               "path_algorithmic_tflops": alg / (ms * 1e-3) / 1e12,
               "path_executed_tflops": path_notes[path]["executed_products"] * thv / (ms * 1e-3) / 1e12,
               "forward_kernel_ms_per_launch": k_ms, "forward_launches_timed": k_n,
               "forward_frac": flops_launch / (k_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS if k_ms > 0 else None,
               "phases": phases, "phase_brackets_dropped": dropped}
        return res, clock.summary(), k_ms, flops_launch, k_n

    head, clock_summary, k_ms, flops_launch, k_n = measure(headline, args.steps, args.warmup)
    ms = head["ms_per_step"]
    tok_s = head["tokens_per_s"]

    # the other ways to the same gradients, timed after the headline with fewer steps
    alt = {}
    if not fwd_only and not args.no_alt_paths:
        for path in ("whole", "recompute", "chunked"):
            if path == headline or (path == "whole" and not whole_ok) or (path == "chunked" and not chunked_ok):
                continue
            try:
                alt[{"whole": "whole_batch_kept"}.get(path, path)] = measure(path, max(3, min(args.steps, 8)), 2)[0]
            except Exception as e:      # noqa: BLE001
                alt[path] = {"error": f"{type(e).__name__}: {e}"[:300]}
            torch.cuda.empty_cache()

    yardstick = None
    if not args.no_library_yardstick:
        try:        # a comparison beside the measurement: its failure must not cost the line
            yardstick = library_yardstick(w.hidden.reshape(T, H).detach(), w.weight.detach(), fwd_only)
        except Exception as e:      # noqa: BLE001
            yardstick = {"error": f"{type(e).__name__}: {e}"[:300]}

    if args.copy_probe:
        # a plain device copy of known size, so that one counter run holds the scale of FETCH_SIZE / WRITE_SIZE
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
    achieved = flops_launch / (k_ms * 1e-3) / 1e12
    prof = PROFILED_TRAFFIC.get((args.config if args.tokens is None else None, headline))

    line = {
        "metric": "packed tokens/sec fused logprob+GRPO fwd/bwd (Qwen2.5-1.5B shape); MFMA % peak",
        "value": tok_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if w.dtype == torch.bfloat16 else "fp32", "data": "synthetic",
        "config": {"workload": f"{args.config}: T={T} packed tokens, H={H}, V={V}, "
                               f"{'forward only' if fwd_only else 'forward+backward (dHidden, dW)'}, "
                               f"{w.n_samples} samples, loss chunk size {chunk_arg}",
                   "tokens": T, "hidden": H, "vocab": V, "samples": w.n_samples,
                   "objective": None if fwd_only else (
                       "north_star: dual clip + k3 KL to the reference policy, mean over samples of per-sample token means"
                       if north_star else "reference: dual clip, token mean, no KL (grpo_loss.py:318-348)"),
                   "tokens_without_gradient": None if fwd_only else float(((adv == 0) | (shifted == -100)).float().mean()) if not north_star
                   else float((shifted == -100).float().mean()),
                   "backward": None if fwd_only else f"{headline}: {path_notes[headline]['what']}",
                   "never_holds_T_x_V": path_notes[headline]["never_holds_T_x_V"],
                   "transient_bytes": path_notes[headline]["transient_bytes"],
                   "input_sets_rotated": len(sets)},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_BF16_TFLOPS,
                     "frac_at_held_clock": (achieved / (PEAK_BF16_TFLOPS * clock_summary["median_mhz"] / PEAK_CLOCK_MHZ))
                     if clock_summary else None,
                     "traffic": prof[0] if prof else None,
                     "traffic_source": (prof[1] + " (rocprofv3 --pmc runs of this command; not measured in this run)") if prof else None,
                     "kernel": head["phases"][0]["kernel"], "kernel_ms": k_ms,
                     "kernel_launches_timed": k_n,
                     "algorithmic_flops_per_launch": flops_launch,
                     "phases": head["phases"], "phase_brackets_dropped": head["phase_brackets_dropped"],
                     "library_yardstick": yardstick,
                     "peak_note": f"published peak = {PEAK_CLOCK_MHZ:.0f} MHz x 256 CUs x 4096 flop/cycle; the clock the "
                                  "device held during the timed steps is under 'clock'"},
        "clock": clock_summary,
        "parity": parity,
        "ms_per_step_median": head["ms_per_step_median"], "ms_per_step_min": head["ms_per_step_min"],
        "path_mfma_frac": head["path_mfma_frac"],
        "path_algorithmic_tflops": head["path_algorithmic_tflops"],
        # what the matrix pipeline executes: three products where numerators are kept, a fourth where logits are recomputed
        "path_executed_tflops": head["path_executed_tflops"],
        "alt_paths": alt or None,
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(args.config, chunk_arg, args.seed)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
