"""Torch-facing wrappers of the C ABI: allocate outputs and workspaces with
torch (device memory and streams are torch's), hand raw pointers to the HIP
library, and wire the forward/backward pair into autograd.

Nothing here computes: every number comes out of ``libfgrpo.so``.  CPU tensors
are rejected - there is no eager fallback."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib

IGNORE_INDEX = -100


# --------------------------------------------------------------------------- helpers
def _require_cuda(*tensors) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("fgrpo: tensors must live on the GPU (the HIP path has no CPU fallback)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError("fgrpo: all tensors must be on the same device")
    if dev is None:
        raise RuntimeError("fgrpo: no tensor given")
    return dev


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.bfloat16:
        return _lib.BF16
    if dtype == torch.float32:
        return _lib.F32
    raise RuntimeError(f"fgrpo: unsupported dtype {dtype} (bf16 and fp32 only)")


def _f32(t: Optional[torch.Tensor], n: int, name: str) -> Optional[torch.Tensor]:
    if t is None:
        return None
    t = t.detach().reshape(-1)
    if t.numel() != n:
        raise RuntimeError(f"fgrpo: {name} has {t.numel()} elements, expected {n}")
    return t.to(torch.float32).contiguous()


def _aligned(t: torch.Tensor) -> torch.Tensor:
    """Contiguous and 16-byte aligned (a sliced view can start anywhere)."""
    t = t.detach().contiguous()
    return t if t.data_ptr() % 16 == 0 else t.clone()


def _ws(nbytes: int, device) -> torch.Tensor:
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


def shift_labels(labels: torch.Tensor) -> torch.Tensor:
    """labels [..., L] -> next-token targets, -100 in the last column."""
    return torch.nn.functional.pad(labels, (0, 1), value=IGNORE_INDEX)[..., 1:].contiguous()


# --------------------------------------------------------------------------- raw ops
# Optional timing hook: when a list is installed, every forward launch appends a pair of events recorded on
# the launch stream right before and right after the library call (nothing is synchronised here).
_fwd_event_sink = None


def set_fwd_event_sink(sink) -> None:
    global _fwd_event_sink
    _fwd_event_sink = sink


def keep_supported(T: int, H: int, V: int, dtype: torch.dtype) -> bool:
    """Whether the kept-logits forward/backward pair handles this problem: bf16, H % 64 == 0 and a vocabulary side
    that fills the device (V/256 x H/256 tiles for at least half the CUs; any token count)."""
    if dtype != torch.bfloat16 or T <= 0:
        return False
    return bool(_lib.load().fgrpo_keep_supported(int(T), int(H), int(V), _lib.BF16))


def logits_keep_bytes(T: int, V: int) -> int:
    return int(_lib.load().fgrpo_logits_keep_bytes(int(T), int(V)))


def lmhead_logprob_fwd(hidden: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                       labels_shifted: torch.Tensor, temperature: float = 1.0,
                       want_entropy: bool = True, want_lse: bool = True, keep: bool = False):
    """hidden [T,H], weight [V,H] (same dtype, bf16 or fp32), labels_shifted [T] int64
    -> (lp [T] fp32, entropy [T] fp32 | None, lse [T] fp32 | None); with ``keep`` a fourth result, the uint8 buffer
    holding the bf16 soft-max numerators in the library's blocked layout, for ``lmhead_bwd_kept``."""
    dev = _require_cuda(hidden, weight, bias, labels_shifted)
    lib = _lib.load()
    if hidden.dim() != 2 or weight.dim() != 2 or hidden.shape[1] != weight.shape[1]:
        raise RuntimeError(f"fgrpo: hidden {tuple(hidden.shape)} / weight {tuple(weight.shape)} mismatch")
    if hidden.dtype != weight.dtype:
        raise RuntimeError("fgrpo: hidden and weight must share a dtype")
    T, H = hidden.shape
    V = weight.shape[0]
    code = _code(weight.dtype)
    hidden = _aligned(hidden)
    weight = _aligned(weight)
    if bias is not None:
        bias = bias.detach().to(weight.dtype).contiguous()
        if bias.numel() != V:
            raise RuntimeError("fgrpo: bias must have V elements")
    labels_shifted = labels_shifted.reshape(-1).to(torch.int64).contiguous()
    if labels_shifted.numel() != T:
        raise RuntimeError("fgrpo: labels must have one entry per token")
    lp = torch.empty(T, dtype=torch.float32, device=dev)
    ent = torch.empty(T, dtype=torch.float32, device=dev) if want_entropy else None
    lse = torch.empty(T, dtype=torch.float32, device=dev) if want_lse else None
    if keep and not keep_supported(T, H, V, weight.dtype):
        raise RuntimeError(f"fgrpo: the kept-logits forward does not handle T={T} H={H} V={V} {weight.dtype}")
    if T == 0:
        return lp, ent, lse
    nbytes = lib.fgrpo_logprob_fwd_workspace(T, H, V, code)
    ws = _ws(nbytes, dev)
    kept = torch.empty(lib.fgrpo_logits_keep_bytes(T, V), dtype=torch.uint8, device=dev) if keep else None
    with torch.cuda.device(dev):
        sink = _fwd_event_sink
        if sink is not None:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
        if keep:
            rc = lib.fgrpo_logprob_fwd_keep(_ptr(hidden), _ptr(weight), _ptr(bias), _ptr(labels_shifted),
                                            1.0 / float(temperature), T, H, V, code,
                                            _ptr(lp), _ptr(ent), _ptr(lse), _ptr(kept), kept.numel(),
                                            _ptr(ws), ws.numel(), _stream())
        else:
            rc = lib.fgrpo_logprob_fwd(_ptr(hidden), _ptr(weight), _ptr(bias), _ptr(labels_shifted),
                                       1.0 / float(temperature), T, H, V, code,
                                       _ptr(lp), _ptr(ent), _ptr(lse), _ptr(ws), ws.numel(), _stream())
        if sink is not None:
            e1.record()
            sink.append((e0, e1))
    _lib.check(rc, "logprob_fwd_keep" if keep else "logprob_fwd")
    return (lp, ent, lse, kept) if keep else (lp, ent, lse)


def phase_timing_begin() -> None:
    """Start bracketing the launches of this thread's backward calls with HIP events (diagnostics)."""
    _lib.check(_lib.load().fgrpo_phase_timing_begin(), "phase_timing_begin")


def phase_timing_end():
    """Stop and read: ({phase: summed ms}, {phase: brackets}, dropped) for the phases dlogits / dh / dw / other / fwd
    (fwd: the forward launches of the chunked step; the stand-alone forward is not bracketed by the library)."""
    import ctypes
    ms = (ctypes.c_float * _lib.NUM_PHASES)()
    cnt = (ctypes.c_int * _lib.NUM_PHASES)()
    rc = _lib.load().fgrpo_phase_timing_end(ctypes.cast(ms, ctypes.c_void_p), ctypes.cast(cnt, ctypes.c_void_p))
    if rc < 0:
        _lib.check(rc, "phase_timing_end")
    names = ("dlogits", "dh", "dw", "other", "fwd")
    return {n: float(ms[i]) for i, n in enumerate(names)}, {n: int(cnt[i]) for i, n in enumerate(names)}, int(rc)


def lmhead_bwd(hidden, weight, bias, labels_shifted, lse, g, gout: Optional[torch.Tensor],
               temperature: float, need_dh: bool, need_dw: bool, need_db: bool,
               panel_elems_hint: int = 0):
    """Gradients of the projection+log-softmax+gather given g = d loss / d lp [T].
    Returns (dH [T,H] | None, dW [V,H] | None, dbias [V] | None) in the input dtype."""
    dev = _require_cuda(hidden, weight, labels_shifted, lse, g)
    lib = _lib.load()
    T, H = hidden.shape
    V = weight.shape[0]
    code = _code(weight.dtype)
    hidden = _aligned(hidden)
    weight = _aligned(weight)
    if bias is not None:
        bias = bias.detach().to(weight.dtype).contiguous()
    labels_shifted = labels_shifted.reshape(-1).to(torch.int64).contiguous()
    lse = _f32(lse, T, "lse")
    g = _f32(g, T, "g")
    if gout is not None:
        gout = gout.detach().reshape(-1)[:1].to(device=dev, dtype=torch.float32).contiguous()
    dH = torch.empty_like(hidden) if need_dh else None
    dW = torch.empty_like(weight) if need_dw else None
    db = torch.empty(V, dtype=weight.dtype, device=dev) if (need_db and bias is not None) else None
    if T == 0 or not (need_dh or need_dw or db is not None):
        if dW is not None:
            dW.zero_()
        if db is not None:
            db.zero_()
        return dH, dW, db
    nbytes = lib.fgrpo_lmhead_bwd_workspace(T, H, V, code, int(panel_elems_hint))
    ws = _ws(nbytes, dev)
    with torch.cuda.device(dev):
        rc = lib.fgrpo_lmhead_bwd(_ptr(hidden), _ptr(weight), _ptr(bias), _ptr(labels_shifted), _ptr(lse), _ptr(g),
                                  _ptr(gout), 1.0 / float(temperature), T, H, V, code,
                                  _ptr(dH), _ptr(dW), _ptr(db), int(panel_elems_hint),
                                  _ptr(ws), ws.numel(), _stream())
    _lib.check(rc, "lmhead_bwd")
    return dH, dW, db


def keep_overflowed(kept: torch.Tensor, T: int, V: int) -> bool:
    """True when the forward flagged that the kept values may have overflowed (a logit more than 123 log-probability
    units above both the target logit and the largest logit of the first 512 vocabulary rows).  Waits for the current
    stream.  A query for tests and reports: the backward reads the flag on the device and recomputes by itself."""
    with torch.cuda.device(kept.device):
        rc = _lib.load().fgrpo_keep_overflowed(_ptr(kept), int(T), int(V), _stream())
    if rc < 0:
        _lib.check(rc, "keep_overflowed")
    return rc != 0


def lmhead_bwd_kept(hidden, weight, bias, labels_shifted, lse, g, gout: Optional[torch.Tensor], temperature: float,
                    kept: torch.Tensor, need_dh: bool, need_dw: bool, need_db: bool):
    """The backward on the soft-max numerators the forward kept (``lmhead_logprob_fwd(..., keep=True)``): one
    element per row of ``kept`` is patched in place, then dH / dW / dbias come from one GEMM each reading the buffer
    as it lies.  When the forward raised the buffer's overflow flag, the library (reading it on the device)
    first overwrites the buffer with dLogits recomputed from the operands: same launches, no host synchronisation."""
    dev = _require_cuda(hidden, weight, labels_shifted, lse, g, kept)
    lib = _lib.load()
    T, H = hidden.shape
    V = weight.shape[0]
    code = _code(weight.dtype)
    hidden = _aligned(hidden)
    weight = _aligned(weight)
    if bias is not None:
        bias = bias.detach().to(weight.dtype).contiguous()
    labels_shifted = labels_shifted.reshape(-1).to(torch.int64).contiguous()
    lse = _f32(lse, T, "lse")
    g = _f32(g, T, "g")
    if gout is not None:
        gout = gout.detach().reshape(-1)[:1].to(device=dev, dtype=torch.float32).contiguous()
    dH = torch.empty_like(hidden) if need_dh else None
    dW = torch.empty_like(weight) if need_dw else None
    db = torch.empty(V, dtype=weight.dtype, device=dev) if (need_db and bias is not None) else None
    if not (need_dh or need_dw or db is not None):
        return dH, dW, db
    ws = _ws(lib.fgrpo_lmhead_bwd_kept_workspace(T, H, V, code), dev)
    with torch.cuda.device(dev):
        rc = lib.fgrpo_lmhead_bwd_kept(_ptr(hidden), _ptr(weight), _ptr(bias), _ptr(labels_shifted), _ptr(lse), _ptr(g),
                                       _ptr(gout), 1.0 / float(temperature), T, H, V, code,
                                       _ptr(kept), kept.numel(), _ptr(dH), _ptr(dW), _ptr(db),
                                       _ptr(ws), ws.numel(), _stream())
    _lib.check(rc, "lmhead_bwd_kept")
    return dH, dW, db


def grpo_loss_fwd(lp, old_lp, ref_lp, adv, labels_shifted, cu_seqlens=None,
                  clip_low=0.2, clip_high=0.4, clip_ratio_c=1e32, kl_beta=0.0,
                  loss_agg_mode="token_mean", denom_override: float = 0.0, want_diag: bool = True):
    """Per-token dual-clip objective on device.
    Returns (loss [] fp32, g [T], log_ratio, clip1, unclipped, clipped, scal [4])."""
    dev = _require_cuda(lp, adv, labels_shifted)
    lib = _lib.load()
    T = lp.numel()
    lp = _f32(lp, T, "lp")
    old_lp = _f32(old_lp, T, "old_logprobs")
    ref_lp = _f32(ref_lp, T, "ref_logprobs")
    adv = _f32(adv, T, "advantages")
    labels_shifted = labels_shifted.reshape(-1).to(torch.int64).contiguous()
    if loss_agg_mode == "token_mean":
        agg = _lib.AGG_TOKEN_MEAN
    elif loss_agg_mode == "sample_mean":
        agg = _lib.AGG_SAMPLE_MEAN
        if cu_seqlens is None:
            raise RuntimeError("fgrpo: loss_agg_mode='sample_mean' needs cu_seqlens")
    else:
        raise ValueError(f"Invalid loss_agg_mode: {loss_agg_mode}")
    nseq = 0
    if cu_seqlens is not None:
        cu_seqlens = cu_seqlens.to(device=dev, dtype=torch.int32).contiguous()
        nseq = cu_seqlens.numel() - 1
    mk = lambda: torch.empty(T, dtype=torch.float32, device=dev)
    loss = torch.empty((), dtype=torch.float32, device=dev)
    g = mk()
    lr, c1, l1, l2 = (mk(), mk(), mk(), mk()) if want_diag else (None, None, None, None)
    scal = torch.empty(4, dtype=torch.float32, device=dev)
    if T == 0:
        loss.zero_()
        scal.zero_()
        return loss, g, lr, c1, l1, l2, scal
    ws = _ws(lib.fgrpo_loss_fwd_workspace(T, nseq), dev)
    clamp = lambda x: float(max(min(float(x), 3.0e38), -3.0e38))
    with torch.cuda.device(dev):
        rc = lib.fgrpo_loss_fwd(_ptr(lp), _ptr(old_lp), _ptr(ref_lp), _ptr(adv), _ptr(labels_shifted),
                                _ptr(cu_seqlens), nseq, T, clamp(clip_low), clamp(clip_high), clamp(clip_ratio_c),
                                clamp(kl_beta), agg, float(denom_override),
                                _ptr(loss), _ptr(g), _ptr(lr), _ptr(c1), _ptr(l1), _ptr(l2), _ptr(scal),
                                _ptr(ws), ws.numel(), _stream())
    _lib.check(rc, "loss_fwd")
    return loss, g, lr, c1, l1, l2, scal


def grpo_metrics(output_indices, log_ratio, entropy, old_entropy, adv, unclipped, clipped,
                 clip_low: float, clip_high: float) -> torch.Tensor:
    """One [16] float64 device vector (layout in include/fgrpo.h): partial sums per work-group, added in a fixed
    order by a second small launch when there are more than 2048 positions."""
    dev = _require_cuda(log_ratio, adv)
    lib = _lib.load()
    T = log_ratio.numel()
    idx = output_indices.to(device=dev, dtype=torch.int64).reshape(-1).contiguous()
    buf = torch.zeros(_lib.NUM_STATS * (1 + _lib.METRIC_BLOCKS), dtype=torch.float64, device=dev)
    stats, partial = buf[:_lib.NUM_STATS], buf[_lib.NUM_STATS:]
    with torch.cuda.device(dev):
        rc = lib.fgrpo_metrics(_ptr(idx), idx.numel(), T, _ptr(_f32(log_ratio, T, "log_ratio")),
                               _ptr(_f32(entropy, T, "entropy")), _ptr(_f32(old_entropy, T, "old_entropy")),
                               _ptr(_f32(adv, T, "advantages")), _ptr(_f32(unclipped, T, "unclipped")),
                               _ptr(_f32(clipped, T, "clipped")), float(clip_low), float(clip_high),
                               _ptr(stats), _ptr(partial), _stream())
    _lib.check(rc, "metrics")
    return stats


def group_advantages(rewards: torch.Tensor, group_offsets: torch.Tensor, eps: float = 1e-4,
                     out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """(r - mean) / (population std + eps) per group; rewards fp32/fp64 on device."""
    dev = _require_cuda(rewards)
    lib = _lib.load()
    if rewards.dtype not in (torch.float32, torch.float64):
        rewards = rewards.to(torch.float64)
    rewards = rewards.reshape(-1).contiguous()
    goff = group_offsets.to(device=dev, dtype=torch.int32).contiguous()
    out = torch.empty(rewards.numel(), dtype=out_dtype, device=dev)
    if rewards.numel() == 0:
        return out
    o32 = _ptr(out) if out_dtype == torch.float32 else None
    o64 = _ptr(out) if out_dtype == torch.float64 else None
    if o32 is None and o64 is None:
        raise RuntimeError("fgrpo: out_dtype must be float32 or float64")
    with torch.cuda.device(dev):
        rc = lib.fgrpo_group_advantages(_ptr(rewards), int(rewards.dtype == torch.float64), _ptr(goff),
                                        goff.numel() - 1, rewards.numel(), float(eps), o32, o64, _stream())
    _lib.check(rc, "group_advantages")
    return out


def segment_broadcast(values: torch.Tensor, cu_seqlens: torch.Tensor, total: int) -> torch.Tensor:
    """out[t] = values[segment(t)], fp32 [total]."""
    dev = _require_cuda(values)
    lib = _lib.load()
    if values.dtype not in (torch.float32, torch.float64):
        values = values.to(torch.float32)
    values = values.reshape(-1).contiguous()
    cu = cu_seqlens.to(device=dev, dtype=torch.int32).contiguous()
    out = torch.zeros(total, dtype=torch.float32, device=dev)
    if values.numel() == 0:
        return out
    with torch.cuda.device(dev):
        rc = lib.fgrpo_segment_broadcast(_ptr(values), int(values.dtype == torch.float64), _ptr(cu), cu.numel() - 1,
                                         int(total), _ptr(out), _stream())
    _lib.check(rc, "segment_broadcast")
    return out


def segment_reduce(x: torch.Tensor, cu_seqlens: torch.Tensor, labels_shifted: Optional[torch.Tensor] = None):
    """Per-segment (sum, mean, count) of a per-token fp32 array, masked by labels != -100 when given."""
    dev = _require_cuda(x)
    lib = _lib.load()
    x = x.detach().reshape(-1).to(torch.float32).contiguous()
    cu = cu_seqlens.to(device=dev, dtype=torch.int32).contiguous()
    n = cu.numel() - 1
    s = torch.empty(n, dtype=torch.float32, device=dev)
    m = torch.empty(n, dtype=torch.float32, device=dev)
    c = torch.empty(n, dtype=torch.int32, device=dev)
    lab = None if labels_shifted is None else labels_shifted.reshape(-1).to(torch.int64).contiguous()
    if lab is not None and lab.numel() != x.numel():
        raise RuntimeError("fgrpo: labels must have one entry per token")
    if n > 0:
        with torch.cuda.device(dev):
            rc = lib.fgrpo_segment_reduce(_ptr(x), _ptr(lab), _ptr(cu), n, x.numel(), _ptr(s), _ptr(m), _ptr(c), _stream())
        _lib.check(rc, "segment_reduce")
    return s, m, c


def output_indices(input_lens, output_lens, device) -> torch.Tensor:
    """int64 positions of the logits scoring every generated token (see fgrpo_output_indices)."""
    lib = _lib.load()
    il = torch.as_tensor(input_lens, dtype=torch.int64).reshape(-1)
    ol = torch.as_tensor(output_lens, dtype=torch.int64).reshape(-1)
    n = il.numel()
    tok_off = torch.zeros(n, dtype=torch.int64)
    out_off = torch.zeros(n + 1, dtype=torch.int64)
    if n:
        tok_off[1:] = torch.cumsum(il + ol, 0)[:-1]
        out_off[1:] = torch.cumsum(ol, 0)
    total = int(out_off[-1])
    out = torch.empty(total, dtype=torch.int64, device=device)
    if n == 0 or total == 0:
        return out
    if int((il + ol).sum()) >= 2 ** 31:
        raise RuntimeError("fgrpo: packed batch longer than 2^31 tokens")
    pack = torch.cat([tok_off.to(torch.int32), il.to(torch.int32), out_off.to(torch.int32)]).to(device)
    with torch.cuda.device(device):
        rc = lib.fgrpo_output_indices(pack.data_ptr(), pack.data_ptr() + 4 * n, pack.data_ptr() + 8 * n, n,
                                      total, _ptr(out), _stream())
    _lib.check(rc, "output_indices")
    return out


def build_labels(ids: torch.Tensor, input_lens, output_lens) -> torch.Tensor:
    """Labels of a packed batch built on the device: ``ids`` [T] (or [1, T]) int64 on the GPU, sample i made of
    ``input_lens[i]`` prompt tokens and ``output_lens[i]`` generated ones; returns int64 of ``ids``' shape with the
    generated tokens kept and -100 elsewhere (what vllm_worker.py:768-774 builds per sample on the host)."""
    dev = _require_cuda(ids)
    lib = _lib.load()
    flat = ids.reshape(-1).to(torch.int64).contiguous()
    T = flat.numel()
    il = torch.as_tensor(input_lens, dtype=torch.int64).reshape(-1)
    ol = torch.as_tensor(output_lens, dtype=torch.int64).reshape(-1)
    n = il.numel()
    if ol.numel() != n:
        raise RuntimeError("fgrpo: input_lens and output_lens must have one entry per sample")
    if int((il + ol).sum()) != T:
        raise RuntimeError(f"fgrpo: the samples hold {int((il + ol).sum())} tokens, ids has {T}")
    out = torch.empty_like(flat)
    if T == 0 or n == 0:
        return out.view(ids.shape)
    if T >= 2 ** 31:
        raise RuntimeError("fgrpo: packed batch longer than 2^31 tokens")
    tok_off = torch.zeros(n + 1, dtype=torch.int64)
    tok_off[1:] = torch.cumsum(il + ol, 0)
    pack = torch.cat([tok_off, il, ol]).to(torch.int32).to(dev)
    base = pack.data_ptr()
    with torch.cuda.device(dev):
        rc = lib.fgrpo_build_labels(_ptr(flat), base, base + 4 * (n + 1), base + 4 * (2 * n + 1), n, T, _ptr(out), _stream())
    _lib.check(rc, "build_labels")
    return out.view(ids.shape)


def cu_seqlens_from_position_ids(position_ids: torch.Tensor, max_segments: Optional[int] = None) -> torch.Tensor:
    """int32 [n+1]: indices where position_ids == 0, then T (one host sync for n)."""
    dev = _require_cuda(position_ids)
    lib = _lib.load()
    pos = position_ids.reshape(-1).to(torch.int64).contiguous()
    T = pos.numel()
    cap = (max_segments if max_segments is not None else T) + 1
    out = torch.empty(cap, dtype=torch.int32, device=dev)
    cnt = torch.zeros(1, dtype=torch.int32, device=dev)
    if T == 0:
        return torch.zeros(1, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        rc = lib.fgrpo_segment_starts(_ptr(pos), T, _ptr(out), cap, _ptr(cnt), _stream())
    _lib.check(rc, "segment_starts")
    n = int(cnt.item())
    if n > cap:
        raise RuntimeError(f"fgrpo: {n - 1} segments exceed max_segments={cap - 1}")
    return out[:n]


def logits_logprob_entropy(logits: torch.Tensor, labels: Optional[torch.Tensor], ignore_index: Optional[int],
                           want_lp=True, want_ent=True, want_lse=True):
    """Row soft-max statistics of materialised logits [N,V] (bf16/fp32, row stride allowed)."""
    dev = _require_cuda(logits)
    lib = _lib.load()
    code = _code(logits.dtype)
    if logits.dim() != 2 or logits.stride(1) != 1:
        raise RuntimeError("fgrpo: logits must be [N,V] with unit column stride")
    N, V = logits.shape
    mk = lambda: torch.empty(N, dtype=torch.float32, device=dev)
    lp, ent, lse = (mk() if want_lp else None), (mk() if want_ent else None), (mk() if want_lse else None)
    if N == 0:
        return lp, ent, lse
    lab = None if labels is None else labels.reshape(-1).to(torch.int64).contiguous()
    with torch.cuda.device(dev):
        rc = lib.fgrpo_logits_logprob_entropy(_ptr(logits), code, logits.stride(0), N, V, _ptr(lab),
                                              int(ignore_index if ignore_index is not None else 0),
                                              int(ignore_index is not None), _ptr(lp), _ptr(ent), _ptr(lse), _stream())
    _lib.check(rc, "logits_logprob_entropy")
    return lp, ent, lse


def logits_logprob_bwd(logits, labels, ignore_index, g, lse) -> torch.Tensor:
    dev = _require_cuda(logits)
    lib = _lib.load()
    N, V = logits.shape
    out = torch.empty((N, V), dtype=logits.dtype, device=dev)
    if N == 0:
        return out
    lab = labels.reshape(-1).to(torch.int64).contiguous()
    with torch.cuda.device(dev):
        rc = lib.fgrpo_logits_logprob_bwd(_ptr(logits), _code(logits.dtype), logits.stride(0), N, V, _ptr(lab),
                                          int(ignore_index if ignore_index is not None else 0),
                                          int(ignore_index is not None), _ptr(_f32(g, N, "g")), _ptr(_f32(lse, N, "lse")),
                                          _ptr(out), out.stride(0), _stream())
    _lib.check(rc, "logits_logprob_bwd")
    return out


def gemm_nt(A: torch.Tensor, B: torch.Tensor, out_dtype=torch.float32, c_in: Optional[torch.Tensor] = None,
            alpha: float = 1.0, variant: int = 0) -> torch.Tensor:
    """Test hook: C = alpha * A @ B.T (+ c_in); A [M,K], B [N,K] bf16, K % 64 == 0."""
    dev = _require_cuda(A, B)
    lib = _lib.load()
    M, K = A.shape
    N = B.shape[0]
    A = A.contiguous()
    B = B.contiguous()
    out = torch.empty((M, N), dtype=out_dtype, device=dev)
    o32 = _ptr(out) if out_dtype == torch.float32 else None
    o16 = _ptr(out) if out_dtype == torch.bfloat16 else None
    with torch.cuda.device(dev):
        rc = lib.fgrpo_gemm_nt(_ptr(A), _ptr(B), M, N, K, K, K, _ptr(c_in), o32, o16, N, float(alpha), int(variant),
                               _stream())
    _lib.check(rc, "gemm_nt")
    return out


def gemm_kmajor(A: torch.Tensor, B: torch.Tensor, a_kmajor: bool, b_kmajor: bool, M: int, N: int, K: int,
                k_valid: int = 0, out_dtype=torch.float32, c_in: Optional[torch.Tensor] = None,
                alpha: float = 1.0, a_blk: int = 0) -> torch.Tensor:
    """Test hook: C[m,n] = alpha * sum_k A(m,k) B(n,k) (+ c_in) with A given as [K', lda] when ``a_kmajor``
    (else [M, K]) and B likewise; leading dimensions are the tensors' row strides.  ``a_blk`` != 0: A is a
    buffer of 256-column blocks, ``a_blk`` elements apart, each with rows of 256."""
    dev = _require_cuda(A, B)
    lib = _lib.load()
    assert A.stride(-1) == 1 and B.stride(1) == 1
    out = torch.empty((M, N), dtype=out_dtype, device=dev)
    o32 = _ptr(out) if out_dtype == torch.float32 else None
    o16 = _ptr(out) if out_dtype == torch.bfloat16 else None
    lda = 256 if a_blk else A.stride(0)
    with torch.cuda.device(dev):
        rc = lib.fgrpo_gemm_kmajor(_ptr(A), _ptr(B), M, N, K, lda, B.stride(0), int(a_kmajor), int(b_kmajor),
                                   int(a_blk), int(k_valid), _ptr(c_in), o32, o16, N, float(alpha), _stream())
    _lib.check(rc, "gemm_kmajor")
    return out


# --------------------------------------------------------------------------- autograd
# Rows whose shifted label is -100 take no part in the objective: their logprob and entropy are 0 by definition and
# they receive no gradient.  With ``compact`` the projection runs on the other rows only (one host sync to learn how
# many there are), which pays off when prompts make up a sizeable part of the packed batch.
COMPACT_MIN_TOKENS = 2048
COMPACT_MAX_VALID_FRACTION = 0.9


def _valid_rows(labels_shifted: torch.Tensor, compact):
    """Row indices the projection runs on, or None for all rows.  ``compact`` is False, True (find the rows whose
    shifted label is valid: one host sync for their number) or an int64 tensor that already lists them in
    ascending order (no sync; the caller vouches that it holds exactly the positions with a valid label)."""
    T = labels_shifted.numel()
    if torch.is_tensor(compact):
        idx = compact.reshape(-1).to(device=labels_shifted.device, dtype=torch.int64)
        return idx if 0 < idx.numel() < T else None
    if not compact or T < COMPACT_MIN_TOKENS:
        return None
    mask = labels_shifted.reshape(-1) != -100
    n = int(mask.sum())
    if n == 0 or n > COMPACT_MAX_VALID_FRACTION * T:
        return None
    return mask.nonzero(as_tuple=False).squeeze(1)


# How a training step gets its gradients (``keep_logits`` of the calls below; None = the module default
# ``KEEP_LOGITS``).  The choice depends on shapes and on these settings only - never on what else happens to be
# resident on the device - so the same inputs give bit-identical gradients whatever the allocator's state.
#   "chunked"   the whole step inside the forward call, token chunk by token chunk (``grpo_step_chunked``): 6 T H V of
#               matrix work with one chunk of soft-max numerators as the transient; what the reference's chunk loop
#               is for (grpo_loss.py:280-316).  Needs the objective fused with the projection (``fused_grpo_loss``).
#   "auto"      "chunked" where the kernels support the shape, else "recompute"; for ``lmhead_logprob`` alone (whose
#               per-token gradient only arrives with backward()): the whole-batch kept buffer when it takes at most
#               ``KEEP_WHOLE_MAX_BYTES``, else "recompute".
#   True / "whole"   soft-max numerators of the whole batch kept for backward() ([T x V] bf16; raises when unsupported).
#   False / "recompute"   logits recomputed in backward(), one vocabulary panel of dLogits at a time (8 T H V).
KEEP_LOGITS = "auto"
KEEP_WHOLE_MAX_BYTES = 4 << 30
# Token chunk of the chunked step: twice the caller's ``loss_chunksize`` (the reference holds a chunk's logits in bf16
# plus fp32 temporaries of the same shape; the one buffer here is 2 * loss_chunksize * V bf16), else this many tokens;
# never more than ``CHUNK_MAX_BYTES`` of kept numerators.
CHUNK_TOKENS = 8192
CHUNK_MAX_BYTES = 8 << 30


def _grad_mode(keep_logits):
    mode = KEEP_LOGITS if keep_logits is None else keep_logits
    if mode is True or mode == "whole":
        return "whole"
    if mode is False or mode == "recompute":
        return "recompute"
    if mode in ("auto", "chunked"):
        return mode
    raise ValueError(f"fgrpo: keep_logits={mode!r} (expected 'auto', 'chunked', 'whole' / True, 'recompute' / False)")


def chunk_bound_for(V: int, loss_chunksize: Optional[int] = None) -> int:
    """Upper bound on the token chunk of the chunked step (a multiple of 256), from the settings above."""
    bound = 2 * int(loss_chunksize) if (loss_chunksize is not None and loss_chunksize > 0) else CHUNK_TOKENS
    by_bytes = CHUNK_MAX_BYTES // (2 * ((V + 255) // 256 * 256))
    return max(256, min(bound, by_bytes) // 256 * 256)


def chunk_tokens_for(T: int, H: int, V: int, loss_chunksize: Optional[int] = None) -> int:
    """Token chunk the chunked step uses for a packed batch of T tokens: under the bound, either the tokens dealt
    evenly over the chunks the bound needs or whole chunks of the bound and a shorter last one (whole 256-token
    tiles; the library picks by how the tile counts fill the device)."""
    return int(_lib.load().fgrpo_grpo_step_chunk_tokens(int(T), int(H), int(V), chunk_bound_for(V, loss_chunksize)))


def _want_keep(T: int, H: int, V: int, dtype, needs_grad: bool, keep_logits=None) -> bool:
    """Whole-batch kept numerators for a forward whose backward comes later (see ``KEEP_LOGITS``)."""
    mode = _grad_mode(keep_logits)
    if not needs_grad or mode == "recompute" or T == 0:
        return False
    ok = keep_supported(T, H, V, dtype)
    if mode == "whole":
        if not ok:
            raise RuntimeError(f"fgrpo: keep_logits=True but T={T} H={H} V={V} {dtype} is not supported")
        return True
    return ok and mode == "auto" and logits_keep_bytes(T, V) <= KEEP_WHOLE_MAX_BYTES


def _logprob_fwd_rows(hidden, weight, bias, labels_shifted, temperature, idx, needs_grad=False, keep_logits=None):
    """Forward on the rows ``idx`` (or on all rows when idx is None); outputs scattered back into [T] vectors.
    Returns (lp, ent, lse, hidden used, labels used, kept logits | None)."""
    if idx is not None:
        hidden = hidden.index_select(0, idx)
        y = labels_shifted.reshape(-1).index_select(0, idx)
    else:
        y = labels_shifted
    keep = _want_keep(hidden.shape[0], hidden.shape[1], weight.shape[0], weight.dtype, needs_grad, keep_logits)
    res = lmhead_logprob_fwd(hidden, weight, bias, y, temperature, keep=keep)
    lp, ent, lse = res[:3]
    kept = res[3] if keep else None
    if idx is not None:
        T = labels_shifted.numel()
        lp = torch.zeros(T, dtype=torch.float32, device=hidden.device).index_copy_(0, idx, lp)
        ent = torch.zeros(T, dtype=torch.float32, device=hidden.device).index_copy_(0, idx, ent)
    return lp, ent, lse, hidden, y, kept


def panel_elems_bound(T: int, V: int, loss_chunksize: Optional[int]) -> int:
    """Upper bound on the elements of one dLogits panel of the backward, as ``panel_elems_hint``: 0 (the library's
    own bound: a quarter of ``T * V``, between 2**25 and 2**30 elements) unless the caller's ``loss_chunksize``
    rows of logits (what the reference holds per chunk, grpo_loss.py:286-313) are more than that."""
    if loss_chunksize is None or loss_chunksize <= 0:
        return 0
    own = min(max(int(T) * int(V) // 4, 1 << 25), 1 << 30)
    asked = int(loss_chunksize) * int(V)
    return asked if asked > own else 0


def _bwd_rows(h_used, weight, bias, y_used, lse, g_full, gout, temperature, need, panel_hint, idx, hidden_shape,
              kept=None):
    g_used = g_full if idx is None else g_full.reshape(-1).index_select(0, idx)
    if kept is not None:
        # an out-of-range batch is recomputed by the library itself (flag read on the device): no host wait here
        dH, dW, db = lmhead_bwd_kept(h_used, weight, bias, y_used, lse, g_used, gout, temperature, kept, need[0],
                                     need[1], need[2])
    else:
        dH, dW, db = lmhead_bwd(h_used, weight, bias, y_used, lse, g_used, gout, temperature, need[0], need[1],
                                need[2], panel_hint)
    if idx is not None and dH is not None:
        dH = torch.zeros(hidden_shape, dtype=dH.dtype, device=dH.device).index_copy_(0, idx, dH)
    return dH, dW, db


def loss_prepare(labels_shifted, cu_seqlens=None, loss_agg_mode="token_mean", denom_override: float = 0.0):
    """The objective's normalisers from the labels and segments alone: (tokw [T] fp32 | None, pre [4] float64) -
    see ``fgrpo_loss_prepare``."""
    dev = _require_cuda(labels_shifted)
    lib = _lib.load()
    y = labels_shifted.reshape(-1).to(torch.int64).contiguous()
    T = y.numel()
    pre = torch.empty(4, dtype=torch.float64, device=dev)
    if loss_agg_mode == "token_mean":
        agg, tokw, segc, cu, nseq = _lib.AGG_TOKEN_MEAN, None, None, None, 0
    elif loss_agg_mode == "sample_mean":
        if cu_seqlens is None:
            raise RuntimeError("fgrpo: loss_agg_mode='sample_mean' needs cu_seqlens")
        agg = _lib.AGG_SAMPLE_MEAN
        cu = cu_seqlens.to(device=dev, dtype=torch.int32).contiguous()
        nseq = cu.numel() - 1
        tokw = torch.empty(T, dtype=torch.float32, device=dev)
        segc = torch.empty(max(nseq, 1), dtype=torch.int32, device=dev)
    else:
        raise ValueError(f"Invalid loss_agg_mode: {loss_agg_mode}")
    with torch.cuda.device(dev):
        rc = lib.fgrpo_loss_prepare(_ptr(y), _ptr(cu), nseq, T, agg, float(denom_override), _ptr(tokw), _ptr(segc),
                                    _ptr(pre), _stream())
    _lib.check(rc, "loss_prepare")
    return tokw, pre


def chunked_supported(T: int, H: int, V: int, dtype: torch.dtype, chunk_tokens: int) -> bool:
    """Whether the chunked step handles this problem under the chunk bound ``chunk_tokens``: the kept-numerators
    kernels must accept every chunk, the shorter last one included."""
    if dtype != torch.bfloat16 or T <= 0:
        return False
    return bool(_lib.load().fgrpo_grpo_step_chunked_supported(int(T), int(H), int(V), _lib.BF16, int(chunk_tokens)))


def grpo_step_chunked(hidden, weight, bias, labels_shifted, old_lp, ref_lp, adv, tokw, pre, temperature, clip_low,
                      clip_high, clip_ratio_c, kl_beta, chunk_tokens, need_dh=True, need_dw=True, need_db=False,
                      want_diag=True):
    """Projection, logprob, objective and gradients of one packed batch, token chunk by token chunk, in one library
    call (``fgrpo_grpo_step_chunked``): hidden [T,H], weight [V,H] bf16; per-token inputs fp32 [T]; ``tokw`` / ``pre``
    from ``loss_prepare``.  Returns (loss, lp, ent, lse, g, log_ratio, clip1, unclipped, clipped, scal, dH, dW, db):
    the gradients are those of the loss itself (upstream gradient 1)."""
    dev = _require_cuda(hidden, weight, bias, labels_shifted, adv, pre)
    lib = _lib.load()
    T, H = hidden.shape
    V = weight.shape[0]
    code = _code(weight.dtype)
    if hidden.dtype != weight.dtype:
        raise RuntimeError("fgrpo: hidden and weight must share a dtype")
    hidden, weight = _aligned(hidden), _aligned(weight)
    if bias is not None:
        bias = bias.detach().to(weight.dtype).contiguous()
    y = labels_shifted.reshape(-1).to(torch.int64).contiguous()
    old_lp, ref_lp, adv, tokw = _f32(old_lp, T, "old_logprobs"), _f32(ref_lp, T, "ref_logprobs"), \
        _f32(adv, T, "advantages"), _f32(tokw, T, "token weights")
    mk = lambda: torch.empty(T, dtype=torch.float32, device=dev)
    lp, ent, lse, g = mk(), mk(), mk(), mk()
    lr, c1, l1, l2 = (mk(), mk(), mk(), mk()) if want_diag else (None, None, None, None)
    loss = torch.empty((), dtype=torch.float32, device=dev)
    scal = torch.empty(4, dtype=torch.float32, device=dev)
    dH = torch.empty_like(hidden) if need_dh else None
    dW = torch.empty_like(weight) if need_dw else None
    db = torch.empty(V, dtype=weight.dtype, device=dev) if (need_db and bias is not None) else None
    ws = _ws(lib.fgrpo_grpo_step_chunked_workspace(T, H, V, code, int(chunk_tokens)), dev)
    clamp = lambda x: float(max(min(float(x), 3.0e38), -3.0e38))
    with torch.cuda.device(dev):
        rc = lib.fgrpo_grpo_step_chunked(_ptr(hidden), _ptr(weight), _ptr(bias), _ptr(y), _ptr(old_lp), _ptr(ref_lp),
                                         _ptr(adv), _ptr(tokw), _ptr(pre), 1.0 / float(temperature), T, H, V, code,
                                         clamp(clip_low), clamp(clip_high), clamp(clip_ratio_c), clamp(kl_beta),
                                         int(chunk_tokens), _ptr(lp), _ptr(ent), _ptr(lse), _ptr(loss), _ptr(g),
                                         _ptr(lr), _ptr(c1), _ptr(l1), _ptr(l2), _ptr(scal), _ptr(dH), _ptr(dW), _ptr(db),
                                         _ptr(ws), ws.numel(), _stream())
    _lib.check(rc, "grpo_step_chunked")
    return loss, lp, ent, lse, g, lr, c1, l1, l2, scal, dH, dW, db


def scale_inplace(x: Optional[torch.Tensor], scale_dev: torch.Tensor) -> None:
    """x *= scale (a one-element fp32 device tensor) in place; exactly 1 leaves x untouched."""
    if x is None or x.numel() == 0:
        return
    if not x.is_contiguous():
        raise RuntimeError("fgrpo: scale_inplace needs a contiguous tensor")
    with torch.cuda.device(x.device):
        rc = _lib.load().fgrpo_scale_inplace(_ptr(x), x.numel(), _code(x.dtype), _ptr(scale_dev), _stream())
    _lib.check(rc, "scale_inplace")


class _LMHeadLogprob(torch.autograd.Function):
    """(hidden, weight, bias, labels_shifted) -> (lp, entropy); entropy carries no gradient."""

    @staticmethod
    def forward(ctx, hidden, weight, bias, labels_shifted, temperature, panel_hint, compact, keep_logits=None):
        idx = _valid_rows(labels_shifted, compact)
        needs_grad = any(ctx.needs_input_grad[:3])
        if _grad_mode(keep_logits) == "chunked":
            keep_logits = "auto"        # the per-token gradient only arrives with backward(): nothing to chunk here
        lp, ent, lse, h_used, y_used, kept = _logprob_fwd_rows(hidden, weight, bias, labels_shifted, temperature, idx,
                                                               needs_grad, keep_logits)
        ctx.save_for_backward(h_used, weight, bias if bias is not None else hidden.new_empty(0), y_used, lse,
                              idx if idx is not None else hidden.new_empty(0))
        ctx.kept = kept       # released by the first backward (a second backward through this node recomputes)
        ctx.has_bias = bias is not None
        ctx.compacted = idx is not None
        ctx.hidden_shape = tuple(hidden.shape)
        ctx.temperature = temperature
        ctx.panel_hint = panel_hint
        ctx.mark_non_differentiable(ent)
        return lp, ent

    @staticmethod
    def backward(ctx, g_lp, _g_ent):
        h_used, weight, bias, y_used, lse, idx = ctx.saved_tensors
        bias = bias if ctx.has_bias else None
        need = (ctx.needs_input_grad[0], ctx.needs_input_grad[1], ctx.has_bias and ctx.needs_input_grad[2])
        kept, ctx.kept = ctx.kept, None
        dH, dW, db = _bwd_rows(h_used, weight, bias, y_used, lse, g_lp, None, ctx.temperature, need, ctx.panel_hint,
                               idx if ctx.compacted else None, ctx.hidden_shape, kept)
        return dH, dW, db, None, None, None, None, None


class _FusedGRPOLoss(torch.autograd.Function):
    """Projection -> logprob -> dual-clip objective in one autograd node.  The
    backward receives the scalar upstream gradient as a device pointer."""

    @staticmethod
    def forward(ctx, hidden, weight, bias, labels_shifted, old_lp, adv, ref_lp, cu_seqlens, temperature,
                clip_low, clip_high, clip_ratio_c, kl_beta, loss_agg_mode, denom_override, panel_hint, compact,
                keep_logits=None, chunk_tokens=0):
        idx = _valid_rows(labels_shifted, compact)
        need = (ctx.needs_input_grad[0], ctx.needs_input_grad[1], bias is not None and ctx.needs_input_grad[2])
        needs_grad = any(ctx.needs_input_grad[:3])
        T_used = hidden.shape[0] if idx is None else idx.numel()
        H, V = hidden.shape[1], weight.shape[0]
        mode = _grad_mode(keep_logits)
        chunk = int(chunk_tokens) if chunk_tokens and chunk_tokens > 0 else chunk_bound_for(V)   # a bound: the library deals the tokens evenly
        chunked = needs_grad and mode in ("auto", "chunked") and weight.dtype == torch.bfloat16 and \
            hidden.dtype == weight.dtype and chunked_supported(T_used, H, V, weight.dtype, chunk)
        if mode == "chunked" and needs_grad and not chunked:
            raise RuntimeError(f"fgrpo: keep_logits='chunked' but T={T_used} H={H} V={V} {weight.dtype} is not supported")
        ctx.has_bias = bias is not None
        ctx.compacted = idx is not None
        ctx.hidden_shape = tuple(hidden.shape)
        ctx.temperature = temperature
        ctx.panel_hint = panel_hint
        ctx.kept = None
        ctx.grads = None
        if chunked:
            # every gradient is formed here, chunk by chunk, for an upstream gradient of 1; backward() scales them
            tokw, pre = loss_prepare(labels_shifted, cu_seqlens, loss_agg_mode, denom_override)
            y_full = labels_shifted.reshape(-1)
            if idx is None:
                h_used, y_used = hidden, y_full
                sel = lambda t: t
            else:
                h_used, y_used = hidden.index_select(0, idx), y_full.index_select(0, idx)
                sel = lambda t: None if t is None else t.detach().reshape(-1).index_select(0, idx)
            loss, lp, ent, lse, g, lr, c1, l1, l2, _scal, dH, dW, db = grpo_step_chunked(
                h_used, weight, bias, y_used, sel(old_lp), sel(ref_lp), sel(adv), sel(tokw), pre, temperature, clip_low,
                clip_high, clip_ratio_c, kl_beta, chunk, need[0], need[1], need[2], want_diag=idx is None)
            if idx is not None:
                # outputs live on all T positions: scatter, and let the objective kernels write the loss and the
                # diagnostics there (as the other paths do; g, the gradients' source, stays the compacted one)
                T = y_full.numel()
                lp = torch.zeros(T, dtype=torch.float32, device=hidden.device).index_copy_(0, idx, lp)
                ent = torch.zeros(T, dtype=torch.float32, device=hidden.device).index_copy_(0, idx, ent)
                g = torch.zeros(T, dtype=torch.float32, device=hidden.device).index_copy_(0, idx, g)
                loss, _g, lr, c1, l1, l2, _scal = grpo_loss_fwd(lp, old_lp, ref_lp, adv, labels_shifted, cu_seqlens,
                                                                clip_low, clip_high, clip_ratio_c, kl_beta, loss_agg_mode,
                                                                denom_override)
                if dH is not None:
                    dH = torch.zeros(ctx.hidden_shape, dtype=dH.dtype, device=dH.device).index_copy_(0, idx, dH)
            ctx.grads = (dH, dW, db)
        else:
            lp, ent, lse, h_used, y_used, kept = _logprob_fwd_rows(hidden, weight, bias, labels_shifted, temperature, idx,
                                                                   needs_grad, "recompute" if mode == "chunked" else keep_logits)
            ctx.kept = kept       # released by the first backward (a second backward through this node recomputes)
            loss, g, lr, c1, l1, l2, scal = grpo_loss_fwd(lp, old_lp, ref_lp, adv, labels_shifted, cu_seqlens,
                                                          clip_low, clip_high, clip_ratio_c, kl_beta, loss_agg_mode,
                                                          denom_override)
        ctx.save_for_backward(h_used, weight, bias if bias is not None else hidden.new_empty(0), y_used, lse, g,
                              idx if idx is not None else hidden.new_empty(0))
        ctx.mark_non_differentiable(ent, lr, c1, l1, l2, lp)
        return loss, ent, lr, c1, l1, l2, lp

    @staticmethod
    def backward(ctx, g_loss, *_unused):
        grads, ctx.grads = ctx.grads, None
        if grads is not None:
            # the chunked step left the gradients of the loss itself: multiply by the upstream scalar (on the device;
            # exactly 1 costs three empty launches).  A second backward through this node recomputes, below.
            scale = g_loss.detach().reshape(-1)[:1].to(torch.float32).contiguous()
            for t in grads:
                scale_inplace(t, scale)
            return tuple(grads) + (None,) * 16
        h_used, weight, bias, y_used, lse, g, idx = ctx.saved_tensors
        bias = bias if ctx.has_bias else None
        need = (ctx.needs_input_grad[0], ctx.needs_input_grad[1], ctx.has_bias and ctx.needs_input_grad[2])
        kept, ctx.kept = ctx.kept, None
        dH, dW, db = _bwd_rows(h_used, weight, bias, y_used, lse, g, g_loss, ctx.temperature, need, ctx.panel_hint,
                               idx if ctx.compacted else None, ctx.hidden_shape, kept)
        return (dH, dW, db) + (None,) * 16


class _GRPOLossFromLogprobs(torch.autograd.Function):
    """The dual-clip objective on per-token logprobs that some other autograd graph produced
    (the materialised-logits path of a caller-supplied ``per_token_fn``)."""

    @staticmethod
    def forward(ctx, lp, labels_shifted, old_lp, adv, ref_lp, cu_seqlens, clip_low, clip_high, clip_ratio_c, kl_beta,
                loss_agg_mode, denom_override):
        loss, g, lr, c1, l1, l2, scal = grpo_loss_fwd(lp.detach(), old_lp, ref_lp, adv, labels_shifted, cu_seqlens,
                                                      clip_low, clip_high, clip_ratio_c, kl_beta, loss_agg_mode,
                                                      denom_override)
        ctx.save_for_backward(g)
        ctx.lp_dtype = lp.dtype
        ctx.mark_non_differentiable(lr, c1, l1, l2)
        return loss, lr, c1, l1, l2

    @staticmethod
    def backward(ctx, g_loss, *_unused):
        (g,) = ctx.saved_tensors
        return ((g * g_loss).to(ctx.lp_dtype),) + (None,) * 11


def grpo_loss_from_logprobs(lp, labels_shifted, old_lp, adv, ref_lp=None, cu_seqlens=None, clip_low=0.2,
                            clip_high=0.4, clip_ratio_c=1e32, kl_beta=0.0, loss_agg_mode="token_mean",
                            denom_override=0.0):
    """(loss, log_ratio, clip1, unclipped, clipped); the gradient flows into ``lp``."""
    return _GRPOLossFromLogprobs.apply(lp.reshape(-1), labels_shifted, old_lp, adv, ref_lp, cu_seqlens, float(clip_low),
                                       float(clip_high), float(clip_ratio_c), float(kl_beta), loss_agg_mode,
                                       float(denom_override))


def lmhead_logprob(hidden, weight, bias, labels_shifted, temperature=1.0, panel_hint=0,
                   compact=False, keep_logits=None) -> Tuple[torch.Tensor, torch.Tensor]:
    return _LMHeadLogprob.apply(hidden, weight, bias, labels_shifted, float(temperature), int(panel_hint), compact if torch.is_tensor(compact) else bool(compact),
                                keep_logits)


def fused_grpo_loss(hidden, weight, bias, labels_shifted, old_lp, adv, ref_lp=None, cu_seqlens=None,
                    temperature=1.0, clip_low=0.2, clip_high=0.4, clip_ratio_c=1e32, kl_beta=0.0,
                    loss_agg_mode="token_mean", denom_override=0.0, panel_hint=0, compact=False, keep_logits=None,
                    chunk_tokens=0):
    """(loss, entropy, log_ratio, clip1, unclipped, clipped, lp); only loss carries a gradient.
    ``keep_logits``: how the gradients are formed, see ``KEEP_LOGITS`` (None = that module default);
    ``chunk_tokens``: token chunk of the chunked step (0 = ``chunk_tokens_for``)."""
    return _FusedGRPOLoss.apply(hidden, weight, bias, labels_shifted, old_lp, adv, ref_lp, cu_seqlens,
                                float(temperature), float(clip_low), float(clip_high), float(clip_ratio_c),
                                float(kl_beta), loss_agg_mode, float(denom_override), int(panel_hint),
                                compact if torch.is_tensor(compact) else bool(compact), keep_logits, int(chunk_tokens))


# --------------------------------------------------------------------------- packed variable-length attention
def _attn_operand(t: torch.Tensor, name: str) -> torch.Tensor:
    """[T, H, D] bf16 view the kernels can read in place (innermost contiguous, strides multiples of 8
    elements, 16-byte aligned base); anything else is copied once."""
    if t.dim() != 3:
        raise RuntimeError(f"fgrpo: {name} must be [tokens, heads, head_dim], got {tuple(t.shape)}")
    if t.dtype != torch.bfloat16:
        raise RuntimeError(f"fgrpo: {name} must be bf16, got {t.dtype}")
    t = t.detach()
    ok = t.stride(2) == 1 and t.stride(0) % 8 == 0 and t.stride(1) % 8 == 0 and t.stride(0) > 0 and t.stride(1) > 0 \
        and t.data_ptr() % 16 == 0
    return t if ok else _aligned(t)


def attention_bounds_numel(T: int) -> int:
    """int32 elements of the attention kernels' segment scratch for ``T`` packed tokens: start and end of each
    token's segment, then the launch order of the key tiles (128 tokens) and of the query tiles (128, 64, 32)."""
    return 2 * T + 2 * ((T + 127) // 128) + (T + 63) // 64 + (T + 31) // 32


def _attn_bounds(bounds: Optional[torch.Tensor], T: int, dev):
    """(buffer, already filled?) for the int32 segment scratch of the attention kernels."""
    n = attention_bounds_numel(T)
    if bounds is None:
        return torch.empty(n, dtype=torch.int32, device=dev), False
    if bounds.dtype != torch.int32 or bounds.numel() != n or bounds.device != dev or not bounds.is_contiguous():
        raise RuntimeError("fgrpo: bounds does not come from an attention call of this shape")
    return bounds, True


def varlen_attn_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens: torch.Tensor,
                    softmax_scale: Optional[float] = None, causal: bool = True, return_bounds: bool = False,
                    bounds: Optional[torch.Tensor] = None):
    """out [T, Hq, D] bf16 and lse [Hq, T] fp32 of packed self-attention: segment i covers tokens
    cu_seqlens[i]:cu_seqlens[i+1]; query head j reads K/V head j // (Hq // Hkv).  ``return_bounds``: also the int32
    scratch (per-token segment bounds, tile order) that ``varlen_attn_bwd`` - or the next layer's forward, through
    ``bounds`` - can take over instead of rebuilding it (same ``cu_seqlens``, ``T`` and ``causal``)."""
    dev = _require_cuda(q, k, v, cu_seqlens)
    lib = _lib.load()
    q, k, v = _attn_operand(q, "q"), _attn_operand(k, "k"), _attn_operand(v, "v")
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    if k.shape != v.shape or k.shape[0] != T or k.shape[2] != D:
        raise RuntimeError(f"fgrpo: q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)} do not fit together")
    cu = cu_seqlens.to(torch.int32).contiguous()
    scale = float(D) ** -0.5 if softmax_scale is None else float(softmax_scale)
    out = torch.empty((T, Hq, D), dtype=torch.bfloat16, device=dev)
    lse = torch.empty((Hq, T), dtype=torch.float32, device=dev)
    bounds, bounds_valid = _attn_bounds(bounds, T, dev)
    if T == 0:
        return (out, lse, bounds) if return_bounds else (out, lse)
    with torch.cuda.device(dev):
        rc = lib.fgrpo_varlen_attn_fwd(_ptr(q), _ptr(k), _ptr(v), q.stride(0), q.stride(1), k.stride(0), k.stride(1),
                                       v.stride(0), v.stride(1), _ptr(cu), cu.numel() - 1, T, Hq, Hkv, D, scale,
                                       int(bool(causal)), _ptr(out), _ptr(lse), _ptr(bounds), int(bounds_valid), _stream())
    _lib.check(rc, "varlen_attn_fwd")
    return (out, lse, bounds) if return_bounds else (out, lse)


def varlen_attn_bwd(dout: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor,
                    lse: torch.Tensor, cu_seqlens: torch.Tensor, softmax_scale: Optional[float] = None,
                    causal: bool = True, bounds: Optional[torch.Tensor] = None):
    """(dq, dk, dv) bf16, contiguous, for the forward above.  ``bounds``: the scratch the forward returned for the
    same ``cu_seqlens`` and ``causal``."""
    dev = _require_cuda(dout, q, k, v, out, lse, cu_seqlens)
    lib = _lib.load()
    q, k, v = _attn_operand(q, "q"), _attn_operand(k, "k"), _attn_operand(v, "v")
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    if dout.dtype != torch.bfloat16 or tuple(dout.shape) != (T, Hq, D):
        raise RuntimeError(f"fgrpo: dout must be bf16 {(T, Hq, D)}, got {dout.dtype} {tuple(dout.shape)}")
    dout, out = _aligned(dout), _aligned(out)
    lse = lse.detach().to(torch.float32).contiguous()
    cu = cu_seqlens.to(torch.int32).contiguous()
    scale = float(D) ** -0.5 if softmax_scale is None else float(softmax_scale)
    dq = torch.empty((T, Hq, D), dtype=torch.bfloat16, device=dev)
    dk = torch.empty((T, Hkv, D), dtype=torch.bfloat16, device=dev)
    dv = torch.empty((T, Hkv, D), dtype=torch.bfloat16, device=dev)
    if T == 0:
        return dq, dk, dv
    delta = torch.empty((Hq, T), dtype=torch.float32, device=dev)
    bounds, bounds_valid = _attn_bounds(bounds, T, dev)
    with torch.cuda.device(dev):
        rc = lib.fgrpo_varlen_attn_bwd(_ptr(dout), _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), q.stride(0),
                                       q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1), _ptr(cu),
                                       cu.numel() - 1, T, Hq, Hkv, D, scale, int(bool(causal)), _ptr(dq), _ptr(dk),
                                       _ptr(dv), _ptr(delta), _ptr(bounds), int(bounds_valid), _stream())
    _lib.check(rc, "varlen_attn_bwd")
    return dq, dk, dv


class _VarlenAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens, softmax_scale, causal, bounds=None):
        out, lse, bounds = varlen_attn_fwd(q, k, v, cu_seqlens, softmax_scale, causal, return_bounds=True, bounds=bounds)
        ctx.save_for_backward(q, k, v, out, lse, cu_seqlens, bounds)
        ctx.softmax_scale, ctx.causal = softmax_scale, causal
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse, cu, bounds = ctx.saved_tensors
        dq, dk, dv = varlen_attn_bwd(dout.to(torch.bfloat16), q, k, v, out, lse, cu, ctx.softmax_scale, ctx.causal, bounds)
        return dq, dk, dv, None, None, None, None


def varlen_attention(q, k, v, cu_seqlens, softmax_scale=None, causal=True, bounds=None) -> torch.Tensor:
    """Differentiable packed self-attention on the HIP kernels (bf16 in, bf16 out).  ``bounds``: segment scratch of an
    earlier call with the same ``cu_seqlens`` and ``causal`` (see ``attention_bounds``)."""
    return _VarlenAttention.apply(q, k, v, cu_seqlens, softmax_scale, causal, bounds)


def attention_bounds(cu_seqlens: torch.Tensor, T: int, causal: bool = True) -> torch.Tensor:
    """The int32 segment scratch of the attention kernels for one packed batch, built once so that every layer can
    pass it as ``bounds``."""
    dev = _require_cuda(cu_seqlens)
    lib = _lib.load()
    cu = cu_seqlens.to(torch.int32).contiguous()
    bounds, _ = _attn_bounds(None, T, dev)
    if T > 0:
        with torch.cuda.device(dev):
            rc = lib.fgrpo_varlen_attn_bounds(_ptr(cu), cu.numel() - 1, T, int(bool(causal)), _ptr(bounds), _stream())
        _lib.check(rc, "varlen_attn_bounds")
    return bounds

