"""ctypes binding of the C ABI declared in ``include/fgrpo.h``.

The library is loaded from ``csrc/libfgrpo.so`` (built in-tree by
``fgrpo.build``).  There is no fallback: a missing library raises."""
from __future__ import annotations

import ctypes as C
import os

from .build import LIB_PATH

ERR = {-1: "bad argument", -2: "unsupported", -3: "workspace", -4: "HIP error", -5: "alignment"}

BF16, F32 = 0, 1
AGG_TOKEN_MEAN, AGG_SAMPLE_MEAN = 0, 1
NUM_STATS = 16
NUM_PHASES = 5           # FGRPO_NUM_PHASES
STATIC_SCRATCH_BYTES = 8 << 20   # FGRPO_STATIC_SCRATCH_BYTES
METRIC_BLOCKS = 128      # work-groups of the diagnostics' first stage (FGRPO_METRIC_BLOCKS)

_vp, _i, _ll, _f, _d, _sz = C.c_void_p, C.c_int, C.c_longlong, C.c_float, C.c_double, C.c_size_t

# name -> (restype, argtypes); mirrors include/fgrpo.h one to one
SIGNATURES = {
    "fgrpo_version": (_i, []),
    "fgrpo_last_error": (C.c_char_p, []),
    "fgrpo_set_tuning": (_i, [C.c_char_p, _i]),
    "fgrpo_get_tuning": (_i, [C.c_char_p]),
    "fgrpo_logprob_fwd_workspace": (_sz, [_i, _i, _i, _i]),
    "fgrpo_logprob_fwd": (_i, [_vp, _vp, _vp, _vp, _f, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _sz, _vp]),
    "fgrpo_logprob_fwd_static": (_i, [_vp, _vp, _vp, _vp, _f, _i, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "fgrpo_lmhead_bwd_workspace": (_sz, [_i, _i, _i, _i, _ll]),
    "fgrpo_lmhead_bwd_panel_cols": (_i, [_i, _i, _i, _i, _ll]),
    "fgrpo_lmhead_bwd": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _f, _i, _i, _i, _i, _vp, _vp, _vp, _ll, _vp, _sz, _vp]),
    "fgrpo_keep_supported": (_i, [_i, _i, _i, _i]),
    "fgrpo_logits_keep_bytes": (_sz, [_i, _i]),
    "fgrpo_logprob_fwd_keep": (_i, [_vp, _vp, _vp, _vp, _f, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _sz, _vp, _sz, _vp]),
    "fgrpo_keep_overflowed": (_i, [_vp, _i, _i, _vp]),
    "fgrpo_lmhead_bwd_kept_workspace": (_sz, [_i, _i, _i, _i]),
    "fgrpo_lmhead_bwd_kept": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _f, _i, _i, _i, _i, _vp, _sz, _vp, _vp, _vp,
                                   _vp, _sz, _vp]),
    "fgrpo_phase_timing_begin": (_i, []),
    "fgrpo_phase_timing_end": (_i, [_vp, _vp]),
    "fgrpo_loss_fwd_workspace": (_sz, [_i, _i]),
    "fgrpo_loss_fwd": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _f, _f, _f, _f, _i, _d,
                            _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "fgrpo_loss_prepare": (_i, [_vp, _vp, _i, _i, _i, _d, _vp, _vp, _vp, _vp]),
    "fgrpo_grpo_step_chunk_tokens": (_i, [_i, _i, _i, _i]),
    "fgrpo_grpo_step_chunked_supported": (_i, [_i, _i, _i, _i, _i]),
    "fgrpo_grpo_step_chunked_workspace": (_sz, [_i, _i, _i, _i, _i]),
    "fgrpo_grpo_step_chunked": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _f, _i, _i, _i, _i, _f, _f, _f, _f, _i,
                                     _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "fgrpo_scale_inplace": (_i, [_vp, _ll, _i, _vp, _vp]),
    "fgrpo_metrics": (_i, [_vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _f, _f, _vp, _vp, _vp]),
    "fgrpo_group_advantages": (_i, [_vp, _i, _vp, _i, _i, _d, _vp, _vp, _vp]),
    "fgrpo_segment_broadcast": (_i, [_vp, _i, _vp, _i, _i, _vp, _vp]),
    "fgrpo_segment_reduce": (_i, [_vp, _vp, _vp, _i, _i, _vp, _vp, _vp, _vp]),
    "fgrpo_output_indices": (_i, [_vp, _vp, _vp, _i, _i, _vp, _vp]),
    "fgrpo_build_labels": (_i, [_vp, _vp, _vp, _vp, _i, _i, _vp, _vp]),
    "fgrpo_segment_starts": (_i, [_vp, _i, _vp, _i, _vp, _vp]),
    "fgrpo_logits_logprob_entropy": (_i, [_vp, _i, _ll, _i, _i, _vp, _ll, _i, _vp, _vp, _vp, _vp]),
    "fgrpo_logits_logprob_bwd": (_i, [_vp, _i, _ll, _i, _i, _vp, _ll, _i, _vp, _vp, _vp, _ll, _vp]),
    "fgrpo_gemm_nt": (_i, [_vp, _vp, _i, _i, _i, _ll, _ll, _vp, _vp, _vp, _ll, _f, _i, _vp]),
    "fgrpo_gemm_kmajor": (_i, [_vp, _vp, _i, _i, _i, _ll, _ll, _i, _i, _ll, _i, _vp, _vp, _vp, _ll, _f, _vp]),
    "fgrpo_varlen_attn_bounds": (_i, [_vp, _i, _i, _i, _vp, _vp]),
    "fgrpo_varlen_attn_fwd": (_i, [_vp, _vp, _vp, _ll, _ll, _ll, _ll, _ll, _ll, _vp, _i, _i, _i, _i, _i, _f, _i,
                                   _vp, _vp, _vp, _i, _vp]),
    "fgrpo_varlen_attn_bwd": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _ll, _ll, _ll, _ll, _ll, _ll, _vp, _i, _i, _i, _i, _i,
                                   _f, _i, _vp, _vp, _vp, _vp, _vp, _i, _vp]),
}

_lib = None


def load() -> C.CDLL:
    """Load (once) and type the shared library; raise if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"fgrpo: {LIB_PATH} is missing - build it with `python -m fgrpo.build` "
            "(hipcc --offload-arch=gfx950); there is no CPU or eager fallback")
    # torch first: the wheel carries its own HIP runtime, and a process must hold one runtime only.  Loaded before
    # torch, this library would bind the system's runtime while the tensors it is handed live in torch's.
    import torch  # noqa: F401
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().fgrpo_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"fgrpo {what} failed ({ERR.get(rc, rc)}): {msg}")


def set_tuning(**kw) -> None:
    lib = load()
    for k, v in kw.items():
        check(lib.fgrpo_set_tuning(k.encode(), int(v)), f"set_tuning({k})")


def get_tuning(key: str) -> int:
    return load().fgrpo_get_tuning(key.encode())
