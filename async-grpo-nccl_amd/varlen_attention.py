"""Packed variable-length attention for the training / logprob workers, on the HIP kernels of ``libfgrpo``.

Mirrors, for this path, what the reference gets from flash-attn and from its local wrapper
(reference ``gpu_process_worker.py:95-387``):

* ``flash_attn_varlen_func`` - same name, argument order and defaults as the flash-attn function the wrapper
  calls (``gpu_process_worker.py:265-276``); the K/V heads are NOT repeated for grouped-query attention
  (``gpu_process_worker.py:154-161, 209-214``): the kernels index K/V head ``j // (Hq // Hkv)``.
* ``prepare_from_position_ids`` - ``cu_seqlens`` / ``max_seqlen`` from the resets of ``position_ids``
  (``gpu_process_worker.py:239-252``).
* ``varlen_attention_forward`` - the attention callable handed to Transformers (the role of
  ``_fa2_forward_wrapper``, ``gpu_process_worker.py:164-318``), in the attention-interface signature of
  current Transformers.
* ``install_explicit_varlen_wrapper`` - the role of ``_install_explicit_fa2_varlen_wrapper``
  (``gpu_process_worker.py:110``): makes a model use the callable above; returns ``True`` when installed.

There is no fallback: inputs the kernels do not cover (dropout, sliding windows, padding masks, head
dimensions other than 128 and 64, CPU tensors) raise."""
from __future__ import annotations

import weakref
from typing import Optional, Tuple

import torch

from fgrpo import ops

ATTENTION_NAME = "fgrpo_varlen"

# (weak reference to the position_ids tensor, its version counter, result) of the last call
_cu_cache = {"ref": None, "version": None, "value": None}
# segment scratch of the attention kernels for a cu_seqlens tensor: (weak reference, its version counter, causal, buffer)
_bounds_cache = {"ref": None, "version": None, "causal": None, "value": None}


def _bounds_for(cu: torch.Tensor, total: int, causal: bool) -> torch.Tensor:
    """The kernels' int32 segment scratch (per-token segment bounds and tile launch order) for ``cu``: built on the
    first call with a ``cu_seqlens`` tensor OBJECT and reused while that object is alive and unmodified - the
    layers of one forward pass, and their backward passes, share the tensor."""
    ref = _bounds_cache["ref"]
    if ref is not None and ref() is cu and _bounds_cache["version"] == cu._version and \
            _bounds_cache["causal"] == causal and _bounds_cache["value"].numel() == ops.attention_bounds_numel(total):
        return _bounds_cache["value"]
    bounds = ops.attention_bounds(cu, total, causal)
    _bounds_cache.update(ref=weakref.ref(cu), version=cu._version, causal=causal, value=bounds)
    return bounds


def prepare_from_position_ids(position_ids: torch.Tensor) -> Tuple[torch.Tensor, int]:
    """``(cu_seqlens int32 [n+1], max_seqlen)`` for ``position_ids`` of shape ``[B, L]`` (or ``[L]``): a segment
    starts wherever the position is 0 and at the start of every row; the last entry is ``B * L``.  Follows
    reference ``gpu_process_worker.py:239-252``.  The result is remembered for the tensor OBJECT it was computed
    from (weak reference + version counter; an address would be reused by the next batch), so that the layers of
    one forward pass pay for it once."""
    ref = _cu_cache["ref"]
    if ref is not None and ref() is position_ids and _cu_cache["version"] == position_ids._version:
        return _cu_cache["value"]
    pos = position_ids if position_ids.dim() == 2 else position_ids.reshape(1, -1)
    if pos.shape[0] > 1:                       # a row start is a boundary whatever its first position says
        pos = pos.clone()
        pos[:, 0] = 0
    cu = ops.cu_seqlens_from_position_ids(pos.reshape(-1))
    if int(cu[0].item()) != 0:                 # tokens before the first reset form a segment of their own
        cu = torch.cat([torch.zeros(1, dtype=torch.int32, device=cu.device), cu])
    max_seqlen = int((cu[1:] - cu[:-1]).max().item())
    _cu_cache["ref"], _cu_cache["version"], _cu_cache["value"] = weakref.ref(position_ids), position_ids._version, (cu, max_seqlen)
    return cu, max_seqlen


def flash_attn_varlen_func(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q=None, max_seqlen_k=None, dropout_p=0.0,
                           softmax_scale=None, causal=False, window_size=(-1, -1), softcap=0.0, alibi_slopes=None,
                           deterministic=False, return_attn_probs=False, block_table=None):
    """``q`` [total, Hq, D], ``k`` / ``v`` [total, Hkv, D] bf16 -> out [total, Hq, D] bf16 (differentiable).
    Self-attention over packed segments: ``cu_seqlens_q`` and ``cu_seqlens_k`` must describe the same segments,
    as they do at the reference's call site (``gpu_process_worker.py:265-276``).  ``max_seqlen_*`` are accepted
    and not needed."""
    if dropout_p not in (0, 0.0):
        raise RuntimeError("fgrpo varlen attention: dropout is not supported (the reference passes 0.0)")
    if tuple(window_size) != (-1, -1) or softcap not in (0, 0.0) or alibi_slopes is not None or block_table is not None:
        raise RuntimeError("fgrpo varlen attention: window_size / softcap / alibi_slopes / block_table are not supported")
    if return_attn_probs:
        raise RuntimeError("fgrpo varlen attention: attention probabilities are never materialised")
    if cu_seqlens_q is not cu_seqlens_k:
        if cu_seqlens_q.shape != cu_seqlens_k.shape or not torch.equal(cu_seqlens_q, cu_seqlens_k):
            raise RuntimeError("fgrpo varlen attention: queries and keys must share their segments (self-attention)")
    bounds = _bounds_for(cu_seqlens_q, q.shape[0], bool(causal)) if q.is_cuda else None
    return ops.varlen_attention(q, k, v, cu_seqlens_q, softmax_scale, bool(causal), bounds)


def varlen_attention_forward(module, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                             attention_mask: Optional[torch.Tensor] = None, dropout: float = 0.0,
                             scaling: Optional[float] = None, is_causal: Optional[bool] = None,
                             sliding_window: Optional[int] = None, position_ids: Optional[torch.Tensor] = None,
                             **kwargs):
    """Attention callable in the Transformers attention-interface form: ``query`` [B, Hq, L, D], ``key`` /
    ``value`` [B, Hkv, L, D] -> ``(attn_output [B, L, Hq, D], None)``.  Segments come from ``position_ids``
    (every reset to 0 starts one, as in the reference wrapper); without ``position_ids`` every row is one
    segment.  A padding mask is not supported: packed batches carry none (the reference routes only
    ``B == 1`` packed inputs to the varlen kernel)."""
    if dropout not in (0, 0.0):
        raise RuntimeError("fgrpo varlen attention: dropout is not supported")
    B, Hq, L, D = query.shape
    if sliding_window is not None and sliding_window < L:
        raise RuntimeError("fgrpo varlen attention: sliding-window attention is not supported")
    if key.shape[2] != L:
        raise RuntimeError("fgrpo varlen attention: a key/value cache (keys longer than queries) is not supported")
    if attention_mask is not None and attention_mask.dim() == 2 and not bool(attention_mask.all()):
        raise RuntimeError("fgrpo varlen attention: padded batches are not supported; pack the samples instead")
    if is_causal is None:
        is_causal = bool(getattr(module, "is_causal", True))
    if position_ids is not None:
        cu, _ = prepare_from_position_ids(position_ids)
    else:
        cu = torch.arange(0, (B + 1) * L, L, dtype=torch.int32, device=query.device)
    # [B, H, L, D] -> packed [B*L, H, D]; for B == 1 this is a view the kernels read in place
    q = query.transpose(1, 2).reshape(B * L, Hq, D)
    k = key.transpose(1, 2).reshape(B * L, key.shape[1], D)
    v = value.transpose(1, 2).reshape(B * L, value.shape[1], D)
    dt = q.dtype
    if dt != torch.bfloat16:
        q, k, v = q.to(torch.bfloat16), k.to(torch.bfloat16), v.to(torch.bfloat16)
    causal = bool(is_causal)
    bounds = _bounds_for(cu, B * L, causal) if position_ids is not None and q.is_cuda else None
    out = ops.varlen_attention(q, k, v, cu, scaling, causal, bounds)
    return out.view(B, L, Hq, D).to(dt), None


def install_explicit_varlen_wrapper(model=None) -> bool:
    """Registers ``varlen_attention_forward`` with Transformers under the name ``fgrpo_varlen`` and, when a model
    is given, switches that model to it.  Counterpart of the reference's
    ``_install_explicit_fa2_varlen_wrapper(model) -> bool`` (``gpu_process_worker.py:110``), which patches
    Transformers' flash-attention shim; current Transformers offers a registry for the purpose."""
    from transformers import AttentionInterface
    AttentionInterface.register(ATTENTION_NAME, varlen_attention_forward)
    if model is not None:
        seen = set()
        for m in model.modules():
            cfg = getattr(m, "config", None)
            if cfg is not None and id(cfg) not in seen:
                seen.add(id(cfg))
                cfg._attn_implementation = ATTENTION_NAME
    return True
