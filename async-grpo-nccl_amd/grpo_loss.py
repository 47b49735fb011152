"""Drop-in for the reference module ``grpo_loss.py`` (same names, positional
order, keyword names and defaults), with every numeric step executed by the
gfx950 HIP library behind ``fgrpo`` instead of eager torch:

* the LM-head projection, log-softmax, target gather and entropy never
  materialise ``[tokens x vocab]`` logits (reference: grpo_loss.py:211-250,
  :286-313);
* the dual-clip objective, its gradient and the diagnostics are single kernels
  (reference: grpo_loss.py:318-348, :408-498);
* the backward recomputes logits per tile (what autograd derives for
  grpo_loss.py:290-296).

Tensors must be on the GPU; there is no CPU or eager path.  Put this directory
on ``sys.path`` and the reference's import line
``from grpo_loss import compute_dual_clip_grpo_loss, make_grpo_forward``
(gpu_process_worker.py:40) resolves here.

Differences a caller can observe, all documented where they occur:
per-token logprobs are returned in fp32 (the reference returns the logits'
dtype on its un-chunked path); entropy is computed from fp32 logits (the
reference rounds logits to bf16 first, grpo_loss.py:245/:310); a foreign
``per_token_fn`` (a function of logits) takes the chunked materialised-logits route, as in the reference.
Extensions reachable through the ``**unused_kwargs`` hole of the reference
signature: ``ref_logprobs``/``kl_beta`` (k3 KL penalty), ``loss_agg_mode``
(``"token_mean"`` = reference, ``"sample_mean"``), ``cu_seqlens``,
``num_samples_total``, ``compact_masked_tokens`` (project only the rows whose
shifted label is not -100: same results, one host sync, worth it when prompts
are a sizeable part of the packed batch).
"""
from __future__ import annotations

from dataclasses import dataclass
from functools import partial
from typing import Callable, List, Optional, Tuple, Union

import torch

from fgrpo import ops

try:  # the reference derives its outputs from transformers' ModelOutput
    from transformers.modeling_outputs import ModelOutput
except Exception:  # pragma: no cover - transformers is optional for the math
    class ModelOutput(dict):  # minimal stand-in: attribute + key access
        def __post_init__(self):
            for k, v in self.__dict__.items():
                if v is not None:
                    self[k] = v

# The Triton cross-entropy of flash-attn is never used here; the HIP row kernel
# serves both logprob entry points (reference flag: grpo_loss.py:14-18).
_FLASH_ATTN_CE_AVAILABLE = False

DEBUG = False


def debug_print(message):
    return


@dataclass
class GRPOOutput(ModelOutput):
    loss: torch.Tensor = None
    entropy: torch.Tensor = None
    neg_log_ratio: torch.Tensor = None
    loss_clip1: torch.Tensor = None
    loss_unclipped: torch.Tensor = None
    loss_clipped: torch.Tensor = None
    policy_logprobs: torch.Tensor = None


@dataclass
class LogProbsOutput(ModelOutput):
    loss: torch.Tensor = None
    entropy: torch.Tensor = None


# ----------------------------------------------------------------------------
# row kernels on materialised logits (reference: grpo_loss.py:146-208)
# ----------------------------------------------------------------------------
class _RowLogprob(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits2d, labels1d, ignore_index):
        lp, _, lse = ops.logits_logprob_entropy(logits2d, labels1d, ignore_index, want_ent=False)
        ctx.save_for_backward(logits2d, labels1d, lse)
        ctx.ignore_index = ignore_index
        return lp

    @staticmethod
    def backward(ctx, g):
        logits2d, labels1d, lse = ctx.saved_tensors
        return ops.logits_logprob_bwd(logits2d, labels1d, ctx.ignore_index, g, lse), None, None


def _rows(logits: torch.Tensor) -> torch.Tensor:
    flat = logits.reshape(-1, logits.shape[-1])
    return flat if flat.stride(-1) == 1 else flat.contiguous()


def logprobs_from_logits(
    logits: torch.Tensor,
    labels: torch.Tensor,
    ignore_index: int = -100,
    **unused_kwargs,
) -> torch.Tensor:
    """logits[y] - logsumexp(logits) per row, ignored rows 0, in the logits' dtype
    (reference: grpo_loss.py:146-173).  One streaming pass per row on the GPU."""
    lp = _RowLogprob.apply(_rows(logits), labels.reshape(-1), ignore_index)
    return lp.to(logits.dtype).view(labels.shape)


def logprobs_from_logits_flash_attn(
    logits: torch.Tensor,
    labels: torch.Tensor,
    ignore_index: int = -100,
    inplace_backward: bool = True,
    **unused_kwargs,
) -> torch.Tensor:
    """Same quantity in fp32, as the flash-attn cross-entropy route returns it
    (reference: grpo_loss.py:175-201).  ``inplace_backward`` is accepted and
    ignored: the HIP backward writes a fresh dlogits tensor."""
    labels = labels.to(logits.device)
    lp = _RowLogprob.apply(_rows(logits), labels.reshape(-1), ignore_index)
    return lp.view(labels.shape)


def entropy_from_logits(logits: torch.Tensor) -> torch.Tensor:
    """H = logsumexp(x) - sum softmax(x) x per row, no grad
    (reference: grpo_loss.py:203-208)."""
    with torch.no_grad():
        _, ent, _ = ops.logits_logprob_entropy(_rows(logits.detach()), None, None, want_lp=False, want_lse=False)
        return ent.to(logits.dtype).view(logits.shape[:-1])


COMPUTE_ENTROPY_FN = entropy_from_logits

_OWN_PER_TOKEN_FNS = (logprobs_from_logits, logprobs_from_logits_flash_attn)


def _is_own_per_token_fn(per_token_fn) -> bool:
    return per_token_fn is None or per_token_fn in _OWN_PER_TOKEN_FNS


def _materialised_log_probs_and_entropy(w, b, hidden_states, shifted_labels, temperature, per_token_fn, chunk):
    """A caller-supplied ``per_token_fn`` is a function of logits, so for it (and only for it) the logits of one
    chunk of positions at a time are formed, exactly as the reference does (grpo_loss.py:227-249, 286-313):
    ``per_token_fn(logits, shifted_labels, vocab_size=V)`` may return the logprobs or ``(logprobs, logits_flat)``;
    entropy comes from the row kernel on the valid rows.  Gradients reach hidden/weight through torch's own
    autograd of the projection."""
    ops._require_cuda(hidden_states, w, shifted_labels)
    B, L = shifted_labels.shape
    V = w.shape[0]
    hs = hidden_states.to(w.dtype)
    step = int(chunk) if (chunk is not None and chunk > 0) else L
    lps, ents = [], []
    for start in range(0, max(L, 1), max(step, 1)):
        end = min(start + step, L)
        logits = torch.matmul(hs[:, start:end, :], w.t())
        if b is not None:
            logits = logits + b
        logits = logits / temperature
        lab = shifted_labels[:, start:end]
        out = per_token_fn(logits, lab, vocab_size=V)
        if isinstance(out, tuple):
            lp_c, logits_flat = out[0], out[1]
        else:
            lp_c, logits_flat = out, logits.reshape(-1, logits.shape[-1])
        lps.append(lp_c.reshape(B, end - start))
        ent_c = torch.zeros(B * (end - start), device=logits.device, dtype=torch.float32)
        valid = lab.reshape(-1) != -100
        if bool(valid.any()):
            ent_c[valid] = COMPUTE_ENTROPY_FN(logits_flat[valid].detach().bfloat16()).to(ent_c.dtype)
        ents.append(ent_c.reshape(B, end - start))
    return torch.cat(lps, dim=1).reshape(-1), torch.cat(ents, dim=1).reshape(-1)


def _prep(lm_head_weights, lm_head_bias, hidden_states):
    """Flatten to [T, H] and align dtypes the way the reference does
    (``hidden_states.to(lm_head_weights.dtype)``, grpo_loss.py:227); under a bf16
    autocast region fp32 operands are cast to bf16 as torch.matmul would."""
    w = lm_head_weights
    if torch.is_autocast_enabled() and w.dtype == torch.float32:
        try:
            ac = torch.get_autocast_dtype("cuda")
        except Exception:  # older torch
            ac = torch.get_autocast_gpu_dtype()
        if ac == torch.bfloat16:
            w = w.to(torch.bfloat16)
    hs = hidden_states.to(w.dtype)
    b = lm_head_bias
    return w, b, hs.reshape(-1, hs.shape[-1])


# ----------------------------------------------------------------------------
# fused projection + logprob + entropy (reference: grpo_loss.py:211-254)
# ----------------------------------------------------------------------------
def fused_log_probs_and_entropy_fn(
    lm_head_weights: torch.Tensor,
    lm_head_bias: Optional[torch.Tensor],
    hidden_states: torch.Tensor,
    labels: torch.Tensor,
    temperature: float = 1.0,
    per_token_fn: Callable = logprobs_from_logits,
    **unused_kwargs,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """(per-token logprob [B*L] fp32, entropy [B*L] fp32); labels are shifted by
    one inside, masked positions give 0 (reference: grpo_loss.py:211-250)."""
    w, b, hs = _prep(lm_head_weights, lm_head_bias, hidden_states)
    if not _is_own_per_token_fn(per_token_fn):
        return _materialised_log_probs_and_entropy(w, b, hidden_states, ops.shift_labels(labels), temperature,
                                                   per_token_fn, None)
    shifted = ops.shift_labels(labels).reshape(-1)
    lp, ent = ops.lmhead_logprob(hs, w, b, shifted, temperature,
                                 compact=unused_kwargs.get("compact_masked_tokens", False),
                                 keep_logits=unused_kwargs.get("keep_logits", None))
    return lp, ent


ce_loss_and_entropy_logsoftmax = partial(
    fused_log_probs_and_entropy_fn, per_token_fn=logprobs_from_logits
)


# ----------------------------------------------------------------------------
# fused GRPO objective (reference: grpo_loss.py:256-352)
# ----------------------------------------------------------------------------
def grpo_loss_and_entropy_ce_fn(
    lm_head_weights: torch.Tensor,
    lm_head_bias: Optional[torch.Tensor],
    hidden_states: torch.Tensor,
    labels: torch.Tensor,
    temperature: float = 1.0,
    old_logprobs: Optional[torch.Tensor] = None,
    advantages: Optional[torch.Tensor] = None,
    clip_low: float = 0.2,
    clip_high: float = 0.4,
    clip_ratio_c: float = 1e32,
    ce_loss_and_entropy_fn: Callable = ce_loss_and_entropy_logsoftmax,
    per_token_fn: Callable = logprobs_from_logits,
    loss_chunksize: int | None = None,
    **unused_kwargs,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """6-tuple ``(loss, entropy, log_ratio, loss_clip1, loss_unclipped,
    loss_clipped)`` of the dual-clip token-mean objective (reference:
    grpo_loss.py:256-348).  When an input needs a gradient the whole step -
    projection, objective and the gradients - runs here, token chunk by token
    chunk as the reference's loop does (grpo_loss.py:280-316), with one chunk
    of bf16 soft-max numerators as the only ``[. x V]`` transient
    (``2 * loss_chunksize`` tokens, 8192 without one; ``backward()`` then only
    multiplies by the upstream scalar).  The loss, the logprobs and the
    diagnostics do not depend on the chunk size.  ``keep_logits`` among the
    keyword arguments picks another way to the same gradients: ``False`` /
    ``"recompute"`` recomputes the logits in ``backward()``, ``True`` /
    ``"whole"`` keeps the numerators of the whole batch (``[T, V]`` bf16)."""
    if advantages is None:
        raise ValueError("grpo_loss_and_entropy_ce_fn: advantages are required")
    ref_logprobs = unused_kwargs.get("ref_logprobs", None)
    kl_beta = float(unused_kwargs.get("kl_beta", 0.0) or 0.0)
    loss_agg_mode = unused_kwargs.get("loss_agg_mode", "token_mean")
    cu_seqlens = unused_kwargs.get("cu_seqlens", None)
    num_samples_total = unused_kwargs.get("num_samples_total", None)
    compact = unused_kwargs.get("compact_masked_tokens", False)      # True / False, or the int64 row indices themselves

    shifted = ops.shift_labels(labels).reshape(-1)
    w, b, hs = _prep(lm_head_weights, lm_head_bias, hidden_states)
    V = w.shape[0]
    hint = ops.panel_elems_bound(hs.shape[0], V, loss_chunksize)
    denom = float(num_samples_total) if (num_samples_total and loss_agg_mode == "sample_mean") else 0.0
    if not _is_own_per_token_fn(per_token_fn):
        lp, ent = _materialised_log_probs_and_entropy(w, b, hidden_states, ops.shift_labels(labels), temperature,
                                                      per_token_fn, loss_chunksize)
        loss, lr, c1, l1, l2 = ops.grpo_loss_from_logprobs(
            lp, shifted, None if old_logprobs is None else old_logprobs.reshape(-1), advantages.reshape(-1),
            None if ref_logprobs is None else ref_logprobs.reshape(-1), cu_seqlens, clip_low, clip_high,
            clip_ratio_c, kl_beta, loss_agg_mode, denom)
        return loss, ent, lr, c1, l1, l2
    loss, ent, lr, c1, l1, l2, _lp = ops.fused_grpo_loss(
        hs, w, b, shifted,
        None if old_logprobs is None else old_logprobs.reshape(-1),
        advantages.reshape(-1),
        None if ref_logprobs is None else ref_logprobs.reshape(-1),
        cu_seqlens, temperature, clip_low, clip_high, clip_ratio_c, kl_beta,
        loss_agg_mode, denom, hint, compact, unused_kwargs.get("keep_logits", None),
        ops.chunk_bound_for(V, loss_chunksize))
    return loss, ent, lr, c1, l1, l2


grpo_loss_and_entropy_ce_from_logsoftmax = partial(
    grpo_loss_and_entropy_ce_fn, ce_loss_and_entropy_fn=ce_loss_and_entropy_logsoftmax
)


# ----------------------------------------------------------------------------
# model.forward replacement (reference: grpo_loss.py:40-144)
# ----------------------------------------------------------------------------
def make_grpo_forward(model, temperature: float = 1.0, mode: str = 'training', use_torch_compile: bool = True, loss_chunksize: int | None = None):
    """Replace ``model.forward`` by a closure that runs the transformer body
    (``model.model``) and then the fused LM-head path: ``mode='training'`` ->
    ``GRPOOutput``, ``mode='eval'`` -> ``LogProbsOutput`` whose ``loss`` field
    holds the per-token logprobs.  ``use_torch_compile`` is accepted for
    signature compatibility; nothing is traced or compiled."""
    global COMPUTE_ENTROPY_FN
    COMPUTE_ENTROPY_FN = entropy_from_logits

    def _forward(
        input_ids: torch.LongTensor = None,
        attention_mask: Optional[torch.Tensor] = None,
        position_ids: Optional[torch.LongTensor] = None,
        past_key_values=None,
        inputs_embeds: Optional[torch.FloatTensor] = None,
        labels: Optional[torch.LongTensor] = None,
        use_cache: Optional[bool] = None,
        output_attentions: Optional[bool] = None,
        output_hidden_states: Optional[bool] = None,
        return_dict: Optional[bool] = None,
        cache_position: Optional[torch.LongTensor] = None,
        num_logits_to_keep: int = 0,
        old_logprobs: Optional[torch.Tensor] = None,
        advantages: Optional[torch.Tensor] = None,
        clip_low: float = 0.2,
        clip_high: float = 0.4,
        clip_ratio_c: float = 1e32,
        compute_entropy: Optional[bool] = None,
        **kwargs,
    ):
        cfg = model.config
        output_attentions = output_attentions if output_attentions is not None else cfg.output_attentions
        output_hidden_states = output_hidden_states if output_hidden_states is not None else cfg.output_hidden_states
        return_dict = return_dict if return_dict is not None else cfg.use_return_dict
        # objective extensions travel in kwargs but are not for the transformer body
        extra = {k: kwargs.pop(k) for k in ("ref_logprobs", "kl_beta", "loss_agg_mode", "cu_seqlens", "num_samples_total",
                                            "compact_masked_tokens", "keep_logits")
                 if k in kwargs}
        body_out = model.model(
            input_ids=input_ids,
            attention_mask=attention_mask,
            position_ids=position_ids,
            past_key_values=past_key_values,
            inputs_embeds=inputs_embeds,
            use_cache=use_cache,
            output_attentions=output_attentions,
            output_hidden_states=output_hidden_states,
            return_dict=return_dict,
            cache_position=cache_position,
            **kwargs,
        )
        hidden_states = body_out[0]
        head = model.lm_head
        bias = head.bias if hasattr(head, "bias") else None

        if mode == 'training':
            out = grpo_loss_and_entropy_ce_from_logsoftmax(
                lm_head_weights=head.weight,
                lm_head_bias=bias,
                hidden_states=hidden_states,
                labels=labels,
                temperature=temperature,
                old_logprobs=old_logprobs,
                advantages=advantages,
                clip_low=clip_low,
                clip_high=clip_high,
                clip_ratio_c=clip_ratio_c,
                loss_chunksize=loss_chunksize,
                per_token_fn=logprobs_from_logits,
                **extra,
            )
            return GRPOOutput(
                loss=out[0],
                entropy=out[1],
                neg_log_ratio=out[2],
                loss_clip1=out[3],
                loss_unclipped=out[4],
                loss_clipped=out[5],
                policy_logprobs=None,
            )
        elif mode == 'eval':
            out = ce_loss_and_entropy_logsoftmax(
                lm_head_weights=head.weight,
                lm_head_bias=bias,
                hidden_states=hidden_states,
                labels=labels,
                temperature=temperature,
                **{k: v for k, v in extra.items() if k in ("compact_masked_tokens", "keep_logits")},
            )
            return LogProbsOutput(loss=out[0], entropy=out[1])
        else:
            raise ValueError(f"Invalid mode: {mode}")

    model.__original_forward = model.forward
    model.forward = _forward
    return model


# ----------------------------------------------------------------------------
# loss + diagnostics wrapper (reference: grpo_loss.py:355-513)
# ----------------------------------------------------------------------------
def compute_dual_clip_grpo_loss(
    policy_model,
    minibatch,
    clip_low: float,
    clip_high: float,
    clip_ratio_c: float,
    compute_entropy: bool = True,
    apply_entropy_bonus: bool = True,
    entropy_coeff: float = 0.0,
) -> Tuple[torch.Tensor, dict]:
    """Run the patched model on a packed minibatch and return ``(loss, metrics)``
    with the metric keys of the reference (grpo_loss.py:478-498).  All
    diagnostics over ``output_indices`` come from one kernel launch and reach the
    host in one copy instead of ~20 ``.item()`` syncs."""
    batch_ids = minibatch["batch_ids"]
    batch_position_ids = minibatch["batch_position_ids"]
    output_indices = minibatch["output_indices"]
    old_logprobs = minibatch["reference_output_logprobs"]
    advantages = minibatch["advantages"]
    labels = minibatch["labels"]

    # Shapes alone (no sync) tell when prompts are a sizeable part of the batch: output_indices lists exactly the
    # positions whose shifted label is valid (sample_processing_utils.py:29-67).  The LM head then skips the rest.
    extra = {}
    if ops.COMPACT_MIN_TOKENS <= int(labels.numel()) and \
            0 < int(output_indices.numel()) < ops.COMPACT_MAX_VALID_FRACTION * int(labels.numel()):
        # output_indices are the rows themselves when post_process_batch has established, on the host, that they
        # list exactly the positions with a valid next-token label; otherwise the rows are found from the labels
        extra["compact_masked_tokens"] = output_indices if minibatch.get("_labels_are_output_tokens", False) else True
    grpo_output = policy_model(
        input_ids=batch_ids,
        attention_mask=minibatch.get("attention_mask", None),
        position_ids=batch_position_ids,
        labels=labels,
        use_cache=False,
        old_logprobs=old_logprobs,
        advantages=advantages,
        clip_low=clip_low,
        clip_high=clip_high,
        clip_ratio_c=clip_ratio_c,
        compute_entropy=compute_entropy,
        **extra,
    )

    old_entropy = minibatch.get("reference_output_entropies", None)
    if old_entropy is not None and old_entropy.numel() == 0:
        old_entropy = None
    with torch.no_grad():
        stats_dev = ops.grpo_metrics(output_indices, grpo_output.neg_log_ratio, grpo_output.entropy, old_entropy,
                                     advantages, grpo_output.loss_unclipped, grpo_output.loss_clipped,
                                     clip_low, clip_high)
        # the one device-to-host copy of this function: diagnostics, loss value and the batch's sample count
        num_samples_tensor = minibatch.get("num_samples", None)
        tail = [grpo_output.loss.detach().double().reshape(1)]
        if torch.is_tensor(num_samples_tensor):
            tail.append(num_samples_tensor.detach().double().reshape(1).to(stats_dev.device))
        host = torch.cat([stats_dev] + tail).cpu().tolist()
    st, loss_sum = host[:ops._lib.NUM_STATS], float(host[ops._lib.NUM_STATS])
    num_samples = int(host[ops._lib.NUM_STATS + 1]) if len(host) > ops._lib.NUM_STATS + 1 else \
        (int(num_samples_tensor) if num_samples_tensor is not None else 0)
    n = st[0]
    mean = (lambda s: s / n) if n > 0 else (lambda s: 0.0)

    def pop_std(s1, s2):
        if n <= 1:
            return 0.0
        m = s1 / n
        return max(s2 / n - m * m, 0.0) ** 0.5

    expected_out = int(output_indices.numel())

    metrics = {
        "loss": loss_sum,
        "loss_per_token": (loss_sum / max(1, expected_out)) if expected_out > 0 else float(loss_sum),
        "loss_per_sample": (loss_sum / max(1, num_samples)) if num_samples > 0 else float(loss_sum),
        "pg_loss": loss_sum,
        "pg_clip": int(st[13]),
        "kl_div": mean(st[1]),
        "entropy": mean(st[7]),
        "old_policy_entropy": mean(st[8]) if old_entropy is not None else 0.0,
        "entropy_coeff": float(entropy_coeff),
        "approx_kl": mean(st[4]),
        "clipfrac_upper": mean(st[5]),
        "clipfrac_lower": mean(st[6]),
        "log_ratio_mean": mean(st[2]),
        "log_ratio_std": pop_std(st[2], st[3]),
        "adv_mean": mean(st[9]),
        "adv_std": pop_std(st[9], st[10]),
        "adv_pos_frac": mean(st[11]),
        "adv_zero_frac": mean(st[12]),
    }

    final_loss = grpo_output.loss
    if compute_entropy and apply_entropy_bonus and float(entropy_coeff) != 0.0 and n > 0:
        # entropy carries no gradient: the bonus shifts the value only (reference: grpo_loss.py:500-511)
        entropy_mean = (stats_dev[7] / stats_dev[0]).to(final_loss.dtype)
        final_loss = final_loss - float(entropy_coeff) * entropy_mean

    return final_loss, metrics
