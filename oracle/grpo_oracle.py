"""CPU oracle for the fused logprob + GRPO hot path.  TEST INFRASTRUCTURE ONLY.

This module is the checker, never the product: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it.  It restates, in plain eager torch on the CPU (fp32 or fp64, chosen by
the dtype of the inputs), the arithmetic of the reference files cited on every
function.  Nothing in the shipped package imports it.

Pinning status (what checks each function independently of its own formula;
the tests live in ``tests/test_oracle_pins.py``):

* ``logprobs_from_logits``      pinned  (``F.cross_entropy``/``log_softmax`` fp64,
                                          uniform / dominant-logit closed forms,
                                          shift invariance, brute force V<=8)
* ``entropy_from_logits``       pinned  (``torch.distributions.Categorical``,
                                          uniform -> ln V, one-hot limit -> 0, bounds)
* ``fused_log_probs_and_entropy`` pinned (equals the two above on an explicit
                                          matmul; shift/mask invariants)
* ``grpo_loss_and_entropy``     pinned  (REINFORCE closed form, five-region clip
                                          truth table, chunk invariance, all-masked
                                          batch, permutation invariance, gradcheck,
                                          finite differences, manual backward)
* ``grpo_backward_manual``      pinned  (against autograd of the function above)
* ``dual_clip_metrics``         pinned  (hand-computed tiny case)
* ``output_logits_indices`` / ``broadcast_values`` / ``group_advantages`` /
  ``cu_seqlens_from_position_ids`` / ``pack_samples``
                                pinned  (numpy constructions, brute force)
* extensions ``kl_beta``/``ref_logprobs`` and ``loss_agg_mode='sample_mean'``:
  the reference has no code for them; pinned by closed form and brute force
  only -> **parity unpinned by the reference**.
* flash-attn Triton cross entropy (flash-attn 2.7.4.post1, reference
  ``grpo_loss.py:175-201``) is absent here; the reference treats it as
  interchangeable with gather - logsumexp (``grpo_loss.py:157-158``) and this
  oracle restates only the latter -> **parity unpinned** for the Triton kernel's
  own rounding behaviour.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch
import torch.nn.functional as F

IGNORE_INDEX = -100


# ----------------------------------------------------------------------------
# L0 math
# ----------------------------------------------------------------------------
def shift_labels(labels: torch.Tensor) -> torch.Tensor:
    """Next-token shift: position t is scored against labels[t+1]; the last
    position of every row gets -100.  Reference: grpo_loss.py:224 and :278."""
    return F.pad(labels, (0, 1), value=IGNORE_INDEX)[..., 1:].contiguous()


def logprobs_from_logits(logits: torch.Tensor, labels: torch.Tensor,
                         ignore_index: Optional[int] = IGNORE_INDEX) -> torch.Tensor:
    """lp = logits[y] - logsumexp(logits); ignored rows gather index 0 and are
    multiplied by 0.  Reference: grpo_loss.py:146-173 (fallback branch 160-173)."""
    safe = labels.clone()
    if ignore_index is not None:
        safe[safe == ignore_index] = 0
    picked = torch.gather(logits, -1, safe.unsqueeze(-1)).squeeze(-1)
    lp = picked - torch.logsumexp(logits, dim=-1)
    if ignore_index is not None:
        lp = lp * (labels != ignore_index)
    return lp


def entropy_from_logits(logits: torch.Tensor) -> torch.Tensor:
    """H = logsumexp(x) - sum softmax(x) * x, no grad.  Reference:
    grpo_loss.py:203-208.  (The reference feeds bf16-cast logits, :245/:310; the
    oracle keeps the dtype it is given.)"""
    with torch.no_grad():
        p = F.softmax(logits, dim=-1)
        return torch.logsumexp(logits, dim=-1) - (p * logits).sum(-1)


def project(lm_head_weights, lm_head_bias, hidden_states, temperature):
    """logits = hs @ W.T (+ b), then / temperature.  Reference:
    grpo_loss.py:227-230 and :290-293."""
    logits = torch.matmul(hidden_states.to(lm_head_weights.dtype), lm_head_weights.t())
    if lm_head_bias is not None:
        logits = logits + lm_head_bias
    return logits / temperature


def fused_log_probs_and_entropy(lm_head_weights, lm_head_bias, hidden_states, labels,
                                temperature: float = 1.0) -> Tuple[torch.Tensor, torch.Tensor]:
    """(lp_flat, ent_flat): shifted labels, projection, per-token logprob, entropy
    scattered into zeros at masked rows.  Reference: grpo_loss.py:211-250."""
    shifted = shift_labels(labels)
    logits = project(lm_head_weights, lm_head_bias, hidden_states, temperature)
    lp = logprobs_from_logits(logits, shifted)
    V = logits.shape[-1]
    flat = logits.reshape(-1, V)
    mask = shifted.reshape(-1) != IGNORE_INDEX
    ent = torch.zeros(flat.shape[0], dtype=torch.float32 if logits.dtype != torch.float64 else torch.float64)
    if mask.any():
        ent[mask] = entropy_from_logits(flat[mask].detach()).to(ent.dtype)
    return lp.reshape(-1), ent


def segment_ids_from_cu_seqlens(cu_seqlens: torch.Tensor, total: int) -> torch.Tensor:
    cu = cu_seqlens.to(torch.int64)
    lens = cu[1:] - cu[:-1]
    assert int(cu[-1]) == total and int(cu[0]) == 0
    return torch.repeat_interleave(torch.arange(len(lens)), lens)


def grpo_token_terms(lp, old, adv, clip_low, clip_high, clip_ratio_c):
    """Per-token dual-clip terms.  Reference: grpo_loss.py:323-339."""
    log_ratio = lp - old
    ratio = torch.exp(log_ratio)
    unclipped = -adv * ratio
    clipped = -adv * torch.clamp(ratio, 1.0 - clip_low, 1.0 + clip_high)
    clip1 = torch.maximum(unclipped, clipped)
    clip2 = torch.minimum(clip1, -adv * clip_ratio_c)
    tok = torch.where(adv < 0, clip2, clip1)
    return log_ratio, ratio, unclipped, clipped, clip1, tok


def grpo_objective_from_logprobs(lp, shifted_labels, old_logprobs, advantages, clip_low, clip_high, clip_ratio_c,
                                 ref_logprobs=None, kl_beta=0.0, loss_agg_mode="token_mean", cu_seqlens=None,
                                 num_samples_total=None):
    """The tail of the objective on per-token vectors [T] (reference: grpo_loss.py:318-348): ratio, dual clip,
    masked mean; plus the two extensions described in ``grpo_loss_and_entropy``.  ``lp`` may require grad.
    Returns (loss, log_ratio, clip1, unclipped, clipped) - the last four attached to ``lp``'s graph."""
    if old_logprobs is None:
        old_logprobs = lp.detach()
    old = old_logprobs.reshape(-1).to(lp.dtype)
    adv = advantages.reshape(-1).to(lp.dtype)
    log_ratio, ratio, unclipped, clipped, clip1, tok = grpo_token_terms(
        lp, old, adv, clip_low, clip_high, clip_ratio_c)
    if ref_logprobs is not None and kl_beta != 0.0:
        d = ref_logprobs.reshape(-1).to(lp.dtype) - lp
        tok = tok + kl_beta * (torch.exp(d) - d - 1.0)
    mask = shifted_labels.reshape(-1) != IGNORE_INDEX
    vec = torch.where(mask, tok, torch.zeros_like(tok))
    if loss_agg_mode == "token_mean":
        denom = mask.sum().clamp(min=1).to(vec.dtype)
        loss = vec.sum() / denom
    elif loss_agg_mode == "sample_mean":
        assert cu_seqlens is not None
        seg = segment_ids_from_cu_seqlens(cu_seqlens, vec.numel())
        n = int(seg.max()) + 1 if seg.numel() else 0
        cnt = torch.zeros(n, dtype=vec.dtype).index_add_(0, seg, mask.to(vec.dtype))
        sums = torch.zeros(n, dtype=vec.dtype).index_add_(0, seg, vec)
        per = sums / cnt.clamp(min=1)
        N = num_samples_total if num_samples_total is not None else int((cnt > 0).sum())
        loss = per.sum() / max(N, 1)
    else:
        raise ValueError(loss_agg_mode)
    return loss, log_ratio, clip1, unclipped, clipped


def grpo_loss_and_entropy(lm_head_weights, lm_head_bias, hidden_states, labels,
                          temperature: float = 1.0,
                          old_logprobs: Optional[torch.Tensor] = None,
                          advantages: Optional[torch.Tensor] = None,
                          clip_low: float = 0.2, clip_high: float = 0.4,
                          clip_ratio_c: float = 1e32,
                          loss_chunksize: Optional[int] = None,
                          # extensions beyond the reference (default = reference):
                          ref_logprobs: Optional[torch.Tensor] = None,
                          kl_beta: float = 0.0,
                          loss_agg_mode: str = "token_mean",
                          cu_seqlens: Optional[torch.Tensor] = None,
                          num_samples_total: Optional[int] = None):
    """6-tuple (loss, entropy, log_ratio, clip1, unclipped, clipped).
    Reference: grpo_loss.py:256-348 (chunk loop 280-316, tail 318-348).

    Extensions (not in the reference): ``kl_beta * k3(ref, lp)`` added per token,
    k3 = exp(ref-lp) - (ref-lp) - 1; ``loss_agg_mode='sample_mean'`` =
    (1/N) sum_samples (1/n_i) sum_{t in i, valid} tok_t over ``cu_seqlens``
    segments, N = samples with >=1 valid token unless ``num_samples_total``."""
    B, T, _ = hidden_states.shape
    if loss_chunksize is not None and 0 < loss_chunksize < T:
        shifted_full = shift_labels(labels)
        lps, ents = [], []
        for s in range(0, T, loss_chunksize):
            e = min(s + loss_chunksize, T)
            logits = project(lm_head_weights, lm_head_bias, hidden_states[:, s:e, :], temperature)
            sh = shifted_full[:, s:e]
            lps.append(logprobs_from_logits(logits, sh))
            V = logits.shape[-1]
            flat = logits.reshape(-1, V)
            m = sh.reshape(-1) != IGNORE_INDEX
            ent = torch.zeros(flat.shape[0], dtype=torch.float32 if logits.dtype != torch.float64 else torch.float64)
            if m.any():
                ent[m] = entropy_from_logits(flat[m].detach()).to(ent.dtype)
            ents.append(ent.reshape(B, e - s))
        lp = torch.cat(lps, dim=1).reshape(-1)
        entropy = torch.cat(ents, dim=1).reshape(-1)
    else:
        lp, entropy = fused_log_probs_and_entropy(lm_head_weights, lm_head_bias, hidden_states,
                                                  labels, temperature)
    loss, log_ratio, clip1, unclipped, clipped = grpo_objective_from_logprobs(
        lp, shift_labels(labels).reshape(-1), old_logprobs, advantages, clip_low, clip_high, clip_ratio_c,
        ref_logprobs, kl_beta, loss_agg_mode, cu_seqlens, num_samples_total)
    return loss, entropy, log_ratio.detach(), clip1.detach(), unclipped.detach(), clipped.detach()


def grpo_backward_manual(lm_head_weights, lm_head_bias, hidden_states, labels, temperature,
                         old_logprobs, advantages, clip_low, clip_high, clip_ratio_c,
                         ref_logprobs=None, kl_beta=0.0, loss_agg_mode="token_mean",
                         cu_seqlens=None, num_samples_total=None):
    """Closed-form gradients of ``grpo_loss_and_entropy`` (what the autograd of
    grpo_loss.py:256-348 evaluates to away from the measure-zero clip kinks):
      g_t = w_t * ( -A r  if (A>0, r<=1+ch) or (A<0, 1-cl<=r<=c), else 0 )
            + w_t * beta * (1 - exp(ref - lp));  w_t = mask/denom (token_mean)
      dX  = g (onehot(y) - softmax(x)) / temperature ; dH = dX W ; dW = dX^T H.
    Returns (g, dH, dW, dbias)."""
    B, T, H = hidden_states.shape
    shifted = shift_labels(labels).reshape(-1)
    mask = shifted != IGNORE_INDEX
    logits = project(lm_head_weights, lm_head_bias, hidden_states, temperature).reshape(B * T, -1)
    lp = logprobs_from_logits(logits, shifted)
    old = lp if old_logprobs is None else old_logprobs.reshape(-1).to(lp.dtype)
    adv = advantages.reshape(-1).to(lp.dtype)
    r = torch.exp(lp - old)
    pos_ok = (adv > 0) & (r <= 1.0 + clip_high)
    neg_ok = (adv < 0) & (r >= 1.0 - clip_low) & (r <= clip_ratio_c)
    dtok = torch.where(pos_ok | neg_ok, -adv * r, torch.zeros_like(r))
    if ref_logprobs is not None and kl_beta != 0.0:
        d = ref_logprobs.reshape(-1).to(lp.dtype) - lp
        dtok = dtok + kl_beta * (1.0 - torch.exp(d))
    if loss_agg_mode == "token_mean":
        w = mask.to(lp.dtype) / mask.sum().clamp(min=1).to(lp.dtype)
    else:
        seg = segment_ids_from_cu_seqlens(cu_seqlens, mask.numel())
        n = int(seg.max()) + 1
        cnt = torch.zeros(n, dtype=lp.dtype).index_add_(0, seg, mask.to(lp.dtype))
        N = num_samples_total if num_samples_total is not None else int((cnt > 0).sum())
        w = mask.to(lp.dtype) / (cnt.clamp(min=1)[seg] * max(N, 1))
    g = w * dtok
    p = F.softmax(logits, dim=-1)
    onehot = torch.zeros_like(p)
    safe = shifted.clone()
    safe[~mask] = 0
    onehot.scatter_(1, safe.unsqueeze(1), 1.0)
    dX = g.unsqueeze(1) * (onehot - p) / temperature
    dH = (dX @ lm_head_weights).reshape(B, T, H)
    dW = dX.t() @ hidden_states.reshape(B * T, H).to(dX.dtype)
    db = dX.sum(0)
    return g, dH, dW, db


# ----------------------------------------------------------------------------
# metrics wrapper
# ----------------------------------------------------------------------------
def dual_clip_metrics(loss: float, entropy, log_ratio, unclipped, clipped, advantages,
                      output_indices, labels, clip_low, clip_high,
                      old_entropy=None, num_samples: int = 0, entropy_coeff: float = 0.0) -> Dict[str, float]:
    """The metric dictionary of the reference, restated.  Reference:
    grpo_loss.py:408-498 (every metric is evaluated on ``output_indices``)."""
    oi = output_indices
    n = int(oi.numel())
    lr = log_ratio[oi].float()
    r = torch.exp(lr)
    adv = advantages.reshape(-1)[oi].float()
    mean = (lambda x: float(x.mean()) if n > 0 else 0.0)
    std = (lambda x: float(x.std(unbiased=False)) if n > 1 else 0.0)
    return {
        "loss": loss,
        "loss_per_token": (loss / max(1, n)) if n > 0 else float(loss),
        "loss_per_sample": (loss / max(1, num_samples)) if num_samples > 0 else float(loss),
        "pg_loss": loss,
        "pg_clip": float((clipped > unclipped)[oi].sum()),
        "kl_div": mean(lr.abs()),
        "entropy": mean(entropy[oi]),
        "old_policy_entropy": (float(old_entropy[oi].mean()) if old_entropy is not None and old_entropy.numel() > 0 and n > 0 else 0.0),
        "entropy_coeff": float(entropy_coeff),
        "approx_kl": mean(r - 1.0 - lr),
        "clipfrac_upper": mean((r > 1.0 + clip_high).float()),
        "clipfrac_lower": mean((r < 1.0 - clip_low).float()),
        "log_ratio_mean": mean(lr),
        "log_ratio_std": std(lr),
        "adv_mean": mean(adv),
        "adv_std": std(adv),
        "adv_pos_frac": mean((adv > 0).float()),
        "adv_zero_frac": mean((adv == 0).float()),
    }


# ----------------------------------------------------------------------------
# batch shaping (CPU numpy in the reference)
# ----------------------------------------------------------------------------
def output_logits_indices(input_lens: Sequence[int], output_lens: Sequence[int]) -> np.ndarray:
    """Sample i starting at packed offset o_i contributes indices
    o_i + Lin_i - 1 ... o_i + Lin_i + Lout_i - 2.
    Reference: sample_processing_utils.py:29-67."""
    out: List[int] = []
    off = 0
    for li, lo in zip(input_lens, output_lens):
        for j in range(int(lo)):
            out.append(off + int(li) - 1 + j)
        off += int(li) + int(lo)
    return np.asarray(out, dtype=np.int64)


def broadcast_values(values: Sequence[float], lens: Sequence[int]) -> np.ndarray:
    """Each per-sample scalar repeated over that sample's token count, float64.
    Reference: sample_processing_utils.py:69-105."""
    out = np.zeros(int(np.sum(lens)) if len(lens) else 0, dtype=np.float64)
    off = 0
    for v, n in zip(values, lens):
        for j in range(int(n)):
            out[off + j] = v
        off += int(n)
    return out


def group_advantages(rewards: np.ndarray, eps: float = 1e-4) -> np.ndarray:
    """(r - mean) / (population std + eps) over one prompt group, float64.
    Reference: vllm_worker.py:788-796 (identical: :77-92, eps 1e-4)."""
    r = np.asarray(rewards, dtype=np.float64)
    return (r - float(np.mean(r))) / float(np.std(r) + eps)


def cu_seqlens_from_position_ids(position_ids: torch.Tensor) -> torch.Tensor:
    """Segment starts are the indices where position_ids == 0; the total length
    is appended.  int32.  Reference: gpu_process_worker.py:239-252."""
    flat = position_ids.reshape(-1)
    idx = torch.arange(flat.numel(), dtype=torch.int32)
    return torch.cat([idx[flat == 0], torch.tensor([flat.numel()], dtype=torch.int32)])


def make_labels(sample_ids: Sequence[int], input_len: int, output_len: int) -> List[int]:
    """-100 on the prompt, the token id on every generated position.
    Reference: vllm_worker.py:768-774."""
    labels = [IGNORE_INDEX] * len(sample_ids)
    for i in range(output_len):
        labels[input_len + i] = sample_ids[input_len + i]
    return labels


def pack_samples(samples: List[dict]) -> Dict[str, torch.Tensor]:
    """Padding-free packing of a list of sample dicts into 1xT tensors plus the
    per-token broadcasts and counters the trainer consumes.
    Reference: sample_processing_utils.py:159-223 (helpers :107-125)."""
    input_lens = np.array([s["input_len"] for s in samples])
    output_lens = np.array([s["output_len"] for s in samples])
    oi = output_logits_indices(input_lens, output_lens)
    sample_lens = input_lens + output_lens
    adv = broadcast_values(np.array([s["advantage"] for s in samples], dtype=np.float64), sample_lens)
    olb = broadcast_values(output_lens.astype(np.float64), sample_lens)
    cat = lambda key: torch.cat([torch.tensor(s[key], dtype=torch.long) for s in samples]).unsqueeze(0)
    labels = cat("labels")
    ref_lp = torch.cat([torch.tensor(s["sample_logprobs"]) for s in samples]).to(torch.float32)
    ents = []
    for s in samples:
        e = s.get("sample_entropies", None)
        if e is None:
            e = [0.0] * len(s.get("sample_logprobs") or [])
        ents.append(torch.tensor(e))
    mod = [s for s in samples if s.get("modified_reward") is not None]
    non = [s for s in samples if s.get("modified_reward") is None]
    f32 = lambda x: torch.tensor(float(x), dtype=torch.float32)
    return {
        "batch_ids": cat("sample_ids"),
        "batch_position_ids": cat("sample_position_ids"),
        "labels": labels,
        "output_indices": torch.from_numpy(oi),
        "advantages": torch.from_numpy(adv).to(torch.float32),
        "reference_output_logprobs": ref_lp,
        "reference_output_entropies": torch.cat(ents).to(torch.float32),
        "output_lens_broadcasted": torch.from_numpy(olb).to(torch.float32),
        "num_output_tokens_non_masked": (labels != IGNORE_INDEX).sum().to(torch.float32),
        "num_output_tokens": f32(output_lens.sum()),
        "num_samples": f32(len(samples)),
        "max_reward_in_group": f32(0.0),
        "total_modified_reward": f32(sum(s["modified_reward"] for s in mod)) if mod else f32(0.0),
        "total_non_modified_reward": f32(sum(s["reward"] for s in non)) if non else f32(0.0),
        "num_modified_samples": f32(len(mod)),
        "delimiter_not_found": f32(sum(s["delimiter_not_found"] for s in mod)) if mod else f32(0.0),
        "total_reward_rank": f32(sum(s["reward"] for s in samples)),
        "truncated_sample": f32(sum(s["truncated_sample"] for s in samples)),
        "advantage_is_zero": f32(0.0),
    }


def scale_microbatch_loss(loss, num_real_samples: int, train_minibatch_sample_size: int, world: int = 1):
    """loss * n_real / local_target with local_target = max(1, minibatch_target // world) when world > 0 (so an
    unset target of 0 becomes 1 and the loss is scaled by n_real), the plain target when world is 0, and no scaling
    when that leaves 0.  Reference: gpu_process_worker.py:1006-1025."""
    local_target = int(train_minibatch_sample_size or 0)
    if world and world > 0:
        local_target = max(1, local_target // world)
    if local_target <= 0:
        return loss
    scale = float(num_real_samples) / float(local_target)
    return loss * scale if scale != 1.0 else loss


def split_logprobs_per_sample(flat_lp: torch.Tensor, flat_ent: Optional[torch.Tensor], lens: Sequence[int]):
    """Per-sample python lists of floats.  Reference: gpu_process_worker.py:1694-1703."""
    lp = torch.split(flat_lp, list(lens))
    en = torch.split(flat_ent, list(lens)) if flat_ent is not None else [None] * len(lens)
    return [{"logprobs": a.tolist(), "entropies": (b.tolist() if b is not None else None)} for a, b in zip(lp, en)]
