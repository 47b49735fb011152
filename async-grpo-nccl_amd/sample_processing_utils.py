"""Drop-in for the batch-shaping functions of the reference module
``sample_processing_utils.py``: a list of sample dicts becomes padding-free
``1 x T`` device tensors plus the per-token broadcasts the trainer consumes.

The reference expands per-sample scalars on the CPU with numba loops and copies
the expanded arrays to the GPU (sample_processing_utils.py:29-105, :159-223).
Here only per-sample arrays and the token lists cross PCIe; the expansion
(``output_indices``, advantage and length broadcasts) runs in HIP kernels over
``cu_seqlens``.  ``device`` must be a GPU: there is no CPU path.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import numpy as np
import torch

from fgrpo import ops


class PackedLogProbs:
    """Wire format of the logprob worker's result: ONE pinned fp32 host buffer ``[2, T]`` (row 0 per-token
    logprobs, row 1 per-token entropies; row 1 is absent, ``[1, T]``, when no entropies were produced) plus int32
    ``offsets [n + 1]`` into it, sample i owning ``offsets[i]:offsets[i+1]``.  The reference ships a Python list of
    floats per sample instead (gpu_process_worker.py:1694-1703), stores the lists on the samples
    (logprob_worker.py:112-121) and re-tensors them in the trainer (sample_processing_utils.py:180-193).
    ``attach`` puts views of the buffer on the samples; ``post_process_batch`` recognises samples that are
    consecutive slices of one buffer and moves them with a single copy, no per-sample loop."""

    def __init__(self, buffer: torch.Tensor, offsets):
        if buffer.dim() != 2 or buffer.shape[0] not in (1, 2) or buffer.dtype != torch.float32 or buffer.is_cuda:
            raise ValueError("PackedLogProbs: buffer must be a host fp32 tensor [1 or 2, T]")
        self.buffer = buffer
        self.offsets = np.ascontiguousarray(np.asarray(offsets, dtype=np.int32))
        if self.offsets.ndim != 1 or self.offsets.size < 1 or int(self.offsets[-1]) != buffer.shape[1] or \
                (np.diff(self.offsets) < 0).any() or int(self.offsets[0]) != 0:
            raise ValueError("PackedLogProbs: offsets must rise from 0 to the buffer's length")

    def __len__(self) -> int:
        return self.offsets.size - 1

    @property
    def has_entropies(self) -> bool:
        return self.buffer.shape[0] == 2

    def sample(self, i: int):
        """(logprobs view, entropies view | None) of sample i, numpy views of the buffer."""
        a, b = int(self.offsets[i]), int(self.offsets[i + 1])
        view = self.buffer.numpy()
        return view[0, a:b], (view[1, a:b] if self.has_entropies else None)

    def to_lists(self) -> List[dict]:
        """The reference's list form (gpu_process_worker.py:1694-1703)."""
        out = []
        for i in range(len(self)):
            lp, ent = self.sample(i)
            out.append({"logprobs": lp.tolist(), "entropies": ent.tolist() if ent is not None else None})
        return out

    def attach(self, samples: list) -> None:
        """What the controller does with the worker's result (logprob_worker.py:112-121), on views: sample i gets
        ``sample_logprobs`` / ``sample_entropies`` and a note of where in which buffer they live."""
        if len(samples) != len(self):
            raise ValueError(f"PackedLogProbs: {len(self)} results for {len(samples)} samples")
        for i, s in enumerate(samples):
            lp, ent = self.sample(i)
            s["sample_logprobs"] = lp
            s["sample_entropies"] = ent
            s["_packed_logprobs"] = (self, i)


def _packed_run(batched_questions):
    """(PackedLogProbs, first, last + 1) when the samples are consecutive entries of one packed result whose views
    they still carry, else None."""
    first = batched_questions[0].get("_packed_logprobs") if batched_questions else None
    if first is None:
        return None
    packed, i0 = first
    for k, s in enumerate(batched_questions):
        ref = s.get("_packed_logprobs")
        if ref is None or ref[0] is not packed or ref[1] != i0 + k:
            return None
        lp = s.get("sample_logprobs")
        a, b = int(packed.offsets[i0 + k]), int(packed.offsets[i0 + k + 1])
        if not isinstance(lp, np.ndarray) or lp.size != b - a or (lp.size and not np.shares_memory(lp, packed.buffer.numpy())):
            return None                           # the field was replaced after attach: take the general route
    return packed, i0, i0 + len(batched_questions)


def _fill(dst: np.ndarray, batched_questions, key: str, lens, default=None) -> None:
    """Writes the per-token values ``s[key]`` of every sample into consecutive pieces of ``dst`` (a numpy view of
    the staging buffer).  Python lists go through ``np.fromiter`` (about half the cost of ``torch.as_tensor`` per
    element, and this conversion is most of the time of packing a batch); arrays and tensors are copied."""
    off = 0
    for s, k in zip(batched_questions, lens):
        x = s.get(key, None)
        if x is None:
            dst[off:off + k] = default
        elif isinstance(x, (list, tuple)):
            if len(x) != k:
                raise ValueError(f"sample field {key!r} has {len(x)} entries for {k} tokens")
            dst[off:off + k] = np.fromiter(x, dtype=dst.dtype, count=k)
        else:
            dst[off:off + k] = np.asarray(x.cpu() if torch.is_tensor(x) else x).reshape(-1)
        off += k


def _lens(batched_questions):
    il = np.fromiter((s["input_len"] for s in batched_questions), dtype=np.int64, count=len(batched_questions))
    ol = np.fromiter((s["output_len"] for s in batched_questions), dtype=np.int64, count=len(batched_questions))
    return il, ol


def get_output_logits_indices_numba(input_lens, output_lens):
    """Host reference form kept for callers that want a numpy array
    (reference: sample_processing_utils.py:29-67), vectorised: sample i starting
    at offset o_i yields o_i + Lin_i - 1 + [0, Lout_i)."""
    il = np.asarray(input_lens, dtype=np.int64)
    ol = np.asarray(output_lens, dtype=np.int64)
    start = np.concatenate(([0], np.cumsum(il + ol)[:-1])) + il - 1 if il.size else np.zeros(0, np.int64)
    first = np.repeat(start, ol)
    within = np.arange(int(ol.sum()), dtype=np.int64) - np.repeat(np.cumsum(ol) - ol, ol)
    return (first + within).astype(np.int64)


def broadcast_values(values, output_lens):
    """float64 repeat of per-sample scalars (reference: sample_processing_utils.py:69-105)."""
    return np.repeat(np.asarray(values, dtype=np.float64), np.asarray(output_lens, dtype=np.int64))


def get_output_logits_indices(batched_questions, device):
    """(output_indices on device, output_lens) - reference: sample_processing_utils.py:107-112."""
    il, ol = _lens(batched_questions)
    return ops.output_indices(il, ol, device), ol


def get_input_for_logprobs(batched_questions, output_indices, device, info=None):
    """Concatenated ids / position ids / labels as [1, T] int64 device tensors
    (reference: sample_processing_utils.py:114-125).  One pinned staging buffer,
    one copy.  Samples that carry no ``labels`` get them built on the device from
    ``input_len`` / ``output_len`` (the rule of vllm_worker.py:768-774).
    ``info`` (a dict, optional) receives what is known on the host while the labels
    are packed: ``num_scored`` (labelled tokens) and ``labels_are_output_tokens``
    (True when the positions whose next-token label is valid are exactly the
    output positions of (input_len, output_len) - by construction when the labels
    are built from those lengths, otherwise checked here on the host copy)."""
    lens = [len(s["sample_ids"]) for s in batched_questions]
    n_tok = sum(lens)
    have_labels = all("labels" in s for s in batched_questions)
    rows = 3 if have_labels else 2
    host = torch.empty((rows, n_tok), dtype=torch.long).pin_memory() if n_tok else torch.empty((rows, 0), dtype=torch.long)
    view = host.numpy()
    _fill(view[0], batched_questions, "sample_ids", lens)
    _fill(view[1], batched_questions, "sample_position_ids", lens)
    if have_labels:
        _fill(view[2], batched_questions, "labels", lens)
        if info is not None:
            info["num_scored"] = int(np.count_nonzero(view[2] != -100))
            same = False
            if all("input_len" in s and "output_len" in s for s in batched_questions):
                il, ol = _lens(batched_questions)
                # position t is scored when the label of token t + 1 is valid (the last position never is)
                same = int((il + ol).sum()) == n_tok and \
                    np.array_equal(np.flatnonzero(view[2][1:] != -100), get_output_logits_indices_numba(il, ol))
            info["labels_are_output_tokens"] = bool(same)
    dev = host.to(device, non_blocking=True)
    if have_labels:
        return dev[0:1], dev[1:2], dev[2:3]
    il, ol = _lens(batched_questions)
    if info is not None:
        info["num_scored"] = int(ol.sum())
        info["labels_are_output_tokens"] = True
    return dev[0:1], dev[1:2], ops.build_labels(dev[0:1], il, ol)


# scalar counters of a packed batch (fp32 device scalars), in the reference's key order
_COUNTER_KEYS = ("num_output_tokens_non_masked", "num_output_tokens", "num_samples", "max_reward_in_group",
                 "total_modified_reward", "total_non_modified_reward", "num_modified_samples", "delimiter_not_found",
                 "total_reward_rank", "truncated_sample", "advantage_is_zero")


def make_dummy_batch(batched_questions, device):
    """All-masked 4-token placeholder that keeps lock-step ranks busy without
    touching the metrics (reference: sample_processing_utils.py:127-157): every
    label is -100, there are no output positions, every counter is zero."""
    n = 4
    batch = {key: torch.zeros((), device=device, dtype=torch.float32) for key in _COUNTER_KEYS}
    for key in ("advantages", "reference_output_logprobs", "output_lens_broadcasted"):
        batch[key] = torch.zeros(n, device=device, dtype=torch.float32)
    batch["batch_ids"] = torch.arange(11, 11 + n, dtype=torch.long, device=device).unsqueeze(0)
    batch["batch_position_ids"] = torch.arange(n, device=device).unsqueeze(0)
    batch["labels"] = torch.full((1, n), -100, dtype=torch.long, device=device)
    batch["output_indices"] = torch.empty((0,), dtype=torch.long, device=device)
    batch["samples"] = batched_questions
    return batch


def post_process_batch(batched_questions, device, constant_length_samples=None):
    """Pack samples for the trainer; same keys, dtypes and shapes as the
    reference (sample_processing_utils.py:159-223)."""
    if len(batched_questions) == 1 and batched_questions[0].get('dummy', False):
        return make_dummy_batch(batched_questions, device)

    il, ol = _lens(batched_questions)
    sample_lens = il + ol
    total = int(sample_lens.sum())
    cu = torch.from_numpy(np.concatenate(([0], np.cumsum(sample_lens))).astype(np.int32)).to(device)
    output_indices = ops.output_indices(il, ol, device)

    per_sample = torch.tensor([[float(s["advantage"]) for s in batched_questions], ol.astype(np.float64).tolist()],
                              dtype=torch.float64).to(device)
    advantages = ops.segment_broadcast(per_sample[0], cu, total)
    if constant_length_samples is None:
        output_lens_broadcasted = ops.segment_broadcast(per_sample[1], cu, total)
    else:
        output_lens_broadcasted = torch.full((total,), float(constant_length_samples), device=device, dtype=torch.float32)

    # old-policy logprobs and entropies (zeros where a sample carries none)
    run = _packed_run(batched_questions)
    if run is not None:
        # consecutive slices of one pinned result buffer: one copy of the column range, no per-sample work
        packed, i0, i1 = run
        a, b = int(packed.offsets[i0]), int(packed.offsets[i1])
        stage_dev = packed.buffer[:, a:b].to(device, non_blocking=True)
        reference_output_logprobs = stage_dev[0]
        reference_output_entropies = stage_dev[1] if packed.has_entropies else torch.zeros_like(stage_dev[0])
    else:
        # lists (the reference's form) or loose arrays: one pinned staging buffer, one copy
        lp_lens = [len(s["sample_logprobs"]) for s in batched_questions]
        n_lp = sum(lp_lens)
        stage = torch.empty((2, n_lp), dtype=torch.float32).pin_memory() if n_lp else torch.empty((2, 0), dtype=torch.float32)
        sv = stage.numpy()
        _fill(sv[0], batched_questions, "sample_logprobs", lp_lens)
        _fill(sv[1], batched_questions, "sample_entropies", lp_lens, default=0.0)
        stage_dev = stage.to(device, non_blocking=True)
        reference_output_logprobs, reference_output_entropies = stage_dev[0], stage_dev[1]

    label_info = {}
    batch_ids, batch_position_ids, labels = get_input_for_logprobs(batched_questions, output_indices, device, label_info)

    modified = [q for q in batched_questions if q['modified_reward'] is not None]
    plain = [q for q in batched_questions if q['modified_reward'] is None]
    # the scalar counters travel as one vector (one copy instead of eleven)
    counters = {
        "num_output_tokens": float(ol.sum()),
        "num_samples": float(len(batched_questions)),
        "max_reward_in_group": 0.0,
        "total_modified_reward": float(sum(s['modified_reward'] for s in modified)) if modified else 0.0,
        "total_non_modified_reward": float(sum(s['reward'] for s in plain)) if plain else 0.0,
        "num_modified_samples": float(len(modified)),
        "delimiter_not_found": float(sum(s['delimiter_not_found'] for s in modified)) if modified else 0.0,
        "total_reward_rank": float(sum(s['reward'] for s in batched_questions)),
        "truncated_sample": float(sum(s['truncated_sample'] for s in batched_questions)),
        "advantage_is_zero": 0.0,
    }
    counter_vec = torch.tensor(list(counters.values()), dtype=torch.float32).to(device)
    out = {
        "batch_ids": batch_ids.contiguous(),
        "batch_position_ids": batch_position_ids.contiguous(),
        "output_indices": output_indices.contiguous(),
        "advantages": advantages.contiguous(),
        "reference_output_logprobs": reference_output_logprobs.contiguous(),
        "reference_output_entropies": reference_output_entropies.contiguous(),
        "output_lens_broadcasted": output_lens_broadcasted.contiguous(),
        "num_output_tokens_non_masked": (labels != -100).sum().to(torch.float32),
        "samples": batched_questions,
        "labels": labels.contiguous(),
        # not in the reference: segment boundaries, so that the loss can aggregate per sample
        "cu_seqlens": cu,
        # not in the reference: the labelled-token count as a host integer (known while the labels are packed), so
        # that the trainer's all-masked check needs no device read
        "_num_output_tokens_non_masked_host": float(label_info["num_scored"]),
        # not in the reference: whether output_indices lists exactly the positions with a valid next-token label
        # (then the loss may hand them to the LM head as its row list without looking at the labels again)
        "_labels_are_output_tokens": bool(label_info["labels_are_output_tokens"]),
    }
    for k, key in enumerate(counters):
        out[key] = counter_vec[k]
    try:
        out["uids"] = torch.tensor([int(s.get("__uid__", -1)) for s in batched_questions], device=device)
    except Exception:
        pass
    return out


def normalize_rewards(rewards, eps: float = 1e-4, group_size: Optional[int] = None):
    """Group-normalised advantages on the GPU: (r - mean) / (population std + eps)
    (reference: vllm_worker.py:77-92 and :788-796).  ``rewards`` is one group, or
    several groups of ``group_size`` laid end to end; returns float64 numpy."""
    r = torch.as_tensor(np.asarray(rewards, dtype=np.float64))
    n = r.numel()
    gs = n if group_size is None else int(group_size)
    if gs <= 0 or n % gs:
        raise ValueError("normalize_rewards: group_size must divide the number of rewards")
    goff = torch.arange(0, n + 1, gs, dtype=torch.int32)
    out = ops.group_advantages(r.cuda(), goff.cuda(), eps, torch.float64)
    return out.cpu().numpy()
