"""Single-GPU harnesses mirroring the two worker methods that drive the hot path
in the reference: ``TrainerGPUWorker.compute_gradients``
(gpu_process_worker.py:963-1050) and
``LogProbGPUWorker.compute_log_probs_from_samples``
(gpu_process_worker.py:1662-1709).  Ray, FSDP and the weight sync around them
are not reproduced; the model is any module patched by
``grpo_loss.make_grpo_forward`` (``prepare_actor_module`` does what the reference does at
load time: attention wrapper, then the forward patch)."""
from __future__ import annotations

from types import SimpleNamespace
from typing import List

import numpy as np
import torch

from grpo_loss import compute_dual_clip_grpo_loss, make_grpo_forward
from sample_processing_utils import PackedLogProbs, _fill, post_process_batch


def prepare_actor_module(model, config=None, mode: str = "training", use_varlen_attention: bool = True):
    """What the reference does to a freshly loaded actor before using it (gpu_process_worker.py:657-693): install the
    packed-attention wrapper when flattened packing is used (``:657-668``), then patch ``forward`` with
    ``make_grpo_forward`` in 'training' or 'eval' mode with the configured temperature and ``loss_chunksize``
    (``:676-693``).  Returns the model."""
    if use_varlen_attention:
        from varlen_attention import install_explicit_varlen_wrapper
        install_explicit_varlen_wrapper(model)
    make_grpo_forward(model, temperature=float(getattr(config, "temperature", 1.0)), mode=mode,
                      use_torch_compile=bool(getattr(config, "use_torch_compile", True)),
                      loss_chunksize=getattr(config, "loss_chunksize", None))
    return model


class TrainerHarness:
    """Forward + backward of one micro-batch with the reference's loss scaling."""

    def __init__(self, model, config=None, device="cuda:0", fsdp_world_size: int = 1):
        self.actor_module_fsdp = model
        self.config = config or SimpleNamespace(clip_low=0.2, clip_high=0.28, clip_ratio_c=3.0,
                                                train_minibatch_sample_size=0, entropy_coeff=0.0)
        self.device = torch.device(device)
        self.fsdp_world_size = fsdp_world_size
        self._mb_count_since_last_step = 0

    def compute_gradients(self, worker_batch: list, total_non_masked_tokens: int = 0) -> dict:
        self.actor_module_fsdp.train()
        batch = post_process_batch(worker_batch, self.device)
        # single GPU: an all-masked batch contributes nothing (gpu_process_worker.py:979-985)
        # (the count is known on the host from packing the labels; the device scalar is only read when it is not)
        n_scored = batch.get("_num_output_tokens_non_masked_host")
        if n_scored is None:
            n_scored = float(batch["num_output_tokens_non_masked"].item())
        if self.fsdp_world_size == 1 and n_scored == 0:
            return {"loss": 0.0, "pg_clip": 0, "kl_div": 0.0, "entropy": 0.0}
        cfg = self.config
        with torch.autocast(device_type="cuda", dtype=torch.bfloat16):
            loss, metrics = compute_dual_clip_grpo_loss(
                self.actor_module_fsdp, batch, cfg.clip_low, cfg.clip_high, cfg.clip_ratio_c,
                compute_entropy=bool(getattr(cfg, "compute_entropy", True)),
                apply_entropy_bonus=bool(getattr(cfg, "apply_entropy_bonus", True)),
                entropy_coeff=float(getattr(cfg, "entropy_coeff", 0.0)))
        # n_real / (minibatch_target // world) before backward (gpu_process_worker.py:1006-1025)
        n_real = sum(1 for s in worker_batch if not s.get("dummy", False))
        target = int(getattr(cfg, "train_minibatch_sample_size", 0) or 0)
        if self.fsdp_world_size and self.fsdp_world_size > 0:
            target = max(1, target // self.fsdp_world_size)          # an unset target of 0 becomes 1, as in the reference
        scale = float(n_real) / float(target) if target > 0 else 1.0
        if scale != 1.0:
            loss = loss * scale
        loss.backward()
        self._mb_count_since_last_step += 1
        return metrics


class LogProbHarness:
    """No-grad per-sample logprobs and entropies of packed samples."""

    def __init__(self, model, device="cuda:0"):
        self.actor_module_fsdp = model
        self.device = torch.device(device)

    @torch.no_grad()
    def compute_log_probs_from_samples(self, samples: list, packed: bool = False):
        """Per-sample logprobs and entropies of ``samples`` (dicts with ``sample_ids`` and ``labels``).
        Default: the reference's result, a list of ``{"logprobs": [float], "entropies": [float] | None}``
        (gpu_process_worker.py:1694-1703).  ``packed=True``: a ``PackedLogProbs`` - one pinned fp32 buffer
        ``[2, T]`` filled by a single device-to-host copy, plus int32 offsets - whose ``to_lists()`` equals the
        default result bit for bit and which ``post_process_batch`` takes without a per-sample loop."""
        self.actor_module_fsdp.eval()
        lens = [len(s["sample_ids"]) for s in samples]
        total = sum(lens)
        host = torch.empty((3, total), dtype=torch.long).pin_memory() if total else torch.empty((3, 0), dtype=torch.long)
        view = host.numpy()
        _fill(view[0], samples, "sample_ids", lens)
        _fill(view[2], samples, "labels", lens, default=-100)
        off = 0
        for k in lens:
            view[1, off:off + k] = np.arange(k)
            off += k
        dev = host.to(self.device, non_blocking=True)
        out = self.actor_module_fsdp(input_ids=dev[0:1], attention_mask=None, position_ids=dev[1:2], labels=dev[2:3])
        # one device->host copy for the whole batch into one pinned buffer
        ent = getattr(out, "entropy", None)
        rows = 2 if ent is not None else 1
        buf = torch.empty((rows, total), dtype=torch.float32).pin_memory() if total else torch.empty((rows, 0), dtype=torch.float32)
        stacked = out.loss.detach().float().reshape(1, -1) if ent is None else \
            torch.stack((out.loss.detach().float().reshape(-1), ent.detach().float().reshape(-1)))
        buf.copy_(stacked, non_blocking=True)
        torch.cuda.current_stream(self.device).synchronize()
        result = PackedLogProbs(buf, np.concatenate(([0], np.cumsum(lens))))
        return result if packed else result.to_lists()
