"""Seeded synthetic workloads for the five benchmark configurations of the fused
logprob + GRPO path.  Data only: hidden states, LM-head weight, packed labels,
segment boundaries, rewards and the logprob perturbations; no arithmetic of the
path itself is done here.

Packing convention: a sample of length n contributes token ids ``ids[0..n-1]``
with labels ``[-100, ids[1], ..., ids[n-1]]`` (prompt length 1), position ids
``0..n-1``; after the next-token shift the first n-1 positions of the segment
are scored and the last is masked.  Samples are concatenated into one row and
the last sample is cut so that the row holds exactly ``tokens`` tokens.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch

CONFIGS: Dict[str, dict] = {
    # fp32 CPU-runnable anchor
    "cfg0": dict(dtype="fp32", H=64, V=1000, prompts=2, group=8, len_lo=16, len_hi=64, len_dist="uniform",
                 tokens=None, w_std=0.02, h_scale=1.0, reward_p=0.5, adv_eps=1e-6, clip_low=0.2, clip_high=0.2,
                 clip_ratio_c=1e32, kl_beta=0.001, chunk=None, forward_only=False),
    # Qwen2.5-1.5B shape (tied embedding)
    "cfg1": dict(dtype="bf16", H=1536, V=151936, prompts=32, group=8, len_lo=128, len_hi=1024, len_dist="uniform",
                 tokens=32768, w_std=0.02, h_scale=None, reward_p=0.3, adv_eps=1e-6, clip_low=0.2, clip_high=0.2,
                 clip_ratio_c=1e32, kl_beta=0.001, chunk=4096, forward_only=False),
    # Qwen2.5-7B shape
    "cfg2": dict(dtype="bf16", H=3584, V=152064, prompts=16, group=16, len_lo=256, len_hi=8192, len_dist="loguniform",
                 tokens=65536, w_std=0.02, h_scale=None, reward_p=0.5, adv_eps=1e-6, clip_low=0.2, clip_high=0.2,
                 clip_ratio_c=1e32, kl_beta=0.04, chunk=8192, forward_only=False),
    # 32B-class reference-logprob forward
    "cfg3": dict(dtype="bf16", H=5120, V=152064, prompts=64, group=1, len_lo=1024, len_hi=4096, len_dist="uniform",
                 tokens=131072, w_std=0.02, h_scale=None, reward_p=0.5, adv_eps=1e-6, clip_low=0.2, clip_high=0.2,
                 clip_ratio_c=1e32, kl_beta=0.0, chunk=None, forward_only=True),
    # 70B-class LM head
    "cfg4": dict(dtype="bf16", H=8192, V=128256, prompts=8, group=4, len_lo=256, len_hi=1024, len_dist="uniform",
                 tokens=16384, w_std=0.02, h_scale=None, reward_p=0.3, adv_eps=1e-6, clip_low=0.2, clip_high=0.2,
                 clip_ratio_c=1e32, kl_beta=0.001, chunk=2048, forward_only=False),
}


@dataclass
class Workload:
    name: str
    T: int
    H: int
    V: int
    dtype: torch.dtype
    hidden: torch.Tensor          # [1, T, H]
    weight: torch.Tensor          # [V, H]
    input_ids: torch.Tensor       # [1, T] int64
    labels: torch.Tensor          # [1, T] int64, unshifted
    position_ids: torch.Tensor    # [1, T] int64
    cu_seqlens: torch.Tensor      # [n+1] int32
    sample_lens: List[int]
    rewards: torch.Tensor         # [n] float64 (per sample)
    group_offsets: torch.Tensor   # [g+1] int32 (samples per prompt group)
    noise_old: torch.Tensor       # [T] fp32, N(0, 0.01): old = lp + noise_old
    noise_ref: torch.Tensor       # [T] fp32, N(0, 0.05): ref = lp + noise_ref
    params: dict = field(default_factory=dict)

    @property
    def n_samples(self) -> int:
        return len(self.sample_lens)


def _sample_lens(cfg: dict, gen: torch.Generator) -> List[int]:
    n = cfg["prompts"] * cfg["group"]
    lo, hi = cfg["len_lo"], cfg["len_hi"]
    if cfg["len_dist"] == "uniform":
        lens = torch.randint(lo, hi + 1, (n,), generator=gen).tolist()
    else:
        u = torch.rand(n, generator=gen, dtype=torch.float64)
        lens = [int(round(math.exp(math.log(lo) + float(x) * (math.log(hi) - math.log(lo))))) for x in u]
    tokens = cfg["tokens"]
    if tokens is None:
        return lens
    # exactly `tokens` tokens: repeat the draw if short, cut the sample that overflows
    out, tot, i = [], 0, 0
    while tot < tokens:
        k = lens[i % n]
        i += 1
        k = min(k, tokens - tot)
        if k < 2 and out:       # a 1-token tail has nothing to score: give it to the previous sample
            out[-1] += k
        else:
            out.append(k)
        tot += k
    return out


def make_workload(name: str, seed: int = 0, device="cpu", overrides: Optional[dict] = None) -> Workload:
    """Build configuration ``name`` ("cfg0".."cfg4").  Small tensors are drawn on the
    CPU generator (identical everywhere); ``hidden`` and ``weight`` are drawn on
    ``device`` (the large configurations would take minutes on a CPU generator)."""
    cfg = dict(CONFIGS[name])
    if overrides:
        cfg.update(overrides)
    gen = torch.Generator().manual_seed(seed)
    lens = _sample_lens(cfg, gen)
    T, H, V = sum(lens), cfg["H"], cfg["V"]
    dtype = torch.float32 if cfg["dtype"] == "fp32" else torch.bfloat16

    ids = torch.randint(0, V, (T,), generator=gen)
    labels = ids.clone()
    pos = torch.empty(T, dtype=torch.long)
    cu = [0]
    for k in lens:
        labels[cu[-1]] = -100
        pos[cu[-1]:cu[-1] + k] = torch.arange(k)
        cu.append(cu[-1] + k)
    n = len(lens)
    rewards = (torch.rand(n, generator=gen) < cfg["reward_p"]).to(torch.float64)
    g = cfg["group"]
    goff = list(range(0, n, g)) + [n]
    noise_old = torch.randn(T, generator=gen) * 0.01
    noise_ref = torch.randn(T, generator=gen) * 0.05

    dgen = torch.Generator(device=device).manual_seed(seed + 1)
    h_scale = cfg["h_scale"] if cfg["h_scale"] is not None else 1.0 / math.sqrt(H)
    hidden = (torch.randn(T, H, generator=dgen, device=device) * h_scale).to(dtype).reshape(1, T, H)
    weight = (torch.randn(V, H, generator=dgen, device=device) * cfg["w_std"]).to(dtype)

    mv = lambda t: t.to(device)
    return Workload(name=name, T=T, H=H, V=V, dtype=dtype, hidden=hidden, weight=weight,
                    input_ids=mv(ids.reshape(1, T)), labels=mv(labels.reshape(1, T)),
                    position_ids=mv(pos.reshape(1, T)), cu_seqlens=mv(torch.tensor(cu, dtype=torch.int32)),
                    sample_lens=lens, rewards=mv(rewards), group_offsets=mv(torch.tensor(goff, dtype=torch.int32)),
                    noise_old=mv(noise_old), noise_ref=mv(noise_ref), params=cfg)
