"""Writes tests/golden/cfg0_oracle_fp64.pt: configuration 0 (fp32 inputs, seed 0)
evaluated by the CPU oracle in float64.  The reference repository ships no golden
vectors for this path; these numbers come from the oracle, which is pinned by
tests/test_oracle_pins.py, and serve as a frozen regression anchor for the GPU
tests.  Run from the repository root:  python tests/golden/make_cfg0_golden.py"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "async-grpo-nccl_amd"))

from oracle import grpo_oracle as O  # noqa: E402
from fgrpo.synthetic import make_workload  # noqa: E402


def main():
    w = make_workload("cfg0", seed=0)
    hs64, W64 = w.hidden.double(), w.weight.double()
    lp0, _ = O.fused_log_probs_and_entropy(W64, None, hs64, w.labels, 1.0)
    old = (lp0 + w.noise_old.double()).float()
    r = w.rewards.numpy()
    go = w.group_offsets.tolist()
    adv = np.concatenate([O.group_advantages(r[a:b], 1e-6) for a, b in zip(go[:-1], go[1:])])
    adv = torch.from_numpy(O.broadcast_values(adv, w.sample_lens)).float()
    hs64.requires_grad_(True)
    W64.requires_grad_(True)
    out = O.grpo_loss_and_entropy(W64, None, hs64, w.labels, 1.0, old.double(), adv.double(), 0.2, 0.2, 1e32)
    out[0].backward()
    gold = dict(hidden=w.hidden, weight=w.weight, labels=w.labels, old=old, adv=adv,
                loss=out[0].detach(), entropy=out[1].detach(), log_ratio=out[2].detach(),
                dH=hs64.grad.float(), dW=W64.grad.float())
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cfg0_oracle_fp64.pt")
    torch.save(gold, path)
    print(path, os.path.getsize(path), "bytes; loss", float(out[0]))


if __name__ == "__main__":
    main()
