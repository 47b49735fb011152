"""Pins of the CPU oracle (oracle/grpo_oracle.py) against facts that do not come
from the oracle's own formulas: torch library routines in fp64, closed forms,
brute force on tiny inputs, invariants, autograd gradcheck and finite
differences.  The reference repository holds no tests, fixtures or golden
vectors for this path, so these are what a wrong sign, index or dropped term
in the restatement would trip over."""
import itertools
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import grpo_oracle as O

torch.manual_seed(0)
D = torch.float64


# ------------------------------------------------------------------ logprob / entropy
def test_logprob_equals_library_cross_entropy():
    x = torch.randn(37, 91, dtype=D) * 3
    y = torch.randint(0, 91, (37,))
    y[::5] = -100
    got = O.logprobs_from_logits(x, y)
    want = -F.cross_entropy(x, y, reduction="none", ignore_index=-100)
    assert torch.allclose(got, want, atol=1e-12)
    want2 = torch.log_softmax(x, -1).gather(1, y.clamp(min=0)[:, None])[:, 0] * (y != -100)
    assert torch.allclose(got, want2, atol=1e-12)
    assert (got[::5] == 0).all()


def test_logprob_closed_forms_and_shift_invariance():
    V = 50
    y = torch.tensor([3, 7])
    assert torch.allclose(O.logprobs_from_logits(torch.full((2, V), 1.7, dtype=D), y), torch.full((2,), -math.log(V), dtype=D))
    x = torch.zeros(2, V, dtype=D)
    x[0, 3] = 80.0
    x[1, 7] = 80.0
    assert O.logprobs_from_logits(x, y).abs().max() < 1e-12          # dominant target -> 0
    x2 = torch.randn(2, V, dtype=D)
    assert torch.allclose(O.logprobs_from_logits(x2, y), O.logprobs_from_logits(x2 + 123.25, y), atol=1e-10)


def test_logprob_brute_force_tiny_vocab():
    x = torch.tensor([[0.3, -1.2, 2.0, 0.0]], dtype=D)
    for k in range(4):
        den = sum(math.exp(v) for v in x[0].tolist())
        want = math.log(math.exp(x[0, k].item()) / den)
        assert abs(O.logprobs_from_logits(x, torch.tensor([k])).item() - want) < 1e-12


def test_entropy_equals_library_and_limits():
    x = torch.randn(23, 67, dtype=D) * 2
    want = torch.distributions.Categorical(logits=x).entropy()
    got = O.entropy_from_logits(x)
    assert torch.allclose(got, want, atol=1e-12)
    assert torch.allclose(O.entropy_from_logits(torch.zeros(3, 67, dtype=D)), torch.full((3,), math.log(67), dtype=D))
    onehot = torch.zeros(1, 67, dtype=D)
    onehot[0, 5] = 200.0
    assert O.entropy_from_logits(onehot).abs().item() < 1e-9
    assert (got >= 0).all() and (got <= math.log(67) + 1e-12).all()


def _toy(B=1, T=29, H=8, V=17, seed=0, dtype=D, bias=True):
    g = torch.Generator().manual_seed(seed)
    hs = torch.randn(B, T, H, generator=g, dtype=dtype)
    W = torch.randn(V, H, generator=g, dtype=dtype) * 0.5
    b = torch.randn(V, generator=g, dtype=dtype) * 0.1 if bias else None
    labels = torch.randint(0, V, (B, T), generator=g)
    labels[:, :3] = -100
    labels[:, 11] = -100
    return hs, W, b, labels


def test_fused_logprob_entropy_is_composition_with_shift():
    hs, W, b, labels = _toy(B=2)
    lp, ent = O.fused_log_probs_and_entropy(W, b, hs, labels, temperature=0.7)
    x = (hs @ W.t() + b) / 0.7
    T = labels.shape[1]
    for bi in range(2):
        for t in range(T):
            k = bi * T + t
            nxt = labels[bi, t + 1].item() if t + 1 < T else -100
            if nxt == -100:
                assert lp[k] == 0 and ent[k] == 0
            else:
                want = torch.log_softmax(x[bi, t], -1)[nxt]
                assert abs(lp[k] - want) < 1e-12
                assert abs(ent[k] - torch.distributions.Categorical(logits=x[bi, t]).entropy()) < 1e-12
    # the last position of every row is masked by the shift
    assert lp[T - 1] == 0 and lp[2 * T - 1] == 0
    # masked rows do not depend on the hidden state there
    hs2 = hs.clone()
    hs2[:, 10] += 5.0            # labels[:, 11] == -100 -> position 10 is masked after the shift
    lp2, _ = O.fused_log_probs_and_entropy(W, b, hs2, labels, temperature=0.7)
    assert torch.equal(lp2[[10, T + 10]], lp[[10, T + 10]])


# ------------------------------------------------------------------ GRPO objective
def test_clip_truth_table():
    """Five regions at cl = ch = 0.2, c = 3: (A, log ratio) -> (token loss, d tok / d lp)."""
    table = [(+1.0, 0.0, -1.0, -1.0), (-1.0, 0.0, 1.0, 1.0), (+1.0, 0.5, -1.2, 0.0),
             (-1.0, -0.5, 0.8, 0.0), (-1.0, 2.0, 3.0, 0.0)]
    for A, lr, want_tok, want_grad in table:
        lp = torch.tensor([lr], dtype=D, requires_grad=True)
        *_, tok = O.grpo_token_terms(lp, torch.zeros(1, dtype=D), torch.tensor([A], dtype=D), 0.2, 0.2, 3.0)
        tok.sum().backward()
        assert abs(tok.item() - want_tok) < 1e-12, (A, lr)
        assert abs(lp.grad.item() - want_grad) < 1e-12, (A, lr)


def test_reinforce_closed_form_when_old_is_none():
    hs, W, b, labels = _toy()
    adv = torch.randn(labels.numel(), dtype=D)
    hs.requires_grad_(True)
    out = O.grpo_loss_and_entropy(W, b, hs, labels, 1.0, None, adv, 0.2, 0.4, 1e32)
    mask = O.shift_labels(labels).reshape(-1) != -100
    assert abs(out[0].item() - (-(adv[mask]).mean().item())) < 1e-12
    assert torch.count_nonzero(out[2]) == 0          # log ratio identically 0
    g, dH, dW, db = O.grpo_backward_manual(W, b, hs.detach(), labels, 1.0, None, adv, 0.2, 0.4, 1e32)
    assert torch.allclose(g, -adv * mask / mask.sum(), atol=1e-14)
    out[0].backward()
    assert torch.allclose(hs.grad, dH, atol=1e-12)


@pytest.mark.parametrize("chunk", [1, 4, 7, 28, 29, 1000])
def test_chunk_invariance(chunk):
    hs, W, b, labels = _toy()
    adv = torch.randn(labels.numel(), dtype=D)
    old = torch.randn(labels.numel(), dtype=D) * 0.3 - 2.5
    a = O.grpo_loss_and_entropy(W, b, hs, labels, 0.9, old, adv, 0.2, 0.28, 3.0, loss_chunksize=None)
    c = O.grpo_loss_and_entropy(W, b, hs, labels, 0.9, old, adv, 0.2, 0.28, 3.0, loss_chunksize=chunk)
    for x, y in zip(a, c):
        assert torch.allclose(x, y, atol=1e-12)


def test_all_masked_batch_gives_zero_loss_and_grads():
    hs, W, b, labels = _toy()
    labels[:] = -100
    hs.requires_grad_(True)
    W.requires_grad_(True)
    out = O.grpo_loss_and_entropy(W, b, hs, labels, 1.0, torch.zeros(labels.numel(), dtype=D),
                                  torch.zeros(labels.numel(), dtype=D), 0.2, 0.4, 1e32)
    out[0].backward()
    assert out[0].item() == 0 and torch.isfinite(out[0])
    assert hs.grad.abs().max() == 0 and W.grad.abs().max() == 0
    assert out[1].abs().max() == 0


def test_sample_permutation_leaves_token_mean_unchanged():
    H, V = 8, 17
    g = torch.Generator().manual_seed(3)
    W = torch.randn(V, H, generator=g, dtype=D)
    segs = []
    for n in (5, 9, 4):
        hs = torch.randn(n, H, generator=g, dtype=D)
        lab = torch.randint(0, V, (n,), generator=g)
        lab[0] = -100
        segs.append((hs, lab, torch.randn(n, generator=g, dtype=D), torch.randn(n, generator=g, dtype=D) * 0.1 - 2.8))
    def run(order):
        hs = torch.cat([segs[i][0] for i in order])[None]
        lab = torch.cat([segs[i][1] for i in order])[None]
        adv = torch.cat([segs[i][2] for i in order])
        old = torch.cat([segs[i][3] for i in order])
        return O.grpo_loss_and_entropy(W, None, hs, lab, 1.0, old, adv, 0.2, 0.2, 1e32)[0]
    # every sample starts with a -100 label, so after the shift the last position of each sample
    # is masked and the scored (position, target) pairs move with their sample
    a, b_ = run([0, 1, 2]), run([2, 0, 1])
    assert abs(a.item() - b_.item()) < 1e-12


def test_gradients_gradcheck_and_manual_backward():
    hs, W, b, labels = _toy(T=13, H=5, V=7)
    n = labels.numel()
    adv = torch.randn(n, dtype=D)
    old = torch.randn(n, dtype=D) * 0.2 - 2.0
    ref = torch.randn(n, dtype=D) * 0.2 - 2.0
    for kw in (dict(), dict(ref_logprobs=ref, kl_beta=0.05)):
        f = lambda h_, W_, b_: O.grpo_loss_and_entropy(W_, b_, h_, labels, 0.8, old, adv, 0.2, 0.28, 3.0, **kw)[0]
        hs_, W_, b_ = hs.clone().requires_grad_(True), W.clone().requires_grad_(True), b.clone().requires_grad_(True)
        assert torch.autograd.gradcheck(f, (hs_, W_, b_), eps=1e-6, atol=1e-7)
        f(hs_, W_, b_).backward()
        g, dH, dW, db = O.grpo_backward_manual(W, b, hs, labels, 0.8, old, adv, 0.2, 0.28, 3.0, **kw)
        assert torch.allclose(hs_.grad, dH, atol=1e-12)
        assert torch.allclose(W_.grad, dW, atol=1e-12)
        assert torch.allclose(b_.grad, db, atol=1e-12)
        # central finite difference on one weight entry
        Wp, Wm = W.clone(), W.clone()
        Wp[2, 3] += 1e-6
        Wm[2, 3] -= 1e-6
        fd = (f(hs, Wp, b) - f(hs, Wm, b)) / 2e-6
        assert abs(fd.item() - dW[2, 3].item()) < 1e-7


def test_kl_extension_closed_form():
    """beta * (exp(d) - d - 1), d = ref - lp: zero at ref == lp, positive elsewhere, added per token."""
    hs, W, b, labels = _toy()
    n = labels.numel()
    adv = torch.zeros(n, dtype=D)            # policy-gradient term vanishes
    lp, _ = O.fused_log_probs_and_entropy(W, b, hs, labels, 1.0)
    mask = O.shift_labels(labels).reshape(-1) != -100
    out0 = O.grpo_loss_and_entropy(W, b, hs, labels, 1.0, None, adv, 0.2, 0.2, 1e32, ref_logprobs=lp.clone(), kl_beta=0.5)
    assert abs(out0[0].item()) < 1e-14
    ref = lp + 0.3
    out1 = O.grpo_loss_and_entropy(W, b, hs, labels, 1.0, None, adv, 0.2, 0.2, 1e32, ref_logprobs=ref, kl_beta=0.5)
    assert abs(out1[0].item() - 0.5 * (math.exp(0.3) - 0.3 - 1.0)) < 1e-12
    assert mask.any()


def test_sample_mean_brute_force():
    hs, W, b, labels = _toy(T=20)
    cu = torch.tensor([0, 6, 13, 20], dtype=torch.int32)
    labels[0, 0] = labels[0, 6] = labels[0, 13] = -100
    n = labels.numel()
    adv = torch.randn(n, dtype=D)
    old = torch.randn(n, dtype=D) * 0.1 - 2.8
    out = O.grpo_loss_and_entropy(W, b, hs, labels, 1.0, old, adv, 0.2, 0.2, 1e32, loss_agg_mode="sample_mean", cu_seqlens=cu)
    lp, _ = O.fused_log_probs_and_entropy(W, b, hs, labels, 1.0)
    *_, tok = O.grpo_token_terms(lp, old, adv, 0.2, 0.2, 1e32)
    mask = O.shift_labels(labels).reshape(-1) != -100
    per = []
    for s in range(3):
        idx = [t for t in range(int(cu[s]), int(cu[s + 1])) if mask[t]]
        per.append(sum(tok[t].item() for t in idx) / len(idx))
    assert abs(out[0].item() - sum(per) / 3) < 1e-12
    out5 = O.grpo_loss_and_entropy(W, b, hs, labels, 1.0, old, adv, 0.2, 0.2, 1e32, loss_agg_mode="sample_mean",
                                   cu_seqlens=cu, num_samples_total=5)
    assert abs(out5[0].item() - sum(per) / 5) < 1e-12


# ------------------------------------------------------------------ metrics
def test_metrics_hand_computed():
    lr = torch.tensor([0.0, 0.5, -0.5, 0.1])
    ent = torch.tensor([1.0, 2.0, 3.0, 9.0])
    adv = torch.tensor([1.0, 0.0, -2.0, 5.0])
    unclipped = -adv * torch.exp(lr)
    clipped = -adv * torch.exp(lr).clamp(0.8, 1.2)
    oi = torch.tensor([0, 1, 2])
    m = O.dual_clip_metrics(0.25, ent, lr, unclipped, clipped, adv, oi, None, 0.2, 0.2, num_samples=2)
    r = [1.0, math.exp(0.5), math.exp(-0.5)]
    assert abs(m["kl_div"] - (0 + 0.5 + 0.5) / 3) < 1e-7
    assert abs(m["entropy"] - 2.0) < 1e-7
    assert abs(m["approx_kl"] - sum(ri - 1 - l for ri, l in zip(r, [0, 0.5, -0.5])) / 3) < 1e-6
    assert abs(m["clipfrac_upper"] - 1 / 3) < 1e-7 and abs(m["clipfrac_lower"] - 1 / 3) < 1e-7
    assert abs(m["log_ratio_mean"]) < 1e-7 and abs(m["log_ratio_std"] - math.sqrt((0.25 + 0.25) / 3)) < 1e-6
    assert abs(m["adv_mean"] + 1 / 3) < 1e-7 and abs(m["adv_pos_frac"] - 1 / 3) < 1e-7 and abs(m["adv_zero_frac"] - 1 / 3) < 1e-7
    # clipped > unclipped: A=-2, r<0.8 -> clipped = 1.6 > unclipped = 1.21 -> 1 hit
    assert m["pg_clip"] == 1.0
    assert m["loss_per_token"] == 0.25 / 3 and m["loss_per_sample"] == 0.125
    # population standard deviation of the advantages {1, 0, -2}: mean -1/3
    assert abs(m["adv_std"] - math.sqrt(((4 / 3) ** 2 + (1 / 3) ** 2 + (5 / 3) ** 2) / 3)) < 1e-6
    assert m["old_policy_entropy"] == 0.0 and m["entropy_coeff"] == 0.0       # nothing given: zeros
    old_ent = torch.tensor([0.5, 1.5, 4.0, 100.0])
    m2 = O.dual_clip_metrics(0.25, ent, lr, unclipped, clipped, adv, oi, None, 0.2, 0.2, old_entropy=old_ent,
                             num_samples=2, entropy_coeff=0.01)
    assert abs(m2["old_policy_entropy"] - 2.0) < 1e-7 and m2["entropy_coeff"] == 0.01      # mean over the indexed positions only
    assert m2["adv_std"] == m["adv_std"] and m2["kl_div"] == m["kl_div"]


# ------------------------------------------------------------------ batch shaping
def test_output_indices_broadcast_and_advantages():
    il, ol = [3, 1, 4], [2, 5, 1]
    oi = O.output_logits_indices(il, ol)
    want, off = [], 0
    for a, b in zip(il, ol):
        want += list(range(off + a - 1, off + a - 1 + b))
        off += a + b
    assert oi.tolist() == want and oi.dtype == np.int64
    bv = O.broadcast_values([0.5, -1.0, 2.0], [5, 6, 5])
    assert np.array_equal(bv, np.repeat([0.5, -1.0, 2.0], [5, 6, 5])) and bv.dtype == np.float64
    r = np.array([1.0, 0.0, 0.0, 1.0, 1.0, 0.0, 0.0, 0.0])
    adv = O.group_advantages(r)
    assert np.allclose(adv, (r - r.mean()) / (r.std(ddof=0) + 1e-4))
    assert abs(adv.mean()) < 1e-12
    assert np.allclose(O.group_advantages(np.ones(4)), 0.0)          # all-equal group -> zeros, no NaN


def test_output_indices_are_the_scored_positions():
    """The index list equals the positions whose shifted label is not -100 when labels follow the
    generation-side construction (prompt masked, every generated token labelled)."""
    rng = np.random.default_rng(0)
    samples = []
    for _ in range(5):
        li, lo = int(rng.integers(1, 6)), int(rng.integers(1, 7))
        ids = rng.integers(0, 50, li + lo).tolist()
        samples.append(dict(sample_ids=ids, input_len=li, output_len=lo, labels=O.make_labels(ids, li, lo)))
    labels = torch.tensor(sum((s["labels"] for s in samples), []))[None]
    scored = torch.nonzero(O.shift_labels(labels)[0] != -100)[:, 0]
    oi = O.output_logits_indices([s["input_len"] for s in samples], [s["output_len"] for s in samples])
    assert scored.tolist() == oi.tolist()


def test_projection_and_segment_ids_by_hand():
    """The two helpers every other oracle function goes through: the projection (grpo_loss.py:227-230) against a
    hand-expanded sum, with bias and temperature; segment ids of a cu_seqlens vector with an empty segment."""
    W = torch.tensor([[1.0, 2.0], [0.5, -1.0], [3.0, 0.0]], dtype=torch.float64)       # [V=3, H=2]
    b = torch.tensor([0.1, -0.2, 0.3], dtype=torch.float64)
    hs = torch.tensor([[[2.0, -1.0], [0.0, 4.0]]], dtype=torch.float64)                # [1, 2, 2]
    got = O.project(W, b, hs, 0.5)
    want = torch.tensor([[[(2 * 1 - 1 * 2 + 0.1) / 0.5, (2 * 0.5 + 1 * 1 - 0.2) / 0.5, (2 * 3 + 0 + 0.3) / 0.5],
                          [(0 + 4 * 2 + 0.1) / 0.5, (0 - 4 - 0.2) / 0.5, (0 + 0 + 0.3) / 0.5]]], dtype=torch.float64)
    assert torch.allclose(got, want, rtol=0, atol=1e-12)
    assert torch.equal(O.project(W, None, hs, 1.0), torch.einsum("blh,vh->blv", hs, W))
    # hidden states arrive in another dtype than the weights: cast to the weights' first (grpo_loss.py:227)
    assert O.project(W.float(), None, hs, 1.0).dtype == torch.float32
    seg = O.segment_ids_from_cu_seqlens(torch.tensor([0, 2, 2, 5], dtype=torch.int32), 5)
    assert seg.tolist() == [0, 0, 2, 2, 2]


def test_cu_seqlens_from_position_ids():
    pos = torch.tensor([[0, 1, 2, 0, 1, 0, 1, 2, 3]])
    cu = O.cu_seqlens_from_position_ids(pos)
    assert cu.tolist() == [0, 3, 5, 9] and cu.dtype == torch.int32


def test_pack_samples_keys_and_values():
    samples = []
    for i, (li, lo) in enumerate([(2, 3), (1, 2)]):
        ids = list(range(10 * i, 10 * i + li + lo))
        samples.append(dict(sample_ids=ids, sample_position_ids=list(range(li + lo)), labels=O.make_labels(ids, li, lo),
                            input_len=li, output_len=lo, advantage=0.5 - i, sample_logprobs=[-0.1 * (k + 1) for k in range(li + lo)],
                            reward=float(i), modified_reward=None, delimiter_not_found=False, truncated_sample=bool(i)))
    b = O.pack_samples(samples)
    assert b["batch_ids"].shape == (1, 8) and b["labels"].shape == (1, 8)
    assert b["advantages"].tolist() == [0.5] * 5 + [-0.5] * 3
    assert b["output_lens_broadcasted"].tolist() == [3.0] * 5 + [2.0] * 3
    assert b["output_indices"].tolist() == [1, 2, 3, 5, 6]
    assert b["num_output_tokens_non_masked"].item() == 5 and b["num_samples"].item() == 2
    assert b["total_non_modified_reward"].item() == 1.0 and b["truncated_sample"].item() == 1.0
    assert b["reference_output_entropies"].abs().sum() == 0
    assert b["total_modified_reward"].item() == 0.0 and b["num_modified_samples"].item() == 0.0
    assert b["delimiter_not_found"].item() == 0.0


def test_pack_samples_modified_rewards():
    """sample_processing_utils.py:167-168, 209-212: samples whose modified_reward is set are counted apart - their
    modified rewards and delimiter flags are summed, the others contribute their plain reward; total_reward_rank
    sums the plain reward of all."""
    spec = [  # (input_len, output_len, reward, modified_reward, delimiter_not_found)
        (2, 3, 1.0, None, False), (1, 2, 0.5, 0.25, True), (3, 1, 0.0, -1.0, False), (1, 1, 2.0, None, True),
        (2, 2, 1.5, 0.0, True)]
    samples = []
    for i, (li, lo, r, mr, dnf) in enumerate(spec):
        ids = list(range(10 * i, 10 * i + li + lo))
        samples.append(dict(sample_ids=ids, sample_position_ids=list(range(li + lo)), labels=O.make_labels(ids, li, lo),
                            input_len=li, output_len=lo, advantage=float(i), sample_logprobs=[-1.0] * (li + lo),
                            sample_entropies=[0.5] * (li + lo) if i % 2 else None,
                            reward=r, modified_reward=mr, delimiter_not_found=dnf, truncated_sample=False))
    b = O.pack_samples(samples)
    assert b["num_modified_samples"].item() == 3.0                      # modified_reward = 0.0 still counts as set
    assert b["total_modified_reward"].item() == 0.25 - 1.0 + 0.0
    assert b["total_non_modified_reward"].item() == 1.0 + 2.0
    assert b["delimiter_not_found"].item() == 2.0                       # flags of the modified samples only
    assert b["total_reward_rank"].item() == 1.0 + 0.5 + 0.0 + 2.0 + 1.5
    # entropies: given lists where present, zeros of the logprob length elsewhere
    want_ent = sum(([0.5] * (li + lo) if i % 2 else [0.0] * (li + lo) for i, (li, lo, *_r) in enumerate(spec)), [])
    assert b["reference_output_entropies"].tolist() == want_ent


def test_loss_scaling():
    """gpu_process_worker.py:1013-1025: local_target = max(1, target // world) whenever world > 0."""
    assert O.scale_microbatch_loss(2.0, 6, 128, world=2) == 2.0 * 6 / 64
    assert O.scale_microbatch_loss(2.0, 6, 0) == 2.0 * 6          # unset target: max(1, 0 // 1) = 1
    assert O.scale_microbatch_loss(2.0, 6, 3, world=8) == 2.0 * 6  # 3 // 8 = 0 -> 1
    assert O.scale_microbatch_loss(2.0, 6, 6, world=1) == 2.0      # scale exactly 1: loss untouched
    assert O.scale_microbatch_loss(2.0, 6, 0, world=0) == 2.0      # no world, no target: no scaling
    assert O.scale_microbatch_loss(2.0, 6, 12, world=0) == 1.0


def test_split_logprobs_per_sample_hand_case():
    """gpu_process_worker.py:1694-1703: torch.split by sample length, then python lists."""
    lp = torch.tensor([-0.5, -1.5, 0.0, -2.0, -3.0, -0.25])
    ent = torch.tensor([1.0, 2.0, 3.0, 4.0, 5.0, 6.0])
    got = O.split_logprobs_per_sample(lp, ent, [2, 1, 3])
    assert got == [{"logprobs": [-0.5, -1.5], "entropies": [1.0, 2.0]},
                   {"logprobs": [0.0], "entropies": [3.0]},
                   {"logprobs": [-2.0, -3.0, -0.25], "entropies": [4.0, 5.0, 6.0]}]
    assert all(isinstance(v, float) for s in got for v in s["logprobs"] + s["entropies"])
    none = O.split_logprobs_per_sample(lp, None, [6])
    assert none == [{"logprobs": lp.tolist(), "entropies": None}]
    assert O.split_logprobs_per_sample(lp[:0], None, []) == []
