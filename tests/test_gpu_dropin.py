"""GPU tests of the drop-in Python surface (grpo_loss.py, sample_processing_utils.py,
workers.py of this package) against the CPU oracle: the patched model forward in both
modes, the metrics dictionary, batch packing, the worker harnesses, and the small
segmented / per-group kernels."""
import math
from types import SimpleNamespace

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import grpo_oracle as O

pytestmark = pytest.mark.gpu


class TinyBody(torch.nn.Module):
    """Stand-in for the transformer body: embedding + one linear layer."""

    def __init__(self, V, H):
        super().__init__()
        self.embed_tokens = torch.nn.Embedding(V, H)
        self.proj = torch.nn.Linear(H, H, bias=False)

    def forward(self, input_ids=None, position_ids=None, **kw):
        h = self.proj(self.embed_tokens(input_ids)) + 0.01 * position_ids.unsqueeze(-1).to(self.proj.weight.dtype)
        return (h,)


class TinyLM(torch.nn.Module):
    def __init__(self, V=512, H=64, tied=True):
        super().__init__()
        self.model = TinyBody(V, H)
        self.lm_head = torch.nn.Linear(H, V, bias=False)
        if tied:
            self.lm_head.weight = self.model.embed_tokens.weight
        self.config = SimpleNamespace(output_attentions=False, output_hidden_states=False, use_return_dict=True)

    def forward(self, *a, **k):
        raise RuntimeError("unpatched forward")


def make_samples(n=6, V=512, seed=0):
    rng = np.random.default_rng(seed)
    samples = []
    for i in range(n):
        li, lo = int(rng.integers(2, 9)), int(rng.integers(3, 20))
        ids = rng.integers(0, V, li + lo).tolist()
        samples.append(dict(sample_ids=ids, sample_position_ids=list(range(li + lo)), labels=O.make_labels(ids, li, lo),
                            input_len=li, output_len=lo, advantage=float(rng.normal()),
                            sample_logprobs=(-rng.random(li + lo) * 0.2 - math.log(V)).tolist(),
                            sample_entropies=(rng.random(li + lo) + 5).tolist() if i % 2 == 0 else None,
                            reward=float(i % 2), modified_reward=(0.25 * i - 0.5 if i % 3 == 1 else None),
                            delimiter_not_found=bool(i % 2 == 1),
                            truncated_sample=bool(i % 3 == 0), __uid__=100 + i))
    return samples


def test_post_process_batch_matches_oracle(dev):
    import sample_processing_utils as spu
    samples = make_samples()
    got = spu.post_process_batch(samples, dev)
    want = O.pack_samples(samples)
    for k, v in want.items():
        assert k in got, k
        g = got[k].cpu()
        assert g.dtype == v.dtype and g.shape == v.shape, k
        assert torch.equal(g, v), k
    assert got["uids"].tolist() == [100 + i for i in range(len(samples))]
    # samples 1 and 4 carry a modified reward (sample_processing_utils.py:167-168, 209-212)
    assert got["num_modified_samples"].item() == 2.0 and got["total_modified_reward"].item() == (-0.25) + 0.5
    assert got["delimiter_not_found"].item() == 1.0 and got["total_non_modified_reward"].item() == 0.0 + 0.0 + 1.0 + 1.0
    cu = got["cu_seqlens"].cpu()
    assert torch.equal(cu, O.cu_seqlens_from_position_ids(want["batch_position_ids"]))
    const = spu.post_process_batch(samples, dev, constant_length_samples=7)
    assert (const["output_lens_broadcasted"] == 7).all()
    dummy = spu.post_process_batch([{"dummy": True}], dev)
    assert dummy["labels"].eq(-100).all() and dummy["output_indices"].numel() == 0
    # the dummy batch has the key set of a real one (reference: sample_processing_utils.py:137-157), zero counters,
    # four tokens, and the same dtypes
    assert set(dummy) == {"batch_ids", "batch_position_ids", "output_indices", "advantages", "reference_output_logprobs",
                          "output_lens_broadcasted", "num_output_tokens_non_masked", "num_output_tokens", "num_samples",
                          "max_reward_in_group", "total_modified_reward", "total_non_modified_reward",
                          "num_modified_samples", "delimiter_not_found", "samples", "labels", "total_reward_rank",
                          "truncated_sample", "advantage_is_zero"}
    assert set(dummy) <= set(got), sorted(set(dummy) - set(got))
    assert dummy["batch_ids"].tolist() == [[11, 12, 13, 14]] and dummy["batch_position_ids"].tolist() == [[0, 1, 2, 3]]
    for k, v in dummy.items():
        if k == "samples":
            continue
        assert v.dtype == got[k].dtype, k
        if v.dim() == 0:
            assert v.item() == 0.0, k
    # labels built on the device when the samples carry none (the rule of vllm_worker.py:768-774)
    bare = [{k: v for k, v in smp.items() if k != "labels"} for smp in samples]
    got_bare = spu.post_process_batch(bare, dev)
    assert torch.equal(got_bare["labels"].cpu(), want["labels"])
    assert got_bare["num_output_tokens_non_masked"].item() == got["num_output_tokens_non_masked"].item()
    from fgrpo import ops as _ops
    with pytest.raises(RuntimeError):
        _ops.build_labels(got["batch_ids"], [1, 2], [3, 4])                 # lens do not add up to the batch
    # the two helpers post_process_batch is built from (reference: sample_processing_utils.py:107-125)
    idx, out_lens = spu.get_output_logits_indices(samples, dev)
    assert torch.equal(idx.cpu(), want["output_indices"]) and list(out_lens) == [s["output_len"] for s in samples]
    ids, pos, lab = spu.get_input_for_logprobs(samples, idx, dev)
    for a, key in ((ids, "batch_ids"), (pos, "batch_position_ids"), (lab, "labels")):
        assert a.dtype == torch.long and torch.equal(a.cpu(), want[key]), key


def test_segment_kernels(dev):
    from fgrpo import ops
    pos = torch.cat([torch.arange(n) for n in (5, 1, 300, 64, 1000, 2)])[None].to(dev)
    cu = ops.cu_seqlens_from_position_ids(pos)
    assert torch.equal(cu.cpu(), O.cu_seqlens_from_position_ids(pos.cpu())) and cu.dtype == torch.int32
    # several rounds of the walk (8192 tokens each), ragged end, dense and sparse hits, and the overflow report
    gen = torch.Generator().manual_seed(5)
    for lens in ([1] * 20001, torch.randint(1, 40, (1500,), generator=gen).tolist(), [8192, 8191, 1, 16385], [70001]):
        pos2 = torch.cat([torch.arange(n) for n in lens])[None].to(dev)
        got = ops.cu_seqlens_from_position_ids(pos2)
        assert torch.equal(got.cpu(), O.cu_seqlens_from_position_ids(pos2.cpu())), len(lens)
    with pytest.raises(RuntimeError, match="max_segments"):
        ops.cu_seqlens_from_position_ids(pos, max_segments=3)
    vals = torch.randn(6, dtype=torch.float64)
    out = ops.segment_broadcast(vals.to(dev), cu, pos.numel())
    assert torch.equal(out.cpu(), torch.from_numpy(O.broadcast_values(vals.numpy(), [5, 1, 300, 64, 1000, 2])).float())
    x = torch.randn(pos.numel())
    lab = torch.randint(0, 9, (pos.numel(),))
    lab[::3] = -100
    s, m, c = ops.segment_reduce(x.to(dev), cu, lab.to(dev))
    off = 0
    for i, n in enumerate((5, 1, 300, 64, 1000, 2)):
        ok = lab[off:off + n] != -100
        assert c[i].item() == int(ok.sum())
        assert abs(s[i].item() - x[off:off + n][ok].sum().item()) < 1e-3
        if ok.any():
            assert abs(m[i].item() - x[off:off + n][ok].mean().item()) < 1e-4
        off += n
    il, ol = [3, 1, 4, 2], [2, 5, 1, 0]
    assert ops.output_indices(il, ol, dev).cpu().tolist() == O.output_logits_indices(il, ol).tolist()


def test_group_advantages(dev):
    from fgrpo import ops
    import sample_processing_utils as spu
    rng = np.random.default_rng(0)
    r = (rng.random(8 * 13) < 0.3).astype(np.float64)
    r[8:16] = 1.0                                   # an all-equal group
    goff = torch.arange(0, 8 * 13 + 1, 8, dtype=torch.int32)
    want = np.concatenate([O.group_advantages(r[i:i + 8]) for i in range(0, len(r), 8)])
    got = ops.group_advantages(torch.from_numpy(r).to(dev), goff.to(dev), 1e-4, torch.float64).cpu().numpy()
    assert np.allclose(got, want, rtol=1e-12, atol=1e-12) and np.all(got[8:16] == 0)
    got32 = ops.group_advantages(torch.from_numpy(r).float().to(dev), goff.to(dev), 1e-6).cpu().numpy()
    want6 = np.concatenate([O.group_advantages(r[i:i + 8], 1e-6) for i in range(0, len(r), 8)])
    assert np.allclose(got32, want6, rtol=1e-5, atol=1e-5)
    assert np.allclose(spu.normalize_rewards(r[:8]), O.group_advantages(r[:8]), atol=1e-12)
    ragged = torch.tensor([0, 3, 4, 104], dtype=torch.int32)
    got_r = ops.group_advantages(torch.from_numpy(r).to(dev), ragged.to(dev), 1e-4, torch.float64).cpu().numpy()
    want_r = np.concatenate([O.group_advantages(r[a:b]) for a, b in ((0, 3), (3, 4), (4, 104))])
    assert np.allclose(got_r, want_r, atol=1e-12)


def test_malformed_offsets_stay_inside_the_arrays(dev):
    """cu_seqlens and group offsets live in device memory, so the host cannot vet them: the kernels clamp every
    offset into the array and make ranges monotone.  A malformed vector gives well-defined results for the rows
    that are well formed and touches nothing outside (checked with guard values around the output)."""
    from fgrpo import ops
    T = 10
    cu = torch.tensor([0, 5, 3, 100000], dtype=torch.int32, device=dev)        # decreasing, then far past the end
    vals = torch.tensor([1.0, 2.0, 3.0], device=dev)
    out = ops.segment_broadcast(vals, cu, T).cpu()
    assert out[:3].tolist() == [1.0, 1.0, 1.0] and out[5:].tolist() == [3.0] * 5
    x = torch.arange(T, dtype=torch.float32, device=dev)
    s, m, c = ops.segment_reduce(x, cu)
    assert s.tolist() == [10.0, 0.0, float(sum(range(3, 10)))] and c.tolist() == [5, 0, 7]
    neg = torch.tensor([-7, 4, 2 ** 31 - 1], dtype=torch.int32, device=dev)
    s2, _, c2 = ops.segment_reduce(x, neg)
    assert s2.tolist() == [6.0, float(sum(range(4, 10)))] and c2.tolist() == [4, 6]
    r = torch.tensor([1.0, 0.0, 1.0, 1.0], dtype=torch.float64, device=dev)
    adv = ops.group_advantages(r, torch.tensor([0, 2, 900], dtype=torch.int32), 1e-4, torch.float64).cpu()
    want = np.concatenate([O.group_advantages(np.array([1.0, 0.0])), O.group_advantages(np.array([1.0, 1.0]))])
    assert np.allclose(adv.numpy(), want, atol=1e-12)
    # sample-mean objective with a cu_seqlens that overruns the batch: finite loss, nothing written past T
    import grpo_loss as G
    g = torch.Generator().manual_seed(0)
    hs = torch.randn(1, 64, 64, generator=g).bfloat16().to(dev)
    W = (torch.randn(300, 64, generator=g) * 0.05).bfloat16().to(dev)
    labels = torch.randint(0, 300, (1, 64), generator=g).to(dev)
    bad_cu = torch.tensor([0, 40, 5000], dtype=torch.int32, device=dev)
    out = G.grpo_loss_and_entropy_ce_fn(W, None, hs, labels, 1.0, None, torch.randn(64, generator=g).to(dev),
                                        loss_agg_mode="sample_mean", cu_seqlens=bad_cu)
    torch.cuda.synchronize()
    assert torch.isfinite(out[0]).item()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_row_kernels_on_materialised_logits(dev, dtype):
    import grpo_loss as G
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(2, 37, 1003, generator=g) * 3).to(dtype)
    y = torch.randint(0, 1003, (2, 37), generator=g)
    y[0, :4] = -100
    xg = x.to(dev).requires_grad_(True)
    lp = G.logprobs_from_logits(xg, y.to(dev))
    want = O.logprobs_from_logits(x.float(), y)
    tol = 1e-5 if dtype == torch.float32 else 0.07          # bf16 output rounding of values near -12
    assert lp.dtype == dtype and lp.shape == y.shape
    assert (lp.float().cpu() - want).abs().max() <= tol
    lp32 = G.logprobs_from_logits_flash_attn(xg, y.to(dev))
    assert lp32.dtype == torch.float32 and (lp32.cpu() - want).abs().max() <= 1e-5
    ent = G.entropy_from_logits(x.to(dev))
    assert (ent.float().cpu() - O.entropy_from_logits(x.float())).abs().max() <= (1e-5 if dtype == torch.float32 else 0.04)
    w = torch.randn(2, 37, generator=g)
    (lp32 * w.to(dev)).sum().backward()
    xo = x.float().requires_grad_(True)
    (O.logprobs_from_logits(xo, y) * w).sum().backward()
    rel = (xg.grad.float().cpu() - xo.grad).norm() / xo.grad.norm()
    assert rel <= (1e-5 if dtype == torch.float32 else 5e-3)
    assert xg.grad[0, :4].abs().max() == 0
    # ignore_index=None: every label is gathered
    lpn = G.logprobs_from_logits(x.to(dev), y.clamp(min=0).to(dev), ignore_index=None)
    assert (lpn.float().cpu() - O.logprobs_from_logits(x.float(), y.clamp(min=0), None)).abs().max() <= tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("V,ld", [(1003, 1008), (1024, 1024), (1003, 1003), (5, 8), (2400, 2400)])
def test_row_kernels_vector_and_tail_paths(dev, dtype, V, ld):
    """Rows that start on 16-byte boundaries are read and written 16 bytes at a time with a scalar tail (V % 8),
    others element by element; labels are placed at chunk edges, inside the tail and on ignored rows."""
    import grpo_loss as G
    g = torch.Generator().manual_seed(V + ld)
    N = 9
    buf = (torch.randn(N, ld, generator=g) * 3).to(dtype)
    x = buf[:, :V]
    y = torch.tensor([0, min(7, V - 1), min(8, V - 1), V - 1, V - 2, V // 2, -100, (V - 1) // 8 * 8, 3 % V])
    xg = buf.to(dev)[:, :V].requires_grad_(True)
    assert xg.stride(0) == ld
    lp = G.logprobs_from_logits_flash_attn(xg, y.to(dev))
    want = O.logprobs_from_logits(x.float(), y)
    assert (lp.cpu() - want).abs().max() <= 1e-5
    ent = G.entropy_from_logits(xg.detach())
    assert (ent.float().cpu() - O.entropy_from_logits(x.float())).abs().max() <= (1e-5 if dtype == torch.float32 else 0.04)
    w = torch.randn(N, generator=g)
    (lp * w.to(dev)).sum().backward()
    xo = x.float().requires_grad_(True)
    (O.logprobs_from_logits(xo, y) * w).sum().backward()
    rel = (xg.grad.float().cpu() - xo.grad).norm() / xo.grad.norm()
    assert rel <= (1e-5 if dtype == torch.float32 else 5e-3)
    assert xg.grad[6].abs().max() == 0                       # the ignored row


def _patched(dev, mode, dtype=torch.float32, chunk=None, temperature=1.0):
    import grpo_loss as G
    torch.manual_seed(0)
    m = TinyLM().to(dev).to(dtype)
    return G.make_grpo_forward(m, temperature=temperature, mode=mode, loss_chunksize=chunk), G


def _oracle_hidden(model, batch):
    with torch.no_grad():
        return model.model(input_ids=batch["batch_ids"], position_ids=batch["batch_position_ids"])[0].float().cpu()


def test_eval_forward_and_logprob_worker(dev):
    from workers import LogProbHarness
    model, G = _patched(dev, "eval", temperature=0.9)
    samples = make_samples(5)
    res = LogProbHarness(model, dev).compute_log_probs_from_samples(samples)
    assert len(res) == 5
    ids = torch.tensor(sum((s["sample_ids"] for s in samples), []))[None]
    pos = torch.cat([torch.arange(len(s["sample_ids"])) for s in samples])[None]
    labels = torch.tensor(sum((s["labels"] for s in samples), []))[None]
    hid = _oracle_hidden(model, dict(batch_ids=ids.to(dev), batch_position_ids=pos.to(dev)))
    lp, ent = O.fused_log_probs_and_entropy(model.lm_head.weight.detach().float().cpu(), None, hid, labels, 0.9)
    want = O.split_logprobs_per_sample(lp, ent, [len(s["sample_ids"]) for s in samples])
    for a, b in zip(res, want):
        assert np.allclose(a["logprobs"], b["logprobs"], atol=1e-4)
        assert np.allclose(a["entropies"], b["entropies"], atol=1e-4)
    with pytest.raises(ValueError):
        G.make_grpo_forward(TinyLM().to(dev), mode="bogus").forward(input_ids=ids.to(dev), position_ids=pos.to(dev), labels=labels.to(dev))


def test_packed_logprob_wire_format_round_trip(dev):
    """compute_log_probs_from_samples(packed=True): one pinned fp32 buffer [2, T] + int32 offsets.  Its list form
    equals the default result bit for bit, and post_process_batch builds the same batch from attached views (one
    copy of a column range) as from the lists (per-sample conversion) - also for a sub-run of the samples, and it
    falls back to the general route when the samples are not consecutive slices of one buffer."""
    import sample_processing_utils as spu
    from workers import LogProbHarness
    model, G = _patched(dev, "eval", temperature=0.9)
    samples = make_samples(7, seed=11)
    h = LogProbHarness(model, dev)
    lists = h.compute_log_probs_from_samples(samples)
    packed = h.compute_log_probs_from_samples(samples, packed=True)
    assert isinstance(packed, spu.PackedLogProbs) and len(packed) == 7 and packed.has_entropies
    assert packed.buffer.is_pinned() and packed.buffer.dtype == torch.float32 and packed.buffer.shape[0] == 2
    assert packed.offsets.dtype == np.int32 and packed.offsets.tolist() == np.concatenate(([0], np.cumsum([len(s["sample_ids"]) for s in samples]))).tolist()
    assert packed.to_lists() == lists                                   # bit for bit: float lists compare exactly

    a = [dict(s) for s in samples]
    for s, r in zip(a, lists):                                          # what the reference's controller stores
        s["sample_logprobs"], s["sample_entropies"] = r["logprobs"], r["entropies"]
    b = [dict(s) for s in samples]
    packed.attach(b)
    for sub in (slice(0, 7), slice(2, 6)):
        from_lists = spu.post_process_batch(a[sub], dev)
        from_packed = spu.post_process_batch(b[sub], dev)
        assert spu._packed_run(b[sub]) is not None
        for k, v in from_lists.items():
            if torch.is_tensor(v):
                assert torch.equal(v, from_packed[k]), k
    shuffled = [b[3], b[1], b[2]]
    assert spu._packed_run(shuffled) is None
    got = spu.post_process_batch(shuffled, dev)
    want = spu.post_process_batch([a[3], a[1], a[2]], dev)
    assert torch.equal(got["reference_output_logprobs"], want["reference_output_logprobs"])
    assert torch.equal(got["reference_output_entropies"], want["reference_output_entropies"])
    b[4]["sample_logprobs"] = list(b[4]["sample_logprobs"])            # replaced after attach: general route again
    assert spu._packed_run(b[3:6]) is None


@pytest.mark.parametrize("entropy_coeff", [0.0, 0.01])
def test_training_forward_metrics_and_backward(dev, entropy_coeff):
    import sample_processing_utils as spu
    model, G = _patched(dev, "training", chunk=16)
    samples = make_samples(7, seed=3)
    batch = spu.post_process_batch(samples, dev)
    loss, metrics = G.compute_dual_clip_grpo_loss(model, batch, 0.2, 0.28, 3.0, entropy_coeff=entropy_coeff)
    loss.backward()
    # oracle on the same hidden states, gradients through the same tiny body on the CPU
    import copy
    cpu_model = copy.deepcopy(model).cpu().float()
    cb = O.pack_samples(samples)
    hid = cpu_model.model(input_ids=cb["batch_ids"], position_ids=cb["batch_position_ids"])[0]
    out = O.grpo_loss_and_entropy(cpu_model.lm_head.weight, None, hid, cb["labels"], 1.0, cb["reference_output_logprobs"],
                                  cb["advantages"], 0.2, 0.28, 3.0)
    want = O.dual_clip_metrics(out[0].item(), out[1], out[2], out[4], out[5], cb["advantages"], cb["output_indices"],
                               cb["labels"], 0.2, 0.28, old_entropy=cb["reference_output_entropies"],
                               num_samples=len(samples), entropy_coeff=entropy_coeff)
    assert set(metrics) == set(want)
    for k, v in want.items():
        assert abs(metrics[k] - v) <= 2e-4 * max(1.0, abs(v)), (k, metrics[k], v)
    want_loss = out[0] - entropy_coeff * out[1][cb["output_indices"]].mean()
    assert abs(loss.item() - want_loss.item()) <= 2e-4 * max(1.0, abs(want_loss.item()))
    out[0].backward()
    ge = model.model.embed_tokens.weight.grad.float().cpu()          # tied: LM-head + embedding gradients summed
    gw = cpu_model.model.embed_tokens.weight.grad
    assert torch.nn.functional.cosine_similarity(ge.flatten(), gw.flatten(), dim=0) > 0.9999
    gp = model.model.proj.weight.grad.float().cpu()
    assert torch.nn.functional.cosine_similarity(gp.flatten(), cpu_model.model.proj.weight.grad.flatten(), dim=0) > 0.9999


def test_labels_that_are_not_the_output_tokens_are_noticed(dev):
    """Labels that mask some generated tokens and score as many prompt tokens hold the same NUMBER of valid entries
    as output_indices but not the same positions.  post_process_batch says so (the flag it sets from a host-side
    comparison), and the loss then finds its rows from the labels instead of taking output_indices for them: the
    loss equals the oracle's on those labels."""
    import sample_processing_utils as spu
    import grpo_loss as G
    from fgrpo import ops
    rng = np.random.default_rng(5)
    V, H = 512, 64
    samples = []
    for i in range(40):
        li, lo = int(rng.integers(20, 60)), int(rng.integers(20, 60))
        ids = rng.integers(0, V, li + lo).tolist()
        labels = O.make_labels(ids, li, lo)
        labels[li], labels[li + 1] = -100, -100           # two generated tokens masked ...
        labels[3], labels[4] = ids[3], ids[4]             # ... two prompt tokens scored instead
        samples.append(dict(sample_ids=ids, sample_position_ids=list(range(li + lo)), labels=labels, input_len=li,
                            output_len=lo, advantage=float(rng.normal()), sample_logprobs=[-6.0] * (li + lo),
                            sample_entropies=None, reward=1.0, modified_reward=None, delimiter_not_found=False,
                            truncated_sample=False))
    batch = spu.post_process_batch(samples, dev)
    assert batch["_labels_are_output_tokens"] is False
    assert int(batch["_num_output_tokens_non_masked_host"]) == int(batch["output_indices"].numel())
    plain = [dict(s, labels=O.make_labels(s["sample_ids"], s["input_len"], s["output_len"])) for s in samples]
    assert spu.post_process_batch(plain, dev)["_labels_are_output_tokens"] is True
    assert spu.post_process_batch([{k: v for k, v in s.items() if k != "labels"} for s in plain], dev)["_labels_are_output_tokens"] is True

    model, G = _patched(dev, "training")
    assert ops.COMPACT_MIN_TOKENS <= batch["labels"].numel()
    loss, _ = G.compute_dual_clip_grpo_loss(model, batch, 0.2, 0.28, 3.0)
    import copy
    cpu_model = copy.deepcopy(model).cpu().float()
    cb = O.pack_samples(samples)
    hid = cpu_model.model(input_ids=cb["batch_ids"], position_ids=cb["batch_position_ids"])[0]
    want = O.grpo_loss_and_entropy(cpu_model.lm_head.weight, None, hid, cb["labels"], 1.0, cb["reference_output_logprobs"],
                                   cb["advantages"], 0.2, 0.28, 3.0)[0]
    assert abs(loss.item() - want.item()) <= 2e-4 * max(1.0, abs(want.item()))


@pytest.mark.parametrize("n_tok", [3000, 50000, 700000])
def test_diagnostics_vector_against_direct_sums(dev, n_tok):
    """The 16 sums behind the metric dictionary (reference: grpo_loss.py:408-498), from one work-group for few
    positions and from a two-stage sum in fixed order for many: compared with float64 sums on the host, and two
    runs agree bit for bit.  Negative and out-of-range positions are wrapped / counted, not dereferenced."""
    from fgrpo import ops
    g = torch.Generator().manual_seed(n_tok)
    lr = torch.randn(n_tok, generator=g) * 0.2
    ent = torch.rand(n_tok, generator=g) * 5
    old_ent = torch.rand(n_tok, generator=g) * 5
    adv = torch.randn(n_tok, generator=g).round(decimals=1)
    l1 = torch.randn(n_tok, generator=g)
    l2 = torch.randn(n_tok, generator=g)
    idx = torch.nonzero(torch.rand(n_tok, generator=g) < 0.8).reshape(-1)
    idx = torch.cat([idx, torch.tensor([-1, n_tok + 5, -n_tok - 9])])            # last token, two out of range
    args = [t.to(dev) for t in (idx, lr, ent, old_ent, adv, l1, l2)]
    got = ops.grpo_metrics(*args, 0.2, 0.28)
    again = ops.grpo_metrics(*args, 0.2, 0.28)
    assert torch.equal(got, again)
    ok = torch.cat([idx[:-3], torch.tensor([n_tok - 1])])
    x, a, r = lr[ok].double(), adv[ok].double(), torch.exp(lr[ok]).double()
    want = [ok.numel(), x.abs().sum(), x.sum(), (x * x).sum(), (torch.exp(lr[ok]) - 1.0 - lr[ok]).double().sum(),
            (torch.exp(lr[ok]) > 1.28).sum(), (torch.exp(lr[ok]) < 0.8).sum(), ent[ok].double().sum(),
            old_ent[ok].double().sum(), a.sum(), (a * a).sum(), (a > 0).sum(), (a == 0).sum(), (l2[ok] > l1[ok]).sum(),
            0, 2]
    for k, (gv, wv) in enumerate(zip(got.cpu().tolist(), want)):
        wv = float(wv)
        assert abs(gv - wv) <= 2e-5 * max(1.0, abs(wv)) + (3 if k in (5, 6) else 0), (k, gv, wv)   # k 5, 6: thresholds met to 1 ulp of exp


def test_trainer_harness_scaling_and_dummy(dev):
    from workers import TrainerHarness
    model, G = _patched(dev, "training", dtype=torch.bfloat16)
    cfg = SimpleNamespace(clip_low=0.2, clip_high=0.28, clip_ratio_c=3.0, train_minibatch_sample_size=16, entropy_coeff=0.0)
    tr = TrainerHarness(model, cfg, dev)
    samples = make_samples(4, seed=5)
    m = tr.compute_gradients(samples, 0)
    g1 = model.model.proj.weight.grad.clone()
    assert set(("loss", "kl_div", "entropy", "pg_clip", "approx_kl")) <= set(m)
    model.zero_grad()
    cfg.train_minibatch_sample_size = 4            # scale 1 instead of 4/16
    tr.compute_gradients(samples, 0)
    g2 = model.model.proj.weight.grad.clone()
    ratio = (g1.float().norm() / g2.float().norm()).item()
    assert abs(ratio - 0.25) < 0.02
    # an unset target becomes max(1, 0 // world) = 1: the loss is scaled by the number of real samples
    # (gpu_process_worker.py:1013-1020)
    model.zero_grad()
    cfg.train_minibatch_sample_size = 0
    tr.compute_gradients(samples, 0)
    g3 = model.model.proj.weight.grad.clone()
    assert abs((g3.float().norm() / g2.float().norm()).item() - 4.0) < 0.3
    assert tr.compute_gradients([{"dummy": True}], 0) == {"loss": 0.0, "pg_clip": 0, "kl_div": 0.0, "entropy": 0.0}


@pytest.mark.parametrize("returns_tuple", [False, True])
def test_foreign_per_token_fn_takes_the_materialised_route(dev, returns_tuple):
    """per_token_fn(logits, shifted_labels, vocab_size=V) supplied by the caller (reference: grpo_loss.py:232-239,
    :296-303, either a tensor or (logprobs, logits_flat)): same loss, diagnostics and gradients as the fused route
    and as the oracle, with and without chunking."""
    import grpo_loss as G
    from fgrpo.synthetic import make_workload
    w = make_workload("cfg1", seed=8, overrides=dict(H=128, V=3000, tokens=700, len_lo=8, len_hi=120, h_scale=1.0))
    p = w.params
    calls = []

    def my_fn(logits, labels, vocab_size=None):
        calls.append(tuple(logits.shape))
        assert vocab_size == w.V
        lp = torch.log_softmax(logits.float(), -1).gather(-1, labels.clamp(min=0).unsqueeze(-1)).squeeze(-1)
        lp = lp * (labels != -100)
        return (lp, logits.reshape(-1, logits.shape[-1])) if returns_tuple else lp

    T = w.T
    adv = torch.randn(T, generator=torch.Generator().manual_seed(3)).to(dev)
    with torch.no_grad():
        lp0, _ = G.fused_log_probs_and_entropy_fn(w.weight.to(dev), None, w.hidden.to(dev), w.labels.to(dev))
    old = lp0 + w.noise_old.to(dev)
    outs = []
    for fn, chunk in ((G.logprobs_from_logits, None), (my_fn, None), (my_fn, 256)):
        hs = w.hidden.to(dev).clone().requires_grad_(True)
        W = w.weight.to(dev).clone().requires_grad_(True)
        out = G.grpo_loss_and_entropy_ce_fn(W, None, hs, w.labels.to(dev), 1.0, old, adv, p["clip_low"], p["clip_high"],
                                            p["clip_ratio_c"], per_token_fn=fn, loss_chunksize=chunk)
        out[0].backward()
        outs.append((out, hs.grad, W.grad))
    assert calls[0] == (1, T, w.V) and len(calls) == 1 + (T + 255) // 256
    ref = outs[0]
    for out, dh, dw in outs[1:]:
        # logits are rounded to bf16 on the materialised route (as in the reference): logprob errors ~1e-2
        assert abs(out[0].item() - ref[0][0].item()) <= 5e-4
        assert (out[2] - ref[0][2]).abs().max().item() <= 2e-2
        assert (out[1] - ref[0][1]).abs().max().item() <= 5e-2
        assert F.cosine_similarity(dh.float().flatten(), ref[1].float().flatten(), dim=0).item() >= 0.999
        assert F.cosine_similarity(dw.float().flatten(), ref[2].float().flatten(), dim=0).item() >= 0.999
    lp_m, ent_m = G.fused_log_probs_and_entropy_fn(w.weight.to(dev), None, w.hidden.to(dev), w.labels.to(dev), per_token_fn=my_fn)
    assert (lp_m - lp0).abs().max().item() <= 2e-2
