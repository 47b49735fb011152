"""GPU parity of the packed variable-length attention kernels (through the C ABI) against the CPU oracle
(oracle/attn_oracle.py, fp32 math on the same bf16-rounded inputs).

Tolerances, bf16 inputs/outputs with fp32 softmax and accumulation: |d out| <= 2e-2 absolute for O(1) values
(bf16 output rounding is 2^-8 relative, P is rounded to bf16 before P V) and mean |d out| <= 2e-3;
|d lse| <= 2e-3; every gradient cosine >= 0.999 and max error <= 3 % of the gradient's largest entry."""
import pytest
import torch
import torch.nn.functional as F

from oracle import attn_oracle as A

pytestmark = pytest.mark.gpu

OUT_ATOL, OUT_MEAN, LSE_ATOL, COS_MIN, GRAD_REL = 2e-2, 2e-3, 2e-3, 0.999, 3e-2


def cos(a, b):
    return F.cosine_similarity(a.detach().float().flatten().cpu(), b.detach().float().flatten().cpu(), dim=0).item()


def make(T, Hq, Hkv, seed, scale_in=1.0, D=128):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(T, Hq, D, generator=g) * scale_in).bfloat16()
    k = (torch.randn(T, Hkv, D, generator=g) * scale_in).bfloat16()
    v = torch.randn(T, Hkv, D, generator=g).bfloat16()
    do = torch.randn(T, Hq, D, generator=g).bfloat16()
    return q, k, v, do


def check(dev, name, T, cu, Hq, Hkv, causal, seed=0, softmax_scale=None, backward=True, D=128):
    from fgrpo import ops
    print(f"[attention case] {name}: T={T} Hq={Hq} Hkv={Hkv} D={D} causal={causal} segments={len(cu) - 1}", flush=True)
    q, k, v, do = make(T, Hq, Hkv, seed, D=D)
    cu_t = torch.tensor(cu, dtype=torch.int32)
    qo, ko, vo = (x.float().requires_grad_(True) for x in (q, k, v))
    want, want_lse = A.varlen_attention(qo, ko, vo, cu_t, softmax_scale=softmax_scale, causal=causal, return_lse=True)
    qg, kg, vg = (x.to(dev).requires_grad_(True) for x in (q, k, v))
    got = ops.varlen_attention(qg, kg, vg, cu_t.to(dev), softmax_scale, causal)
    _, lse = ops.varlen_attn_fwd(qg, kg, vg, cu_t.to(dev), softmax_scale, causal)
    torch.cuda.synchronize()
    err = (got.float().cpu() - want.detach()).abs()
    assert err.max().item() <= OUT_ATOL, f"{name}: out max err {err.max().item()}"
    assert err.mean().item() <= OUT_MEAN, f"{name}: out mean err {err.mean().item()}"
    assert (lse.cpu() - want_lse).abs().max().item() <= LSE_ATOL, f"{name}: lse"
    if not backward:
        return
    want.backward(do.float())
    got.backward(do.to(dev))
    torch.cuda.synchronize()
    for nm, a, b in (("dq", qg.grad, qo.grad), ("dk", kg.grad, ko.grad), ("dv", vg.grad, vo.grad)):
        if b.abs().max().item() < 1e-6:      # e.g. one-token segments: dq = dk = 0 exactly; a cosine says nothing
            assert a.float().abs().max().item() <= 1e-3, f"{name}: {nm} should vanish"
            continue
        c = cos(a, b)
        rel = (a.float().cpu() - b).abs().max().item() / max(b.abs().max().item(), 1e-12)
        assert c >= COS_MIN, f"{name}: {nm} cosine {c}"
        assert rel <= GRAD_REL, f"{name}: {nm} max error {rel} of the largest entry"


@pytest.mark.parametrize("causal", [True, False])
def test_small_segments_share_a_tile(dev, causal):
    check(dev, "short segments", 200, [0, 5, 6, 70, 71, 72, 200], 4, 2, causal, seed=1)


@pytest.mark.parametrize("causal", [True, False])
def test_segments_cross_tile_boundaries(dev, causal):
    check(dev, "crossing tiles", 1000, [0, 130, 385, 390, 900, 1000], 4, 4, causal, seed=2)


@pytest.mark.parametrize("causal", [True, False])
def test_head_dimension_64(dev, causal):
    # 14 query heads over 2 K/V heads of 64: the attention shape of Qwen2.5-0.5B
    check(dev, "head dim 64, short segments", 200, [0, 5, 6, 70, 71, 72, 200], 4, 2, causal, seed=21, D=64)
    check(dev, "head dim 64, crossing tiles", 1000, [0, 130, 385, 390, 900, 1000], 14, 2, causal, seed=22, D=64)


def test_one_long_segment(dev):
    check(dev, "one segment", 777, [0, 777], 2, 1, True, seed=3)


def test_grouped_query_shape_of_the_1_5b_model(dev):
    # Qwen2.5-1.5B: 12 query heads, 2 K/V heads, head dimension 128
    check(dev, "12/2 heads", 1536, [0, 300, 301, 900, 1536], 12, 2, True, seed=4)


def test_single_token_segments_and_explicit_scale(dev):
    T = 140
    check(dev, "single tokens", T, list(range(T + 1)), 2, 2, True, seed=5)
    check(dev, "explicit scale", 300, [0, 100, 300], 2, 1, True, seed=6, softmax_scale=0.05)


def test_empty_segments_in_cu_seqlens(dev):
    check(dev, "empty segments", 260, [0, 0, 100, 100, 100, 260], 2, 2, True, seed=7)


def test_strided_operands_are_read_in_place(dev):
    """q, k, v as slices of one fused [T, (Hq + 2 Hkv) * 128] projection, the way a fused QKV layer hands them over."""
    from fgrpo import ops
    T, Hq, Hkv = 500, 4, 2
    print("[attention case] strided qkv", flush=True)
    g = torch.Generator().manual_seed(8)
    qkv = torch.randn(T, (Hq + 2 * Hkv) * 128, generator=g).bfloat16().to(dev)
    q = qkv[:, :Hq * 128].view(T, Hq, 128)
    k = qkv[:, Hq * 128:(Hq + Hkv) * 128].view(T, Hkv, 128)
    v = qkv[:, (Hq + Hkv) * 128:].view(T, Hkv, 128)
    cu = torch.tensor([0, 123, 500], dtype=torch.int32, device=dev)
    out, lse = ops.varlen_attn_fwd(q, k, v, cu)
    out2, lse2 = ops.varlen_attn_fwd(q.contiguous(), k.contiguous(), v.contiguous(), cu)
    assert torch.equal(out, out2) and torch.equal(lse, lse2)
    do = torch.randn(T, Hq, 128, generator=g).bfloat16().to(dev)
    g1 = ops.varlen_attn_bwd(do, q, k, v, out, lse, cu)
    g2 = ops.varlen_attn_bwd(do, q.contiguous(), k.contiguous(), v.contiguous(), out, lse, cu)
    for a, b in zip(g1, g2):
        assert torch.equal(a, b)


def test_full_size_properties(dev):
    """T = 32768 packed like the benchmark micro-batch (too large for the oracle): size-independent properties.
    Segments do not see each other (perturbing one segment leaves every other token bit-identical) and a
    segment computed alone equals the same segment inside the pack."""
    from fgrpo import ops
    print("[attention case] full size", flush=True)
    T, Hq, Hkv = 32768, 12, 2
    g = torch.Generator().manual_seed(9)
    lens = []
    while sum(lens) < T:
        lens.append(int(torch.randint(128, 1025, (1,), generator=g)))
    lens[-1] -= sum(lens) - T
    cu_l = [0]
    for n in lens:
        cu_l.append(cu_l[-1] + n)
    cu = torch.tensor(cu_l, dtype=torch.int32, device=dev)
    q = torch.randn(T, Hq, 128, generator=g).bfloat16().to(dev)
    k = torch.randn(T, Hkv, 128, generator=g).bfloat16().to(dev)
    v = torch.randn(T, Hkv, 128, generator=g).bfloat16().to(dev)
    out, lse = ops.varlen_attn_fwd(q, k, v, cu)
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
    a, b = cu_l[3], cu_l[4]
    k2, v2 = k.clone(), v.clone()
    k2[a:b] += 1.0
    v2[a:b] -= 1.0
    out2, _ = ops.varlen_attn_fwd(q, k2, v2, cu)
    assert torch.equal(out[:a], out2[:a]) and torch.equal(out[b:], out2[b:]) and not torch.equal(out[a:b], out2[a:b])
    # the segment alone: same keys per query, but a different split into 64-key steps -> equal up to the
    # rounding of the running rescale
    alone, lse_alone = ops.varlen_attn_fwd(q[a:b], k[a:b], v[a:b], torch.tensor([0, b - a], dtype=torch.int32, device=dev))
    assert (alone.float() - out[a:b].float()).abs().max().item() <= 2e-2
    assert (lse_alone - lse[:, a:b]).abs().max().item() <= 1e-3
    # one segment against the oracle
    want, want_lse = A.varlen_attention(q[a:b].float().cpu(), k[a:b].float().cpu(), v[a:b].float().cpu(),
                                        torch.tensor([0, b - a], dtype=torch.int32), return_lse=True)
    assert (out[a:b].float().cpu() - want).abs().max().item() <= OUT_ATOL
    assert (lse[:, a:b].cpu() - want_lse).abs().max().item() <= LSE_ATOL
    # backward runs at this size and stays finite; dK/dV of a segment do not depend on the others
    do = torch.randn(T, Hq, 128, generator=g).bfloat16().to(dev)
    dq, dk, dv = ops.varlen_attn_bwd(do, q, k, v, out, lse, cu)
    for t in (dq, dk, dv):
        assert torch.isfinite(t.float()).all()
    do2 = do.clone()
    do2[a:b] *= 2
    dq2, dk2, dv2 = ops.varlen_attn_bwd(do2, q, k, v, out, lse, cu)
    for x, y in ((dq, dq2), (dk, dk2), (dv, dv2)):
        assert torch.equal(x[:a], y[:a]) and torch.equal(x[b:], y[b:])


def test_argument_errors(dev):
    from fgrpo import ops
    cu = torch.tensor([0, 16], dtype=torch.int32, device=dev)
    q96 = torch.zeros(16, 2, 96, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="head dimension"):
        ops.varlen_attn_fwd(q96, q96, q96, cu)
    q = torch.zeros(16, 3, 128, dtype=torch.bfloat16, device=dev)
    kv = torch.zeros(16, 2, 128, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError):
        ops.varlen_attn_fwd(q, kv, kv, cu)          # 3 query heads over 2 K/V heads
    with pytest.raises(RuntimeError, match="bf16"):
        ops.varlen_attn_fwd(q.float(), kv.float(), kv.float(), cu)
    with pytest.raises(RuntimeError, match="GPU"):
        ops.varlen_attn_fwd(q.cpu(), kv.cpu(), kv.cpu(), cu.cpu())


def test_transformers_model_with_packed_position_ids(dev):
    """A small random Qwen2 model (head dimension 128, 4 query heads over 2 K/V heads) on one packed row with
    position_ids resets, attention routed through install_explicit_varlen_wrapper: logits and weight gradients
    against the same model run segment by segment with Transformers' own eager attention."""
    from transformers import Qwen2Config, Qwen2ForCausalLM
    import varlen_attention as VA
    print("[attention case] tiny Qwen2 model, packed row", flush=True)
    cfg = Qwen2Config(vocab_size=512, hidden_size=512, intermediate_size=1024, num_hidden_layers=2,
                      num_attention_heads=4, num_key_value_heads=2, max_position_embeddings=1024)
    torch.manual_seed(0)
    model = Qwen2ForCausalLM(cfg).to(dev).to(torch.bfloat16)
    lens = [37, 1, 200, 130]
    T = sum(lens)
    g = torch.Generator().manual_seed(1)
    ids = torch.randint(0, 512, (1, T), generator=g).to(dev)
    pos = torch.cat([torch.arange(n) for n in lens]).unsqueeze(0).to(dev)
    wsel = torch.randn(T, 512, generator=g).to(dev)

    model.config._attn_implementation = "eager"
    ref_logits = []
    a = 0
    for n in lens:
        ref_logits.append(model(input_ids=ids[:, a:a + n], position_ids=pos[:, a:a + n]).logits[0])
        a += n
    ref_logits = torch.cat(ref_logits, 0).float()
    model.zero_grad()
    (ref_logits * wsel).mean().backward()
    ref_grad = model.model.layers[0].self_attn.q_proj.weight.grad.float().clone()
    ref_grad_v = model.model.layers[0].self_attn.v_proj.weight.grad.float().clone()

    assert VA.install_explicit_varlen_wrapper(model) is True
    assert model.config._attn_implementation == VA.ATTENTION_NAME
    model.zero_grad()
    got = model(input_ids=ids, position_ids=pos).logits[0].float()
    (got * wsel).mean().backward()
    torch.cuda.synchronize()
    assert cos(got, ref_logits) >= 0.9995
    assert (got - ref_logits).abs().max().item() <= 0.05 * ref_logits.abs().max().item()
    assert cos(model.model.layers[0].self_attn.q_proj.weight.grad, ref_grad) >= 0.995
    assert cos(model.model.layers[0].self_attn.v_proj.weight.grad, ref_grad_v) >= 0.995


def test_flash_attn_varlen_func_signature(dev):
    import varlen_attention as VA
    q, k, v, _ = make(96, 4, 2, 11)
    cu = torch.tensor([0, 40, 96], dtype=torch.int32)
    want = A.varlen_attention(q.float(), k.float(), v.float(), cu, causal=True)
    got = VA.flash_attn_varlen_func(q.to(dev), k.to(dev), v.to(dev), cu.to(dev), cu.to(dev).clone(), 56, 56,
                                    dropout_p=0.0, softmax_scale=None, causal=True)
    assert (got.float().cpu() - want).abs().max().item() <= OUT_ATOL
    pos = torch.cat([torch.arange(40), torch.arange(56)]).unsqueeze(0).to(dev)
    cu2, mx = VA.prepare_from_position_ids(pos)
    assert cu2.tolist() == [0, 40, 96] and mx == 56
    assert VA.prepare_from_position_ids(pos)[0] is cu2                     # same tensor object: remembered
    ptr = pos.data_ptr()
    del pos
    pos = torch.cat([torch.arange(10), torch.arange(86)]).unsqueeze(0).to(dev)   # typically lands on the same address
    cu3, mx3 = VA.prepare_from_position_ids(pos)
    assert cu3.tolist() == [0, 10, 96] and mx3 == 86, (ptr == pos.data_ptr())
    pos[0, 50] = 0                                                          # in-place edit bumps the version
    assert VA.prepare_from_position_ids(pos)[0].tolist() == [0, 10, 50, 96]
    # the segment scratch is remembered per cu_seqlens OBJECT: a second layer reuses it, an in-place edit rebuilds it
    cud = cu.to(dev)
    a = VA.flash_attn_varlen_func(q.to(dev), k.to(dev), v.to(dev), cud, cud, causal=True)
    held = VA._bounds_cache["value"]
    b = VA.flash_attn_varlen_func(q.to(dev), k.to(dev), v.to(dev), cud, cud, causal=True)
    assert VA._bounds_cache["value"] is held and torch.equal(a, b) and torch.equal(a, got)
    cud[1] = 70
    want2 = A.varlen_attention(q.float(), k.float(), v.float(), torch.tensor([0, 70, 96]), causal=True)
    c = VA.flash_attn_varlen_func(q.to(dev), k.to(dev), v.to(dev), cud, cud, causal=True)
    assert VA._bounds_cache["value"] is not held
    assert (c.float().cpu() - want2).abs().max().item() <= OUT_ATOL
    d = VA.flash_attn_varlen_func(q.to(dev), k.to(dev), v.to(dev), cud, cud, causal=False)     # other mask: rebuilt too
    want3 = A.varlen_attention(q.float(), k.float(), v.float(), torch.tensor([0, 70, 96]), causal=False)
    assert (d.float().cpu() - want3).abs().max().item() <= OUT_ATOL


def test_workers_on_a_transformers_model_end_to_end(dev):
    """The whole replaced path on a real Transformers model: packed attention (install_explicit_varlen_wrapper) feeding
    the fused logprob / GRPO kernels (make_grpo_forward), driven by the two worker harnesses.  Logprobs of the packed
    batch are checked against the same model run sample by sample with eager attention and torch log-softmax."""
    from types import SimpleNamespace
    from transformers import Qwen2Config, Qwen2ForCausalLM
    import numpy as np
    import grpo_loss as G
    import varlen_attention as VA
    from oracle import grpo_oracle as O
    from workers import LogProbHarness, TrainerHarness
    print("[attention case] worker harnesses on a tiny Qwen2 model", flush=True)
    V = 512
    cfg = Qwen2Config(vocab_size=V, hidden_size=512, intermediate_size=1024, num_hidden_layers=2,
                      num_attention_heads=4, num_key_value_heads=2, max_position_embeddings=1024)
    torch.manual_seed(0)
    model = Qwen2ForCausalLM(cfg).to(dev).to(torch.bfloat16)
    rng = np.random.default_rng(0)
    samples = []
    for i in range(5):
        li, lo = int(rng.integers(3, 40)), int(rng.integers(5, 150))
        ids = rng.integers(0, V, li + lo).tolist()
        samples.append(dict(sample_ids=ids, sample_position_ids=list(range(li + lo)), labels=O.make_labels(ids, li, lo),
                            input_len=li, output_len=lo, advantage=float(rng.normal()),
                            sample_logprobs=(-rng.random(li + lo) * 0.2 - 6.0).tolist(), sample_entropies=None,
                            reward=float(i % 2), modified_reward=None, delimiter_not_found=False,
                            truncated_sample=False, __uid__=i))
    # reference numbers: one sample at a time, eager attention, plain log-softmax of the logits
    model.config._attn_implementation = "eager"
    want = []
    with torch.no_grad():
        for s in samples:
            ids = torch.tensor(s["sample_ids"], device=dev)[None]
            logits = model(input_ids=ids, position_ids=torch.arange(ids.shape[1], device=dev)[None]).logits[0].float()
            lab = torch.tensor(s["labels"][1:] + [-100], device=dev)
            lp = torch.log_softmax(logits, -1).gather(-1, lab.clamp(min=0)[:, None])[:, 0] * (lab != -100)
            want.append(lp.cpu())

    from workers import prepare_actor_module
    prepare_actor_module(model, SimpleNamespace(temperature=1.0), mode="eval")
    assert model.config._attn_implementation == VA.ATTENTION_NAME
    res = LogProbHarness(model, dev).compute_log_probs_from_samples(samples)
    for r, w_lp in zip(res, want):
        got = torch.tensor(r["logprobs"])
        assert got.shape == w_lp.shape
        assert (got - w_lp).abs().max().item() <= 0.08      # bf16 model: logits differ at the 1e-2 level
        assert (got - w_lp).abs().mean().item() <= 0.015

    model.forward = model.__original_forward
    G.make_grpo_forward(model, temperature=1.0, mode="training", loss_chunksize=128)
    tcfg = SimpleNamespace(clip_low=0.2, clip_high=0.28, clip_ratio_c=3.0, train_minibatch_sample_size=5, entropy_coeff=0.0)
    model.zero_grad()
    m = TrainerHarness(model, tcfg, dev).compute_gradients(samples, 0)
    assert all(np.isfinite(float(m[k])) for k in ("loss", "kl_div", "entropy", "approx_kl"))
    for p_ in (model.model.layers[0].self_attn.q_proj.weight, model.model.layers[1].self_attn.v_proj.weight,
               model.lm_head.weight):
        assert p_.grad is not None and torch.isfinite(p_.grad.float()).all() and p_.grad.float().abs().max().item() > 0


def test_random_shapes_and_segmentations(dev):
    """Seeded sweep over awkward sizes (T = 1, tile edges +-1), both head dimensions, grouped-query ratios up to 7,
    empty and one-token segments, causal and full attention - forward and backward against the oracle."""
    import random
    rnd = random.Random(0)
    for case in range(30):
        T = rnd.choice([1, 2, 31, 32, 33, 63, 64, 65, 127, 128, 129, 200, 255, 256, 257, 300, 511])
        D = rnd.choice([64, 128])
        Hkv = rnd.choice([1, 2, 3])
        Hq = Hkv * rnd.choice([1, 2, 4, 7])
        causal = rnd.random() < 0.7
        cuts = sorted(set(rnd.sample(range(1, T), min(T - 1, rnd.randint(0, 6))))) if T > 1 else []
        cu = [0] + cuts + [T]
        if rnd.random() < 0.3:
            cu = cu[:1] + [cu[1]] + cu[1:]                  # an empty segment
        check(dev, f"random {case}", T, cu, Hq, Hkv, causal, seed=100 + case, D=D)


@pytest.mark.parametrize("scale_in", [0.01, 4.0, 64.0])
def test_input_scales_from_flat_to_saturated_softmax(dev, scale_in):
    """Scores from nearly constant (softmax flat) to hundreds in magnitude (softmax one-hot, exponents far below
    the fp32 range on the masked side): outputs and gradients stay finite and follow the fp32 oracle."""
    from fgrpo import ops
    T, Hq, Hkv, D = 300, 4, 2, 128
    for causal in (True, False):
        g = torch.Generator().manual_seed(int(scale_in * 100) + causal)
        q = (torch.randn(T, Hq, D, generator=g) * scale_in).bfloat16()
        k = (torch.randn(T, Hkv, D, generator=g) * scale_in).bfloat16()
        v = torch.randn(T, Hkv, D, generator=g).bfloat16()
        do = torch.randn(T, Hq, D, generator=g).bfloat16()
        cu = torch.tensor([0, 37, 38, 200, 300], dtype=torch.int32)
        qo, ko, vo = (x.float().requires_grad_(True) for x in (q, k, v))
        want = A.varlen_attention(qo, ko, vo, cu, causal=causal)
        want.backward(do.float())
        qg, kg, vg = (x.to(dev).requires_grad_(True) for x in (q, k, v))
        got = ops.varlen_attention(qg, kg, vg, cu.to(dev), None, causal)
        got.backward(do.to(dev))
        torch.cuda.synchronize()
        assert (got.float().cpu() - want.detach()).abs().max().item() <= OUT_ATOL
        for a, b in ((qg.grad, qo.grad), (kg.grad, ko.grad), (vg.grad, vo.grad)):
            assert torch.isfinite(a.float()).all()
            assert ((a.float().cpu() - b).norm() / (b.norm() + 1e-30)).item() <= 3e-2


def test_every_heads_per_work_group_shape(dev):
    """The forward and dQ kernels come in three shapes (1, 2 or 4 query heads of a K/V group per work-group over
    128-, 64- or 32-token tiles).  Each is forced in turn over group sizes it divides and does not divide
    (idle wavefronts past the last head), tile-edge token counts and both masks; the default choice is restored."""
    from fgrpo import _lib
    try:
        for hb in (1, 2, 4):
            _lib.set_tuning(attn_heads=hb)
            for i, (T, Hq, Hkv, D, causal) in enumerate([(129, 3, 1, 128, True), (97, 10, 2, 128, True),
                                                         (300, 6, 1, 64, False), (64, 7, 7, 128, True),
                                                         (31, 8, 1, 64, True), (513, 5, 1, 128, False)]):
                cu = [0, T // 3, T // 3 + 1, T]
                check(dev, f"heads/wg={hb} #{i}", T, cu, Hq, Hkv, causal, seed=300 + 10 * hb + i, D=D)
    finally:
        _lib.set_tuning(attn_heads=0)


def test_shared_segment_scratch_gives_identical_results(dev):
    """The segment scratch built once (ops.attention_bounds) and handed to forward and backward gives bit-identical
    results to calls that build their own; a scratch of another shape is refused."""
    from fgrpo import ops
    q, k, v, do = (x.to(dev) for x in make(700, 4, 2, 31))
    cu = torch.tensor([0, 5, 300, 301, 700], dtype=torch.int32, device=dev)
    for causal in (True, False):
        bounds = ops.attention_bounds(cu, 700, causal)
        o1, l1 = ops.varlen_attn_fwd(q, k, v, cu, None, causal)
        o2, l2 = ops.varlen_attn_fwd(q, k, v, cu, None, causal, bounds=bounds)
        assert torch.equal(o1, o2) and torch.equal(l1, l2)
        g1 = ops.varlen_attn_bwd(do, q, k, v, o1, l1, cu, None, causal)
        g2 = ops.varlen_attn_bwd(do, q, k, v, o1, l1, cu, None, causal, bounds=bounds)
        assert all(torch.equal(a, b) for a, b in zip(g1, g2))
    with pytest.raises(RuntimeError, match="bounds"):
        ops.varlen_attn_fwd(q, k, v, cu, None, True, bounds=bounds[:-1])


def test_both_key_side_kernels_give_identical_gradients(dev):
    """dK/dV comes in two kernels: one wavefront per 32 keys, and a pair of wavefronts per 32 keys (the default: one
    computes S and P, the other dP and dS, each accumulates half of the head dimension).  Same products in the same
    order: bit-identical dK and dV over short and long segments, tile-edge token counts, both masks, both head
    dimensions, grouped heads; the single-wavefront kernel also against the oracle.  Twice, so that a result that
    depended on timing would show."""
    import random
    from fgrpo import _lib, ops
    cases = [(200, [0, 5, 6, 70, 71, 72, 200], 4, 2, True, 128), (200, [0, 5, 6, 70, 71, 72, 200], 4, 2, False, 128),
             (1000, [0, 130, 385, 390, 900, 1000], 4, 4, True, 128), (1000, [0, 130, 385, 390, 900, 1000], 14, 2, False, 64),
             (777, [0, 777], 2, 1, True, 128), (4096, [0, 1000, 1001, 3000, 4096], 12, 2, True, 128),
             (4096, [0, 1000, 1001, 3000, 4096], 12, 2, False, 128), (3000, [0, 3000], 6, 2, True, 64),
             (1, [0, 1], 2, 2, True, 128), (129, [0, 64, 129], 3, 1, True, 64)]
    rnd = random.Random(5)
    for _ in range(10):
        T = rnd.randint(2, 2500)
        cuts = sorted(rnd.sample(range(1, T), min(rnd.randint(0, 7), T - 1)))
        cases.append((T, [0] + cuts + [T], rnd.choice([2, 4, 6]), 2, rnd.random() < 0.7, rnd.choice([64, 128])))
    try:
        for i, (T, cu, Hq, Hkv, causal, D) in enumerate(cases):
            print(f"[attention case] key-side kernels #{i}: T={T} segments={len(cu) - 1} Hq={Hq} Hkv={Hkv} causal={causal} D={D}", flush=True)
            q, k, v, do = (x.to(dev) for x in make(T, Hq, Hkv, 500 + i, D=D))
            cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
            out, lse = ops.varlen_attn_fwd(q, k, v, cu_t, None, causal)
            got = {}
            for variant in (1, 2, 2):
                _lib.set_tuning(attn_dkv=variant)
                g = ops.varlen_attn_bwd(do, q, k, v, out, lse, cu_t, None, causal)
                torch.cuda.synchronize()
                if variant in got:
                    assert all(torch.equal(a, b) for a, b in zip(got[variant], g)), f"case {i}: the paired kernel is not reproducible"
                got[variant] = g
            for nm, a, b in zip(("dq", "dk", "dv"), got[1], got[2]):
                assert torch.equal(a, b), f"case {i}: {nm} differs between the two kernels"
        _lib.set_tuning(attn_dkv=1)
        check(dev, "single-wavefront key-side kernel", 1000, [0, 130, 385, 390, 900, 1000], 4, 4, True, seed=2)
        check(dev, "single-wavefront key-side kernel, head dim 64", 1000, [0, 130, 385, 390, 900, 1000], 14, 2, False, seed=22, D=64)
    finally:
        _lib.set_tuning(attn_dkv=0)


def test_both_query_side_kernels_give_identical_results(dev):
    """The forward and the dQ kernel come in two forms: tiles staged through registers with compiler-scheduled LDS
    reads, and the default with tiles loaded direct to LDS and hand-scheduled fragment reads.  Same products in the
    same order: bit-identical out, lse and gradients for every heads-per-work-group shape, both head dimensions,
    both masks, tile-edge token counts; the register-staged kernels also against the oracle.  The default runs twice."""
    import random
    from fgrpo import _lib, ops
    rnd = random.Random(11)
    cases = [(200, [0, 5, 6, 70, 71, 72, 200], 4, 2, True, 128, 0), (1000, [0, 130, 385, 390, 900, 1000], 14, 2, False, 64, 0),
             (777, [0, 777], 2, 1, True, 128, 1), (4096, [0, 1000, 1001, 3000, 4096], 12, 2, True, 128, 2),
             (4096, [0, 1000, 1001, 3000, 4096], 12, 2, False, 128, 4), (3000, [0, 3000], 6, 2, True, 64, 4),
             (1, [0, 1], 2, 2, True, 128, 0), (129, [0, 64, 129], 3, 1, True, 64, 2), (97, [0, 32, 33, 97], 10, 2, True, 128, 4)]
    for _ in range(10):
        T = rnd.randint(2, 2500)
        cuts = sorted(rnd.sample(range(1, T), min(rnd.randint(0, 7), T - 1)))
        cases.append((T, [0] + cuts + [T], rnd.choice([2, 4, 6, 14]), 2, rnd.random() < 0.7, rnd.choice([64, 128]), rnd.choice([0, 1, 2, 4])))
    try:
        for i, (T, cu, Hq, Hkv, causal, D, hb) in enumerate(cases):
            print(f"[attention case] forward kernels #{i}: T={T} segments={len(cu) - 1} Hq={Hq} Hkv={Hkv} causal={causal} D={D} heads/wg={hb}", flush=True)
            q, k, v, do = (x.to(dev) for x in make(T, Hq, Hkv, 700 + i, D=D))
            cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
            got = {}
            for variant in (1, 2, 2):
                _lib.set_tuning(attn_qside=variant, attn_heads=hb)
                out, lse = ops.varlen_attn_fwd(q, k, v, cu_t, None, causal)
                r = (out, lse) + tuple(ops.varlen_attn_bwd(do, q, k, v, out, lse, cu_t, None, causal))
                torch.cuda.synchronize()
                if variant in got:
                    assert all(torch.equal(a, b) for a, b in zip(got[variant], r)), f"case {i}: the default kernels are not reproducible"
                got[variant] = r
            for nm, a, b in zip(("out", "lse", "dq", "dk", "dv"), got[1], got[2]):
                assert torch.equal(a, b), f"case {i}: {nm} differs between the two forms"
        _lib.set_tuning(attn_qside=1, attn_heads=0)
        check(dev, "register-staged query-side kernels", 1000, [0, 130, 385, 390, 900, 1000], 4, 4, True, seed=2)
        check(dev, "register-staged query-side kernels, head dim 64", 1000, [0, 130, 385, 390, 900, 1000], 14, 2, False, seed=22, D=64)
    finally:
        _lib.set_tuning(attn_qside=0, attn_heads=0)
