"""fgrpo_logprob_fwd_static (the entry point that allocates nothing) against fgrpo_logprob_fwd with a caller
workspace: same kernels, so the outputs must be bit-identical.  Called through the C ABI, twice in a row, the second
call on a smaller input (the built-in scratch keeps the first call's contents)."""
import pytest
import torch

from fgrpo import _lib

pytestmark = pytest.mark.gpu


def _inputs(T, H, V, seed, dev, with_bias):
    g = torch.Generator().manual_seed(seed)
    hidden = (torch.randn(T, H, generator=g) / H ** 0.5).bfloat16().to(dev)
    weight = (torch.randn(V, H, generator=g) * 0.05).bfloat16().to(dev)
    bias = (torch.randn(V, generator=g) * 0.1).bfloat16().to(dev) if with_bias else None
    labels = torch.randint(0, V, (T,), generator=g)
    labels[torch.rand(T, generator=g) < 0.2] = -100
    return hidden, weight, bias, labels.to(dev)


def _call(lib, static, hidden, weight, bias, labels, inv_temp):
    T, H = hidden.shape
    V = weight.shape[0]
    dev = hidden.device
    # poisoned outputs: every element must be written by the call
    lp, ent, lse = (torch.full((T,), float("nan"), dtype=torch.float32, device=dev) for _ in range(3))
    stream = torch.cuda.current_stream().cuda_stream
    bp = None if bias is None else bias.data_ptr()
    if static:
        rc = lib.fgrpo_logprob_fwd_static(hidden.data_ptr(), weight.data_ptr(), bp, labels.data_ptr(), inv_temp,
                                          T, H, V, _lib.BF16, lp.data_ptr(), ent.data_ptr(), lse.data_ptr(), stream)
    else:
        n = lib.fgrpo_logprob_fwd_workspace(T, H, V, _lib.BF16)
        ws = torch.empty(n, dtype=torch.uint8, device=dev)
        rc = lib.fgrpo_logprob_fwd(hidden.data_ptr(), weight.data_ptr(), bp, labels.data_ptr(), inv_temp,
                                   T, H, V, _lib.BF16, lp.data_ptr(), ent.data_ptr(), lse.data_ptr(),
                                   ws.data_ptr(), n, stream)
    _lib.check(rc, "logprob_fwd_static" if static else "logprob_fwd")
    torch.cuda.synchronize()
    return lp, ent, lse


def test_static_entry_point_matches_workspace_entry_point_twice(dev):
    lib = _lib.load()
    # first call: several token tiles and vocabulary splits, with a bias; second call: smaller in T, H and V
    for (T, H, V, with_bias, inv_temp, seed) in ((3000, 256, 5000, True, 1.0 / 0.7, 11), (777, 128, 1900, False, 1.0, 12)):
        hidden, weight, bias, labels = _inputs(T, H, V, seed, dev, with_bias)
        want = _call(lib, False, hidden, weight, bias, labels, inv_temp)
        got = _call(lib, True, hidden, weight, bias, labels, inv_temp)
        for name, a, b in zip(("logprob", "entropy", "lse"), got, want):
            assert not torch.isnan(a).any(), f"{name}: unwritten output (T={T})"
            assert torch.equal(a, b), f"{name} differs from fgrpo_logprob_fwd at T={T}, H={H}, V={V}"
        assert (got[0][labels == -100] == 0).all()


def test_static_entry_point_rejects_what_does_not_fit(dev):
    lib = _lib.load()
    # fp32 inputs stage split operand copies in the scratch: 4 * (V + T) * H bytes do not fit 8 MiB here
    T, H, V = 512, 1024, 8192
    assert lib.fgrpo_logprob_fwd_workspace(T, H, V, _lib.F32) > _lib.STATIC_SCRATCH_BYTES
    hidden = torch.zeros(T, H, device=dev)
    weight = torch.zeros(V, H, device=dev)
    labels = torch.zeros(T, dtype=torch.int64, device=dev)
    lp = torch.empty(T, device=dev)
    rc = lib.fgrpo_logprob_fwd_static(hidden.data_ptr(), weight.data_ptr(), None, labels.data_ptr(), 1.0, T, H, V,
                                      _lib.F32, lp.data_ptr(), None, None, torch.cuda.current_stream().cuda_stream)
    assert rc == -3
    assert b"scratch" in lib.fgrpo_last_error()
