"""The C-ABI library loads on a machine without a GPU and exports every symbol
that include/fgrpo.h declares; the ctypes table covers the header one to one.
No compute call is made here."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "fgrpo.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fgrpo_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib_path():
    from fgrpo.build import LIB_PATH, build
    if not os.path.exists(LIB_PATH):
        build(verbose=False)
    return LIB_PATH


def test_header_declares_the_expected_surface():
    names = declared_functions()
    for must in ("fgrpo_logprob_fwd", "fgrpo_lmhead_bwd", "fgrpo_loss_fwd", "fgrpo_metrics", "fgrpo_group_advantages",
                 "fgrpo_segment_broadcast", "fgrpo_segment_reduce", "fgrpo_output_indices", "fgrpo_segment_starts",
                 "fgrpo_logits_logprob_entropy", "fgrpo_logits_logprob_bwd", "fgrpo_last_error", "fgrpo_version"):
        assert must in names


def test_library_exports_every_declared_symbol(lib_path):
    lib = ctypes.CDLL(lib_path)
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} declared in include/fgrpo.h but not exported"


def test_ctypes_table_matches_header(lib_path):
    from fgrpo import _lib
    assert sorted(_lib.SIGNATURES) == declared_functions()
    lib = _lib.load()
    assert lib.fgrpo_version() >= 100
    # argument counts of the table equal the header's
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    for name, (_, args) in _lib.SIGNATURES.items():
        m = re.search(r"\b" + name + r"\s*\((.*?)\)\s*;", text, flags=re.S)
        assert m, name
        params = m.group(1).strip()
        n = 0 if params in ("", "void") else len([p for p in params.split(",")])
        assert n == len(args), f"{name}: header has {n} parameters, ctypes table {len(args)}"


def test_argument_errors_are_reported_without_a_gpu(lib_path):
    from fgrpo import _lib
    lib = _lib.load()
    assert lib.fgrpo_set_tuning(b"no_such_key", 1) == -1
    assert b"no_such_key" in lib.fgrpo_last_error()
    assert lib.fgrpo_logprob_fwd(None, None, None, None, 1.0, 8, 8, 8, 0, None, None, None, None, 0, None) == -1
    assert lib.fgrpo_logprob_fwd_workspace(32768, 1536, 151936, 0) > 0
    assert lib.fgrpo_lmhead_bwd_workspace(32768, 1536, 151936, 0, 0) > 0
    assert lib.fgrpo_get_tuning(b"panel_cols") >= 0


def test_backward_panel_plan_respects_the_bound(lib_path):
    """The dLogits panel of the backward: a multiple of 256 columns, never above the caller's bound (rounded up to
    one 256-column block), at most three panels more than the bound alone would need, and by default at most a
    quarter of [T x V] / 2**30 elements.  Host logic only: no GPU call."""
    import random
    from fgrpo import _lib
    lib = _lib.load()
    rnd = random.Random(0)
    cases = [(32768, 1536, 151936), (65536, 3584, 152064), (16384, 8192, 128256), (131072, 5120, 152064),
             (640, 64, 1000), (4096, 1000, 32000)]
    for _ in range(40):
        cases.append((rnd.randrange(1, 70000), rnd.choice([64, 256, 1536, 4096, 1000]), rnd.randrange(1, 200000)))
    for T, H, V in cases:
        for hint in (0, 256 * T, 4096 * V, rnd.randrange(1, 1 << 31)):
            cols = lib.fgrpo_lmhead_bwd_panel_cols(T, H, V, 0, hint)
            assert cols > 0 and cols % 256 == 0, (T, H, V, hint, cols)
            bound = hint if hint > 0 else min(max(T * V // 4, 1 << 25), 1 << 30)
            max_cols = max(bound // T, 256)
            assert cols <= (max_cols + 255) // 256 * 256, (T, H, V, hint, cols, max_cols)
            np_min = -(-V // max_cols)
            assert -(-V // cols) <= np_min + 3, (T, H, V, hint, cols, np_min)
            assert lib.fgrpo_lmhead_bwd_workspace(T, H, V, 0, hint) >= 2 * cols * T
    assert lib.fgrpo_lmhead_bwd_panel_cols(32768, 1536, 151936, 0, 0) == 21760      # 7 panels: 510 dW tiles each
    assert lib.fgrpo_lmhead_bwd_panel_cols(0, 1536, 151936, 0, 0) < 0
