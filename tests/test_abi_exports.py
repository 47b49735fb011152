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
