"""The C-ABI library loads without a GPU, exports every symbol include/gnnhip.h
declares, validates arguments on the host and reports errors through status codes."""
import ctypes
import os
import re

import numpy as np
import pytest

from graphnn_amd import _lib as binding

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "gnnhip.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gnnhip_[a-z0-9_]+)\s*\(", text)))


def test_library_is_built_in_tree():
    assert os.path.exists(binding.library_path()), "run `python -m graphnn_amd.build`"


def test_every_declared_symbol_is_exported_and_bound():
    lib = ctypes.CDLL(binding.library_path())
    declared = _declared_symbols()
    assert len(declared) >= 30
    for name in declared:
        assert hasattr(lib, name), "declared in gnnhip.h but not exported: " + name
    # the Python binding declares a prototype for each of them, and nothing else
    assert sorted(binding.SIGNATURES) == declared


def test_header_cites_the_reference_for_every_entry():
    text = open(HEADER).read()
    # each block comment introducing entry points names a reference file
    blocks = re.findall(r"/\* ----(.*?)\*/", text, flags=re.S)
    assert len(blocks) >= 20
    for b in blocks:
        if "No counterpart in the reference" in b:      # the entry for callers that cannot allocate
            continue
        assert re.search(r"(src|include|examples)/[\w/]+\.(cpp|cu|h)", b), b[:80]


def test_argument_validation_needs_no_gpu():
    lib = binding.load_library()
    f = ctypes.c_float
    # negative sizes, bad op codes, null pointers: rejected before any device work
    assert lib.gnnhip_spmm_csr_f32(-1, 1, 1, 0, f(1), None, None, None, None, 1, f(0), None, 1, None) == -1
    assert b"negative" in lib.gnnhip_last_error()
    assert lib.gnnhip_spmm_csr_f32(4, 4, 8, 0, f(1), None, None, None, None, 8, f(0), None, 8, None) == -1
    assert lib.gnnhip_gemm_f32(2, 0, 1, 1, 1, f(1), None, 1, None, 1, f(0), None, 1, None) == -1
    assert lib.gnnhip_unary_f32(99, None, 10, f(0), f(0), None) == -1
    assert lib.gnnhip_reduce_f32(9, None, 10, None, None) == -1
    assert lib.gnnhip_row_argmax_f32(None, 3, 0, None, None) == -1
    assert lib.gnnhip_s2v_forward_f32(0, 1, 1, 1, 1, 1, 1, 0, *([None] * 19), None, None) == -1
    x = np.zeros(8, np.float32)
    p = x.ctypes.data_as(ctypes.c_void_p)
    assert lib.gnnhip_s2v_level_f32(2, 4, 0, p, p, p, p, p, None, None, p, None) == -1      # in place is refused
    assert b"in place" in lib.gnnhip_last_error()
    # empty work is a successful no-op
    assert lib.gnnhip_unary_f32(6, None, 0, f(0), f(0), None) == 0
    assert lib.gnnhip_spmm_csr_f32(0, 0, 0, 0, f(1), None, None, None, None, 0, f(0), None, 0, None) == 0
    assert lib.gnnhip_memset0(None, 0, None) == 0


def test_plan_entries_reject_what_is_not_a_plan():
    lib = binding.load_library()
    x = np.zeros(8, np.float32)
    p = x.ctypes.data_as(ctypes.c_void_p)
    f = ctypes.c_float
    assert lib.gnnhip_spmm_csr_planned_f32(p, 4, f(1), p, 4, f(0), p, 4, None) == -1
    assert b"not a live CSR plan" in lib.gnnhip_last_error()
    assert lib.gnnhip_s2v_level_planned_f32(None, 64, p, p, None, None, p, None) == -1
    assert lib.gnnhip_csr_plan_destroy(None) == 0
    assert lib.gnnhip_csr_plan_destroy(p) == -1
    n = ctypes.c_size_t()
    assert lib.gnnhip_csr_plan_bytes(p, ctypes.byref(n)) == -1
    h = ctypes.c_void_p()
    assert lib.gnnhip_csr_plan_create(-1, 1, p, p, p, None, ctypes.byref(h)) == -1
    assert lib.gnnhip_csr_plan_create(1, 1, None, p, p, None, ctypes.byref(h)) == -1
    assert lib.gnnhip_csr_plan_create(1, 1, p, p, p, None, None) == -1


def test_compute_before_init_is_refused():
    import torch
    if torch.cuda.is_available():
        pytest.skip("on a GPU box another test may already have initialised the library")
    lib = binding.load_library()
    x = np.zeros(8, np.float32)
    p = x.ctypes.data_as(ctypes.c_void_p)
    assert lib.gnnhip_unary_f32(6, p, 8, ctypes.c_float(0), ctypes.c_float(0), None) == -4
    assert b"gnnhip_init" in lib.gnnhip_last_error()
    out = ctypes.c_void_p()
    assert lib.gnnhip_malloc(ctypes.byref(out), 1024) == -4
    # no device here: init reports it instead of crashing
    assert lib.gnnhip_init(0) in (-3, -1)
    assert lib.gnnhip_shutdown() == 0


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(binding, "_lib", None)
    monkeypatch.setattr(binding, "_LIB_PATH", str(tmp_path / "libgnnhip.so"))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        binding.load_library()
