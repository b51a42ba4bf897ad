"""gnnhip_jagged_softmax_static_f32 (the entry point that allocates nothing) gives the bits of
gnnhip_jagged_softmax_f32 on two calls in a row, the second smaller than the first, and refuses more
segments than its static array holds."""
import ctypes

import numpy as np
import pytest

from conftest import PARITY_TOL, max_rel

pytestmark = pytest.mark.gpu


def _pair(ops, torch, gpu, x, lens):
    xd = torch.from_numpy(x).to(gpu)
    ld = torch.from_numpy(lens).to(gpu)
    want = ops.jagged_softmax(xd.clone(), ld)
    got = ops.jagged_softmax_static(xd.clone(), ld)
    torch.cuda.synchronize()
    return got.cpu().numpy(), want.cpu().numpy()


def test_static_jagged_softmax_two_calls_second_smaller(gpu, oracle):
    import torch
    from graphnn_amd import ops
    from graphnn_amd._lib import load_library
    rng = np.random.default_rng(41)
    # first call: 50,000 ragged segments (empty, length-1 and one long segment among them)
    lens1 = rng.integers(0, 30, 50000).astype(np.int32)
    lens1[[0, 7, 49999]] = 0
    lens1[3] = 1
    lens1[25000] = 30000
    x1 = (rng.standard_normal(int(lens1.sum())) * 2).astype(np.float32)
    got1, want1 = _pair(ops, torch, gpu, x1, lens1)
    assert np.array_equal(got1, want1)
    assert max_rel(got1, oracle.jagged_softmax(x1, lens1)) < PARITY_TOL
    # second call, smaller: the offsets the first call left behind must not show
    lens2 = np.array([2, 3, 5], np.int32)                        # gpu_tensor_test.cpp:182-209, bound 1e-5
    x2 = (1.0 + rng.random(10)).astype(np.float32)
    got2, want2 = _pair(ops, torch, gpu, x2, lens2)
    assert np.array_equal(got2, want2)
    assert float(np.abs(got2 - oracle.jagged_softmax(x2, lens2)).sum()) <= 1e-5
    # the largest size it takes, then one past it
    lens3 = np.full(65536, 3, np.int32)
    x3 = rng.standard_normal(3 * 65536).astype(np.float32)
    got3, want3 = _pair(ops, torch, gpu, x3, lens3)
    assert np.array_equal(got3, want3)
    lib = load_library()
    assert lib.gnnhip_jagged_softmax_static_f32(None, None, 65537, None) == -1
    assert b"at most 65536" in lib.gnnhip_last_error()
    assert lib.gnnhip_jagged_softmax_static_f32(None, None, 0, None) == 0


def test_static_jagged_softmax_makes_no_driver_allocation(gpu):
    """the library's own allocation counter and torch's do not move across the call"""
    import torch
    from graphnn_amd import ops
    from graphnn_amd._lib import load_library
    lib = load_library()
    lens = torch.full((4096,), 1024, dtype=torch.int32, device=gpu)
    x = torch.randn(4096 * 1024, device=gpu)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    z = [ctypes.c_size_t() for _ in range(3)]
    lib.gnnhip_pool_stats(*[ctypes.byref(c) for c in z])
    before = z[2].value
    ops.jagged_softmax_static(x, lens)
    torch.cuda.synchronize()
    lib.gnnhip_pool_stats(*[ctypes.byref(c) for c in z])
    free1, _ = torch.cuda.mem_get_info()
    assert z[2].value == before
    assert free1 == free0
    seg = x.view(4096, 1024).double().sum(dim=1)
    assert float((seg - 1.0).abs().max()) < 1e-5
