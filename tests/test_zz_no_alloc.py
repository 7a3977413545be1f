"""The dot entry point that allocates nothing, against the allocating one it is a variant of."""
import ctypes

import numpy as np
import pytest
import torch

from gpu_util import dev
from lapis_amd import generators as gen

pytestmark = pytest.mark.gpu


def _dot_pair(lib, x, y, init):
    """(allocating entry, no-alloc entry) results of the same dot, both through the C ABI."""
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    n = ctypes.c_int64(x.shape[0])
    a = torch.full((1,), -7.0, dtype=torch.float64, device="cuda")
    b = torch.full((1,), -9.0, dtype=torch.float64, device="cuda")
    xp, yp = ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(y.data_ptr())
    assert lib.lapis_hip_dot_f64(n, xp, yp, ctypes.c_double(init), ctypes.c_void_p(a.data_ptr()), stream) == 0
    assert lib.lapis_hip_dot_f64_noalloc(n, xp, yp, ctypes.c_double(init), ctypes.c_void_p(b.data_ptr()), stream) == 0
    torch.cuda.synchronize()
    return a.item(), b.item()


def test_noalloc_dot_equals_the_allocating_dot_on_two_calls_in_a_row(gpu, oracle):
    lib = gpu.load()
    # the second call is smaller: it must not see anything the first left in the shared scratch
    for n, seed in ((3_000_001, 11), (70_001, 12)):
        xh, yh = gen.uniform_vector(n, seed), gen.uniform_vector(n, seed + 100)
        want_alloc, got = _dot_pair(lib, dev(xh), dev(yh), 0.25)
        assert got == want_alloc, "no-alloc dot differs from lapis_hip_dot_f64 at n=%d" % n
        want = oracle.dot(xh, yh, init=0.25)
        assert abs(got - want) <= 1e-12 * (np.abs(xh * yh).sum() + 0.25)


def test_noalloc_dot_edge_sizes_and_limit(gpu):
    lib = gpu.load()
    for n in (0, 1, 63, 257):
        xh, yh = np.arange(n, dtype=np.float64), np.ones(n)
        a, b = _dot_pair(lib, dev(xh), dev(yh), 1.5)
        assert a == b == 1.5 + n * (n - 1) / 2
    x = torch.zeros(8, dtype=torch.float64, device="cuda")
    res = torch.zeros(1, dtype=torch.float64, device="cuda")
    too_many = ctypes.c_int64((1 << 34) + 1)
    rc = lib.lapis_hip_dot_f64_noalloc(too_many, ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(x.data_ptr()),
                                       ctypes.c_double(0.0), ctypes.c_void_p(res.data_ptr()), None)
    assert rc == 1 and b"exceeds the maximum" in lib.lapis_hip_last_error()
