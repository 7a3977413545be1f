"""Helpers of the GPU parity tests: device copies and the tolerance rule.

Tolerance (stated once, used by every SpMV/SpMM parity test): the HIP result may
differ from the sequential-order oracle by at most
    tol * (sum_j |a_ij * x_j| + |y_in_i|)        tol = 1e-12 for fp64, 1e-5 for fp32
per row -- the relative bound the task states, taken against the magnitude of the
summed terms because rows of a Laplacian cancel to ~0 and |y_i| is no usable scale.
"""
import numpy as np
import torch

from lapis_amd import generators as gen
from lapis_amd.generators import CSR

TOL = {np.dtype(np.float64): 1e-12, np.dtype(np.float32): 1e-5}


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def dev_unaligned(a):
    """Device copy whose first element sits 4 or 8 bytes past a 16-byte boundary."""
    a = np.ascontiguousarray(a)
    buf = torch.empty(a.shape[0] + 1, dtype=torch.from_numpy(a[:0]).dtype, device="cuda")
    view = buf[1:]
    view.copy_(torch.from_numpy(a))
    assert view.data_ptr() % 16 != 0
    return view


def assert_rows_close(got, want, scale, dtype, what=""):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    tol = TOL[np.dtype(dtype)]
    err = np.abs(got - want)
    bound = tol * np.maximum(scale, np.finfo(np.float64).tiny)
    bad = np.nonzero(~(err <= bound))[0]
    assert bad.size == 0, "%s: %d rows outside %g * sum|a x|; first row %d: got %r want %r scale %r" % (
        what, bad.size, tol, bad[0], got[bad[0]], want[bad[0]], scale[bad[0]])


def from_lengths(lengths, ncols, seed, dtype):
    rng = np.random.Generator(np.random.PCG64(seed))
    lengths = np.asarray(lengths, dtype=np.int64)
    crd = gen.random_sorted_columns(rng, lengths, ncols)
    val = (rng.random(crd.shape[0]) * 2 - 1).astype(dtype)
    pos = np.zeros(lengths.shape[0] + 1, np.int32)
    pos[1:] = np.cumsum(lengths)
    return CSR(lengths.shape[0], ncols, pos, crd, val)
