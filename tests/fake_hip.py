"""A stand-in for lapis_amd.hip on CPU tensors, for the tests of the executor's HOST logic (which buffer an
operation may overwrite, control flow, calls, refusals): every function computes with numpy what the kernel
library's entry point of the same name computes on the device.  Test infrastructure only."""
import numpy as np
import scipy.sparse as sp

calls = []


def _np(t):
    return t.numpy()


class CsrPlan:
    live = 0

    def __init__(self, nrows, ncols, pos, crd, value_bytes=8, stream=None, nnz=None):
        CsrPlan.live += 1
        self.analysed = 0

    def analyze(self, crd, val, stream=None):
        self.analysed += 1
        calls.append("analyze")
        return self

    def destroy(self):
        CsrPlan.live -= 1


def _matrix(nrows, ncols, pos, crd, val):
    return sp.csr_matrix((_np(val), _np(crd), _np(pos)), shape=(nrows, ncols))


def spmv(plan, nrows, ncols, pos, crd, val, x, y, stream=None):
    calls.append("spmv")
    _np(y)[:] += _matrix(nrows, ncols, pos, crd, val) @ _np(x)
    return y


def spmm(nrows, ncols, pos, crd, val, B, C, stream=None, plan=None):
    calls.append("spmm")
    _np(C)[:] += _matrix(nrows, ncols, pos, crd, val) @ _np(B)
    return C


def dot_host(x, y, init_value=0.0, stream=None):
    calls.append("dot")
    return float(init_value + np.dot(_np(x).astype(np.float64), _np(y).astype(np.float64)))


def axpby(a, x, b, y, dst, stream=None):
    calls.append("axpby")
    t = _np(x) * _np(x).dtype.type(a) + _np(y) * _np(y).dtype.type(b)
    _np(dst)[:] = t
    return dst


def mult(x, y, dst, stream=None):
    calls.append("mult")
    _np(dst)[:] = _np(x) * _np(y)
    return dst


def div(x, y, dst, stream=None):
    calls.append("div")
    _np(dst)[:] = _np(x) / _np(y)
    return dst


def fill(dst, value, stream=None):
    calls.append("fill")
    _np(dst)[:] = value
    return dst


def copy(src, dst, stream=None):
    calls.append("copy")
    _np(dst)[:] = _np(src)
    return dst
