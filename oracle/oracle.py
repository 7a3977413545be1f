"""ctypes front of the CPU oracle (oracle/lapis_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke()`` and
by the ``cpu_baseline`` leg of bench.py.  Nothing under ``lapis_amd/`` imports it.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_c_i64 = ctypes.c_int64
_c_u64 = ctypes.c_uint64
_c_dbl = ctypes.c_double
_c_flt = ctypes.c_float
_vp = ctypes.c_void_p


def build(force=False):
    """Compile both oracle libraries with the committed Makefile."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE, "all"], check=True, capture_output=True)


def _load(name):
    path = os.path.join(_HERE, name)
    if not os.path.exists(path):
        build()
    return ctypes.CDLL(path)


def _ptr(a):
    return ctypes.c_void_p(a.ctypes.data)


def _req(a, dtype):
    return np.require(a, dtype=dtype, requirements=["C", "A"])


class Oracle:
    """Sequential (``omp=False``) or OpenMP (``omp=True``) build of the oracle."""

    def __init__(self, omp=False):
        self.omp = omp
        self.lib = _load("liblapis_oracle_omp.so" if omp else "liblapis_oracle.so")
        L = self.lib
        L.oracle_dot_f64.restype = _c_dbl
        L.oracle_dot_f64.argtypes = [_c_i64, _vp, _vp, _c_dbl]
        L.oracle_dot_f64_omp.restype = _c_dbl
        L.oracle_dot_f64_omp.argtypes = [_c_i64, _vp, _vp, _c_dbl]
        L.oracle_dot_f32.restype = _c_flt
        L.oracle_dot_f32.argtypes = [_c_i64, _vp, _vp, _c_flt]
        L.oracle_plus_norm_f64.restype = _c_dbl
        L.oracle_csr_parallelism_hint.restype = _c_u64
        L.oracle_csr_parallelism_hint.argtypes = [_c_i64, _vp]
        L.oracle_thread_parallel_vector_length.restype = ctypes.c_int
        L.oracle_thread_parallel_vector_length.argtypes = [_c_i64, ctypes.c_int]
        L.oracle_pcg_f64_i32.restype = _c_u64
        L.oracle_pcg_masked_f64_i32.restype = _c_u64
        L.oracle_omp_max_threads.restype = ctypes.c_int

    # -- SpMV ---------------------------------------------------------------
    def spmv(self, pos, crd, val, x, y, parallel=False):
        """In place y = A*x + y in the reference's summation order."""
        dt = val.dtype
        assert dt in (np.float64, np.float32)
        pos, crd = _req(pos, np.int32), _req(crd, np.int32)
        val, x = _req(val, dt), _req(x, dt)
        assert y.dtype == dt and y.flags.c_contiguous
        n = pos.shape[0] - 1
        name = "oracle_spmv_csr_%s_i32" % ("f64" if dt == np.float64 else "f32")
        if parallel:
            name += "_omp"
        getattr(self.lib, name)(_c_i64(n), _ptr(pos), _ptr(crd), _ptr(val), _ptr(x), _ptr(y))
        return y

    def spmv_abs_scale(self, pos, crd, val, x, yin=None):
        dt = val.dtype
        pos, crd = _req(pos, np.int32), _req(crd, np.int32)
        val, x = _req(val, dt), _req(x, dt)
        n = pos.shape[0] - 1
        out = np.empty(n, dtype=np.float64)
        name = "oracle_spmv_abs_scale_%s_i32" % ("f64" if dt == np.float64 else "f32")
        yin = _req(yin, dt) if yin is not None else None  # held in a local: the pointer below must stay valid
        yp = _ptr(yin) if yin is not None else None
        getattr(self.lib, name)(_c_i64(n), _ptr(pos), _ptr(crd), _ptr(val), _ptr(x), yp, _ptr(out))
        return out

    # -- SpMM ---------------------------------------------------------------
    def spmm(self, pos, crd, val, B, C, parallel=False):
        """In place C += A*B (row-major B, C)."""
        dt = val.dtype
        pos, crd = _req(pos, np.int32), _req(crd, np.int32)
        val, B = _req(val, dt), _req(B, dt)
        assert C.dtype == dt and C.flags.c_contiguous
        n, k = C.shape
        name = "oracle_spmm_csr_%s_i32" % ("f64" if dt == np.float64 else "f32")
        if parallel:
            name += "_omp"
        getattr(self.lib, name)(_c_i64(n), _c_i64(k), _ptr(pos), _ptr(crd), _ptr(val),
                                _ptr(B), _c_i64(B.shape[1]), _ptr(C), _c_i64(C.shape[1]))
        return C

    def bspmm_csrv(self, pos, crd, val, V, n1):
        pos, crd = _req(pos, np.int32), _req(crd, np.int32)
        val, V = _req(val, np.float32), _req(V, np.float32)
        _, dh, nh = V.shape
        out = np.zeros((n1, dh, nh), dtype=np.float32)
        self.lib.oracle_bspmm_csrv_f32_i32(_c_i64(n1), _c_i64(dh), _c_i64(nh), _ptr(pos),
                                           _ptr(crd), _ptr(val), _ptr(V), _ptr(out))
        return out

    # -- vector ops ---------------------------------------------------------
    def dot(self, x, y, init=0.0, parallel=False):
        if x.dtype == np.float32:
            x, y = _req(x, np.float32), _req(y, np.float32)
            return np.float32(self.lib.oracle_dot_f32(_c_i64(x.shape[0]), _ptr(x), _ptr(y), _c_flt(init)))
        x, y = _req(x, np.float64), _req(y, np.float64)
        fn = self.lib.oracle_dot_f64_omp if parallel else self.lib.oracle_dot_f64
        return fn(_c_i64(x.shape[0]), _ptr(x), _ptr(y), _c_dbl(init))

    def axpby(self, a, x, b, y, dst=None, parallel=False):
        dt = x.dtype
        x, y = _req(x, dt), _req(y, dt)
        if dst is None:
            dst = np.empty_like(x)
        if dt == np.float32:
            self.lib.oracle_axpby_f32(_c_i64(x.shape[0]), _c_flt(a), _ptr(x), _c_flt(b), _ptr(y), _ptr(dst))
        else:
            fn = self.lib.oracle_axpby_f64_omp if parallel else self.lib.oracle_axpby_f64
            fn(_c_i64(x.shape[0]), _c_dbl(a), _ptr(x), _c_dbl(b), _ptr(y), _ptr(dst))
        return dst

    def mult(self, x, y):
        x, y = _req(x, np.float64), _req(y, np.float64)
        dst = np.empty_like(x)
        self.lib.oracle_mult_f64(_c_i64(x.shape[0]), _ptr(x), _ptr(y), _ptr(dst))
        return dst

    def plus_norm(self, x, y):
        x, y = _req(x, np.float64), _req(y, np.float64)
        out = np.empty_like(x)
        nrm = self.lib.oracle_plus_norm_f64(_c_i64(x.shape[0]), _ptr(x), _ptr(y), _ptr(out))
        return out, nrm

    # -- launch-shape rule ----------------------------------------------------
    def csr_parallelism_hint(self, pos):
        pos = _req(pos, np.int32)
        return int(self.lib.oracle_csr_parallelism_hint(_c_i64(pos.shape[0] - 1), _ptr(pos)))

    def thread_parallel_vector_length(self, hint, max_vector_length):
        return int(self.lib.oracle_thread_parallel_vector_length(_c_i64(hint), max_vector_length))

    # -- CG -------------------------------------------------------------------
    def pcg(self, pos, crd, val, b, dinv, tol, maxiter):
        """examples/pcg_solve.py:52 -> (x, iters, relres)."""
        pos, crd = _req(pos, np.int32), _req(crd, np.int32)
        val, b, dinv = _req(val, np.float64), _req(b, np.float64), _req(dinv, np.float64)
        n = b.shape[0]
        x = np.empty(n)
        work = np.empty(4 * n)
        relres = _c_dbl(0.0)
        it = self.lib.oracle_pcg_f64_i32(_c_i64(n), _ptr(pos), _ptr(crd), _ptr(val), _ptr(b), _ptr(dinv),
                                         _c_dbl(tol), _c_u64(maxiter), _ptr(x), ctypes.byref(relres), _ptr(work))
        return x, int(it), relres.value

    def pcg_masked(self, pos, crd, val, b, mask, d, tol, maxiter):
        """examples/hitting_times.py:97 -> (x, iters, relres)."""
        pos, crd = _req(pos, np.int32), _req(crd, np.int32)
        val, b = _req(val, np.float64), _req(b, np.float64)
        mask, d = _req(mask, np.float64), _req(d, np.float64)
        n = b.shape[0]
        x, work = np.empty(n), np.empty(5 * n)
        relres = _c_dbl(0.0)
        it = self.lib.oracle_pcg_masked_f64_i32(_c_i64(n), _ptr(pos), _ptr(crd), _ptr(val), _ptr(b), _ptr(mask),
                                                _ptr(d), _c_dbl(tol), _c_u64(maxiter), _ptr(x), ctypes.byref(relres),
                                                _ptr(work))
        return x, int(it), relres.value

    def mht(self, pos, crd, val, mask, d, alpha, tol, maxiter):
        """examples/hitting_times.py:153 -> (mom1, mom2); scales ``val`` in place."""
        pos, crd = _req(pos, np.int32), _req(crd, np.int32)
        assert val.dtype == np.float64 and val.flags.c_contiguous
        mask, d = _req(mask, np.float64), _req(d, np.float64)
        n = d.shape[0]
        mom1, mom2, work = np.empty(n), np.empty(n), np.empty(6 * n)
        self.lib.oracle_mht_f64_i32(_c_i64(n), _c_i64(val.shape[0]), _ptr(pos), _ptr(crd), _ptr(val), _ptr(mask),
                                    _ptr(d), _c_dbl(alpha), _c_dbl(tol), _c_u64(maxiter), _ptr(mom1), _ptr(mom2),
                                    _ptr(work))
        return mom1, mom2

    def normalize_mom2(self, mom1, mom2):
        mom1, mom2 = _req(mom1, np.float64), _req(mom2, np.float64)
        out = np.empty_like(mom1)
        self.lib.oracle_normalize_mom2_f64(_c_i64(mom1.shape[0]), _ptr(mom1), _ptr(mom2), _ptr(out))
        return out

    def max_threads(self):
        return int(self.lib.oracle_omp_max_threads())
