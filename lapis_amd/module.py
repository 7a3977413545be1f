"""``LAPISModule``: the Python class a LAPIS-generated package exposes, bound to the
prebuilt gfx950 module.

Mirrors what the reference's emitter writes next to every generated ``.so``
(TranslateToKokkosCpp.cpp:4393-4411 for the class, :2757-2977 per function): the
constructor loads the library and calls ``lapis_initialize()``, ``__del__`` calls
``lapis_finalize()``, and each module function is a method taking ``param0..``
positionally.  Dense inputs are coerced with ``numpy.require(dtype, 'C')``, a
sparse tensor's storage specifier is given as the nested tuple
``((m, n), (m+1, nnz, nnz))``, scalars go through ctypes, memref results come back
as numpy arrays aliasing module-owned (or caller-owned, for in-place results)
memory.
"""
import ctypes
import os

import numpy

from . import memref as rt

_HERE = os.path.dirname(os.path.abspath(__file__))
DEFAULT_MODULE_PATH = os.path.join(_HERE, "lib", "liblapis_package_module.so")


def _flatten_specifier(spec):
    flat = numpy.zeros(5, dtype=numpy.int64)
    for i in range(2):
        flat[0 + i] = spec[0][i]
    for i in range(3):
        flat[2 + i] = spec[1][i]
    return flat


class DualView:
    """A numpy array paired with a device copy that stays allocated between calls: the role of
    LAPIS::DualView (LAPISSupport.hpp:136-426) with its lazy modified-host / modified-device flags.
    ``host`` is the numpy side; after writing to it call ``modify_host()``; ``sync_host()`` brings a
    result back (and waits for the kernels that produce it)."""

    def __init__(self, lib, array):
        self._lib = lib
        self.host = numpy.require(array, dtype=numpy.float64, requirements=['C', 'W'])
        self._handle = ctypes.c_void_p(lib.lapis_dualview_f64_create(self.host.ctypes.data_as(ctypes.c_void_p),
                                                                     ctypes.c_int64(self.host.shape[0])))

    def modify_host(self):
        self._lib.lapis_dualview_f64_modify_host(self._handle)
        return self

    def sync_host(self):
        self._lib.lapis_dualview_f64_sync_host(self._handle)
        return self.host

    def sync_device(self):
        self._lib.lapis_dualview_f64_sync_device(self._handle)
        return self

    def release(self):
        if self._handle:
            self._lib.lapis_dualview_f64_destroy(self._handle)
            self._handle = None

    def __del__(self):
        try:
            self.release()
        except Exception:
            pass


class ResidentCsr:
    """A CSR matrix uploaded once (``LAPISModule.bind_csr``): device copies, plan and, where the library
    recommends it, the column-blocked copy are reused by every ``spmv``."""

    def __init__(self, module, pos, crd, val, spec):
        self._module = module  # keeps the library initialised for as long as the matrix lives
        self._lib = module.libHandle
        pos = numpy.require(pos, dtype=numpy.int32, requirements=['C'])
        crd = numpy.require(crd, dtype=numpy.int32, requirements=['C'])
        val = numpy.require(val, dtype=numpy.float64, requirements=['C'])
        flat = _flatten_specifier(spec)
        self.shape = (int(flat[0]), int(flat[1]))
        self._handle = ctypes.c_void_p(self._lib.lapis_resident_csr_create(
            ctypes.pointer(rt.get_ranked_memref_descriptor(pos)), ctypes.pointer(rt.get_ranked_memref_descriptor(crd)),
            ctypes.pointer(rt.get_ranked_memref_descriptor(val)), flat.ctypes.data_as(ctypes.c_void_p)))

    def update_values(self, val):
        val = numpy.require(val, dtype=numpy.float64, requirements=['C'])
        self._lib.lapis_resident_csr_update_values(self._handle, ctypes.pointer(rt.get_ranked_memref_descriptor(val)))

    def spmv(self, x, y):
        """y += A x.  With ``DualView`` operands nothing crosses PCIe and the call returns before the kernel
        has run (``y.sync_host()`` fetches the result); numpy operands are copied in and out as
        ``LAPISModule.spmv`` does, and the updated ``y`` is returned."""
        if isinstance(x, DualView) and isinstance(y, DualView):
            self._lib.lapis_resident_csr_spmv(self._handle, x._handle, y._handle)
            return y
        xv = x if isinstance(x, DualView) else DualView(self._lib, x)
        yv = y if isinstance(y, DualView) else DualView(self._lib, y)
        self._lib.lapis_resident_csr_spmv(self._handle, xv._handle, yv._handle)
        out = yv.sync_host()
        if out is not y and isinstance(y, numpy.ndarray):
            y[...] = out  # numpy.require had to copy (dtype or layout): keep the in-place contract
            out = y
        for v, given in ((xv, x), (yv, y)):
            if v is not given:
                v.release()
        return out

    def release(self):
        if self._handle:
            self._lib.lapis_resident_csr_destroy(self._handle)
            self._handle = None

    def __del__(self):
        try:
            self.release()
        except Exception:
            pass


class LAPISModule:
    def __init__(self, libPath=None):
        libPath = libPath or DEFAULT_MODULE_PATH
        if not os.path.exists(libPath):
            raise FileNotFoundError(
                "%s not found: build the HIP libraries first (python -m lapis_amd.build)" % libPath)
        self.libHandle = ctypes.CDLL(libPath)
        self.libHandle.lapis_initialize.restype = None
        self.libHandle.lapis_finalize.restype = None
        self.libHandle.lapis_dualview_f64_create.restype = ctypes.c_void_p
        self.libHandle.lapis_dualview_f64_create.argtypes = [ctypes.c_void_p, ctypes.c_int64]
        for fn in ("modify_host", "modify_device", "sync_host", "sync_device", "destroy"):
            f = getattr(self.libHandle, "lapis_dualview_f64_" + fn)
            f.restype, f.argtypes = None, [ctypes.c_void_p]
        self.libHandle.lapis_resident_csr_create.restype = ctypes.c_void_p
        self.libHandle.lapis_resident_csr_update_values.restype = None
        self.libHandle.lapis_resident_csr_update_values.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        self.libHandle.lapis_resident_csr_spmv.restype = None
        self.libHandle.lapis_resident_csr_spmv.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
        self.libHandle.lapis_resident_csr_destroy.restype = None
        self.libHandle.lapis_resident_csr_destroy.argtypes = [ctypes.c_void_p]
        self.libHandle.lapis_initialize()

    def __del__(self):
        handle = getattr(self, "libHandle", None)
        if handle is not None:
            handle.lapis_finalize()

    # ---- operands that stay on the device (opt-in; the methods below copy per call as the reference does) ----
    def bind_csr(self, param0, param1, param2, param3):
        """Upload a CSR matrix (positions, coordinates, values, storage specifier) once; the returned
        object's ``spmv(x, y)`` reuses the device copies, the plan and the column-blocked layout."""
        return ResidentCsr(self, param0, param1, param2, param3)

    def dual_view(self, array):
        """A float64 vector that keeps a device copy between calls (see ``DualView``)."""
        return DualView(self.libHandle, array)

    # func @spmv(A, x, y) -> y          (examples/spmv_noalloc.py:9, benchmarks/spmv/spmv.mlir)
    def spmv(self, param0, param1, param2, param3, param4, param5):
        val_dtype = numpy.float32 if numpy.asarray(param2).dtype == numpy.float32 else numpy.float64
        param0 = numpy.require(param0, dtype=numpy.int32, requirements=['C'])
        param1 = numpy.require(param1, dtype=numpy.int32, requirements=['C'])
        param2 = numpy.require(param2, dtype=val_dtype, requirements=['C'])
        param3 = _flatten_specifier(param3)
        param4 = numpy.require(param4, dtype=val_dtype, requirements=['C'])
        param5 = numpy.require(param5, dtype=val_dtype, requirements=['C'])
        ctype = ctypes.c_float if val_dtype == numpy.float32 else ctypes.c_double
        ret0 = ctypes.pointer(ctypes.pointer(rt.make_nd_memref_descriptor(1, ctype)()))
        entry = self.libHandle.py_spmv_f32 if val_dtype == numpy.float32 else self.libHandle.py_spmv
        entry(ret0,
              ctypes.pointer(rt.get_ranked_memref_descriptor(param0)),
              ctypes.pointer(rt.get_ranked_memref_descriptor(param1)),
              ctypes.pointer(rt.get_ranked_memref_descriptor(param2)),
              param3.ctypes.data_as(ctypes.c_void_p),
              ctypes.pointer(rt.get_ranked_memref_descriptor(param4)),
              ctypes.pointer(rt.get_ranked_memref_descriptor(param5)))
        return (rt.ranked_memref_to_numpy(ret0[0]))

    # torch.mv export, entry `main` renamed lapis_main      (examples/spmv.py:47)
    def lapis_main(self, param0, param1, param2, param3, param4):
        param0 = numpy.require(param0, dtype=numpy.int32, requirements=['C'])
        param1 = numpy.require(param1, dtype=numpy.int32, requirements=['C'])
        param2 = numpy.require(param2, dtype=numpy.float64, requirements=['C'])
        param3 = _flatten_specifier(param3)
        param4 = numpy.require(param4, dtype=numpy.float64, requirements=['C'])
        ret0 = ctypes.pointer(ctypes.pointer(rt.make_nd_memref_descriptor(1, ctypes.c_double)()))
        self.libHandle.py_lapis_main(ret0,
                                     ctypes.pointer(rt.get_ranked_memref_descriptor(param0)),
                                     ctypes.pointer(rt.get_ranked_memref_descriptor(param1)),
                                     ctypes.pointer(rt.get_ranked_memref_descriptor(param2)),
                                     param3.ctypes.data_as(ctypes.c_void_p),
                                     ctypes.pointer(rt.get_ranked_memref_descriptor(param4)))
        return (rt.ranked_memref_to_numpy(ret0[0]))

    # func @pcg(A, b, dinv, tol, maxiter) -> (x, iters, relres)      (examples/pcg_solve.py:52,129)
    def pcg(self, param0, param1, param2, param3, param4, param5, param6, param7):
        param0 = numpy.require(param0, dtype=numpy.int32, requirements=['C'])
        param1 = numpy.require(param1, dtype=numpy.int32, requirements=['C'])
        param2 = numpy.require(param2, dtype=numpy.float64, requirements=['C'])
        param3 = _flatten_specifier(param3)
        param4 = numpy.require(param4, dtype=numpy.float64, requirements=['C'])
        param5 = numpy.require(param5, dtype=numpy.float64, requirements=['C'])
        param6 = ctypes.c_double(param6)
        param7 = ctypes.c_ulong(param7)
        ret0 = ctypes.pointer(ctypes.pointer(rt.make_nd_memref_descriptor(1, ctypes.c_double)()))
        ret1 = numpy.zeros(1, dtype=numpy.uint64)
        ret2 = numpy.zeros(1, dtype=numpy.float64)
        self.libHandle.py_pcg(ret0, ret1.ctypes.data_as(ctypes.c_void_p), ret2.ctypes.data_as(ctypes.c_void_p),
                              ctypes.pointer(rt.get_ranked_memref_descriptor(param0)),
                              ctypes.pointer(rt.get_ranked_memref_descriptor(param1)),
                              ctypes.pointer(rt.get_ranked_memref_descriptor(param2)),
                              param3.ctypes.data_as(ctypes.c_void_p),
                              ctypes.pointer(rt.get_ranked_memref_descriptor(param4)),
                              ctypes.pointer(rt.get_ranked_memref_descriptor(param5)),
                              param6, param7)
        return (rt.ranked_memref_to_numpy(ret0[0]), ret1[0], ret2[0])

    # CSR x dense matmul, C += A B in place     (decomposed-CSR form of examples/spmm_dcsr_opdsl.py:73-110)
    def spmm(self, param0, param1, param2, param3, param4, param5):
        val_dtype = numpy.float64 if numpy.asarray(param2).dtype == numpy.float64 else numpy.float32
        param0 = numpy.require(param0, dtype=numpy.int32, requirements=['C'])
        param1 = numpy.require(param1, dtype=numpy.int32, requirements=['C'])
        param2 = numpy.require(param2, dtype=val_dtype, requirements=['C'])
        param3 = _flatten_specifier(param3)
        param4 = numpy.require(param4, dtype=val_dtype, requirements=['C'])
        param5 = numpy.require(param5, dtype=val_dtype, requirements=['C'])
        ctype = ctypes.c_double if val_dtype == numpy.float64 else ctypes.c_float
        ret0 = ctypes.pointer(ctypes.pointer(rt.make_nd_memref_descriptor(2, ctype)()))
        entry = self.libHandle.py_spmm_f64 if val_dtype == numpy.float64 else self.libHandle.py_spmm
        entry(ret0,
              ctypes.pointer(rt.get_ranked_memref_descriptor(param0)),
              ctypes.pointer(rt.get_ranked_memref_descriptor(param1)),
              ctypes.pointer(rt.get_ranked_memref_descriptor(param2)),
              param3.ctypes.data_as(ctypes.c_void_p),
              ctypes.pointer(rt.get_ranked_memref_descriptor(param4)),
              ctypes.pointer(rt.get_ranked_memref_descriptor(param5)))
        return (rt.ranked_memref_to_numpy(ret0[0]))

    # func @pte_local_bspmm(A: CSRV, B) -> out      (examples/bspmm.py:26-52, called at :103)
    def pte_local_bspmm(self, param0, param1, param2, param3, param4):
        param0 = numpy.require(param0, dtype=numpy.int32, requirements=['C'])
        param1 = numpy.require(param1, dtype=numpy.int32, requirements=['C'])
        param2 = numpy.require(param2, dtype=numpy.float32, requirements=['C'])
        spec = numpy.zeros(6, dtype=numpy.int64)  # ((n1, n2, nh), (n1+1, nnz, nnz*nh)) flattened
        spec[0:3] = param3[0]
        spec[3:6] = param3[1]
        param4 = numpy.require(param4, dtype=numpy.float32, requirements=['C'])
        ret0 = ctypes.pointer(ctypes.pointer(rt.make_nd_memref_descriptor(3, ctypes.c_float)()))
        self.libHandle.py_pte_local_bspmm(ret0,
                                          ctypes.pointer(rt.get_ranked_memref_descriptor(param0)),
                                          ctypes.pointer(rt.get_ranked_memref_descriptor(param1)),
                                          ctypes.pointer(rt.get_ranked_memref_descriptor(param2)),
                                          spec.ctypes.data_as(ctypes.c_void_p),
                                          ctypes.pointer(rt.get_ranked_memref_descriptor(param4)))
        return (rt.ranked_memref_to_numpy(ret0[0]))

    # func @plus_norm(x, y) -> (x+y, norm)      (examples/multiple_results.py:8,34)
    def plus_norm(self, param0, param1):
        param0 = numpy.require(param0, dtype=numpy.float64, requirements=['C'])
        param1 = numpy.require(param1, dtype=numpy.float64, requirements=['C'])
        ret0 = ctypes.pointer(ctypes.pointer(rt.make_nd_memref_descriptor(1, ctypes.c_double)()))
        ret1 = numpy.zeros(1, dtype=numpy.float64)
        self.libHandle.py_plus_norm(ret0, ret1.ctypes.data_as(ctypes.c_void_p),
                                    ctypes.pointer(rt.get_ranked_memref_descriptor(param0)),
                                    ctypes.pointer(rt.get_ranked_memref_descriptor(param1)))
        return (rt.ranked_memref_to_numpy(ret0[0]), ret1[0])

    # func @mht(A, mask, d, alpha, tol, maxiter) -> (mom1, mom2)      (examples/hitting_times.py:153,216)
    def mht(self, param0, param1, param2, param3, param4, param5, param6, param7, param8):
        param0 = numpy.require(param0, dtype=numpy.int32, requirements=['C'])
        param1 = numpy.require(param1, dtype=numpy.int32, requirements=['C'])
        param2 = numpy.require(param2, dtype=numpy.float64, requirements=['C'])
        param3 = _flatten_specifier(param3)
        param4 = numpy.require(param4, dtype=numpy.float64, requirements=['C'])
        param5 = numpy.require(param5, dtype=numpy.float64, requirements=['C'])
        param6 = ctypes.c_double(param6)
        param7 = ctypes.c_double(param7)
        param8 = ctypes.c_ulong(param8)
        ret0 = ctypes.pointer(ctypes.pointer(rt.make_nd_memref_descriptor(1, ctypes.c_double)()))
        ret1 = ctypes.pointer(ctypes.pointer(rt.make_nd_memref_descriptor(1, ctypes.c_double)()))
        self.libHandle.py_mht(ret0, ret1,
                              ctypes.pointer(rt.get_ranked_memref_descriptor(param0)),
                              ctypes.pointer(rt.get_ranked_memref_descriptor(param1)),
                              ctypes.pointer(rt.get_ranked_memref_descriptor(param2)),
                              param3.ctypes.data_as(ctypes.c_void_p),
                              ctypes.pointer(rt.get_ranked_memref_descriptor(param4)),
                              ctypes.pointer(rt.get_ranked_memref_descriptor(param5)),
                              param6, param7, param8)
        return (rt.ranked_memref_to_numpy(ret0[0]), rt.ranked_memref_to_numpy(ret1[0]))

    # func @normalize_mom2(mom1, mom2) -> stdev      (examples/hitting_times.py:181,218)
    def normalize_mom2(self, param0, param1):
        param0 = numpy.require(param0, dtype=numpy.float64, requirements=['C'])
        param1 = numpy.require(param1, dtype=numpy.float64, requirements=['C'])
        ret0 = ctypes.pointer(ctypes.pointer(rt.make_nd_memref_descriptor(1, ctypes.c_double)()))
        self.libHandle.py_normalize_mom2(ret0,
                                         ctypes.pointer(rt.get_ranked_memref_descriptor(param0)),
                                         ctypes.pointer(rt.get_ranked_memref_descriptor(param1)))
        return (rt.ranked_memref_to_numpy(ret0[0]))
