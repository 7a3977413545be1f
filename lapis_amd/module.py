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


class LAPISModule:
    def __init__(self, libPath=None):
        libPath = libPath or DEFAULT_MODULE_PATH
        if not os.path.exists(libPath):
            raise FileNotFoundError(
                "%s not found: build the HIP libraries first (python -m lapis_amd.build)" % libPath)
        self.libHandle = ctypes.CDLL(libPath)
        self.libHandle.lapis_initialize.restype = None
        self.libHandle.lapis_finalize.restype = None
        self.libHandle.lapis_initialize()

    def __del__(self):
        handle = getattr(self, "libHandle", None)
        if handle is not None:
            handle.lapis_finalize()

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
