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


def _value_dtype(array):
    return numpy.float32 if numpy.asarray(array).dtype == numpy.float32 else numpy.float64


class DualView:
    """A numpy array (float64, or float32 if it is given as such) paired with a device copy that stays
    allocated between calls: the role of LAPIS::DualView (LAPISSupport.hpp:136-426) with its lazy
    modified-host / modified-device flags.  ``host`` is the numpy side; after writing to it call
    ``modify_host()``; ``sync_host()`` brings a result back (and waits for the kernels that produce it).
    Arrays of more than one dimension are kept row-major; ``host`` has the caller's shape."""

    def __init__(self, module, array):
        self._module = module  # keeps the library initialised for as long as the view lives
        self._lib = module.libHandle
        self.dtype = _value_dtype(array)
        self._tag = "f32" if self.dtype == numpy.float32 else "f64"
        self.host = numpy.require(array, dtype=self.dtype, requirements=['C', 'W'])
        create = getattr(self._lib, "lapis_dualview_%s_create" % self._tag)
        self._handle = ctypes.c_void_p(create(self.host.ctypes.data_as(ctypes.c_void_p), ctypes.c_int64(self.host.size)))

    def _call(self, what):
        getattr(self._lib, "lapis_dualview_%s_%s" % (self._tag, what))(self._handle)

    def modify_host(self):
        self._call("modify_host")
        return self

    def sync_host(self):
        self._call("sync_host")
        return self.host

    def sync_device(self):
        self._call("sync_device")
        return self

    def release(self):
        if self._handle:
            self._call("destroy")
            self._handle = None

    def __del__(self):
        try:
            self.release()
        except Exception:
            pass


class ResidentCsr:
    """A CSR matrix uploaded once (``LAPISModule.bind_csr``): device copies, plan and, where the library
    recommends it, the column-blocked copy are reused by every ``spmv`` / ``spmm`` / ``pcg``.  The values
    are float64, or float32 if they are given as such; vector operands must have the matrix's type."""

    def __init__(self, module, pos, crd, val, spec):
        self._module = module  # keeps the library initialised for as long as the matrix lives
        self._lib = module.libHandle
        self.dtype = _value_dtype(val)
        self._prefix = "lapis_resident_csr_f32_" if self.dtype == numpy.float32 else "lapis_resident_csr_"
        pos = numpy.require(pos, dtype=numpy.int32, requirements=['C'])
        crd = numpy.require(crd, dtype=numpy.int32, requirements=['C'])
        val = numpy.require(val, dtype=self.dtype, requirements=['C'])
        flat = _flatten_specifier(spec)
        self.shape = (int(flat[0]), int(flat[1]))
        self._handle = ctypes.c_void_p(self._fn("create")(
            ctypes.pointer(rt.get_ranked_memref_descriptor(pos)), ctypes.pointer(rt.get_ranked_memref_descriptor(crd)),
            ctypes.pointer(rt.get_ranked_memref_descriptor(val)), flat.ctypes.data_as(ctypes.c_void_p)))

    def _fn(self, what):
        return getattr(self._lib, self._prefix + what)

    def _views(self, *operands):
        """DualViews of the operands (made for the call where numpy arrays are given) and which ones are ours."""
        views = [v if isinstance(v, DualView) else DualView(self._module, numpy.asarray(v, dtype=self.dtype)) for v in operands]
        for v in views:
            if v.dtype != self.dtype:
                raise TypeError("operand is %s, the matrix holds %s" % (v.dtype.__name__, self.dtype.__name__))
        return views

    def update_values(self, val):
        val = numpy.require(val, dtype=self.dtype, requirements=['C'])
        self._fn("update_values")(self._handle, ctypes.pointer(rt.get_ranked_memref_descriptor(val)))

    def _finish(self, out_view, given, views, operands):
        """In-place contract for numpy operands: fetch the result, write it through to the caller's array."""
        out = out_view.sync_host()
        if isinstance(given, numpy.ndarray) and out is not given:
            given[...] = out.reshape(given.shape)  # numpy.require had to copy (dtype or layout)
            out = given
        for v, g in zip(views, operands):
            if v is not g:
                v.release()
        return out

    def spmv(self, x, y):
        """y += A x.  With ``DualView`` operands nothing crosses PCIe and the call returns before the kernel
        has run (``y.sync_host()`` fetches the result); numpy operands are copied in and out as
        ``LAPISModule.spmv`` does, and the updated ``y`` is returned."""
        xv, yv = self._views(x, y)
        self._fn("spmv")(self._handle, xv._handle, yv._handle)
        if xv is x and yv is y:
            return y
        return self._finish(yv, y, (xv, yv), (x, y))

    def spmm(self, B, C):
        """C += A B for row-major B (columns x k) and C (rows x k); operands as in ``spmv``."""
        Bv, Cv = self._views(B, C)
        if Bv.host.ndim != 2 or Cv.host.ndim != 2 or Bv.host.shape[1] != Cv.host.shape[1]:
            raise ValueError("spmm takes two-dimensional B and C with the same number of columns")
        if Bv.host.shape[0] < self.shape[1] or Cv.host.shape[0] < self.shape[0]:
            raise ValueError("spmm: B needs %d rows and C %d" % (self.shape[1], self.shape[0]))
        self._fn("spmm")(self._handle, Bv._handle, ctypes.c_int64(Bv.host.shape[1]), Cv._handle)
        if Bv is B and Cv is C:
            return C
        return self._finish(Cv, C, (Bv, Cv), (B, C))

    def pcg(self, b, dinv, tol, maxiter, x=None):
        """``func @pcg`` of examples/pcg_solve.py:52 on the resident matrix (float64): returns (x, iterations,
        relative residual).  ``dinv`` None runs unpreconditioned CG.  With a ``DualView`` x the solution stays on
        the device (``x.sync_host()`` fetches it)."""
        if self.dtype != numpy.float64:
            raise TypeError("pcg is implemented for float64 matrices")
        n = self.shape[0]
        given_x = x
        if x is None:
            x = numpy.zeros(n, dtype=numpy.float64)
        operands = [b, x] + ([dinv] if dinv is not None else [])
        views = self._views(*operands)
        bv, xv = views[0], views[1]
        dv = views[2]._handle if dinv is not None else None
        iters, relres = ctypes.c_size_t(0), ctypes.c_double(0.0)
        self._lib.lapis_resident_csr_pcg(self._handle, bv._handle, dv, ctypes.c_double(tol), ctypes.c_size_t(maxiter),
                                         xv._handle, ctypes.byref(iters), ctypes.byref(relres))
        if isinstance(given_x, DualView):
            out = given_x
            for v, g in zip(views, operands):
                if v is not g:
                    v.release()
        else:
            out = self._finish(xv, x, views, operands)
        return out, iters.value, relres.value

    def release(self):
        if self._handle:
            self._fn("destroy")(self._handle)
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
        vp = ctypes.c_void_p
        for tag in ("f64", "f32"):
            create = getattr(self.libHandle, "lapis_dualview_%s_create" % tag)
            create.restype, create.argtypes = vp, [vp, ctypes.c_int64]
            for fn in ("modify_host", "modify_device", "sync_host", "sync_device", "destroy"):
                f = getattr(self.libHandle, "lapis_dualview_%s_%s" % (tag, fn))
                f.restype, f.argtypes = None, [vp]
        for prefix in ("lapis_resident_csr_", "lapis_resident_csr_f32_"):
            fn = lambda what: getattr(self.libHandle, prefix + what)
            fn("create").restype = vp
            fn("update_values").restype, fn("update_values").argtypes = None, [vp, vp]
            fn("spmv").restype, fn("spmv").argtypes = None, [vp, vp, vp]
            fn("spmm").restype, fn("spmm").argtypes = None, [vp, vp, ctypes.c_int64, vp]
            fn("destroy").restype, fn("destroy").argtypes = None, [vp]
        self.libHandle.lapis_resident_csr_pcg.restype = None
        self.libHandle.lapis_resident_csr_pcg.argtypes = [vp, vp, vp, ctypes.c_double, ctypes.c_size_t, vp,
                                                          ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_double)]
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
        """An array (float64, or float32 if given as such) that keeps a device copy between calls (see ``DualView``)."""
        return DualView(self, array)

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
