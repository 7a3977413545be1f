"""ctypes binding of the C-ABI kernel library (include/lapis_hip.h).

Pointers are DEVICE addresses: pass ``torch`` CUDA tensors (their ``data_ptr()`` is
taken), or plain integers.  ``stream`` is a ``torch.cuda.Stream``, a raw
``hipStream_t`` value, or None for torch's current stream.  The library has no CPU
path: loading fails loudly when it has not been built.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "liblapis_hip.so")

SPMV_AUTO, SPMV_SUBWARP, SPMV_ROWBLOCK, SPMV_NNZSPLIT, SPMV_COLBLOCK = 0, 1, 2, 3, 4
KERNEL_NAMES = {SPMV_AUTO: "auto", SPMV_SUBWARP: "subwarp", SPMV_ROWBLOCK: "rowblock", SPMV_NNZSPLIT: "nnzsplit",
                SPMV_COLBLOCK: "colblock"}

_i64, _u64, _vp, _int = ctypes.c_int64, ctypes.c_uint64, ctypes.c_void_p, ctypes.c_int
_dbl, _flt = ctypes.c_double, ctypes.c_float


class LapisHipError(RuntimeError):
    def __init__(self, status, name, message):
        super().__init__("%s (%d): %s" % (name, status, message))
        self.status = status
        self.status_name = name


class CsrStats(ctypes.Structure):
    _fields_ = [("nrows", _i64), ("ncols", _i64), ("nnz", _i64),
                ("min_row_len", _i64), ("max_row_len", _i64), ("empty_rows", _i64),
                ("mean_row_len", _dbl), ("var_row_len", _dbl), ("mean_chunk_col_span", _dbl),
                ("reference_hint", _i64), ("reference_vector_length", ctypes.c_int32),
                ("kernel", ctypes.c_int32), ("width", ctypes.c_int32), ("chunk", ctypes.c_int32),
                ("colblock_recommended", ctypes.c_int32), ("colblock_layout", ctypes.c_int32),
                ("near_diagonal_fraction", _dbl * 4)]

    def as_dict(self):
        d = {k: getattr(self, k) for k, _ in self._fields_}
        d["near_diagonal_fraction"] = list(self.near_diagonal_fraction)
        d["kernel_name"] = KERNEL_NAMES.get(self.kernel, "?")
        d["colblock_layout_name"] = {0: None, 1: "wave", 2: "group"}.get(self.colblock_layout)
        return d


class _CalibrateMode(ctypes.Structure):
    _fields_ = [(name, ctypes.c_int) for name in (
        "threads", "workgroups", "stream_in_flight", "gathers_in_flight", "lanes_per_line", "roles", "producers",
        "stream_behind", "stream_policy", "stream_in_l2", "scalar", "scalar_ahead", "scalar_stride")]


_SIGNATURES = {
    "lapis_hip_init": [],
    "lapis_hip_finalize": [],
    "lapis_hip_stream_synchronize": [_vp],
    "lapis_hip_kernel_timing_start": [_int],
    "lapis_hip_kernel_timing_stop": [ctypes.POINTER(_int), ctypes.POINTER(_dbl), ctypes.POINTER(_dbl),
                                     ctypes.POINTER(_dbl)],
    "lapis_hip_calibrate_gather": [_vp, _i64, _int, _vp, _i64, _i64, _vp, ctypes.POINTER(_dbl), ctypes.POINTER(_dbl),
                                   ctypes.POINTER(_dbl), _vp],
    "lapis_hip_calibrate_mix": [ctypes.POINTER(_CalibrateMode), _vp, _i64, _vp, _i64, _i64, _i64, _vp, _vp,
                                ctypes.POINTER(_dbl), ctypes.POINTER(_dbl), ctypes.POINTER(_dbl), ctypes.POINTER(_int),
                                _vp],
    "lapis_hip_csr_plan_create": [ctypes.POINTER(_vp), _i64, _i64, _i64, _vp, _vp, _int, _vp],
    "lapis_hip_csr_plan_set_kernel": [_vp, _int, _int],
    "lapis_hip_csr_plan_get_stats": [_vp, ctypes.POINTER(CsrStats)],
    "lapis_hip_csr_plan_destroy": [_vp],
    "lapis_hip_csr_plan_build_colblock": [_vp, _vp, _vp, _int, _int, _int, _vp],
    "lapis_hip_csr_plan_analyze": [_vp, _vp, _vp, _int, _vp],
    "lapis_hip_csr_plan_update_values": [_vp, _vp, _int, _vp],
    "lapis_hip_csr_plan_check": [_vp, _vp],
    "lapis_hip_csr_plan_matches": [_vp, _i64, _i64, _i64, _vp, _vp],
    "lapis_hip_csr_plan_analyze_reproducible": [_vp, _vp, _vp, _int, _vp],
    "lapis_hip_spmv_csr_f64_i32": [_vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp],
    "lapis_hip_spmv_csr_f32_i32": [_vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp],
    "lapis_hip_spmm_csr_f32_i32": [_i64, _i64, _i64, _vp, _vp, _vp, _vp, _i64, _vp, _i64, _vp],
    "lapis_hip_spmm_csr_f64_i32": [_i64, _i64, _i64, _vp, _vp, _vp, _vp, _i64, _vp, _i64, _vp],
    "lapis_hip_spmm_csr_f32_i32_plan": [_vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _i64, _vp, _i64, _vp],
    "lapis_hip_spmm_csr_f64_i32_plan": [_vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _i64, _vp, _i64, _vp],
    "lapis_hip_bspmm_csrv_f32_i32": [_i64, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp],
    "lapis_hip_dot_f64": [_i64, _vp, _vp, _dbl, _vp, _vp],
    "lapis_hip_dot_f32": [_i64, _vp, _vp, _flt, _vp, _vp],
    "lapis_hip_dot_f64_noalloc": [_i64, _vp, _vp, _dbl, _vp, _vp],
    "lapis_hip_dot_f64_host": [_i64, _vp, _vp, _dbl, ctypes.POINTER(_dbl), _vp],
    "lapis_hip_dot_f32_host": [_i64, _vp, _vp, _flt, ctypes.POINTER(_flt), _vp],
    "lapis_hip_axpby_dot_f64": [_i64, _dbl, _vp, _dbl, _vp, _vp, _vp, _dbl, _vp, _vp],
    "lapis_hip_axpby_dot_f32": [_i64, _flt, _vp, _flt, _vp, _vp, _vp, _flt, _vp, _vp],
    "lapis_hip_axpby_f64": [_i64, _dbl, _vp, _dbl, _vp, _vp, _vp],
    "lapis_hip_axpby_f32": [_i64, _flt, _vp, _flt, _vp, _vp, _vp],
    "lapis_hip_mult_f64": [_i64, _vp, _vp, _vp, _vp],
    "lapis_hip_mult_f32": [_i64, _vp, _vp, _vp, _vp],
    "lapis_hip_div_f64": [_i64, _vp, _vp, _vp, _vp],
    "lapis_hip_div_f32": [_i64, _vp, _vp, _vp, _vp],
    "lapis_hip_fill_f64": [_i64, _dbl, _vp, _vp],
    "lapis_hip_fill_f32": [_i64, _flt, _vp, _vp],
    "lapis_hip_copy_f64": [_i64, _vp, _vp, _vp],
    "lapis_hip_copy_f32": [_i64, _vp, _vp, _vp],
    "lapis_hip_scale_f64": [_i64, _dbl, _vp, _vp],
    "lapis_hip_pcg_masked_f64_i32": [_vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _dbl, _u64, _vp,
                                     ctypes.POINTER(_u64), ctypes.POINTER(_dbl), _vp, _vp],
    "lapis_hip_mht_f64_i32": [_vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _dbl, _dbl, _u64, _vp, _vp, _vp],
    "lapis_hip_normalize_mom2_f64": [_i64, _vp, _vp, _vp, _vp],
    "lapis_hip_pcg_f64_i32": [_vp, _i64, _vp, _vp, _vp, _vp, _vp, _dbl, _u64, _vp,
                              ctypes.POINTER(_u64), ctypes.POINTER(_dbl), _vp, _vp],
}

# every symbol include/lapis_hip.h declares
EXPORTED_SYMBOLS = sorted(list(_SIGNATURES) + ["lapis_hip_last_error", "lapis_hip_status_name",
                                             "lapis_hip_spmm_last_kernel", "lapis_hip_kernel_timing_median_ms",
                                             "lapis_hip_csr_plan_kernel_name"])

_lib = None


def load(path=None):
    """Load the kernel library (without initialising the device)."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    path = path or LIB_PATH
    if not os.path.exists(path):
        raise FileNotFoundError("%s not found: build it first (python -m lapis_amd.build); "
                                "there is no CPU fallback" % path)
    lib = ctypes.CDLL(path)
    for name, argtypes in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = _int
    lib.lapis_hip_last_error.restype = ctypes.c_char_p
    lib.lapis_hip_spmm_last_kernel.restype = ctypes.c_char_p
    lib.lapis_hip_csr_plan_kernel_name.restype = ctypes.c_char_p
    lib.lapis_hip_csr_plan_kernel_name.argtypes = [_vp]
    lib.lapis_hip_kernel_timing_median_ms.restype = _dbl
    lib.lapis_hip_kernel_timing_median_ms.argtypes = []
    lib.lapis_hip_status_name.restype = ctypes.c_char_p
    lib.lapis_hip_status_name.argtypes = [_int]
    _lib = lib
    return lib


def check(status):
    if status != 0:
        lib = load()
        raise LapisHipError(status, lib.lapis_hip_status_name(status).decode(), lib.lapis_hip_last_error().decode())


_initialized = False


def init():
    """lapis_hip_init() once per process (needs a gfx950 device)."""
    global _initialized
    lib = load()
    if not _initialized:
        check(lib.lapis_hip_init())
        _initialized = True
    return lib


def _ptr(t):
    if t is None:
        return None
    if isinstance(t, int):
        return t
    return t.data_ptr()


def _stream(stream):
    if stream is None:
        import torch
        return torch.cuda.current_stream().cuda_stream
    if isinstance(stream, int):
        return stream
    return stream.cuda_stream


def kernel_timing_start(capacity):
    """Attach HIP event pairs to the next ``capacity`` dominant-kernel launches."""
    check(init().lapis_hip_kernel_timing_start(capacity))


def kernel_timing_stop():
    """-> dict(count, mean_ms, median_ms, min_ms, max_ms) of the launches timed since the start call."""
    n, mean, mn, mx = _int(0), _dbl(0), _dbl(0), _dbl(0)
    lib = init()
    check(lib.lapis_hip_kernel_timing_stop(ctypes.byref(n), ctypes.byref(mean), ctypes.byref(mn), ctypes.byref(mx)))
    return {"count": n.value, "mean_ms": mean.value, "median_ms": lib.lapis_hip_kernel_timing_median_ms(),
            "min_ms": mn.value, "max_ms": mx.value}


COLBLOCK_LAYOUTS = {"auto": 0, "wave": 1, "group": 2}


class CsrPlan:
    """Row-length statistics of one CSR matrix and the SpMV kernel chosen from them."""

    def __init__(self, nrows, ncols, pos, crd, value_bytes=8, stream=None, nnz=None):
        lib = init()
        self._lib = lib
        self._handle = _vp()
        self.pos, self.crd = pos, crd  # keep the buffers alive: the plan holds pos by address
        if nnz is None:
            nnz = int(crd.shape[0])
        check(lib.lapis_hip_csr_plan_create(ctypes.byref(self._handle), nrows, ncols, nnz, _ptr(pos), _ptr(crd),
                                            value_bytes, _stream(stream)))

    @property
    def handle(self):
        return self._handle

    def stats(self):
        s = CsrStats()
        check(self._lib.lapis_hip_csr_plan_get_stats(self._handle, ctypes.byref(s)))
        return s.as_dict()

    def set_kernel(self, kernel, width=0):
        check(self._lib.lapis_hip_csr_plan_set_kernel(self._handle, kernel, width))
        return self

    def build_colblock(self, crd, val, slice_log2_cols=0, layout="auto", stream=None):
        """Copy the matrix into a column-blocked layout ("wave", "group" or "auto") and select that kernel."""
        check(self._lib.lapis_hip_csr_plan_build_colblock(self._handle, _ptr(crd), _ptr(val), val.element_size(),
                                                          COLBLOCK_LAYOUTS[layout], slice_log2_cols,
                                                          _stream(stream)))
        return self.set_kernel(SPMV_COLBLOCK)

    def analyze(self, crd, val, stream=None):
        """Let the library decide, with the values in hand, whether the column-blocked copy pays; builds it if so."""
        check(self._lib.lapis_hip_csr_plan_analyze(self._handle, _ptr(crd), _ptr(val), val.element_size(),
                                                   _stream(stream)))
        return self

    def analyze_reproducible(self, crd, val, stream=None):
        """analyze() for callers that need the same bits from every run (per-wavefront layout where the copy pays)."""
        check(self._lib.lapis_hip_csr_plan_analyze_reproducible(self._handle, _ptr(crd), _ptr(val), val.element_size(),
                                                                _stream(stream)))
        return self

    def kernel_name(self):
        """Name of the SpMV kernel a launch with this plan runs."""
        return self._lib.lapis_hip_csr_plan_kernel_name(self._handle).decode()

    def matches(self, nrows, ncols, nnz, pos, crd):
        """Was this plan made for exactly this structure (sizes, number of non-zeros, position and coordinate buffers)?"""
        return bool(self._lib.lapis_hip_csr_plan_matches(self._handle, nrows, ncols, nnz, _ptr(pos), _ptr(crd)))

    def update_values(self, val, stream=None):
        """Refresh the values of the column-blocked copy after ``val`` changed (no-op without a copy)."""
        check(self._lib.lapis_hip_csr_plan_update_values(self._handle, _ptr(val), val.element_size(), _stream(stream)))
        return self

    def check(self, stream=None):
        """Wait for the stream and raise if a kernel of this plan gave up a bounded wait between its wavefronts."""
        check(self._lib.lapis_hip_csr_plan_check(self._handle, _stream(stream)))
        return self

    def destroy(self):
        if self._handle:
            self._lib.lapis_hip_csr_plan_destroy(self._handle)
            self._handle = _vp()

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


def _suffix(t):
    import torch
    if t.dtype == torch.float64:
        return "f64"
    if t.dtype == torch.float32:
        return "f32"
    raise TypeError("values must be float32 or float64, got %s" % t.dtype)


def _holds(what, n, *tensors, like=None):
    """The C ABI takes pointers and counts: a tensor with fewer than ``n`` elements, of another element type
    than ``like`` or with gaps between its elements would be read or written past its end on the device, so it
    is refused here.  Raw addresses (ints) and None pass: the caller vouches for them."""
    for t in tensors:
        if t is None or isinstance(t, int):
            continue
        if t.numel() < n:
            raise ValueError("%s: an operand of %d elements where %d are needed" % (what, t.numel(), n))
        if like is not None and not isinstance(like, int) and t.dtype != like.dtype:
            raise TypeError("%s: operands of %s and %s" % (what, t.dtype, like.dtype))
        if not t.is_contiguous():
            raise ValueError("%s: an operand that is not contiguous" % what)


def _indices(what, *tensors):
    import torch
    for t in tensors:
        if t is not None and not isinstance(t, int) and t.dtype != torch.int32:
            raise TypeError("%s: positions and coordinates are int32, got %s" % (what, t.dtype))


def spmv(plan, nrows, ncols, pos, crd, val, x, y, stream=None):
    """y += A x.  ``plan`` may be None: the launch then follows the reference's own rule."""
    _indices("spmv", pos, crd)
    _holds("spmv", nrows + 1, pos)
    _holds("spmv", ncols, x, like=val)
    _holds("spmv", nrows, y, like=val)
    if not isinstance(crd, int) and not isinstance(val, int) and crd is not None and val is not None:
        _holds("spmv", crd.numel(), val)
    lib = init()
    fn = getattr(lib, "lapis_hip_spmv_csr_%s_i32" % _suffix(val))
    check(fn(plan.handle if plan is not None else None, nrows, ncols, _ptr(pos), _ptr(crd), _ptr(val), _ptr(x),
             _ptr(y), _stream(stream)))
    return y


def spmm(nrows, ncols, pos, crd, val, B, C, stream=None, plan=None):
    """C += A B with row-major B (ncols x k) and C (nrows x k); with a plan its statistics pick the kernel."""
    k = int(C.shape[1])
    _indices("spmm", pos, crd)
    _holds("spmm", nrows + 1, pos)
    _holds("spmm", crd.numel(), val)
    if B.dim() != 2 or C.dim() != 2 or int(B.shape[1]) != k or B.shape[0] < ncols or C.shape[0] < nrows or \
            B.stride(1) != 1 or C.stride(1) != 1 or B.dtype != val.dtype or C.dtype != val.dtype:
        raise ValueError("spmm: a %d x %d matrix of %s times B %s into C %s" % (
            nrows, ncols, val.dtype, tuple(B.shape), tuple(C.shape)))
    lib = init()
    if plan is not None:
        fn = getattr(lib, "lapis_hip_spmm_csr_%s_i32_plan" % _suffix(val))
        check(fn(plan.handle, nrows, ncols, k, _ptr(pos), _ptr(crd), _ptr(val), _ptr(B), int(B.stride(0)), _ptr(C),
                 int(C.stride(0)), _stream(stream)))
        return C
    fn = getattr(lib, "lapis_hip_spmm_csr_%s_i32" % _suffix(val))
    check(fn(nrows, ncols, k, _ptr(pos), _ptr(crd), _ptr(val), _ptr(B), int(B.stride(0)), _ptr(C), int(C.stride(0)),
             _stream(stream)))
    return C


def spmm_last_kernel():
    """Name of the kernel this thread's last ``spmm`` call launched."""
    return init().lapis_hip_spmm_last_kernel().decode()


def dot(x, y, result, init_value=0.0, stream=None):
    """result[0] = init + x.y, with ``result`` a one-element device tensor (no host sync)."""
    _holds("dot", int(x.shape[0]), x, y, like=x)
    _holds("dot", 1, result, like=x)
    lib = init()
    fn = getattr(lib, "lapis_hip_dot_%s" % _suffix(x))
    check(fn(int(x.shape[0]), _ptr(x), _ptr(y), init_value, _ptr(result), _stream(stream)))
    return result


def calibrate_gather(x, window_bytes, lanes_per_line, stream_buf, gathers, sink, stream=None):
    """One row of the gather/stream calibration table: dict(ms, gathers, stream_bytes)."""
    lib = init()
    ms, done, sbytes = _dbl(0.0), _dbl(0.0), _dbl(0.0)
    check(lib.lapis_hip_calibrate_gather(_ptr(x) if x is not None else None, window_bytes, lanes_per_line,
                                         _ptr(stream_buf) if stream_buf is not None else None,
                                         stream_buf.numel() * stream_buf.element_size() if stream_buf is not None else 0,
                                         gathers, _ptr(sink), ctypes.byref(ms), ctypes.byref(done), ctypes.byref(sbytes),
                                         _stream(stream)))
    return {"ms": ms.value, "gathers": done.value, "stream_bytes": sbytes.value}


def calibrate_mix(mode, x, window_bytes, stream_buf, stream_bytes, gathers, cu_count, sink, stream=None):
    """One arrangement of streaming and gathering wavefronts (lapis_hip_calibrate_mix): ``mode`` is a dict of the
    fields of lapis_hip_calibrate_mode (missing ones are 0, lanes_per_line 1).  Returns dict(ms, gathers,
    stream_bytes, cus_with_both_roles)."""
    lib = init()
    fn = lib.lapis_hip_calibrate_mix
    m = _CalibrateMode(**dict({"lanes_per_line": 1}, **mode))
    ms, done, sbytes, both = _dbl(0.0), _dbl(0.0), _dbl(0.0), _int(-1)
    check(fn(ctypes.byref(m), _ptr(x) if x is not None else None, window_bytes,
             _ptr(stream_buf) if stream_buf is not None else None,
             stream_buf.numel() * stream_buf.element_size() if stream_buf is not None else 0, int(stream_bytes),
             int(gathers), _ptr(cu_count) if cu_count is not None else None, _ptr(sink), ctypes.byref(ms),
             ctypes.byref(done), ctypes.byref(sbytes), ctypes.byref(both), _stream(stream)))
    return {"ms": ms.value, "gathers": done.value, "stream_bytes": sbytes.value, "cus_with_both_roles": both.value}


def dot_host(x, y, init_value=0.0, stream=None):
    """init + x . y as a Python float: the entry point that returns the scalar to the host (blocking)."""
    _holds("dot", int(x.shape[0]), x, y, like=x)
    lib = init()
    out = (_dbl if x.element_size() == 8 else _flt)(0.0)
    fn = getattr(lib, "lapis_hip_dot_%s_host" % _suffix(x))
    check(fn(int(x.shape[0]), _ptr(x), _ptr(y), init_value, ctypes.byref(out), _stream(stream)))
    return out.value


def axpby_dot(a, x, b, y, dst, z, result, init_value=0.0, stream=None):
    """dst = a*x + b*y and result = init + dst . z (z None: dst . dst) in one pass."""
    _holds("axpby_dot", int(x.shape[0]), x, y, dst, z, like=x)
    _holds("axpby_dot", 1, result, like=x)
    lib = init()
    fn = getattr(lib, "lapis_hip_axpby_dot_%s" % _suffix(x))
    check(fn(int(x.shape[0]), a, _ptr(x), b, _ptr(y), _ptr(dst), _ptr(z) if z is not None else None, init_value,
             _ptr(result), _stream(stream)))
    return result


def dot_noalloc(x, y, result, init_value=0.0, stream=None):
    """dot() through the entry point that allocates nothing (fp64; fixed scratch inside the library)."""
    _holds("dot_noalloc", int(x.shape[0]), x, y, like=x)
    _holds("dot_noalloc", 1, result, like=x)
    lib = init()
    check(lib.lapis_hip_dot_f64_noalloc(int(x.shape[0]), _ptr(x), _ptr(y), init_value, _ptr(result), _stream(stream)))
    return result


def axpby(a, x, b, y, dst, stream=None):
    _holds("axpby", int(x.shape[0]), x, y, dst, like=x)
    lib = init()
    fn = getattr(lib, "lapis_hip_axpby_%s" % _suffix(x))
    check(fn(int(x.shape[0]), a, _ptr(x), b, _ptr(y), _ptr(dst), _stream(stream)))
    return dst


def mult(x, y, dst, stream=None):
    _holds("mult", int(x.shape[0]), x, y, dst, like=x)
    check(getattr(init(), "lapis_hip_mult_%s" % _suffix(x))(int(x.shape[0]), _ptr(x), _ptr(y), _ptr(dst), _stream(stream)))
    return dst


def div(x, y, dst, stream=None):
    _holds("div", int(x.shape[0]), x, y, dst, like=x)
    check(getattr(init(), "lapis_hip_div_%s" % _suffix(x))(int(x.shape[0]), _ptr(x), _ptr(y), _ptr(dst), _stream(stream)))
    return dst


def fill(dst, value, stream=None):
    lib = init()
    fn = getattr(lib, "lapis_hip_fill_%s" % _suffix(dst))
    check(fn(int(dst.shape[0]), value, _ptr(dst), _stream(stream)))
    return dst


def copy(src, dst, stream=None):
    _holds("copy", int(src.shape[0]), src, dst, like=src)
    check(getattr(init(), "lapis_hip_copy_%s" % _suffix(src))(int(src.shape[0]), _ptr(src), _ptr(dst), _stream(stream)))
    return dst


def scale(alpha, val, stream=None):
    check(init().lapis_hip_scale_f64(int(val.shape[0]), alpha, _ptr(val), _stream(stream)))
    return val


def pcg(plan, n, pos, crd, val, b, dinv, tol, maxiter, x, work=None, stream=None):
    """CG of examples/pcg_solve.py on device buffers -> (iters, relres); x is filled in place."""
    _indices("pcg", pos, crd)
    _holds("pcg", n + 1, pos)
    _holds("pcg", n, b, dinv, x, like=val)
    _holds("pcg", 4 * n, work, like=val)
    if not isinstance(crd, int) and not isinstance(val, int):
        _holds("pcg", crd.numel(), val)
    lib = init()
    iters, relres = _u64(0), _dbl(0.0)
    check(lib.lapis_hip_pcg_f64_i32(plan.handle if plan is not None else None, n, _ptr(pos), _ptr(crd), _ptr(val),
                                    _ptr(b), _ptr(dinv), tol, maxiter, _ptr(x), ctypes.byref(iters),
                                    ctypes.byref(relres), _ptr(work), _stream(stream)))
    return int(iters.value), relres.value


def pcg_masked(plan, n, pos, crd, val, b, mask, d, tol, maxiter, x, work=None, stream=None):
    """Masked CG of examples/hitting_times.py:97 on device buffers -> (iters, relres)."""
    _indices("pcg_masked", pos, crd)
    _holds("pcg_masked", n + 1, pos)
    _holds("pcg_masked", n, b, mask, d, x, like=val)
    _holds("pcg_masked", 5 * n, work, like=val)
    lib = init()
    iters, relres = _u64(0), _dbl(0.0)
    check(lib.lapis_hip_pcg_masked_f64_i32(plan.handle if plan is not None else None, n, _ptr(pos), _ptr(crd),
                                           _ptr(val), _ptr(b), _ptr(mask), _ptr(d), tol, maxiter, _ptr(x),
                                           ctypes.byref(iters), ctypes.byref(relres), _ptr(work), _stream(stream)))
    return int(iters.value), relres.value


def mht(plan, n, pos, crd, val, mask, d, alpha, tol, maxiter, mom1, mom2, stream=None):
    """Hitting-time moments of examples/hitting_times.py:153; scales ``val`` in place."""
    check(init().lapis_hip_mht_f64_i32(plan.handle if plan is not None else None, n, int(val.shape[0]), _ptr(pos),
                                       _ptr(crd), _ptr(val), _ptr(mask), _ptr(d), alpha, tol, maxiter, _ptr(mom1),
                                       _ptr(mom2), _stream(stream)))
    return mom1, mom2


def normalize_mom2(mom1, mom2, out, stream=None):
    check(init().lapis_hip_normalize_mom2_f64(int(mom1.shape[0]), _ptr(mom1), _ptr(mom2), _ptr(out), _stream(stream)))
    return out


def bspmm_csrv(n1, n2, pos, crd, val, V, out, stream=None):
    """out(n1,dh,nh) += A(n1,n2,nh) * V(n2,dh,nh) with CSRV A (examples/bspmm.py)."""
    dh, nh = int(V.shape[1]), int(V.shape[2])
    check(init().lapis_hip_bspmm_csrv_f32_i32(n1, n2, dh, nh, _ptr(pos), _ptr(crd), _ptr(val), _ptr(V), _ptr(out),
                                              _stream(stream)))
    return out
