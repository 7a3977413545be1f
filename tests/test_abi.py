"""CPU checks of the drop-in boundary: both shared libraries load without a GPU and
export every symbol the headers under include/ declare; error paths that need no
device answer with status codes."""
import ctypes
import os
import re

import numpy as np
import pytest

from conftest import ROOT
from lapis_amd import hip, memref, module


def _declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
    return sorted(set(re.findall(r"\b((?:lapis|py)_[a-z0-9_]+)\s*\(", text)))


def test_kernel_library_exports_every_declared_symbol():
    lib = hip.load()
    declared = _declared_functions("lapis_hip.h")
    assert len(declared) >= 24
    missing = [name for name in declared if not hasattr(lib, name)]
    assert missing == []
    assert sorted(hip.EXPORTED_SYMBOLS) == declared  # the Python binding covers the whole header


def test_module_library_exports_the_generated_module_symbols():
    lib = ctypes.CDLL(module.DEFAULT_MODULE_PATH)
    declared = _declared_functions("lapis_module.h")
    for required in ("lapis_initialize", "lapis_finalize", "py_spmv", "py_lapis_main", "py_pcg"):
        assert required in declared
    assert [name for name in declared if not hasattr(lib, name)] == []


def test_calls_before_init_report_not_initialized():
    lib = hip.load()
    rc = lib.lapis_hip_fill_f64(16, 0.0, None, None)
    assert lib.lapis_hip_status_name(rc) == b"LAPIS_HIP_ERR_NOT_INITIALIZED"
    assert b"lapis_hip_init" in lib.lapis_hip_last_error()
    rc = lib.lapis_hip_spmv_csr_f64_i32(None, 4, 4, None, None, None, None, None, None)
    assert lib.lapis_hip_status_name(rc) == b"LAPIS_HIP_ERR_NOT_INITIALIZED"


def test_status_names_are_distinct():
    lib = hip.load()
    names = {lib.lapis_hip_status_name(i) for i in range(8)}
    assert len(names) == 8 and lib.lapis_hip_status_name(99) == b"LAPIS_HIP_ERR_UNKNOWN"


def test_stats_struct_matches_header_layout():
    # 6 int64 + 3 double + int64 + 6 int32 + 4 double = 136 bytes, no padding surprises
    assert ctypes.sizeof(hip.CsrStats) == 6 * 8 + 3 * 8 + 8 + 6 * 4 + 4 * 8
    assert hip.CsrStats.near_diagonal_fraction.offset == 104


@pytest.mark.parametrize("dtype", [np.float64, np.float32, np.int32])
def test_memref_descriptor_round_trip(dtype):
    a = np.arange(24, dtype=dtype).reshape(4, 6)
    d = memref.get_ranked_memref_descriptor(a)
    assert list(d.shape) == [4, 6] and list(d.strides) == [6, 1] and d.offset == 0
    back = memref.ranked_memref_to_numpy(d)
    assert back.dtype == a.dtype and np.array_equal(back, a)
    back[1, 2] = 77  # aliases, does not copy
    assert a[1, 2] == 77
    v = a[:, 1]  # strided view: the descriptor reports the stride the module shim would reject
    dv = memref.get_ranked_memref_descriptor(v)
    assert list(dv.strides) == [6] and np.array_equal(memref.ranked_memref_to_numpy(dv), v)


def test_memref_descriptor_layout_is_stridedmemreftype():
    cls = memref.make_nd_memref_descriptor(1, ctypes.c_double)
    assert [f[0] for f in cls._fields_] == ["allocated", "aligned", "offset", "shape", "strides"]
    assert ctypes.sizeof(cls) == 5 * 8
    assert ctypes.sizeof(memref.make_nd_memref_descriptor(2, ctypes.c_float)) == 7 * 8


def test_specifier_flattening_matches_emitted_wrapper():
    flat = module._flatten_specifier(((5, 6), (6, 8, 8)))
    assert flat.dtype == np.int64 and list(flat) == [5, 6, 6, 8, 8]


def test_missing_library_is_an_error_not_a_fallback(tmp_path):
    with pytest.raises(FileNotFoundError, match="no CPU fallback"):
        hip.load(str(tmp_path / "liblapis_hip.so"))
    with pytest.raises(FileNotFoundError):
        module.LAPISModule(str(tmp_path / "liblapis_package_module.so"))


def test_nothing_under_the_package_reaches_for_the_oracle():
    # the oracle is test infrastructure: the product must not import, load or run it
    import os
    import re
    pkg = os.path.dirname(hip.__file__)
    offenders = []
    for root, _, files in os.walk(pkg):
        for name in files:
            if name.endswith((".py", ".hip", ".hpp", ".cpp", ".h")):
                text = open(os.path.join(root, name), errors="ignore").read()
                if re.search(r"liblapis_oracle|oracle\.oracle|from oracle|import oracle|lapis_oracle\.c", text):
                    offenders.append(os.path.join(root, name))
    assert offenders == []


def test_the_python_binding_refuses_operands_the_kernels_would_overrun():
    """lapis_amd.hip passes addresses and counts through ctypes: tensors that are too short, of another
    element type, or not contiguous are refused before the library is asked for anything (no GPU needed)."""
    import torch
    from lapis_amd import hip
    f64 = lambda n: torch.ones(n, dtype=torch.float64)
    i32 = lambda n: torch.zeros(n, dtype=torch.int32)
    x5, y4 = f64(5), f64(4)
    for call in (lambda: hip.axpby(1.0, x5, 1.0, y4, x5), lambda: hip.dot_host(x5, y4), lambda: hip.mult(x5, y4, x5),
                 lambda: hip.div(x5, x5, y4), lambda: hip.copy(x5, y4),
                 lambda: hip.spmv(None, 5, 5, i32(6), i32(9), f64(9), y4, x5),        # x shorter than the columns
                 lambda: hip.spmv(None, 5, 5, i32(5), i32(9), f64(9), x5, x5),        # positions for four rows
                 lambda: hip.spmv(None, 5, 5, i32(6), i32(9), f64(8), x5, x5),        # fewer values than coordinates
                 lambda: hip.pcg(None, 5, i32(6), i32(9), f64(9), x5, None, 0.0, 1, y4),
                 lambda: hip.pcg(None, 5, i32(6), i32(9), f64(9), x5, None, 0.0, 1, x5, work=f64(19)),
                 lambda: hip.copy(f64(10)[::2], x5),
                 lambda: hip.spmm(5, 5, i32(6), i32(9), torch.ones(9), torch.ones(4, 3), torch.ones(5, 3))):
        with pytest.raises(ValueError):
            call()
    for call in (lambda: hip.axpby(1.0, x5, 1.0, torch.ones(5), x5),
                 lambda: hip.spmv(None, 5, 5, i32(6).long(), i32(9), f64(9), x5, x5),
                 lambda: hip.spmv(None, 5, 5, i32(6), i32(9), f64(9), torch.ones(5), x5)):
        with pytest.raises(TypeError):
            call()
