"""lapis_spmv_bench (the counterpart of the reference's benchmarks/spmv/main.cpp) run as a child process:
its MatrixMarket reader (general / symmetric / skew-symmetric, real / integer / pattern) and the product it
computes are checked against the oracle through the --check / --dump-y output."""
import os
import re
import subprocess

import numpy as np
import pytest

from conftest import GOLDEN, ROOT, read_mtx_csr
from gpu_util import assert_rows_close

pytestmark = pytest.mark.gpu

BENCH = os.path.join(ROOT, "lapis_amd", "bin", "lapis_spmv_bench")


def _run(matrix, trials, kernel, tmp_path):
    dump = str(tmp_path / "y.bin")
    assert os.path.exists(BENCH), "lapis_spmv_bench has not been built (python -m lapis_amd.build)"
    proc = subprocess.run([BENCH, matrix, str(trials), kernel, "--check", "--dump-y", dump], capture_output=True,
                          text=True, timeout=300)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    y = np.fromfile(dump, dtype=np.float64)
    total = float(re.search(r"check: sum\(y\) = (\S+)", proc.stdout).group(1))
    picked = {int(i): float(v) for i, v in re.findall(r"check: y\[(\d+)\] = (\S+)", proc.stdout)}
    # the protocol strings of the reference driver (benchmarks/spmv/main.cpp:39-47,61)
    assert "Reading matrix from" in proc.stdout and "Read matrix (" in proc.stdout and "spmv avg time = " in proc.stdout
    return y, total, picked, proc.stdout


def _expect(oracle, pos, crd, val, shape):
    x = np.arange(1, shape[1] + 1, dtype=np.float64)
    want = np.zeros(shape[0])
    oracle.spmv(pos, crd, val, x, want)
    return want, oracle.spmv_abs_scale(pos, crd, val, x)


@pytest.mark.parametrize("name", ["nos4.mtx", "mht_A.mtx", "mht_D.mtx"])
@pytest.mark.parametrize("kernel", ["auto", "reference", "nnzsplit"])
def test_driver_reads_the_reference_matrices(gpu, oracle, tmp_path, name, kernel):
    pos, crd, val, shape = read_mtx_csr(name)  # scipy's reader: an independent parse of the same file
    y, total, picked, out = _run(os.path.join(GOLDEN, name), 3, kernel, tmp_path)
    want, scale = _expect(oracle, pos, crd, val, shape)
    assert "Read matrix (%dx%d with %d entries)" % (shape[0], shape[1], crd.shape[0]) in out
    assert_rows_close(y, want, scale, np.float64, "%s/%s" % (name, kernel))
    assert abs(total - want.sum()) <= 1e-12 * scale.sum()
    for i, v in picked.items():
        assert v == y[i]


def _write_mtx(path, header, rows, cols, vals, shape):
    with open(path, "w") as f:
        f.write("%%MatrixMarket matrix coordinate " + header + "\n% written by the test\n")
        f.write("%d %d %d\n" % (shape[0], shape[1], len(rows)))
        for k in range(len(rows)):
            if vals is None:
                f.write("%d %d\n" % (rows[k] + 1, cols[k] + 1))
            else:
                f.write("%d %d %s\n" % (rows[k] + 1, cols[k] + 1, repr(vals[k])))


@pytest.mark.parametrize("flavour", ["real general", "integer general", "pattern general", "real skew-symmetric",
                                     "pattern symmetric"])
def test_driver_reads_every_supported_flavour(gpu, oracle, tmp_path, flavour):
    import scipy.sparse as sp
    rng = np.random.Generator(np.random.PCG64(7))
    n, m = 300, 260
    field, symmetry = flavour.split()
    if symmetry == "general":
        rows = rng.integers(0, n, 2500)
        cols = rng.integers(0, m, 2500)
        keep = np.unique(rows * m + cols, return_index=True)[1]  # the format lists each position once
        rows, cols = rows[keep], cols[keep]
        shape = (n, m)
    else:
        rows = rng.integers(0, n, 2500)
        cols = rng.integers(0, n, 2500)
        lower = rows > cols if symmetry == "skew-symmetric" else rows >= cols
        rows, cols = rows[lower], cols[lower]
        keep = np.unique(rows * n + cols, return_index=True)[1]
        rows, cols = rows[keep], cols[keep]
        shape = (n, n)
    if field == "pattern":
        vals = None
        v = np.ones(rows.shape[0])
    elif field == "integer":
        vals = [int(t) for t in rng.integers(-9, 10, rows.shape[0])]
        v = np.asarray(vals, dtype=np.float64)
    else:
        v = rng.random(rows.shape[0]) * 2 - 1
        vals = [float(t) for t in v]
    path = str(tmp_path / "m.mtx")
    _write_mtx(path, flavour, rows, cols, vals, shape)
    A = sp.coo_matrix((v, (rows, cols)), shape=shape)
    if symmetry == "symmetric":
        off = rows != cols
        A = A + sp.coo_matrix((v[off], (cols[off], rows[off])), shape=shape)
    elif symmetry == "skew-symmetric":
        A = A - sp.coo_matrix((v, (cols, rows)), shape=shape)
    A = sp.csr_matrix(A)
    A.sort_indices()
    pos, crd, val = A.indptr.astype(np.int32), A.indices.astype(np.int32), A.data.astype(np.float64)
    y, total, picked, out = _run(path, 2, "auto", tmp_path)
    want, scale = _expect(oracle, pos, crd, val, shape)
    assert_rows_close(y, want, scale, np.float64, flavour)


def test_driver_auto_picks_the_column_blocked_kernel_for_wide_random_columns(gpu, oracle, tmp_path):
    from lapis_amd import generators as gen
    A = gen.poisson_random(300000, 4.0, seed=51)
    rows = np.repeat(np.arange(A.nrows), np.diff(A.pos))
    path = str(tmp_path / "wide.mtx")
    with open(path, "w") as f:
        f.write("%%MatrixMarket matrix coordinate real general\n")
        f.write("%d %d %d\n" % (A.nrows, A.ncols, A.nnz))
        np.savetxt(f, np.column_stack([rows + 1, A.crd + 1, A.val]), fmt="%d %d %.17g")
    y, total, picked, out = _run(path, 64, "auto", tmp_path)
    assert re.search(r"kernel 4 ", out), out  # LAPIS_HIP_SPMV_COLBLOCK, chosen inside the library
    want, scale = _expect(oracle, A.pos, A.crd, A.val, (A.nrows, A.ncols))
    assert_rows_close(y, want, scale, np.float64, "auto/colblock")
    # too few calls for the copy to pay back: the plan keeps its CSR kernel
    y2, _, _, out2 = _run(path, 8, "auto", tmp_path)
    assert not re.search(r"kernel 4 ", out2)
    assert_rows_close(y2, want, scale, np.float64, "auto/csr")
