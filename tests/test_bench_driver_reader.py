"""The MatrixMarket reader of lapis_spmv_bench (the counterpart of benchmarks/spmv/main.cpp:37-47 of the
reference, which reads through KokkosKernels) on every header variant it accepts, without a GPU:
`--parse-only` prints what the reader made of the file and scipy.io.mmread says what it should be."""
import os
import re
import subprocess

import numpy as np
import pytest
import scipy.io
import scipy.sparse as sp

from conftest import ROOT

BENCH = os.path.join(ROOT, "lapis_amd", "bin", "lapis_spmv_bench")


def parse_only(path):
    if not os.path.exists(BENCH):
        pytest.skip("lapis_spmv_bench is not built")
    proc = subprocess.run([BENCH, str(path), "--parse-only"], capture_output=True, text=True, timeout=60)
    return proc


def expected(A):
    A = sp.csr_matrix(A)
    A.sum_duplicates()
    coo = A.tocoo()
    weighted = float(np.sum((coo.row + 1.0) * (2.0 * coo.col + 1.0) * coo.data))
    return A.shape, A.nnz, float(coo.data.sum()), weighted


def check(path, A):
    proc = parse_only(path)
    assert proc.returncode == 0, proc.stderr
    shape, nnz, total, weighted = expected(A)
    m = re.search(r"Read matrix \((\d+)x(\d+) with (\d+) entries\)", proc.stdout)
    assert m and (int(m.group(1)), int(m.group(2))) == shape and int(m.group(3)) == nnz, proc.stdout
    got_sum = float(re.search(r"parse: sum\(val\) = (\S+)", proc.stdout).group(1))
    got_w = float(re.search(r"parse: sum\(\(row\+1\)\*\(2\*col\+1\)\*val\) = (\S+)", proc.stdout).group(1))
    assert got_sum == pytest.approx(total, rel=1e-13, abs=1e-13)
    assert got_w == pytest.approx(weighted, rel=1e-13, abs=1e-11)
    assert "columns ascend in every row = yes" in proc.stdout


CASES = {
    "general_real": """%%MatrixMarket matrix coordinate real general
% a comment line
4 5 6
1 1 1.5
3 2 -2.25
1 5 4.0
4 4 1e-3
2 3 7
4 1 -8.5
""",
    "symmetric_real": """%%MatrixMarket matrix coordinate real symmetric
4 4 5
1 1 2.0
2 1 -1.0
3 2 -1.5
4 4 3.0
4 1 0.25
""",
    "skew_symmetric": """%%MatrixMarket matrix coordinate real skew-symmetric
4 4 3
2 1 1.0
4 2 -2.5
3 1 0.5
""",
    "pattern_symmetric": """%%MatrixMarket matrix coordinate pattern symmetric
5 5 6
1 1
2 1
3 3
5 2
5 4
4 4
""",
    "pattern_general": """%%MatrixMarket matrix coordinate pattern general
3 6 4
1 6
2 2
3 1
1 2
""",
    "integer_general": """%%MatrixMarket matrix coordinate integer general
3 3 4
1 1 2
2 3 -7
3 1 5
3 3 11
""",
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_reader_expands_every_header_variant_like_scipy(tmp_path, name):
    path = tmp_path / (name + ".mtx")
    path.write_text(CASES[name])
    check(path, scipy.io.mmread(str(path)))


@pytest.mark.parametrize("name", ["nos4.mtx", "mht_A.mtx", "mht_D.mtx"])
def test_reader_on_the_reference_matrices(name):
    path = os.path.join(ROOT, "tests", "golden", name)
    check(path, scipy.io.mmread(path))


@pytest.mark.parametrize("text, why", [
    ("%%MatrixMarket matrix array real general\n2 2\n1\n2\n3\n4\n", "array"),
    ("%%MatrixMarket matrix coordinate complex general\n2 2 1\n1 1 1.0 0.0\n", "complex"),
    ("%%MatrixMarket matrix coordinate real general\n2 2 2\n1 1 1.0\n3 1 2.0\n", "outside"),
    ("%%MatrixMarket matrix coordinate real general\n2 2 3\n1 1 1.0\n", "entries"),
    ("not a matrix market file\n", "header"),
    # a header that claims more entries than the file can hold must not make the reader set memory aside for them
    ("%%MatrixMarket matrix coordinate real symmetric\n4 4 42147483647\n1 1 2\n2 1 -1\n", "claimed entries"),
    ("%%MatrixMarket matrix coordinate pattern general\n3 3 2000000000\n1 2\n2 3\n3 1\n", "claimed entries"),
    ("%%MatrixMarket matrix coordinate real general\n4294967296 4 1\n1 1 1.0\n", "int32 rows"),
    ("%%MatrixMarket matrix coordinate real general\n4 4294967296 1\n1 1 1.0\n", "int32 columns"),
])
def test_reader_refuses_what_it_cannot_represent(tmp_path, text, why):
    path = tmp_path / "bad.mtx"
    path.write_text(text)
    proc = parse_only(path)
    assert proc.returncode != 0
    assert "error" in proc.stderr.lower()
