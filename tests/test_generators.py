"""The seeded synthetic inputs: structure, sizes and reproducibility."""
import numpy as np
import pytest

from lapis_amd import generators as gen


def _check_structure(A):
    assert A.pos.dtype == np.int32 and A.crd.dtype == np.int32
    assert A.pos[0] == 0 and A.pos[-1] == A.nnz and A.pos.shape[0] == A.nrows + 1
    assert np.all(np.diff(A.pos) >= 0)
    assert A.crd.min() >= 0 and A.crd.max() < A.ncols
    d = np.diff(A.crd.astype(np.int64))
    inner = np.ones(A.nnz - 1, bool)
    cuts = A.pos[1:-1]
    cuts = cuts[(cuts > 0) & (cuts < A.nnz)]
    inner[cuts - 1] = False
    assert np.all(d[inner] > 0), "columns must be strictly ascending inside a row"


def test_config1_is_the_named_laplacian():
    A, x = gen.config1()
    assert (A.nrows, A.nnz) == (65536, 326656) and A.spmv_bytes() == 5230596
    _check_structure(A)
    assert x.dtype == np.float64 and -1 <= x.min() and x.max() < 1
    assert set(np.unique(A.val)) == {-1.0, 4.0}


def test_config5_sizes_at_small_scale_and_full_formula():
    A, b = gen.config5(scale=(16 / 192) ** 3)
    nx = 16
    assert A.nrows == nx ** 3 and A.nnz == 7 * nx ** 3 - 6 * nx ** 2
    _check_structure(A)
    assert 7 * 192 ** 3 - 6 * 192 ** 2 == 49324032
    assert 0 <= b.min() and b.max() < 1


@pytest.mark.parametrize("cfg", [gen.config2, gen.config3, gen.config4])
def test_random_configs_are_valid_and_reproducible(cfg):
    A, v = cfg(scale=1 / 256)
    B, w = cfg(scale=1 / 256)
    _check_structure(A)
    assert np.array_equal(A.pos, B.pos) and np.array_equal(A.crd, B.crd) and np.array_equal(A.val, B.val)
    assert np.array_equal(v, w)


def test_config2_row_lengths_are_poisson_16():
    A, _ = gen.config2(scale=1 / 64)
    L = np.diff(A.pos)
    assert abs(L.mean() - 16) < 0.1 and abs(L.var() - 16) < 0.5
    assert A.val.dtype == np.float64


def test_config3_power_law_shape():
    A, x = gen.config3(scale=1 / 8)
    L = np.diff(A.pos)
    assert L.min() == 1 and L.max() <= 200000
    assert 20 < L.mean() < 40
    assert L.max() > 100 * L.mean()  # a heavy tail, not a bell
    # exponent 2: P(K >= 10k) is about ten times smaller than P(K >= k)
    r = (L >= 100).mean() / (L >= 1000).mean()
    assert 6 < r < 16
    assert A.val.dtype == np.float32 and x.dtype == np.float32


def test_config4_has_exactly_32_per_row():
    A, B = gen.config4(scale=1 / 128)
    assert np.all(np.diff(A.pos) == 32) and B.shape == (A.nrows, 64) and B.dtype == np.float32


def test_sorted_columns_handle_rows_as_long_as_the_matrix():
    rng = np.random.Generator(np.random.PCG64(1))
    crd = gen.random_sorted_columns(rng, np.array([5, 0, 3]), 5)
    assert list(crd[:5]) == [0, 1, 2, 3, 4] and len(crd) == 8
