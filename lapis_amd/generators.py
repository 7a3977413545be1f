"""Seeded synthetic CSR inputs for the five benchmark configurations.

Every generator returns host numpy arrays in the decomposed-CSR form the
generated modules take: ``pos`` int32[n+1], ``crd`` int32[nnz] (ascending and
distinct inside each row), ``val`` T[nnz].  Random draws come from
``numpy.random.Generator(PCG64(seed))`` so a (config, seed) pair names one matrix.
"""
from dataclasses import dataclass

import numpy as np


@dataclass
class CSR:
    nrows: int
    ncols: int
    pos: np.ndarray
    crd: np.ndarray
    val: np.ndarray

    @property
    def nnz(self):
        return int(self.crd.shape[0])

    def spec(self):
        """Storage specifier tuple ``((m, n), (m+1, nnz, nnz))`` of a decomposed CSR argument."""
        return ((self.nrows, self.ncols), (self.nrows + 1, self.nnz, self.nnz))

    def spmv_bytes(self):
        """Algorithmic bytes of one SpMV: x read once, y written once, pos/crd/val streamed."""
        w = self.val.dtype.itemsize
        return 2 * w * self.nrows + (4 + w) * self.nnz + 4 * (self.nrows + 1)


def _rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def _pos_from_lengths(lengths):
    pos = np.zeros(lengths.shape[0] + 1, dtype=np.int64)
    np.cumsum(lengths, out=pos[1:])
    if pos[-1] >= 2 ** 31:
        raise ValueError("nnz does not fit the int32 positions of the CSR encoding")
    return pos.astype(np.int32)


def random_sorted_columns(rng, lengths, ncols):
    """Distinct ascending column indices for rows of the given lengths.

    Row i draws ``lengths[i]`` values u uniformly from ``[0, ncols - lengths[i]]``,
    sorts them, and takes ``u_j + j``: sorted draws with repetition map one-to-one
    onto strictly increasing sequences in ``[0, ncols)``, so no rejection loop is
    needed whatever the row length.
    """
    lengths = np.asarray(lengths, dtype=np.int64)
    if lengths.size and lengths.max() > ncols:
        raise ValueError("a row cannot hold more distinct columns than the matrix has")
    nnz = int(lengths.sum())
    nrows = lengths.shape[0]
    row_of = np.repeat(np.arange(nrows, dtype=np.int64), lengths)
    span = (ncols - lengths + 1).astype(np.float64)
    u = np.floor(rng.random(nnz) * span[row_of]).astype(np.int64)
    np.minimum(u, (ncols - lengths)[row_of], out=u)
    bits = max(1, int(ncols - 1).bit_length())
    key = (row_of << bits) | u
    del row_of
    key.sort()
    u = key & ((1 << bits) - 1)
    del key
    starts = np.zeros(nrows + 1, dtype=np.int64)
    np.cumsum(lengths, out=starts[1:])
    rank = np.arange(nnz, dtype=np.int64) - np.repeat(starts[:-1], lengths)
    return (u + rank).astype(np.int32)


def laplace2d(nx, dtype=np.float64):
    """5-point Laplacian on an nx-by-nx grid, row-major numbering, diag 4, off-diag -1."""
    n = nx * nx
    idx = np.arange(n, dtype=np.int64)
    ix, iy = idx % nx, idx // nx
    cand = np.stack([idx - nx, idx - 1, idx, idx + 1, idx + nx], axis=1)
    ok = np.stack([iy > 0, ix > 0, np.ones(n, bool), ix < nx - 1, iy < nx - 1], axis=1)
    vals = np.broadcast_to(np.array([-1, -1, 4, -1, -1], dtype=dtype), (n, 5))
    lengths = ok.sum(axis=1)
    return CSR(n, n, _pos_from_lengths(lengths), cand[ok].astype(np.int32), np.ascontiguousarray(vals[ok]))


def laplace3d(nx, dtype=np.float64):
    """7-point Laplacian on an nx^3 grid, x fastest, diag 6, off-diag -1."""
    n = nx ** 3
    idx = np.arange(n, dtype=np.int32)
    ix, iy, iz = idx % nx, (idx // nx) % nx, idx // (nx * nx)
    offs = np.array([-nx * nx, -nx, -1, 0, 1, nx, nx * nx], dtype=np.int32)
    ok = np.stack([iz > 0, iy > 0, ix > 0, np.ones(n, bool), ix < nx - 1, iy < nx - 1, iz < nx - 1], axis=1)
    del ix, iy, iz
    crd = (idx[:, None] + offs[None, :])[ok]
    val = np.broadcast_to(np.array([-1, -1, -1, 6, -1, -1, -1], dtype=dtype), (n, 7))[ok]
    return CSR(n, n, _pos_from_lengths(ok.sum(axis=1, dtype=np.int64)), crd, np.ascontiguousarray(val))


def elasticity3d(nx, dtype=np.float64):
    """Structure of a 3-D elasticity operator on an nx^3 node grid: 3 unknowns per node,
    27-point node stencil, a full 3x3 block per node pair (rows 3*nx^3, nnz 9*(3nx-2)^3).
    nx = 60 gives the size of the reference's published matrix Elasticity3D_60
    (648 000 rows, 50 757 768 non-zeros, benchmarks/plots/plotSPMV.py:14-15); the values
    (diagonal 100, rest -1) are stand-ins, SpMV time does not depend on them."""
    n = nx ** 3
    idx = np.arange(n, dtype=np.int64)
    ix, iy, iz = idx % nx, (idx // nx) % nx, idx // (nx * nx)
    cands, oks = [], []
    for dz in (-1, 0, 1):
        for dy in (-1, 0, 1):
            for dx in (-1, 0, 1):
                ok = ((ix + dx >= 0) & (ix + dx < nx) & (iy + dy >= 0) & (iy + dy < nx) & (iz + dz >= 0) & (iz + dz < nx))
                cands.append(idx + dx + dy * nx + dz * nx * nx)
                oks.append(ok)
    cand = np.stack(cands, axis=1)
    ok = np.stack(oks, axis=1)
    nb = cand[ok]                                   # neighbour nodes, node-major, ascending inside a node
    cnt = ok.sum(axis=1)                            # neighbours per node
    node_start = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(cnt, out=node_start[1:])
    row_len = np.repeat(3 * cnt, 3)                 # three rows per node, 3 columns per neighbour
    pos = _pos_from_lengths(row_len)
    nnz = int(pos[-1])
    row_of = np.repeat(np.arange(3 * n, dtype=np.int64), row_len)
    k = np.arange(nnz, dtype=np.int64) - pos[:-1].astype(np.int64)[row_of]
    crd = (nb[node_start[row_of // 3] + k // 3] * 3 + k % 3).astype(np.int32)
    val = np.where(crd == row_of, 100.0, -1.0).astype(dtype)
    return CSR(3 * n, 3 * n, pos, crd, val)


def poisson_random(n, mean=16.0, seed=2002, dtype=np.float64):
    """Square matrix, row length ~ Poisson(mean), uniform distinct sorted columns, values U[-1,1)."""
    rng = _rng(seed)
    lengths = np.minimum(rng.poisson(mean, n).astype(np.int64), n)
    crd = random_sorted_columns(rng, lengths, n)
    val = (rng.random(crd.shape[0]) * 2.0 - 1.0).astype(dtype)
    return CSR(n, n, _pos_from_lengths(lengths), crd, val)


def _zipf_shift_for_mean(mean, cap):
    """Shift q of the Zipf-Mandelbrot tail P(K>=k) = (q+1)/(k+q), 1<=k<=cap, giving the asked mean."""
    k = np.arange(1, cap + 1, dtype=np.float64)
    lo, hi = 0.0, 64.0
    for _ in range(60):
        q = 0.5 * (lo + hi)
        m = ((q + 1.0) / (k + q)).sum()
        lo, hi = (q, hi) if m < mean else (lo, q)
    return 0.5 * (lo + hi)


def powerlaw_random(n, mean=30.0, cap=200000, seed=3003, dtype=np.float32):
    """Square matrix with exponent-2 power-law row lengths (min 1, capped), values N(0,1).

    Lengths follow the Zipf-Mandelbrot law P(K>=k) = (q+1)/(k+q): pmf ~ k^-2 in the
    tail, minimum 1, truncated at ``cap``; the shift q is solved so that the expected
    length equals ``mean`` (a plain Zipf(2) truncated at 200000 has mean 7.8).
    """
    rng = _rng(seed)
    cap = min(cap, n)
    q = _zipf_shift_for_mean(mean, cap)
    u = 1.0 - rng.random(n)  # (0, 1]
    lengths = np.floor((q + 1.0) / u - q).astype(np.int64)
    np.clip(lengths, 1, cap, out=lengths)
    crd = random_sorted_columns(rng, lengths, n)
    val = rng.standard_normal(crd.shape[0], dtype=np.float32).astype(dtype, copy=False)
    return CSR(n, n, _pos_from_lengths(lengths), crd, val)


def fixed_degree_random(n, degree=32, seed=4004, dtype=np.float32):
    """Square matrix with exactly ``degree`` uniform distinct sorted columns per row, values N(0,1)."""
    rng = _rng(seed)
    lengths = np.full(n, min(degree, n), dtype=np.int64)
    crd = random_sorted_columns(rng, lengths, n)
    val = rng.standard_normal(crd.shape[0], dtype=np.float32).astype(dtype, copy=False)
    return CSR(n, n, _pos_from_lengths(lengths), crd, val)


def uniform_vector(n, seed, lo=-1.0, hi=1.0, dtype=np.float64):
    return (_rng(seed).random(n) * (hi - lo) + lo).astype(dtype)


def uniform_matrix(rows, cols, seed, lo=-1.0, hi=1.0, dtype=np.float32):
    rng = _rng(seed)
    return (rng.random((rows, cols), dtype=np.float32) * (hi - lo) + lo).astype(dtype, copy=False)


# The five named configurations.  ``scale`` < 1 shrinks the row count (for parity
# tests the oracle can finish in seconds); scale = 1 is the benchmark size.
def config1(scale=1.0):
    nx = max(4, int(round(256 * np.sqrt(scale))))
    A = laplace2d(nx)
    return A, uniform_vector(A.ncols, 1001)


def config2(scale=1.0):
    n = max(64, int(4194304 * scale))
    A = poisson_random(n, 16.0, seed=2002)
    return A, uniform_vector(A.ncols, 2002 + 1)


def config3(scale=1.0):
    n = max(64, int(2097152 * scale))
    A = powerlaw_random(n, 30.0, 200000, seed=3003)
    return A, uniform_vector(A.ncols, 3003 + 1, dtype=np.float32)


def config4(scale=1.0, k=64):
    n = max(64, int(1048576 * scale))
    A = fixed_degree_random(n, 32, seed=4004)
    return A, uniform_matrix(n, k, 4004 + 1)


# Matrices of the reference's published SpMV table whose structure is a formula
# (benchmarks/plots/spmv.csv:3,8): name -> (maker, published mean seconds on MI300A, on H100)
PUBLISHED = {
    "Laplace3D_100": (lambda: laplace3d(100), 5.44e-05, 7.29e-05),
    "Elasticity3D_60": (lambda: elasticity3d(60), 2.85281e-04, 2.65587e-04),
}


def config5(scale=1.0):
    nx = max(4, int(round(192 * scale ** (1.0 / 3.0))))
    A = laplace3d(nx)
    return A, uniform_vector(A.nrows, 5005, lo=0.0, hi=1.0)
