"""Seeded random CSR structures through every SpMV kernel family, the SpMM and CG, against the CPU oracle.

The fixed-shape tests name their edge cases; this one draws shapes nobody thought of: rectangular matrices with a
single row or column, power-law rows with empty ones and a few that hold most of the entries, bands, and wide
matrices with so many columns that the column-blocked copies have something to block.  Every structure goes through
the call without a plan (the reference's own launch rule), the plan's choice, each CSR kernel forced, the library's
analysis, and both column-blocked layouts."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch

from gpu_util import TOL, assert_rows_close, dev

pytestmark = pytest.mark.gpu


def _structure(rng, kind, dt):
    if kind == 0:
        m, n = int(rng.integers(1, 3000)), int(rng.integers(1, 3000))
        A = sp.random(m, n, density=min(1.0, rng.uniform(0.5, 40) / n),
                      random_state=np.random.RandomState(int(rng.integers(1 << 30))), format="csr")
    elif kind == 1:
        m, n = int(rng.integers(100, 20000)), int(rng.integers(100, 20000))
        lens = np.minimum((rng.pareto(1.2, m) * rng.uniform(0.2, 3)).astype(np.int64), n)
        lens[rng.integers(0, m, 3)] = np.minimum(n, rng.integers(1000, 20000, 3))
        pos = np.concatenate([[0], np.cumsum(lens)])
        crd = np.concatenate([np.sort(rng.choice(n, l, replace=False)) for l in lens])
        A = sp.csr_matrix((rng.standard_normal(pos[-1]), crd, pos), shape=(m, n))
    elif kind == 2:
        m = n = int(rng.integers(10, 30000))
        offs = np.unique(rng.integers(-50, 50, int(rng.integers(1, 9))))
        A = sp.diags([rng.standard_normal(m - abs(o)) for o in offs], offs, shape=(m, n), format="csr")
    else:
        m, n = int(rng.integers(1000, 40000)), int(rng.integers(300000, 900000))
        k = int(rng.integers(1, 12))
        crd = rng.integers(0, n, (m, k))
        crd.sort(axis=1)
        A = sp.csr_matrix((rng.standard_normal(m * k), crd.ravel(), np.arange(0, m * k + 1, k)), shape=(m, n))
        A.sum_duplicates()
    A = sp.csr_matrix(A, dtype=dt)
    A.sort_indices()
    return A


@pytest.mark.parametrize("seed", [101, 102, 103])
def test_random_structures_through_every_kernel_family(gpu, oracle, seed):
    rng = np.random.default_rng(seed)
    ran = set()
    for case in range(40):
        kind = int(rng.integers(0, 4))
        dt = np.float64 if rng.random() < 0.6 else np.float32
        A = _structure(rng, kind, dt)
        m, n = A.shape
        hp, hc, hv = A.indptr.astype(np.int32), A.indices.astype(np.int32), A.data.astype(dt)
        pos, crd, val = dev(hp), dev(hc), dev(hv)
        x, y0 = rng.standard_normal(n).astype(dt), rng.standard_normal(m).astype(dt)
        want = oracle.spmv(hp, hc, hv, x, y0.copy())
        scale = oracle.spmv_abs_scale(hp, hc, hv, x, y0)
        dx = dev(x)
        what = "seed %d case %d kind %d %s %dx%d nnz %d" % (seed, case, kind, dt.__name__, m, n, A.nnz)
        for name, how in (("no plan", None), ("plan", "plan"), ("subwarp", 1), ("rowblock", 2), ("row split", 3),
                          ("analyze", "analyze"), ("group", "group"), ("wave", "wave")):
            y = dev(y0.copy())
            plan = None
            try:
                if how is not None:
                    plan = gpu.CsrPlan(m, n, pos, crd, value_bytes=np.dtype(dt).itemsize)
                    if isinstance(how, int):
                        plan.set_kernel(how, 4 if how == 1 else 0)
                    elif how == "analyze":
                        plan.analyze(crd, val)
                    elif how in ("group", "wave"):
                        try:
                            plan.build_colblock(crd, val, layout=how)
                        except gpu.LapisHipError as e:
                            if e.status_name != "LAPIS_HIP_ERR_NO_TILING":
                                raise
                            continue
                gpu.spmv(plan, m, n, pos, crd, val, dx, y)
                if plan is not None:
                    plan.check()
                    ran.add(plan.kernel_name())
                assert_rows_close(y.cpu().numpy(), want, scale, dt, what + " / " + name)
            finally:
                if plan is not None:
                    plan.destroy()
        k = int(rng.choice([1, 3, 16, 64]))
        if A.nnz * k < 4e6 and n * k < 3e7:
            B, C0 = rng.standard_normal((n, k)).astype(dt), rng.standard_normal((m, k)).astype(dt)
            wantC = oracle.spmm(hp, hc, hv, B, C0.copy())
            C = dev(C0.copy())
            plan = gpu.CsrPlan(m, n, pos, crd, value_bytes=np.dtype(dt).itemsize)
            gpu.spmm(m, n, pos, crd, val, dev(B), C, plan=plan if case % 2 else None)
            plan.destroy()
            sc = np.abs(C0).astype(np.float64) + abs(A).astype(np.float64) @ np.abs(B).astype(np.float64)
            assert np.all(np.abs(C.cpu().numpy().astype(np.float64) - wantC) <= TOL[np.dtype(dt)] * (sc + 1e-300)), \
                what + " / spmm k=%d" % k
        if dt == np.float64 and m == n and kind in (0, 2):
            S = sp.csr_matrix(A + A.T)
            S = sp.csr_matrix(S + sp.diags(np.asarray(abs(S).sum(axis=1)).ravel() + 1.0))
            S.sort_indices()
            b = S @ np.ones(m)
            sp_, sc_, sv_ = S.indptr.astype(np.int32), S.indices.astype(np.int32), S.data
            xo, io, ro = oracle.pcg(sp_, sc_, sv_, b, np.ones(m), 1e-10, 2000)
            dp, dc, dv = dev(sp_), dev(sc_), dev(sv_)
            for forced in (None, 3):  # the plan's own kernel, then the row-split kernel with its fused p.Ap sums
                plan = gpu.CsrPlan(m, m, dp, dc)
                if forced:
                    plan.set_kernel(forced, 0)
                xs = torch.zeros(m, dtype=torch.float64, device="cuda")
                its, rel = gpu.pcg(plan, m, dp, dc, dv, dev(b), None, 1e-10, 2000, xs)
                plan.destroy()
                assert abs(its - io) <= 1 and rel <= 1e-10, what + " / cg"
                assert np.allclose(xs.cpu().numpy(), xo, rtol=1e-7, atol=1e-9), what + " / cg"
    assert {"spmv_subwarp_kernel", "spmv_rowblock_kernel", "spmv_nnzsplit_kernel", "spmv_colblock_kernel",
            "spmv_colgroup_kernel"} <= ran
