"""SpMV parity on the GPU: every kernel family of the HIP library, called through the
C ABI, against the sequential-order CPU oracle on the same seeded inputs."""
import numpy as np
import pytest
import torch

from gpu_util import assert_rows_close, dev, dev_unaligned, from_lengths as _from_lengths
from lapis_amd import generators as gen
from lapis_amd.generators import CSR

pytestmark = pytest.mark.gpu

# (kernel, width) choices a plan can be forced to, plus None = automatic choice
KERNELS = [("auto", 0), ("subwarp", 1), ("subwarp", 2), ("subwarp", 4), ("subwarp", 8), ("subwarp", 16),
           ("subwarp", 32), ("subwarp", 64), ("rowblock", 0), ("nnzsplit", 0)]
KID = {"auto": 0, "subwarp": 1, "rowblock": 2, "nnzsplit": 3}


def _matrices(dtype):
    """name -> CSR.  Sizes are chosen so the oracle needs well under a second each."""
    out = {}
    out["golden5x5"] = CSR(5, 5, np.array([0, 1, 5, 6, 8, 8], np.int32),
                           np.array([1, 0, 2, 3, 4, 2, 0, 1], np.int32),
                           np.array([1.1, 0.3, 2.2, 3.7, -4, -19, -2, 1], dtype))
    A, _ = gen.config1(scale=1 / 16)
    out["laplace2d_64"] = CSR(A.nrows, A.ncols, A.pos, A.crd, A.val.astype(dtype))
    A, _ = gen.config5(scale=(20 / 192) ** 3)
    out["laplace3d_20"] = CSR(A.nrows, A.ncols, A.pos, A.crd, A.val.astype(dtype))
    A = gen.poisson_random(65536 + 37, 16.0, seed=2002, dtype=dtype)
    out["poisson16_65573"] = A
    A = gen.powerlaw_random(131072, 30.0, 200000, seed=3003, dtype=dtype)
    out["powerlaw_131072"] = A
    # ragged edge cases
    out["all_rows_empty"] = _from_lengths([0] * 300, 300, 1, dtype)
    out["one_long_row"] = _from_lengths([5000], 8000, 2, dtype)
    out["long_rows_between_empties"] = _from_lengths([0, 0, 3000, 0, 1, 0, 2047, 1025, 0, 0, 1, 4096, 0], 5000, 3, dtype)
    out["chunk_boundary_exact"] = _from_lengths([1024, 1024, 512, 512, 1, 1023, 2048], 4096, 4, dtype)
    out["wide_gap_of_empty_rows"] = _from_lengths([7] * 10 + [0] * 1000 + [9] * 10, 64, 5, dtype)
    out["dense_short"] = _from_lengths([64] * 257, 64, 6, dtype)
    out["mean_100"] = gen.poisson_random(3000, 100.0, seed=7, dtype=dtype)
    # rectangular: more columns than rows and the other way round
    out["wide_300x100000"] = _from_lengths([40] * 150 + [3000] + [0] * 49 + [700] * 100, 100000, 8, dtype)
    out["tall_50000x37"] = _from_lengths([5, 0, 37, 1] * 12500, 37, 9, dtype)
    return out


@pytest.fixture(scope="module", params=[np.float64, np.float32], ids=["f64", "f32"])
def cases(request, oracle):
    dtype = request.param
    built = {}
    for name, A in _matrices(dtype).items():
        x = gen.uniform_vector(A.ncols, 11, dtype=dtype)
        y_in = gen.uniform_vector(A.nrows, 12, dtype=dtype)
        want = y_in.copy()
        oracle.spmv(A.pos, A.crd, A.val, x, want)
        scale = oracle.spmv_abs_scale(A.pos, A.crd, A.val, x, y_in)
        built[name] = (A, x, y_in, want, scale)
    return dtype, built


@pytest.mark.parametrize("kernel,width", KERNELS, ids=["%s%s" % (k, w or "") for k, w in KERNELS])
def test_spmv_matches_oracle(gpu, cases, kernel, width):
    dtype, built = cases
    for name, (A, x, y_in, want, scale) in built.items():
        print("case", name, kernel, width, np.dtype(dtype).name, flush=True)
        pos, crd, val = dev(A.pos), dev(A.crd), dev(A.val)
        plan = gpu.CsrPlan(A.nrows, A.ncols, pos, crd, value_bytes=np.dtype(dtype).itemsize)
        if kernel != "auto":
            plan.set_kernel(KID[kernel], width)
        y = dev(y_in)
        gpu.spmv(plan, A.nrows, A.ncols, pos, crd, val, dev(x), y)
        torch.cuda.synchronize()
        got = y.cpu().numpy()
        assert_rows_close(got, want, scale, dtype, "%s/%s%d" % (name, kernel, width))
        if kernel == "subwarp" and width == 1:
            # one lane per row sums in the reference's order with separate multiply and add
            assert np.array_equal(got, want), name + ": thread-per-row must be bit-identical to the oracle"
        plan.destroy()


@pytest.mark.parametrize("chunk,waves", [(512, 4), (512, 8), (1024, 2), (1024, 4), (1024, 8), (2048, 2), (2048, 4)])
def test_row_split_kernel_at_every_chunk_size(gpu, cases, monkeypatch, chunk, waves):
    dtype, built = cases
    monkeypatch.setenv("LAPIS_HIP_SPMV_CHUNK", str(chunk))
    monkeypatch.setenv("LAPIS_HIP_SPMV_WAVES", str(waves))
    for name, (A, x, y_in, want, scale) in built.items():
        print("case", name, "nnzsplit", chunk, waves, np.dtype(dtype).name, flush=True)
        pos, crd, val = dev(A.pos), dev(A.crd), dev(A.val)
        plan = gpu.CsrPlan(A.nrows, A.ncols, pos, crd, value_bytes=np.dtype(dtype).itemsize).set_kernel(3)
        if A.nnz:
            assert plan.stats()["chunk"] == chunk
        y = dev(y_in)
        gpu.spmv(plan, A.nrows, A.ncols, pos, crd, val, dev(x), y)
        torch.cuda.synchronize()
        assert_rows_close(y.cpu().numpy(), want, scale, dtype, "%s/nnzsplit%dx%d" % (name, chunk, waves))
        plan.destroy()


@pytest.mark.parametrize("layout", ["wave", "group"])
@pytest.mark.parametrize("slice_log2", [0, 4, 9])
def test_column_blocked_copy_matches_oracle(gpu, cases, slice_log2, layout):
    dtype, built = cases
    for name, (A, x, y_in, want, scale) in built.items():
        if A.nnz == 0:
            continue
        print("case", name, "colblock", layout, slice_log2, np.dtype(dtype).name, flush=True)
        pos, crd, val = dev(A.pos), dev(A.crd), dev(A.val)
        plan = gpu.CsrPlan(A.nrows, A.ncols, pos, crd, value_bytes=np.dtype(dtype).itemsize)
        plan.build_colblock(crd, val, slice_log2, layout=layout)
        assert plan.stats()["kernel_name"] == "colblock"
        runs = []
        for _ in range(2):
            y = dev(y_in)
            gpu.spmv(plan, A.nrows, A.ncols, pos, crd, val, dev(x), y)
            torch.cuda.synchronize()
            runs.append(y.cpu().numpy())
        assert_rows_close(runs[0], want, scale, dtype, "%s/colblock-%s" % (name, layout))
        if layout == "wave":
            assert np.array_equal(runs[0], runs[1]), name + ": two runs of the column-blocked kernel differ"
        else:  # row sums are LDS atomics shared by a workgroup: the order of additions is not fixed
            assert_rows_close(runs[1], want, scale, dtype, "%s/colblock-%s, second run" % (name, layout))
        plan.destroy()


# (producer wavefronts, threads per workgroup) of the workgroup kernel; 0 = every wavefront streams and gathers
ROLE_SPLITS = [(0, 0), (4, 1024), (6, 1024), (3, 768), (4, 640), (2, 512)]


def _set_role_split(monkeypatch, split):
    monkeypatch.setenv("LAPIS_HIP_COLBLOCK_PC", str(split[0]))
    if split[0]:
        monkeypatch.setenv("LAPIS_HIP_COLBLOCK_PC_THREADS", str(split[1]))


@pytest.mark.parametrize("split", ROLE_SPLITS)
@pytest.mark.parametrize("long_threshold,unit,rows", [(2, 100, 4096), (64, 5000, 4096), (1024, 0, 8192),
                                                      (100000000, 33333, 16384)])
def test_workgroup_layout_with_forced_long_rows_and_units(gpu, cases, monkeypatch, long_threshold, unit, rows, split):
    # the tuning overrides move rows between their natural blocks and the blocks of long rows
    # and change how many work units a block is cut into: every combination must give the same y,
    # with every wavefront streaming and gathering and with the roles split between wavefronts
    _set_role_split(monkeypatch, split)
    monkeypatch.setenv("LAPIS_HIP_COLBLOCK_LONG", str(long_threshold))
    monkeypatch.setenv("LAPIS_HIP_COLBLOCK_UNIT", str(unit))
    monkeypatch.setenv("LAPIS_HIP_COLBLOCK_ROWS", str(rows))
    dtype, built = cases
    for name, (A, x, y_in, want, scale) in built.items():
        if A.nnz == 0:
            continue
        print("case", name, "group", long_threshold, unit, rows, split, np.dtype(dtype).name, flush=True)
        pos, crd, val = dev(A.pos), dev(A.crd), dev(A.val)
        plan = gpu.CsrPlan(A.nrows, A.ncols, pos, crd, value_bytes=np.dtype(dtype).itemsize)
        plan.build_colblock(crd, val, 7, layout="group")
        y = dev(y_in)
        gpu.spmv(plan, A.nrows, A.ncols, pos, crd, val, dev(x), y)
        torch.cuda.synchronize()
        assert_rows_close(y.cpu().numpy(), want, scale, dtype, "%s/group long>=%d unit %d" % (name, long_threshold, unit))
        plan.check()
        plan.destroy()


@pytest.mark.parametrize("split", ROLE_SPLITS[:3])
def test_workgroup_layout_on_seeded_random_shapes(gpu, oracle, monkeypatch, split):
    _set_role_split(monkeypatch, split)
    # 40 matrices of random shape, density and skew, each with its own slice width, work-unit size,
    # long-row threshold and block size: unit borders fall inside tiles, on tile borders and
    # next to empty tiles
    rng = np.random.Generator(np.random.PCG64(20240607))
    for case in range(40):
        dtype = [np.float64, np.float32][case % 2]
        nrows = int(rng.integers(1, 40000))
        ncols = int(rng.integers(1, 300000))
        mean = float(rng.choice([0.3, 2.0, 9.0, 40.0]))
        lengths = np.minimum(rng.poisson(mean, nrows), ncols)
        for _ in range(int(rng.integers(0, 4))):  # a few long rows
            lengths[int(rng.integers(0, nrows))] = min(ncols, int(rng.integers(500, 60000)))
        A = _from_lengths(lengths, ncols, 1000 + case, dtype)
        if A.nnz == 0:
            continue
        slice_log2 = int(rng.integers(1, 19))
        monkeypatch.setenv("LAPIS_HIP_COLBLOCK_UNIT", str(int(rng.choice([0, 64, 1000, 4096, 50000]))))
        monkeypatch.setenv("LAPIS_HIP_COLBLOCK_LONG", str(int(rng.choice([0, 2, 300, 5000]))))
        monkeypatch.setenv("LAPIS_HIP_COLBLOCK_ROWS", str(int(rng.choice([0, 4096, 8192, 16384]))))
        x = gen.uniform_vector(A.ncols, 11, dtype=dtype)
        y_in = gen.uniform_vector(A.nrows, 12, dtype=dtype)
        want = y_in.copy()
        oracle.spmv(A.pos, A.crd, A.val, x, want)
        scale = oracle.spmv_abs_scale(A.pos, A.crd, A.val, x, y_in)
        print("random case", case, nrows, ncols, A.nnz, int(lengths.max()), slice_log2, np.dtype(dtype).name, flush=True)
        pos, crd, val = dev(A.pos), dev(A.crd), dev(A.val)
        plan = gpu.CsrPlan(A.nrows, A.ncols, pos, crd, value_bytes=np.dtype(dtype).itemsize)
        plan.build_colblock(crd, val, slice_log2, layout="group")
        y = dev(y_in)
        gpu.spmv(plan, A.nrows, A.ncols, pos, crd, val, dev(x), y)
        torch.cuda.synchronize()
        assert_rows_close(y.cpu().numpy(), want, scale, dtype, "random case %d" % case)
        plan.check()
        plan.destroy()


def test_column_blocked_copy_refuses_what_it_cannot_encode(gpu):
    # per-wavefront layout: 2^23 columns need 23 bits; an entry has 22
    pos = dev(np.array([0, 1], np.int32))
    crd = dev(np.array([5], np.int32))
    plan = gpu.CsrPlan(1, 1 << 23, pos, crd)
    with pytest.raises(gpu.LapisHipError) as e:
        plan.build_colblock(crd, dev(np.ones(1)), layout="wave")
    assert e.value.status_name == "LAPIS_HIP_ERR_NO_TILING"
    with pytest.raises(gpu.LapisHipError):
        plan.set_kernel(4)  # nothing was built


def test_spmv_without_plan_follows_the_reference_rule(gpu, cases):
    dtype, built = cases
    for name, (A, x, y_in, want, scale) in built.items():
        print("case", name, "no plan", flush=True)
        y = dev(y_in)
        gpu.spmv(None, A.nrows, A.ncols, dev(A.pos), dev(A.crd), dev(A.val), dev(x), y)
        torch.cuda.synchronize()
        assert_rows_close(y.cpu().numpy(), want, scale, dtype, name + "/noplan")


def test_plan_statistics_and_reference_decision(gpu, oracle):
    A, _ = gen.config2(scale=1 / 64)
    pos, crd = dev(A.pos), dev(A.crd)
    s = gpu.CsrPlan(A.nrows, A.ncols, pos, crd).stats()
    L = np.diff(A.pos)
    assert (s["nrows"], s["ncols"], s["nnz"]) == (A.nrows, A.ncols, A.nnz)
    assert (s["min_row_len"], s["max_row_len"], s["empty_rows"]) == (L.min(), L.max(), int((L == 0).sum()))
    assert abs(s["mean_row_len"] - L.mean()) < 1e-12 and abs(s["var_row_len"] - L.var()) < 1e-6
    # index outputs are bit-exact: the reference's hint and vector length for this matrix
    hint = oracle.csr_parallelism_hint(A.pos)
    assert hint in (16, 17) and s["reference_hint"] == hint
    assert s["reference_vector_length"] == oracle.thread_parallel_vector_length(hint, 64) == 4
    assert s["kernel_name"] == "rowblock"  # about a million non-zeros: one launch beats two
    assert s["mean_chunk_col_span"] > 0.9 * A.ncols and s["colblock_recommended"] == 0
    B, _ = gen.config3(scale=1 / 16)
    sb = gpu.CsrPlan(B.nrows, B.ncols, dev(B.pos), dev(B.crd), value_bytes=4).stats()
    assert sb["kernel_name"] == "nnzsplit" and sb["reference_vector_length"] == 8
    C = gen.poisson_random(6000, 2400.0, seed=3)
    sc = gpu.CsrPlan(C.nrows, C.ncols, dev(C.pos), dev(C.crd)).stats()
    assert sc["kernel_name"] == "subwarp" and sc["width"] == 64
    D, _ = gen.config5(scale=(110 / 192) ** 3)
    sd = gpu.CsrPlan(D.nrows, D.ncols, dev(D.pos), dev(D.crd)).stats()
    assert sd["kernel_name"] == "nnzsplit" and sd["mean_chunk_col_span"] < 3 * 110 * 110


def test_unaligned_buffers_take_the_scalar_path(gpu, oracle):
    A = gen.poisson_random(5000, 20.0, seed=9)
    x = gen.uniform_vector(A.ncols, 1)
    want = np.zeros(A.nrows)
    oracle.spmv(A.pos, A.crd, A.val, x, want)
    scale = oracle.spmv_abs_scale(A.pos, A.crd, A.val, x)
    pos, crd, val = dev(A.pos), dev_unaligned(A.crd), dev_unaligned(A.val)
    for kid in (2, 3):
        plan = gpu.CsrPlan(A.nrows, A.ncols, pos, crd).set_kernel(kid)
        y = torch.zeros(A.nrows, dtype=torch.float64, device="cuda")
        gpu.spmv(plan, A.nrows, A.ncols, pos, crd, val, dev(x), y)
        torch.cuda.synchronize()
        assert_rows_close(y.cpu().numpy(), want, scale, np.float64, "unaligned/%d" % kid)


def test_repeated_calls_accumulate_and_are_deterministic(gpu, oracle):
    A = gen.powerlaw_random(20000, 30.0, 200000, seed=5, dtype=np.float64)
    x = gen.uniform_vector(A.ncols, 2)
    pos, crd, val, dx = dev(A.pos), dev(A.crd), dev(A.val), dev(x)
    plan = gpu.CsrPlan(A.nrows, A.ncols, pos, crd)
    runs = []
    for _ in range(2):
        y = torch.zeros(A.nrows, dtype=torch.float64, device="cuda")
        for _ in range(3):
            gpu.spmv(plan, A.nrows, A.ncols, pos, crd, val, dx, y)
        torch.cuda.synchronize()
        runs.append(y.cpu().numpy())
    assert np.array_equal(runs[0], runs[1])  # fixed summation order, no atomics on y
    want = np.zeros(A.nrows)
    for _ in range(3):
        oracle.spmv(A.pos, A.crd, A.val, x, want)
    assert_rows_close(runs[0], want, 3 * oracle.spmv_abs_scale(A.pos, A.crd, A.val, x), np.float64, "3 calls")


def test_bad_structure_is_rejected_before_any_kernel_reads_it(gpu):
    pos = dev(np.array([0, 2, 1, 3], np.int32))
    crd = dev(np.array([0, 1, 2], np.int32))
    with pytest.raises(gpu.LapisHipError) as e:
        gpu.CsrPlan(3, 3, pos, crd)
    assert e.value.status_name == "LAPIS_HIP_ERR_BAD_CSR"
    pos = dev(np.array([0, 1, 2, 3], np.int32))
    with pytest.raises(gpu.LapisHipError) as e:
        gpu.CsrPlan(3, 3, pos, dev(np.array([0, 3, 1], np.int32)))
    assert e.value.status_name == "LAPIS_HIP_ERR_BAD_CSR"
    with pytest.raises(gpu.LapisHipError) as e:
        gpu.CsrPlan(3, 3, pos, crd, nnz=5)
    assert e.value.status_name == "LAPIS_HIP_ERR_BAD_CSR"
    plan = gpu.CsrPlan(3, 3, pos, crd)
    other = dev(np.array([0, 1, 2, 3], np.int32))
    y = torch.zeros(3, dtype=torch.float64, device="cuda")
    with pytest.raises(gpu.LapisHipError) as e:
        gpu.spmv(plan, 3, 3, other, crd, y, y, y)
    assert e.value.status_name == "LAPIS_HIP_ERR_PLAN_MISMATCH"


def test_empty_matrix_is_a_no_op(gpu):
    pos = dev(np.zeros(1, np.int32))
    crd = torch.empty(0, dtype=torch.int32, device="cuda")
    plan = gpu.CsrPlan(0, 0, pos, crd)
    y = torch.empty(0, dtype=torch.float64, device="cuda")
    gpu.spmv(plan, 0, 0, pos, crd, y, y, y)
    torch.cuda.synchronize()


@pytest.mark.parametrize("kernel", ["rowblock", "nnzsplit", "colblock-group", "colblock-wave"])
def test_spmv_replays_from_a_hip_graph(gpu, oracle, kernel):
    # A planned SpMV is kernel launches only (no allocation, no host read, no memset), so a
    # caller can capture it.  The graph is replayed several times with eager work and
    # synchronisation in between, and every replay is checked against the eager result.
    A, x = gen.config2(scale=1 / 64)
    pos, crd, val, dx = dev(A.pos), dev(A.crd), dev(A.val), dev(x)
    plan = gpu.CsrPlan(A.nrows, A.ncols, pos, crd)
    if kernel.startswith("colblock"):
        plan.build_colblock(crd, val, layout=kernel.split("-")[1])
    else:
        plan.set_kernel(KID[kernel], 0)
    want = np.zeros(A.nrows)
    oracle.spmv(A.pos, A.crd, A.val, x, want)
    scale = oracle.spmv_abs_scale(A.pos, A.crd, A.val, x)
    y = torch.zeros(A.nrows, dtype=torch.float64, device="cuda")
    gpu.spmv(plan, A.nrows, A.ncols, pos, crd, val, dx, y)  # eager: also does the one-time kernel attribute call
    torch.cuda.synchronize()
    assert_rows_close(y.cpu().numpy(), want, scale, np.float64, kernel + " eager")
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        y.zero_()
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            gpu.spmv(plan, A.nrows, A.ncols, pos, crd, val, dx, y)
    torch.cuda.synchronize()
    for replay in range(3):
        y.zero_()                       # eager work between the replays
        scratch = (dx * 2.0).sum().item()  # and a host synchronisation
        assert np.isfinite(scratch)
        graph.replay()
        torch.cuda.synchronize()
        assert_rows_close(y.cpu().numpy(), want, scale, np.float64, "%s replay %d" % (kernel, replay))
    plan.destroy()


def test_plans_give_back_their_device_memory(gpu):
    # build and destroy plans with both column-blocked layouts (long rows included) many times:
    # the free device memory must come back to where it was
    A = gen.powerlaw_random(131072, 30.0, 200000, seed=3003, dtype=np.float64)
    pos, crd, val = dev(A.pos), dev(A.crd), dev(A.val)
    torch.cuda.synchronize()

    def cycle():
        for layout in ("group", "wave", "group"):
            plan = gpu.CsrPlan(A.nrows, A.ncols, pos, crd)
            plan.build_colblock(crd, val, 0, layout=layout)
            plan.build_colblock(crd, val, 9, layout="group")  # rebuilding replaces the copy
            plan.destroy()

    cycle()  # first use may grow library-internal pools (radix sort, kernel code)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(5):
        cycle()
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free0 - free1 < (8 << 20), "plans leak %.1f MB over 15 build/destroy cycles" % ((free0 - free1) / 1e6)


@pytest.mark.parametrize("layout", ["group", "wave"])
def test_column_blocked_copy_follows_value_updates_and_refuses_other_buffers(gpu, oracle, layout):
    # the reference reads val on every call; a copy has to be told: update_values refreshes it in one
    # gather pass, and a call with buffers the copy was not made from is refused
    A = gen.poisson_random(30000, 9.0, seed=21)
    x = gen.uniform_vector(A.ncols, 22)
    pos, crd, val, dx = dev(A.pos), dev(A.crd), dev(A.val), dev(x)
    plan = gpu.CsrPlan(A.nrows, A.ncols, pos, crd)
    plan.build_colblock(crd, val, 9, layout=layout)

    def run(values):
        y = torch.zeros(A.nrows, dtype=torch.float64, device="cuda")
        gpu.spmv(plan, A.nrows, A.ncols, pos, crd, values, dx, y)
        torch.cuda.synchronize()
        return y.cpu().numpy()

    def expect(values_host):
        want = np.zeros(A.nrows)
        oracle.spmv(A.pos, A.crd, values_host, x, want)
        return want, oracle.spmv_abs_scale(A.pos, A.crd, values_host, x)

    want, scale = expect(A.val)
    assert_rows_close(run(val), want, scale, np.float64, "as built")
    # scale the values in place, as scale_csr of examples/hitting_times.py:51-71 does
    gpu.scale(-0.375, val)
    plan.update_values(val)
    want2, scale2 = expect(A.val * -0.375)
    assert_rows_close(run(val), want2, scale2, np.float64, "after update_values")
    # other values in another buffer: refused until update_values is given that buffer
    other_host = gen.uniform_vector(A.nnz, 23)
    other = dev(other_host)
    with pytest.raises(gpu.LapisHipError) as e:
        run(other)
    assert e.value.status_name == "LAPIS_HIP_ERR_PLAN_MISMATCH"
    with pytest.raises(gpu.LapisHipError) as e:
        y = torch.zeros(A.nrows, dtype=torch.float64, device="cuda")
        gpu.spmv(plan, A.nrows, A.ncols, pos, dev(A.crd), val, dx, y)  # same coordinates, another buffer
    assert e.value.status_name == "LAPIS_HIP_ERR_PLAN_MISMATCH"
    plan.update_values(other)
    want3, scale3 = expect(other_host)
    assert_rows_close(run(other), want3, scale3, np.float64, "after update_values with another buffer")
    plan.destroy()


def test_analyze_builds_the_copy_only_where_it_is_recommended(gpu, oracle):
    # wide uniformly random columns, more than 2^20 non-zeros: the gathers of a chunk range over all of x
    A = gen.poisson_random(600000, 4.0, seed=31)
    x = gen.uniform_vector(A.ncols, 32)
    pos, crd, val = dev(A.pos), dev(A.crd), dev(A.val)
    plan = gpu.CsrPlan(A.nrows, A.ncols, pos, crd)
    assert plan.stats()["colblock_recommended"] == 1 and plan.stats()["kernel_name"] in ("rowblock", "nnzsplit")
    plan.analyze(crd, val)
    s = plan.stats()
    assert s["kernel_name"] == "colblock" and s["colblock_layout_name"] == "group"
    y = torch.zeros(A.nrows, dtype=torch.float64, device="cuda")
    gpu.spmv(plan, A.nrows, A.ncols, pos, crd, val, dev(x), y)
    torch.cuda.synchronize()
    want = np.zeros(A.nrows)
    oracle.spmv(A.pos, A.crd, A.val, x, want)
    assert_rows_close(y.cpu().numpy(), want, oracle.spmv_abs_scale(A.pos, A.crd, A.val, x), np.float64, "analyze")
    plan.analyze(crd, val)  # a second call keeps the copy and refreshes its values
    assert plan.stats()["kernel_name"] == "colblock"
    plan.destroy()
    # a stencil: the gathers stay inside a window L2 holds, the plan keeps its CSR kernel
    L, _ = gen.config5(scale=(110 / 192) ** 3)
    lp, lc, lv = dev(L.pos), dev(L.crd), dev(L.val)
    plan = gpu.CsrPlan(L.nrows, L.ncols, lp, lc)
    plan.analyze(lc, lv)
    assert plan.stats()["kernel_name"] == "nnzsplit" and plan.stats()["colblock_layout_name"] is None


def test_a_kept_plan_is_never_used_on_another_structure_in_the_same_buffers(gpu, oracle):
    # What emitted code that keeps a plan between calls of a generated function has to survive: the
    # function's operands are uploaded anew at every call and a second matrix of the same shape lands at
    # the same device addresses.  lapis_hip_csr_plan_matches tells the plan of A from matrix B (another
    # number of non-zeros); with the plan rebuilt the answer is B's, never A's.
    n = 20000
    A = gen.poisson_random(n, 9.0, seed=51)
    B = gen.poisson_random(n, 5.0, seed=52)
    assert A.nnz > B.nnz and A.nrows == B.nrows and A.ncols == B.ncols
    x = gen.uniform_vector(n, 53)
    pos = torch.empty(n + 1, dtype=torch.int32, device="cuda")
    crd = torch.empty(A.nnz, dtype=torch.int32, device="cuda")
    val = torch.empty(A.nnz, dtype=torch.float64, device="cuda")
    dx = dev(x)

    def upload(M):
        pos.copy_(torch.from_numpy(M.pos))
        crd[:M.nnz].copy_(torch.from_numpy(M.crd))
        val[:M.nnz].copy_(torch.from_numpy(M.val))

    def multiply(plan, M):
        y = torch.zeros(n, dtype=torch.float64, device="cuda")
        gpu.spmv(plan, n, n, pos, crd, val, dx, y)
        torch.cuda.synchronize()
        want = np.zeros(n)
        oracle.spmv(M.pos, M.crd, M.val, x, want)
        return y.cpu().numpy(), want, oracle.spmv_abs_scale(M.pos, M.crd, M.val, x)

    upload(A)
    plan = gpu.CsrPlan(n, n, pos, crd, nnz=A.nnz)
    got, want, scale = multiply(plan, A)
    assert_rows_close(got, want, scale, np.float64, "A with its own plan")
    assert plan.matches(n, n, A.nnz, pos, crd)
    upload(B)  # same buffers, same shape, other structure
    assert not plan.matches(n, n, B.nnz, pos, crd), "the plan of A must not pass for B"
    assert not plan.matches(n, n, A.nnz, pos, dev(A.crd)) and not plan.matches(n + 1, n, A.nnz, pos, crd)
    plan.destroy()
    plan = gpu.CsrPlan(n, n, pos, crd, nnz=B.nnz)  # what the emitted call does on a mismatch
    got, want, scale = multiply(plan, B)
    assert_rows_close(got, want, scale, np.float64, "B after the rebuild")
    wrong = np.zeros(n)
    oracle.spmv(A.pos, A.crd, A.val, x, wrong)
    assert not np.allclose(got, wrong)
    plan.destroy()


def test_reproducible_analysis_gives_the_same_bits_every_run(gpu, oracle):
    A = gen.poisson_random(600000, 4.0, seed=31)
    x = gen.uniform_vector(A.ncols, 32)
    pos, crd, val, dx = dev(A.pos), dev(A.crd), dev(A.val), dev(x)
    plan = gpu.CsrPlan(A.nrows, A.ncols, pos, crd)
    plan.analyze_reproducible(crd, val)
    s = plan.stats()
    assert s["kernel_name"] == "colblock" and s["colblock_layout_name"] == "wave"
    runs = []
    for _ in range(3):
        y = torch.zeros(A.nrows, dtype=torch.float64, device="cuda")
        gpu.spmv(plan, A.nrows, A.ncols, pos, crd, val, dx, y)
        torch.cuda.synchronize()
        runs.append(y.cpu().numpy())
    assert np.array_equal(runs[0], runs[1]) and np.array_equal(runs[0], runs[2])
    want = np.zeros(A.nrows)
    oracle.spmv(A.pos, A.crd, A.val, x, want)
    assert_rows_close(runs[0], want, oracle.spmv_abs_scale(A.pos, A.crd, A.val, x), np.float64, "reproducible")
    plan.analyze(crd, val)  # the other layout on request: the copy is rebuilt, not reused
    assert plan.stats()["colblock_layout_name"] == "group"
    plan.destroy()


@pytest.mark.parametrize("kernel", ["nnzsplit", "rowblock"])
def test_long_runs_of_empty_rows(gpu, oracle, kernel):
    # three million empty rows between the rows that hold the entries of one chunk, and again before the last row
    rng = np.random.default_rng(5)
    lengths = np.zeros(4_000_000, dtype=np.int64)
    lengths[[0, 1, 2, 70, 3_000_000, 3_000_001, 3_999_999]] = [3, 600, 2, 90, 700, 5, 40]
    lengths[rng.integers(3_000_002, 3_999_000, 50)] = rng.integers(1, 30, 50)
    A = _from_lengths(lengths, 5000, 77, np.float64)
    x = gen.uniform_vector(A.ncols, 78)
    y_in = gen.uniform_vector(A.nrows, 79)
    want = y_in.copy()
    oracle.spmv(A.pos, A.crd, A.val, x, want)
    scale = oracle.spmv_abs_scale(A.pos, A.crd, A.val, x, y_in)
    pos, crd, val = dev(A.pos), dev(A.crd), dev(A.val)
    plan = gpu.CsrPlan(A.nrows, A.ncols, pos, crd)
    plan.set_kernel({"rowblock": 2, "nnzsplit": 3}[kernel])
    y = dev(y_in)
    gpu.spmv(plan, A.nrows, A.ncols, pos, crd, val, dev(x), y)
    torch.cuda.synchronize()
    assert_rows_close(y.cpu().numpy(), want, scale, np.float64, "empty runs/" + kernel)


def test_config1_at_its_full_size(gpu, oracle):
    # the first benchmark configuration itself: the 5-point Laplacian on the 256 x 256 grid (65 536 rows, 326 656 non-zeros)
    A, x = gen.config1()
    assert (A.nrows, A.nnz) == (65536, 326656)
    want = np.zeros(A.nrows)
    oracle.spmv(A.pos, A.crd, A.val, x, want)
    scale = oracle.spmv_abs_scale(A.pos, A.crd, A.val, x)
    pos, crd, val, dx = dev(A.pos), dev(A.crd), dev(A.val), dev(x)
    for kernel in (0, 1, 2, 3):  # the plan's choice, then each CSR kernel family
        plan = gpu.CsrPlan(A.nrows, A.ncols, pos, crd)
        if kernel:
            plan.set_kernel(kernel, 1 if kernel == 1 else 0)
        y = torch.zeros(A.nrows, dtype=torch.float64, device="cuda")
        gpu.spmv(plan, A.nrows, A.ncols, pos, crd, val, dx, y)
        torch.cuda.synchronize()
        got = y.cpu().numpy()
        assert_rows_close(got, want, scale, np.float64, "config1/kernel %d" % kernel)
        if kernel in (1, 2):  # one lane per row and the row-block kernel add in the oracle's order: bit for bit
            assert np.array_equal(got, want)
    # interior rows of a Laplacian annihilate the constant vector
    ones = torch.ones(A.ncols, dtype=torch.float64, device="cuda")
    y = torch.zeros(A.nrows, dtype=torch.float64, device="cuda")
    gpu.spmv(gpu.CsrPlan(A.nrows, A.ncols, pos, crd), A.nrows, A.ncols, pos, crd, val, ones, y)
    interior = np.diff(A.pos) == 5
    assert np.all(y.cpu().numpy()[interior] == 0.0)


def test_kernel_timing_counts_the_dominant_kernel_launches(gpu):
    # what bench.py's roofline figure rests on: one event pair per launch of the SpMV main kernel
    A = gen.laplace2d(64)
    pos, crd, val = dev(A.pos), dev(A.crd), dev(A.val)
    x, y = dev(gen.uniform_vector(A.ncols, 3)), dev(np.zeros(A.nrows))
    plan = gpu.CsrPlan(A.nrows, A.ncols, pos, crd, value_bytes=8)
    gpu.kernel_timing_start(5)
    for _ in range(7):  # more launches than capacity: the later ones are not timed
        gpu.spmv(plan, A.nrows, A.ncols, pos, crd, val, x, y)
    t = gpu.kernel_timing_stop()
    assert t["count"] == 5
    assert 0.0 < t["min_ms"] <= t["median_ms"] <= t["max_ms"] < 50.0
    assert t["min_ms"] <= t["mean_ms"] <= t["max_ms"]
    with pytest.raises(gpu.LapisHipError):
        gpu.kernel_timing_stop()  # not started
