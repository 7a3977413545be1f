"""dot / axpby / mult / div / fill / copy / scale parity on the GPU through the C ABI."""
import numpy as np
import pytest
import torch

from gpu_util import dev, dev_unaligned
from lapis_amd import generators as gen

pytestmark = pytest.mark.gpu

SIZES = [0, 1, 2, 3, 63, 64, 255, 256, 257, 4099, 1 << 20, (1 << 20) + 7]


@pytest.mark.parametrize("n", SIZES)
def test_elementwise_ops_are_bit_exact(gpu, oracle, n):
    # elementwise results have no summation order: they must equal the oracle bit for bit
    x = gen.uniform_vector(n, 1) if n else np.zeros(0)
    y = gen.uniform_vector(n, 2) + 1.5 if n else np.zeros(0)
    dx, dy = dev(x), dev(y)
    out = torch.empty(n, dtype=torch.float64, device="cuda")
    gpu.axpby(0.75, dx, -1.25, dy, out)
    assert np.array_equal(out.cpu().numpy(), oracle.axpby(0.75, x, -1.25, y))
    gpu.mult(dx, dy, out)
    assert np.array_equal(out.cpu().numpy(), x * y)
    gpu.div(dx, dy, out)
    assert np.array_equal(out.cpu().numpy(), x / y)
    gpu.copy(dx, out)
    assert np.array_equal(out.cpu().numpy(), x)
    gpu.fill(out, 3.25)
    assert np.array_equal(out.cpu().numpy(), np.full(n, 3.25))
    gpu.scale(-2.0, dx)
    assert np.array_equal(dx.cpu().numpy(), x * -2.0)
    # in place, as CG uses it: x = 1*x + a*p
    acc = dev(y)
    gpu.axpby(1.0, acc, 0.5, dev(x), acc)
    assert np.array_equal(acc.cpu().numpy(), oracle.axpby(1.0, y, 0.5, x))


def test_elementwise_f32_and_unaligned(gpu, oracle):
    n = 10007
    x = gen.uniform_vector(n, 3, dtype=np.float32)
    y = gen.uniform_vector(n, 4, dtype=np.float32)
    out = torch.empty(n, dtype=torch.float32, device="cuda")
    gpu.axpby(2.0, dev(x), 3.0, dev(y), out)
    assert np.array_equal(out.cpu().numpy(), oracle.axpby(2.0, x, 3.0, y))
    x64, y64 = x.astype(np.float64), y.astype(np.float64)
    out64 = dev_unaligned(np.zeros(n))
    gpu.axpby(2.0, dev_unaligned(x64), 3.0, dev(y64), out64)
    assert np.array_equal(out64.cpu().numpy(), oracle.axpby(2.0, x64, 3.0, y64))


@pytest.mark.parametrize("n", SIZES)
def test_dot_matches_oracle_within_summation_error(gpu, oracle, n):
    x = gen.uniform_vector(n, 5) if n else np.zeros(0)
    y = gen.uniform_vector(n, 6) if n else np.zeros(0)
    res = torch.full((1,), 123.0, dtype=torch.float64, device="cuda")
    gpu.dot(dev(x), dev(y), res, init_value=0.5)
    want = oracle.dot(x, y, init=0.5)
    scale = np.abs(x * y).sum() + 0.5
    assert abs(res.item() - want) <= 1e-12 * scale
    # the same call twice gives the same bits (fixed reduction order)
    res2 = torch.zeros(1, dtype=torch.float64, device="cuda")
    gpu.dot(dev(x), dev(y), res2, init_value=0.5)
    assert res.item() == res2.item()


def test_dot_f32_and_closed_form(gpu):
    n = 100000
    i = np.arange(1, n + 1, dtype=np.float64)
    res = torch.zeros(1, dtype=torch.float64, device="cuda")
    gpu.dot(dev(i), dev(np.ones(n)), res)
    assert res.item() == n * (n + 1) / 2  # integers below 2^53: exact in any order
    xf = gen.uniform_vector(n, 7, dtype=np.float32)
    resf = torch.zeros(1, dtype=torch.float32, device="cuda")
    gpu.dot(dev(xf), dev(xf), resf)
    assert abs(resf.item() - float((xf.astype(np.float64) ** 2).sum())) <= 1e-5 * float((xf.astype(np.float64) ** 2).sum())


def test_many_dots_in_flight_use_separate_scratch(gpu):
    n = 50000
    xs = [dev(gen.uniform_vector(n, 100 + k)) for k in range(8)]
    res = torch.zeros(8, dtype=torch.float64, device="cuda")
    for rep in range(20):
        for k in range(8):
            gpu.dot(xs[k], xs[k], res[k:k + 1])
    torch.cuda.synchronize()
    want = [float((x.cpu().numpy() ** 2).sum()) for x in xs]
    assert np.allclose(res.cpu().numpy(), want, rtol=1e-13)


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("n", [0, 1, 3, 1000, 4097, 1 << 20, (1 << 20) + 3])
def test_dot_with_its_result_on_the_host(gpu, oracle, dtype, n):
    # the entry emitted code calls where the reference reduces into a host scalar: same bits as the
    # device-scalar entry, and the oracle's value within the reordering tolerance
    x, y = gen.uniform_vector(n, 21, dtype=dtype), gen.uniform_vector(n, 22, dtype=dtype)
    dx, dy = dev(x), dev(y)
    got = gpu.dot_host(dx, dy, 0.5)
    res = torch.zeros(1, dtype=dx.dtype, device="cuda")
    gpu.dot(dx, dy, res, 0.5)
    torch.cuda.synchronize()
    assert np.asarray(got, dtype=dtype) == res.cpu().numpy()[0]
    want = oracle.dot(x.astype(np.float64), y.astype(np.float64), 0.5)
    scale = float(np.abs(x.astype(np.float64) * y.astype(np.float64)).sum()) + 0.5
    assert abs(got - want) <= (1e-12 if dtype == np.float64 else 1e-5) * scale


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("n", [1, 2, 255, 4096, 100003, 1 << 21])
@pytest.mark.parametrize("other_z", [False, True])
def test_fused_axpby_dot_has_the_bits_of_the_two_calls(gpu, dtype, n, other_z):
    # r = r - alpha * Ap followed by r . r (examples/pcg_solve.py:80-82) in one pass
    x, y, z = (gen.uniform_vector(n, s, dtype=dtype) for s in (31, 32, 33))
    a, b = 1.0, -0.37
    dx, dy, dz = dev(x), dev(y), dev(z)
    dst1, res1 = torch.empty_like(dx), torch.zeros(1, dtype=dx.dtype, device="cuda")
    gpu.axpby(a, dx, b, dy, dst1)
    gpu.dot(dst1, dz if other_z else dst1, res1, 0.25)
    dst2, res2 = dx.clone(), torch.zeros(1, dtype=dx.dtype, device="cuda")  # in place on x, as CG does with r
    gpu.axpby_dot(a, dst2, b, dy, dst2, dz if other_z else None, res2, 0.25)
    torch.cuda.synchronize()
    assert torch.equal(dst1, dst2)
    assert torch.equal(res1, res2)
    want = dtype(a) * x + dtype(b) * y  # separate multiply and add, as the oracle's axpby
    assert np.array_equal(dst2.cpu().numpy(), want.astype(dtype))


def test_fused_axpby_dot_on_unaligned_buffers_stays_within_tolerance(gpu):
    n = 5001
    x, y = gen.uniform_vector(n + 1, 41), gen.uniform_vector(n + 1, 42)
    dx, dy = dev(x)[1:], dev(y)[1:]  # 8 bytes past a 16-byte boundary
    dst, res = torch.empty(n, dtype=torch.float64, device="cuda"), torch.zeros(1, dtype=torch.float64, device="cuda")
    gpu.axpby_dot(2.0, dx, -1.0, dy, dst, None, res)
    torch.cuda.synchronize()
    want = 2.0 * x[1:] + -1.0 * y[1:]
    assert np.array_equal(dst.cpu().numpy(), want)
    assert abs(res.item() - float(want @ want)) <= 1e-12 * float(want @ want)


def test_vector_kernels_beyond_two_to_the_31_elements(gpu):
    """2.3 thousand million fp32 elements: the element count does not fit 32 bits.  Constant vectors, so that
    every result is known exactly and the far end of the arrays is checked as well as the start."""
    import torch
    n = 2_300_000_000
    x = torch.full((n,), 0.5, device="cuda", dtype=torch.float32)
    y = torch.full((n,), 2.0, device="cuda", dtype=torch.float32)
    d = torch.empty(n, device="cuda", dtype=torch.float32)
    assert gpu.dot_host(x, y) == float(n)
    gpu.axpby(2.0, x, 0.25, y, d)
    assert d.min().item() == 1.5 and d.max().item() == 1.5 and d[n - 1].item() == 1.5
    gpu.mult(x, y, d)
    assert d.min().item() == 1.0 and d.max().item() == 1.0
    gpu.fill(d, 3.0)
    assert d.min().item() == 3.0 and d[n - 1].item() == 3.0
    gpu.copy(x, d)
    assert d.max().item() == 0.5 and d[n - 1].item() == 0.5
