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
