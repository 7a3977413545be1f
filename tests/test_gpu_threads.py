"""Host threads calling the library at once, each on a stream of its own: the scratch ring of the dot
products, the per-thread error text and the plans must not get in each other's way."""
import threading

import numpy as np
import pytest
import scipy.sparse as sp
import torch

from gpu_util import dev

pytestmark = pytest.mark.gpu


def test_four_host_threads_on_four_streams(gpu, oracle):
    results, errors = {}, []

    def work(tid):
        try:
            rng = np.random.default_rng(900 + tid)
            n = 20000 + 3000 * tid
            cols = rng.integers(0, n, (n, 8))
            A = sp.csr_matrix((rng.standard_normal(8 * n), cols.ravel(), np.arange(0, 8 * n + 1, 8)), shape=(n, n))
            A.sum_duplicates()
            A.sort_indices()
            hp, hc, hv = A.indptr.astype(np.int32), A.indices.astype(np.int32), A.data
            x = rng.standard_normal(n)
            want = oracle.spmv(hp, hc, hv, x, np.zeros(n))
            stream = torch.cuda.Stream()  # default priority
            with torch.cuda.stream(stream):
                pos, crd, val, dx = dev(hp), dev(hc), dev(hv), dev(x)
                plan = gpu.CsrPlan(n, n, pos, crd, stream=stream)
                out = torch.zeros(1, dtype=torch.float64, device="cuda")
                worst, dots = 0.0, []
                for it in range(40):
                    y = torch.zeros(n, dtype=torch.float64, device="cuda")
                    gpu.spmv(plan, n, n, pos, crd, val, dx, y, stream=stream)
                    gpu.dot(y, dx, out, stream=stream)
                    dots.append(gpu.dot_host(y, y, stream=stream))
                    stream.synchronize()
                    worst = max(worst, float(np.max(np.abs(y.cpu().numpy() - want))))
                    dots.append(out.item())
                # an error raised in this thread carries this thread's text
                try:
                    gpu.spmv(plan, n + 1, n, pos, crd, val, dx, torch.zeros(n + 1, dtype=torch.float64, device="cuda"),
                             stream=stream)
                    errors.append("thread %d: a plan for n rows took n + 1" % tid)
                except (gpu.LapisHipError, ValueError) as e:
                    if isinstance(e, gpu.LapisHipError) and str(n + 1) not in str(e):
                        errors.append("thread %d got another thread's error text: %s" % (tid, e))
                plan.destroy()
            results[tid] = (worst, dots, float(want @ x), float(want @ want), np.abs(want).sum())
        except Exception as e:  # noqa: BLE001 - reported by the main thread
            errors.append("thread %d: %r" % (tid, e))

    threads = [threading.Thread(target=work, args=(t,)) for t in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a thread did not finish"
    assert not errors, errors
    for tid, (worst, dots, yx, yy, scale) in results.items():
        assert worst <= 1e-11 * max(1.0, scale / 1000), (tid, worst)
        for a, b in zip(dots[0::2], dots[1::2]):
            assert abs(a - yy) <= 1e-9 * abs(yy) and abs(b - yx) <= 1e-9 * (abs(yx) + scale), (tid, a, yy, b, yx)
