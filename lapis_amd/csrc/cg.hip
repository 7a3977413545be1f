// Conjugate gradients on the device: the solver examples/pcg_solve.py:52-101
// lowers to, with its scalars kept in device memory between kernels.
//
// Reference iteration (one pass of the scf.while, :74-98):
//   Ap = A p ; pAp = p.Ap ; rz = r.z ; alpha = rz/pAp
//   x = 1*x + alpha*p ; r = 1*r + (-alpha)*Ap ; rr = r.r
//   relres = sqrt(rr)/sqrt(r0.r0) ; leave if !(relres > tol) or i == maxiter
//   z = r*dinv ; rz' = r.z ; beta = rz'/rz ; p = 1*z + beta*p ; i = i+1
// r.z at the top of an iteration is the rz' of the one before (same vectors), so
// it is carried instead of recomputed; without a preconditioner z is r and rz' is rr.
#include <algorithm>
#include <cmath>

#include "blas1.hpp"
#include "common.hpp"
#include "plan.hpp"

namespace lapis {

struct CgState {
  double pAp;      // p . Ap
  double rz;       // r . z of the current residual
  double rz_next;  // r . z after the update
  double rr;       // r . r after the update
  double initres;  // sqrt(r0 . r0)
  double relres;
  unsigned long long iter;  // the reference's counter i (starts at 1)
  unsigned long long maxiter;
  double tol;
  int done;
  unsigned ticket[3];
};

__device__ __forceinline__ double block_sum_256d(double v, double *lds4) {
  v = group_sum<64>(v);
  if ((threadIdx.x & 63) == 0) lds4[threadIdx.x >> 6] = v;
  __syncthreads();
  const double total = ((lds4[0] + lds4[1]) + lds4[2]) + lds4[3];
  __syncthreads();
  return total;
}

// Publishes this block's partial and tells whether this block is the last to do so;
// the last block then owns the ordered final sum.
__device__ __forceinline__ bool publish_partial(double v, double *partials, unsigned *ticket, bool *flag) {
  if (threadIdx.x == 0) {
    partials[blockIdx.x] = v;
    __threadfence();
    *flag = (atomicAdd(ticket, 1u) == gridDim.x - 1);
  }
  __syncthreads();
  const bool last = *flag;
  if (last) __threadfence();
  return last;
}

__device__ __forceinline__ double ordered_total(const double *partials, double *lds4) {
  double s = 0.0;
  for (unsigned i = threadIdx.x; i < gridDim.x; i += 256) s = s + partials[i];
  return block_sum_256d(s, lds4);
}

// r0 = b, z0 = r0*dinv (or r0), p0 = z0, x0 = 0; partial sums of r0.r0 and r0.z0.
__global__ __launch_bounds__(256) void cg_init_kernel(long long n, const double *__restrict__ b,
                                                      const double *__restrict__ dinv, double *__restrict__ x,
                                                      double *__restrict__ r, double *__restrict__ z,
                                                      double *__restrict__ p, CgState *st,
                                                      double *__restrict__ partials) {
  __shared__ double lds4[4];
  __shared__ bool flag;
  double rr = 0.0, rz = 0.0;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) {
    const double ri = b[i];
    const double zi = dinv ? ri * dinv[i] : ri;
    r[i] = ri;
    if (dinv) z[i] = zi;
    p[i] = zi;
    x[i] = 0.0;
    rr = rr + ri * ri;
    rz = rz + ri * zi;
  }
  const double brr = block_sum_256d(rr, lds4);
  const double brz = block_sum_256d(rz, lds4);
  if (threadIdx.x == 0) partials[kDotMaxBlocks + blockIdx.x] = brz;
  if (!publish_partial(brr, partials, &st->ticket[0], &flag)) return;
  const double trr = ordered_total(partials, lds4);
  const double trz = ordered_total(partials + kDotMaxBlocks, lds4);
  if (threadIdx.x == 0) {
    st->initres = sqrt(trr);
    st->rz = trz;
    st->iter = 1;
    st->done = 0;
    st->ticket[0] = 0u;
  }
}

// pAp = p . Ap
__global__ __launch_bounds__(256) void cg_pap_kernel(long long n, const double *__restrict__ p,
                                                     const double *__restrict__ Ap, CgState *st,
                                                     double *__restrict__ partials) {
  __shared__ double lds4[4];
  __shared__ bool flag;
  double acc = 0.0;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256)
    acc = acc + p[i] * Ap[i];
  const double bsum = block_sum_256d(acc, lds4);
  if (!publish_partial(bsum, partials, &st->ticket[0], &flag)) return;
  const double total = ordered_total(partials, lds4);
  if (threadIdx.x == 0) {
    st->pAp = total;
    st->ticket[0] = 0u;
  }
}

// x += alpha p ; r -= alpha Ap ; rr = r.r ; the last block decides convergence.
__global__ __launch_bounds__(256) void cg_update_xr_kernel(long long n, const double *__restrict__ p,
                                                           const double *__restrict__ Ap, double *__restrict__ x,
                                                           double *__restrict__ r, CgState *st,
                                                           double *__restrict__ partials, int preconditioned) {
  __shared__ double lds4[4];
  __shared__ bool flag;
  if (st->done) return;
  const double alpha = st->rz / st->pAp;
  const double malpha = -alpha;
  double rr = 0.0;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) {
    const double xt = p[i] * alpha;
    const double xi = x[i] + xt;
    const double rt = Ap[i] * malpha;
    const double ri = r[i] + rt;
    x[i] = xi;
    r[i] = ri;
    rr = rr + ri * ri;
  }
  const double bsum = block_sum_256d(rr, lds4);
  if (!publish_partial(bsum, partials, &st->ticket[1], &flag)) return;
  const double total = ordered_total(partials, lds4);
  if (threadIdx.x == 0) {
    const double relres = sqrt(total) / st->initres;
    st->rr = total;
    st->relres = relres;
    if (!preconditioned) st->rz_next = total;
    const bool go_on = (relres > st->tol) && (st->iter != st->maxiter);
    if (!go_on) st->done = 1;
    st->ticket[1] = 0u;
  }
}

// z = r * dinv ; rz_next = r.z     (preconditioned runs only)
__global__ __launch_bounds__(256) void cg_precond_kernel(long long n, const double *__restrict__ r,
                                                         const double *__restrict__ dinv, double *__restrict__ z,
                                                         CgState *st, double *__restrict__ partials) {
  __shared__ double lds4[4];
  __shared__ bool flag;
  if (st->done) return;
  double acc = 0.0;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) {
    const double ri = r[i];
    const double zi = ri * dinv[i];
    z[i] = zi;
    acc = acc + ri * zi;
  }
  const double bsum = block_sum_256d(acc, lds4);
  if (!publish_partial(bsum, partials, &st->ticket[2], &flag)) return;
  const double total = ordered_total(partials, lds4);
  if (threadIdx.x == 0) {
    st->rz_next = total;
    st->ticket[2] = 0u;
  }
}

// p = z + beta p with beta = rz_next/rz.  The scalars are rolled forward
// (rz = rz_next, i = i+1) by a separate one-thread kernel queued behind this one, so
// that every block of this kernel still reads the pair it needs.
__global__ __launch_bounds__(256) void cg_update_p_kernel(long long n, const double *__restrict__ z,
                                                          double *__restrict__ p, const CgState *st) {
  if (st->done) return;
  const double beta = st->rz_next / st->rz;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) {
    const double pt = p[i] * beta;
    p[i] = z[i] + pt;
  }
}

__global__ void cg_roll_kernel(CgState *st) {
  if (st->done) return;
  st->rz = st->rz_next;
  st->iter = st->iter + 1;
}

}  // namespace lapis

using namespace lapis;

extern "C" int lapis_hip_pcg_f64_i32(lapis_hip_csr_plan *plan, int64_t n, const int32_t *pos, const int32_t *crd,
                                     const double *val, const double *b, const double *dinv, double tol,
                                     uint64_t maxiter, double *x, uint64_t *iters, double *relres, double *work,
                                     lapis_hip_stream_t stream) {
  LAPIS_CHECK_INIT();
  LAPIS_REQUIRE(n >= 0, "pcg: negative size");
  LAPIS_REQUIRE(iters && relres, "pcg: null iters/relres output");
  hipStream_t st = as_stream(stream);
  if (n == 0) {
    // r0.r0 = 0: relres is 0/0 = NaN, `relres > tol` is false, the loop leaves at i = 1
    *iters = 1;
    *relres = std::nan("");
    return LAPIS_HIP_OK;
  }
  LAPIS_REQUIRE(pos && b && x, "pcg: null positions, right-hand side or solution");

  int rc = LAPIS_HIP_OK;
  lapis_hip_csr_plan *own_plan = nullptr;
  double *own_work = nullptr;
  CgState *state = nullptr;
  double *partials = nullptr;
  bool finished = false;

  // one-exit cleanup
  auto cleanup = [&]() {
    if (own_plan) lapis_hip_csr_plan_destroy(own_plan);
    if (own_work) (void)hipFree(own_work);
    if (state) (void)hipFree(state);
    if (partials) (void)hipFree(partials);
  };
#define PCG_TRY(expr)                                                                          \
  do {                                                                                         \
    hipError_t e_ = (expr);                                                                    \
    if (e_ != hipSuccess) {                                                                    \
      cleanup();                                                                               \
      return set_error(LAPIS_HIP_ERR_RUNTIME, "pcg: %s failed: %s", #expr, hipGetErrorString(e_)); \
    }                                                                                          \
  } while (0)
#define PCG_RC(expr)      \
  do {                    \
    rc = (expr);          \
    if (rc != LAPIS_HIP_OK) { \
      cleanup();          \
      return rc;          \
    }                     \
  } while (0)

  if (!plan) {
    int32_t nnz32 = 0;
    PCG_TRY(hipMemcpyAsync(&nnz32, pos + n, sizeof(int32_t), hipMemcpyDeviceToHost, st));
    PCG_TRY(hipStreamSynchronize(st));
    PCG_RC(lapis_hip_csr_plan_create(&own_plan, n, n, nnz32, pos, crd, 8, stream));
    plan = own_plan;
  }
  if (!work) {
    PCG_TRY(hipMalloc(&own_work, sizeof(double) * 4 * (size_t)n));
    work = own_work;
  }
  double *r = work, *z = dinv ? work + n : work, *p = work + 2 * n, *Ap = work + 3 * n;
  PCG_TRY(hipMalloc(&state, sizeof(CgState)));
  PCG_TRY(hipMalloc(&partials, sizeof(double) * 2 * kDotMaxBlocks));
  CgState h{};
  h.maxiter = maxiter;
  h.tol = tol;
  PCG_TRY(hipMemcpyAsync(state, &h, sizeof(h), hipMemcpyHostToDevice, st));

  const int grid = dot_grid(n);
  const int pre = dinv ? 1 : 0;
  hipLaunchKernelGGL(cg_init_kernel, dim3(grid), dim3(256), 0, st, (long long)n, b, dinv, x, r, z, p, state,
                     partials);
  PCG_TRY(hipGetLastError());

  // The host looks at the device's `done` flag after each batch of iterations; a
  // batch queued past convergence costs launches only (its kernels return at once
  // or touch scratch vectors only).
  struct Peek {
    unsigned long long iter;
    int done;
  };
  uint64_t launched = 0;
  int batch = 1;
  while (!finished) {
    int todo = batch;
    if (maxiter != 0) todo = (int)std::min<uint64_t>((uint64_t)todo, maxiter - launched);
    if (todo <= 0) {
      // iteration `maxiter` always raises the flag, so this is unreachable unless the state was corrupted
      cleanup();
      return set_error(LAPIS_HIP_ERR_RUNTIME, "pcg: %llu iterations queued and the device never reported an exit",
                       (unsigned long long)launched);
    }
    for (int it = 0; it < todo; ++it) {
      // Ap = A p: the reference zero-fills Ap and accumulates (examples/pcg_solve.py:12-19)
      PCG_RC(spmv_overwrite_f64(plan, n, n, pos, crd, val, p, Ap, stream));
      hipLaunchKernelGGL(cg_pap_kernel, dim3(grid), dim3(256), 0, st, (long long)n, p, Ap, state, partials);
      hipLaunchKernelGGL(cg_update_xr_kernel, dim3(grid), dim3(256), 0, st, (long long)n, p, Ap, x, r, state,
                         partials, pre);
      if (pre)
        hipLaunchKernelGGL(cg_precond_kernel, dim3(grid), dim3(256), 0, st, (long long)n, r, dinv, z, state,
                           partials);
      hipLaunchKernelGGL(cg_update_p_kernel, dim3(grid), dim3(256), 0, st, (long long)n, z, p, state);
      hipLaunchKernelGGL(cg_roll_kernel, dim3(1), dim3(1), 0, st, state);
      PCG_TRY(hipGetLastError());
    }
    launched += (uint64_t)todo;
    CgState now;
    PCG_TRY(hipMemcpyAsync(&now, state, sizeof(now), hipMemcpyDeviceToHost, st));
    PCG_TRY(hipStreamSynchronize(st));
    if (now.done) {
      *iters = now.iter;
      *relres = now.relres;
      finished = true;
    }
    batch = std::min(batch * 2, 32);
  }
  cleanup();
#undef PCG_TRY
#undef PCG_RC
  return LAPIS_HIP_OK;
}
