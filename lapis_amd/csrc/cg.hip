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
//
// A dot product never needs a launch of its own: the vector kernel that produces the
// operands leaves one partial per block, and EVERY block of the next vector kernel
// adds those partials (at most 2048 doubles, from L2) in index order before it
// starts, so all blocks hold the same bits of alpha, beta and relres.  Kernel
// boundaries do the ordering; no block needs a device-scope fence (on a multi-XCD
// part such a fence writes back and invalidates L2, and two thousand of them per
// kernel cost more than the vector pass itself).  The iteration number is a kernel
// argument (the host knows which iteration it is queueing); scalars that one kernel
// both reads and replaces (r.z) are kept twice, indexed by iteration parity.
//
// x is needed by nobody until the solve ends, so x += alpha p is made by the kernel
// that reads p anyway to replace it (p = z + beta p), not by the one that updates r:
// p is then read twice per iteration (by the SpMV's gathers and by that kernel), not
// three times.  The pass that decides to leave still adds its alpha p and leaves p alone.
#include <algorithm>
#include <cmath>

#include "blas1.hpp"
#include "common.hpp"
#include "plan.hpp"
#include "rowsplit_fix.hpp"

namespace lapis {

struct CgState {
  double pAp;      // p . Ap of the last iteration (diagnostic)
  double rz[2];    // r . z entering iteration i is rz[i & 1]
  double rr;       // r . r after the update
  double initres;  // sqrt(r0 . r0)
  double relres;
  double alpha;    // r.z / p.Ap of the iteration under way
  unsigned long long done_iter;  // 0 while iterating, then the reference's counter i at exit (it starts at 1)
  unsigned long long maxiter;
  double tol;
};

__device__ __forceinline__ double block_sum_256d(double v, double *lds4) {
  v = group_sum<64>(v);
  if ((threadIdx.x & 63) == 0) lds4[threadIdx.x >> 6] = v;
  __syncthreads();
  const double total = ((lds4[0] + lds4[1]) + lds4[2]) + lds4[3];
  __syncthreads();
  return total;
}

// The exit mark, read once per block: block 0 of the kernel that makes the convergence
// test sets it while other blocks of the same kernel may still be starting, and
// every thread of a block has to take the same way past the barriers below.
__device__ __forceinline__ unsigned long long block_done_iter(const CgState *st) {
  __shared__ unsigned long long seen;
  if (threadIdx.x == 0) seen = st->done_iter;
  __syncthreads();
  const unsigned long long d = seen;
  __syncthreads();
  return d;
}

// Sum of partials[0..count) in a fixed order, by one block of 256 threads.
__device__ __forceinline__ double ordered_total(const double *partials, int count, double *lds4) {
  double s = 0.0;
  for (int i = threadIdx.x; i < count; i += 256) s = s + partials[i];
  return block_sum_256d(s, lds4);
}

// The vector passes below walk their arrays two doubles (one 128-bit access) per
// thread and trip when every array is 16-byte aligned (`vec`), element by element
// otherwise; an odd last element is taken by the scalar tail.
#define CG_GRID_STRIDE(i, first, count) \
  for (long long i = (first) + (long long)blockIdx.x * 256 + threadIdx.x; i < (count); i += (long long)gridDim.x * 256)

__device__ __forceinline__ v2d ld2(const double *p, long long i) { return reinterpret_cast<const v2d *>(p)[i]; }
__device__ __forceinline__ void st2(double *p, long long i, v2d v) { reinterpret_cast<v2d *>(p)[i] = v; }

// r0 = b, z0 = r0*dinv (or r0), p0 = z0, x0 = 0; block partials of r0.r0 and r0.z0.
__global__ __launch_bounds__(256) void cg_init_kernel(long long n, const double *__restrict__ b,
                                                      const double *__restrict__ dinv, double *__restrict__ x,
                                                      double *__restrict__ r, double *__restrict__ z,
                                                      double *__restrict__ p, double *__restrict__ partials,
                                                      int divide) {
  __shared__ double lds4[4];
  double rr = 0.0, rz = 0.0;
  CG_GRID_STRIDE(i, 0, n) {
    const double ri = b[i];
    const double zi = dinv ? (divide ? ri / dinv[i] : ri * dinv[i]) : ri;
    r[i] = ri;
    if (dinv) z[i] = zi;
    p[i] = zi;
    x[i] = 0.0;
    rr = rr + ri * ri;
    rz = rz + ri * zi;
  }
  const double brr = block_sum_256d(rr, lds4);
  const double brz = block_sum_256d(rz, lds4);
  if (threadIdx.x == 0) {
    partials[blockIdx.x] = brr;
    partials[kDotMaxBlocks + blockIdx.x] = brz;
  }
}

// block partials of p . Ap
__global__ __launch_bounds__(256) void cg_pap_kernel(long long n, const double *__restrict__ p,
                                                     const double *__restrict__ Ap, double *__restrict__ partials,
                                                     int vec) {
  __shared__ double lds4[4];
  double acc = 0.0;
  const long long nv = vec ? n / 2 : 0;
  CG_GRID_STRIDE(i, 0, nv) {
    const v2d a = ld2(p, i), b = ld2(Ap, i);
    acc = acc + a.x * b.x;
    acc = acc + a.y * b.y;
  }
  CG_GRID_STRIDE(i, 2 * nv, n) acc = acc + p[i] * Ap[i];
  const double bsum = block_sum_256d(acc, lds4);
  if (threadIdx.x == 0) partials[blockIdx.x] = bsum;
}

// The same partials when Ap came from the row-split SpMV kernel with its fix-up left out
// and the chunk sums of p[r]*Ap[r] over uncut rows taken (`chunk_pap`): thread t of a
// block completes the row cut at chunk boundary c (if that boundary is the first to cut
// it), adds that row's p[r]*Ap[r], and adds chunk c's sum.  Neither vector is read in
// full again.  Chunks and boundaries are dealt to blocks and lanes in a fixed order.
template <int CH>
__global__ __launch_bounds__(256) void cg_pap_fix_kernel(int nchunks, int chunks_per_block,
                                                         const double *__restrict__ p, double *Ap,
                                                         const double *__restrict__ chunk_pap,
                                                         double *__restrict__ partials,
                                                         const int *__restrict__ pos,
                                                         const int *__restrict__ chunk_row,
                                                         const double *__restrict__ part_first,
                                                         const double *__restrict__ part_last) {
  __shared__ double lds4[4];
  const long long c0 = (long long)blockIdx.x * chunks_per_block;
  const long long c1 = std::min<long long>(nchunks, c0 + chunks_per_block);
  double acc = 0.0;
  for (long long base = c0; base < c1; base += 256) {
    const long long c = base + threadIdx.x;
    const bool mine = c < c1;
    bool owner;
    int r;
    const double total = rowsplit_row_total<double, CH>((mine && c >= 1) ? c : nchunks, nchunks, pos, chunk_row,
                                                        part_first, part_last, owner, r);
    if (owner) {
      Ap[r] = total;
      acc = acc + p[r] * total;
    }
    if (mine) acc = acc + chunk_pap[c];
  }
  const double bsum = block_sum_256d(acc, lds4);
  if (threadIdx.x == 0) partials[blockIdx.x] = bsum;
}

// r -= alpha Ap ; block partials of r.r.   alpha = r.z / p.Ap with p.Ap summed here from the
// partials the p.Ap kernel left; block 0 keeps alpha for the kernel that updates x and p.
// Ap is read here for the last time: it goes through streaming accesses, so that it does not
// push p, which the next SpMV gathers from, out of the caches.
__global__ __launch_bounds__(256) void cg_update_r_kernel(long long n, const double *__restrict__ Ap,
                                                          double *__restrict__ r, CgState *st,
                                                          unsigned long long iter, int count,
                                                          const double *__restrict__ pap_partials,
                                                          double *__restrict__ rr_partials, int vec) {
  __shared__ double lds4[4];
  if (block_done_iter(st)) return;
  const double pAp = ordered_total(pap_partials, count, lds4);
  const double alpha = st->rz[iter & 1] / pAp;
  const double malpha = -alpha;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    st->pAp = pAp;
    st->alpha = alpha;
  }
  double rr = 0.0;
  const long long nv = vec ? n / 2 : 0;
  CG_GRID_STRIDE(i, 0, nv) {
    const v2d av = load_stream(reinterpret_cast<const v2d *>(Ap) + i);
    v2d rv = ld2(r, i);
    rv.x = rv.x + av.x * malpha;
    rv.y = rv.y + av.y * malpha;
    st2(r, i, rv);
    rr = rr + rv.x * rv.x;
    rr = rr + rv.y * rv.y;
  }
  CG_GRID_STRIDE(i, 2 * nv, n) {
    const double rt = Ap[i] * malpha;
    const double ri = r[i] + rt;
    r[i] = ri;
    rr = rr + ri * ri;
  }
  const double bsum = block_sum_256d(rr, lds4);
  if (threadIdx.x == 0) rr_partials[blockIdx.x] = bsum;
}

// The convergence test of examples/pcg_solve.py:84-90, made by every block from the
// r.r partials: leave when !(relres > tol) or i == maxiter.  Block 0 records the exit.
__device__ __forceinline__ bool cg_continues(CgState *st, unsigned long long iter, double rr) {
  const double relres = sqrt(rr) / st->initres;
  const bool go_on = (relres > st->tol) && (iter != st->maxiter);
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    st->rr = rr;
    st->relres = relres;
    if (!go_on) st->done_iter = iter;
  }
  return go_on;
}

// Convergence test, then z = r * dinv (or r / dinv) ; block partials of r.z     (preconditioned runs only)
__global__ __launch_bounds__(256) void cg_precond_kernel(long long n, const double *__restrict__ r,
                                                         const double *__restrict__ dinv, double *__restrict__ z,
                                                         CgState *st, unsigned long long iter, int count,
                                                         const double *__restrict__ rr_partials,
                                                         double *__restrict__ rz_partials, int vec, int divide) {
  __shared__ double lds4[4];
  if (block_done_iter(st)) return;  // an earlier pass left, or block 0 of this kernel has just decided to
  const double rr = ordered_total(rr_partials, count, lds4);
  if (!cg_continues(st, iter, rr)) return;
  double acc = 0.0;
  const long long nv = vec ? n / 2 : 0;
  CG_GRID_STRIDE(i, 0, nv) {
    // r and the preconditioner are read here for the last time in this iteration
    const v2d rv = load_stream(reinterpret_cast<const v2d *>(r) + i);
    const v2d dv = load_stream(reinterpret_cast<const v2d *>(dinv) + i);
    v2d zv;
    zv.x = divide ? rv.x / dv.x : rv.x * dv.x;
    zv.y = divide ? rv.y / dv.y : rv.y * dv.y;
    st2(z, i, zv);
    acc = acc + rv.x * zv.x;
    acc = acc + rv.y * zv.y;
  }
  CG_GRID_STRIDE(i, 2 * nv, n) {
    const double ri = r[i];
    const double zi = divide ? ri / dinv[i] : ri * dinv[i];
    z[i] = zi;
    acc = acc + ri * zi;
  }
  const double bsum = block_sum_256d(acc, lds4);
  if (threadIdx.x == 0) rz_partials[blockIdx.x] = bsum;
}

// Elementwise pieces of the masked operator and of the moment right-hand sides
// (examples/hitting_times.py:73-93, :166-177, :181-198).
// mode 0: out = (d*t - out) * m     (end of plpt; t = mask*x, out holds A t)
// mode 1: out = (d*t + out) * m     (right-hand side of the second moment; t = mom1, out holds A mom1)
__global__ __launch_bounds__(256) void masked_combine_kernel(long long n, int mode, const double *__restrict__ d,
                                                             const double *__restrict__ t,
                                                             const double *__restrict__ m, double *out) {
  CG_GRID_STRIDE(i, 0, n) {
    const double t1 = d[i] * t[i];
    const double t2 = mode == 0 ? t1 - out[i] : t1 + out[i];
    out[i] = t2 * m[i];
  }
}

__global__ __launch_bounds__(256) void normalize_mom2_kernel(long long n, const double *__restrict__ m1,
                                                             const double *__restrict__ m2, double *__restrict__ out) {
  CG_GRID_STRIDE(i, 0, n) {
    const double sq = m1[i] * m1[i];
    out[i] = sqrt(m2[i] - sq);
  }
}

// x += alpha p ; p = z + beta p with beta = (new r.z) / (old r.z).  Unpreconditioned, z is r
// and the new r.z is r.r: this kernel then makes the convergence test itself; preconditioned,
// the test was made by cg_precond_kernel and `partials` holds r.z.  The pass that leaves
// (the exit mark names this very iteration) still owes x its alpha p and keeps p as it is;
// passes queued behind it find an older mark and touch nothing.  x goes through streaming
// accesses: it is touched once per iteration and must not push p out of the caches.
__global__ __launch_bounds__(256) void cg_update_xp_kernel(long long n, const double *__restrict__ z,
                                                           double *__restrict__ p, double *__restrict__ x,
                                                           CgState *st, unsigned long long iter, int count,
                                                           const double *__restrict__ partials, int preconditioned,
                                                           int vec) {
  __shared__ double lds4[4];
  const unsigned long long mark = block_done_iter(st);
  if (mark != 0 && mark != iter) return;
  const double rz_new = ordered_total(partials, count, lds4);
  const bool go_on = preconditioned ? mark == 0 : cg_continues(st, iter, rz_new);
  const double alpha = st->alpha;
  const long long nv = vec ? n / 2 : 0;
  if (!go_on) {
    CG_GRID_STRIDE(i, 0, nv) {
      const v2d pv = ld2(p, i);
      v2d xv = load_stream(reinterpret_cast<const v2d *>(x) + i);
      xv.x = xv.x + pv.x * alpha;
      xv.y = xv.y + pv.y * alpha;
      store_stream(reinterpret_cast<v2d *>(x) + i, xv);
    }
    CG_GRID_STRIDE(i, 2 * nv, n) {
      const double xt = p[i] * alpha;
      x[i] = x[i] + xt;
    }
    return;
  }
  const double beta = rz_new / st->rz[iter & 1];
  if (blockIdx.x == 0 && threadIdx.x == 0) st->rz[(iter + 1) & 1] = rz_new;
  CG_GRID_STRIDE(i, 0, nv) {
    const v2d zv = load_stream(reinterpret_cast<const v2d *>(z) + i);
    v2d pv = ld2(p, i);
    v2d xv = load_stream(reinterpret_cast<const v2d *>(x) + i);
    xv.x = xv.x + pv.x * alpha;
    xv.y = xv.y + pv.y * alpha;
    store_stream(reinterpret_cast<v2d *>(x) + i, xv);
    pv.x = zv.x + pv.x * beta;
    pv.y = zv.y + pv.y * beta;
    st2(p, i, pv);
  }
  CG_GRID_STRIDE(i, 2 * nv, n) {
    const double pi = p[i];
    const double xt = pi * alpha;
    x[i] = x[i] + xt;
    const double pt = pi * beta;
    p[i] = z[i] + pt;
  }
}

// One block, once per solve: the scalars of the initial residual.
__global__ __launch_bounds__(256) void cg_init_scalar_kernel(int count, const double *__restrict__ partials,
                                                             CgState *st) {
  __shared__ double lds4[4];
  const double trr = ordered_total(partials, count, lds4);
  const double trz = ordered_total(partials + kDotMaxBlocks, count, lds4);
  if (threadIdx.x == 0) {
    st->initres = sqrt(trr);
    st->rz[1] = trz;  // the first iteration is i = 1
    st->done_iter = 0;
  }
}

}  // namespace lapis

using namespace lapis;

namespace {

// What the solver applies as A and as the preconditioner.
//   mask == nullptr: A p is the SpMV, z = r * prec (prec may be null: z = r)      examples/pcg_solve.py:52-101
//   mask != nullptr: A p is plpt, y = mask*(d*(mask*p) - A (mask*p)), z = r / d   examples/hitting_times.py:97-149
// work holds 4 vectors (5 with a mask), `stride` apart.
int pcg_run(lapis_hip_csr_plan *plan, int64_t n, const int32_t *pos, const int32_t *crd, const double *val,
            const double *b, const double *dinv, const double *mask, double tol, uint64_t maxiter, double *x,
            uint64_t *iters, double *relres, double *work, lapis_hip_stream_t stream) {
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
  int64_t stride = n;  // distance between the four work vectors
  CgState *state = nullptr;
  double *partials = nullptr;
  double *chunk_pap = nullptr;  // per chunk of the row-split SpMV: p.Ap over the rows inside it
  bool finished = false;

  // one-exit cleanup
  auto cleanup = [&]() {
    if (own_plan) lapis_hip_csr_plan_destroy(own_plan);
    if (own_work) (void)hipFree(own_work);
    if (state) (void)hipFree(state);
    if (partials) (void)hipFree(partials);
    if (chunk_pap) (void)hipFree(chunk_pap);
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
    // the column-blocked copy costs about as much as 40 SpMVs of such a matrix: build it
    // only when the iteration limit allows it to pay back
    if (maxiter >= 64) PCG_RC(lapis_hip_csr_plan_analyze(own_plan, crd, val, 8, stream));
  }
  if (!work) {
    // own scratch: an even stride keeps all four vectors 16-byte aligned
    stride = (n + 1) & ~(int64_t)1;
    PCG_TRY(hipMalloc(&own_work, sizeof(double) * (mask ? 5 : 4) * (size_t)stride));
    work = own_work;
  }
  double *r = work, *z = dinv ? work + stride : work, *p = work + 2 * stride, *Ap = work + 3 * stride;
  double *tmp = mask ? work + 4 * stride : nullptr;
  const int divide = mask ? 1 : 0;
  PCG_TRY(hipMalloc(&state, sizeof(CgState)));
  PCG_TRY(hipMalloc(&partials, sizeof(double) * 3 * kDotMaxBlocks));
  if (!mask && plan->stats.kernel == LAPIS_HIP_SPMV_NNZSPLIT && plan->nchunks > 1)
    PCG_TRY(hipMalloc(&chunk_pap, sizeof(double) * (size_t)plan->nchunks));
  CgState h{};
  h.maxiter = maxiter;
  h.tol = tol;
  PCG_TRY(hipMemcpyAsync(state, &h, sizeof(h), hipMemcpyHostToDevice, st));

  const int grid = dot_grid(n);
  const int pre = dinv ? 1 : 0;
  const int vec = (aligned16(x) && aligned16(r) && aligned16(z) && aligned16(p) && aligned16(Ap) &&
                   (!dinv || aligned16(dinv)))
                      ? 1
                      : 0;
  hipLaunchKernelGGL(cg_init_kernel, dim3(grid), dim3(256), 0, st, (long long)n, b, dinv, x, r, z, p, partials,
                     divide);
  hipLaunchKernelGGL(cg_init_scalar_kernel, dim3(1), dim3(256), 0, st, grid, partials, state);
  PCG_TRY(hipGetLastError());
  double *pap_partials = partials, *rr_partials = partials + kDotMaxBlocks, *rz_partials = partials + 2 * kDotMaxBlocks;
  // The host looks at the device's exit mark after each batch of iterations; a
  // batch queued past convergence costs launches only (its kernels return at once
  // or touch scratch vectors only).
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
      int deferred = 0;  // chunk length when the SpMV left its cut rows to the p.Ap kernel
      if (mask) {
        // plpt: tmp = mask*p ; Ap = A tmp ; Ap = (d*tmp - Ap)*mask
        PCG_RC(lapis_hip_mult_f64(n, p, mask, tmp, stream));
        PCG_RC(spmv_overwrite_f64(plan, n, n, pos, crd, val, tmp, Ap, stream));
        hipLaunchKernelGGL(masked_combine_kernel, dim3(grid), dim3(256), 0, st, (long long)n, 0, dinv, tmp, mask, Ap);
      } else {
        // Ap = A p: the reference zero-fills Ap and accumulates (examples/pcg_solve.py:12-19)
        PCG_RC(spmv_overwrite_f64(plan, n, n, pos, crd, val, p, Ap, stream, chunk_pap ? &deferred : nullptr,
                                  chunk_pap));
      }
      const unsigned long long iter = launched + (uint64_t)it + 1;  // the reference's counter for this pass
      int pap_count = grid;
      if (deferred) {
        // one thread per chunk, at most kDotMaxBlocks blocks
        const int nchunks = plan->nchunks;
        const int per_block = (int)std::max<int64_t>(256, ceil_div(ceil_div(nchunks, kDotMaxBlocks), 256) * 256);
        pap_count = (int)ceil_div(nchunks, per_block);
#define PCG_PAP_FIX(CH)                                                                                         \
  hipLaunchKernelGGL(cg_pap_fix_kernel<CH>, dim3(pap_count), dim3(256), 0, st, nchunks, per_block, p, Ap,        \
                     (const double *)chunk_pap, pap_partials, pos, (const int *)plan->chunk_row,                \
                     (const double *)plan->part_first, (const double *)plan->part_last)
        switch (deferred) {
          case 512: PCG_PAP_FIX(512); break;
          case 1024: PCG_PAP_FIX(1024); break;
          case 2048: PCG_PAP_FIX(2048); break;
          default:
            cleanup();
            return set_error(LAPIS_HIP_ERR_RUNTIME, "pcg: no p.Ap kernel for chunks of %d non-zeros", deferred);
        }
#undef PCG_PAP_FIX
      } else {
        hipLaunchKernelGGL(cg_pap_kernel, dim3(grid), dim3(256), 0, st, (long long)n, p, Ap, pap_partials, vec);
      }
      hipLaunchKernelGGL(cg_update_r_kernel, dim3(grid), dim3(256), 0, st, (long long)n, Ap, r, state, iter,
                         pap_count, pap_partials, rr_partials, vec);
      if (pre)
        hipLaunchKernelGGL(cg_precond_kernel, dim3(grid), dim3(256), 0, st, (long long)n, r, dinv, z, state, iter,
                           grid, rr_partials, rz_partials, vec, divide);
      hipLaunchKernelGGL(cg_update_xp_kernel, dim3(grid), dim3(256), 0, st, (long long)n, z, p, x, state, iter,
                         grid, pre ? rz_partials : rr_partials, pre, vec);
      PCG_TRY(hipGetLastError());
    }
    launched += (uint64_t)todo;
    CgState now;
    PCG_TRY(hipMemcpyAsync(&now, state, sizeof(now), hipMemcpyDeviceToHost, st));
    PCG_TRY(hipStreamSynchronize(st));
    if (now.done_iter != 0) {
      *iters = now.done_iter;
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

}  // namespace

extern "C" int lapis_hip_pcg_f64_i32(lapis_hip_csr_plan *plan, int64_t n, const int32_t *pos, const int32_t *crd,
                                     const double *val, const double *b, const double *dinv, double tol,
                                     uint64_t maxiter, double *x, uint64_t *iters, double *relres, double *work,
                                     lapis_hip_stream_t stream) {
  return pcg_run(plan, n, pos, crd, val, b, dinv, nullptr, tol, maxiter, x, iters, relres, work, stream);
}

extern "C" int lapis_hip_pcg_masked_f64_i32(lapis_hip_csr_plan *plan, int64_t n, const int32_t *pos,
                                            const int32_t *crd, const double *val, const double *b,
                                            const double *mask, const double *d, double tol, uint64_t maxiter,
                                            double *x, uint64_t *iters, double *relres, double *work,
                                            lapis_hip_stream_t stream) {
  LAPIS_REQUIRE(n == 0 || (mask && d), "pcg_masked: null mask or diagonal");
  return pcg_run(plan, n, pos, crd, val, b, d, mask, tol, maxiter, x, iters, relres, work, stream);
}

extern "C" int lapis_hip_mht_f64_i32(lapis_hip_csr_plan *plan, int64_t n, int64_t nnz, const int32_t *pos,
                                     const int32_t *crd, double *val, const double *mask, const double *d,
                                     double alpha, double tol, uint64_t maxiter, double *mom1, double *mom2,
                                     lapis_hip_stream_t stream) {
  LAPIS_CHECK_INIT();
  LAPIS_REQUIRE(n >= 0 && nnz >= 0, "mht: negative size");
  if (n == 0) return LAPIS_HIP_OK;
  LAPIS_REQUIRE(pos && mask && d && mom1 && mom2 && (nnz == 0 || (crd && val)), "mht: null argument");
  hipStream_t st = as_stream(stream);
  double *bbuf = nullptr;
  LAPIS_HIP_TRY(hipMalloc(&bbuf, sizeof(double) * (size_t)n));
  uint64_t its = 0;
  double res = 0.0;
  int rc = lapis_hip_scale_f64(nnz, alpha, val, stream);  // scale_csr, in place
  // a column-blocked copy inside the caller's plan still holds the unscaled values
  if (rc == LAPIS_HIP_OK && plan) rc = lapis_hip_csr_plan_update_values(plan, val, 8, stream);
  if (rc == LAPIS_HIP_OK) rc = lapis_hip_mult_f64(n, d, mask, bbuf, stream);
  if (rc == LAPIS_HIP_OK)
    rc = lapis_hip_pcg_masked_f64_i32(plan, n, pos, crd, val, bbuf, mask, d, tol, maxiter, mom1, &its, &res, nullptr,
                                      stream);
  if (rc == LAPIS_HIP_OK) rc = spmv_overwrite_f64(plan, n, n, pos, crd, val, mom1, bbuf, stream);
  if (rc == LAPIS_HIP_OK) {
    hipLaunchKernelGGL(masked_combine_kernel, dim3(dot_grid(n)), dim3(256), 0, st, (long long)n, 1, d,
                       (const double *)mom1, mask, bbuf);
    if (hipGetLastError() != hipSuccess) rc = set_error(LAPIS_HIP_ERR_RUNTIME, "mht: kernel launch failed");
  }
  if (rc == LAPIS_HIP_OK)
    rc = lapis_hip_pcg_masked_f64_i32(plan, n, pos, crd, val, bbuf, mask, d, tol, maxiter, mom2, &its, &res, nullptr,
                                      stream);
  (void)hipStreamSynchronize(st);
  (void)hipFree(bbuf);
  return rc;
}

extern "C" int lapis_hip_normalize_mom2_f64(int64_t n, const double *mom1, const double *mom2, double *out,
                                            lapis_hip_stream_t stream) {
  LAPIS_CHECK_INIT();
  LAPIS_REQUIRE(n >= 0, "normalize_mom2: negative size");
  if (n == 0) return LAPIS_HIP_OK;
  LAPIS_REQUIRE(mom1 && mom2 && out, "normalize_mom2: null argument");
  hipLaunchKernelGGL(normalize_mom2_kernel, dim3(dot_grid(n)), dim3(256), 0, as_stream(stream), (long long)n, mom1,
                     mom2, out);
  LAPIS_LAUNCH_CHECK();
  return LAPIS_HIP_OK;
}
