/*
 * CPU oracle for the CSR SpMV / SpMM / CG hot path of LAPIS-generated modules.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP library is
 * compared against; nothing in the shipped library links or calls it.  It is a
 * plain-C restatement of the loop nests that the reference emits for its Kokkos
 * Serial / OpenMP host backends, in the reference's own summation order, with
 * separate multiply and add (build with -ffp-contract=off).  All paths cited
 * below are relative to the reference tree.
 *
 * Pinning status (see tests/test_oracle_*.py):
 *   spmv_*      : literal answer of examples/spmv_noalloc.py, scipy.sparse,
 *                 dense brute force, stencil eigenvectors           -> pinned
 *   spmm_*      : literal 3x4 case of examples/spmm_dcsr_opdsl.py, numpy
 *                 matmul, brute force                               -> pinned
 *   dot/axpby/mult/fill/copy : examples/multiple_results.py vectors, numpy
 *                 closed forms                                       -> pinned
 *   pcg         : nos4 vs scipy cg (examples/pcg_solve.py), exact solve of a
 *                 Laplacian with known solution                      -> pinned
 *   mht chain   : literal gold vectors of examples/hitting_times.py -> pinned
 *   vector-length rule : table of values derived from
 *                 LAPISSupport.hpp:428-435                           -> pinned
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------- */
/* SpMV: y[i] = (sum_{j=pos[i]}^{pos[i+1]-1} val[j]*x[crd[j]]) + y_in[i]     */
/* Loop shape: tests/Dialect/Kokkos/loop_mapping_2.mlir.gold:12-37.          */
/* The inner reduction starts from the Sum identity 0 and adds products in   */
/* ascending j (Kokkos host backends run ThreadVectorRange sequentially);    */
/* the incoming y is joined last: TranslateToKokkosCpp.cpp:1671-1690         */
/* (joinReductionInit) and :2127-2157 (lreduce = lreduce + prod).            */
/* ------------------------------------------------------------------------- */
#define DEFINE_SPMV(NAME, T)                                                   \
  void NAME(int64_t nrows, const int32_t *pos, const int32_t *crd,             \
            const T *val, const T *x, T *y) {                                  \
    for (int64_t i = 0; i < nrows; i++) {                                      \
      T yin = y[i];                                                            \
      T acc = (T)0;                                                            \
      for (int64_t j = pos[i]; j < pos[i + 1]; j++) {                          \
        T prod = val[j] * x[crd[j]];                                           \
        acc = acc + prod;                                                      \
      }                                                                        \
      y[i] = acc + yin;                                                        \
    }                                                                          \
  }

DEFINE_SPMV(oracle_spmv_csr_f64_i32, double)
DEFINE_SPMV(oracle_spmv_csr_f32_i32, float)

/* Same loop nest with the row loop distributed over OpenMP threads, as the
 * Kokkos OpenMP backend distributes the league (static schedule).  Used only
 * as the timed CPU baseline. */
#define DEFINE_SPMV_OMP(NAME, T)                                               \
  void NAME(int64_t nrows, const int32_t *pos, const int32_t *crd,             \
            const T *val, const T *x, T *y) {                                  \
    _Pragma("omp parallel for schedule(static)")                               \
    for (int64_t i = 0; i < nrows; i++) {                                      \
      T yin = y[i];                                                            \
      T acc = (T)0;                                                            \
      for (int64_t j = pos[i]; j < pos[i + 1]; j++) {                          \
        T prod = val[j] * x[crd[j]];                                           \
        acc = acc + prod;                                                      \
      }                                                                        \
      y[i] = acc + yin;                                                        \
    }                                                                          \
  }

DEFINE_SPMV_OMP(oracle_spmv_csr_f64_i32_omp, double)
DEFINE_SPMV_OMP(oracle_spmv_csr_f32_i32_omp, float)

int oracle_omp_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* Row-wise sum of |val*x| — the scale the parity tolerance is taken against
 * (rows of a Laplacian cancel to ~0, so |y| itself is not a usable scale). */
#define DEFINE_SPMV_ABS(NAME, T)                                               \
  void NAME(int64_t nrows, const int32_t *pos, const int32_t *crd,             \
            const T *val, const T *x, const T *yin, double *scale) {           \
    for (int64_t i = 0; i < nrows; i++) {                                      \
      double acc = yin ? fabs((double)yin[i]) : 0.0;                           \
      for (int64_t j = pos[i]; j < pos[i + 1]; j++)                            \
        acc += fabs((double)val[j] * (double)x[crd[j]]);                       \
      scale[i] = acc;                                                          \
    }                                                                          \
  }
DEFINE_SPMV_ABS(oracle_spmv_abs_scale_f64_i32, double)
DEFINE_SPMV_ABS(oracle_spmv_abs_scale_f32_i32, float)

/* ------------------------------------------------------------------------- */
/* SpMM: C[i,:] += sum_kk val[kk] * B[crd[kk],:]  (CSR A, row-major B and C) */
/* Loop order i -> kk -> j with C updated in place at every kk, as the       */
/* sparsifier emits for linalg.matmul / the generic of                       */
/* examples/spmm_dcsr_opdsl.py:73-110 under the race-free strategies         */
/* (Pipelines/Passes.h:41-56; examples/bspmm.py:92-100).                     */
/* ------------------------------------------------------------------------- */
#define DEFINE_SPMM(NAME, T)                                                   \
  void NAME(int64_t nrows, int64_t k, const int32_t *pos, const int32_t *crd,  \
            const T *val, const T *B, int64_t ldb, T *C, int64_t ldc) {        \
    for (int64_t i = 0; i < nrows; i++) {                                      \
      for (int64_t kk = pos[i]; kk < pos[i + 1]; kk++) {                       \
        T a = val[kk];                                                         \
        const T *brow = B + (int64_t)crd[kk] * ldb;                            \
        for (int64_t j = 0; j < k; j++) {                                      \
          T prod = a * brow[j];                                                \
          C[i * ldc + j] = C[i * ldc + j] + prod;                              \
        }                                                                      \
      }                                                                        \
    }                                                                          \
  }
DEFINE_SPMM(oracle_spmm_csr_f32_i32, float)
DEFINE_SPMM(oracle_spmm_csr_f64_i32, double)

#define DEFINE_SPMM_OMP(NAME, T)                                               \
  void NAME(int64_t nrows, int64_t k, const int32_t *pos, const int32_t *crd,  \
            const T *val, const T *B, int64_t ldb, T *C, int64_t ldc) {        \
    _Pragma("omp parallel for schedule(static)")                               \
    for (int64_t i = 0; i < nrows; i++) {                                      \
      for (int64_t kk = pos[i]; kk < pos[i + 1]; kk++) {                       \
        T a = val[kk];                                                         \
        const T *brow = B + (int64_t)crd[kk] * ldb;                            \
        for (int64_t j = 0; j < k; j++) {                                      \
          T prod = a * brow[j];                                                \
          C[i * ldc + j] = C[i * ldc + j] + prod;                              \
        }                                                                      \
      }                                                                        \
    }                                                                          \
  }
DEFINE_SPMM_OMP(oracle_spmm_csr_f32_i32_omp, float)

/* Batched CSRV SpMM of examples/bspmm.py:22-50:
 * out(n1, dh, nh) += attn(n1, n2, nh) * v(n2, dh, nh); attn is CSR over
 * (n1, n2) whose values carry a trailing dense batch of length nh. */
void oracle_bspmm_csrv_f32_i32(int64_t n1, int64_t dh, int64_t nh,
                               const int32_t *pos, const int32_t *crd,
                               const float *val, const float *V, float *out) {
  for (int64_t i = 0; i < n1; i++)
    for (int64_t kk = pos[i]; kk < pos[i + 1]; kk++) {
      int64_t c = crd[kk];
      for (int64_t d = 0; d < dh; d++)
        for (int64_t h = 0; h < nh; h++) {
          float prod = val[kk * nh + h] * V[(c * dh + d) * nh + h];
          out[(i * dh + d) * nh + h] = prod + out[(i * dh + d) * nh + h];
        }
    }
}

/* ------------------------------------------------------------------------- */
/* Dense vector ops of examples/pcg_solve.py:22-47 after                     */
/* DenseLinalgToParallelLoops.cpp:227-272,349-393.                           */
/* ------------------------------------------------------------------------- */

/* linalg.dot -> scf.parallel + scf.reduce(addf)
 * (tests/Dialect/Kokkos/linalg_to_loops_0.mlir.gold:7-18): partial sum from 0
 * in ascending i, then joined with the initial value of the 0-d output. */
double oracle_dot_f64(int64_t n, const double *x, const double *y, double init) {
  double acc = 0.0;
  for (int64_t i = 0; i < n; i++) {
    double prod = x[i] * y[i];
    acc = acc + prod;
  }
  return acc + init;
}

float oracle_dot_f32(int64_t n, const float *x, const float *y, float init) {
  float acc = 0.0f;
  for (int64_t i = 0; i < n; i++) {
    float prod = x[i] * y[i];
    acc = acc + prod;
  }
  return acc + init;
}

double oracle_dot_f64_omp(int64_t n, const double *x, const double *y, double init) {
  double acc = 0.0;
  _Pragma("omp parallel for schedule(static) reduction(+ : acc)")
  for (int64_t i = 0; i < n; i++) acc += x[i] * y[i];
  return acc + init;
}

/* examples/pcg_solve.py:30-38: dst = x*a + y*b (two multiplies, one add). */
void oracle_axpby_f64(int64_t n, double a, const double *x, double b,
                      const double *y, double *dst) {
  for (int64_t i = 0; i < n; i++) {
    double t0 = x[i] * a;
    double t1 = y[i] * b;
    dst[i] = t0 + t1;
  }
}

void oracle_axpby_f32(int64_t n, float a, const float *x, float b,
                      const float *y, float *dst) {
  for (int64_t i = 0; i < n; i++) {
    float t0 = x[i] * a;
    float t1 = y[i] * b;
    dst[i] = t0 + t1;
  }
}

void oracle_axpby_f64_omp(int64_t n, double a, const double *x, double b,
                          const double *y, double *dst) {
  _Pragma("omp parallel for schedule(static)")
  for (int64_t i = 0; i < n; i++) {
    double t0 = x[i] * a;
    double t1 = y[i] * b;
    dst[i] = t0 + t1;
  }
}

/* examples/pcg_solve.py:40-47: dst = x*y. */
void oracle_mult_f64(int64_t n, const double *x, const double *y, double *dst) {
  for (int64_t i = 0; i < n; i++) dst[i] = x[i] * y[i];
}

/* linalg.div of examples/hitting_times.py:120,146: dst = x/y. */
void oracle_div_f64(int64_t n, const double *x, const double *y, double *dst) {
  for (int64_t i = 0; i < n; i++) dst[i] = x[i] / y[i];
}

/* linalg.add of examples/multiple_results.py:12. */
void oracle_add_f64(int64_t n, const double *x, const double *y, double *dst) {
  for (int64_t i = 0; i < n; i++) dst[i] = x[i] + y[i];
}

void oracle_fill_f64(int64_t n, double v, double *dst) {
  for (int64_t i = 0; i < n; i++) dst[i] = v;
}

void oracle_copy_f64(int64_t n, const double *src, double *dst) {
  memcpy(dst, src, (size_t)n * sizeof(double));
}

/* examples/multiple_results.py:8-19: returns x+y and ||x+y||_2. */
double oracle_plus_norm_f64(int64_t n, const double *x, const double *y,
                            double *x_plus_y) {
  oracle_add_f64(n, x, y, x_plus_y);
  /* the 0-d accumulator is tensor.empty: Kokkos view allocations are
   * zero-initialised unless WithoutInitializing is requested */
  double s = oracle_dot_f64(n, x_plus_y, x_plus_y, 0.0);
  return sqrt(s);
}

/* ------------------------------------------------------------------------- */
/* Launch-shape rule of the reference.                                       */
/* ------------------------------------------------------------------------- */

/* KokkosLoopMapping.cpp:279-323 (pinned by loop_mapping_2.mlir.gold:6-11):
 * ceil((R[N]-R[0])/N) in unsigned index arithmetic. */
uint64_t oracle_csr_parallelism_hint(int64_t nrows, const int32_t *pos) {
  uint64_t hi = (uint64_t)(int64_t)pos[nrows];
  uint64_t lo = (uint64_t)(int64_t)pos[0];
  uint64_t N = (uint64_t)nrows;
  if (N == 0) return 0;
  return (hi - lo + N - 1) / N;
}

/* LAPISSupport.hpp:428-435, with TranslateToKokkosCpp.cpp:2013-2019 for the
 * "no hint" case (hint 0 -> 8). */
int oracle_thread_parallel_vector_length(int64_t hint, int max_vector_length) {
  if (hint == 0) return 8;
  int par = (int)hint;
  if (par < 1) return 1;
  int v = 1;
  while (v < max_vector_length && v * 6 < par) v *= 2;
  return v;
}

/* ------------------------------------------------------------------------- */
/* Preconditioned CG of examples/pcg_solve.py:52-101.                        */
/* x0 = 0; the iteration counter starts at 1 and the loop leaves when        */
/* relres <= tol or i == maxiter (:84-90). Returns iters, writes x, relres.  */
/* work: 4*n doubles.                                                        */
/* ------------------------------------------------------------------------- */
static void spmv_zeroed(int64_t n, const int32_t *pos, const int32_t *crd,
                        const double *val, const double *x, double *y) {
  /* examples/pcg_solve.py:12-19: linalg.fill 0 then matvec accumulates */
  oracle_fill_f64(n, 0.0, y);
  oracle_spmv_csr_f64_i32(n, pos, crd, val, x, y);
}

uint64_t oracle_pcg_f64_i32(int64_t n, const int32_t *pos, const int32_t *crd,
                            const double *val, const double *b,
                            const double *dinv, double tol, uint64_t maxiter,
                            double *x, double *relres_out, double *work) {
  double *r = work, *z = work + n, *p = work + 2 * n, *Ap = work + 3 * n;
  oracle_copy_f64(n, b, r);
  oracle_mult_f64(n, r, dinv, z);
  oracle_copy_f64(n, z, p);
  oracle_fill_f64(n, 0.0, x);
  double rr0 = oracle_dot_f64(n, r, r, 0.0);
  double initres = sqrt(rr0);
  uint64_t i = 1;
  double relres;
  for (;;) {
    spmv_zeroed(n, pos, crd, val, p, Ap);
    double pAp = oracle_dot_f64(n, p, Ap, 0.0);
    double rz = oracle_dot_f64(n, r, z, 0.0);
    double alpha = rz / pAp;
    double malpha = -alpha;
    oracle_axpby_f64(n, 1.0, x, alpha, p, x);
    oracle_axpby_f64(n, 1.0, r, malpha, Ap, r);
    double rr = oracle_dot_f64(n, r, r, 0.0);
    double rnorm = sqrt(rr);
    relres = rnorm / initres;
    int not_converged = relres > tol;
    int below_maxiter = i != maxiter;
    if (!(not_converged && below_maxiter)) break;
    oracle_mult_f64(n, r, dinv, z);
    double rznext = oracle_dot_f64(n, r, z, 0.0);
    double beta = rznext / rz;
    oracle_axpby_f64(n, 1.0, z, beta, p, p);
    i = i + 1;
  }
  *relres_out = relres;
  return i;
}

/* ------------------------------------------------------------------------- */
/* Hitting-time moments of examples/hitting_times.py:49-198.                 */
/* ------------------------------------------------------------------------- */

/* :51-71 scale_csr, in place on the values. */
void oracle_scale_csr_f64(int64_t nnz, double alpha, double *val) {
  for (int64_t j = 0; j < nnz; j++) val[j] = val[j] * alpha;
}

/* :73-93 plpt: dst = mask*(d*(mask*x) - Aalpha*(mask*x)); tmp holds mask*x. */
void oracle_plpt_f64_i32(int64_t n, const int32_t *pos, const int32_t *crd,
                         const double *val, const double *x, const double *d,
                         const double *mask, double *tmp, double *dst) {
  oracle_mult_f64(n, x, mask, tmp);
  spmv_zeroed(n, pos, crd, val, tmp, dst);
  for (int64_t i = 0; i < n; i++) {
    double t1 = d[i] * tmp[i];
    double t2 = t1 - dst[i];
    dst[i] = t2 * mask[i];
  }
}

/* :97-149: the pcg variant whose operator is plpt and whose preconditioner is
 * an elementwise division by d.  work: 5*n doubles. */
uint64_t oracle_pcg_masked_f64_i32(int64_t n, const int32_t *pos,
                                   const int32_t *crd, const double *val,
                                   const double *b, const double *mask,
                                   const double *d, double tol,
                                   uint64_t maxiter, double *x,
                                   double *relres_out, double *work) {
  double *r = work, *z = work + n, *p = work + 2 * n, *Ap = work + 3 * n,
         *tmp = work + 4 * n;
  oracle_copy_f64(n, b, r);
  oracle_div_f64(n, r, d, z);
  oracle_copy_f64(n, z, p);
  oracle_fill_f64(n, 0.0, x);
  double rr0 = oracle_dot_f64(n, r, r, 0.0);
  double initres = sqrt(rr0);
  uint64_t i = 1;
  double relres;
  for (;;) {
    oracle_plpt_f64_i32(n, pos, crd, val, p, d, mask, tmp, Ap);
    double pAp = oracle_dot_f64(n, p, Ap, 0.0);
    double rz = oracle_dot_f64(n, r, z, 0.0);
    double alpha = rz / pAp;
    double malpha = -alpha;
    oracle_axpby_f64(n, 1.0, x, alpha, p, x);
    oracle_axpby_f64(n, 1.0, r, malpha, Ap, r);
    double rr = oracle_dot_f64(n, r, r, 0.0);
    relres = sqrt(rr) / initres;
    if (!((relres > tol) && (i != maxiter))) break;
    oracle_div_f64(n, r, d, z);
    double rznext = oracle_dot_f64(n, r, z, 0.0);
    double beta = rznext / rz;
    oracle_axpby_f64(n, 1.0, z, beta, p, p);
    i = i + 1;
  }
  *relres_out = relres;
  return i;
}

/* :153-179 mht: scales val by alpha IN PLACE, then two masked CG solves.
 * work: 6*n doubles. */
void oracle_mht_f64_i32(int64_t n, int64_t nnz, const int32_t *pos,
                        const int32_t *crd, double *val, const double *mask,
                        const double *d, double alpha, double tol,
                        uint64_t maxiter, double *mom1, double *mom2,
                        double *work) {
  double *bbuf = work, *cgwork = work + n;
  double relres;
  oracle_scale_csr_f64(nnz, alpha, val);
  oracle_mult_f64(n, d, mask, bbuf);
  oracle_pcg_masked_f64_i32(n, pos, crd, val, bbuf, mask, d, tol, maxiter, mom1,
                            &relres, cgwork);
  spmv_zeroed(n, pos, crd, val, mom1, bbuf);
  for (int64_t i = 0; i < n; i++) {
    double t1 = d[i] * mom1[i];
    double t2 = t1 + bbuf[i];
    bbuf[i] = t2 * mask[i];
  }
  oracle_pcg_masked_f64_i32(n, pos, crd, val, bbuf, mask, d, tol, maxiter, mom2,
                            &relres, cgwork);
}

/* :181-198 normalize_mom2: sqrt(m2 - m1*m1). */
void oracle_normalize_mom2_f64(int64_t n, const double *mom1, const double *mom2,
                               double *out) {
  for (int64_t i = 0; i < n; i++) {
    double sq = mom1[i] * mom1[i];
    double var = mom2[i] - sq;
    out[i] = sqrt(var);
  }
}
