/*
 * lapis_module.h -- the calling convention of a LAPIS-generated module, as
 * exported by the prebuilt gfx950 module (liblapis_package_module.so).
 *
 * These are the symbols the reference's emitter writes into every generated
 * module (mlir/lib/Target/KokkosCpp/TranslateToKokkosCpp.cpp, "emitter"):
 *   lapis_initialize / lapis_finalize          emitter :4277-4378
 *   py_<func>(results..., params...)           emitter :2541-2684
 * Result slots come first; a memref result is StridedMemRefType<T,N>**, a
 * scalar result T*; a memref parameter is StridedMemRefType<T,N>*, a sparse
 * tensor's storage specifier is a struct of five int64 passed by reference
 * ({dimSizes[2], memSizes[3]} = ((m, n), (m+1, nnz, nnz))), scalars by value.
 * All buffers are HOST memory; a returned memref either aliases an input
 * parameter (updated in place) or points at memory the module owns until
 * lapis_finalize().  As in the reference there are no status codes: a memref
 * that is not unit-stride, an invalid CSR structure or a failed HIP call prints
 * a message and aborts.
 */
#ifndef LAPIS_MODULE_H
#define LAPIS_MODULE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* StridedMemRefType<T,1> of mlir/lib/Target/KokkosCpp/LAPISSupport.hpp:7-14 */
#define LAPIS_DECLARE_MEMREF_1D(NAME, T) \
  typedef struct NAME {                  \
    T *basePtr;                          \
    T *data;                             \
    int64_t offset;                      \
    int64_t sizes[1];                    \
    int64_t strides[1];                  \
  } NAME

LAPIS_DECLARE_MEMREF_1D(lapis_memref_1d_i32, int32_t);
LAPIS_DECLARE_MEMREF_1D(lapis_memref_1d_f64, double);
LAPIS_DECLARE_MEMREF_1D(lapis_memref_1d_f32, float);

/* StridedMemRefType<T,2> */
#define LAPIS_DECLARE_MEMREF_2D(NAME, T) \
  typedef struct NAME {                  \
    T *basePtr;                          \
    T *data;                             \
    int64_t offset;                      \
    int64_t sizes[2];                    \
    int64_t strides[2];                  \
  } NAME

LAPIS_DECLARE_MEMREF_2D(lapis_memref_2d_f32, float);
LAPIS_DECLARE_MEMREF_2D(lapis_memref_2d_f64, double);

/* StridedMemRefType<T,3> */
typedef struct lapis_memref_3d_f32 {
  float *basePtr;
  float *data;
  int64_t offset;
  int64_t sizes[3];
  int64_t strides[3];
} lapis_memref_3d_f32;

/* storage specifier of a decomposed 3-D CSRV tensor (dense, compressed, dense):
 * ((n1, n2, nh), (n1+1, nnz, nnz*nh)) as examples/bspmm.py:103 passes it */
typedef struct lapis_csrv_specifier {
  int64_t dimSizes[3];
  int64_t memSizes[3];
} lapis_csrv_specifier;

/* storage specifier of a decomposed 2-D CSR tensor (benchmarks/spmv/main.cpp:48-51) */
typedef struct lapis_csr_specifier {
  int64_t dimSizes[2];
  int64_t memSizes[3];
} lapis_csr_specifier;

/* One prebuilt library serves every LAPISModule object of a process, where the
 * reference has one generated library (and one alives list) per package: the
 * two calls are counted, and only the last lapis_finalize() frees the results
 * handed out and finalises the kernel library. */
void lapis_initialize(void);
void lapis_finalize(void);

/* ---- operands that stay on the device between calls -----------------------
 * The role of LAPIS::DualView (LAPISSupport.hpp:136-426), which lets a C++
 * caller of a generated module keep operands resident across calls
 * (benchmarks/spmv/main.cpp:42-56), offered through the C ABI: a host buffer
 * the caller owns paired with a device copy, with the DualView's lazy
 * modified_host / modified_device flags.  The py_<func> entry points above
 * keep the reference's copy-per-call behaviour; these are opt-in. */
typedef struct lapis_dualview_f64 lapis_dualview_f64;
/* Pairs `n` doubles at `host` (borrowed: they must outlive the view) with a
 * device allocation; the view starts out modified on the host
 * (the host-view constructor, LAPISSupport.hpp:214-226). */
lapis_dualview_f64 *lapis_dualview_f64_create(double *host, int64_t n);
void lapis_dualview_f64_modify_host(lapis_dualview_f64 *v);   /* modifyHost()  :229 */
void lapis_dualview_f64_modify_device(lapis_dualview_f64 *v); /* modifyDevice():234 */
void lapis_dualview_f64_sync_host(lapis_dualview_f64 *v);     /* syncHost()    :251: copies back only if modified on the device */
void lapis_dualview_f64_sync_device(lapis_dualview_f64 *v);   /* syncDevice()  :271: uploads only if modified on the host */
void lapis_dualview_f64_destroy(lapis_dualview_f64 *v);
/* the same for floats (LAPIS::DualView is a template over the element type, LAPISSupport.hpp:136) */
typedef struct lapis_dualview_f32 lapis_dualview_f32;
lapis_dualview_f32 *lapis_dualview_f32_create(float *host, int64_t n);
void lapis_dualview_f32_modify_host(lapis_dualview_f32 *v);
void lapis_dualview_f32_modify_device(lapis_dualview_f32 *v);
void lapis_dualview_f32_sync_host(lapis_dualview_f32 *v);
void lapis_dualview_f32_sync_device(lapis_dualview_f32 *v);
void lapis_dualview_f32_destroy(lapis_dualview_f32 *v);

/* A CSR matrix uploaded once: device copies of positions, coordinates and
 * values, its plan (row statistics -> kernel) and, where the library
 * recommends it, the column-blocked copy (lapis_hip_csr_plan_analyze). */
typedef struct lapis_resident_csr lapis_resident_csr;
lapis_resident_csr *lapis_resident_csr_create(lapis_memref_1d_i32 *pos, lapis_memref_1d_i32 *crd,
                                              lapis_memref_1d_f64 *val, const lapis_csr_specifier *spec);
/* new values in the same sparsity pattern (same length and order as at creation) */
void lapis_resident_csr_update_values(lapis_resident_csr *A, lapis_memref_1d_f64 *val);
/* func @spmv on resident operands: y += A*x.  x and y are brought to the device
 * if (and only if) they are marked modified on the host, y is left marked
 * modified on the device; nothing is copied back and the call does not wait
 * for the kernel -- lapis_dualview_f64_sync_host(y) does both. */
void lapis_resident_csr_spmv(lapis_resident_csr *A, lapis_dualview_f64 *x, lapis_dualview_f64 *y);
/* func @spmm on resident operands: C += A*B, B (columns x k) and C (rows x k) row-major
 * in their views; same copy and wait rules as lapis_resident_csr_spmv. */
void lapis_resident_csr_spmm(lapis_resident_csr *A, lapis_dualview_f64 *B, int64_t k, lapis_dualview_f64 *C);
/* func @pcg of examples/pcg_solve.py:52 on resident operands: solves A x = b from x = 0 with
 * the Jacobi preconditioner dinv (NULL: none), at most maxiter iterations, until the relative
 * residual is at most tol.  x is a view of the caller's, overwritten and left marked modified
 * on the device; *iters and *relres as the function returns them.  Waits for the solve. */
void lapis_resident_csr_pcg(lapis_resident_csr *A, lapis_dualview_f64 *b, lapis_dualview_f64 *dinv, double tol,
                            size_t maxiter, lapis_dualview_f64 *x, size_t *iters, double *relres);
void lapis_resident_csr_destroy(lapis_resident_csr *A);
/* the fp32 matrix (config 3 and the SpMM operand of config 4 are fp32) */
typedef struct lapis_resident_csr_f32 lapis_resident_csr_f32;
lapis_resident_csr_f32 *lapis_resident_csr_f32_create(lapis_memref_1d_i32 *pos, lapis_memref_1d_i32 *crd,
                                                      lapis_memref_1d_f32 *val, const lapis_csr_specifier *spec);
void lapis_resident_csr_f32_update_values(lapis_resident_csr_f32 *A, lapis_memref_1d_f32 *val);
void lapis_resident_csr_f32_spmv(lapis_resident_csr_f32 *A, lapis_dualview_f32 *x, lapis_dualview_f32 *y);
void lapis_resident_csr_f32_spmm(lapis_resident_csr_f32 *A, lapis_dualview_f32 *B, int64_t k, lapis_dualview_f32 *C);
void lapis_resident_csr_f32_destroy(lapis_resident_csr_f32 *A);

/* func @spmv(A, x, y) -> y of examples/spmv_noalloc.py:9-14 and
 * benchmarks/spmv/spmv.mlir:3-6: y += A*x, y updated in place and returned. */
void py_spmv(lapis_memref_1d_f64 **ret0, lapis_memref_1d_i32 *pos, lapis_memref_1d_i32 *crd,
             lapis_memref_1d_f64 *val, const lapis_csr_specifier *spec, lapis_memref_1d_f64 *x,
             lapis_memref_1d_f64 *y);

/* the fp32 instance of the same function (config 3 of the benchmark set) */
void py_spmv_f32(lapis_memref_1d_f32 **ret0, lapis_memref_1d_i32 *pos, lapis_memref_1d_i32 *crd,
                 lapis_memref_1d_f32 *val, const lapis_csr_specifier *spec, lapis_memref_1d_f32 *x,
                 lapis_memref_1d_f32 *y);

/* torch.mv export of examples/spmv.py:13-18,47 (entry `main` is renamed
 * lapis_main, emitter :2351-2355): y = A*x with y allocated by the module. */
void py_lapis_main(lapis_memref_1d_f64 **ret0, lapis_memref_1d_i32 *pos, lapis_memref_1d_i32 *crd,
                   lapis_memref_1d_f64 *val, const lapis_csr_specifier *spec, lapis_memref_1d_f64 *x);

/* func @pcg(A, b, dinv, tol, maxiter) -> (x, iters, relres) of examples/pcg_solve.py:52. */
void py_pcg(lapis_memref_1d_f64 **ret0, size_t *ret1, double *ret2, lapis_memref_1d_i32 *pos,
            lapis_memref_1d_i32 *crd, lapis_memref_1d_f64 *val, const lapis_csr_specifier *spec,
            lapis_memref_1d_f64 *b, lapis_memref_1d_f64 *dinv, double tol, size_t maxiter);

/* CSR x dense matmul, C += A*B with C updated in place and returned (the
 * decomposed-CSR form of spMxM, examples/spmm_dcsr_opdsl.py:73-110). */
void py_spmm(lapis_memref_2d_f32 **ret0, lapis_memref_1d_i32 *pos, lapis_memref_1d_i32 *crd,
             lapis_memref_1d_f32 *val, const lapis_csr_specifier *spec, lapis_memref_2d_f32 *B,
             lapis_memref_2d_f32 *C);
void py_spmm_f64(lapis_memref_2d_f64 **ret0, lapis_memref_1d_i32 *pos, lapis_memref_1d_i32 *crd,
                 lapis_memref_1d_f64 *val, const lapis_csr_specifier *spec, lapis_memref_2d_f64 *B,
                 lapis_memref_2d_f64 *C);

/* func @pte_local_bspmm(A: ?x?x?xf32 #csrv, B: ?x?x?xf32) -> ?x?x?xf32 of examples/bspmm.py:26-52:
 * out(i, d, h) = sum_c A(i, c, h) * B(c, d, h); the result is allocated and zero-filled inside. */
void py_pte_local_bspmm(lapis_memref_3d_f32 **ret0, lapis_memref_1d_i32 *pos, lapis_memref_1d_i32 *crd,
                        lapis_memref_1d_f32 *val, const lapis_csrv_specifier *spec, lapis_memref_3d_f32 *B);

/* func @plus_norm(x, y) -> (x+y, ||x+y||) of examples/multiple_results.py:8-19. */
void py_plus_norm(lapis_memref_1d_f64 **ret0, double *ret1, lapis_memref_1d_f64 *x, lapis_memref_1d_f64 *y);

/* func @mht(A, mask, d, alpha, tol, maxiter) -> (mom1, mom2) and
 * func @normalize_mom2(mom1, mom2) -> stdev of examples/hitting_times.py:153-198. */
void py_mht(lapis_memref_1d_f64 **ret0, lapis_memref_1d_f64 **ret1, lapis_memref_1d_i32 *pos,
            lapis_memref_1d_i32 *crd, lapis_memref_1d_f64 *val, const lapis_csr_specifier *spec,
            lapis_memref_1d_f64 *mask, lapis_memref_1d_f64 *d, double alpha, double tol, size_t maxiter);
void py_normalize_mom2(lapis_memref_1d_f64 **ret0, lapis_memref_1d_f64 *mom1, lapis_memref_1d_f64 *mom2);

#ifdef __cplusplus
}
#endif
#endif /* LAPIS_MODULE_H */
