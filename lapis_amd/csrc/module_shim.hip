// The generated-module calling convention (lapis_initialize / lapis_finalize /
// py_<func> over StridedMemRefType descriptors of HOST buffers) on top of the
// gfx950 kernel library.  This file plays the role of the C++ a LAPIS module is
// emitted as: the py_ wrappers (TranslateToKokkosCpp.cpp:2541-2684), the
// host<->device mirroring of LAPIS::DualView (LAPISSupport.hpp:136-426) and the
// keep-alive list for results handed to Python (LAPISSupport.hpp:101-120).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <vector>

#include "lapis_hip.h"
#include "lapis_module.h"

namespace {

[[noreturn]] void module_abort(const char *msg) {
  // the counterpart of Kokkos::abort (LAPISSupport.hpp:76,86): no status channel exists
  fprintf(stderr, "lapis module: %s\n", msg);
  fflush(stderr);
  abort();
}

void check(int status, const char *what) {
  if (status != LAPIS_HIP_OK) {
    char buf[768];
    snprintf(buf, sizeof(buf), "%s failed: %s (%s)", what, lapis_hip_status_name(status), lapis_hip_last_error());
    module_abort(buf);
  }
}

void check_hip(hipError_t e, const char *what) {
  if (e != hipSuccess) {
    char buf[512];
    snprintf(buf, sizeof(buf), "%s failed: %s", what, hipGetErrorString(e));
    module_abort(buf);
  }
}

// Results returned to Python stay allocated until lapis_finalize().
std::mutex g_mutex;
std::vector<void *> g_alives;
int g_initialized = 0;

void *keep_alive_alloc(size_t bytes) {
  void *p = malloc(bytes ? bytes : 1);
  if (!p) module_abort("out of host memory for a result");
  std::lock_guard<std::mutex> lock(g_mutex);
  g_alives.push_back(p);
  return p;
}

// stridedMemrefToView<LayoutRight> (LAPISSupport.hpp:36-91): unit innermost stride,
// each outer stride the product of the inner extents, else abort.
template <typename M>
auto *host_data(const M *m, int rank, const char *name) {
  int64_t expected = 1;
  for (int i = rank - 1; i >= 0; --i) {
    if (m->strides[i] != expected) {
      char buf[256];
      snprintf(buf, sizeof(buf),
               "Cannot shallow-copy StridedMemRefType that is not contiguous and LayoutRight (%s)", name);
      module_abort(buf);
    }
    expected *= m->sizes[i];
  }
  return m->data + m->offset;
}

// The device half of a DualView built from a host view: allocated and filled from
// the host buffer at construction ("modified_host" then syncDevice), copied back on
// request (syncHost), freed at scope exit.
template <typename T>
struct DeviceMirror {
  T *dev = nullptr;
  T *host = nullptr;
  size_t count = 0;
  DeviceMirror() = default;
  DeviceMirror(T *h, size_t n, bool upload = true) : host(h), count(n) {
    if (n == 0) return;
    check_hip(hipMalloc(&dev, n * sizeof(T)), "hipMalloc");
    if (upload) check_hip(hipMemcpy(dev, h, n * sizeof(T), hipMemcpyHostToDevice), "host-to-device copy");
  }
  DeviceMirror(const DeviceMirror &) = delete;
  DeviceMirror &operator=(const DeviceMirror &) = delete;
  ~DeviceMirror() {
    if (dev) (void)hipFree(dev);
  }
  void sync_host() {
    if (count) check_hip(hipMemcpy(host, dev, count * sizeof(T), hipMemcpyDeviceToHost), "device-to-host copy");
  }
};

template <typename M, typename T>
void set_result_1d(M **ret, T *data, int64_t n) {
  (*ret)->basePtr = data;
  (*ret)->data = data;
  (*ret)->offset = 0;
  (*ret)->sizes[0] = n;
  (*ret)->strides[0] = 1;
}

struct CsrArgs {
  int64_t nrows, ncols, nnz;
};

CsrArgs csr_args(const lapis_memref_1d_i32 *pos, const lapis_memref_1d_i32 *crd, int64_t val_size,
                 const lapis_csr_specifier *spec) {
  CsrArgs a;
  a.nrows = spec->dimSizes[0];
  a.ncols = spec->dimSizes[1];
  if (a.nrows < 0 || a.ncols < 0) module_abort("negative dimension in the storage specifier");
  if (pos->sizes[0] < a.nrows + 1) module_abort("positions buffer shorter than rows+1");
  const int32_t *p = pos->data + pos->offset;
  a.nnz = p[a.nrows];
  if (a.nnz < 0 || crd->sizes[0] < a.nnz || val_size < a.nnz)
    module_abort("coordinates/values buffer shorter than pos[rows]");
  return a;
}

template <typename T, typename MV>
void spmv_entry(MV **ret0, lapis_memref_1d_i32 *pos, lapis_memref_1d_i32 *crd, MV *val,
                const lapis_csr_specifier *spec, MV *x, MV *y, bool allocate_y) {
  int32_t *hpos = host_data(pos, 1, "positions");
  int32_t *hcrd = host_data(crd, 1, "coordinates");
  T *hval = host_data(val, 1, "values");
  T *hx = host_data(x, 1, "x");
  const CsrArgs a = csr_args(pos, crd, val->sizes[0], spec);
  if (x->sizes[0] < a.ncols) module_abort("x is shorter than the number of columns");
  T *hy = nullptr;
  if (allocate_y) {
    // the torch.mv export allocates and zero-fills its result inside the function
    hy = static_cast<T *>(keep_alive_alloc(sizeof(T) * (size_t)a.nrows));
    memset(hy, 0, sizeof(T) * (size_t)a.nrows);
  } else {
    hy = host_data(y, 1, "y");
    if (y->sizes[0] < a.nrows) module_abort("y is shorter than the number of rows");
  }
  {
    DeviceMirror<int32_t> dpos(hpos, (size_t)a.nrows + 1), dcrd(hcrd, (size_t)a.nnz);
    DeviceMirror<T> dval(hval, (size_t)a.nnz), dx(hx, (size_t)a.ncols), dy(hy, (size_t)a.nrows);
    lapis_hip_csr_plan *plan = nullptr;
    check(lapis_hip_csr_plan_create(&plan, a.nrows, a.ncols, a.nnz, dpos.dev, dcrd.dev, (int)sizeof(T), nullptr),
          "lapis_hip_csr_plan_create");
    int rc;
    if (sizeof(T) == 8)
      rc = lapis_hip_spmv_csr_f64_i32(plan, a.nrows, a.ncols, dpos.dev, dcrd.dev, (const double *)dval.dev,
                                      (const double *)dx.dev, (double *)dy.dev, nullptr);
    else
      rc = lapis_hip_spmv_csr_f32_i32(plan, a.nrows, a.ncols, dpos.dev, dcrd.dev, (const float *)dval.dev,
                                      (const float *)dx.dev, (float *)dy.dev, nullptr);
    check(rc, "lapis_hip_spmv_csr");
    check(lapis_hip_stream_synchronize(nullptr), "stream synchronize");
    lapis_hip_csr_plan_destroy(plan);
    dy.sync_host();  // results.syncHost(): the caller's y (or the module's) now holds the result
  }
  set_result_1d(ret0, hy, a.nrows);
}

template <typename T, typename MV, typename MM>
void spmm_entry(MM **ret0, lapis_memref_1d_i32 *pos, lapis_memref_1d_i32 *crd, MV *val,
                const lapis_csr_specifier *spec, MM *B, MM *C) {
  int32_t *hpos = host_data(pos, 1, "positions");
  int32_t *hcrd = host_data(crd, 1, "coordinates");
  T *hval = host_data(val, 1, "values");
  T *hB = host_data(B, 2, "B");
  T *hC = host_data(C, 2, "C");
  const CsrArgs a = csr_args(pos, crd, val->sizes[0], spec);
  const int64_t k = C->sizes[1];
  if (B->sizes[0] < a.ncols || B->sizes[1] != k || C->sizes[0] < a.nrows)
    module_abort("SpMM operand shapes do not agree");
  {
    DeviceMirror<int32_t> dpos(hpos, (size_t)a.nrows + 1), dcrd(hcrd, (size_t)a.nnz);
    DeviceMirror<T> dval(hval, (size_t)a.nnz), dB(hB, (size_t)(a.ncols * k)), dC(hC, (size_t)(a.nrows * k));
    // the plan checks the structure (a bad coordinate must not reach the kernel) and its statistics pick the kernel
    lapis_hip_csr_plan *plan = nullptr;
    check(lapis_hip_csr_plan_create(&plan, a.nrows, a.ncols, a.nnz, dpos.dev, dcrd.dev, (int)sizeof(T), nullptr),
          "lapis_hip_csr_plan_create");
    int rc;
    if (sizeof(T) == 8)
      rc = lapis_hip_spmm_csr_f64_i32_plan(plan, a.nrows, a.ncols, k, dpos.dev, dcrd.dev, (const double *)dval.dev,
                                           (const double *)dB.dev, k, (double *)dC.dev, k, nullptr);
    else
      rc = lapis_hip_spmm_csr_f32_i32_plan(plan, a.nrows, a.ncols, k, dpos.dev, dcrd.dev, (const float *)dval.dev,
                                           (const float *)dB.dev, k, (float *)dC.dev, k, nullptr);
    check(rc, "lapis_hip_spmm_csr");
    check(lapis_hip_stream_synchronize(nullptr), "stream synchronize");
    lapis_hip_csr_plan_destroy(plan);
    dC.sync_host();
  }
  (*ret0)->basePtr = hC;
  (*ret0)->data = hC;
  (*ret0)->offset = 0;
  (*ret0)->sizes[0] = C->sizes[0];
  (*ret0)->sizes[1] = k;
  (*ret0)->strides[0] = k;
  (*ret0)->strides[1] = 1;
}

}  // namespace

extern "C" void lapis_initialize(void) {
  std::lock_guard<std::mutex> lock(g_mutex);
  // `if (!Kokkos::is_initialized())`: only the first call initialises; every call is counted, because
  // this one library stands in for all the generated packages of a process
  if (g_initialized++ > 0) return;
  check(lapis_hip_init(), "lapis_hip_init");
}

extern "C" void lapis_finalize(void) {
  std::lock_guard<std::mutex> lock(g_mutex);
  if (g_initialized == 0) return;
  if (--g_initialized > 0) return;  // another module object is alive: its results must stay valid
  for (void *p : g_alives) free(p);  // LAPIS::alives.clear()
  g_alives.clear();
  lapis_hip_finalize();
}

// ---- resident operands ----------------------------------------------------------------------------

template <typename T>
struct DualViewOf {
  T *host = nullptr;
  T *dev = nullptr;
  int64_t n = 0;
  bool modified_host = false;
  bool modified_device = false;
};
struct lapis_dualview_f64 : DualViewOf<double> {};
struct lapis_dualview_f32 : DualViewOf<float> {};

template <typename T>
struct ResidentCsrOf {
  int64_t nrows = 0, ncols = 0, nnz = 0;
  int32_t *pos = nullptr, *crd = nullptr;
  T *val = nullptr;
  lapis_hip_csr_plan *plan = nullptr;
};
struct lapis_resident_csr : ResidentCsrOf<double> {};
struct lapis_resident_csr_f32 : ResidentCsrOf<float> {};

namespace {
template <typename V, typename T>
V *dualview_create(T *host, int64_t n) {
  if (n < 0 || (n > 0 && !host)) module_abort("dualview: null host buffer or negative length");
  V *v = new V();
  v->host = host;
  v->n = n;
  if (n > 0) check_hip(hipMalloc(&v->dev, sizeof(T) * (size_t)n), "hipMalloc");
  v->modified_host = true;
  return v;
}
template <typename T>
void dualview_sync_host(DualViewOf<T> *v) {
  if (!v->modified_device) return;
  // hipMemcpy on the null stream waits for the kernels queued there before it copies
  if (v->n > 0) check_hip(hipMemcpy(v->host, v->dev, sizeof(T) * (size_t)v->n, hipMemcpyDeviceToHost), "device-to-host copy");
  v->modified_device = false;
}
template <typename T>
void dualview_sync_device(DualViewOf<T> *v) {
  if (!v->modified_host) return;
  if (v->n > 0) check_hip(hipMemcpy(v->dev, v->host, sizeof(T) * (size_t)v->n, hipMemcpyHostToDevice), "host-to-device copy");
  v->modified_host = false;
}
template <typename T>
void dualview_destroy(DualViewOf<T> *v) {
  if (v && v->dev) (void)hipFree(v->dev);
}

template <typename R, typename T, typename ValMemref>
R *resident_create(lapis_memref_1d_i32 *pos, lapis_memref_1d_i32 *crd, ValMemref *val, const lapis_csr_specifier *spec) {
  int32_t *hpos = host_data(pos, 1, "positions");
  int32_t *hcrd = host_data(crd, 1, "coordinates");
  T *hval = host_data(val, 1, "values");
  const CsrArgs a = csr_args(pos, crd, val->sizes[0], spec);
  R *A = new R();
  A->nrows = a.nrows;
  A->ncols = a.ncols;
  A->nnz = a.nnz;
  check_hip(hipMalloc(&A->pos, sizeof(int32_t) * ((size_t)a.nrows + 1)), "hipMalloc");
  check_hip(hipMalloc(&A->crd, sizeof(int32_t) * (size_t)std::max<int64_t>(a.nnz, 1)), "hipMalloc");
  check_hip(hipMalloc(&A->val, sizeof(T) * (size_t)std::max<int64_t>(a.nnz, 1)), "hipMalloc");
  check_hip(hipMemcpy(A->pos, hpos, sizeof(int32_t) * ((size_t)a.nrows + 1), hipMemcpyHostToDevice), "host-to-device copy");
  check_hip(hipMemcpy(A->crd, hcrd, sizeof(int32_t) * (size_t)a.nnz, hipMemcpyHostToDevice), "host-to-device copy");
  check_hip(hipMemcpy(A->val, hval, sizeof(T) * (size_t)a.nnz, hipMemcpyHostToDevice), "host-to-device copy");
  check(lapis_hip_csr_plan_create(&A->plan, a.nrows, a.ncols, a.nnz, A->pos, A->crd, (int)sizeof(T), nullptr),
        "lapis_hip_csr_plan_create");
  // a resident matrix is there to be multiplied many times: let the library build the copy it recommends
  check(lapis_hip_csr_plan_analyze(A->plan, A->crd, A->val, (int)sizeof(T), nullptr), "lapis_hip_csr_plan_analyze");
  return A;
}
template <typename T, typename ValMemref>
void resident_update_values(ResidentCsrOf<T> *A, ValMemref *val) {
  T *hval = host_data(val, 1, "values");
  if (val->sizes[0] < A->nnz) module_abort("update_values: fewer values than the matrix has non-zeros");
  check_hip(hipMemcpy(A->val, hval, sizeof(T) * (size_t)A->nnz, hipMemcpyHostToDevice), "host-to-device copy");
  check(lapis_hip_csr_plan_update_values(A->plan, A->val, (int)sizeof(T), nullptr), "lapis_hip_csr_plan_update_values");
}
template <typename T>
void resident_spmv(ResidentCsrOf<T> *A, DualViewOf<T> *x, DualViewOf<T> *y) {
  if (x->n < A->ncols) module_abort("x is shorter than the number of columns");
  if (y->n < A->nrows) module_abort("y is shorter than the number of rows");
  if (x == y) module_abort("x and y must be different views");
  dualview_sync_device(x);
  dualview_sync_device(y);
  if constexpr (sizeof(T) == 8)
    check(lapis_hip_spmv_csr_f64_i32(A->plan, A->nrows, A->ncols, A->pos, A->crd, A->val, x->dev, y->dev, nullptr),
          "lapis_hip_spmv_csr_f64_i32");
  else
    check(lapis_hip_spmv_csr_f32_i32(A->plan, A->nrows, A->ncols, A->pos, A->crd, A->val, x->dev, y->dev, nullptr),
          "lapis_hip_spmv_csr_f32_i32");
  y->modified_device = true;
}
// C += A*B with B (ncols x k) and C (nrows x k) row-major in their views
template <typename T>
void resident_spmm(ResidentCsrOf<T> *A, DualViewOf<T> *B, int64_t k, DualViewOf<T> *C) {
  if (k < 0 || B->n < A->ncols * k) module_abort("B is smaller than columns x k");
  if (C->n < A->nrows * k) module_abort("C is smaller than rows x k");
  if (B == C) module_abort("B and C must be different views");
  dualview_sync_device(B);
  dualview_sync_device(C);
  if constexpr (sizeof(T) == 8)
    check(lapis_hip_spmm_csr_f64_i32_plan(A->plan, A->nrows, A->ncols, k, A->pos, A->crd, A->val, B->dev, k, C->dev, k,
                                          nullptr),
          "lapis_hip_spmm_csr_f64_i32_plan");
  else
    check(lapis_hip_spmm_csr_f32_i32_plan(A->plan, A->nrows, A->ncols, k, A->pos, A->crd, A->val, B->dev, k, C->dev, k,
                                          nullptr),
          "lapis_hip_spmm_csr_f32_i32_plan");
  C->modified_device = true;
}
template <typename T>
void resident_destroy(ResidentCsrOf<T> *A) {
  if (!A) return;
  lapis_hip_csr_plan_destroy(A->plan);
  if (A->pos) (void)hipFree(A->pos);
  if (A->crd) (void)hipFree(A->crd);
  if (A->val) (void)hipFree(A->val);
}
}  // namespace

extern "C" lapis_dualview_f64 *lapis_dualview_f64_create(double *host, int64_t n) {
  return dualview_create<lapis_dualview_f64>(host, n);
}
extern "C" void lapis_dualview_f64_modify_host(lapis_dualview_f64 *v) { v->modified_host = true; }
extern "C" void lapis_dualview_f64_modify_device(lapis_dualview_f64 *v) { v->modified_device = true; }
extern "C" void lapis_dualview_f64_sync_host(lapis_dualview_f64 *v) { dualview_sync_host<double>(v); }
extern "C" void lapis_dualview_f64_sync_device(lapis_dualview_f64 *v) { dualview_sync_device<double>(v); }
extern "C" void lapis_dualview_f64_destroy(lapis_dualview_f64 *v) {
  dualview_destroy<double>(v);
  delete v;
}
extern "C" lapis_dualview_f32 *lapis_dualview_f32_create(float *host, int64_t n) {
  return dualview_create<lapis_dualview_f32>(host, n);
}
extern "C" void lapis_dualview_f32_modify_host(lapis_dualview_f32 *v) { v->modified_host = true; }
extern "C" void lapis_dualview_f32_modify_device(lapis_dualview_f32 *v) { v->modified_device = true; }
extern "C" void lapis_dualview_f32_sync_host(lapis_dualview_f32 *v) { dualview_sync_host<float>(v); }
extern "C" void lapis_dualview_f32_sync_device(lapis_dualview_f32 *v) { dualview_sync_device<float>(v); }
extern "C" void lapis_dualview_f32_destroy(lapis_dualview_f32 *v) {
  dualview_destroy<float>(v);
  delete v;
}

extern "C" lapis_resident_csr *lapis_resident_csr_create(lapis_memref_1d_i32 *pos, lapis_memref_1d_i32 *crd,
                                                         lapis_memref_1d_f64 *val, const lapis_csr_specifier *spec) {
  return resident_create<lapis_resident_csr, double>(pos, crd, val, spec);
}
extern "C" void lapis_resident_csr_update_values(lapis_resident_csr *A, lapis_memref_1d_f64 *val) {
  resident_update_values<double>(A, val);
}
extern "C" void lapis_resident_csr_spmv(lapis_resident_csr *A, lapis_dualview_f64 *x, lapis_dualview_f64 *y) {
  resident_spmv<double>(A, x, y);
}
extern "C" void lapis_resident_csr_spmm(lapis_resident_csr *A, lapis_dualview_f64 *B, int64_t k, lapis_dualview_f64 *C) {
  resident_spmm<double>(A, B, k, C);
}
// func @pcg on resident operands: x (allocated by the caller, overwritten) = the solution
extern "C" void lapis_resident_csr_pcg(lapis_resident_csr *A, lapis_dualview_f64 *b, lapis_dualview_f64 *dinv, double tol,
                                       size_t maxiter, lapis_dualview_f64 *x, size_t *iters, double *relres) {
  const int64_t n = A->nrows;
  if (A->ncols != n) module_abort("pcg: A must be square");
  if (b->n < n || x->n < n || (dinv && dinv->n < n)) module_abort("pcg: b, dinv and x need n elements");
  if (x == b || x == dinv) module_abort("pcg: x must be a view of its own");
  dualview_sync_device<double>(b);
  if (dinv) dualview_sync_device<double>(dinv);
  uint64_t it = 0;
  double rr = 0.0;
  check(lapis_hip_pcg_f64_i32(A->plan, n, A->pos, A->crd, A->val, b->dev, dinv ? dinv->dev : nullptr, tol, (uint64_t)maxiter,
                              x->dev, &it, &rr, nullptr, nullptr),
        "lapis_hip_pcg_f64_i32");
  x->modified_device = true;
  x->modified_host = false;
  if (iters) *iters = (size_t)it;
  if (relres) *relres = rr;
}
extern "C" void lapis_resident_csr_destroy(lapis_resident_csr *A) {
  resident_destroy<double>(A);
  delete A;
}

extern "C" lapis_resident_csr_f32 *lapis_resident_csr_f32_create(lapis_memref_1d_i32 *pos, lapis_memref_1d_i32 *crd,
                                                                 lapis_memref_1d_f32 *val, const lapis_csr_specifier *spec) {
  return resident_create<lapis_resident_csr_f32, float>(pos, crd, val, spec);
}
extern "C" void lapis_resident_csr_f32_update_values(lapis_resident_csr_f32 *A, lapis_memref_1d_f32 *val) {
  resident_update_values<float>(A, val);
}
extern "C" void lapis_resident_csr_f32_spmv(lapis_resident_csr_f32 *A, lapis_dualview_f32 *x, lapis_dualview_f32 *y) {
  resident_spmv<float>(A, x, y);
}
extern "C" void lapis_resident_csr_f32_spmm(lapis_resident_csr_f32 *A, lapis_dualview_f32 *B, int64_t k,
                                            lapis_dualview_f32 *C) {
  resident_spmm<float>(A, B, k, C);
}
extern "C" void lapis_resident_csr_f32_destroy(lapis_resident_csr_f32 *A) {
  resident_destroy<float>(A);
  delete A;
}

extern "C" void py_spmv(lapis_memref_1d_f64 **ret0, lapis_memref_1d_i32 *pos, lapis_memref_1d_i32 *crd,
                        lapis_memref_1d_f64 *val, const lapis_csr_specifier *spec, lapis_memref_1d_f64 *x,
                        lapis_memref_1d_f64 *y) {
  spmv_entry<double>(ret0, pos, crd, val, spec, x, y, false);
}

extern "C" void py_spmv_f32(lapis_memref_1d_f32 **ret0, lapis_memref_1d_i32 *pos, lapis_memref_1d_i32 *crd,
                            lapis_memref_1d_f32 *val, const lapis_csr_specifier *spec, lapis_memref_1d_f32 *x,
                            lapis_memref_1d_f32 *y) {
  spmv_entry<float>(ret0, pos, crd, val, spec, x, y, false);
}

extern "C" void py_lapis_main(lapis_memref_1d_f64 **ret0, lapis_memref_1d_i32 *pos, lapis_memref_1d_i32 *crd,
                              lapis_memref_1d_f64 *val, const lapis_csr_specifier *spec, lapis_memref_1d_f64 *x) {
  spmv_entry<double>(ret0, pos, crd, val, spec, x, (lapis_memref_1d_f64 *)nullptr, true);
}

extern "C" void py_pcg(lapis_memref_1d_f64 **ret0, size_t *ret1, double *ret2, lapis_memref_1d_i32 *pos,
                       lapis_memref_1d_i32 *crd, lapis_memref_1d_f64 *val, const lapis_csr_specifier *spec,
                       lapis_memref_1d_f64 *b, lapis_memref_1d_f64 *dinv, double tol, size_t maxiter) {
  int32_t *hpos = host_data(pos, 1, "positions");
  int32_t *hcrd = host_data(crd, 1, "coordinates");
  double *hval = host_data(val, 1, "values");
  double *hb = host_data(b, 1, "b");
  double *hdinv = host_data(dinv, 1, "dinv");
  const CsrArgs a = csr_args(pos, crd, val->sizes[0], spec);
  const int64_t n = b->sizes[0];  // %n = tensor.dim %b (examples/pcg_solve.py:55)
  if (a.nrows != n || a.ncols != n || dinv->sizes[0] < n) module_abort("pcg: A must be n x n and dinv of length n");
  double *hx = static_cast<double *>(keep_alive_alloc(sizeof(double) * (size_t)n));
  uint64_t iters = 0;
  double relres = 0.0;
  {
    DeviceMirror<int32_t> dpos(hpos, (size_t)n + 1), dcrd(hcrd, (size_t)a.nnz);
    DeviceMirror<double> dval(hval, (size_t)a.nnz), db(hb, (size_t)n), ddinv(hdinv, (size_t)n);
    DeviceMirror<double> dx(hx, (size_t)n, false);
    lapis_hip_csr_plan *plan = nullptr;
    check(lapis_hip_csr_plan_create(&plan, n, n, a.nnz, dpos.dev, dcrd.dev, 8, nullptr), "lapis_hip_csr_plan_create");
    // enough iterations for the column-blocked copy to pay back where the library recommends one
    if (maxiter >= 64) check(lapis_hip_csr_plan_analyze(plan, dcrd.dev, dval.dev, 8, nullptr), "lapis_hip_csr_plan_analyze");
    check(lapis_hip_pcg_f64_i32(plan, n, dpos.dev, dcrd.dev, dval.dev, db.dev, ddinv.dev, tol, (uint64_t)maxiter,
                                dx.dev, &iters, &relres, nullptr, nullptr),
          "lapis_hip_pcg_f64_i32");
    lapis_hip_csr_plan_destroy(plan);
    dx.sync_host();
  }
  set_result_1d(ret0, hx, n);
  *ret1 = (size_t)iters;
  *ret2 = relres;
}

extern "C" void py_spmm(lapis_memref_2d_f32 **ret0, lapis_memref_1d_i32 *pos, lapis_memref_1d_i32 *crd,
                        lapis_memref_1d_f32 *val, const lapis_csr_specifier *spec, lapis_memref_2d_f32 *B,
                        lapis_memref_2d_f32 *C) {
  spmm_entry<float>(ret0, pos, crd, val, spec, B, C);
}

extern "C" void py_spmm_f64(lapis_memref_2d_f64 **ret0, lapis_memref_1d_i32 *pos, lapis_memref_1d_i32 *crd,
                            lapis_memref_1d_f64 *val, const lapis_csr_specifier *spec, lapis_memref_2d_f64 *B,
                            lapis_memref_2d_f64 *C) {
  spmm_entry<double>(ret0, pos, crd, val, spec, B, C);
}

extern "C" void py_pte_local_bspmm(lapis_memref_3d_f32 **ret0, lapis_memref_1d_i32 *pos, lapis_memref_1d_i32 *crd,
                                   lapis_memref_1d_f32 *val, const lapis_csrv_specifier *spec,
                                   lapis_memref_3d_f32 *B) {
  int32_t *hpos = host_data(pos, 1, "positions");
  int32_t *hcrd = host_data(crd, 1, "coordinates");
  float *hval = host_data(val, 1, "values");
  float *hB = host_data(B, 3, "B");
  const int64_t n1 = spec->dimSizes[0], n2 = spec->dimSizes[1], nh = spec->dimSizes[2];
  const int64_t nnz = spec->memSizes[1];
  const int64_t dh = B->sizes[1];
  if (n1 < 0 || n2 < 0 || nh < 0 || nnz < 0 || spec->memSizes[0] != n1 + 1 || spec->memSizes[2] != nnz * nh ||
      pos->sizes[0] < n1 + 1 || crd->sizes[0] < nnz || val->sizes[0] < nnz * nh)
    module_abort("bspmm: storage specifier and buffers do not agree");
  if (B->sizes[0] < n2 || B->sizes[2] != nh) module_abort("bspmm: operand shapes do not agree");
  const size_t out_count = (size_t)(n1 * dh * nh);
  float *hout = static_cast<float *>(keep_alive_alloc(sizeof(float) * out_count));
  memset(hout, 0, sizeof(float) * out_count);  // linalg.fill of the result (examples/bspmm.py:40-42)
  if (out_count > 0) {
    DeviceMirror<int32_t> dpos(hpos, (size_t)n1 + 1), dcrd(hcrd, (size_t)nnz);
    DeviceMirror<float> dval(hval, (size_t)(nnz * nh)), dB(hB, (size_t)(n2 * dh * nh)), dout(hout, out_count);
    // the plan is built only for its structure check: a bad coordinate must not reach the kernel
    lapis_hip_csr_plan *plan = nullptr;
    check(lapis_hip_csr_plan_create(&plan, n1, n2, nnz, dpos.dev, dcrd.dev, 4, nullptr), "lapis_hip_csr_plan_create");
    lapis_hip_csr_plan_destroy(plan);
    check(lapis_hip_bspmm_csrv_f32_i32(n1, n2, dh, nh, dpos.dev, dcrd.dev, dval.dev, dB.dev, dout.dev, nullptr),
          "lapis_hip_bspmm_csrv_f32_i32");
    check(lapis_hip_stream_synchronize(nullptr), "stream synchronize");
    dout.sync_host();
  }
  (*ret0)->basePtr = hout;
  (*ret0)->data = hout;
  (*ret0)->offset = 0;
  (*ret0)->sizes[0] = n1;
  (*ret0)->sizes[1] = dh;
  (*ret0)->sizes[2] = nh;
  (*ret0)->strides[0] = dh * nh;
  (*ret0)->strides[1] = nh;
  (*ret0)->strides[2] = 1;
}

extern "C" void py_plus_norm(lapis_memref_1d_f64 **ret0, double *ret1, lapis_memref_1d_f64 *x,
                             lapis_memref_1d_f64 *y) {
  double *hx = host_data(x, 1, "x");
  double *hy = host_data(y, 1, "y");
  const int64_t n = y->sizes[0];  // %n = tensor.dim %y (examples/multiple_results.py:10)
  if (x->sizes[0] < n) module_abort("plus_norm: x shorter than y");
  double *hout = static_cast<double *>(keep_alive_alloc(sizeof(double) * (size_t)n));
  double sum = 0.0;
  {
    DeviceMirror<double> dx(hx, (size_t)n), dy(hy, (size_t)n), dout(hout, (size_t)n, false);
    double *dsum = nullptr;
    check_hip(hipMalloc(&dsum, sizeof(double)), "hipMalloc");
    check(lapis_hip_axpby_f64(n, 1.0, dx.dev, 1.0, dy.dev, dout.dev, nullptr), "lapis_hip_axpby_f64");
    check(lapis_hip_dot_f64(n, dout.dev, dout.dev, 0.0, dsum, nullptr), "lapis_hip_dot_f64");
    check_hip(hipMemcpy(&sum, dsum, sizeof(double), hipMemcpyDeviceToHost), "device-to-host copy");
    (void)hipFree(dsum);
    dout.sync_host();
  }
  set_result_1d(ret0, hout, n);
  *ret1 = sqrt(sum);
}

extern "C" void py_mht(lapis_memref_1d_f64 **ret0, lapis_memref_1d_f64 **ret1, lapis_memref_1d_i32 *pos,
                       lapis_memref_1d_i32 *crd, lapis_memref_1d_f64 *val, const lapis_csr_specifier *spec,
                       lapis_memref_1d_f64 *mask, lapis_memref_1d_f64 *d, double alpha, double tol, size_t maxiter) {
  int32_t *hpos = host_data(pos, 1, "positions");
  int32_t *hcrd = host_data(crd, 1, "coordinates");
  double *hval = host_data(val, 1, "values");
  double *hmask = host_data(mask, 1, "mask");
  double *hd = host_data(d, 1, "d");
  const CsrArgs a = csr_args(pos, crd, val->sizes[0], spec);
  const int64_t n = d->sizes[0];  // %n = tensor.dim %d (examples/hitting_times.py:157)
  if (a.nrows != n || a.ncols != n || mask->sizes[0] < n) module_abort("mht: A must be n x n and mask of length n");
  double *h1 = static_cast<double *>(keep_alive_alloc(sizeof(double) * (size_t)n));
  double *h2 = static_cast<double *>(keep_alive_alloc(sizeof(double) * (size_t)n));
  {
    DeviceMirror<int32_t> dpos(hpos, (size_t)n + 1), dcrd(hcrd, (size_t)a.nnz);
    DeviceMirror<double> dval(hval, (size_t)a.nnz), dmask(hmask, (size_t)n), dd(hd, (size_t)n);
    DeviceMirror<double> d1(h1, (size_t)n, false), d2(h2, (size_t)n, false);
    lapis_hip_csr_plan *plan = nullptr;
    check(lapis_hip_csr_plan_create(&plan, n, n, a.nnz, dpos.dev, dcrd.dev, 8, nullptr), "lapis_hip_csr_plan_create");
    // two solves of up to maxiter iterations each; mht refreshes the copy's values after it has scaled the matrix
    if (maxiter >= 32) check(lapis_hip_csr_plan_analyze(plan, dcrd.dev, dval.dev, 8, nullptr), "lapis_hip_csr_plan_analyze");
    check(lapis_hip_mht_f64_i32(plan, n, a.nnz, dpos.dev, dcrd.dev, dval.dev, dmask.dev, dd.dev, alpha, tol,
                                (uint64_t)maxiter, d1.dev, d2.dev, nullptr),
          "lapis_hip_mht_f64_i32");
    lapis_hip_csr_plan_destroy(plan);
    d1.sync_host();
    d2.sync_host();
    // the scaled values stay on the device: they are no result of the function, and a
    // DualView built from host memory is not copied back unless it is one
  }
  set_result_1d(ret0, h1, n);
  set_result_1d(ret1, h2, n);
}

extern "C" void py_normalize_mom2(lapis_memref_1d_f64 **ret0, lapis_memref_1d_f64 *mom1, lapis_memref_1d_f64 *mom2) {
  double *h1 = host_data(mom1, 1, "mom1");
  double *h2 = host_data(mom2, 1, "mom2");
  const int64_t n = mom1->sizes[0];
  if (mom2->sizes[0] < n) module_abort("normalize_mom2: mom2 shorter than mom1");
  double *hout = static_cast<double *>(keep_alive_alloc(sizeof(double) * (size_t)n));
  {
    DeviceMirror<double> d1(h1, (size_t)n), d2(h2, (size_t)n), dout(hout, (size_t)n, false);
    check(lapis_hip_normalize_mom2_f64(n, d1.dev, d2.dev, dout.dev, nullptr), "lapis_hip_normalize_mom2_f64");
    check(lapis_hip_stream_synchronize(nullptr), "stream synchronize");
    dout.sync_host();
  }
  set_result_1d(ret0, hout, n);
}
