// SpMV benchmark driver over a MatrixMarket file, the counterpart of the
// reference's benchmarks/spmv/main.cpp: read the matrix, keep it resident on the
// device, one warm-up call, then `trials` calls each followed by a fence, print the
// mean time.  Usage: lapis_spmv_bench matrix.mtx [trials=1000] [kernel] [--check] [--dump-y FILE]
//   kernel: auto (default) | reference | subwarpN | rowblock | nnzsplit | colblock
//   auto lets the library decide (plan statistics, and with 64 trials or more
//   lapis_hip_csr_plan_analyze, which builds the column-blocked copy where it pays).
//   --check       run one product with x = 1, 2, 3, ... and y = 0 before the timing and print
//                 sum(y) and four entries of y with 17 digits (the reference driver prints
//                 nothing that can be verified; this is what the tests compare)
//   --dump-y FILE also write that y as raw doubles
// Instead of a file, `gen:laplace3d:N` builds the 7-point Laplacian on an N^3 grid
// (N = 100 is the size of the reference's Laplace3D_100).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <sstream>
#include <string>
#include <vector>

#include "lapis_hip.h"

namespace {

struct Csr {
  int64_t nrows = 0, ncols = 0;
  std::vector<int32_t> pos, crd;
  std::vector<double> val;
};

bool read_matrix_market(const std::string &path, Csr &A, std::string &err) {
  std::ifstream in(path);
  if (!in) {
    err = "cannot open " + path;
    return false;
  }
  std::string line;
  if (!std::getline(in, line) || line.rfind("%%MatrixMarket", 0) != 0) {
    err = "not a MatrixMarket file";
    return false;
  }
  std::string banner, object, format, field, symmetry;
  {
    std::istringstream hs(line);
    hs >> banner >> object >> format >> field >> symmetry;
  }
  auto lower = [](std::string s) {
    std::transform(s.begin(), s.end(), s.begin(), ::tolower);
    return s;
  };
  format = lower(format);
  field = lower(field);
  symmetry = lower(symmetry);
  if (lower(object) != "matrix" || format != "coordinate") {
    err = "only 'matrix coordinate' files are supported";
    return false;
  }
  if (field != "real" && field != "integer" && field != "pattern" && field != "double") {
    err = "unsupported field type " + field;
    return false;
  }
  const bool pattern = field == "pattern";
  const bool sym = symmetry == "symmetric", skew = symmetry == "skew-symmetric";
  if (!sym && !skew && symmetry != "general") {
    err = "unsupported symmetry " + symmetry;
    return false;
  }
  while (std::getline(in, line))
    if (!line.empty() && line[0] != '%') break;
  long long m = 0, n = 0, entries = 0;
  if (sscanf(line.c_str(), "%lld %lld %lld", &m, &n, &entries) != 3 || m < 0 || n < 0 || entries < 0) {
    err = "bad size line";
    return false;
  }
  if (m > INT32_MAX - 64 || n > INT32_MAX || entries > INT32_MAX) {
    err = "sizes exceed the int32 index range";
    return false;
  }
  // A header may claim anything: an entry takes at least four characters ("1 1\n"), so a
  // count the rest of the file cannot hold is refused before memory is set aside for it.
  {
    const std::streamoff here = in.tellg();
    in.seekg(0, std::ios::end);
    const std::streamoff end = in.tellg();
    in.seekg(here);
    if (here < 0 || end < here || entries > (end - here) / 4 + 1) {
      err = "file ends before all entries were read";
      return false;
    }
  }
  struct Entry {
    int32_t r, c;
    double v;
  };
  std::vector<Entry> coo;
  coo.reserve((size_t)entries * ((sym || skew) ? 2 : 1));
  for (long long k = 0; k < entries; ++k) {
    long long r, c;
    double v = 1.0;
    if (!(in >> r >> c)) {
      err = "file ends before all entries were read";
      return false;
    }
    if (!pattern && !(in >> v)) {
      err = "missing value";
      return false;
    }
    if (r < 1 || r > m || c < 1 || c > n) {
      err = "entry outside the matrix";
      return false;
    }
    coo.push_back({(int32_t)(r - 1), (int32_t)(c - 1), v});
    if ((sym || skew) && r != c) coo.push_back({(int32_t)(c - 1), (int32_t)(r - 1), skew ? -v : v});
  }
  if (coo.size() > (size_t)INT32_MAX) {
    err = "more non-zeros than int32 positions can address";
    return false;
  }
  std::sort(coo.begin(), coo.end(), [](const Entry &a, const Entry &b) { return a.r != b.r ? a.r < b.r : a.c < b.c; });
  A.nrows = m;
  A.ncols = n;
  A.pos.assign((size_t)m + 1, 0);
  A.crd.resize(coo.size());
  A.val.resize(coo.size());
  for (size_t k = 0; k < coo.size(); ++k) {
    A.pos[(size_t)coo[k].r + 1]++;
    A.crd[k] = coo[k].c;
    A.val[k] = coo[k].v;
  }
  for (int64_t i = 0; i < m; ++i) A.pos[(size_t)i + 1] += A.pos[(size_t)i];
  return true;
}

// 7-point Laplacian on an n^3 grid, x fastest, diagonal 6 and off-diagonals -1.
void laplace3d(int n, Csr &A) {
  const int64_t N = (int64_t)n * n * n;
  A.nrows = A.ncols = N;
  A.pos.assign((size_t)N + 1, 0);
  A.crd.clear();
  A.val.clear();
  A.crd.reserve((size_t)N * 7);
  A.val.reserve((size_t)N * 7);
  for (int64_t i = 0; i < N; ++i) {
    const int ix = (int)(i % n), iy = (int)((i / n) % n), iz = (int)(i / ((int64_t)n * n));
    auto put = [&](int64_t c, double v) {
      A.crd.push_back((int32_t)c);
      A.val.push_back(v);
    };
    if (iz > 0) put(i - (int64_t)n * n, -1);
    if (iy > 0) put(i - n, -1);
    if (ix > 0) put(i - 1, -1);
    put(i, 6);
    if (ix < n - 1) put(i + 1, -1);
    if (iy < n - 1) put(i + n, -1);
    if (iz < n - 1) put(i + (int64_t)n * n, -1);
    A.pos[(size_t)i + 1] = (int32_t)A.crd.size();
  }
}

#define CHECK_HIP(expr)                                                              \
  do {                                                                               \
    hipError_t e_ = (expr);                                                          \
    if (e_ != hipSuccess) {                                                          \
      fprintf(stderr, "%s failed: %s\n", #expr, hipGetErrorString(e_));              \
      return 2;                                                                      \
    }                                                                                \
  } while (0)
#define CHECK_LAPIS(expr)                                                            \
  do {                                                                               \
    int s_ = (expr);                                                                 \
    if (s_ != LAPIS_HIP_OK) {                                                        \
      fprintf(stderr, "%s failed: %s: %s\n", #expr, lapis_hip_status_name(s_), lapis_hip_last_error()); \
      return 2;                                                                      \
    }                                                                                \
  } while (0)

}  // namespace

int main(int argc, const char **argv) {
  std::vector<std::string> positional;
  bool check = false, parse_only = false;
  std::string dump_path;
  for (int i = 1; i < argc; ++i) {
    const std::string a = argv[i];
    if (a == "--check") check = true;
    else if (a == "--parse-only") parse_only = true;
    else if (a == "--dump-y" && i + 1 < argc) dump_path = argv[++i];
    else if (a.rfind("--", 0) == 0) {
      std::cerr << "unknown option " << a << "\n";
      return 1;
    } else positional.push_back(a);
  }
  if (positional.empty() || positional.size() > 3) {
    std::cout << "Expected: matrix file in MatrixMarket format [trials] [kernel] [--check] [--dump-y FILE] [--parse-only]\n";
    return 1;
  }
  const std::string mfile = positional[0];
  const int trials = positional.size() > 1 ? std::max(1, atoi(positional[1].c_str())) : 1000;
  const std::string kernel = positional.size() > 2 ? positional[2] : "auto";
  Csr A;
  std::string err;
  if (mfile.rfind("gen:laplace3d:", 0) == 0) {
    const int n = atoi(mfile.c_str() + 14);
    if (n < 1 || n > 1000) {
      std::cerr << "error: grid size outside [1, 1000]\n";
      return 1;
    }
    std::cout << "Generating the 7-point Laplacian on a " << n << "^3 grid...\n";
    laplace3d(n, A);
  } else {
    std::cout << "Reading matrix from " << mfile << "...\n";
    if (!read_matrix_market(mfile, A, err)) {
      std::cerr << "error: " << err << "\n";
      return 1;
    }
  }
  const int64_t nnz = (int64_t)A.crd.size();
  std::cout << "Read matrix (" << A.nrows << "x" << A.ncols << " with " << nnz << " entries)\n";
  if (parse_only) {
    // what the reader made of the file, without touching the GPU: sums that change with a dropped, doubled,
    // transposed or sign-flipped entry, and whether every row's columns ascend
    double sum = 0.0, weighted = 0.0;
    bool sorted = true;
    for (int64_t r = 0; r < A.nrows; ++r)
      for (int64_t j = A.pos[r]; j < A.pos[r + 1]; ++j) {
        sum += A.val[j];
        weighted += (double)(r + 1) * (double)(2 * (int64_t)A.crd[j] + 1) * A.val[j];
        if (j > A.pos[r] && A.crd[j] <= A.crd[j - 1]) sorted = false;
      }
    std::cout.precision(17);
    std::cout << "parse: sum(val) = " << sum << "\n";
    std::cout << "parse: sum((row+1)*(2*col+1)*val) = " << weighted << "\n";
    std::cout << "parse: columns ascend in every row = " << (sorted ? "yes" : "no") << "\n";
    return 0;
  }
  CHECK_LAPIS(lapis_hip_init());

  int32_t *pos = nullptr, *crd = nullptr;
  double *val = nullptr, *x = nullptr, *y = nullptr;
  CHECK_HIP(hipMalloc(&pos, sizeof(int32_t) * (A.nrows + 1)));
  CHECK_HIP(hipMalloc(&crd, sizeof(int32_t) * std::max<int64_t>(nnz, 1)));
  CHECK_HIP(hipMalloc(&val, sizeof(double) * std::max<int64_t>(nnz, 1)));
  CHECK_HIP(hipMalloc(&x, sizeof(double) * std::max<int64_t>(A.ncols, 1)));
  CHECK_HIP(hipMalloc(&y, sizeof(double) * std::max<int64_t>(A.nrows, 1)));
  CHECK_HIP(hipMemcpy(pos, A.pos.data(), sizeof(int32_t) * (A.nrows + 1), hipMemcpyHostToDevice));
  CHECK_HIP(hipMemcpy(crd, A.crd.data(), sizeof(int32_t) * nnz, hipMemcpyHostToDevice));
  CHECK_HIP(hipMemcpy(val, A.val.data(), sizeof(double) * nnz, hipMemcpyHostToDevice));
  // x and y start at zero, as the Kokkos views of the reference driver do
  CHECK_HIP(hipMemset(x, 0, sizeof(double) * std::max<int64_t>(A.ncols, 1)));
  CHECK_HIP(hipMemset(y, 0, sizeof(double) * std::max<int64_t>(A.nrows, 1)));

  lapis_hip_csr_plan *plan = nullptr;
  if (kernel != "reference") {
    CHECK_LAPIS(lapis_hip_csr_plan_create(&plan, A.nrows, A.ncols, nnz, pos, crd, 8, nullptr));
    if (kernel == "rowblock") CHECK_LAPIS(lapis_hip_csr_plan_set_kernel(plan, LAPIS_HIP_SPMV_ROWBLOCK, 0));
    else if (kernel == "nnzsplit") CHECK_LAPIS(lapis_hip_csr_plan_set_kernel(plan, LAPIS_HIP_SPMV_NNZSPLIT, 0));
    else if (kernel == "colblock") CHECK_LAPIS(lapis_hip_csr_plan_build_colblock(plan, crd, val, 8, LAPIS_HIP_COLBLOCK_AUTO, 0, nullptr));
    else if (kernel.rfind("subwarp", 0) == 0)
      CHECK_LAPIS(lapis_hip_csr_plan_set_kernel(plan, LAPIS_HIP_SPMV_SUBWARP, atoi(kernel.c_str() + 7)));
    else if (kernel != "auto") {
      std::cerr << "unknown kernel " << kernel << "\n";
      return 1;
    } else if (trials >= 64) {
      // enough calls for a column-blocked copy to pay back where the library recommends one
      CHECK_LAPIS(lapis_hip_csr_plan_analyze(plan, crd, val, 8, nullptr));
    }
    lapis_hip_csr_stats s;
    CHECK_LAPIS(lapis_hip_csr_plan_get_stats(plan, &s));
    std::cout << "rows: min " << s.min_row_len << " mean " << s.mean_row_len << " max " << s.max_row_len
              << "; kernel " << s.kernel << " width " << s.width << "; reference vector length "
              << s.reference_vector_length << "\n";
  }
  if (check || !dump_path.empty()) {
    std::vector<double> hx((size_t)A.ncols), hy((size_t)A.nrows);
    for (int64_t i = 0; i < A.ncols; ++i) hx[(size_t)i] = (double)(i + 1);
    CHECK_HIP(hipMemcpy(x, hx.data(), sizeof(double) * hx.size(), hipMemcpyHostToDevice));
    CHECK_LAPIS(lapis_hip_spmv_csr_f64_i32(plan, A.nrows, A.ncols, pos, crd, val, x, y, nullptr));
    CHECK_LAPIS(lapis_hip_stream_synchronize(nullptr));
    CHECK_HIP(hipMemcpy(hy.data(), y, sizeof(double) * hy.size(), hipMemcpyDeviceToHost));
    double sum = 0.0;
    for (double v : hy) sum += v;  // ascending index order
    printf("check: sum(y) = %.17g\n", sum);
    if (A.nrows > 0) {
      const int64_t at[4] = {0, A.nrows / 3, A.nrows / 2, A.nrows - 1};
      for (int64_t i : at) printf("check: y[%lld] = %.17g\n", (long long)i, hy[(size_t)i]);
    }
    if (!dump_path.empty()) {
      FILE *f = fopen(dump_path.c_str(), "wb");
      if (!f || fwrite(hy.data(), sizeof(double), hy.size(), f) != hy.size()) {
        std::cerr << "error: cannot write " << dump_path << "\n";
        return 1;
      }
      fclose(f);
    }
    // back to the reference driver's state: x and y zero
    CHECK_HIP(hipMemset(x, 0, sizeof(double) * std::max<int64_t>(A.ncols, 1)));
    CHECK_HIP(hipMemset(y, 0, sizeof(double) * std::max<int64_t>(A.nrows, 1)));
  }
  // Warmup
  CHECK_LAPIS(lapis_hip_spmv_csr_f64_i32(plan, A.nrows, A.ncols, pos, crd, val, x, y, nullptr));
  CHECK_LAPIS(lapis_hip_stream_synchronize(nullptr));
  const auto t0 = std::chrono::steady_clock::now();
  for (int i = 0; i < trials; i++) {
    CHECK_LAPIS(lapis_hip_spmv_csr_f64_i32(plan, A.nrows, A.ncols, pos, crd, val, x, y, nullptr));
    CHECK_LAPIS(lapis_hip_stream_synchronize(nullptr));
  }
  const double elapsed = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
  const double avg = elapsed / trials;
  const double bytes = 2.0 * 8 * A.nrows + 12.0 * nnz + 4.0 * (A.nrows + 1);  // benchmarks/plots/plotSPMV.py:20
  std::cout << "spmv avg time = " << avg << "\n";
  std::cout << "bandwidth = " << bytes / avg / 1e9 << " GB/s, " << 2.0 * nnz / avg / 1e9 << " GFLOP/s\n";
  lapis_hip_csr_plan_destroy(plan);
  (void)hipFree(pos);
  (void)hipFree(crd);
  (void)hipFree(val);
  (void)hipFree(x);
  (void)hipFree(y);
  lapis_hip_finalize();
  return 0;
}
