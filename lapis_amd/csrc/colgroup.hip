// Column-blocked SpMV, workgroup layout (what lapis_hip_csr_plan_build_colblock builds
// for LAPIS_HIP_COLBLOCK_GROUP / AUTO).
//
// The matrix is copied once into tiles = (block of up to 16384 rows) x (slice of 2^s
// columns of x).  A workgroup keeps the row sums of its block in LDS (doubles) and
// walks the block's tiles slice by slice; the blocks are resident together and walk
// together, so the chip gathers from the same few slices of x at a time and they stay
// in L2.  A tile is stored in COLUMN order and the threads take it 64 neighbours per
// wave instruction: with about as many entries in a tile as the slice has 128-byte
// lines, neighbouring lanes fall into the same lines and the address unit merges them
// into one request.  Requests to L2 are what bounds these matrices: the calibration
// kernel of calibrate.hip sustains 250-270 G line requests/s on this chip whatever a
// request carries (67 M single-line gathers in 0.246 ms, two neighbours per line in 0.128 ms).
//
// Entry word = (row within the block << s) | column within the slice; the value array
// runs parallel to it.  tile_ptr[block * (nslices + 1) + k] is where slice k of the
// block starts.
//
// Long rows.  Rows of `long_threshold` entries or more would put hundreds of entries
// into one tile that all add to one LDS word.  They are taken out of their natural
// blocks and numbered among themselves; blocks nblocks_nat, nblocks_nat + 1, ... hold
// up to 16384 of them each.  Such a block is dense (thousands of entries per line of
// x), so almost all of its gathers merge, and no single row dominates a tile.
//
// Work units.  One workgroup = one unit = a contiguous range of the entries of one
// block (blocks differ in size: a block of long rows can hold half the matrix).  A
// block that is one unit adds its sums to y with plain stores; the units of a split
// block, and blocks of long rows, use floating-point atomics on y.  Because several
// wavefronts add into one row sum, the order of the additions of a row is not fixed:
// the last bits of the result can differ from run to run.
#include <hipcub/hipcub.hpp>

#include <algorithm>
#include <cstdlib>
#include <mutex>
#include <vector>

#include "common.hpp"
#include "plan.hpp"

namespace lapis {

constexpr int kMaxSlicesInLds = 6000;  // tile pointers of one block sit in LDS beside 128 KB of row sums

template <typename T, int THREADS, int U, bool NT>
__global__ __launch_bounds__(THREADS) void spmv_colgroup_kernel(int nrows, int rows_per_block, int nblocks_nat,
                                                                int nlong, int nslices, int slice_log2,
                                                                const int *__restrict__ units,
                                                                const int *__restrict__ tile_ptr,
                                                                const int *__restrict__ long_rows,
                                                                const unsigned *__restrict__ bidx,
                                                                const T *__restrict__ bval, const T *__restrict__ x,
                                                                T *__restrict__ y) {
  extern __shared__ __align__(16) unsigned char colgroup_lds[];
  double *acc = reinterpret_cast<double *>(colgroup_lds);
  int *tp = reinterpret_cast<int *>(acc + rows_per_block);  // tile pointers of the block, indexed by slice
  const int tid = threadIdx.x;
  const int block = units[4 * blockIdx.x];
  const int e_first = units[4 * blockIdx.x + 1];
  const int e_last = units[4 * blockIdx.x + 2];
  const int sole = units[4 * blockIdx.x + 3];
  for (int i = tid; i < rows_per_block; i += THREADS) acc[i] = 0.0;
  {
    const int *gtp = tile_ptr + (long long)block * (nslices + 1);
    for (int i = tid; i <= nslices; i += THREADS) tp[i] = gtp[i];
  }
  __syncthreads();

  // the tile that holds entry e_first: last slice s with tp[s] <= e_first
  int s;
  {
    int lo = 0, hi = nslices;  // answer in [lo, hi)
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (tp[mid] <= e_first) lo = mid; else hi = mid;
    }
    s = lo;
  }
  const unsigned cmask = (1u << slice_log2) - 1u;
  constexpr int TRIP = U * THREADS;
  // A trip is up to TRIP consecutive entries of ONE tile, [off, min(off + TRIP, end)):
  // the slice, and with it the base of the gathers, is uniform over the workgroup.
  // (Trips running across tile borders, and a third trip's gathers kept in flight,
  // both measured 10-30 % slower.)
  int off = e_first, end = min(tp[s + 1], e_last);
  while (off >= end && end < e_last) {  // e_first sits at the border of empty tiles
    ++s;
    end = min(tp[s + 1], e_last);
  }
  bool have = off < end;
  unsigned ci[U];
  T cv[U];
  auto load_trip = [&](int o, int e, unsigned (&li)[U], T (&lv)[U]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int p = o + u * THREADS + tid;
      if (p < e) {
        li[u] = ldv<NT>(bidx + p);
        lv[u] = ldv<NT>(bval + p);
      }
    }
  };
  if (have) load_trip(off, end, ci, cv);
  while (have) {
    int ns = s, noff = off + TRIP, nend = end;
    while (noff >= nend && nend < e_last) {  // tile finished: the next one starts where it ends
      ++ns;
      noff = nend;
      nend = min(tp[ns + 1], e_last);
    }
    const bool more = noff < nend;
    unsigned ni[U];
    T nv[U];
    if (more) load_trip(noff, nend, ni, nv);  // in flight while this trip gathers and adds
    const T *xs = x + ((long long)s << slice_log2);
    T pr[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (off + u * THREADS + tid < end) pr[u] = cv[u] * xs[ci[u] & cmask];
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (off + u * THREADS + tid < end) lds_add(acc + (ci[u] >> slice_log2), (double)pr[u]);
    if (more) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        ci[u] = ni[u];
        cv[u] = nv[u];
      }
    }
    s = ns;
    off = noff;
    end = nend;
    have = more;
  }
  __syncthreads();
  // A sum that is exactly zero leaves y alone (y + 0 is y).  This is what keeps the plain
  // stores of a natural block off the long rows inside its range, which other
  // workgroups are updating atomically at the same time.
  if (block < nblocks_nat) {
    const long long row0 = (long long)block * rows_per_block;
    const int rows_here = (int)std::min<long long>(rows_per_block, nrows - row0);
    if (sole) {
      for (int i = tid; i < rows_here; i += THREADS)
        if (acc[i] != 0.0) y[row0 + i] = T(acc[i]) + y[row0 + i];
    } else {
      for (int i = tid; i < rows_here; i += THREADS)
        if (acc[i] != 0.0) unsafeAtomicAdd(y + row0 + i, T(acc[i]));
    }
  } else {
    const long long base = (long long)(block - nblocks_nat) * rows_per_block;
    const int rows_here = (int)std::min<long long>(rows_per_block, nlong - base);
    for (int i = tid; i < rows_here; i += THREADS)
      if (acc[i] != 0.0) unsafeAtomicAdd(y + long_rows[base + i], T(acc[i]));
  }
}

// ---- the same walk with producer and consumer wavefronts -------------------------------
//
// A wavefront that both streams its entries and gathers x waits, at every step, for
// whatever it has in flight: loads of one wavefront return in issue order, so the wait
// for a gather that hits L2 is also a wait for the entry loads issued before it, which
// come from HBM.  Here the roles are split.  PROD wavefronts of the workgroup only
// stream: 512 entries (index words and values, 128-bit loads) per step, one step in
// flight, handed over through a ring of kPcSlots x 512 entries in LDS.  The other
// wavefronts only consume: they copy a chunk from the ring into registers, give the slot
// back, gather x and add into the row sums.  Chunk k is loaded by producer k % PROD,
// passes through slot k % kPcSlots and is consumed by consumer k % CONS; `ready[slot]`
// and `taken[slot]` count how often the slot was filled and emptied.  LDS operations of a
// wavefront execute in issue order, so a flag written after the data is seen after it.
// Every wait is bounded: a flag that never comes makes the wavefront give up and set
// *fault (lapis_hip_csr_plan_check reports it), so the grid drains whatever happens.
constexpr int kPcChunk = 512;
constexpr int kPcSlots = 4;
constexpr int kPcPad = 1024;  // entries allocated behind the copy: the last chunk is loaded whole

// The flags are read and written with the LDS instructions themselves: a volatile access would make the
// compiler wait for every load the wavefront has in flight, the producers' next chunk included.
typedef __attribute__((address_space(3))) int lds_int;
__device__ __forceinline__ int pc_flag_load(const int *flag) {
  int v;
  const unsigned a = (unsigned)(uintptr_t)(const lds_int *)flag;
  asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(a) : "memory");
  return v;
}
__device__ __forceinline__ void pc_flag_store(int *flag, int v) {
  const unsigned a = (unsigned)(uintptr_t)(lds_int *)flag;
  asm volatile("ds_write_b32 %0, %1" : : "v"(a), "v"(v) : "memory");
}

__device__ __forceinline__ bool pc_wait(const int *flag, int want) {
  for (int spin = 0; spin < (1 << 22); ++spin) {
    const int v = __builtin_amdgcn_readfirstlane(pc_flag_load(flag));
    if (v == want) return true;
    __builtin_amdgcn_s_sleep(1);
  }
  return false;
}

__device__ __forceinline__ void pc_compiler_fence() { __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront"); }

template <typename T> struct PcVal;
template <> struct PcVal<double> { typedef v2d vec; static constexpr int per = 2; };
template <> struct PcVal<float> { typedef v4f vec; static constexpr int per = 4; };

template <typename T, int THREADS, int PROD, bool NT>
__global__ __launch_bounds__(THREADS) void spmv_colgroup_pc_kernel(int nrows, int rows_per_block, int nblocks_nat,
                                                                   int nlong, int nslices, int slice_log2,
                                                                   const int *__restrict__ units,
                                                                   const int *__restrict__ tile_ptr,
                                                                   const int *__restrict__ long_rows,
                                                                   const unsigned *__restrict__ bidx,
                                                                   const T *__restrict__ bval, const T *__restrict__ x,
                                                                   T *__restrict__ y, int *__restrict__ fault) {
  typedef typename PcVal<T>::vec VV;
  constexpr int VPER = PcVal<T>::per;            // values per 16-byte vector
  constexpr int NIV = kPcChunk / (64 * 4);       // index vectors per lane and chunk (2)
  constexpr int NVV = kPcChunk / (64 * VPER);    // value vectors per lane and chunk (4 fp64, 2 fp32)
  constexpr int EPL = kPcChunk / 64;             // entries per consumer lane and chunk (8)
  constexpr int CONS = THREADS / 64 - PROD;
  constexpr int DEPTH = 1;                       // chunks a producer has in flight
  static_assert(CONS >= 1 && PROD >= 1, "both roles need a wavefront");
  extern __shared__ __align__(16) unsigned char colgroup_lds[];
  double *acc = reinterpret_cast<double *>(colgroup_lds);
  T *rval = reinterpret_cast<T *>(acc + rows_per_block);
  unsigned *ridx = reinterpret_cast<unsigned *>(rval + kPcSlots * kPcChunk);
  int *ready = reinterpret_cast<int *>(ridx + kPcSlots * kPcChunk);
  int *taken = ready + kPcSlots;
  int *tp = taken + kPcSlots;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int block = units[4 * blockIdx.x];
  const int e_first = units[4 * blockIdx.x + 1];
  const int e_last = units[4 * blockIdx.x + 2];
  const int sole = units[4 * blockIdx.x + 3];
  for (int i = tid; i < rows_per_block; i += THREADS) acc[i] = 0.0;
  {
    const int *gtp = tile_ptr + (long long)block * (nslices + 1);
    for (int i = tid; i <= nslices; i += THREADS) tp[i] = gtp[i];
  }
  if (tid < 2 * kPcSlots) ready[tid] = 0;  // ready[] and taken[] are neighbours
  __syncthreads();

  const int base0 = e_first & ~3;  // chunks start on 16-byte boundaries of both arrays
  const int nchunks = e_last > e_first ? (e_last - base0 + kPcChunk - 1) / kPcChunk : 0;
  bool ok = true;
  if (wave < PROD) {
    v4i ci[DEPTH][NIV];
    VV cv[DEPTH][NVV];
    auto load_chunk = [&](int k, v4i (&li)[NIV], VV (&lv)[NVV]) {
      const long long cb = (long long)base0 + (long long)k * kPcChunk;
      const v4i *pi = reinterpret_cast<const v4i *>(bidx + cb) + lane;
      const VV *pv = reinterpret_cast<const VV *>(bval + cb) + lane;
#pragma unroll
      for (int j = 0; j < NIV; ++j) li[j] = ldv<NT>(pi + j * 64);
#pragma unroll
      for (int j = 0; j < NVV; ++j) lv[j] = ldv<NT>(pv + j * 64);
    };
    // chunk k: wait until its slot was emptied, copy it there, say so
    auto hand_over = [&](int k, const v4i (&li)[NIV], const VV (&lv)[NVV]) {
      const int slot = k % kPcSlots, round = k / kPcSlots;
      if (!pc_wait(taken + slot, round)) return false;
      pc_compiler_fence();
      v4i *wi = reinterpret_cast<v4i *>(ridx + slot * kPcChunk) + lane;
      VV *wv = reinterpret_cast<VV *>(rval + slot * kPcChunk) + lane;
#pragma unroll
      for (int j = 0; j < NIV; ++j) wi[j * 64] = li[j];
#pragma unroll
      for (int j = 0; j < NVV; ++j) wv[j * 64] = lv[j];
      pc_compiler_fence();
      pc_flag_store(ready + slot, round + 1);
      return true;
    };
    // ONE chunk in flight per producer: wait for it, hand it over, ask for the next.  Keeping more of
    // the copy in flight is slower here (two chunks per producer, refilled in turns: config 2 in
    // 0.30-0.31 ms against 0.28): a streamed line waits for HBM, and while it does it holds room in the
    // compute unit's memory pipeline that the consumers' gathers, which come back from L2, would use.
    if (wave < nchunks) {
      int k = wave;
      load_chunk(k, ci[0], cv[0]);
      while (ok && k < nchunks) {
        ok = hand_over(k, ci[0], cv[0]);
        k += PROD;
        load_chunk(min(k, nchunks - 1), ci[0], cv[0]);
      }
    }
  } else {
    const int c = wave - PROD;
    const unsigned cmask = (1u << slice_log2) - 1u;
    // the slice of this lane's entries: tp[s] <= position < tp[s + 1]; positions only grow
    int s = 0, nb = tp[1];
    for (int k = c; k < nchunks && ok; k += CONS) {
      const int slot = k % kPcSlots, round = k / kPcSlots;
      ok = pc_wait(ready + slot, round + 1);
      if (!ok) break;
      pc_compiler_fence();
      unsigned w[EPL];
      T v[EPL];
#pragma unroll
      for (int u = 0; u < EPL; ++u) {
        w[u] = ridx[slot * kPcChunk + u * 64 + lane];
        v[u] = rval[slot * kPcChunk + u * 64 + lane];
      }
      pc_compiler_fence();
      pc_flag_store(taken + slot, round + 1);
      const int cb = base0 + k * kPcChunk;
      T xv[EPL];
      bool act[EPL];
      unsigned xi[EPL];  // an entry outside the unit's range reads x[0] and adds nothing
#pragma unroll
      for (int u = 0; u < EPL; ++u) {
        const int p = cb + u * 64 + lane;
        act[u] = p >= e_first && p < e_last;
        xi[u] = 0;
        if (act[u]) {
          while (p >= nb) {
            ++s;
            nb = tp[s + 1];
          }
          xi[u] = ((unsigned)s << slice_log2) + (w[u] & cmask);
        }
      }
#pragma unroll
      for (int u = 0; u < EPL; ++u) xv[u] = x[xi[u]];
#pragma unroll
      for (int u = 0; u < EPL; ++u) {
        const T pr = v[u] * xv[u];
        if (act[u]) lds_add(acc + (w[u] >> slice_log2), (double)pr);
      }
    }
  }
  if (!ok && lane == 0) atomicExch(fault, 1);
  __syncthreads();
  if (block < nblocks_nat) {
    const long long row0 = (long long)block * rows_per_block;
    const int rows_here = (int)std::min<long long>(rows_per_block, nrows - row0);
    if (sole) {
      for (int i = tid; i < rows_here; i += THREADS)
        if (acc[i] != 0.0) y[row0 + i] = T(acc[i]) + y[row0 + i];
    } else {
      for (int i = tid; i < rows_here; i += THREADS)
        if (acc[i] != 0.0) unsafeAtomicAdd(y + row0 + i, T(acc[i]));
    }
  } else {
    const long long base = (long long)(block - nblocks_nat) * rows_per_block;
    const int rows_here = (int)std::min<long long>(rows_per_block, nlong - base);
    for (int i = tid; i < rows_here; i += THREADS)
      if (acc[i] != 0.0) unsafeAtomicAdd(y + long_rows[base + i], T(acc[i]));
  }
}

// ---- plan-time kernels ---------------------------------------------------------

__global__ __launch_bounds__(256) void long_row_flag_kernel(int nrows, int long_threshold,
                                                            const int *__restrict__ pos, int *__restrict__ flag) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < nrows) flag[i] = pos[i + 1] - pos[i] >= long_threshold ? 1 : 0;
}

__global__ __launch_bounds__(256) void long_row_list_kernel(int nrows, const int *__restrict__ flag,
                                                            const int *__restrict__ rank, int *__restrict__ rows) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < nrows && flag[i]) rows[rank[i]] = (int)i;
}

// key = (block << (col_bits + row_bits)) | (column << row_bits) | row in block: sorted,
// the entries of a block come slice by slice and by column inside a slice.  A long row
// (flag set) belongs to block nblocks_nat + rank / rows, as row rank % rows.
// One wavefront per 1024 consecutive entries; the rows of the entries come from the positions
// (rows_of_chunk), so the cost does not depend on how the entries are spread over the rows.
__global__ __launch_bounds__(256) void colgroup_keys_kernel(int nrows, long long nnz, int row_bits, int col_bits,
                                                            int nblocks_nat, const int *__restrict__ long_flag,
                                                            const int *__restrict__ long_rank,
                                                            const int *__restrict__ pos,
                                                            const int *__restrict__ crd,
                                                            unsigned long long *__restrict__ keys) {
  __shared__ int s_rows[4][1024];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long long j0 = ((long long)blockIdx.x * 4 + wave) * 1024;
  if (j0 >= nnz) return;
  const long long j1 = std::min(nnz, j0 + 1024);
  rows_of_chunk(pos, nrows, j0, j1, s_rows[wave]);
  for (long long j = j0 + lane; j < j1; j += 64) {
    const int row = s_rows[wave][j - j0];
    long long v = row;  // position in the blocked numbering
    if (long_flag && long_flag[row]) v = ((long long)nblocks_nat << row_bits) + long_rank[row];
    const unsigned long long rb = (unsigned long long)(v >> row_bits);
    const unsigned long long rl = (unsigned long long)(v & ((1LL << row_bits) - 1));
    const unsigned long long c = (unsigned long long)(unsigned)crd[j];
    keys[j] = (rb << (col_bits + row_bits)) | (c << row_bits) | rl;
  }
}

__global__ __launch_bounds__(256) void colgroup_entry_kernel(long long n, int row_bits, int slice_log2,
                                                             const unsigned long long *__restrict__ keys,
                                                             unsigned *__restrict__ out) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const unsigned long long k = keys[i];
  const unsigned rl = (unsigned)(k & ((1ull << row_bits) - 1ull));
  const unsigned cs = (unsigned)((k >> row_bits) & ((1ull << slice_log2) - 1ull));
  out[i] = (rl << slice_log2) | cs;
}

// tile_ptr[b * (nslices + 1) + s] = first sorted entry whose key is >= (block b, slice s);
// block_range[2b], [2b+1] = the block's first entry and one past its last
__global__ __launch_bounds__(256) void colgroup_tile_ptr_kernel(long long nnz, int nblocks, int nslices, int row_bits,
                                                                int col_bits, int slice_log2,
                                                                const unsigned long long *__restrict__ keys,
                                                                int *__restrict__ tile_ptr,
                                                                int *__restrict__ block_range) {
  const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
  if (t >= (long long)nblocks * (nslices + 1)) return;
  const unsigned long long b = (unsigned long long)(t / (nslices + 1));
  const int s = (int)(t % (nslices + 1));
  const unsigned long long target =
      s == nslices ? ((b + 1) << (col_bits + row_bits))
                   : ((b << (col_bits + row_bits)) | (((unsigned long long)s << slice_log2) << row_bits));
  long long lo = 0, hi = nnz;
  while (lo < hi) {
    const long long mid = (lo + hi) >> 1;
    if (keys[mid] < target) lo = mid + 1; else hi = mid;
  }
  tile_ptr[t] = (int)lo;
  if (s == 0) block_range[2 * b] = (int)lo;
  if (s == nslices) block_range[2 * b + 1] = (int)lo;
}

// ---- launch ----------------------------------------------------------------------

template <typename T, int THREADS, int U, bool NT>
int launch_colgroup_cfg(const lapis_hip_csr_plan *p, const T *x, T *y, hipStream_t st) {
  auto kernel = spmv_colgroup_kernel<T, THREADS, U, NT>;
  const size_t lds_bytes = sizeof(double) * (size_t)p->colblock_rows + sizeof(int) * ((size_t)p->colblock_nslices + 2);
  // one per instantiation; more than 64 KB of dynamic LDS has to be asked for
  static std::once_flag attribute_once;
  static hipError_t attribute_status = hipSuccess;
  std::call_once(attribute_once, [&] {
    attribute_status = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
  });
  LAPIS_HIP_TRY(attribute_status);
  const dim3 grid((unsigned)p->colblock_nunits), block(THREADS);
  hipEvent_t e0, e1;
  if (timing_next_events(&e0, &e1))
    hipExtLaunchKernelGGL(kernel, grid, block, lds_bytes, st, e0, e1, 0, (int)p->stats.nrows, p->colblock_rows,
                          p->colblock_nblocks_nat, p->colblock_nlong, p->colblock_nslices, p->colblock_slice_log2,
                          (const int *)p->colblock_units, (const int *)p->colblock_tile_ptr,
                          (const int *)p->colblock_long_rows, (const unsigned *)p->colblock_idx,
                          (const T *)p->colblock_val, x, y);
  else
    hipLaunchKernelGGL(kernel, grid, block, lds_bytes, st, (int)p->stats.nrows, p->colblock_rows,
                       p->colblock_nblocks_nat, p->colblock_nlong, p->colblock_nslices, p->colblock_slice_log2,
                       (const int *)p->colblock_units, (const int *)p->colblock_tile_ptr,
                       (const int *)p->colblock_long_rows, (const unsigned *)p->colblock_idx,
                       (const T *)p->colblock_val, x, y);
  LAPIS_LAUNCH_CHECK();
  return LAPIS_HIP_OK;
}

template <typename T, int THREADS>
int launch_colgroup_threads(const lapis_hip_csr_plan *p, const T *x, T *y, hipStream_t st) {
  const bool nt = p->nontemporal;
  if (p->colblock_epl == 4)
    return nt ? launch_colgroup_cfg<T, THREADS, 4, true>(p, x, y, st)
              : launch_colgroup_cfg<T, THREADS, 4, false>(p, x, y, st);

  return nt ? launch_colgroup_cfg<T, THREADS, 8, true>(p, x, y, st)
            : launch_colgroup_cfg<T, THREADS, 8, false>(p, x, y, st);
}

size_t colgroup_pc_lds_bytes(int rows, int nslices, int value_bytes) {
  return sizeof(double) * (size_t)rows + (size_t)kPcSlots * kPcChunk * (value_bytes + 4) + sizeof(int) * 2 * kPcSlots +
         sizeof(int) * ((size_t)nslices + 2);
}

template <typename T, int THREADS, int PROD, bool NT>
int launch_colgroup_pc_cfg(const lapis_hip_csr_plan *p, const T *x, T *y, hipStream_t st) {
  auto kernel = spmv_colgroup_pc_kernel<T, THREADS, PROD, NT>;
  const size_t lds_bytes = colgroup_pc_lds_bytes(p->colblock_rows, p->colblock_nslices, (int)sizeof(T));
  static std::once_flag attribute_once;
  static hipError_t attribute_status = hipSuccess;
  std::call_once(attribute_once, [&] {
    attribute_status = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
  });
  LAPIS_HIP_TRY(attribute_status);
  const dim3 grid((unsigned)p->colblock_nunits), block(THREADS);
  hipEvent_t e0, e1;
  if (timing_next_events(&e0, &e1))
    hipExtLaunchKernelGGL(kernel, grid, block, lds_bytes, st, e0, e1, 0, (int)p->stats.nrows, p->colblock_rows,
                          p->colblock_nblocks_nat, p->colblock_nlong, p->colblock_nslices, p->colblock_slice_log2,
                          (const int *)p->colblock_units, (const int *)p->colblock_tile_ptr,
                          (const int *)p->colblock_long_rows, (const unsigned *)p->colblock_idx,
                          (const T *)p->colblock_val, x, y, p->colblock_fault);
  else
    hipLaunchKernelGGL(kernel, grid, block, lds_bytes, st, (int)p->stats.nrows, p->colblock_rows,
                       p->colblock_nblocks_nat, p->colblock_nlong, p->colblock_nslices, p->colblock_slice_log2,
                       (const int *)p->colblock_units, (const int *)p->colblock_tile_ptr,
                       (const int *)p->colblock_long_rows, (const unsigned *)p->colblock_idx,
                       (const T *)p->colblock_val, x, y, p->colblock_fault);
  LAPIS_LAUNCH_CHECK();
  return LAPIS_HIP_OK;
}

template <typename T>
int launch_colgroup_pc(const lapis_hip_csr_plan *p, const T *x, T *y, hipStream_t st) {
  const bool nt = p->nontemporal;
#define LAPIS_PC_CASE(THREADS, PROD)                                                        \
  case THREADS * 16 + PROD:                                                                 \
    return nt ? launch_colgroup_pc_cfg<T, THREADS, PROD, true>(p, x, y, st)                 \
              : launch_colgroup_pc_cfg<T, THREADS, PROD, false>(p, x, y, st)
  switch (p->colblock_pc_threads * 16 + p->colblock_pc_prod) {
    LAPIS_PC_CASE(1024, 4);
    LAPIS_PC_CASE(1024, 2);
    LAPIS_PC_CASE(768, 2);
    LAPIS_PC_CASE(1024, 6);
    LAPIS_PC_CASE(768, 3);
    LAPIS_PC_CASE(640, 4);
    LAPIS_PC_CASE(512, 3);
    LAPIS_PC_CASE(512, 2);
    default:
      return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT,
                       "colblock: no producer/consumer kernel with %d threads and %d producer wavefronts",
                       p->colblock_pc_threads, p->colblock_pc_prod);
  }
#undef LAPIS_PC_CASE
}

template <typename T>
int launch_colgroup(const lapis_hip_csr_plan *p, const T *x, T *y, hipStream_t st) {
  if (p->colblock_nunits == 0) return LAPIS_HIP_OK;
  if (p->colblock_pc_prod > 0) return launch_colgroup_pc<T>(p, x, y, st);
  switch (p->colblock_threads) {
    case 1024: return launch_colgroup_threads<T, 1024>(p, x, y, st);
    case 512: return launch_colgroup_threads<T, 512>(p, x, y, st);
    case 256: return launch_colgroup_threads<T, 256>(p, x, y, st);
    default:
      return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT, "colblock: no workgroup kernel with %d threads",
                       p->colblock_threads);
  }
}
template int launch_colgroup<double>(const lapis_hip_csr_plan *, const double *, double *, hipStream_t);
template int launch_colgroup<float>(const lapis_hip_csr_plan *, const float *, float *, hipStream_t);

// ---- build -------------------------------------------------------------------------

template <typename T>
int build_colgroup(lapis_hip_csr_plan *p, const int32_t *crd, const T *val, int slice_log2, hipStream_t st) {
  const int64_t nnz = p->stats.nnz, nrows = p->stats.nrows;
  const int col_bits = std::max(1, bits_for(p->stats.ncols));
  auto env_or = [](const char *name, int fallback) {
    const char *v = getenv(name);
    return v ? atoi(v) : fallback;
  };
  // 16 rows per thread.  The more rows share a tile, the more lanes fall into one line
  // of x, so the block is as large as LDS allows unless the matrix is smaller.
  int rows = env_or("LAPIS_HIP_COLBLOCK_ROWS", 0);
  if (rows != 4096 && rows != 8192 && rows != 16384) rows = nrows > 8192 ? 16384 : (nrows > 4096 ? 8192 : 4096);
  const int row_bits = bits_for(rows);
  slice_log2 = std::min(slice_log2, 32 - row_bits);  // an entry word holds row in block | column in slice
  // Threads per workgroup: 16 rows per thread, but half of that where a tile holds at most
  // about two entries per 128-byte line of x.  Such matrices are bound by requests to L2,
  // and 8 wavefronts per CU, each with one gather in flight, measured 2-6 % faster than 16
  // (4.2 M rows with 16 / 24 / 32 per row: 0.305 / 0.423 / 0.538 against 0.325 / 0.445 /
  // 0.546 ms).  Dense tiles are bound by instruction issue and lose up to 40 % with half the
  // threads (2.1 M rows, 32 per row: 0.265 against 0.248 ms; config 3: 0.225 against 0.161).
  // With a quarter of an entry per line it is 0.123 against 0.129 ms (4.2 M rows, 4 per row)
  // but 0.519 against 0.509 ms when the blocks need two rounds (8.4 M rows, 8 per row).
  int threads = rows / 16;
  {
    const double per_line = (double)rows * p->stats.mean_row_len * (128.0 / sizeof(T)) /
                            (double)std::max<int64_t>(1, p->stats.ncols);
    if (rows == 16384 && per_line < 2.5) threads = 512;
    const int forced = env_or("LAPIS_HIP_COLBLOCK_THREADS", 0);
    if (forced == 256 || forced == 512 || forced == 1024) threads = forced;
  }
  const int nblocks_nat = (int)ceil_div(nrows, rows);
  // finer slices than LDS has room for tile pointers are widened (a matter of speed only)
  while (slice_log2 < 32 - row_bits && ceil_div(p->stats.ncols, 1LL << slice_log2) > kMaxSlicesInLds) ++slice_log2;
  const int64_t nslices64 = ceil_div(p->stats.ncols, 1LL << slice_log2);
  if (slice_log2 < 1 || nslices64 > kMaxSlicesInLds)
    return set_error(LAPIS_HIP_ERR_NO_TILING,
                     "csr_plan_build_colblock: %lld slices of 2^%d columns; the workgroup layout takes at most %d",
                     (long long)nslices64, slice_log2, kMaxSlicesInLds);
  const int nslices = (int)nslices64;
  // Long rows: a fixed floor, raised for matrices whose rows are long throughout (there
  // a tile holds few rows' worth of entries anyway and nothing is gained by moving them).
  int long_threshold = env_or("LAPIS_HIP_COLBLOCK_LONG", 0);
  if (long_threshold <= 0) long_threshold = (int)std::max<double>(2048.0, 16.0 * p->stats.mean_row_len);
  long_threshold = std::max(2, long_threshold);

  unsigned long long *keys_in = nullptr, *keys_out = nullptr;
  T *val_out = nullptr;
  unsigned *idx = nullptr, *perm = nullptr;
  int *tile_ptr = nullptr, *block_range = nullptr, *long_flag = nullptr, *long_rank = nullptr, *long_rows = nullptr,
      *units = nullptr, *fault = nullptr;
  void *scan_temp = nullptr;
  size_t scan_bytes = 0;
  auto release = [&](bool all) {
    if (keys_in) (void)hipFree(keys_in);
    if (keys_out) (void)hipFree(keys_out);
    if (scan_temp) (void)hipFree(scan_temp);
    if (long_flag) (void)hipFree(long_flag);
    if (long_rank) (void)hipFree(long_rank);
    if (block_range) (void)hipFree(block_range);
    if (all) {
      if (val_out) (void)hipFree(val_out);
      if (idx) (void)hipFree(idx);
      if (perm) (void)hipFree(perm);
      if (tile_ptr) (void)hipFree(tile_ptr);
      if (long_rows) (void)hipFree(long_rows);
      if (units) (void)hipFree(units);
      if (fault) (void)hipFree(fault);
    }
  };
  auto fail = [&](hipError_t e, const char *what) {
    release(true);
    return set_error(LAPIS_HIP_ERR_RUNTIME, "csr_plan_build_colblock: %s failed: %s", what, hipGetErrorString(e));
  };
  hipError_t e;

  // 1. the long rows and their numbering
  int nlong = 0;
  if (p->stats.max_row_len >= long_threshold) {
    const dim3 row_grid((unsigned)ceil_div(nrows, 256));
    if ((e = hipMalloc(&long_flag, sizeof(int) * (size_t)nrows)) != hipSuccess) return fail(e, "hipMalloc");
    if ((e = hipMalloc(&long_rank, sizeof(int) * (size_t)nrows)) != hipSuccess) return fail(e, "hipMalloc");
    hipLaunchKernelGGL(long_row_flag_kernel, row_grid, dim3(256), 0, st, (int)nrows, long_threshold, p->pos, long_flag);
    if ((e = hipGetLastError()) != hipSuccess) return fail(e, "long row flag kernel");
    if ((e = hipcub::DeviceScan::ExclusiveSum(nullptr, scan_bytes, long_flag, long_rank, (int)nrows, st)) != hipSuccess)
      return fail(e, "scan sizing");
    if ((e = hipMalloc(&scan_temp, scan_bytes ? scan_bytes : 1)) != hipSuccess) return fail(e, "hipMalloc");
    if ((e = hipcub::DeviceScan::ExclusiveSum(scan_temp, scan_bytes, long_flag, long_rank, (int)nrows, st)) !=
        hipSuccess)
      return fail(e, "scan");
    int tail[2] = {0, 0};
    if ((e = hipMemcpyAsync(&tail[0], long_flag + (nrows - 1), sizeof(int), hipMemcpyDeviceToHost, st)) != hipSuccess)
      return fail(e, "copy");
    if ((e = hipMemcpyAsync(&tail[1], long_rank + (nrows - 1), sizeof(int), hipMemcpyDeviceToHost, st)) != hipSuccess)
      return fail(e, "copy");
    if ((e = hipStreamSynchronize(st)) != hipSuccess) return fail(e, "synchronize");
    nlong = tail[0] + tail[1];
    if (nlong > 0) {
      if ((e = hipMalloc(&long_rows, sizeof(int) * (size_t)nlong)) != hipSuccess) return fail(e, "hipMalloc");
      hipLaunchKernelGGL(long_row_list_kernel, row_grid, dim3(256), 0, st, (int)nrows, long_flag, long_rank, long_rows);
      if ((e = hipGetLastError()) != hipSuccess) return fail(e, "long row list kernel");
    }
  }
  const int nblocks = nblocks_nat + (int)ceil_div(nlong, rows);
  const int end_bit = bits_for((int64_t)nblocks) + col_bits + row_bits;
  if (end_bit > 64 || (int64_t)nblocks * (nslices + 1) > (1LL << 27)) {
    release(true);
    return set_error(LAPIS_HIP_ERR_NO_TILING,
                     "csr_plan_build_colblock: %d row blocks x %d slices of 2^%d columns is not a usable tiling",
                     nblocks, nslices, slice_log2);
  }

  // 2. sort the entries by (block, column, row in block): the entries arrive by rows and the sort is
  // stable, so the bits of the row in its block need no passes of their own
  const size_t ntiles = (size_t)nblocks * ((size_t)nslices + 1);
  if ((e = hipMalloc(&keys_in, sizeof(unsigned long long) * (size_t)nnz)) != hipSuccess) return fail(e, "hipMalloc");
  // kPcPad entries behind both arrays: the producer wavefronts load whole chunks
  if ((e = hipMalloc(&val_out, sizeof(T) * ((size_t)nnz + kPcPad))) != hipSuccess) return fail(e, "hipMalloc");
  if ((e = hipMalloc(&idx, sizeof(unsigned) * ((size_t)nnz + kPcPad))) != hipSuccess) return fail(e, "hipMalloc");
  if ((e = hipMemsetAsync(val_out + nnz, 0, sizeof(T) * kPcPad, st)) != hipSuccess) return fail(e, "hipMemsetAsync");
  if ((e = hipMemsetAsync(idx + nnz, 0, sizeof(unsigned) * kPcPad, st)) != hipSuccess) return fail(e, "hipMemsetAsync");
  if ((e = hipMalloc(&fault, sizeof(int))) != hipSuccess) return fail(e, "hipMalloc");
  if ((e = hipMemsetAsync(fault, 0, sizeof(int), st)) != hipSuccess) return fail(e, "hipMemsetAsync");
  if ((e = hipMalloc(&tile_ptr, sizeof(int) * ntiles)) != hipSuccess) return fail(e, "hipMalloc");
  if ((e = hipMalloc(&block_range, sizeof(int) * 2 * (size_t)nblocks)) != hipSuccess) return fail(e, "hipMalloc");
  hipLaunchKernelGGL(colgroup_keys_kernel, dim3((unsigned)ceil_div(ceil_div(nnz, 1024), 4)), dim3(256), 0, st,
                     (int)nrows, (long long)nnz, row_bits, col_bits, nblocks_nat, nlong > 0 ? (const int *)long_flag : (const int *)nullptr,
                     (const int *)long_rank, p->pos, crd, keys_in);
  if ((e = hipGetLastError()) != hipSuccess) return fail(e, "key kernel");
  // the permutation of the sort is kept: lapis_hip_csr_plan_update_values refreshes the copy's values with it
  {
    const int rc = sort_keys_with_perm(keys_in, nnz, row_bits, end_bit, &keys_out, &perm, st);
    if (rc != LAPIS_HIP_OK) {
      release(true);
      return rc;
    }
    if (gather_values<T>(perm, val, val_out, nnz, st) != LAPIS_HIP_OK) return fail(hipGetLastError(), "value gather");
  }
  hipLaunchKernelGGL(colgroup_entry_kernel, dim3((unsigned)ceil_div(nnz, 256)), dim3(256), 0, st, (long long)nnz,
                     row_bits, slice_log2, keys_out, idx);
  if ((e = hipGetLastError()) != hipSuccess) return fail(e, "entry kernel");
  hipLaunchKernelGGL(colgroup_tile_ptr_kernel, dim3((unsigned)ceil_div((int64_t)ntiles, 256)), dim3(256), 0, st,
                     (long long)nnz, nblocks, nslices, row_bits, col_bits, slice_log2, keys_out, tile_ptr, block_range);
  if ((e = hipGetLastError()) != hipSuccess) return fail(e, "tile pointer kernel");

  // 3. work units: every block's entries in equal parts of at most `unit` entries
  std::vector<int> ranges(2 * (size_t)nblocks);
  if ((e = hipMemcpyAsync(ranges.data(), block_range, sizeof(int) * ranges.size(), hipMemcpyDeviceToHost, st)) !=
      hipSuccess)
    return fail(e, "copy");
  if ((e = hipStreamSynchronize(st)) != hipSuccess) return fail(e, "synchronize");
  // The units run in rounds of as many workgroups as the chip holds: with no more
  // blocks than that, take the smallest unit size that still gives a single round;
  // otherwise 1.25 x the mean block, so that only outsized blocks are cut.
  int64_t unit = env_or("LAPIS_HIP_COLBLOCK_UNIT", 0);
  if (unit <= 0) {
    // workgroups of 16384 / 8192 / 4096 rows fit 1 / 2 / 4 to a CU (LDS limit)
    const int64_t cus = (int64_t)std::max(1, device_cu_count()) * (16384 / rows);
    int64_t nonempty = 0, longest = 1;
    for (int b = 0; b < nblocks; ++b) {
      const int64_t len = (int64_t)ranges[2 * (size_t)b + 1] - ranges[2 * (size_t)b];
      if (len > 0) ++nonempty;
      longest = std::max(longest, len);
    }
    if (nonempty <= cus) {
      int64_t lo = 1, hi = longest;  // smallest unit with sum(ceil(len / unit)) <= cus
      while (lo < hi) {
        const int64_t mid = (lo + hi) / 2;
        int64_t count = 0;
        for (int b = 0; b < nblocks; ++b)
          count += ceil_div((int64_t)ranges[2 * (size_t)b + 1] - ranges[2 * (size_t)b], mid);
        if (count <= cus) hi = mid; else lo = mid + 1;
      }
      unit = lo;
    } else {
      unit = ceil_div(5 * nnz, 4 * nonempty);
    }
    unit = std::max<int64_t>(unit, 4096);
  }
  std::vector<int> hunits;
  for (int b = 0; b < nblocks; ++b) {
    const int64_t first = ranges[2 * (size_t)b], last = ranges[2 * (size_t)b + 1];
    if (last <= first) continue;  // nothing to add for this block
    const int64_t parts = ceil_div(last - first, unit);
    for (int64_t k = 0; k < parts; ++k) {
      hunits.push_back(b);
      hunits.push_back((int)(first + (last - first) * k / parts));
      hunits.push_back((int)(first + (last - first) * (k + 1) / parts));
      hunits.push_back(parts == 1 ? 1 : 0);
    }
  }
  const int nunits = (int)(hunits.size() / 4);
  if (nunits > 0) {
    if ((e = hipMalloc(&units, sizeof(int) * hunits.size())) != hipSuccess) return fail(e, "hipMalloc");
    if ((e = hipMemcpyAsync(units, hunits.data(), sizeof(int) * hunits.size(), hipMemcpyHostToDevice, st)) != hipSuccess)
      return fail(e, "copy");
  }
  if ((e = hipStreamSynchronize(st)) != hipSuccess) return fail(e, "synchronize");
  release(false);
  free_colblock(p);
  p->colblock_group = 1;
  p->colblock_epl = env_or("LAPIS_HIP_COLBLOCK_EPL", 8);  // entries per thread and trip
  p->colblock_rows = rows;
  p->colblock_threads = threads;
  p->colblock_fault = fault;
  {
    // Producer and consumer wavefronts: the ring and the tile pointers have to fit beside the row sums,
    // and a consumer lane finds its slice by walking the tile pointers, which wants tiles of some size.
    // Instantiated: 1024 threads with 2, 4 or 6 producers; 768 with 2 or 3; 640 with 4; 512 with 2 or 3.
    // LAPIS_HIP_COLBLOCK_PC unset: chosen here; 0: never; n > 0: n producers of LAPIS_HIP_COLBLOCK_PC_THREADS.
    int prod = env_or("LAPIS_HIP_COLBLOCK_PC", -1);
    int pc_threads = env_or("LAPIS_HIP_COLBLOCK_PC_THREADS", 1024);
    if (prod < 0) {
      // doubles in request-bound tiles (the rule that also picks 512 threads) gain 8 % from the split
      // (config 2: 0.280 against 0.306 ms); floats and dense tiles lose (config 3: 0.168-0.18 against 0.160 ms)
      prod = (sizeof(T) == 8 && threads == 512) ? 2 : 0;
      pc_threads = 512;
    }
    if (colgroup_pc_lds_bytes(rows, nslices, (int)sizeof(T)) > 160 * 1024) prod = 0;
    p->colblock_pc_prod = std::max(0, prod);
    p->colblock_pc_threads = pc_threads;
  }
  p->colblock_nblocks = nblocks;
  p->colblock_nblocks_nat = nblocks_nat;
  p->colblock_nslices = nslices;
  p->colblock_nunits = nunits;
  p->colblock_units = units;
  p->colblock_nlong = nlong;
  p->colblock_long_rows = long_rows;
  p->colblock_long_threshold = long_threshold;
  p->colblock_tile_ptr = tile_ptr;
  p->colblock_idx = idx;
  p->colblock_val = val_out;
  p->colblock_perm = perm;
  p->colblock_src_crd = crd;
  p->colblock_src_val = val;
  p->colblock_value_bytes = (int)sizeof(T);
  p->colblock_col_bits = col_bits;
  p->colblock_slice_log2 = slice_log2;
  p->colblock_built = true;
  p->colblock_pace_fp = 0;  // the workgroups keep pace by themselves: clock pacing measured no gain here
  p->colblock_free_ms = p->colblock_paced_ms = 0.0;
  if (getenv("LAPIS_HIP_VERBOSE"))
    fprintf(stderr,
            "lapis_hip: workgroup-blocked copy: %d blocks of %d rows (%d of them for %d rows with >= %d entries) x %d "
            "slices of 2^%d columns, %d work units of at most %lld entries\n",
            nblocks, rows, nblocks - nblocks_nat, nlong, long_threshold, nslices, slice_log2, nunits, (long long)unit);
  return LAPIS_HIP_OK;
}
template int build_colgroup<double>(lapis_hip_csr_plan *, const int32_t *, const double *, int, hipStream_t);
template int build_colgroup<float>(lapis_hip_csr_plan *, const int32_t *, const float *, int, hipStream_t);

}  // namespace lapis
