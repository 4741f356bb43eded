// Mask pre-passes that run on the device before the attention kernels:
//   - COO entries -> row buckets (histogram, exclusive scan, scatter), any entry order;
//   - global-token list -> per-row flag bytes.
#include "spfa_prep.hpp"

#include "spfa_common.hpp"

namespace spfa {

namespace {

constexpr int kScanThreads = 256;
constexpr int kScanPerThread = 8;
constexpr int kScanTile = kScanThreads * kScanPerThread;

__global__ void fill_u32_kernel(uint32_t* p, int64_t n, uint32_t value) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) p[i] = value;
}

__device__ __forceinline__ int64_t load_index(const void* p, int64_t i, int wide) {
  return wide ? (int64_t)((const uint64_t*)p)[i] : (int64_t)((const uint32_t*)p)[i];
}

// 1 -> *flag when the entries are not sorted by row or hold a row outside [0, n_rows)
__global__ void coo_check_sorted_kernel(const void* row_ind, int wide, int64_t nnz, int64_t n_rows,
                                        uint32_t* flag) {
  int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  bool bad = false;
  for (; e < nnz; e += stride) {
    const int64_t r = load_index(row_ind, e, wide);
    if (r < 0 || r >= n_rows) bad = true;
    if (e > 0 && load_index(row_ind, e - 1, wide) > r) bad = true;
  }
  if (bad) *flag = 1u;
}

// sorted entries: row_off[r] = first entry whose row is >= r
__global__ void coo_sorted_offsets_kernel(const void* row_ind, int wide, int64_t nnz, int64_t n_rows,
                                          const uint32_t* flag, uint32_t* row_off) {
  if (*flag) return;
  int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; e <= nnz; e += stride) {
    const int64_t prev = e > 0 ? load_index(row_ind, e - 1, wide) : -1;
    const int64_t cur = e < nnz ? load_index(row_ind, e, wide) : n_rows;
    for (int64_t r = prev + 1; r <= cur; r++) row_off[r] = (uint32_t)e;
  }
}

__global__ void coo_histogram_kernel(const void* row_ind, int wide, int64_t nnz, int64_t n_rows,
                                     const uint32_t* flag, uint32_t* counts) {
  if (!*flag) return;
  int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; e < nnz; e += stride) {
    int64_t r = load_index(row_ind, e, wide);
    if (r >= 0 && r < n_rows) atomicAdd(&counts[r], 1u);
  }
}

__global__ void coo_scatter_kernel(const void* row_ind, int wide, const uint32_t* col_ind,
                                   int64_t nnz, int64_t n_rows, const uint32_t* flag,
                                   uint32_t* cursor, uint32_t* cols_out) {
  if (!*flag) return;
  int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; e < nnz; e += stride) {
    int64_t r = load_index(row_ind, e, wide);
    if (r >= 0 && r < n_rows) {
      uint32_t pos = atomicAdd(&cursor[r], 1u);
      cols_out[pos] = col_ind[e];
    }
  }
}

// inclusive scan over the wavefront
__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t x, int lane) {
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    uint32_t y = (uint32_t)__builtin_amdgcn_ds_bpermute(((lane - off) & 63) << 2, (int)x);
    if (lane >= off) x += y;
  }
  return x;
}

// exclusive scan of one value per thread over a 256-thread block; returns the thread's prefix
// and the block total
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t x, uint32_t& total,
                                                         uint32_t* lds /*[4]*/) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t inc = wave_inclusive_scan(x, lane);
  if (lane == 63) lds[wave] = inc;
  __syncthreads();
  uint32_t wave_prefix = 0, tot = 0;
#pragma unroll
  for (int w = 0; w < kScanThreads / kWave; w++) {
    uint32_t s = lds[w];
    if (w < wave) wave_prefix += s;
    tot += s;
  }
  __syncthreads();
  total = tot;
  return wave_prefix + inc - x;
}

// (the scan kernels take an optional gate: they return at once when *gate == 0)
__global__ __launch_bounds__(kScanThreads) void scan_tile_sums_kernel(const uint32_t* in, int64_t n,
                                                                      uint32_t* tile_sums,
                                                                      const uint32_t* gate) {
  __shared__ uint32_t lds[4];
  if (gate != nullptr && !*gate) return;
  const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanPerThread;
  uint32_t s = 0;
#pragma unroll
  for (int j = 0; j < kScanPerThread; j++)
    if (base + j < n) s += in[base + j];
  uint32_t total;
  block_exclusive_scan(s, total, lds);
  if (threadIdx.x == 0) tile_sums[blockIdx.x] = total;
}

// single block: exclusive scan of the tile sums in place
__global__ __launch_bounds__(kScanThreads) void scan_sums_kernel(uint32_t* tile_sums, int64_t n_tiles,
                                                                 const uint32_t* gate) {
  __shared__ uint32_t lds[4];
  if (gate != nullptr && !*gate) return;
  uint32_t carry = 0;
  for (int64_t base = 0; base < n_tiles; base += kScanThreads) {
    int64_t i = base + threadIdx.x;
    uint32_t x = i < n_tiles ? tile_sums[i] : 0u;
    uint32_t total;
    uint32_t ex = block_exclusive_scan(x, total, lds);
    if (i < n_tiles) tile_sums[i] = carry + ex;
    carry += total;
  }
}

// exclusive scan of in[0..n) into out[0..n) and out2[0..n); out[n] = out2[n] = grand total is
// written by the block that owns element n-1
__global__ __launch_bounds__(kScanThreads) void scan_apply_kernel(const uint32_t* in, int64_t n,
                                                                  const uint32_t* tile_sums,
                                                                  uint32_t* out, uint32_t* out2,
                                                                  const uint32_t* gate) {
  __shared__ uint32_t lds[4];
  if (gate != nullptr && !*gate) return;
  const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanPerThread;
  uint32_t v[kScanPerThread];
  uint32_t s = 0;
#pragma unroll
  for (int j = 0; j < kScanPerThread; j++) {
    v[j] = (base + j < n) ? in[base + j] : 0u;
    s += v[j];
  }
  uint32_t total;
  uint32_t run = block_exclusive_scan(s, total, lds) + tile_sums[blockIdx.x];
#pragma unroll
  for (int j = 0; j < kScanPerThread; j++) {
    if (base + j < n) {
      out[base + j] = run;
      out2[base + j] = run;
    }
    run += v[j];
    if (base + j == n - 1) {
      out[n] = run;
      out2[n] = run;
    }
  }
}

__global__ void mark_globals_kernel(const int32_t* globs, int64_t n_globs, int64_t n, uint32_t* bits,
                                    uint32_t* count, int32_t* uq) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n_globs) {
    int64_t g = globs[i];
    if (g >= 0 && g < n) {
      const uint32_t bit = 1u << (g & 31);
      const uint32_t old = atomicOr(&bits[g >> 5], bit);
      if (!(old & bit)) uq[atomicAdd(count, 1u)] = (int32_t)g;  // first time this row is listed
    }
  }
}

// ---- two-pass partition of unsorted COO entries by row -----------------------------------
// Pass 1 stages a whole tile in LDS (152 KB with the bucket tables: one workgroup per CU), so the
// workgroup is as large as it can be: 1024 threads and 16384 entries measured 0.35 ms for 50 M
// entries against 0.78 ms with 256 threads and 8192 entries (and longer runs per bucket).
constexpr int kPartThreads = 1024;
constexpr int kPartTile = 16384;     // entries per workgroup in pass 1
constexpr int kPartMaxBuckets = 2048;

// pass 1a: per-tile histogram of the high digit, stored bucket-major: hist[b * n_tiles + tile].
// The same pass over the row indices decides whether the entries need bucketing at all: it sets
// *flag when they are not sorted by row or hold a row outside [0, n_rows) (so the sortedness check
// costs no pass of its own; for sorted entries the histogram is simply not used).
__global__ __launch_bounds__(kPartThreads) void coo_part_count_kernel(
    const void* row_ind, int wide, int64_t nnz, int64_t n_rows, int lo_bits, int n_hi,
    int64_t n_tiles, uint32_t* flag, uint32_t* hist) {
  __shared__ uint32_t cnt[kPartMaxBuckets];
  for (int b = threadIdx.x; b < n_hi; b += kPartThreads) cnt[b] = 0;
  __syncthreads();
  const int64_t beg = (int64_t)blockIdx.x * kPartTile;
  const int64_t end = beg + kPartTile < nnz ? beg + kPartTile : nnz;
  bool bad = false;
  // (the tile's loads are issued together: one trip instead of sixteen dependent ones)
  int64_t rows[kPartTile / kPartThreads], prev[kPartTile / kPartThreads];
#pragma unroll
  for (int i = 0; i < kPartTile / kPartThreads; i++) {
    const int64_t e = beg + (int64_t)i * kPartThreads + threadIdx.x;
    const int64_t ec = e < end ? e : end - 1;  // (end > beg: the grid has no empty tile)
    rows[i] = load_index(row_ind, ec, wide);
    prev[i] = load_index(row_ind, ec > 0 ? ec - 1 : 0, wide);
  }
#pragma unroll
  for (int i = 0; i < kPartTile / kPartThreads; i++) {
    const int64_t e = beg + (int64_t)i * kPartThreads + threadIdx.x;
    if (e < end) {
      const int64_t r = rows[i];
      if (r >= 0 && r < n_rows) atomicAdd(&cnt[r >> lo_bits], 1u);
      else bad = true;
      if (e > 0 && prev[i] > r) bad = true;
    }
  }
  if (bad) *flag = 1u;
  __syncthreads();
  for (int b = threadIdx.x; b < n_hi; b += kPartThreads) hist[(int64_t)b * n_tiles + blockIdx.x] = cnt[b];
}

// pass 1b: hist now holds exclusive prefixes.  The tile is first sorted by high digit inside LDS,
// then written out, so that the entries a tile sends to one bucket leave as one contiguous run
// of (row, col) pairs instead of as isolated 4-byte stores.
constexpr int kPartPerThread = kPartTile / kPartThreads;
constexpr size_t kPartScatterLds = (size_t)kPartTile * 8 + 3 * (size_t)kPartMaxBuckets * 4;

__global__ __launch_bounds__(kPartThreads) void coo_part_scatter_kernel(
    const void* row_ind, int wide, const uint32_t* col_ind, int64_t nnz, int64_t n_rows, int lo_bits,
    int n_hi, int64_t n_tiles, const uint32_t* flag, const uint32_t* hist, uint64_t* tmp_pairs,
    int col_bits, uint32_t col_max) {
  extern __shared__ __attribute__((aligned(16))) unsigned char part_lds[];
  uint64_t* stage = reinterpret_cast<uint64_t*>(part_lds);
  uint32_t* cnt = reinterpret_cast<uint32_t*>(part_lds + (size_t)kPartTile * 8);
  uint32_t* lstart = cnt + kPartMaxBuckets;
  uint32_t* gstart = lstart + kPartMaxBuckets;
  __shared__ uint32_t wave_sums[kPartThreads / kWave];
  if (!*flag) return;
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  for (int b = tid; b < n_hi; b += kPartThreads) {
    cnt[b] = 0;
    gstart[b] = hist[(int64_t)b * n_tiles + blockIdx.x];
  }
  __syncthreads();
  const int64_t beg = (int64_t)blockIdx.x * kPartTile;
  const int64_t end = beg + kPartTile < nnz ? beg + kPartTile : nnz;
  uint32_t rows[kPartPerThread], cols[kPartPerThread], rank[kPartPerThread];
#pragma unroll
  for (int i = 0; i < kPartPerThread; i++) {
    const int64_t e = beg + (int64_t)i * kPartThreads + tid;
    rows[i] = 0xffffffffu;  // dropped
    if (e < end) {
      const int64_t r = load_index(row_ind, e, wide);
      if (r >= 0 && r < n_rows) {
        rows[i] = (uint32_t)r;
        cols[i] = col_ind[e];
        rank[i] = atomicAdd(&cnt[r >> lo_bits], 1u);
      }
    }
  }
  __syncthreads();
  // exclusive scan of cnt -> lstart
  uint32_t carry = 0;
  for (int base = 0; base < n_hi; base += kPartThreads) {
    const int i = base + tid;
    const uint32_t x = i < n_hi ? cnt[i] : 0u;
    const uint32_t inc = wave_inclusive_scan(x, lane);
    if (lane == kWave - 1) wave_sums[wave] = inc;
    __syncthreads();
    uint32_t prefix = 0, total = 0;
#pragma unroll
    for (int w = 0; w < kPartThreads / kWave; w++) {
      const uint32_t sw = wave_sums[w];
      if (w < wave) prefix += sw;
      total += sw;
    }
    if (i < n_hi) lstart[i] = carry + prefix + inc - x;
    carry += total;
    __syncthreads();
  }
  const uint32_t kept = carry;
#pragma unroll
  for (int i = 0; i < kPartPerThread; i++) {
    if (rows[i] != 0xffffffffu)
      stage[lstart[rows[i] >> lo_bits] + rank[i]] = ((uint64_t)rows[i] << 32) | cols[i];
  }
  __syncthreads();
  if (col_bits > 0) {
    // (row inside the bucket, column) fit 32 bits: half the bytes to write here and to read in
    // pass 2; a column past the last key (masked later whatever its value) becomes col_max
    uint32_t* tmp_packed = reinterpret_cast<uint32_t*>(tmp_pairs);
    const uint32_t lo_mask = (1u << lo_bits) - 1u;
    for (uint32_t i = tid; i < kept; i += kPartThreads) {
      const uint64_t x = stage[i];
      const uint32_t row = (uint32_t)(x >> 32), col = (uint32_t)x;
      const uint32_t b = row >> lo_bits;
      tmp_packed[gstart[b] + (i - lstart[b])] = ((row & lo_mask) << col_bits) | (col < col_max ? col : col_max);
    }
    return;
  }
  for (uint32_t i = tid; i < kept; i += kPartThreads) {
    const uint64_t x = stage[i];
    const uint32_t b = (uint32_t)(x >> 32) >> lo_bits;
    tmp_pairs[gstart[b] + (i - lstart[b])] = x;
  }
}

// pass 2: one workgroup per high bucket; its (row, col) pairs are contiguous in tmp_pairs.
// Count the low digit in LDS, scan, emit the row offsets of the bucket's rows and place the
// columns.
constexpr int kPartRowsThreads = 1024;
constexpr int kPartKeep = 32;  // pairs per thread that pass 2 keeps in registers

// LDS counters under skew: a row that holds a large share of its bucket's entries (power-law
// masks) has most lanes of every wavefront adding to the same counter, which the LDS serialises
// lane by lane.  The lanes that share the key of the first lane not dealt with yet are counted
// with a ballot and added once; after kAggRounds such rounds the remaining lanes add one by one.
constexpr int kAggRounds = 2;

__device__ __forceinline__ int wave_lane() {
  return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

// cnt[key] += 1 for every lane with valid set
__device__ __forceinline__ void lds_count(uint32_t* cnt, uint32_t key, bool valid) {
  const int lane = wave_lane();
  uint64_t todo = __builtin_amdgcn_ballot_w64(valid);
#pragma unroll
  for (int round = 0; round < kAggRounds; round++) {
    if (todo == 0) break;
    const int leader = __builtin_ctzll(todo);
    const uint32_t k0 = (uint32_t)__builtin_amdgcn_readlane((int)key, leader);
    const uint64_t same = __builtin_amdgcn_ballot_w64(valid && key == k0) & todo;
    if (lane == leader) atomicAdd(&cnt[k0], (uint32_t)__builtin_popcountll(same));
    todo &= ~same;
  }
  if ((todo >> lane) & 1ull) atomicAdd(&cnt[key], 1u);
}

// the same, returning the counter's value before this lane's own increment (a distinct slot per
// lane): pos = atomicAdd(&cnt[key], 1)
__device__ __forceinline__ uint32_t lds_take_slot(uint32_t* cnt, uint32_t key, bool valid) {
  const int lane = wave_lane();
  uint64_t todo = __builtin_amdgcn_ballot_w64(valid);
  uint32_t pos = 0;
#pragma unroll
  for (int round = 0; round < kAggRounds; round++) {
    if (todo == 0) break;
    const int leader = __builtin_ctzll(todo);
    const uint32_t k0 = (uint32_t)__builtin_amdgcn_readlane((int)key, leader);
    const uint64_t same = __builtin_amdgcn_ballot_w64(valid && key == k0) & todo;
    uint32_t base = 0;
    if (lane == leader) base = atomicAdd(&cnt[k0], (uint32_t)__builtin_popcountll(same));
    base = (uint32_t)__builtin_amdgcn_readlane((int)base, leader);
    if ((same >> lane) & 1ull) pos = base + (uint32_t)__builtin_popcountll(same & ((1ull << lane) - 1ull));
    todo &= ~same;
  }
  if ((todo >> lane) & 1ull) pos = atomicAdd(&cnt[key], 1u);
  return pos;
}

// PACKED: the entries are 32-bit (row inside the bucket << col_bits | column).  A bucket of up to
// kPartKeep * kPartRowsThreads entries is then read once, all loads in flight together, and stays
// in registers between the count and the placement (32 registers; two workgroups share a CU).
// Larger buckets, and 64-bit (row, column) pairs, are walked twice, four loads in flight.
template <bool PACKED>
__global__ __launch_bounds__(kPartRowsThreads, PACKED ? 8 : 4) void coo_part_rows_kernel(
    int64_t n_rows, int lo_bits, int n_hi, int64_t n_tiles, int64_t n_hist, const uint32_t* flag,
    const uint32_t* hist, const uint64_t* tmp_pairs, uint32_t* row_off, uint32_t* cols_out, int col_bits) {
  __shared__ uint32_t cnt[kPartMaxBuckets];
  __shared__ uint32_t wave_sums[kPartRowsThreads / kWave];
  if (!*flag) return;
  const int b = blockIdx.x;
  const int n_lo = 1 << lo_bits;
  const uint32_t beg = hist[(int64_t)b * n_tiles];
  const uint32_t end = (b + 1 < n_hi) ? hist[(int64_t)(b + 1) * n_tiles] : hist[n_hist];
  for (int i = threadIdx.x; i < n_lo; i += kPartRowsThreads) cnt[i] = 0;
  __syncthreads();
  const uint32_t lo_mask = (uint32_t)n_lo - 1u;
  const uint32_t col_mask = PACKED ? (1u << col_bits) - 1u : 0xffffffffu;
  const uint32_t* tmp_packed = reinterpret_cast<const uint32_t*>(tmp_pairs);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  // entry e as (row inside the bucket, column)
  auto key_of = [&](uint64_t x) -> uint32_t {
    return PACKED ? (uint32_t)x >> col_bits : (uint32_t)(x >> 32) & lo_mask;
  };
  auto load_entry = [&](uint32_t e) -> uint64_t {
    if constexpr (PACKED) return tmp_packed[e];
    else return tmp_pairs[e];
  };
  // exclusive scan of cnt[0 .. n_lo) in place, kPartRowsThreads values at a time; the scanned
  // values are the row offsets of the bucket's rows and the cursors of the placement
  auto scan_counts = [&]() {
    uint32_t carry = beg;
    for (int base = 0; base < n_lo; base += kPartRowsThreads) {
      const int i = base + threadIdx.x;
      const uint32_t x = i < n_lo ? cnt[i] : 0u;
      const uint32_t inc = wave_inclusive_scan(x, lane);
      if (lane == kWave - 1) wave_sums[wave] = inc;
      __syncthreads();
      uint32_t prefix = 0, total = 0;
#pragma unroll
      for (int w = 0; w < kPartRowsThreads / kWave; w++) {
        const uint32_t sw = wave_sums[w];
        if (w < wave) prefix += sw;
        total += sw;
      }
      const uint32_t ex = carry + prefix + inc - x;
      if (i < n_lo) {
        cnt[i] = ex;  // becomes the cursor of this row
        const int64_t row = ((int64_t)b << lo_bits) + i;
        if (row < n_rows) row_off[row] = ex;
      }
      carry += total;
      __syncthreads();
    }
    if (b == n_hi - 1 && threadIdx.x == 0) row_off[n_rows] = end;
  };
  if constexpr (PACKED) {
    if (end - beg <= (uint32_t)(kPartKeep * kPartRowsThreads)) {
      if (end == beg) {
        scan_counts();  // (an empty bucket still owes its rows their offsets)
        return;
      }
      // (every load reads a valid entry: past the end, the bucket's last one, which is not counted)
      uint32_t x[kPartKeep];
      const uint32_t* bp = tmp_packed + beg;
      const uint32_t last = end - beg - 1;
#pragma unroll
      for (int i = 0; i < kPartKeep; i++) {
        const uint32_t e = i * kPartRowsThreads + threadIdx.x;
        x[i] = bp[e < last ? e : last];
      }
      // (a few entries at a time: with all of them unrolled into one stretch the slots that come
      // back from LDS pile up in registers beside the entries)
#pragma unroll
      for (int i = 0; i < kPartKeep; i++) {
        lds_count(cnt, x[i] >> col_bits, beg + i * kPartRowsThreads + threadIdx.x < end);
        if (i % 4 == 3) __builtin_amdgcn_sched_barrier(0);
      }
      __syncthreads();
      scan_counts();
#pragma unroll
      for (int i = 0; i < kPartKeep; i++) {
        const bool valid = beg + i * kPartRowsThreads + threadIdx.x < end;
        const uint32_t pos = lds_take_slot(cnt, x[i] >> col_bits, valid);
        if (valid) cols_out[pos] = x[i] & col_mask;
        if (i % 4 == 3) __builtin_amdgcn_sched_barrier(0);
      }
      return;
    }
  }
  constexpr uint32_t kStep = 4 * kPartRowsThreads;
  for (uint32_t e0 = beg; e0 < end; e0 += kStep) {
    uint64_t x[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t e = e0 + i * kPartRowsThreads + threadIdx.x;
      x[i] = e < end ? load_entry(e) : 0ull;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) lds_count(cnt, key_of(x[i]), e0 + i * kPartRowsThreads + threadIdx.x < end);
  }
  __syncthreads();
  scan_counts();
  for (uint32_t e0 = beg; e0 < end; e0 += kStep) {
    uint64_t x[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t e = e0 + i * kPartRowsThreads + threadIdx.x;
      x[i] = e < end ? load_entry(e) : 0ull;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const bool valid = e0 + i * kPartRowsThreads + threadIdx.x < end;
      const uint32_t pos = lds_take_slot(cnt, key_of(x[i]), valid);
      if (valid) cols_out[pos] = (uint32_t)x[i] & col_mask;
    }
  }
}

// one wavefront per row: lanes stride over the row's entries
__global__ __launch_bounds__(256) void csr_entry_list_kernel(const void* row_off, int off64,
                                                             const uint32_t* cols,
                                                             const uint32_t* alt_cols,
                                                             const uint32_t* use_alt, int64_t n_rows,
                                                             uint32_t* rows_out, uint32_t* cols_out) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t stride = (int64_t)gridDim.x * 4;
  const uint32_t* cp = (use_alt != nullptr && *use_alt != 0u) ? alt_cols : cols;
  for (int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); r < n_rows; r += stride) {
    const int64_t a = load_index(row_off, r, off64), b = load_index(row_off, r + 1, off64);
    for (int64_t e = a + lane; e < b; e += kWave) {
      rows_out[e] = (uint32_t)r;
      cols_out[e] = cp[e];
    }
  }
}

__global__ void coo_csr_export_kernel(const uint32_t* row_off, const uint32_t* bucketed,
                                      const uint32_t* given, const uint32_t* unsorted, int64_t n_rows,
                                      int64_t nnz, uint32_t* row_off_out, uint32_t* cols_out) {
  const uint32_t* src = *unsorted ? bucketed : given;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nnz + n_rows + 1; i += stride) {
    if (i < nnz) cols_out[i] = src[i];
    else row_off_out[i - nnz] = row_off[i - nnz];
  }
}

inline unsigned grid_for(int64_t n, int threads, int64_t cap) {
  int64_t g = (n + threads - 1) / threads;
  if (g > cap) g = cap;
  if (g < 1) g = 1;
  return (unsigned)g;
}

}  // namespace

CooWorkspace coo_workspace(int64_t n_rows, int64_t nnz) {
  CooWorkspace w{};
  int bits = 1;
  while (((int64_t)1 << bits) < n_rows) bits++;
  w.partition = (bits <= 22 && nnz > 0) ? 1 : 0;
  const int hi_bits = (bits + 1) / 2;
  w.lo_bits = bits - hi_bits;
  w.n_hi = ((n_rows > 0 ? n_rows : 1) + ((int64_t)1 << w.lo_bits) - 1) >> w.lo_bits;
  w.n_tiles1 = (nnz + kPartTile - 1) / kPartTile;
  const int64_t n_hist = w.partition ? w.n_hi * w.n_tiles1 : 0;
  const int64_t scan_len = n_hist > n_rows ? n_hist : n_rows;
  const int64_t n_tiles = (scan_len + kScanTile - 1) / kScanTile + 1;
  size_t off = 0;
  w.off_row_off = off; off = align_up(off + (size_t)(n_rows + 1) * 4, 256);
  w.off_cols = off;    off = align_up(off + (size_t)(nnz > 0 ? nnz : 1) * 4, 256);
  w.off_flag = off;    off = align_up(off + 4, 256);
  w.keep_total = off;
  w.off_counts = off;  off = align_up(off + (size_t)(n_rows + 1) * 4, 256);
  w.off_cursor = off;  off = align_up(off + (size_t)(n_rows + 1) * 4, 256);
  w.off_tiles = off;   off = align_up(off + (size_t)n_tiles * 4, 256);
  w.off_hist = off;    off = align_up(off + (size_t)(n_hist + 1) * 4, 256);
  w.off_tmp_pairs = off; off = align_up(off + (size_t)(w.partition ? nnz : 0) * 8, 256);
  w.total = off;
  return w;
}

int coo_to_csr(const void* row_ind, int row_wide, const uint32_t* col_ind, int64_t nnz,
               int64_t n_rows, int64_t n_cols, void* keep, void* scratch, hipStream_t stream, CooCsr* out) {
  CooWorkspace w = coo_workspace(n_rows, nnz);
  char* kbase = (char*)keep;
  char* base = (char*)scratch - w.keep_total;  // scratch offsets are counted from the start of keep
  uint32_t* counts = (uint32_t*)(base + w.off_counts);
  uint32_t* row_off = (uint32_t*)(kbase + w.off_row_off);
  uint32_t* cursor = (uint32_t*)(base + w.off_cursor);
  uint32_t* tiles = (uint32_t*)(base + w.off_tiles);
  uint32_t* cols = (uint32_t*)(kbase + w.off_cols);
  uint32_t* flag = (uint32_t*)(kbase + w.off_flag);
  const int64_t n_tiles = (n_rows + kScanTile - 1) / kScanTile;

  hipLaunchKernelGGL(fill_u32_kernel, dim3(grid_for(n_rows + 1, 256, 4096)), dim3(256), 0, stream,
                     counts, n_rows + 1, 0u);
  hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(64), 0, stream, flag, (int64_t)1, 0u);
  // sorted or not: decided on the device (by the first pass of the partition where there is one)
  const bool part = nnz > 0 && w.partition;
  if (part)
    hipLaunchKernelGGL(coo_part_count_kernel, dim3((unsigned)w.n_tiles1), dim3(kPartThreads), 0, stream,
                       row_ind, row_wide, nnz, n_rows, w.lo_bits, (int)w.n_hi, w.n_tiles1, flag,
                       (uint32_t*)(base + w.off_hist));
  else if (nnz > 0)
    hipLaunchKernelGGL(coo_check_sorted_kernel, dim3(grid_for(nnz, 256, 8192)), dim3(256), 0, stream,
                       row_ind, row_wide, nnz, n_rows, flag);
  // sorted: offsets straight from the row array
  hipLaunchKernelGGL(coo_sorted_offsets_kernel, dim3(grid_for(nnz + 1, 256, 16384)), dim3(256), 0,
                     stream, row_ind, row_wide, nnz, n_rows, flag, row_off);
  // unsorted: bucket by row
  if (part) {
    uint32_t* hist = (uint32_t*)(base + w.off_hist);
    uint64_t* tmp_pairs = (uint64_t*)(base + w.off_tmp_pairs);
    // 152 KB of LDS per workgroup: above the 64 KB a kernel gets without asking (set once per
    // device: the attribute belongs to the device's copy of the kernel)
    constexpr int kMaxDevices = 64;
    static bool lds_attr_set[kMaxDevices];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 4;
    if (dev < 0 || dev >= kMaxDevices || !lds_attr_set[dev]) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(coo_part_scatter_kernel),
                              hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)kPartScatterLds) != hipSuccess)
        return 4;
      if (dev >= 0 && dev < kMaxDevices) lds_attr_set[dev] = true;
    }
    const int64_t n_hist = w.n_hi * w.n_tiles1;
    const int64_t hist_tiles = (n_hist + kScanTile - 1) / kScanTile;
    hipLaunchKernelGGL(scan_tile_sums_kernel, dim3((unsigned)hist_tiles), dim3(kScanThreads), 0, stream,
                       hist, n_hist, tiles, flag);
    hipLaunchKernelGGL(scan_sums_kernel, dim3(1), dim3(kScanThreads), 0, stream, tiles, hist_tiles, flag);
    hipLaunchKernelGGL(scan_apply_kernel, dim3((unsigned)hist_tiles), dim3(kScanThreads), 0, stream,
                       hist, n_hist, tiles, hist, hist, flag);
    // 32-bit entries between the passes when the columns leave room for the row inside its bucket
    // (n_cols known and n_cols < 2^(32 - lo_bits)); columns >= n_cols are stored as n_cols
    int col_bits = 0;
    if (n_cols > 0) {
      int need = 1;
      while (need < 32 && ((int64_t)1 << need) <= n_cols) need++;  // n_cols itself must fit
      if (need + w.lo_bits <= 32) col_bits = need;
    }
    hipLaunchKernelGGL(coo_part_scatter_kernel, dim3((unsigned)w.n_tiles1), dim3(kPartThreads),
                       kPartScatterLds, stream, row_ind, row_wide, col_ind, nnz, n_rows, w.lo_bits,
                       (int)w.n_hi, w.n_tiles1, flag, hist, tmp_pairs, col_bits, (uint32_t)(col_bits ? n_cols : 0));
    if (col_bits)
      hipLaunchKernelGGL(coo_part_rows_kernel<true>, dim3((unsigned)w.n_hi), dim3(kPartRowsThreads), 0, stream,
                         n_rows, w.lo_bits, (int)w.n_hi, w.n_tiles1, n_hist, flag, hist, tmp_pairs, row_off,
                         cols, col_bits);
    else
      hipLaunchKernelGGL(coo_part_rows_kernel<false>, dim3((unsigned)w.n_hi), dim3(kPartRowsThreads), 0, stream,
                         n_rows, w.lo_bits, (int)w.n_hi, w.n_tiles1, n_hist, flag, hist, tmp_pairs, row_off,
                         cols, 0);
  } else if (nnz > 0) {
    hipLaunchKernelGGL(coo_histogram_kernel, dim3(grid_for(nnz, 256, 16384)), dim3(256), 0, stream,
                       row_ind, row_wide, nnz, n_rows, flag, counts);
    hipLaunchKernelGGL(scan_tile_sums_kernel, dim3((unsigned)n_tiles), dim3(kScanThreads), 0, stream,
                       counts, n_rows, tiles, flag);
    hipLaunchKernelGGL(scan_sums_kernel, dim3(1), dim3(kScanThreads), 0, stream, tiles, n_tiles, flag);
    hipLaunchKernelGGL(scan_apply_kernel, dim3((unsigned)n_tiles), dim3(kScanThreads), 0, stream,
                       counts, n_rows, tiles, row_off, cursor, flag);
    hipLaunchKernelGGL(coo_scatter_kernel, dim3(grid_for(nnz, 256, 16384)), dim3(256), 0, stream,
                       row_ind, row_wide, col_ind, nnz, n_rows, flag, cursor, cols);
  }
  out->row_off = row_off;
  out->cols = cols;
  out->unsorted = flag;
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

int csr_entry_list(const void* row_off, int off64, const uint32_t* cols, const uint32_t* alt_cols,
                   const uint32_t* use_alt, int64_t n_rows, uint32_t* rows_out, uint32_t* cols_out,
                   hipStream_t stream) {
  if (n_rows <= 0) return 0;
  hipLaunchKernelGGL(csr_entry_list_kernel, dim3(grid_for(n_rows, 4, 1 << 20)), dim3(256), 0, stream,
                     row_off, off64, cols, alt_cols, use_alt, n_rows, rows_out, cols_out);
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

int coo_csr_export(const CooCsr& csr, const uint32_t* given_cols, int64_t n_rows, int64_t nnz,
                   uint32_t* row_off_out, uint32_t* cols_out, hipStream_t stream) {
  hipLaunchKernelGGL(coo_csr_export_kernel, dim3(grid_for(nnz + n_rows + 1, 256, 16384)), dim3(256), 0,
                     stream, csr.row_off, csr.cols, given_cols, csr.unsorted, n_rows, nnz, row_off_out,
                     cols_out);
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

int prepare_global_rows(const int32_t* globs, int64_t n_globs, int64_t n, uint32_t* bits,
                        int32_t* uq, hipStream_t stream) {
  const int64_t words = (int64_t)global_bits_words(n);
  hipLaunchKernelGGL(fill_u32_kernel, dim3(grid_for(words, 256, 4096)), dim3(256), 0, stream, bits,
                     words, 0u);
  hipLaunchKernelGGL(mark_globals_kernel, dim3(grid_for(n_globs, 256, 1 << 30)), dim3(256), 0,
                     stream, globs, n_globs, n, bits, bits + (words - 1), uq);
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

}  // namespace spfa
