// Mask pre-passes that run on the device before the attention kernels:
//   - COO entries -> row buckets (histogram, exclusive scan, scatter), any entry order;
//   - global-token list -> per-row flag bytes.
#include <atomic>
#include "spfa_prep.hpp"

#include <type_traits>

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
// The kernels of pass 1 take the row type as a template argument: a run-time choice between a
// 32-bit and a 64-bit load puts a branch, and with it a wait for the data, between every two
// loads of a thread, and the sixteen loads of a thread become sixteen round trips.
constexpr int kPartPerThread = kPartTile / kPartThreads;
constexpr uint32_t kPartBadRow = 0xffffffffu;  // a row outside [0, n_rows)

// Tile of a workgroup of pass 1.  Workgroups go to the 8 XCDs in turn, each with an L2 of its
// own; a tile's stores land next to those of the tiles before and after it (hist[b][tile - 1],
// hist[b][tile + 1]; the runs of one bucket), so consecutive tiles go to one XCD, where the
// partly written lines meet in one L2 (measured at 50 M entries: scatter 231 -> 200 us, count
// 100 -> 91 us).  The grid is padded to a multiple of 8; tiles past the last return at once.
constexpr int kXcds = 8;
__device__ __forceinline__ int64_t part_tile_of_block(int64_t n_tiles) {
  const int64_t per_xcd = (n_tiles + kXcds - 1) / kXcds;
  return (int64_t)(blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds;
}
inline unsigned part_grid(int64_t n_tiles) { return (unsigned)((n_tiles + kXcds - 1) / kXcds * kXcds); }

template <typename RowT>
__global__ __launch_bounds__(kPartThreads, 8) void coo_part_count_kernel(
    const RowT* row_ind, int64_t nnz, int64_t n_rows, int lo_bits, int n_hi, int64_t n_tiles,
    uint32_t* flag, uint32_t* hist) {
  __shared__ uint32_t cnt[kPartMaxBuckets];
  __shared__ uint32_t last_of[kPartPerThread][kPartThreads / kWave];
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int64_t tile = part_tile_of_block(n_tiles);
  if (tile >= n_tiles) return;
  for (int b = tid; b < n_hi; b += kPartThreads) cnt[b] = 0;
  const int64_t beg = tile * kPartTile;
  const uint32_t n_tile = (uint32_t)(nnz - beg < kPartTile ? nnz - beg : kPartTile);  // (> 0)
  const RowT* rp = row_ind + beg;
  RowT raw[kPartPerThread];
#pragma unroll
  for (int i = 0; i < kPartPerThread; i++) {
    const uint32_t idx = (uint32_t)(i * kPartThreads + tid);
    raw[i] = rp[idx < n_tile ? idx : n_tile - 1];
  }
  // the row of the entry before the tile (thread 0 compares its first entry with it)
  uint32_t before = 0;
  if (tid == 0 && beg > 0) {
    const RowT pr = rp[-1];
    before = pr < (RowT)n_rows ? (uint32_t)pr : kPartBadRow;
  }
  uint32_t row[kPartPerThread];
#pragma unroll
  for (int i = 0; i < kPartPerThread; i++) {
    row[i] = raw[i] < (RowT)n_rows ? (uint32_t)raw[i] : kPartBadRow;
    if (lane == kWave - 1) last_of[i][wave] = row[i];
  }
  __syncthreads();
  // entry idx follows entry idx - 1: the lane before, the last lane of the wavefront before, or
  // the last thread's previous entry
  bool bad = false;
#pragma unroll
  for (int i = 0; i < kPartPerThread; i++) {
    const uint32_t idx = (uint32_t)(i * kPartThreads + tid);
    uint32_t prev = (uint32_t)__builtin_amdgcn_ds_bpermute(((lane - 1) & 63) << 2, (int)row[i]);
    if (lane == 0) prev = wave > 0 ? last_of[i][wave - 1] : i > 0 ? last_of[i > 0 ? i - 1 : 0][kPartThreads / kWave - 1] : before;
    if (idx < n_tile) {
      if (row[i] == kPartBadRow) bad = true;
      else atomicAdd(&cnt[row[i] >> lo_bits], 1u);
      if (prev > row[i]) bad = true;  // (a bad row before this one has raised the flag already)
    }
  }
  if (bad) *flag = 1u;
  __syncthreads();
  for (int b = tid; b < n_hi; b += kPartThreads) hist[(int64_t)b * n_tiles + tile] = cnt[b];
}

// pass 1b: hist now holds exclusive prefixes.  The tile is first sorted by high digit inside LDS,
// then written out, so that the entries a tile sends to one bucket leave as one contiguous run
// of (row, col) pairs instead of as isolated 4-byte stores.
constexpr size_t kPartScatterLds = (size_t)kPartTile * 8 + 3 * (size_t)kPartMaxBuckets * 4;

template <typename RowT>
__global__ __launch_bounds__(kPartThreads) void coo_part_scatter_kernel(
    const RowT* row_ind, const uint32_t* col_ind, int64_t nnz, int64_t n_rows, int lo_bits,
    int n_hi, int64_t n_tiles, const uint32_t* flag, const uint32_t* hist, uint64_t* tmp_pairs) {
  extern __shared__ __attribute__((aligned(16))) unsigned char part_lds[];
  uint64_t* stage = reinterpret_cast<uint64_t*>(part_lds);
  uint32_t* cnt = reinterpret_cast<uint32_t*>(part_lds + (size_t)kPartTile * 8);
  uint32_t* lstart = cnt + kPartMaxBuckets;
  uint32_t* gstart = lstart + kPartMaxBuckets;
  __shared__ uint32_t wave_sums[kPartThreads / kWave];
  if (!*flag) return;
  const int64_t tile = part_tile_of_block(n_tiles);
  if (tile >= n_tiles) return;
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  for (int b = tid; b < n_hi; b += kPartThreads) {
    cnt[b] = 0;
    gstart[b] = hist[(int64_t)b * n_tiles + tile];
  }
  __syncthreads();
  const int64_t beg = tile * kPartTile;
  const uint32_t n_tile = (uint32_t)(nnz - beg < kPartTile ? nnz - beg : kPartTile);  // (> 0)
  const RowT* rp = row_ind + beg;
  const uint32_t* cp = col_ind + beg;
  RowT raw[kPartPerThread];
  uint32_t rows[kPartPerThread], cols[kPartPerThread], rank[kPartPerThread];
#pragma unroll
  for (int i = 0; i < kPartPerThread; i++) {
    const uint32_t idx = (uint32_t)(i * kPartThreads + tid);
    raw[i] = rp[idx < n_tile ? idx : n_tile - 1];
    cols[i] = cp[idx < n_tile ? idx : n_tile - 1];
  }
#pragma unroll
  for (int i = 0; i < kPartPerThread; i++) {
    const uint32_t idx = (uint32_t)(i * kPartThreads + tid);
    rows[i] = kPartBadRow;  // dropped
    if (idx < n_tile && raw[i] < (RowT)n_rows) {
      rows[i] = (uint32_t)raw[i];
      rank[i] = atomicAdd(&cnt[rows[i] >> lo_bits], 1u);
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
    if (rows[i] != kPartBadRow)
      stage[lstart[rows[i] >> lo_bits] + rank[i]] = ((uint64_t)rows[i] << 32) | cols[i];
  }
  __syncthreads();
  for (uint32_t i = tid; i < kept; i += kPartThreads) {
    const uint64_t x = stage[i];
    const uint32_t b = (uint32_t)(x >> 32) >> lo_bits;
    tmp_pairs[gstart[b] + (i - lstart[b])] = x;
  }
}

// pass 1b when an entry leaves as one 32-bit word (row inside the bucket << col_bits | column;
// a column past the last key, masked later whatever its value, becomes col_max): half the bytes to
// write here and to read in pass 2, and a staged tile of 64 KB, so that two workgroups share a CU
// (up to 1024 buckets; one with 2048) and one loads while the other sorts.  Where the tile's entries of a bucket go inside the staged
// tile follows from the scanned histogram alone (the tile's count of bucket b is the distance to
// the next element of hist), so an entry is staged as soon as it is loaded and nothing is kept in
// registers across a barrier.  The staged words no longer say which bucket they belong to, so
// the tile leaves bucket by bucket: a group of 16 lanes copies the run of one bucket (16 entries
// on average); runs of more than kPartLongRun entries are left to the whole workgroup.
constexpr int kPartLongRun = 256;
constexpr int kPartMaxLongRuns = kPartTile / kPartLongRun;

inline size_t part_scatter_packed_lds(int64_t n_hi) { return (size_t)kPartTile * 4 + 2 * (size_t)n_hi * 4; }

template <typename RowT>
__global__ __launch_bounds__(kPartThreads, 8) void coo_part_scatter_packed_kernel(
    const RowT* row_ind, const uint32_t* col_ind, int64_t nnz, int64_t n_rows, int lo_bits,
    int n_hi, int64_t n_tiles, const uint32_t* flag, const uint32_t* hist, uint32_t* tmp_packed,
    int col_bits, uint32_t col_max) {
  extern __shared__ __attribute__((aligned(16))) uint32_t packed_lds[];
  uint32_t* stage = packed_lds;              // kPartTile words
  uint32_t* cursor = packed_lds + kPartTile;  // n_hi: next free staged position of each bucket
  uint32_t* gstart = cursor + n_hi;           // n_hi: where the tile's run of each bucket goes
  __shared__ uint32_t wave_sums[kPartThreads / kWave];
  __shared__ uint32_t long_runs[kPartMaxLongRuns];
  __shared__ uint32_t n_long;
  if (!*flag) return;
  const int64_t tile = part_tile_of_block(n_tiles);
  if (tile >= n_tiles) return;
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  if (tid == 0) n_long = 0;
  const int64_t beg = tile * kPartTile;
  const uint32_t n_tile = (uint32_t)(nnz - beg < kPartTile ? nnz - beg : kPartTile);  // (> 0)
  const RowT* rp = row_ind + beg;
  const uint32_t* cp = col_ind + beg;
  const uint32_t lo_mask = (1u << lo_bits) - 1u;
  // (half of the thread's entries at a time: 64 registers)
  constexpr int kHalf = kPartPerThread / 2;
  RowT r[kHalf];
  uint32_t c[kHalf];
  auto load_half = [&](int h) {
#pragma unroll
    for (int i = 0; i < kHalf; i++) {
      const uint32_t idx = (uint32_t)((h * kHalf + i) * kPartThreads + tid);
      r[i] = rp[idx < n_tile ? idx : n_tile - 1];
      c[i] = cp[idx < n_tile ? idx : n_tile - 1];
    }
  };
  auto stage_half = [&](int h) {
#pragma unroll
    for (int i = 0; i < kHalf; i++) {
      const uint32_t idx = (uint32_t)((h * kHalf + i) * kPartThreads + tid);
      if (idx < n_tile && r[i] < (RowT)n_rows) {
        const uint32_t row = (uint32_t)r[i];
        stage[atomicAdd(&cursor[row >> lo_bits], 1u)] =
            ((row & lo_mask) << col_bits) | (c[i] < col_max ? c[i] : col_max);
      }
    }
  };
  // cursor[b] = number of entries the tile holds of the buckets before b
  uint32_t carry = 0;
  for (int base = 0; base < n_hi; base += kPartThreads) {
    const int i = base + tid;
    uint32_t x = 0;
    if (i < n_hi) {
      const uint32_t* h = hist + (int64_t)i * n_tiles + tile;
      const uint32_t h0 = h[0];
      x = h[1] - h0;
      gstart[i] = h0;
    }
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
    if (i < n_hi) {
      cursor[i] = carry + prefix + inc - x;
      if (x > (uint32_t)kPartLongRun) long_runs[atomicAdd(&n_long, 1u)] = (uint32_t)i;
    }
    carry += total;
    __syncthreads();
  }
  load_half(0);
  stage_half(0);
  load_half(1);
  stage_half(1);
  __syncthreads();
  // (cursor[b] is now the end of bucket b's run, and the start of the next bucket's)
  // short runs: bucket b to the 16-lane group b % 64 of the workgroup
  constexpr int kRunLanes = 16;  // (measured: 8 lanes 254 us, 16 lanes 245 us, 32 lanes 272 us at 50 M entries)
  const int group = tid / kRunLanes, sub = tid % kRunLanes;
  for (int b = group; b < n_hi; b += kPartThreads / kRunLanes) {
    const uint32_t s = b > 0 ? cursor[b - 1] : 0u, n = cursor[b] - s;
    if (n == 0 || n > (uint32_t)kPartLongRun) continue;
    uint32_t* out = tmp_packed + gstart[b];
    for (uint32_t j = sub; j < n; j += kRunLanes) out[j] = stage[s + j];
  }
  const uint32_t longs = n_long;
  for (uint32_t q = 0; q < longs; q++) {
    const int b = (int)long_runs[q];
    const uint32_t s = b > 0 ? cursor[b - 1] : 0u, n = cursor[b] - s;
    uint32_t* out = tmp_packed + gstart[b];
    for (uint32_t j = tid; j < n; j += kPartThreads) out[j] = stage[s + j];
  }
}

// pass 2: one workgroup per high bucket; its (row, col) pairs are contiguous in tmp_pairs.
// Count the low digit in LDS, scan, emit the row offsets of the bucket's rows and place the
// columns.
constexpr int kPartRowsThreads = 1024;
constexpr int kPartKeep = 64;        // entries per thread that pass 2 keeps in registers
constexpr int kPartWindow = 36864;   // positions of a bucket's output staged in LDS at a time
constexpr int kPartMaxWindows = 8;
constexpr size_t kPartRowsLds = (size_t)kPartWindow * 4;

// LDS counters under skew: when one row holds most of its bucket's entries, most lanes of every
// wavefront add to the same counter, which the LDS serialises lane by lane.  With ROUNDS > 0 the
// lanes that share the key of the first lane not dealt with yet are counted with a ballot and
// added once; after ROUNDS such rounds the remaining lanes add one by one.  The rounds cost about
// forty dependent instructions per 64 entries, more than the serialised adds of a mask whose rows
// hold up to a tenth of a bucket each (measured, 20 M entries in 1024 buckets: rows of 20 entries
// 89 against 159 us with two rounds, rows of 20000 entries 142 against 191 us; a quarter of all
// entries in one row 8.4 against 3.0 ms), so only a bucket that a sample shows to be dominated by
// one row takes them.
constexpr int kAggRounds = 2;
constexpr int kAggSampleLanes = 16;  // lanes of a wavefront on one key that make a bucket "skewed"

// number of set bits of `mask` below this lane
__device__ __forceinline__ uint32_t bits_below_lane(uint64_t mask) {
  return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

// cnt[key] += 1 for every lane with valid set
template <int ROUNDS>
__device__ __forceinline__ void lds_count(uint32_t* cnt, uint32_t key, bool valid) {
  bool pending = valid;
#pragma unroll
  for (int round = 0; round < ROUNDS; round++) {
    const uint64_t todo = __builtin_amdgcn_ballot_w64(pending);
    if (todo == 0) break;
    const uint32_t k0 = (uint32_t)__builtin_amdgcn_readlane((int)key, __builtin_ctzll(todo));
    const bool hit = pending && key == k0;
    const uint64_t same = __builtin_amdgcn_ballot_w64(hit);
    // (the lowest lane of `same` is the leader)
    if (hit && bits_below_lane(same) == 0) atomicAdd(&cnt[k0], (uint32_t)__builtin_popcountll(same));
    pending = pending && !hit;
  }
  if (pending) atomicAdd(&cnt[key], 1u);
}

// the same, returning the counter's value before this lane's own increment (a distinct slot per
// lane): pos = atomicAdd(&cnt[key], 1)
template <int ROUNDS>
__device__ __forceinline__ uint32_t lds_take_slot(uint32_t* cnt, uint32_t key, bool valid) {
  bool pending = valid;
  uint32_t pos = 0;
#pragma unroll
  for (int round = 0; round < ROUNDS; round++) {
    const uint64_t todo = __builtin_amdgcn_ballot_w64(pending);
    if (todo == 0) break;
    const int leader = __builtin_ctzll(todo);
    const uint32_t k0 = (uint32_t)__builtin_amdgcn_readlane((int)key, leader);
    const bool hit = pending && key == k0;
    const uint64_t same = __builtin_amdgcn_ballot_w64(hit);
    const uint32_t below = bits_below_lane(same);
    uint32_t base = 0;
    if (hit && below == 0) base = atomicAdd(&cnt[k0], (uint32_t)__builtin_popcountll(same));
    base = (uint32_t)__builtin_amdgcn_readlane((int)base, leader);
    if (hit) pos = base + below;
    pending = pending && !hit;
  }
  if (pending) pos = atomicAdd(&cnt[key], 1u);
  return pos;
}

// PACKED: the entries are 32-bit (row inside the bucket << col_bits | column).  The first
// kPartKeep * kPartRowsThreads of them are read once, all loads in flight together, and stay in
// registers from the count to the placement; what a larger bucket holds beyond them is walked
// again from memory.  The columns do not leave as isolated 4-byte stores (one memory request
// each: 50 M of them take longer than everything else in this kernel): the bucket's output is
// cut into windows of kPartWindow positions, a window takes the rows that start inside it, their
// columns are placed in LDS and leave as contiguous runs.  The tail of a row that runs past its
// window's end is stored directly.  Buckets of more than kPartMaxWindows windows, and 64-bit
// (row, column) pairs, are walked twice with direct stores.
// (One workgroup per CU: the staged window and 64 entries per thread in 128 registers.)
template <bool PACKED>
__global__ __launch_bounds__(kPartRowsThreads, 4) void coo_part_rows_kernel(
    int64_t n_rows, int lo_bits, int n_hi, int64_t n_tiles, int64_t n_hist, const uint32_t* flag,
    const uint32_t* hist, const uint64_t* tmp_pairs, uint32_t* row_off, uint32_t* cols_out, int col_bits) {
  extern __shared__ __attribute__((aligned(16))) uint32_t rows_stage[];  // PACKED: kPartWindow words
  __shared__ uint32_t cnt[kPartMaxBuckets];
  __shared__ uint32_t wave_sums[kPartRowsThreads / kWave];
  __shared__ uint32_t win_row[kPartMaxWindows + 1], win_pos[kPartMaxWindows + 1];
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
  constexpr uint32_t kStep = 4 * kPartRowsThreads;
  if constexpr (PACKED) {
    const uint32_t size = end - beg;
    if (size == 0) {
      scan_counts();  // (an empty bucket still owes its rows their offsets)
      return;
    }
    constexpr uint32_t kKept = (uint32_t)kPartKeep * kPartRowsThreads;
    constexpr uint32_t kWin = (uint32_t)kPartWindow;
    if (size <= kWin * (uint32_t)kPartMaxWindows) {
      const uint32_t n_win = (size + kWin - 1) / kWin;
      const uint32_t kept = size < kKept ? size : kKept;
      // This thread keeps the entries threadIdx.x + i * kPartRowsThreads, i < n_mine.  (The loads
      // are not clamped to the bucket, so that they need no register per address: the buffer is
      // padded by what a bucket's loads can run past its end; what they read there is not used.)
      uint32_t x[kPartKeep];
      const uint32_t* bp = tmp_packed + beg;
      const uint32_t n_mine = threadIdx.x < kept ? (kept - threadIdx.x + kPartRowsThreads - 1) / kPartRowsThreads : 0u;
#pragma unroll
      for (int i = 0; i < kPartKeep; i++) x[i] = bp[i * kPartRowsThreads + threadIdx.x];
#pragma unroll
      for (int i = 0; i < kPartKeep; i++) {
        lds_count<0>(cnt, x[i] >> col_bits, (uint32_t)i < n_mine);
        if (i % 4 == 3) __builtin_amdgcn_sched_barrier(0);
      }
      for (uint32_t e0 = kKept; e0 < size; e0 += kStep) {
        uint32_t y[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const uint32_t e = e0 + i * kPartRowsThreads + threadIdx.x;
          y[i] = bp[e < size ? e : size - 1];
        }
#pragma unroll
        for (int i = 0; i < 4; i++) lds_count<0>(cnt, y[i] >> col_bits, e0 + i * kPartRowsThreads + threadIdx.x < size);
      }
      __syncthreads();
      scan_counts();
      // window k takes the rows [win_row[k], win_row[k + 1]): those whose first position lies in
      // [k * kWin, (k + 1) * kWin); win_pos[k] is the first position of row win_row[k]
      for (int i = threadIdx.x; i < n_lo; i += kPartRowsThreads) {
        const uint32_t start = cnt[i] - beg;
        uint32_t wi = start / kWin;
        if (wi > n_win) wi = n_win;
        uint32_t k = i > 0 ? (cnt[i - 1] - beg) / kWin + 1 : 0u;
        for (; k <= wi; k++) {
          win_row[k] = (uint32_t)i;
          win_pos[k] = start;
        }
        if (i == n_lo - 1)
          for (k = wi + 1; k <= n_win; k++) {
            win_row[k] = (uint32_t)n_lo;
            win_pos[k] = size;
          }
      }
      __syncthreads();
      uint32_t* outp = cols_out + beg;
      for (uint32_t k = 0; k < n_win; k++) {
        const uint32_t first = win_row[k], n_in = win_row[k + 1] - first;
        if (n_in == 0) continue;  // (the same for every thread)
        const uint32_t lo = k * kWin;
        // (the entries and their number are made opaque in every trip, or the compiler keeps the
        // 64 row numbers and the 64 validity masks of the trip-invariant part in registers)
        uint32_t n_mine_k = n_mine;
        asm volatile("" : "+v"(n_mine_k));
#pragma unroll
        for (int i = 0; i < kPartKeep; i++) {
          uint32_t xi = x[i];
          asm volatile("" : "+v"(xi));
          const uint32_t r = xi >> col_bits;
          const bool in = (uint32_t)i < n_mine_k && r - first < n_in;
          const uint32_t pos = lds_take_slot<0>(cnt, r, in) - beg;
          if (in) {
            if (pos - lo < kWin) rows_stage[pos - lo] = xi & col_mask;
            else outp[pos] = xi & col_mask;
          }
          if (i % 4 == 3) __builtin_amdgcn_sched_barrier(0);
        }
        for (uint32_t e0 = kKept; e0 < size; e0 += kStep) {
          uint32_t y[4];
#pragma unroll
          for (int i = 0; i < 4; i++) {
            const uint32_t e = e0 + i * kPartRowsThreads + threadIdx.x;
            y[i] = bp[e < size ? e : size - 1];
          }
#pragma unroll
          for (int i = 0; i < 4; i++) {
            const uint32_t r = y[i] >> col_bits;
            const bool in = e0 + i * kPartRowsThreads + threadIdx.x < size && r - first < n_in;
            const uint32_t pos = lds_take_slot<0>(cnt, r, in) - beg;
            if (in) {
              if (pos - lo < kWin) rows_stage[pos - lo] = y[i] & col_mask;
              else outp[pos] = y[i] & col_mask;
            }
          }
        }
        __syncthreads();
        const uint32_t stop = win_pos[k + 1] < lo + kWin ? win_pos[k + 1] : lo + kWin;
        for (uint32_t p = win_pos[k] + threadIdx.x; p < stop; p += kPartRowsThreads) outp[p] = rows_stage[p - lo];
        __syncthreads();
      }
      return;
    }
  }
  // the bucket's first entries as a sample: is one row on a quarter of a wavefront's lanes?
  bool heavy = false;
  {
    const uint32_t e = beg + threadIdx.x;
    const bool valid = e < end;
    const uint32_t key = valid ? key_of(load_entry(e)) : 0u;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const uint32_t k0 = (uint32_t)__builtin_amdgcn_readlane((int)key, 16 * j);
      heavy |= __builtin_popcountll(__builtin_amdgcn_ballot_w64(valid && key == k0)) >= kAggSampleLanes;
    }
  }
  const bool skewed = __syncthreads_or(heavy) != 0;
  auto count_all = [&](auto rounds) {
    for (uint32_t e0 = beg; e0 < end; e0 += kStep) {
      uint64_t x[4];
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const uint32_t e = e0 + i * kPartRowsThreads + threadIdx.x;
        x[i] = e < end ? load_entry(e) : 0ull;
      }
#pragma unroll
      for (int i = 0; i < 4; i++)
        lds_count<decltype(rounds)::value>(cnt, key_of(x[i]), e0 + i * kPartRowsThreads + threadIdx.x < end);
    }
  };
  auto place_all = [&](auto rounds) {
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
        const uint32_t pos = lds_take_slot<decltype(rounds)::value>(cnt, key_of(x[i]), valid);
        if (valid) cols_out[pos] = (uint32_t)x[i] & col_mask;
      }
    }
  };
  if (skewed) count_all(std::integral_constant<int, kAggRounds>{});
  else count_all(std::integral_constant<int, 0>{});
  __syncthreads();
  scan_counts();
  if (skewed) place_all(std::integral_constant<int, kAggRounds>{});
  else place_all(std::integral_constant<int, 0>{});
}

// Row offset `r` of a CSR mask held to [0, nnz] (nnz < 2^32).
__device__ __forceinline__ uint32_t held_offset(const void* row_off, int64_t r, int off64, int64_t nnz) {
  int64_t v = load_index(row_off, r, off64);
  v = v < 0 ? 0 : v;
  return (uint32_t)(v > nnz ? nnz : v);
}

// How many of the offsets [lo, hi) are at or below x, plus lo, for offsets in ascending order
// (all of those before lo are taken to be at or below x).  The wavefront searches together: every
// lane looks at one of 64 evenly spaced offsets per round, so 2^17 offsets take three dependent
// loads where a bisection takes seventeen.  Offsets in any other order give some value in
// [lo, hi].
__device__ __forceinline__ int64_t wave_offsets_at_or_below(const void* row_off, int off64, int64_t nnz,
                                                            int64_t lo, int64_t hi, uint32_t x, int lane) {
  while (lo < hi) {
    const int64_t step = (hi - lo + kWave - 1) / kWave;
    const int64_t r = lo + (int64_t)lane * step;
    const bool below = r < hi && held_offset(row_off, r, off64, nnz) <= x;
    const uint64_t not_below = ~__ballot(below);
    const int k = not_below == 0 ? kWave : __builtin_ctzll(not_below);
    if (k == 0) break;
    const int64_t next_hi = lo + (int64_t)k * step;
    lo += (int64_t)(k - 1) * step + 1;
    hi = next_hi < hi ? next_hi : hi;
  }
  return lo;
}

constexpr int kEntryListInFlight = 8;
constexpr int kEntryListChunk = 4 * kEntryListInFlight * kWave;

// (row, column) of every entry of a CSR mask.  A wavefront takes 2048 consecutive ENTRIES, finds
// how many row offsets lie at or below its first entry (the search above) and then holds 64
// consecutive offsets at a time, one per lane: an entry below the last of them lies in the row
// given by the number of held offsets at or below it (six cross-lane reads).  When all the held
// offsets are passed the window moves on by 63, or, over a long run of empty rows, by another
// search.  (Sharing out rows instead - 16 per wavefront - left the wavefronts that met a few rows
// of 4096 entries running long after the rest on a power-law mask; a wavefront per row spends most
// of its time on the empty rows of a mask that has many.)
// Offsets are held to [0, nnz] as in CsrMask::row; entries before the first offset or at and after
// the last belong to no row and get a column that the bucketing drops.  Offsets that are not in
// ascending order give entries of the wrong row or none; every entry of [0, nnz) is written once
// and nothing outside.
__global__ __launch_bounds__(256) void csr_entry_list_kernel(const void* row_off, int off64,
                                                             const uint32_t* __restrict__ cols,
                                                             const uint32_t* __restrict__ alt_cols,
                                                             const uint32_t* use_alt, int64_t n_rows,
                                                             int64_t nnz, uint32_t* __restrict__ rows_out,
                                                             uint32_t* __restrict__ cols_out) {
  const int lane = threadIdx.x & (kWave - 1);
  const uint32_t* __restrict__ cp = (use_alt != nullptr && *use_alt != 0u) ? alt_cols : cols;
  const int64_t begin = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * kEntryListChunk;
  if (begin >= nnz) return;
  // (nnz < 2^32: the offsets of the bucketed mask are 32 bits wide)
  const uint32_t end = (uint32_t)(nnz - begin < kEntryListChunk ? nnz : begin + kEntryListChunk);
  const int64_t n_off = n_rows + 1;
  uint32_t pos = (uint32_t)begin;
  // offsets [0, c) are at or below pos
  int64_t c = wave_offsets_at_or_below(row_off, off64, nnz, 0, n_off, pos, lane);
  // lane l: offset c + l; past the last offset: one that no entry reaches
  auto hold = [&](int64_t first) -> uint32_t {
    return first + lane < n_off ? held_offset(row_off, first + lane, off64, nnz) : 0xffffffffu;
  };
  uint32_t held = hold(c);
  while (pos < end) {
    uint32_t held_last = (uint32_t)__builtin_amdgcn_readlane((int)held, kWave - 1);
    if (held_last <= pos) {
      const int64_t from = c + kWave < n_off ? c + kWave : n_off;
      c = wave_offsets_at_or_below(row_off, off64, nnz, from, n_off, pos, lane);
      held = hold(c);
      held_last = (uint32_t)__builtin_amdgcn_readlane((int)held, kWave - 1);
      if (held_last <= pos) {  // offsets out of order: go on window by window
        c = c + kWave < n_off ? c + kWave : n_off;
        held = hold(c);
        continue;
      }
    }
    // (the next window's offsets are on their way while this one's entries are written)
    const uint32_t held_next = hold(c + kWave - 1);
    const uint32_t stop = held_last < end ? held_last : end;
    // (eight loads in flight per lane: one load per trip makes a row of 4096 entries a chain of 64
    // memory round trips)
    for (uint32_t e0 = pos; e0 < stop; e0 += kEntryListInFlight * kWave) {
      uint32_t col[kEntryListInFlight];
#pragma unroll
      for (int u = 0; u < kEntryListInFlight; u++) {
        const uint32_t e = e0 + u * kWave + lane;
        col[u] = e < stop ? cp[e] : 0u;
      }
#pragma unroll
      for (int u = 0; u < kEntryListInFlight; u++) {
        const uint32_t e = e0 + u * kWave + lane;
        // number of held offsets at or below e (fewer than 64 for e < stop)
        int lo = 0;
#pragma unroll
        for (int step = kWave / 2; step >= 1; step >>= 1) {
          const uint32_t v = (uint32_t)__builtin_amdgcn_ds_bpermute((lo + step - 1) << 2, (int)held);
          if (v <= e) lo += step;
        }
        if (e < stop) {
          const int64_t row = c + lo - 1;
          const bool in_a_row = row >= 0 && row < n_rows;
          rows_out[e] = in_a_row ? (uint32_t)row : 0u;
          cols_out[e] = in_a_row ? col[u] : 0xffffffffu;
        }
      }
    }
    pos = stop;
    c += kWave - 1;
    held = held_next;
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
  // (pass 2 reads kPartKeep * kPartRowsThreads packed entries from a bucket's start whatever the
  // bucket's size: the padding keeps the last buckets' loads inside the buffer)
  w.off_tmp_pairs = off;
  off = align_up(off + (w.partition ? (size_t)nnz * 8 + (size_t)kPartKeep * kPartRowsThreads * 4 : 0), 256);
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

  hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(64), 0, stream, flag, (int64_t)1, 0u);
  // sorted or not: decided on the device (by the first pass of the partition where there is one)
  const bool part = nnz > 0 && w.partition;
  // (the per-row counts belong to the histogram path below; the partition keeps its own)
  if (!part && nnz > 0)
    hipLaunchKernelGGL(fill_u32_kernel, dim3(grid_for(n_rows + 1, 256, 4096)), dim3(256), 0, stream,
                       counts, n_rows + 1, 0u);
  if (part) {
    const dim3 grid_c(part_grid(w.n_tiles1));
    if (row_wide)
      hipLaunchKernelGGL(coo_part_count_kernel<uint64_t>, grid_c, dim3(kPartThreads), 0,
                         stream, (const uint64_t*)row_ind, nnz, n_rows, w.lo_bits, (int)w.n_hi, w.n_tiles1,
                         flag, (uint32_t*)(base + w.off_hist));
    else
      hipLaunchKernelGGL(coo_part_count_kernel<uint32_t>, grid_c, dim3(kPartThreads), 0,
                         stream, (const uint32_t*)row_ind, nnz, n_rows, w.lo_bits, (int)w.n_hi, w.n_tiles1,
                         flag, (uint32_t*)(base + w.off_hist));
  }
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
    // 152 KB of LDS per workgroup in both passes: above the 64 KB a kernel gets without asking
    // (set once per device: the attribute belongs to the device's copy of the kernel)
    // (atomic flags: callers may be on several host threads; two that meet here both set the
    // attributes, which is idempotent)
    constexpr int kMaxDevices = 64;
    static std::atomic<bool> lds_attr_set[kMaxDevices];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 4;
    if (dev < 0 || dev >= kMaxDevices || !lds_attr_set[dev].load(std::memory_order_acquire)) {
      const int packed_max = (int)part_scatter_packed_lds(kPartMaxBuckets);
      const struct { const void* kernel; int bytes; } big_lds[] = {
          {reinterpret_cast<const void*>(coo_part_scatter_kernel<uint64_t>), (int)kPartScatterLds},
          {reinterpret_cast<const void*>(coo_part_scatter_kernel<uint32_t>), (int)kPartScatterLds},
          {reinterpret_cast<const void*>(coo_part_scatter_packed_kernel<uint64_t>), packed_max},
          {reinterpret_cast<const void*>(coo_part_scatter_packed_kernel<uint32_t>), packed_max},
          {reinterpret_cast<const void*>(coo_part_rows_kernel<true>), (int)kPartRowsLds},
      };
      for (const auto& k : big_lds)
        if (hipFuncSetAttribute(k.kernel, hipFuncAttributeMaxDynamicSharedMemorySize, k.bytes) != hipSuccess)
          return 4;
      if (dev >= 0 && dev < kMaxDevices) lds_attr_set[dev].store(true, std::memory_order_release);
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
    const dim3 grid1(part_grid(w.n_tiles1)), block1(kPartThreads);
    const size_t packed_lds = part_scatter_packed_lds(w.n_hi);
    uint32_t* tmp_packed = (uint32_t*)tmp_pairs;
    const uint32_t col_max = (uint32_t)n_cols;
    if (col_bits && row_wide)
      hipLaunchKernelGGL(coo_part_scatter_packed_kernel<uint64_t>, grid1, block1, packed_lds, stream,
                         (const uint64_t*)row_ind, col_ind, nnz, n_rows, w.lo_bits, (int)w.n_hi, w.n_tiles1,
                         flag, hist, tmp_packed, col_bits, col_max);
    else if (col_bits)
      hipLaunchKernelGGL(coo_part_scatter_packed_kernel<uint32_t>, grid1, block1, packed_lds, stream,
                         (const uint32_t*)row_ind, col_ind, nnz, n_rows, w.lo_bits, (int)w.n_hi, w.n_tiles1,
                         flag, hist, tmp_packed, col_bits, col_max);
    else if (row_wide)
      hipLaunchKernelGGL(coo_part_scatter_kernel<uint64_t>, grid1, block1, kPartScatterLds, stream,
                         (const uint64_t*)row_ind, col_ind, nnz, n_rows, w.lo_bits, (int)w.n_hi, w.n_tiles1,
                         flag, hist, tmp_pairs);
    else
      hipLaunchKernelGGL(coo_part_scatter_kernel<uint32_t>, grid1, block1, kPartScatterLds, stream,
                         (const uint32_t*)row_ind, col_ind, nnz, n_rows, w.lo_bits, (int)w.n_hi, w.n_tiles1,
                         flag, hist, tmp_pairs);
    if (col_bits)
      hipLaunchKernelGGL(coo_part_rows_kernel<true>, dim3((unsigned)w.n_hi), dim3(kPartRowsThreads), kPartRowsLds, stream,
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
                   const uint32_t* use_alt, int64_t n_rows, int64_t nnz, uint32_t* rows_out,
                   uint32_t* cols_out, hipStream_t stream) {
  if (n_rows <= 0 || nnz <= 0) return 0;
  const int64_t per_block = 4 * (int64_t)kEntryListChunk;
  hipLaunchKernelGGL(csr_entry_list_kernel, dim3((unsigned)((nnz + per_block - 1) / per_block)), dim3(256), 0,
                     stream, row_off, off64, cols, alt_cols, use_alt, n_rows, nnz, rows_out, cols_out);
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
