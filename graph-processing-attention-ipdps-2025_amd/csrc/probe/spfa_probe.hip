// Measurement aid: the gather of the explicit-mask kernels with the arithmetic taken out.
//
// segments_kernel spends its time fetching one K row and one V row per live position.  What the
// memory system can deliver to exactly that access pattern - rows of `row_bytes` bytes picked by a
// column list, 16 bytes per lane, a batch of 2 * U row loads issued back to back per lane group,
// persistent wavefronts pulling chunks of the list off an atomic cursor - is the
// ceiling that kernel can be priced against when K and V sit in the memory-side cache and the
// HBM figure no longer binds.  This kernel does those loads and nothing else: no dot products, no
// softmax, no output.  The loaded registers are handed to an empty asm statement so that the
// loads stay.
//
// Built into libspfa_probe.so, apart from the attention library: benchmarks load it, the drop-in
// boundary does not carry it.
#include "spfa_probe.h"

#include "spfa_hip.h"

#include "spfa_common.hpp"
#include "spfa_engine.hpp"

namespace spfa {
namespace {

__global__ void probe_reset_kernel(uint32_t* cursor) {
  if (threadIdx.x == 0) *cursor = 0;
}

// an entry of the list: a row below n_rows, else (top bit set, or out of range) skipped.  The
// value is consumed one trip after it is loaded, so the comparison costs no wait.
__device__ __forceinline__ int probe_entry(uint32_t x, uint32_t n_rows) { return x < n_rows ? (int)x : -1; }

template <int LPR, int U>
__global__ __launch_bounds__(256) void gather_probe_kernel(const char* __restrict__ k,
                                                           const char* __restrict__ v, int64_t row_bytes,
                                                           uint32_t n_rows,
                                                           const uint32_t* __restrict__ idx, int64_t n_idx,
                                                           int64_t chunk, uint32_t* cursor) {
  constexpr int GS = kWave / LPR;  // rows per wavefront-wide load
  constexpr int PER = U * GS;      // list entries per batch
  constexpr int PARTS = kWave / PER;
  static_assert(PARTS >= 1 && PARTS * PER == kWave, "a batch must divide an index chunk");
  const int lane = lane_id();
  const int gi = lane / LPR;
  const int c = lane % LPR;
  const int64_t n_chunks = (n_idx + chunk - 1) / chunk;
  // (as in the attention kernel: a wavefront's first chunk is the one with its own number, the
  // later ones come off the cursor)
  const uint32_t n_waves = gridDim.x * 4u;
  uint32_t w = (uint32_t)__builtin_amdgcn_readfirstlane((int)(blockIdx.x * 4u + (threadIdx.x >> 6)));
  while ((int64_t)w < n_chunks) {
    const int64_t t0 = (int64_t)w * chunk;
    const int64_t t1 = t0 + chunk < n_idx ? t0 + chunk : n_idx;
    int next = t0 + lane < t1 ? probe_entry(idx[t0 + lane], n_rows) : -1;
    for (int64_t tb = t0; tb < t1; tb += kWave) {
      const int cur = next;
      if (tb + kWave < t1) next = tb + kWave + lane < t1 ? probe_entry(idx[tb + kWave + lane], n_rows) : -1;
#pragma unroll 1
      for (int part = 0; part < PARTS; part++) {
        if (tb + part * PER >= t1) break;
        int cols[U];
#pragma unroll
        for (int u = 0; u < U; u++) cols[u] = shfl_i32(cur, part * PER + u * GS + gi);
        uint4v kr[U], vr[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
          if (cols[u] >= 0) {
            kr[u] = *reinterpret_cast<const uint4v*>(k + (int64_t)cols[u] * row_bytes + c * 16);
            vr[u] = *reinterpret_cast<const uint4v*>(v + (int64_t)cols[u] * row_bytes + c * 16);
          }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
          if (cols[u] >= 0) asm volatile("" ::"v"(kr[u]), "v"(vr[u]));
        }
        __builtin_amdgcn_sched_barrier(0);  // (one batch in flight at a time, as in the attention kernel)
      }
    }
    if ((int64_t)n_waves >= n_chunks) break;  // (an ordinary grid: a chunk per wavefront, no cursor)
    uint32_t nx = 0;
    if (lane == 0) nx = atomicAdd(cursor, 1u);
    w = n_waves + (uint32_t)__builtin_amdgcn_readfirstlane((int)nx);
    __builtin_amdgcn_wave_barrier();
  }
}

// Two index chunks (2 * 64 entries) per trip, the row loads of both issued before any is consumed:
// twice the loads in flight per wavefront, for row sizes where a batch of U = 64 / groups rows
// already covers a whole chunk.
template <int LPR>
__global__ __launch_bounds__(256) void gather_probe_deep_kernel(const char* __restrict__ k,
                                                                const char* __restrict__ v, int64_t row_bytes,
                                                                uint32_t n_rows,
                                                                const uint32_t* __restrict__ idx, int64_t n_idx,
                                                                int64_t chunk, uint32_t* cursor) {
  constexpr int GS = kWave / LPR;
  constexpr int U = kWave / GS;
  const int lane = lane_id();
  const int gi = lane / LPR;
  const int c = lane % LPR;
  const int64_t n_chunks = (n_idx + chunk - 1) / chunk;
  // (as in the attention kernel: a wavefront's first chunk is the one with its own number, the
  // later ones come off the cursor)
  const uint32_t n_waves = gridDim.x * 4u;
  uint32_t w = (uint32_t)__builtin_amdgcn_readfirstlane((int)(blockIdx.x * 4u + (threadIdx.x >> 6)));
  while ((int64_t)w < n_chunks) {
    const int64_t t0 = (int64_t)w * chunk;
    const int64_t t1 = t0 + chunk < n_idx ? t0 + chunk : n_idx;
    auto fetch = [&](int64_t t) -> int { return t + lane < t1 ? probe_entry(idx[t + lane], n_rows) : -1; };
    int next0 = fetch(t0), next1 = fetch(t0 + kWave);
    for (int64_t tb = t0; tb < t1; tb += 2 * kWave) {
      const int cur0 = next0, cur1 = next1;
      next0 = fetch(tb + 2 * kWave);
      next1 = fetch(tb + 3 * kWave);
      int cols[2 * U];
#pragma unroll
      for (int u = 0; u < U; u++) {
        cols[u] = shfl_i32(cur0, u * GS + gi);
        cols[U + u] = shfl_i32(cur1, u * GS + gi);
      }
      uint4v kr[2 * U], vr[2 * U];
#pragma unroll
      for (int u = 0; u < 2 * U; u++) {
        if (cols[u] >= 0) {
          kr[u] = *reinterpret_cast<const uint4v*>(k + (int64_t)cols[u] * row_bytes + c * 16);
          vr[u] = *reinterpret_cast<const uint4v*>(v + (int64_t)cols[u] * row_bytes + c * 16);
        }
      }
#pragma unroll
      for (int u = 0; u < 2 * U; u++) {
        if (cols[u] >= 0) asm volatile("" ::"v"(kr[u]), "v"(vr[u]));
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if ((int64_t)n_waves >= n_chunks) break;  // (an ordinary grid: a chunk per wavefront, no cursor)
    uint32_t nx = 0;
    if (lane == 0) nx = atomicAdd(cursor, 1u);
    w = n_waves + (uint32_t)__builtin_amdgcn_readfirstlane((int)nx);
    __builtin_amdgcn_wave_barrier();
  }
}

template <int LPR>
int launch_probe(const void* k, const void* v, int64_t row_bytes, uint32_t n_rows, const uint32_t* idx,
                 int64_t n_idx, int64_t chunk, int wg_per_cu, int in_flight, uint32_t* cursor,
                 const KernelEvents& ev, hipStream_t stream) {
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess)
    (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  // wg_per_cu == 0: an ordinary grid, one wavefront per chunk of the list (items_grid_kernel's shape)
  const int64_t n_chunks = (n_idx + chunk - 1) / chunk;
  const dim3 grid((unsigned)(wg_per_cu > 0 ? (int64_t)cus * wg_per_cu : (n_chunks + 3) / 4)), block(256);
  hipLaunchKernelGGL(probe_reset_kernel, dim3(1), dim3(64), 0, stream, cursor);
  // (the gather itself takes the caller's event pair, as the kernel it stands in for does)
  constexpr int UMAX = LPR;  // a batch of U rows per group covers at most one 64-entry chunk
  if constexpr (LPR <= 16) {
    if (in_flight >= 2 * UMAX) {
      launch_maybe_timed(ev, gather_probe_deep_kernel<LPR>, grid, block, stream, (const char*)k, (const char*)v,
                         row_bytes, n_rows, idx, n_idx, chunk, cursor);
      return hipGetLastError() == hipSuccess ? SPFA_OK : SPFA_ERR_LAUNCH;
    }
  }
  if (in_flight >= 16 && UMAX >= 16)
    launch_maybe_timed(ev, gather_probe_kernel<LPR, (UMAX >= 16 ? 16 : UMAX)>, grid, block, stream,
                       (const char*)k, (const char*)v, row_bytes, n_rows, idx, n_idx, chunk, cursor);
  else if (in_flight >= 8 && UMAX >= 8)
    launch_maybe_timed(ev, gather_probe_kernel<LPR, (UMAX >= 8 ? 8 : UMAX)>, grid, block, stream,
                       (const char*)k, (const char*)v, row_bytes, n_rows, idx, n_idx, chunk, cursor);
  else
    launch_maybe_timed(ev, gather_probe_kernel<LPR, 4>, grid, block, stream, (const char*)k, (const char*)v,
                       row_bytes, n_rows, idx, n_idx, chunk, cursor);
  return hipGetLastError() == hipSuccess ? SPFA_OK : SPFA_ERR_LAUNCH;
}

}  // namespace
}  // namespace spfa

extern "C" int spfa_probe_gather(const void* k, const void* v, int64_t n_rows, int64_t row_bytes,
                                 const uint32_t* idx, int64_t n_idx, int64_t chunk, int wg_per_cu,
                                 int in_flight, void* cursor, void* ev_start, void* ev_stop, void* stream) {
  using namespace spfa;
  if (!k || !v || !idx || !cursor || n_rows < 1 || n_rows > (int64_t)0x7fffffff || n_idx < 1 || chunk < 64 ||
      wg_per_cu < 0 || wg_per_cu > 8 || (n_idx + chunk - 1) / chunk > (int64_t)0x7fffffff)
    return SPFA_ERR_BAD_ARG;
  KernelEvents ev;
  ev.start = (hipEvent_t)ev_start;
  ev.stop = (hipEvent_t)ev_stop;
  const uint32_t nr = (uint32_t)n_rows;
  if ((((uintptr_t)k | (uintptr_t)v) & 15u) != 0) return SPFA_ERR_BAD_ARG;
  hipStream_t s = (hipStream_t)stream;
  switch (row_bytes) {
    case 64: return launch_probe<4>(k, v, row_bytes, nr, idx, n_idx, chunk, wg_per_cu, in_flight, (uint32_t*)cursor, ev, s);
    case 128: return launch_probe<8>(k, v, row_bytes, nr, idx, n_idx, chunk, wg_per_cu, in_flight, (uint32_t*)cursor, ev, s);
    case 256: return launch_probe<16>(k, v, row_bytes, nr, idx, n_idx, chunk, wg_per_cu, in_flight, (uint32_t*)cursor, ev, s);
    case 512: return launch_probe<32>(k, v, row_bytes, nr, idx, n_idx, chunk, wg_per_cu, in_flight, (uint32_t*)cursor, ev, s);
  }
  return SPFA_ERR_UNSUPPORTED;
}
