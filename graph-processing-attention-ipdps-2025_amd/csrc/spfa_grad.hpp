// Gradients of masked attention by two gather passes, no atomics on the hot path (the reference
// has no backward pass; the m and l it leaves behind are the statistics one needs).
//
// With lse_i = m_i + log l_i, p_ij = exp(q_i.k_j / sqrt(d) - lse_i) on live positions,
// delta_i = dO_i . O_i and dS_ij = p_ij (dO_i . v_j - delta_i) / sqrt(d):
//     query pass, owner = query row i, candidates = its live columns j (gathers K_j, V_j):
//         dQ_i += sum_j dS_ij k_j
//     key pass, owner = key row j, candidates = the query rows i that attend it (gathers Q_i,
//     dO_i, lse_i, delta_i):
//         dK_j += sum_i dS_ij q_i          dV_j += sum_i p_ij dO_i
// The key pass walks the mask by column: the implicit masks are symmetric and answer that with
// the same functor (the global mask with a column functor that knows about repeated list
// entries), an explicit mask is transposed first (spfa_api.hip).
//
// Both passes are one kernel template.  One wavefront per owner row: the row's two vectors sit in
// registers, replicated in every lane group; each group of LPR lanes takes one candidate at a
// time (16 bytes per lane of each of its two rows, U candidates in flight per group), does both
// dot products with in-group reductions and adds the weighted candidate rows to its
// accumulators; the groups are summed at the end.  Owners with more than `own_max` candidates
// leave their segments of `seg` candidates on a work list instead, which is handed out in the
// forward engine's order (segments at the same place in their rows together) to the persistent
// wavefronts of grad_segments_kernel; their results are added with floating-point atomics.
#pragma once

#include "spfa_engine.hpp"
#include "spfa_masks.hpp"

namespace spfa {

struct GradArgs {
  const void* q;      // element type T; [n_batch, n_q, d]
  const void* k;      // [n_batch, n_k, d]
  const void* v;
  const void* d_out;  // [n_batch, n_q, d]
  float* lse;         // [n_batch * n_q]  m + log l, +inf for rows that never saw a live column
  float* delta;       // [n_batch * n_q]  dO . O (0 for those rows)
  float2* stat;       // [n_batch * n_q]  (lse, delta) side by side, for the gather engine's key pass:
                      // a candidate's two numbers then cost one cache line, not two (measured, 50 M
                      // candidates of 1 M rows: as many line fills went to the two arrays as to Q)
  float* d_q;         // fp32 gradients, added to
  float* d_k;
  float* d_v;
  int64_t n_q;
  int64_t n_k;
  int64_t n_batch;
  int32_t d;
  int32_t seg;          // candidates one wavefront takes of a row
  int32_t own_max;      // owners of more candidates leave all their segments on the work list
  // the work lists of the two passes (query pass, key pass): the forward engine's items, `row`
  // being the owner among all problems (32 bits), and its counters (item count, cursor, overflow)
  Counters* cnt[2];
  Phases* phases[2];
  Item* listed[2];      // as appended
  Item* ordered[2];     // in the order they are handed out in
  uint32_t cap_items;
  uint32_t* status;     // the device's sticky status word (may be null)
  int32_t items_on_grid;  // the work lists are walked by an ordinary grid, a wavefront per item
  int32_t items_as_listed;  // ... and in the order they were appended in (no order_kernel): the
                            // gathered tensors fit the L2s, the hand-out order is worth nothing
};

constexpr int kGradWaves = 4;        // owners per workgroup

// Candidates in flight per lane group in grad_rows_kernel.  One wavefront per owner row makes the
// kernel live on the number of rows in flight, not on the loads in flight per row: with 2 instead
// of 8 (57 / 78 registers instead of 108 / 131 in the query / key pass at fp32 d = 64, 8 / 6
// wavefronts per SIMD instead of 4 / 3) the two passes of the Zipf masks take 1.48 ms instead of
// 1.66 (131 K rows, 12.8 M positions) and 9.7 ms instead of 10.9 (1 M rows, 50 M positions);
// 16 in flight: 1.95 and 11.2 ms; forcing 8 wavefronts per SIMD on 4 in flight spills: 3.3 ms.
template <class Lay>
constexpr int grad_rows_unroll() {
  return Lay::U_SHORT >= 2 ? Lay::U_SHORT / 2 : 1;
}

template <class Lay>
__device__ __forceinline__ int grad_elem_index(int c, int e) {
  return Lay::elem_index(c, e);
}

// lse and delta of every query row: 16 lanes per row, 16 bytes per lane and step
// Clears the counters and phase counts of both work lists (64 lanes).
__device__ __forceinline__ void grad_reset(const GradArgs& g, int lane) {
  static_assert(kPhases == kWave, "one lane per phase");
  for (int p = 0; p < 2; p++) {
    g.phases[p]->count[lane] = 0;
    g.phases[p]->taken[lane] = 0;
    if (lane == 0) {
      g.cnt[p]->n_items = 0;
      g.cnt[p]->next_item = 0;
      g.cnt[p]->overflow = 0;
    }
  }
}

// (RESET: the first wavefront also clears the gather passes' work lists - a launch of its own for
// that costs a short call 4 - 5 us)
template <typename T, bool RESET = false>
__global__ __launch_bounds__(256) void grad_prologue_kernel(Tensors t, GradArgs g) {
  constexpr int V = 16 / (int)sizeof(T);
  typedef T vec __attribute__((ext_vector_type(V)));
  const int c = threadIdx.x & 15;
  const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  if constexpr (RESET) {
    if (blockIdx.x == 0 && threadIdx.x < kWave) grad_reset(g, (int)threadIdx.x);
  }
  if (row >= t.n_q * t.n_batch) return;
  const bool sf = t.state_f32 != 0;
  const float m = load_state<T>(t.m, row, sf);
  const float l = load_state<T>(t.l, row, sf);
  const bool live = l > 0.f;
  float acc = 0.f;
  // (the rows are read whether the row is live or not, so that their loads do not wait for l; a
  // dead row's product - its out row may hold NaN - is dropped below)
  {
    const T* orow = (const T*)t.out + row * t.d;
    const T* drow = (const T*)g.d_out + row * t.d;
    if ((t.d % V) == 0 && (((uintptr_t)t.out | (uintptr_t)g.d_out) & 15) == 0) {
      for (int e = c * V; e < t.d; e += 16 * V) {
        const vec a = *reinterpret_cast<const vec*>(orow + e);
        const vec b = *reinterpret_cast<const vec*>(drow + e);
#pragma unroll
        for (int x = 0; x < V; x++) acc += to_f32((T)a[x]) * to_f32((T)b[x]);
      }
    } else {
      for (int e = c; e < t.d; e += 16) acc += to_f32(orow[e]) * to_f32(drow[e]);
    }
  }
  acc = group_sum<16>(acc);
  if (c == 0) {
    const float lse = live ? m + __logf(l) : __builtin_inff();
    const float delta = live ? acc : 0.f;
    g.lse[row] = lse;
    g.delta[row] = delta;
    g.stat[row] = make_float2(lse, delta);
  }
}

// The work list of a pass as the forward engine's kernels see it (order_kernel, work_list()).
__host__ __device__ inline Plan grad_plan(const GradArgs& g, int pass) {
  Plan plan{};
  plan.cnt = g.cnt[pass];
  plan.cursor = &g.cnt[pass]->next_item;
  plan.phases = g.phases[pass];
  plan.listed = g.listed[pass];
  plan.items = g.ordered[pass];
  plan.cap_items = g.cap_items;
  plan.seg = g.seg;
  return plan;
}

// Candidates t_begin .. t_end of one owner, walked by the whole wavefront.
//   KEYS == false: owner is a query row, (a, b) = (q_i, dO_i), X = K, Y = V, and lse_o / delta_o
//                  are the owner's; acc1 collects dQ_i.
//   KEYS == true:  owner is a key row, (a, b) = (k_j, v_j), X = Q, Y = dO, (lse, delta) are read
//                  per candidate; acc1 collects dK_j, acc2 dV_j.
template <class Lay, class Mask, bool KEYS, int U_>
__device__ __forceinline__ void grad_walk(const Mask& mask, const typename Mask::Row& rc,
                                          const typename Lay::elem* __restrict__ X,
                                          const typename Lay::elem* __restrict__ Y,
                                          const float2* __restrict__ stat_c, float lse_o,
                                          float delta_o, int d, float scale,
                                          const float (&a)[Lay::NE], const float (&b)[Lay::NE],
                                          int64_t t_begin, int64_t t_end, int lane,
                                          float (&acc1)[Lay::NE], float (&acc2)[Lay::NE]) {
  constexpr int NE = Lay::NE;
  constexpr int LPR = Lay::LPR;
  constexpr int GS = kWave / LPR;
  constexpr int U = (U_ * GS > kWave) ? kWave / GS : U_;
  constexpr int PER = U * GS;
  constexpr int PARTS = kWave / PER;
  const int gi = lane / LPR;
  const int c = lane % LPR;

  // (an explicit mask's column is range-checked when the chunk is used, one trip after its load)
  auto fetch = [&](int64_t t) -> int {
    const int64_t tt = t + lane;
    bool valid = tt < t_end;
    int64_t col = 0;
    if constexpr (Mask::kExplicit) {
      if (valid) col = mask.col_unchecked(rc, tt);
    } else {
      if (valid) col = mask.col(rc, tt, valid);
    }
    return valid ? (int)col : -1;
  };

  // (the owner's two vectors came out of the element type: see Lay::packed_dot)
  typename Lay::raw ap{}, bp{};
  if constexpr (Lay::kPackedDot) {
    ap = Lay::pack_exact(a);
    bp = Lay::pack_exact(b);
  }
  int next = fetch(t_begin);
  for (int64_t tb = t_begin; tb < t_end; tb += kWave) {
    int cur = next;
    if constexpr (Mask::kExplicit) cur = mask.in_range(cur) ? cur : -1;
    if (tb + kWave < t_end) next = fetch(tb + kWave);
#pragma unroll 1
    for (int part = 0; part < PARTS; part++) {
      if (tb + part * PER >= t_end) break;
      int cols[U];
#pragma unroll
      for (int u = 0; u < U; u++) cols[u] = shfl_i32(cur, part * PER + u * GS + gi);
      typename Lay::raw xr[U], yr[U];
      float ls[U], dl[U];
#pragma unroll
      for (int u = 0; u < U; u++) {
        ls[u] = lse_o;
        dl[u] = delta_o;
        if (cols[u] >= 0) {
          xr[u] = Lay::load_gather(X + (int64_t)cols[u] * d, c, d);
          yr[u] = Lay::load_gather(Y + (int64_t)cols[u] * d, c, d);
          if constexpr (KEYS) {
            // (two 4-byte loads of the one line: as one 8-byte load the key pass of 131 K rows
            // took 533 us instead of 440)
            const float* sp = reinterpret_cast<const float*>(stat_c + cols[u]);
            ls[u] = sp[0];
            const float* sp1 = sp + 1;
            asm volatile("" : "+v"(sp1));
            dl[u] = *sp1;
          }
        }
      }
#pragma unroll
      for (int u = 0; u < U; u++) {
        float xf[NE], yf[NE];
        float s = 0.f, t = 0.f;
        if (cols[u] >= 0) {
          Lay::unpack(xr[u], xf);
          if constexpr (Lay::kPackedDot) {
            s = Lay::packed_dot(xr[u], ap);
            t = Lay::packed_dot(yr[u], bp);
            if constexpr (KEYS) Lay::unpack(yr[u], yf);
          } else {
            Lay::unpack(yr[u], yf);
#pragma unroll
            for (int e = 0; e < NE; e++) {
              s += a[e] * xf[e];
              t += b[e] * yf[e];
            }
          }
        }
        s = group_sum<LPR>(s);
        t = group_sum<LPR>(t);
        if (cols[u] >= 0) {
          float p = __expf(s * scale - ls[u]);
          if constexpr (Mask::kWeighted) p *= mask.weight(rc, (int64_t)cols[u]);
          const float ds = p * (t - dl[u]) * scale;
#pragma unroll
          for (int e = 0; e < NE; e++) acc1[e] += ds * xf[e];
          if constexpr (KEYS) {
#pragma unroll
            for (int e = 0; e < NE; e++) acc2[e] += p * yf[e];
          }
        }
      }
    }
  }
  // every group has walked its share: add the groups up (group 0 ends up with the total too)
#pragma unroll
  for (int off = LPR; off < kWave; off <<= 1) {
#pragma unroll
    for (int e = 0; e < NE; e++) {
      acc1[e] += shfl_xor_f32(acc1[e], off);
      if constexpr (KEYS) acc2[e] += shfl_xor_f32(acc2[e], off);
    }
  }
}

// What one owner (row `r` among all problems) needs: pointers of its pass.
template <class Lay, bool KEYS>
struct GradOwner {
  using T = typename Lay::elem;
  const T* X;
  const T* Y;
  const float2* stat_c;
  float lse_o, delta_o;
  float a[Lay::NE], b[Lay::NE];
  float* out1;
  float* out2;
  int64_t ri;  // row inside its problem
  __device__ __forceinline__ void load(const GradArgs& g, int64_t r, int c) {
    const int d = g.d;
    const int64_t n_own = KEYS ? g.n_k : g.n_q;
    int64_t bb = 0;
    ri = r;
    if (g.n_batch > 1) {
      bb = r / n_own;
      ri = r - bb * n_own;
    }
    const T* arow;
    const T* brow;
    if constexpr (KEYS) {
      arow = (const T*)g.k + r * d;
      brow = (const T*)g.v + r * d;
      X = (const T*)g.q + bb * g.n_q * d;
      Y = (const T*)g.d_out + bb * g.n_q * d;
      stat_c = g.stat + bb * g.n_q;
      lse_o = 0.f;
      delta_o = 0.f;
      out1 = g.d_k + r * d;
      out2 = g.d_v + r * d;
    } else {
      arow = (const T*)g.q + r * d;
      brow = (const T*)g.d_out + r * d;
      X = (const T*)g.k + bb * g.n_k * d;
      Y = (const T*)g.v + bb * g.n_k * d;
      stat_c = nullptr;
      lse_o = g.lse[r];
      delta_o = g.delta[r];
      out1 = g.d_q + r * d;
      out2 = nullptr;
    }
    Lay::unpack(Lay::load(arow, c, d), a);
    Lay::unpack(Lay::load(brow, c, d), b);
  }
};

template <class Lay, class Mask, bool KEYS>
__device__ __forceinline__ void grad_rows_body(const GradArgs& g, const Mask& mask, int64_t block) {
  constexpr int NE = Lay::NE;
  const int lane = threadIdx.x & (kWave - 1);
  const int c = lane % Lay::LPR;
  const int64_t n_own = KEYS ? g.n_k : g.n_q;
  const int64_t r = block * kGradWaves + (threadIdx.x >> 6);
  if (r >= n_own * g.n_batch) return;
  GradOwner<Lay, KEYS> o;
  o.load(g, r, c);
  const typename Mask::Row rc = mask.row(o.ri);
  const int64_t deg = rc.deg;
  if (deg <= 0) return;
  if (!KEYS && o.lse_o == __builtin_inff()) return;  // the row never saw a live column
  if (deg > g.own_max) {
    // all of the row goes on the work list, a segment per lane
    const int pass = KEYS ? 1 : 0;
    const int64_t seg = g.seg;
    const uint32_t nseg = (uint32_t)((deg + seg - 1) / seg);
    uint32_t base = 0;
    if (lane == 0) base = atomicAdd(&g.cnt[pass]->n_items, nseg);
    base = (uint32_t)__builtin_amdgcn_readfirstlane((int)base);
    if (base + nseg > g.cap_items || base + nseg < base) {
      if (lane == 0) {  // (only a mask whose arrays disagree with the nnz passed can get here)
        atomicOr(&g.cnt[pass]->overflow, 1u);
        if (g.status != nullptr) atomicOr(g.status, kStatusWorkListOverflow);
      }
      return;
    }
    for (uint32_t j = (uint32_t)lane; j < nseg; j += kWave) {
      Item it;
      it.row = (int32_t)(uint32_t)r;
      it.seg = (int32_t)j;
      it.slot = -1;
      it.phase = (int32_t)segment_phase(j, nseg, deg, seg);
      g.listed[pass][base + j] = it;
      atomicAdd(&g.phases[pass]->count[it.phase], 1u);
    }
    return;
  }
  float acc1[NE], acc2[NE];
#pragma unroll
  for (int e = 0; e < NE; e++) {
    acc1[e] = 0.f;
    acc2[e] = 0.f;
  }
  const float scale = 1.0f / sqrtf((float)g.d);
  grad_walk<Lay, Mask, KEYS, grad_rows_unroll<Lay>()>(mask, rc, o.X, o.Y, o.stat_c, o.lse_o, o.delta_o,
                                            g.d, scale, o.a, o.b, 0, deg, lane,
                                            acc1, acc2);
  if (lane < Lay::LPR) {  // this wavefront is the only one that touches the row in this launch
    float cur[NE];
    Lay::load_f32(o.out1, c, g.d, cur);
#pragma unroll
    for (int e = 0; e < NE; e++) cur[e] += acc1[e];
    Lay::store_f32(o.out1, c, g.d, cur);
    if constexpr (KEYS) {
      Lay::load_f32(o.out2, c, g.d, cur);
#pragma unroll
      for (int e = 0; e < NE; e++) cur[e] += acc2[e];
      Lay::store_f32(o.out2, c, g.d, cur);
    }
  }
}

template <class Lay, class Mask, bool KEYS>
__global__ __launch_bounds__(kGradWaves* kWave) void grad_rows_kernel(GradArgs g, Mask mask) {
  grad_rows_body<Lay, Mask, KEYS>(g, mask, (int64_t)blockIdx.x);
}

// The owners of both passes in one launch, query rows first: the passes do not depend on each
// other (one adds to dQ, the other to dK and dV), and in a call of a few ten thousand owners
// neither fills the device - each wavefront is a chain of dependent round trips -, so one after
// the other they take the sum of their latencies, side by side the longer of the two (the Zipf
// mask at 16384 tokens: 60 + 53 us).  In larger calls the query rows would pay for running at the
// key pass's register count.
constexpr int64_t kGradBothOwnersMax = 65536;
template <class Lay, class RowMask, class ColMask>
__global__ __launch_bounds__(kGradWaves* kWave) void grad_rows_both_kernel(GradArgs g, RowMask rows, ColMask cols,
                                                                           uint32_t query_blocks) {
  if (blockIdx.x < query_blocks)
    grad_rows_body<Lay, RowMask, false>(g, rows, (int64_t)blockIdx.x);
  else
    grad_rows_body<Lay, ColMask, true>(g, cols, (int64_t)(blockIdx.x - query_blocks));
}

// Candidates in flight per lane group in grad_segments_kernel: the forward segment kernel's, as
// long as the two owner vectors, the two accumulators and the rows in flight fit 256 registers.
template <class Lay, bool KEYS>
constexpr int grad_segments_unroll() {
  return KEYS ? Lay::U_MEDIUM : Lay::U;
}

// The segments grad_rows_kernel left on the work list: a persistent grid, two workgroups per CU,
// each wavefront pulls items off the ordered list (the forward engine's segments_kernel with the
// gradient's arithmetic), results added atomically.
// GRID: an ordinary grid of one wavefront per item instead (the forward engine's
// items_grid_kernel: the better shape while the gathered tensors stay in the caches).
template <class Lay, class Mask, bool KEYS, bool GRID = false>
__global__ __launch_bounds__(256) void grad_segments_kernel(GradArgs g, Mask mask) {
  constexpr int NE = Lay::NE;
  const int lane = threadIdx.x & (kWave - 1);
  const int c = lane % Lay::LPR;
  const Plan plan = grad_plan(g, KEYS ? 1 : 0);
  if (plan.cnt->overflow) return;
  uint32_t n_items = plan.cnt->n_items;
  if (n_items > plan.cap_items) n_items = plan.cap_items;
  if (n_items == 0) return;  // (else every wavefront would still queue up at the cursor once)
  const Item* const items = work_list(plan, n_items, lane);
  const float scale = 1.0f / sqrtf((float)g.d);
  // (a wavefront's first item is the one with its own number, the later ones come off the cursor)
  const uint32_t n_waves = gridDim.x * 4u;
  uint32_t idx = (uint32_t)__builtin_amdgcn_readfirstlane((int)(blockIdx.x * 4u + (threadIdx.x >> 6)));
  while (idx < n_items) {
    const Item it = items[idx];
    const int64_t r = (int64_t)(uint32_t)it.row;
    GradOwner<Lay, KEYS> o;
    o.load(g, r, c);
    const typename Mask::Row rc = mask.row(o.ri);
    const int64_t t0 = (int64_t)it.seg * g.seg;
    const int64_t t1 = rc.deg < t0 + g.seg ? rc.deg : t0 + g.seg;
    float acc1[NE], acc2[NE];
#pragma unroll
    for (int e = 0; e < NE; e++) {
      acc1[e] = 0.f;
      acc2[e] = 0.f;
    }
    grad_walk<Lay, Mask, KEYS, (GRID ? Lay::U_MEDIUM : grad_segments_unroll<Lay, KEYS>())>(mask, rc, o.X, o.Y, o.stat_c, o.lse_o,
                                                                 o.delta_o, g.d, scale, o.a, o.b, t0, t1,
                                                                 lane, acc1, acc2);
    if (lane < Lay::LPR) {
#pragma unroll
      for (int e = 0; e < NE; e++) {
        const int idx_e = grad_elem_index<Lay>(c, e);
        if (idx_e < g.d) {
          unsafeAtomicAdd(o.out1 + idx_e, acc1[e]);
          if constexpr (KEYS) unsafeAtomicAdd(o.out2 + idx_e, acc2[e]);
        }
      }
    }
    if constexpr (GRID) break;
    uint32_t next = 0;
    if (lane == 0) next = atomicAdd(plan.cursor, 1u);
    idx = n_waves + (uint32_t)__builtin_amdgcn_readfirstlane((int)next);
    // (every lane takes the next trip together: the work index is read across lanes)
    __builtin_amdgcn_wave_barrier();
  }
}

template <class Lay, class RowMask, class ColMask>
int launch_grad(const Tensors& t, const GradArgs& g, const RowMask& rows, const ColMask& cols,
                hipStream_t stream) {
  using T = typename Lay::elem;
  const int64_t nq = g.n_q * g.n_batch, nk = g.n_k * g.n_batch;
  if (nq == 0 || nk == 0) return 0;
  if (nq >= ((int64_t)1 << 32) || nk >= ((int64_t)1 << 32)) return 1;  // items hold 32-bit owners
  const dim3 block(kGradWaves * kWave);
  const bool lists = g.cap_items > 1;  // (no owner of this call can have more than own_max candidates otherwise)
  // (the lists walked as they were appended, see GradArgs::items_as_listed)
  const bool as_listed = g.items_as_listed != 0;
  GradArgs gl = g;
  if (as_listed) {
    gl.ordered[0] = gl.listed[0];
    gl.ordered[1] = gl.listed[1];
  }
  const dim3 grid_order((g.cap_items + 255u) / 256u);
  int64_t grid_seg = (int64_t)device_cu_count() * kSegmentWorkgroupsPerCu;
  if (grid_seg > ((int64_t)g.cap_items + 3) / 4) grid_seg = ((int64_t)g.cap_items + 3) / 4;
  hipLaunchKernelGGL((grad_prologue_kernel<T, true>), dim3((unsigned)((nq + 15) / 16)), dim3(256), 0, stream,
                     t, g);
  const int64_t q_blocks = (nq + kGradWaves - 1) / kGradWaves, k_blocks = (nk + kGradWaves - 1) / kGradWaves;
  const bool both = nq + nk <= kGradBothOwnersMax;
  if (both)
    hipLaunchKernelGGL((grad_rows_both_kernel<Lay, RowMask, ColMask>), dim3((unsigned)(q_blocks + k_blocks)), block,
                       0, stream, g, rows, cols, (uint32_t)q_blocks);
  else
    hipLaunchKernelGGL((grad_rows_kernel<Lay, RowMask, false>), dim3((unsigned)q_blocks), block, 0, stream, g, rows);
  if (lists) {
    if (!as_listed) hipLaunchKernelGGL(order_kernel, grid_order, dim3(256), 0, stream, grad_plan(g, 0));
    if (g.items_on_grid)
      hipLaunchKernelGGL((grad_segments_kernel<Lay, RowMask, false, true>), dim3((g.cap_items + 3u) / 4u),
                         dim3(256), 0, stream, gl, rows);
    else
      hipLaunchKernelGGL((grad_segments_kernel<Lay, RowMask, false>), dim3((unsigned)grid_seg), dim3(256), 0,
                         stream, gl, rows);
  }
  if (!both)
    hipLaunchKernelGGL((grad_rows_kernel<Lay, ColMask, true>), dim3((unsigned)k_blocks), block, 0, stream, g, cols);
  if (lists) {
    if (!as_listed) hipLaunchKernelGGL(order_kernel, grid_order, dim3(256), 0, stream, grad_plan(g, 1));
    if (g.items_on_grid)
      hipLaunchKernelGGL((grad_segments_kernel<Lay, ColMask, true, true>), dim3((g.cap_items + 3u) / 4u),
                         dim3(256), 0, stream, gl, cols);
    else
      hipLaunchKernelGGL((grad_segments_kernel<Lay, ColMask, true>), dim3((unsigned)grid_seg), dim3(256), 0,
                         stream, gl, cols);
  }
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

template <typename T, class RowMask, class ColMask>
int run_grad(const Tensors& t, const GradArgs& g, const RowMask& rows, const ColMask& cols,
             hipStream_t stream) {
  const int64_t row_bytes = (int64_t)t.d * (int64_t)sizeof(T);
  if (row_bytes == 64) return launch_grad<VecLay<T, 4>>(t, g, rows, cols, stream);
  if (row_bytes == 128) return launch_grad<VecLay<T, 8>>(t, g, rows, cols, stream);
  if (row_bytes == 256) return launch_grad<VecLay<T, 16>>(t, g, rows, cols, stream);
  if (row_bytes == 512) return launch_grad<VecLay<T, 32>>(t, g, rows, cols, stream);
  if (row_bytes % 16 == 0) {  // (the padded layouts of the forward engine)
    if (row_bytes < 64) return launch_grad<VecLay<T, 4, true>>(t, g, rows, cols, stream);
    if (row_bytes < 128) return launch_grad<VecLay<T, 8, true>>(t, g, rows, cols, stream);
    if (row_bytes < 256) return launch_grad<VecLay<T, 16, true>>(t, g, rows, cols, stream);
    if (row_bytes < 512) return launch_grad<VecLay<T, 32, true>>(t, g, rows, cols, stream);
    if (row_bytes <= 1024) return launch_grad<WideLay<T, 2>>(t, g, rows, cols, stream);
    if (row_bytes <= 2048) return launch_grad<WideLay<T, 4>>(t, g, rows, cols, stream);
    if constexpr (sizeof(T) == 4) {  // (d <= 1024: only fp32 rows get this long)
      if (row_bytes <= 4096) return launch_grad<WideLay<T, 8>>(t, g, rows, cols, stream);
    }
  }
  if (t.d <= 128) return launch_grad<GenLay<T, 2>>(t, g, rows, cols, stream);
  if (t.d <= 1024) return launch_grad<GenLay<T, 16>>(t, g, rows, cols, stream);
  return 5;
}

}  // namespace spfa
