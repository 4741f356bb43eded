// Row-gather attention engine for gfx950 (wave64).
//
// A mask is a functor that answers two questions for a query row: how many candidate columns
// it has (deg) and which column the t-th candidate is.  The engine walks those candidates with
// an online softmax.  Work decomposition:
//
//   plan_kernel        one thread per query row: rows with short_max < deg <= medium_max go on a
//                      list of their own, longer rows are cut into segments of `seg` candidates
//                      that are appended to a work list.
//   order_kernel       copies the work list into the order it is handed out in: segments that
//                      lie at the same place in their rows together.
//   rows_kernel        one group of LPR lanes per query row (64/LPR rows per wavefront) finishes
//                      the rows with deg <= short_max on the spot.
//   medium_rows_kernel one wavefront per listed medium row, its 64/LPR groups share the row.
//   segments_kernel    persistent grid; each wavefront pulls segments off the work list, its
//                      64/LPR groups take interleaved candidates, the groups are merged with
//                      cross-lane moves, and the result is either final (single-segment row) or
//                      a partial (m, l, acc[d]) in the workspace.
//   merge_kernel       one group per multi-segment row folds that row's partials together.
//
// All of them finish a row the same way: fold the incoming (m, l, out) state in, write back.
// A batch of problems that share the mask is walked by the same kernels: rows of all problems
// form one grid, the work list is shared, partial results are per problem.
#pragma once

#include <atomic>
#include <hip/hip_ext.h>

#include "spfa_common.hpp"
#include "spfa_prep.hpp"

namespace spfa {

struct Tensors {
  const void* q;
  const void* k;
  const void* v;
  void* m;
  void* l;
  void* out;
  int64_t n_q;        // rows of one problem
  int32_t d;
  int32_t state_f32;
  // batch of independent problems that share the mask: q, out are [n_batch, n_q, d], m, l
  // [n_batch, n_q], k, v [n_batch, n_k, d]
  int64_t n_batch;    // >= 1
  int64_t kv_stride;  // n_k * d, elements between the K (V) tensors of two problems
};

// Row r of the stacked problems is row i of problem b.
__device__ __forceinline__ void split_row(const Tensors& t, int64_t r, int64_t& b, int64_t& i) {
  b = 0;
  i = r;
  if (t.n_batch > 1) {
    b = r / t.n_q;
    i = r - b * t.n_q;
  }
}

struct Counters {
  uint32_t n_items;
  uint32_t n_partials;
  uint32_t n_multi;
  uint32_t next_item;
  uint32_t overflow;
  uint32_t n_medium;
  uint32_t n_short;
  uint32_t pad[1];
};

struct Item {
  int32_t row;
  int32_t seg;
  int32_t slot;   // partial slot, or -1 when the row has a single segment
  int32_t phase;  // its place in the order the list is handed out in: segment_phase()
};

// The work list is handed out ordered by `phase`: segment j of every row that has the same number
// of segments comes at the same time, and in rows whose columns are sorted (the usual form of a
// CSR mask) these segments hold about the same columns, so the wavefronts at work at any one time
// keep to one part of K and V and meet each other's rows in the caches.  Rows of 4096 sorted
// uniform columns, fp32 d = 64, listed row by row against by phase: K + V of 16 MiB 12.1 -> 15.0
// TB/s of gathered rows, 64 MiB 8.7 -> 11.9, 256 MiB 8.0 -> 8.6.
constexpr int kPhases = 64;

struct Phases {
  uint32_t count[kPhases];  // items per phase (plan_kernel)
  uint32_t taken[kPhases];  // ... already placed (order_kernel)
};

struct MultiRow {
  int32_t row;
  int32_t slot0;
  int32_t nseg;
  int32_t pad;
};

struct Plan {
  Counters* cnt;
  uint32_t* cursor;  // next work item of segments_kernel (separate from cnt so that a plan can
                     // be shared by calls that each bring their own scratch)
  Item* items;       // ordered by phase: what segments_kernel walks
  Item* listed;      // as plan_kernel appended them
  Phases* phases;
  MultiRow* multi;
  int32_t* medium;   // rows with short_max < deg <= medium_max: one wavefront each, no queue
  int32_t* shorts;   // rows with 0 < deg <= short_max (null: no list was made)
  float* pm;
  float* pl;
  float* pacc;
  uint32_t cap_items;
  uint32_t cap_partials;
  uint32_t cap_multi;
  uint32_t cap_medium;
  uint32_t* status;  // the device's sticky status word (may be null): see device_status_word()
  int32_t use_nan;
  int64_t short_max;
  int64_t medium_max;  // == short_max: no medium rows
  int64_t seg;
};

// Bits of the device's sticky status word (spfa_device_status): what kernels found wrong with mask
// arrays they could only look at on the device.
constexpr uint32_t kStatusWorkListOverflow = 1u;  // more long-row segments than the nnz passed allows
constexpr uint32_t kStatusRowOffsets = 2u;        // row offsets decreasing or beyond nnz

// Device address of the current device's status word, or null when it cannot be looked up.
uint32_t* device_status_word();

static __global__ void reset_cursor_kernel(uint32_t* cursor) {
  if (threadIdx.x == 0) *cursor = 0;
}

static __global__ void reset_counters_kernel(Counters* cnt, Phases* ph) {
  static_assert(kPhases == kWave, "one lane per phase");
  ph->count[threadIdx.x] = 0;
  ph->taken[threadIdx.x] = 0;
  if (threadIdx.x == 0) {
    cnt->n_items = 0;
    cnt->n_partials = 0;
    cnt->n_multi = 0;
    cnt->next_item = 0;
    cnt->overflow = 0;
    cnt->n_medium = 0;
    cnt->n_short = 0;
  }
}

// Fold partial B into partial A (both un-normalised, relative to their own running max).
template <int NE>
__device__ __forceinline__ void merge_partial(float& m, float& l, float (&acc)[NE], float m2,
                                              float l2, const float (&acc2)[NE]) {
  float m_new = fmaxf(m, m2);
  if (m_new == kNegInf) return;
  float a = __expf(m - m_new);
  float b = __expf(m2 - m_new);
  l = l * a + l2 * b;
#pragma unroll
  for (int e = 0; e < NE; e++) acc[e] = acc[e] * a + acc2[e] * b;
  m = m_new;
}

// Candidates t_begin .. t_end of one row, walked by SPAN consecutive lanes (the whole wavefront
// in segments_kernel, one lane group in rows_kernel).
//
// Column indices are fetched SPAN at a time, one per lane (a coalesced load for CSR), one chunk
// ahead of their use, and handed to the groups with cross-lane reads - a column index is never
// waited for inside the gather sequence.  A batch is U candidates per group: all 2*U row loads
// of a batch are issued back to back before any is consumed.
template <class Lay, class Mask, int U_, int SPAN>
__device__ __forceinline__ void attend(const Mask& mask, const typename Mask::Row& rc,
                                       const typename Lay::elem* __restrict__ K,
                                       const typename Lay::elem* __restrict__ V, int d, float scale,
                                       const float (&q)[Lay::NE], int64_t t_begin, int64_t t_end,
                                       int lane, float& m, float& l, float (&acc)[Lay::NE]) {
  constexpr int NE = Lay::NE;
  constexpr int LPR = Lay::LPR;
  constexpr int GS = SPAN / LPR;                  // groups sharing the row
  constexpr int U = (U_ * GS > SPAN) ? SPAN / GS : U_;
  constexpr int PER = U * GS;                     // candidates per batch
  constexpr int PARTS = SPAN / PER;               // batches per index chunk
  static_assert(SPAN % LPR == 0 && PARTS >= 1 && PARTS * PER == SPAN, "bad span / unroll");
  const int ls = lane % SPAN;   // slot of this lane in an index chunk
  const int lb = lane - ls;     // first lane of the span
  const int gi = ls / LPR;      // group within the span
  const int c = lane % LPR;

  // column of candidate t + ls, or -1 (past the end / masked)
  // (an explicit mask's column is range-checked when the chunk is used, one trip after its load)
  auto fetch = [&](int64_t t) -> int {
    const int64_t tt = t + ls;
    bool valid = tt < t_end;
    int64_t col = 0;
    if constexpr (Mask::kExplicit) {
      if (valid) col = mask.col_unchecked(rc, tt);
    } else {
      if (valid) col = mask.col(rc, tt, valid);
    }
    return valid ? (int)col : -1;
  };

  typename Lay::raw qp{};
  if constexpr (Lay::kPackedDot) qp = Lay::pack_exact(q);
  int next = fetch(t_begin);
  for (int64_t tb = t_begin; tb < t_end; tb += SPAN) {
    int cur = next;
    if constexpr (Mask::kExplicit) cur = mask.in_range(cur) ? cur : -1;
    if (tb + SPAN < t_end) next = fetch(tb + SPAN);
#pragma unroll(PARTS <= 2 ? PARTS : 1)
    for (int part = 0; part < PARTS; part++) {
      if (tb + part * PER >= t_end) break;
      int cols[U];
#pragma unroll
      for (int u = 0; u < U; u++) cols[u] = shfl_i32(cur, lb + part * PER + u * GS + gi);
      typename Lay::raw kr[U], vr[U];
#pragma unroll
      for (int u = 0; u < U; u++) {
        if (cols[u] >= 0) {
          kr[u] = Lay::load_gather(K + (int64_t)cols[u] * d, c, d);
          vr[u] = Lay::load_gather(V + (int64_t)cols[u] * d, c, d);
        }
      }
      float s[U];
      float mb = kNegInf;
#pragma unroll
      for (int u = 0; u < U; u++) {
        float part_dot = 0.f;
        if (cols[u] >= 0) {
          if constexpr (Lay::kPackedDot) {
            part_dot = Lay::packed_dot(kr[u], qp);
          } else {
            float kf[NE];
            Lay::unpack(kr[u], kf);
#pragma unroll
            for (int e = 0; e < NE; e++) part_dot += q[e] * kf[e];
          }
        }
        float tot = group_sum<LPR>(part_dot) * scale;
        s[u] = cols[u] >= 0 ? tot : kNegInf;
        mb = fmaxf(mb, s[u]);
      }
      if (mb > kNegInf) {
        float m_new = fmaxf(m, mb);
        float corr = __expf(m - m_new);
        l *= corr;
#pragma unroll
        for (int e = 0; e < NE; e++) acc[e] *= corr;
#pragma unroll
        for (int u = 0; u < U; u++) {
          if (cols[u] >= 0) {
            float p = __expf(s[u] - m_new);
            l += p;
            float vf[NE];
            Lay::unpack(vr[u], vf);
#pragma unroll
            for (int e = 0; e < NE; e++) acc[e] += p * vf[e];
          }
        }
        m = m_new;
      }
    }
  }
}

// Fold the state already in memory into (m, l, acc) and write the row back.  A row that saw
// no live column (l == 0) is left untouched.
template <class Lay>
__device__ __forceinline__ void finish_row_with(const Tensors& t, int64_t row, int c, float m, float l,
                                                float (&acc)[Lay::NE], float m_in, float l_in) {
  using T = typename Lay::elem;
  constexpr int NE = Lay::NE;
  if (!(l > 0.f)) return;
  const bool sf = t.state_f32 != 0;
  T* orow = (T*)t.out + row * t.d;
  float m_new = m, l_new = l;
  if (l_in != 0.f) {
    float o_in[NE];
    typename Lay::raw r = Lay::load(orow, c, t.d);
    Lay::unpack(r, o_in);
    m_new = fmaxf(m, m_in);
    float wa = l_in * __expf(m_in - m_new);
    float wb = __expf(m - m_new);
    l_new = wa + l * wb;
    float inv = 1.f / l_new;
#pragma unroll
    for (int e = 0; e < NE; e++) acc[e] = (wa * o_in[e] + wb * acc[e]) * inv;
  } else {
    float inv = 1.f / l;
#pragma unroll
    for (int e = 0; e < NE; e++) acc[e] *= inv;
  }
  Lay::store(orow, c, t.d, acc);
  if (c == 0) {
    store_state<T>(t.m, row, m_new, sf);
    store_state<T>(t.l, row, l_new, sf);
  }
}

template <class Lay>
__device__ __forceinline__ void finish_row(const Tensors& t, int64_t row, int c, float m, float l,
                                           float (&acc)[Lay::NE]) {
  using T = typename Lay::elem;
  if (!(l > 0.f)) return;
  const bool sf = t.state_f32 != 0;
  const float m_in = load_state<T>(t.m, row, sf);
  const float l_in = load_state<T>(t.l, row, sf);
  finish_row_with<Lay>(t, row, c, m, l, acc, m_in, l_in);
}

template <class Lay>
__device__ __forceinline__ void load_q(const Tensors& t, int64_t row, int c, float (&q)[Lay::NE]) {
  using T = typename Lay::elem;
  typename Lay::raw r = Lay::load((const T*)t.q + row * t.d, c, t.d);
  Lay::unpack(r, q);
}

// inclusive prefix sum over the wavefront
__device__ __forceinline__ uint32_t wave_inclusive_sum(uint32_t x, int lane) {
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    uint32_t y = (uint32_t)__builtin_amdgcn_ds_bpermute(((lane - off) & (kWave - 1)) << 2, (int)x);
    if (lane >= off) x += y;
  }
  return x;
}

// One thread per query row: rows longer than short_max are cut into segments of plan.seg
// candidates.  A workgroup of 1024 rows reserves room for all its rows with one atomic per
// counter (the counters are shared by the whole grid: per-row, even per-wavefront, atomics
// serialise on them and dominate the kernel).
constexpr int kPlanThreads = 1024;

// The phase of segment j of the nseg of a row with deg candidates: where its middle lies in the
// row, in kPhases-ths.  The last segment of a row, the only one that can be short, comes the later
// the shorter it is (within the half phase step above its middle): the list then ends in short
// items, and the wavefronts that find it empty wait for short last items, not for full ones.
// A row of a single segment is all "last segment": such rows spread over the second half of the
// list, longest first, instead of coming all at once in the middle (their columns span all of K
// and V, so they are better taken between the others than as a block: the Zipf headline 0.707 ->
// 0.678 ms fp32, 0.406 -> 0.411 ms bf16, eight heads of it 5.72 -> 5.08 ms; starting them at the
// front, at a quarter or at three quarters of the list instead of the middle: 0.696, 0.686, 0.700).
__device__ __forceinline__ uint32_t segment_phase(uint32_t j, uint32_t nseg, int64_t deg, int64_t seg) {
  uint32_t ph = (uint32_t)(((uint64_t)(2 * j + 1) * kPhases) / (2 * (uint64_t)nseg));
  if (j + 1 == nseg) {
    const uint32_t room = kPhases - ph;  // phases from the middle to the end of the row
    const int64_t missing = (int64_t)nseg * seg - deg;  // 0 ... seg - 1
    ph += (uint32_t)((missing * room) / seg);
  }
  return ph < (uint32_t)kPhases ? ph : (uint32_t)kPhases - 1u;
}

template <class Mask>
__global__ __launch_bounds__(kPlanThreads) void plan_kernel(int64_t n_q, Mask mask, Plan plan) {
  constexpr int NW = kPlanThreads / kWave;
  __shared__ uint32_t wave_tot[NW][5];
  __shared__ uint32_t block_base[5];
  __shared__ uint32_t block_ok;
  __shared__ uint32_t phase_count[kPhases];
  const int lane = lane_id();
  const int wave = threadIdx.x / kWave;
  const int64_t row = (int64_t)blockIdx.x * kPlanThreads + threadIdx.x;
  if (threadIdx.x < kPhases) phase_count[threadIdx.x] = 0;
  int64_t deg = 0;
  if (row < n_q) {
    deg = mask.row(row).deg;
    if constexpr (Mask::kExplicit) {
      // offsets that run backwards or past the entry count: the row was cut to what exists
      if (plan.status != nullptr && !mask.consistent(row)) atomicOr(plan.status, kStatusRowOffsets);
    }
  }
  const bool is_medium = deg > plan.short_max && deg <= plan.medium_max;
  const bool is_long = deg > plan.medium_max;
  const uint32_t nseg = is_long ? (uint32_t)((deg + plan.seg - 1) / plan.seg) : 0u;
  const uint32_t multi = nseg > 1 ? 1u : 0u;
  const uint32_t npart = multi ? nseg : 0u;
  __syncthreads();  // (phase_count is zero)
  for (uint32_t j = 0; j < nseg; j++) atomicAdd(&phase_count[segment_phase(j, nseg, deg, plan.seg)], 1u);
  const uint32_t med = is_medium ? 1u : 0u;
  const uint32_t sht = (deg > 0 && deg <= plan.short_max) ? 1u : 0u;
  const uint32_t inc_items = wave_inclusive_sum(nseg, lane);
  const uint32_t inc_part = wave_inclusive_sum(npart, lane);
  const uint32_t inc_multi = wave_inclusive_sum(multi, lane);
  const uint32_t inc_med = wave_inclusive_sum(med, lane);
  const uint32_t inc_sht = wave_inclusive_sum(sht, lane);
  if (lane == kWave - 1) {
    wave_tot[wave][0] = inc_items;
    wave_tot[wave][1] = inc_part;
    wave_tot[wave][2] = inc_multi;
    wave_tot[wave][3] = inc_med;
    wave_tot[wave][4] = inc_sht;
  }
  __syncthreads();
  if (threadIdx.x < 5) {
    // one lane per counter (work items, partial results, multi-segment rows, medium rows, short
    // rows): its exclusive prefix over the wavefronts, then ONE reservation for the workgroup -
    // the five atomics travel together instead of one after the other
    const int kk = threadIdx.x;
    uint32_t tot = 0;
    for (int w = 0; w < NW; w++) {
      const uint32_t x = wave_tot[w][kk];
      wave_tot[w][kk] = tot;
      tot += x;
    }
    uint32_t* const counter = kk == 0 ? &plan.cnt->n_items : kk == 1 ? &plan.cnt->n_partials
                            : kk == 2 ? &plan.cnt->n_multi : kk == 3 ? &plan.cnt->n_medium : &plan.cnt->n_short;
    // (as many short-row slots as rows: that list cannot overflow)
    const uint32_t cap = kk == 0 ? plan.cap_items : kk == 1 ? plan.cap_partials : kk == 2 ? plan.cap_multi
                       : kk == 3 ? plan.cap_medium : 0xffffffffu;
    uint32_t base = 0;
    bool bad = false;
    if (tot) {
      base = atomicAdd(counter, tot);
      bad = base + tot > cap || base + tot < base;
    }
    block_base[kk] = base;
    const bool any_bad = __ballot(bad) != 0;
    if (kk == 0) {
      block_ok = any_bad ? 0u : 1u;
      if (any_bad) {
        atomicOr(&plan.cnt->overflow, 1u);
        if (plan.status != nullptr) atomicOr(plan.status, kStatusWorkListOverflow);
      }
    }
  }
  __syncthreads();
  if (sht) plan.shorts[block_base[4] + wave_tot[wave][4] + inc_sht - 1] = (int32_t)row;
  if (!block_ok) return;
  if (threadIdx.x < kPhases && phase_count[threadIdx.x] != 0)
    atomicAdd(&plan.phases->count[threadIdx.x], phase_count[threadIdx.x]);
  if (is_medium) plan.medium[block_base[3] + wave_tot[wave][3] + inc_med - 1] = (int32_t)row;
  if (!is_long) return;
  const uint32_t my_item = block_base[0] + wave_tot[wave][0] + inc_items - nseg;
  const uint32_t my_slot = block_base[1] + wave_tot[wave][1] + inc_part - npart;
  if (multi) {
    MultiRow mr;
    mr.row = (int32_t)row;
    mr.slot0 = (int32_t)my_slot;
    mr.nseg = (int32_t)nseg;
    mr.pad = 0;
    plan.multi[block_base[2] + wave_tot[wave][2] + inc_multi - 1] = mr;
  }
  for (uint32_t j = 0; j < nseg; j++) {
    Item it;
    it.row = (int32_t)row;
    it.seg = (int32_t)j;
    it.slot = multi ? (int32_t)(my_slot + j) : -1;
    it.phase = (int32_t)segment_phase(j, nseg, deg, plan.seg);
    plan.listed[my_item + j] = it;
  }
}

// Copies the work list into the order segments_kernel takes it in: by phase, in any order inside
// a phase (which item a wavefront gets has no influence on any result).  The work of one
// wavefront on 64 items.  When every item has the same phase (single-segment rows of one length)
// the list stays where it is and segments_kernel reads it there: one reservation per wavefront
// on the one phase's counter took 17 us for 66 K items.
// (Done by extra workgroups of the rows_kernel launch, which does not look at the list, this cost
// every workgroup of that kernel a scalar load and a wait before its first useful instruction:
// 224 -> 242 us on the 65 K tiny workgroups of a 1 M-row call, against 5 us for a launch.)
__device__ __forceinline__ void order_wave(const Plan& plan, uint32_t wave_index, int lane) {
  if (plan.cnt->overflow) return;
  uint32_t n_items = plan.cnt->n_items;
  if (n_items > plan.cap_items) n_items = plan.cap_items;
  if (wave_index * (uint32_t)kWave >= n_items) return;
  // lane p: first place of phase p in the ordered list
  const uint32_t n_ph = plan.phases->count[lane];
  if (__ballot(n_ph == n_items) != 0) return;  // one phase: see work_list()
  const uint32_t start = wave_inclusive_sum(n_ph, lane) - n_ph;
  const uint32_t i = wave_index * (uint32_t)kWave + (uint32_t)lane;
  const bool live = i < n_items;
  Item it{};
  uint32_t ph = 0;
  if (live) {
    it = plan.listed[i];
    ph = (uint32_t)it.phase & (kPhases - 1);
  }
  // the lanes that hold the same phase, and the first of them
  uint64_t same = 0;
  int leader = lane;
  uint64_t todo = __ballot(live);
  while (todo) {
    const int first = __ffsll((long long)todo) - 1;
    const uint32_t ph0 = (uint32_t)shfl_i32((int)ph, first);
    const uint64_t grp = __ballot(live && ph == ph0);
    if (live && ph == ph0) {
      same = grp;
      leader = first;
    }
    todo &= ~grp;
  }
  // one reservation per wavefront and phase (an atomic per item on the few phases a mask of
  // equally long rows has would take longer than the attention), all of them in one round trip
  uint32_t base = 0;
  if (live && lane == leader) base = atomicAdd(&plan.phases->taken[ph], (uint32_t)__popcll(same));
  base = (uint32_t)shfl_i32((int)base, leader);
  const uint32_t first_place = (uint32_t)shfl_i32((int)start, (int)ph);
  if (live) {
    const uint32_t at = first_place + base + (uint32_t)__popcll(same & (((uint64_t)1 << lane) - 1));
    if (at < n_items) plan.items[at] = it;
  }
}

template <class Lay, class Mask>
__device__ __forceinline__ void rows_body(const Tensors& t, const Mask& mask, const Plan& plan, int64_t block) {
  using T = typename Lay::elem;
  constexpr int NE = Lay::NE;
  constexpr int LPR = Lay::LPR;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int g = lane / LPR;
  const int c = lane % LPR;
  const int64_t idx = (block * 4 + wave) * Lay::GROUPS + g;
  // A mask whose rows are mostly empty (and stay untouched) would spend a lane group on every
  // empty row and a wavefront on every four rows that hold one short row among them: the rows are
  // then taken from the list of non-empty short rows that plan_kernel made.
  int64_t row, b, ri;  // row among all problems, problem, row inside the problem
  const uint32_t n_short = plan.shorts != nullptr ? plan.cnt->n_short : 0u;
  if (plan.shorts != nullptr && !plan.use_nan && !plan.cnt->overflow && (int64_t)n_short * 2 <= t.n_q) {
    if (idx >= (int64_t)n_short * t.n_batch) return;
    b = idx / n_short;
    ri = plan.shorts[idx - b * n_short];
    row = b * t.n_q + ri;
  } else {
    row = idx;
    if (row >= t.n_q * t.n_batch) return;
    split_row(t, row, b, ri);
  }

  const typename Mask::Row rc = mask.row(ri);
  const int64_t deg = rc.deg;
  if (deg <= 0) {
    if (plan.use_nan) {
      float nanv[NE];
#pragma unroll
      for (int e = 0; e < NE; e++) nanv[e] = __builtin_nanf("");
      Lay::store((T*)t.out + row * t.d, c, t.d, nanv);
    }
    return;
  }

  if (deg <= plan.short_max) {
    float q[NE];
    load_q<Lay>(t, row, c, q);
    float m = kNegInf, l = 0.f, acc[NE];
#pragma unroll
    for (int e = 0; e < NE; e++) acc[e] = 0.f;
    const float scale = 1.0f / sqrtf((float)t.d);
    attend<Lay, Mask, Lay::U_SHORT, LPR>(mask, rc, (const T*)t.k + b * t.kv_stride,
                                         (const T*)t.v + b * t.kv_stride, t.d, scale, q, 0, deg, lane,
                                         m, l, acc);
    finish_row<Lay>(t, row, c, m, l, acc);
  }
  // longer rows were cut into segments by plan_kernel and belong to segments_kernel
}

template <class Lay, class Mask>
__global__ __launch_bounds__(256) void rows_kernel(Tensors t, Mask mask, Plan plan) {
  rows_body<Lay, Mask>(t, mask, plan, (int64_t)blockIdx.x);
}

// The list segments_kernel walks: the ordered one, or the list as appended when all its items
// have one phase (order_wave then leaves it alone).
__device__ __forceinline__ const Item* work_list(const Plan& plan, uint32_t n_items, int lane) {
  const uint32_t n_ph = plan.phases->count[lane];
  return __ballot(n_ph == n_items) != 0 ? plan.listed : plan.items;
}

static __global__ __launch_bounds__(256) void order_kernel(Plan plan) {
  order_wave(plan, blockIdx.x * 4u + (threadIdx.x >> 6), (int)(threadIdx.x & (kWave - 1)));
}

template <class Lay, class Mask>
__global__ __launch_bounds__(256) void segments_kernel(Tensors t, Mask mask, Plan plan) {
  using T = typename Lay::elem;
  constexpr int NE = Lay::NE;
  constexpr int LPR = Lay::LPR;
  const int lane = threadIdx.x & (kWave - 1);
  const int g = lane / LPR;
  const int c = lane % LPR;
  if (plan.cnt->overflow) return;
  uint32_t n_items = plan.cnt->n_items;
  if (n_items > plan.cap_items) n_items = plan.cap_items;
  // (an empty list: without this every wavefront would still queue up at the cursor once, 20 us
  // for the 2048 of them)
  if (n_items == 0) return;
  // every problem of the batch walks the same work list (the host keeps items * batch < 2^32)
  const uint32_t n_work = n_items * (uint32_t)t.n_batch;
  const float scale = 1.0f / sqrtf((float)t.d);
  const Item* const items = work_list(plan, n_items, lane);

  // The first item of a wavefront is the one with its own number, the later ones come off the
  // cursor: 2048 wavefronts that all begin with an atomic on the one address wait up to 20 us
  // for each other before the first K row is asked for.
  const uint32_t n_waves = gridDim.x * 4u;
  uint32_t work = (uint32_t)__builtin_amdgcn_readfirstlane((int)(blockIdx.x * 4u + (threadIdx.x >> 6)));
  while (work < n_work) {
    uint32_t idx = work;
    uint32_t b = 0;
    if (t.n_batch > 1) {
      b = idx / n_items;
      idx -= b * n_items;
    }
    const Item it = items[idx];
    const int64_t row = (int64_t)b * t.n_q + it.row;
    const int64_t slot = (int64_t)b * plan.cap_partials + it.slot;
    const typename Mask::Row rc = mask.row(it.row);
    const int64_t t0 = (int64_t)it.seg * plan.seg;
    int64_t t1 = t0 + plan.seg;
    if (t1 > rc.deg) t1 = rc.deg;

    float q[NE];
    load_q<Lay>(t, row, c, q);
    float m = kNegInf, l = 0.f, acc[NE];
#pragma unroll
    for (int e = 0; e < NE; e++) acc[e] = 0.f;
    attend<Lay, Mask, Lay::U, kWave>(mask, rc, (const T*)t.k + (int64_t)b * t.kv_stride,
                                     (const T*)t.v + (int64_t)b * t.kv_stride, t.d, scale, q, t0, t1,
                                     lane, m, l, acc);

    // butterfly over the groups of the wavefront
#pragma unroll
    for (int off = LPR; off < kWave; off <<= 1) {
      float m2 = shfl_xor_f32(m, off);
      float l2 = shfl_xor_f32(l, off);
      float acc2[NE];
#pragma unroll
      for (int e = 0; e < NE; e++) acc2[e] = shfl_xor_f32(acc[e], off);
      merge_partial<NE>(m, l, acc, m2, l2, acc2);
    }

    if (g == 0) {
      if (it.slot < 0) {
        finish_row<Lay>(t, row, c, m, l, acc);
      } else {
        Lay::store_f32(plan.pacc + slot * t.d, c, t.d, acc);
        if (c == 0) {
          plan.pm[slot] = m;
          plan.pl[slot] = l;
        }
      }
    }
    uint32_t next = 0;
    if (lane == 0) next = atomicAdd(plan.cursor, 1u);
    work = n_waves + (uint32_t)__builtin_amdgcn_readfirstlane((int)next);
    // Every lane of the wavefront must take the next trip together: the work index is read
    // across lanes.  A convergent operation in the only latch keeps the optimiser from giving
    // the lanes that wrote the statistics a back edge of their own.
    __builtin_amdgcn_wave_barrier();
  }
}

// Rows of medium length (short_max < deg <= medium_max): one wavefront per row and problem, the
// lane groups share the row's candidates as in segments_kernel, but launched as an ordinary
// grid.  A row of this size is a handful of dependent memory round trips and little else: in
// the persistent kernel (two wavefronts per SIMD) little hides them, here the other resident
// wavefronts do.  (A device-sized grid with a stride loop instead of one wavefront per list
// slot was measured slower: 1.02 against 0.66 ms on 64 x 4096 rows of ~83 entries.)
// UM: neighbours in flight per lane group.  Rows whose columns are sorted (the usual form of a CSR
// mask) are walked from low to high columns by every wavefront, so the wavefronts resident at a
// time touch about the same part of K and V at the same time; smaller batches with more
// wavefronts resident keep them closer together, and while K and V are not much larger than the
// caches that is worth more than the loads in flight per wavefront (uniform rows of 192 sorted
// columns, 65536 tokens, fp32 d = 64: 8.8 TB/s of gathered rows with 8, 11.1 with 4, 9.1 with 2;
// 20000 tokens: 14.1 / 15.2 / 16.5; from 262144 tokens on it makes no difference).
template <class Lay, class Mask, int UM>
__device__ __forceinline__ void medium_rows_body(const Tensors& t, const Mask& mask, const Plan& plan, int64_t block) {
  using T = typename Lay::elem;
  constexpr int NE = Lay::NE;
  constexpr int LPR = Lay::LPR;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int g = lane / LPR;
  const int c = lane % LPR;
  if (plan.cnt->overflow) return;
  uint32_t n_medium = plan.cnt->n_medium;
  if (n_medium > plan.cap_medium) n_medium = plan.cap_medium;
  int64_t idx = block * 4 + wave;
  if (idx >= (int64_t)n_medium * t.n_batch) return;
  int64_t b = 0;
  if (t.n_batch > 1) {
    b = idx / n_medium;
    idx -= b * n_medium;
  }
  const int64_t ri = plan.medium[idx];
  const int64_t row = b * t.n_q + ri;
  const typename Mask::Row rc = mask.row(ri);
  const float scale = 1.0f / sqrtf((float)t.d);

  float q[NE];
  load_q<Lay>(t, row, c, q);
  float m = kNegInf, l = 0.f, acc[NE];
#pragma unroll
  for (int e = 0; e < NE; e++) acc[e] = 0.f;
  attend<Lay, Mask, UM, kWave>(mask, rc, (const T*)t.k + b * t.kv_stride, (const T*)t.v + b * t.kv_stride,
                               t.d, scale, q, 0, rc.deg, lane, m, l, acc);
#pragma unroll
  for (int off = LPR; off < kWave; off <<= 1) {
    float m2 = shfl_xor_f32(m, off);
    float l2 = shfl_xor_f32(l, off);
    float acc2[NE];
#pragma unroll
    for (int e = 0; e < NE; e++) acc2[e] = shfl_xor_f32(acc[e], off);
    merge_partial<NE>(m, l, acc, m2, l2, acc2);
  }
  if (g == 0) finish_row<Lay>(t, row, c, m, l, acc);
}

template <class Lay, class Mask, int UM = Lay::U_MEDIUM>
__global__ __launch_bounds__(256) void medium_rows_kernel(Tensors t, Mask mask, Plan plan) {
  medium_rows_body<Lay, Mask, UM>(t, mask, plan, (int64_t)blockIdx.x);
}

// The work list walked by an ordinary grid, one wavefront per item in list order, instead of by
// segments_kernel's persistent wavefronts: the better of the two while K and V are not much
// larger than the caches.  Three or four wavefronts per SIMD (127 / 139 registers at fp32 / bf16
// d = 64) with eight neighbours in flight per lane group then draw more from the caches than two
// with sixteen, and, dispatched in list order, they stay as close together in the list as the
// persistent ones.  The Zipf mask at N = 16 K /
// 32 K / 64 K / 128 K / 256 K / 512 K / 1 M tokens, persistent -> grid, whole call: fp32 d = 64
// - 33 / - 23 / - 13 / - 2 / + 1 / + 2 / + 3 %, bf16 d = 64 - 42 / - 38 / - 29 / - 19 / - 8 / 0 / + 3 %,
// fp32 d = 128 - 14 / - 6 / + 1 / + 2 %, bf16 d = 128 - 28 / - 17 / - 8 / - 1 / + 2 %; eight heads of
// the 128 K fp32 mask in one call + 5 %.  Taken when K + V of one problem are at most 48 MiB (96 MiB for rows of at most 128 bytes).
template <class Lay, class Mask, int UM>
__device__ __forceinline__ void items_grid_body(const Tensors& t, const Mask& mask, const Plan& plan, int64_t block) {
  using T = typename Lay::elem;
  constexpr int NE = Lay::NE;
  constexpr int LPR = Lay::LPR;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int g = lane / LPR;
  const int c = lane % LPR;
  if (plan.cnt->overflow) return;
  uint32_t n_items = plan.cnt->n_items;
  if (n_items > plan.cap_items) n_items = plan.cap_items;
  int64_t idx = block * 4 + wave;
  if (idx >= (int64_t)n_items * t.n_batch) return;
  int64_t b = 0;
  if (t.n_batch > 1) {
    b = idx / n_items;
    idx -= b * n_items;
  }
  const Item* const items = work_list(plan, n_items, lane);
  const Item it = items[idx];
  const int64_t row = b * t.n_q + it.row;
  const int64_t slot = b * plan.cap_partials + it.slot;
  const typename Mask::Row rc = mask.row(it.row);
  const int64_t t0 = (int64_t)it.seg * plan.seg;
  int64_t t1 = t0 + plan.seg;
  if (t1 > rc.deg) t1 = rc.deg;
  const float scale = 1.0f / sqrtf((float)t.d);
  float q[NE];
  load_q<Lay>(t, row, c, q);
  float m = kNegInf, l = 0.f, acc[NE];
#pragma unroll
  for (int e = 0; e < NE; e++) acc[e] = 0.f;
  attend<Lay, Mask, UM, kWave>(mask, rc, (const T*)t.k + b * t.kv_stride, (const T*)t.v + b * t.kv_stride,
                               t.d, scale, q, t0, t1, lane, m, l, acc);
#pragma unroll
  for (int off = LPR; off < kWave; off <<= 1) {
    float m2 = shfl_xor_f32(m, off);
    float l2 = shfl_xor_f32(l, off);
    float acc2[NE];
#pragma unroll
    for (int e = 0; e < NE; e++) acc2[e] = shfl_xor_f32(acc[e], off);
    merge_partial<NE>(m, l, acc, m2, l2, acc2);
  }
  if (g == 0) {
    if (it.slot < 0) {
      finish_row<Lay>(t, row, c, m, l, acc);
    } else {
      Lay::store_f32(plan.pacc + slot * t.d, c, t.d, acc);
      if (c == 0) {
        plan.pm[slot] = m;
        plan.pl[slot] = l;
      }
    }
  }
}

template <class Lay, class Mask, int UM = Lay::U_MEDIUM>
__global__ __launch_bounds__(256) void items_grid_kernel(Tensors t, Mask mask, Plan plan) {
  items_grid_body<Lay, Mask, UM>(t, mask, plan, (int64_t)blockIdx.x);
}

// The three row kernels of an explicit mask in one launch: the workgroups of the long rows' items
// first, then those of the medium rows, then those of the short rows.  None of the three fills
// the device alone at moderate sizes (a chain of dependent round trips per wavefront each), so
// one after the other they add up to the sum of their latencies, side by side to the longest.
// The Zipf mask at 8192 / 16384 / 32768 / 65536 tokens, three launches -> one: fp32 0.085 -> 0.060 /
// 0.104 -> 0.086 / 0.179 -> 0.154 / 0.300 -> 0.291 ms, bf16 0.064 -> 0.044 / 0.074 -> 0.064 / 0.106 ->
// 0.101 / 0.168 -> 0.172 ms (and 0.316 -> 0.334 at 131072: the short rows then run at the register
// count of the long rows' kernel, and there are enough of them to notice); planned calls at 2048
// ... 16384 tokens 0.048 -> 0.029, 0.050 -> 0.031, 0.067 -> 0.043, 0.086 -> 0.068 ms fp32.  Taken for
// calls of up to kFusedRowsMax rows whose long rows are walked by an ordinary grid anyway.
constexpr int64_t kFusedRowsMax = 32768;
template <class Lay, class Mask, int UM = Lay::U_MEDIUM>  // (UM: the medium rows' batch size)
__global__ __launch_bounds__(256) void explicit_rows_kernel(Tensors t, Mask mask, Plan plan,
                                                            uint32_t item_blocks, uint32_t medium_blocks) {
  if (blockIdx.x < item_blocks)
    items_grid_body<Lay, Mask, Lay::U_MEDIUM>(t, mask, plan, (int64_t)blockIdx.x);
  else if (blockIdx.x < item_blocks + medium_blocks)
    medium_rows_body<Lay, Mask, UM>(t, mask, plan, (int64_t)(blockIdx.x - item_blocks));
  else
    rows_body<Lay, Mask>(t, mask, plan, (int64_t)(blockIdx.x - item_blocks - medium_blocks));
}

// Small problems in one launch: one wavefront per row and problem (empty rows included), eight
// rows per workgroup.  The general path is five launches and a work list; below a few tens of
// thousands of rows those cost more than the attention (4096 rows of ~83 entries: 37 us, against
// 13 us here).  A row of more than kWholeRowsLong candidates is left for a second phase in which
// the eight wavefronts of the workgroup share it (a contiguous run of candidates each) and fold
// their partial results through LDS, so that one very long row costs an eighth of what a single
// wavefront would take (256, not 1024: 4096 rows of the Zipf mask 0.068 -> 0.056 ms fp32, 0.052 ->
// 0.049 ms bf16; rows of ~83 entries do not notice).
constexpr int kWholeRowsWaves = 8;
constexpr int64_t kWholeRowsLong = 256;

template <class Lay, class Mask>
__global__ __launch_bounds__(kWholeRowsWaves* kWave) void whole_rows_kernel(Tensors t, Mask mask, int use_nan,
                                                                            uint32_t* status) {
  using T = typename Lay::elem;
  constexpr int NE = Lay::NE;
  constexpr int LPR = Lay::LPR;
  constexpr int W = kWholeRowsWaves;
  constexpr int DP = NE * LPR;  // padded row length
  __shared__ float part_acc[W * DP];
  __shared__ float part_m[W], part_l[W];
  __shared__ int long_rows[W];
  __shared__ int n_long_s;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int g = lane / LPR;
  const int c = lane % LPR;
  const int64_t total = t.n_q * t.n_batch;
  const int64_t row0 = (int64_t)blockIdx.x * W;
  const float scale = 1.0f / sqrtf((float)t.d);
  if (threadIdx.x == 0) n_long_s = 0;
  __syncthreads();

  // the gather over candidates [t0, t1) of row `row`, folded over the groups of the wavefront
  auto walk = [&](int64_t row, int64_t t0, int64_t t1, float& m, float& l, float (&acc)[NE]) {
    int64_t b, ri;
    split_row(t, row, b, ri);
    const typename Mask::Row rc = mask.row(ri);
    float q[NE];
    load_q<Lay>(t, row, c, q);
    m = kNegInf;
    l = 0.f;
#pragma unroll
    for (int e = 0; e < NE; e++) acc[e] = 0.f;
    if (t1 > rc.deg) t1 = rc.deg;
    if (t0 < t1)
      attend<Lay, Mask, Lay::U_MEDIUM, kWave>(mask, rc, (const T*)t.k + b * t.kv_stride,
                                              (const T*)t.v + b * t.kv_stride, t.d, scale, q, t0, t1, lane,
                                              m, l, acc);
#pragma unroll
    for (int off = LPR; off < kWave; off <<= 1) {
      float m2 = shfl_xor_f32(m, off);
      float l2 = shfl_xor_f32(l, off);
      float acc2[NE];
#pragma unroll
      for (int e = 0; e < NE; e++) acc2[e] = shfl_xor_f32(acc[e], off);
      merge_partial<NE>(m, l, acc, m2, l2, acc2);
    }
  };

  // ---- phase 1: a wavefront per row
  {
    const int64_t row = row0 + wave;
    if (row < total) {
      int64_t b, ri;
      split_row(t, row, b, ri);
      const int64_t deg = mask.row(ri).deg;
      if constexpr (Mask::kExplicit) {
        if (status != nullptr && lane == 0 && !mask.consistent(ri)) atomicOr(status, kStatusRowOffsets);
      }
      if (deg <= 0) {
        if (use_nan && g == 0) {
          float nanv[NE];
#pragma unroll
          for (int e = 0; e < NE; e++) nanv[e] = __builtin_nanf("");
          Lay::store((T*)t.out + row * t.d, c, t.d, nanv);
        }
      } else if (deg > kWholeRowsLong) {
        if (lane == 0) long_rows[atomicAdd(&n_long_s, 1)] = wave;
      } else {
        float m, l, acc[NE];
        walk(row, 0, deg, m, l, acc);
        if (g == 0) finish_row<Lay>(t, row, c, m, l, acc);
      }
    }
  }
  __syncthreads();

  // ---- phase 2: the workgroup's long rows, one after the other, shared by all wavefronts
  const int n_long = n_long_s;
  for (int i = 0; i < n_long; i++) {
    const int64_t row = row0 + long_rows[i];
    int64_t b, ri;
    split_row(t, row, b, ri);
    const int64_t deg = mask.row(ri).deg;
    int64_t per = (deg + W - 1) / W;
    per = (per + kWave - 1) / kWave * kWave;
    float m, l, acc[NE];
    walk(row, wave * per, (wave + 1) * per, m, l, acc);
    if (g == 0) {
      Lay::store_f32(part_acc + wave * DP, c, t.d, acc);
      if (c == 0) {
        part_m[wave] = m;
        part_l[wave] = l;
      }
    }
    __syncthreads();
    if (wave == 0 && g == 0) {
      // (wavefront 0 still holds its own partial in registers)
      for (int w2 = 1; w2 < W; w2++) {
        float acc2[NE];
        Lay::load_f32(part_acc + w2 * DP, c, t.d, acc2);
        merge_partial<NE>(m, l, acc, part_m[w2], part_l[w2], acc2);
      }
      finish_row<Lay>(t, row, c, m, l, acc);
    }
    __syncthreads();
  }
}

template <class Lay>
__global__ __launch_bounds__(256) void merge_kernel(Tensors t, Plan plan) {
  constexpr int NE = Lay::NE;
  constexpr int LPR = Lay::LPR;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int g = lane / LPR;
  const int c = lane % LPR;
  if (plan.cnt->overflow) return;
  uint32_t n_multi = plan.cnt->n_multi;
  if (n_multi > plan.cap_multi) n_multi = plan.cap_multi;
  int64_t idx = ((int64_t)blockIdx.x * 4 + wave) * Lay::GROUPS + g;
  if (idx >= (int64_t)n_multi * t.n_batch) return;
  int64_t b = 0;
  if (t.n_batch > 1) {
    b = idx / n_multi;
    idx -= b * n_multi;
  }
  const MultiRow mr = plan.multi[idx];
  float m = kNegInf, l = 0.f, acc[NE];
#pragma unroll
  for (int e = 0; e < NE; e++) acc[e] = 0.f;
  // four partials per trip, all of them asked for before the first is folded in (a trip per
  // partial is a memory round trip per partial: 8.1 -> 5 us for rows of up to eight segments)
  for (int j0 = 0; j0 < mr.nseg; j0 += 4) {
    float pm4[4], pl4[4], acc4[4][NE];
#pragma unroll
    for (int u = 0; u < 4; u++) {
      pm4[u] = kNegInf;
      pl4[u] = 0.f;
#pragma unroll
      for (int e = 0; e < NE; e++) acc4[u][e] = 0.f;
      if (j0 + u < mr.nseg) {
        const int64_t slot = b * plan.cap_partials + mr.slot0 + j0 + u;
        Lay::load_f32(plan.pacc + slot * t.d, c, t.d, acc4[u]);
        pm4[u] = plan.pm[slot];
        pl4[u] = plan.pl[slot];
      }
    }
#pragma unroll
    for (int u = 0; u < 4; u++) merge_partial<NE>(m, l, acc, pm4[u], pl4[u], acc4[u]);
  }
  finish_row<Lay>(t, b * t.n_q + mr.row, c, m, l, acc);
}

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------
struct EngineSizing {
  int64_t nnz_bound;     // upper bound on the sum of deg over all rows
  int64_t max_deg;       // upper bound on deg of one row
  int64_t short_max;     // rows up to this many candidates are finished by rows_kernel
  int64_t medium_max;    // rows up to this many get a wavefront of their own (0: same as short_max)
  int64_t seg;           // segment length for longer rows
  int64_t n_long_bound;  // upper bound on the number of rows with deg > short_max
  int medium_batch;      // neighbours in flight per lane group in medium_rows_kernel (0: the layout's)
  bool items_on_grid;    // the work list is walked by items_grid_kernel (explicit masks)
  bool items_as_listed;  // ... in the order plan_kernel appended it in: no order_kernel (plain calls only)
};

struct WorkspaceLayout {
  size_t off_cnt, off_phases, off_items, off_listed, off_multi, off_medium, off_short, off_pm, off_pl, off_pacc, total;
  uint32_t cap_items, cap_partials, cap_multi, cap_medium, cap_short;
};


inline int64_t pow2_ceil(int64_t x) {
  int64_t p = 1;
  while (p < x) p <<= 1;
  return p;
}

inline WorkspaceLayout engine_workspace(const EngineSizing& s, int64_t n_q, int64_t d,
                                        int64_t n_batch = 1) {
  WorkspaceLayout w{};
  int64_t cap_items = 0, cap_partials = 0, cap_multi = 0, cap_medium = 0, cap_short = 0;
  if (s.max_deg > s.short_max) {
    cap_short = n_q;
    int64_t n_long = s.nnz_bound / (s.short_max + 1);
    if (n_long > n_q) n_long = n_q;
    if (n_long > s.n_long_bound) n_long = s.n_long_bound;
    if (s.medium_max > s.short_max) cap_medium = n_long + 1;
    cap_items = s.nnz_bound / s.seg + n_long + 1;
    int64_t n_multi = s.nnz_bound / (s.seg + 1);
    if (n_multi > n_long) n_multi = n_long;
    cap_multi = n_multi + 1;
    cap_partials = s.nnz_bound / s.seg + n_multi + 1;
  }
  w.cap_items = (uint32_t)cap_items;
  w.cap_partials = (uint32_t)cap_partials;
  w.cap_multi = (uint32_t)cap_multi;
  w.cap_medium = (uint32_t)cap_medium;
  w.cap_short = (uint32_t)cap_short;
  size_t off = 0;
  w.off_cnt = off;      off = align_up(off + sizeof(Counters), 256);
  w.off_phases = off;   off = align_up(off + sizeof(Phases), 256);
  w.off_items = off;    off = align_up(off + (size_t)cap_items * sizeof(Item), 256);
  w.off_listed = off;   off = align_up(off + (size_t)cap_items * sizeof(Item), 256);
  w.off_multi = off;    off = align_up(off + (size_t)cap_multi * sizeof(MultiRow), 256);
  w.off_medium = off;   off = align_up(off + (size_t)cap_medium * sizeof(int32_t), 256);
  w.off_short = off;    off = align_up(off + (size_t)cap_short * sizeof(int32_t), 256);
  // (the work list is shared by the problems of a batch, the partial results are not)
  const size_t nb = (size_t)(n_batch > 1 ? n_batch : 1);
  w.off_pm = off;       off = align_up(off + nb * (size_t)cap_partials * sizeof(float), 256);
  w.off_pl = off;       off = align_up(off + nb * (size_t)cap_partials * sizeof(float), 256);
  w.off_pacc = off;     off = align_up(off + nb * (size_t)cap_partials * (size_t)d * sizeof(float), 256);
  w.total = off;
  return w;
}

// Raises a kernel's dynamic-LDS limit to `bytes`, once per device: `raised` is the caller's table
// of kLdsLimitDevices flags for that kernel (atomic: callers may be on several host threads; two
// that meet here both set the attribute, which is idempotent).  A device beyond the table gets
// the attribute set on every call.  False when the runtime refuses.
constexpr int kLdsLimitDevices = 64;
inline bool raise_lds_limit(const void* kernel, int bytes, std::atomic<bool>* raised) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) return false;
  const bool tabled = dev >= 0 && dev < kLdsLimitDevices;
  if (tabled && raised[dev].load(std::memory_order_acquire)) return true;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  if (tabled) raised[dev].store(true, std::memory_order_release);
  return true;
}

// optional event pair recorded around the dominant kernel (see spfa_set_kernel_events)
struct KernelEvents {
  hipEvent_t start = nullptr;
  hipEvent_t stop = nullptr;
};
KernelEvents& kernel_events();

// Launches `kernel`; with a pair of events set, the pair receives the start and end time stamps
// of this very dispatch (no extra packets in the queue), so that their difference is the
// kernel's own duration even when launches follow each other back to back on the stream.
template <typename... KArgs, typename... Args>
inline void launch_maybe_timed(const KernelEvents& ev, void (*kernel)(KArgs...), dim3 grid, dim3 block,
                               hipStream_t stream, Args&&... args) {
  if (ev.start != nullptr && ev.stop != nullptr)
    hipExtLaunchKernelGGL(kernel, grid, block, 0, stream, ev.start, ev.stop, 0, static_cast<KArgs>(args)...);
  else
    hipLaunchKernelGGL(kernel, grid, block, 0, stream, static_cast<KArgs>(args)...);
}

constexpr int kSegmentWorkgroupsPerCu = 2;
// whole_rows_kernel takes a call of at most this many rows (over all problems), keys and
// candidates.  What it cannot do is share one very long row over the device, so the limits keep
// such a row short: K and V of 16384 keys stay in the caches, a row of distinct columns is at
// most 16384 long (8 wavefronts x 32 trips); only repeated columns can make a row longer, up to
// all the candidates (measured: 500 K candidates in one row of 64, K and V of 512 K rows, 4.8 ms
// here against 1.5 ms on the general path - hence the limit on keys).
constexpr int64_t kWholeRowsMaxRows = 16384;
constexpr int64_t kWholeRowsMaxKeys = 16384;
constexpr int64_t kWholeRowsMaxEntries = (int64_t)1 << 19;

// compute units of the current device (looked up once per device)
inline int device_cu_count() {
  constexpr int kMaxDevices = 64;
  static int cus[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
  if (cus[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cus[dev] = n;
  }
  return cus[dev];
}

// What a call does: the whole thing, only the work list of the mask (a "plan": counters, items,
// multi-segment rows - the first off_pm bytes of the workspace layout, independent of Q, K, V), or
// only the attention against a work list built earlier (`plan_buf`, read-only; `ws` then only
// provides the work cursor and the partial results, in the same layout).
enum { kEngineAll = 0, kEnginePlanOnly = 1, kEngineRunOnly = 2 };

template <class Lay, class Mask>
int launch_engine(const Tensors& t, const Mask& mask, const EngineSizing& s, int use_nan, void* ws,
                  hipStream_t stream, int phase = kEngineAll, const void* plan_buf = nullptr) {
  WorkspaceLayout w = engine_workspace(s, t.n_q, t.d, t.n_batch);
  char* base = (char*)ws;
  char* pbase = (phase == kEngineRunOnly) ? (char*)const_cast<void*>(plan_buf) : base;
  Plan plan{};
  plan.cnt = (Counters*)(pbase + w.off_cnt);
  plan.items = (Item*)(pbase + w.off_items);
  plan.listed = (Item*)(pbase + w.off_listed);
  plan.phases = (Phases*)(pbase + w.off_phases);
  plan.multi = (MultiRow*)(pbase + w.off_multi);
  plan.medium = (int32_t*)(pbase + w.off_medium);
  plan.shorts = w.cap_short > 0 ? (int32_t*)(pbase + w.off_short) : nullptr;
  plan.cursor = &((Counters*)(base + w.off_cnt))->next_item;
  plan.pm = (float*)(base + w.off_pm);
  plan.pl = (float*)(base + w.off_pl);
  plan.pacc = (float*)(base + w.off_pacc);
  plan.cap_items = w.cap_items;
  plan.cap_partials = w.cap_partials;
  plan.cap_multi = w.cap_multi;
  plan.cap_medium = w.cap_medium;
  plan.status = device_status_word();
  plan.use_nan = use_nan;
  plan.short_max = s.short_max;
  plan.medium_max = s.medium_max > s.short_max ? s.medium_max : s.short_max;
  plan.seg = s.seg;
  if (t.n_q == 0) return 0;

  const bool has_long = s.max_deg > s.short_max;
  const KernelEvents ev = kernel_events();
  if (has_long && phase == kEngineAll && t.n_q * t.n_batch <= kWholeRowsMaxRows &&
      t.kv_stride <= kWholeRowsMaxKeys * (int64_t)t.d && s.nnz_bound <= kWholeRowsMaxEntries) {
    const int64_t grid = (t.n_q * t.n_batch + kWholeRowsWaves - 1) / kWholeRowsWaves;
    launch_maybe_timed(ev, whole_rows_kernel<Lay, Mask>, dim3((unsigned)grid), dim3(kWholeRowsWaves * kWave),
                       stream, t, mask, use_nan, device_status_word());
    return hipGetLastError() == hipSuccess ? 0 : 4;
  }
  if (has_long && phase != kEngineRunOnly) {
    hipLaunchKernelGGL(reset_counters_kernel, dim3(1), dim3(64), 0, stream, plan.cnt, plan.phases);
    hipLaunchKernelGGL((plan_kernel<Mask>), dim3((unsigned)((t.n_q + kPlanThreads - 1) / kPlanThreads)),
                       dim3(kPlanThreads), 0, stream, t.n_q, mask, plan);
    // (a plan that is kept is always ordered: it is made without knowing K and V)
    if (phase == kEngineAll && s.items_as_listed)
      plan.items = plan.listed;
    else
      hipLaunchKernelGGL(order_kernel, dim3((w.cap_items + 255u) / 256u), dim3(256), 0, stream, plan);
  }
  if (phase == kEnginePlanOnly) return hipGetLastError() == hipSuccess ? 0 : 4;
  if (has_long && phase == kEngineRunOnly)
    hipLaunchKernelGGL(reset_cursor_kernel, dim3(1), dim3(64), 0, stream, plan.cursor);

  const int64_t rows_per_wg = 4 * Lay::GROUPS;
  const int64_t grid1 = (t.n_q * t.n_batch + rows_per_wg - 1) / rows_per_wg;
  if constexpr (Mask::kExplicit) {
    if (has_long && s.items_on_grid && w.cap_medium > 0 && t.n_q * t.n_batch <= kFusedRowsMax) {
      const int64_t gridm = ((int64_t)w.cap_medium * t.n_batch + 3) / 4;
      const int64_t need = ((int64_t)w.cap_items * t.n_batch + 3) / 4;
      if (need + gridm + grid1 < ((int64_t)1 << 31)) {
        const dim3 grid_all((unsigned)(need + gridm + grid1));
        if (s.medium_batch == 2 && Lay::U_MEDIUM > 2)
          launch_maybe_timed(ev, explicit_rows_kernel<Lay, Mask, (Lay::U_MEDIUM > 2 ? 2 : Lay::U_MEDIUM)>, grid_all,
                             dim3(256), stream, t, mask, plan, (uint32_t)need, (uint32_t)gridm);
        else if (s.medium_batch == 4 && Lay::U_MEDIUM > 4)
          launch_maybe_timed(ev, explicit_rows_kernel<Lay, Mask, (Lay::U_MEDIUM > 4 ? 4 : Lay::U_MEDIUM)>, grid_all,
                             dim3(256), stream, t, mask, plan, (uint32_t)need, (uint32_t)gridm);
        else
          launch_maybe_timed(ev, explicit_rows_kernel<Lay, Mask>, grid_all, dim3(256), stream, t, mask, plan,
                             (uint32_t)need, (uint32_t)gridm);
        const int64_t grid3 = ((int64_t)w.cap_multi * t.n_batch + rows_per_wg - 1) / rows_per_wg;
        hipLaunchKernelGGL((merge_kernel<Lay>), dim3((unsigned)grid3), dim3(256), 0, stream, t, plan);
        return hipGetLastError() == hipSuccess ? 0 : 4;
      }
    }
  }
  launch_maybe_timed(has_long ? KernelEvents{} : ev, rows_kernel<Lay, Mask>, dim3((unsigned)grid1), dim3(256),
                     stream, t, mask, plan);
  if (has_long && w.cap_medium > 0) {
    const int64_t gridm = ((int64_t)w.cap_medium * t.n_batch + 3) / 4;
    bool launched = false;
    if constexpr (Mask::kExplicit && Lay::U_MEDIUM > 2) {
      if (s.medium_batch == 2) {
        hipLaunchKernelGGL((medium_rows_kernel<Lay, Mask, 2>), dim3((unsigned)gridm), dim3(256), 0, stream, t,
                           mask, plan);
        launched = true;
      } else if (s.medium_batch == 4 && Lay::U_MEDIUM > 4) {
        hipLaunchKernelGGL((medium_rows_kernel<Lay, Mask, (Lay::U_MEDIUM > 4 ? 4 : Lay::U_MEDIUM)>),
                           dim3((unsigned)gridm), dim3(256), 0, stream, t, mask, plan);
        launched = true;
      }
    }
    if (!launched)
      hipLaunchKernelGGL((medium_rows_kernel<Lay, Mask>), dim3((unsigned)gridm), dim3(256), 0, stream, t,
                         mask, plan);
  }
  if (has_long) {
    // Two workgroups (two wavefronts per SIMD) per CU with 16 neighbours in flight per lane
    // group.  With the work list in phase order, on the 12.8 M-position Zipf mask: 1 / 2 / 3 / 4
    // workgroups per CU 0.730 / 0.716 / 0.728 / 0.740 ms fp32, 0.479 / 0.411 / 0.403 / 0.411 ms
    // bf16; with K and V far larger than the caches (4 M tokens) the number makes no difference.
    // Smaller batches with more wavefronts (8 neighbours x 4 workgroups, 4 x 8) lose: 0.752 /
    // 0.776 ms fp32, 0.410 / 0.470 ms bf16.
    // (Listed row by row, one workgroup was the fastest, 0.79 ms fp32 against 0.98 with 8: the
    // wavefronts then spread over all of K and V and only added contention in the vector L1.)
    int64_t grid2 = (int64_t)device_cu_count() * kSegmentWorkgroupsPerCu;
    int64_t need = ((int64_t)w.cap_items * t.n_batch + 3) / 4;
    if (grid2 > need) grid2 = need;
    if (grid2 < 1) grid2 = 1;
    bool on_grid = false;
    if constexpr (Mask::kExplicit) {
      if (s.items_on_grid) {
        launch_maybe_timed(ev, items_grid_kernel<Lay, Mask>, dim3((unsigned)need), dim3(256), stream, t, mask,
                           plan);
        on_grid = true;
      }
    }
    if (!on_grid)
      launch_maybe_timed(ev, segments_kernel<Lay, Mask>, dim3((unsigned)grid2), dim3(256), stream, t, mask,
                         plan);
    const int64_t grid3 = ((int64_t)w.cap_multi * t.n_batch + rows_per_wg - 1) / rows_per_wg;
    hipLaunchKernelGGL((merge_kernel<Lay>), dim3((unsigned)grid3), dim3(256), 0, stream, t, plan);
  }
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// Pick the lane layout for (T, d).
template <typename T, class Mask>
int run_engine(const Tensors& t, const Mask& mask, const EngineSizing& s, int use_nan, void* ws,
               hipStream_t stream, int phase = kEngineAll, const void* plan_buf = nullptr) {
  const int64_t row_bytes = (int64_t)t.d * (int64_t)sizeof(T);
  const bool vec_ok = aligned16(t.q) && aligned16(t.k) && aligned16(t.v) && aligned16(t.out);
  if (vec_ok) {
    if (row_bytes == 64) return launch_engine<VecLay<T, 4>, Mask>(t, mask, s, use_nan, ws, stream, phase, plan_buf);
    if (row_bytes == 128) return launch_engine<VecLay<T, 8>, Mask>(t, mask, s, use_nan, ws, stream, phase, plan_buf);
    if (row_bytes == 256) return launch_engine<VecLay<T, 16>, Mask>(t, mask, s, use_nan, ws, stream, phase, plan_buf);
    if (row_bytes == 512) return launch_engine<VecLay<T, 32>, Mask>(t, mask, s, use_nan, ws, stream, phase, plan_buf);
    // other multiples of 16 bytes: the next layout up with its last lanes idle, then two chunks
    // per lane up to 1024 bytes
    if (row_bytes % 16 == 0) {
      if (row_bytes < 64) return launch_engine<VecLay<T, 4, true>, Mask>(t, mask, s, use_nan, ws, stream, phase, plan_buf);
      if (row_bytes < 128) return launch_engine<VecLay<T, 8, true>, Mask>(t, mask, s, use_nan, ws, stream, phase, plan_buf);
      if (row_bytes < 256) return launch_engine<VecLay<T, 16, true>, Mask>(t, mask, s, use_nan, ws, stream, phase, plan_buf);
      if (row_bytes < 512) return launch_engine<VecLay<T, 32, true>, Mask>(t, mask, s, use_nan, ws, stream, phase, plan_buf);
      if (row_bytes <= 1024) return launch_engine<WideLay<T, 2>, Mask>(t, mask, s, use_nan, ws, stream, phase, plan_buf);
      if (row_bytes <= 2048) return launch_engine<WideLay<T, 4>, Mask>(t, mask, s, use_nan, ws, stream, phase, plan_buf);
      if constexpr (sizeof(T) == 4) {  // (d <= 1024: only fp32 rows get this long)
        if (row_bytes <= 4096) return launch_engine<WideLay<T, 8>, Mask>(t, mask, s, use_nan, ws, stream, phase, plan_buf);
      }
    }
  }
  if (t.d <= 128) return launch_engine<GenLay<T, 2>, Mask>(t, mask, s, use_nan, ws, stream, phase, plan_buf);
  if (t.d <= 1024) return launch_engine<GenLay<T, 16>, Mask>(t, mask, s, use_nan, ws, stream, phase, plan_buf);
  return 5;
}

}  // namespace spfa
