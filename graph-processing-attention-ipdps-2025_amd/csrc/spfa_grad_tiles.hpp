// Gradients of band / block masks on the matrix cores: the dense-tile counterpart of the two
// gather passes of spfa_grad.hpp, for the shapes the forward tile kernels cover.
//
// The masks are symmetric inside a subsequence (|t - u| <= w), so both passes are the same tile
// problem with the roles swapped: 128 consecutive OWNER positions per workgroup (32 per
// wavefront, one per lane column), the positions within w of them STREAMED through LDS in tiles.
//   query pass: owner = query (q_i, dO_i in registers, lse_i, delta_i per lane), streamed = keys
//               (K, V tiles);  dQ_i += sum_j dS_ij k_j
//   key pass:   owner = key (k_j, v_j in registers), streamed = queries (Q, dO tiles, lse and
//               delta of the tile in LDS);  dK_j += sum_i dS_ij q_i,  dV_j += sum_i p_ij dO_i
// Everything is computed transposed, as in the forward tiles (streamed index on the rows of a
// 32x32 result, owner on the columns):
//     S^T = X A^T,  dP^T = Y B^T            (X, Y the streamed tiles; A, B the owner's vectors)
//     P^T = exp2(S^T sc - lse),  dS^T = P^T (dP^T - delta)      (the 1/sqrt(d) of dS is applied once,
//                                                               to G1, at the end)
//     G1^T += X^T dS^T,  G2^T += Y^T P^T    (G2 in the key pass only)
// The streamed tiles are row-major in LDS and serve as both operands: by rows for the first two
// products, transposed for the last two: 8-byte transposing reads for the half types; for fp32
// row i of result block eb stands for element (D/32) * i + eb of the gradient row, so that the
// D/32 values a lane feeds to the blocks for one streamed row are adjacent in LDS (one 8- or
// 16-byte read for D/32 instructions).  No atomics: an owner row belongs to one wavefront.
//
// The global-minus-local mask is two more tile problems of the same kind (the window test
// |i - j| > w is symmetric as well):
//   kTileGlobalRows: owners = the distinct listed tokens, streamed = every token, the streamed
//                    range split over workgroups; every workgroup writes partial sums, which
//                    global_grad_merge_kernel adds up (atomic adds of all the splits into the
//                    same few rows were measured: they took longer than the products);
//   kTileGlobalCols: owners = every token that is not listed, streamed = the listed tokens (the
//                    list as given for the query pass - an ordinary row walks repeated entries
//                    repeatedly - and the distinct ones for the key pass).
// In the key pass over the listed tokens an ordinary query row counts once per occurrence of the
// owner in the list, a listed one once.
#pragma once

#include "spfa_grad.hpp"
#include "spfa_tiles.hpp"

namespace spfa {

template <typename T, int D>
struct GradTileCfg {
  static constexpr bool kF32 = sizeof(T) == 4;
  static constexpr int BM = 128;
  static constexpr int BN = (kF32 && D > 64) ? 32 : 64;  // streamed positions per tile
  static constexpr int NB = BN / 32;
  // row stride in elements: rows are 16-byte aligned and 4 banks apart (a 16-byte read by 16
  // consecutive rows then covers every bank once)
  static constexpr int STRIDE = kF32 ? D + 4 : D + 8;
  static constexpr int TILE = BN * STRIDE;
  static constexpr int EB = D / 32;
  static constexpr int AREGS = kF32 ? D / 2 : D / 16;
};

// d = 128 needs more than 256 registers per lane (owner vectors plus accumulators) except for the
// query pass of the half types: one workgroup per CU there, two otherwise.  (Splitting the d = 128
// key pass into a dK and a dV launch, each at two workgroups per CU, was measured: 308 + 206 us
// against 512 us for the combined one - no gain for 25 % more products.)
template <typename T, int D, bool KEYS>
constexpr int grad_tile_min_blocks() {
  if (D <= 64 && sizeof(T) == 2 && !KEYS) return 3;
  if (D > 128) return 1;
  return (D > 64 && (KEYS || sizeof(T) == 4)) ? 1 : 2;
}

template <typename T, int D, bool KEYS, int MODE, bool PAD = false>
__global__ __launch_bounds__(256, (grad_tile_min_blocks<T, D, KEYS>())) void tile_grad_kernel(TileArgs a,
                                                                                             GradArgs g) {
  using C = GradTileCfg<T, D>;
  constexpr bool kF32 = C::kF32;
  constexpr int BM = C::BM, BN = C::BN, EB = C::EB, NB = C::NB, ST = C::STRIDE;
  __shared__ __attribute__((aligned(16))) T lds[2 * C::TILE];
  __shared__ float lse_s[BN], delta_s[BN];
  __shared__ int ktok_s[BN];    // GlobalCols: token of every streamed row of the tile
  __shared__ float once_s[BN];  // GlobalRows key pass: 1 when the streamed query is a listed token
  T* Xs = lds;
  T* Ys = lds + C::TILE;

  // len: owner positions; [u_lo, u_hi): streamed positions of this workgroup; tok_off: first row
  // of the problem in the stacked tensors (band mode folds it into base)
  int64_t base = 0, len, t0, u_lo, u_hi, tok_off = 0;
  int64_t part_bb = 0, part_split = 0;  // GlobalRows: where this workgroup's partial sums go
  if constexpr (MODE == kTileBand) {
    // the tile list of the forward band kernels: [problem][subsequence][tile], dealt to the XCDs
    // in contiguous runs
    const int64_t n_all = a.n_tiles * a.t.n_batch;
    const int64_t per_xcd = (n_all + 7) / 8;
    int64_t lt = (int64_t)(blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (lt >= n_all) return;
    const int64_t pb = lt / a.n_tiles;
    lt -= pb * a.n_tiles;
    const int64_t sub = lt / a.tiles_per_sub;
    const int64_t tile = lt - sub * a.tiles_per_sub;
    if (a.block > 0) {
      base = sub * a.block + pb * a.n;
      len = a.cnt;
    } else {
      base = sub + pb * a.n;
      len = (a.n - sub + a.s - 1) / a.s;
    }
    t0 = tile * BM;
    if (t0 >= len) return;
    u_lo = t0 - a.w;
    if (u_lo < 0) u_lo = 0;
    u_hi = t0 + BM + a.w;
    if (u_hi > len || u_hi < 0) u_hi = len;
  } else if constexpr (MODE == kTileGlobalRows) {
    // grid: [problem][owner tile][split of the streamed range]
    const int64_t per_problem = (int64_t)gridDim.x / a.t.n_batch;
    const int64_t bb = blockIdx.x / per_problem;
    const int64_t in_problem = blockIdx.x - bb * per_problem;
    const int64_t qt = in_problem / a.n_split;
    const int64_t split = in_problem - qt * a.n_split;
    tok_off = bb * a.n;
    part_bb = bb;
    part_split = split;
    len = (int64_t)*a.n_uq;
    t0 = qt * BM;
    if (t0 >= len) return;
    u_lo = split * a.key_run;
    u_hi = u_lo + a.key_run;
    if (u_hi > a.n) u_hi = a.n;
  } else {
    tok_off = (int64_t)blockIdx.y * a.n;  // one grid row per problem
    len = a.n;
    t0 = (int64_t)blockIdx.x * BM;
    if (t0 >= len) return;
    u_lo = 0;
    u_hi = KEYS ? (int64_t)*a.n_uq : a.n_globs;
  }

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, h = lane >> 5;
  const T* Ap = (const T*)(KEYS ? g.k : g.q);      // owner vectors
  const T* Bp = (const T*)(KEYS ? g.v : g.d_out);
  const T* Xp = (const T*)(KEYS ? g.q : g.k);      // streamed rows
  const T* Yp = (const T*)(KEYS ? g.d_out : g.v);
  // PAD: rows of dr < D elements (a multiple of 16 bytes); the owner vectors and the streamed
  // tiles are filled up with zeros, which add nothing to a product, and the gradient elements
  // from dr on are not written
  const int dr = PAD ? (int)a.t.d : D;
  const float scale = 1.0f / sqrtf((float)dr);
  const float sc = 1.4426950408889634f * scale;

  // GlobalRows with at most 64 listed tokens: only two wavefronts would have owners.  Wavefronts
  // 0, 1 then take the first 32 streamed rows of every tile and wavefronts 2, 3 the second 32, for
  // the same two owner blocks (two partial sums per split).
  const bool pair_split = (MODE == kTileGlobalRows) && NB == 2 && len <= 64;
  const int wave_q = pair_split ? (wave & 1) : wave;
  const int wave_k = pair_split ? (wave >> 1) : -1;  // streamed block it is restricted to (-1: all)
  const int64_t tw0 = t0 + 32 * wave_q;  // first owner of this wavefront
  const int64_t tq = tw0 + r;          // this lane's owner position
  bool own_ok = tq < len;
  int64_t own_tok;  // the owner's token (band: already its row of the stacked tensors)
  if constexpr (MODE == kTileBand) {
    own_tok = base + (own_ok ? tq : len - 1) * a.s;
  } else if constexpr (MODE == kTileGlobalRows) {
    own_tok = a.uq[own_ok ? tq : len - 1];
  } else {
    own_tok = own_ok ? tq : len - 1;
    if (own_ok && bit_is_set(a.gbits, own_tok)) own_ok = false;  // listed tokens belong to GlobalRows
  }
  const int64_t own_row = own_tok + tok_off;
  // GlobalRows key pass: how often the owner is listed (what an ordinary query row counts it as)
  float mult_o = 1.f;
  if constexpr (MODE == kTileGlobalRows && KEYS) {
    int cnt = 0;
    for (int64_t t = 0; t < a.n_globs; t++) cnt += (a.globs[t] == (int32_t)own_tok) ? 1 : 0;
    mult_o = (float)cnt;
  }

  // ---- the owner's two vectors as B operands, kept in registers
  uint4v ah[kF32 ? 1 : C::AREGS], bh[kF32 ? 1 : C::AREGS];
  float af[kF32 ? C::AREGS : 1], bf[kF32 ? C::AREGS : 1];
  {
    const T* arow = Ap + own_row * dr;
    const T* brow = Bp + own_row * dr;
    if constexpr (kF32) {
      // the 32x32x2 product takes two k per instruction, one per half of the wavefront: half h
      // takes k = h * D/2 + ks in step ks (any pairing works as long as both operands use it),
      // so that a lane's operands are consecutive in memory and in LDS
#pragma unroll
      for (int c4 = 0; c4 < D / 8; c4++) {
        float4v x = {0.f, 0.f, 0.f, 0.f}, y = {0.f, 0.f, 0.f, 0.f};
        if (!PAD || h * (D / 2) + 4 * c4 < dr) {
          x = *reinterpret_cast<const float4v*>(arow + h * (D / 2) + 4 * c4);
          y = *reinterpret_cast<const float4v*>(brow + h * (D / 2) + 4 * c4);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
          af[4 * c4 + i] = x[i];
          bf[4 * c4 + i] = y[i];
        }
      }
    } else {
#pragma unroll
      for (int ks = 0; ks < C::AREGS; ks++) {
        ah[ks] = uint4v{0u, 0u, 0u, 0u};
        bh[ks] = uint4v{0u, 0u, 0u, 0u};
        if (!PAD || 16 * ks + 8 * h < dr) {
          ah[ks] = *reinterpret_cast<const uint4v*>(arow + 16 * ks + 8 * h);
          bh[ks] = *reinterpret_cast<const uint4v*>(brow + 16 * ks + 8 * h);
        }
      }
    }
  }
  // query pass: the owner's statistics (log2 units for the exponent)
  float lse_o = 0.f, delta_o = 0.f;
  if constexpr (!KEYS) {
    lse_o = g.lse[own_row] * 1.4426950408889634f;
    delta_o = g.delta[own_row];
  }

  f32x16 g1[EB], g2[KEYS ? EB : 1];
#pragma unroll
  for (int eb = 0; eb < EB; eb++)
#pragma unroll
    for (int v = 0; v < 16; v++) {
      g1[eb][v] = 0.f;
      if constexpr (KEYS) g2[eb][v] = 0.f;
    }

  // ---- streamed tiles, fetched one ahead through registers
  constexpr int CH = kF32 ? D / 4 : D / 8;  // 16-byte chunks per row
  constexpr int KIT = BN * CH / 256;        // chunks per thread, tile and matrix
  uint4v xreg[KIT], yreg[KIT];
  float lse_reg = 0.f, delta_reg = 0.f, once_reg = 0.f;
  int ktok_reg = 0;

  // row of the stacked tensors of streamed position u
  auto streamed_row = [&](int64_t u) -> int64_t {
    if constexpr (MODE == kTileBand) return base + u * a.s;
    else if constexpr (MODE == kTileGlobalRows) return u + tok_off;
    else {
      // (an out-of-range listed entry reads row 0 and is masked below)
      const int g = KEYS ? a.uq[u] : listed_token(a.globs[u], a.n);
      return (int64_t)(g < 0 ? 0 : g) + tok_off;
    }
  };
  auto fetch = [&](int64_t ut) {
#pragma unroll
    for (int it = 0; it < KIT; it++) {
      const int idx = it * 256 + tid;
      const int j = idx / CH, c = idx % CH;
      const int64_t u = ut + j;
      uint4v xx = {0u, 0u, 0u, 0u}, yy = {0u, 0u, 0u, 0u};
      if (u < u_hi && (!PAD || (16 / (int)sizeof(T)) * c < dr)) {
        const int64_t off = streamed_row(u) * dr + (16 / (int)sizeof(T)) * c;
        xx = *reinterpret_cast<const uint4v*>(Xp + off);
        yy = *reinterpret_cast<const uint4v*>(Yp + off);
      }
      xreg[it] = xx;
      yreg[it] = yy;
    }
    if (tid < BN) {
      const bool ok = ut + tid < u_hi;
      const int64_t row = ok ? streamed_row(ut + tid) : 0;
      if constexpr (KEYS) {
        lse_reg = ok ? g.lse[row] * 1.4426950408889634f : __builtin_inff();
        delta_reg = ok ? g.delta[row] : 0.f;
      }
      if constexpr (MODE == kTileGlobalCols)
        ktok_reg = ok ? (KEYS ? (int)(row - tok_off) : listed_token(a.globs[ut + tid], a.n)) : 0;
      if constexpr (MODE == kTileGlobalRows && KEYS)
        once_reg = (ok && bit_is_set(a.gbits, row - tok_off)) ? 1.f : 0.f;
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int it = 0; it < KIT; it++) {
      const int idx = it * 256 + tid;
      const int j = idx / CH, c = idx % CH;
      if constexpr (kF32) {
        *reinterpret_cast<uint4v*>((float*)Xs + j * ST + 4 * c) = xreg[it];
        *reinterpret_cast<uint4v*>((float*)Ys + j * ST + 4 * c) = yreg[it];
      } else {
        *reinterpret_cast<uint4v*>(Xs + j * ST + 8 * c) = xreg[it];
        *reinterpret_cast<uint4v*>(Ys + j * ST + 8 * c) = yreg[it];
      }
    }
    if (tid < BN) {
      if constexpr (KEYS) {
        lse_s[tid] = lse_reg;
        delta_s[tid] = delta_reg;
      }
      if constexpr (MODE == kTileGlobalCols) ktok_s[tid] = ktok_reg;
      if constexpr (MODE == kTileGlobalRows && KEYS) once_s[tid] = once_reg;
    }
  };

  // transposing reads (half types): lane 4*x + y of a group of 16 points at streamed row
  // 4*h + x, columns 16*r_hi + 4*y .. +3 of a 32-column block; lane i of the group receives
  // column i of the four rows
  const int tx = (lane & 15) >> 2, ty = lane & 3, r_hi = (lane >> 4) & 1;
  const int tadr = (4 * h + tx) * ST + 16 * r_hi + 4 * ty;  // elements

  if (u_lo < u_hi) fetch(u_lo);
  for (int64_t ut = u_lo; ut < u_hi; ut += BN) {
    __syncthreads();  // the previous tile has been consumed
    stash();
    __syncthreads();
    if (ut + BN < u_hi) fetch(ut + BN);

    const uint32_t w32 = (uint32_t)a.w, w2 = 2u * (uint32_t)a.w;
    const int rem = (int)((u_hi - ut) < BN ? (u_hi - ut) : BN);
    (void)rem;
    // a streamed row is live iff (unsigned)(delta + w) <= 2w (band; delta in positions) or > 2w
    // (global; delta in tokens)
    // band: the end of the subsequence is folded into the same comparison (a streamed position u
    // is past the end iff u - tq + w > u_hi - 1 - tq + w, which is not negative for a valid owner)
    uint32_t d0, band_hi = w2;
    if constexpr (MODE == kTileBand) {
      const uint32_t end_hi = (uint32_t)(int32_t)(u_hi - 1 - tq) + w32;
      band_hi = own_ok && end_hi < w2 ? end_hi : w2;
    }
    if constexpr (MODE == kTileBand) d0 = (uint32_t)(int32_t)(ut - tq) + w32;
    else if constexpr (MODE == kTileGlobalRows) d0 = (uint32_t)(int32_t)(ut - own_tok) + w32;
    else d0 = w32 - (uint32_t)(int32_t)own_tok;
#pragma unroll
    for (int jb = 0; jb < NB; jb++) {
      const int64_t ub = ut + 32 * jb;
      // band: the block matters iff it overlaps the band of this wavefront's owners
      bool need = (tw0 < len) && (ub < u_hi) && (wave_k < 0 || wave_k == jb);
      if constexpr (MODE == kTileBand) need = need && (ub <= tw0 + 31 + a.w) && (ub + 31 + a.w >= tw0);
      if (!need) continue;
      const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      // the dO.V product starts at -delta, so that it comes out as (dP - delta)
      f32x16 s = zero16, dp;
#pragma unroll
      for (int v = 0; v < 16; v++) {
        if constexpr (KEYS) dp[v] = -delta_s[32 * jb + 8 * (v / 4) + 4 * h + (v % 4)];
        else dp[v] = -delta_o;
      }
      if constexpr (kF32) {
        const float* xrow = (const float*)Xs + (32 * jb + r) * ST + h * (D / 2);
        const float* yrow = (const float*)Ys + (32 * jb + r) * ST + h * (D / 2);
#pragma unroll
        for (int k4 = 0; k4 < D / 8; k4++) {
          const float4v xa = *reinterpret_cast<const float4v*>(xrow + 4 * k4);
          const float4v ya = *reinterpret_cast<const float4v*>(yrow + 4 * k4);
#pragma unroll
          for (int i = 0; i < 4; i++) {
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(xa[i], af[4 * k4 + i], s, 0, 0, 0);
            dp = __builtin_amdgcn_mfma_f32_32x32x2f32(ya[i], bf[4 * k4 + i], dp, 0, 0, 0);
          }
        }
      } else {
        const T* xrow = Xs + (32 * jb + r) * ST + 8 * h;
        const T* yrow = Ys + (32 * jb + r) * ST + 8 * h;
#pragma unroll
        for (int ks = 0; ks < D / 16; ks++) {
          s = mfma16<T>(*reinterpret_cast<const uint4v*>(xrow + 16 * ks), ah[ks], s);
          dp = mfma16<T>(*reinterpret_cast<const uint4v*>(yrow + 16 * ks), bh[ks], dp);
        }
      }
      // ---- weights: p (kept in s) and dS (kept in dp)
      bool full = false;  // every (streamed, owner) pair of the block is live
      if constexpr (MODE == kTileBand) {
        full = (ub + 31 < u_hi) && (ub + a.w >= tw0 + 31) && (ub + 31 <= tw0 + a.w);
      } else if constexpr (MODE == kTileGlobalRows) {
        const bool hit = (ub + 31 + a.w >= own_tok) && (ub <= own_tok + a.w);
        full = (ub + 31 < u_hi) && (__builtin_amdgcn_ballot_w64(hit) == 0);
      }
      // Band masks: the test is a pass of its own under a wave-uniform branch (most blocks of a band
      // are full and skip it).  Global masks: folded into the weights (measured: the separate pass
      // costs the fp32 global kernels 6 %).
      if constexpr (MODE == kTileBand) {
        if (!full) {
#pragma unroll
          for (int v = 0; v < 16; v++) {
            const int j = 32 * jb + 8 * (v / 4) + 4 * h + (v % 4);
            s[v] = (d0 + (uint32_t)j <= band_hi) ? s[v] : kNegInf;  // exp2(-inf) = 0
          }
          __builtin_amdgcn_sched_barrier(0);  // (keeps the two passes apart)
        }
      }
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int j = 32 * jb + 8 * (v / 4) + 4 * h + (v % 4);
        float ls = lse_o;
        if constexpr (KEYS) ls = lse_s[j];
        float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], sc, -ls));
        if constexpr (MODE == kTileGlobalRows && KEYS) p *= (once_s[j] != 0.f) ? 1.f : mult_o;
        if constexpr (MODE != kTileBand) {
          if (!full) {
            bool ok;
            if constexpr (MODE == kTileGlobalRows) ok = (d0 + (uint32_t)j > w2) && (j < rem);
            else ok = (d0 + (uint32_t)ktok_s[j] > w2) && (j < rem) && ktok_s[j] >= 0;
            p = ok ? p : 0.f;
          }
        }
        s[v] = p;
        dp[v] *= p;  // dS without its 1/sqrt(d), which the write-out applies
      }
      // ---- G1^T += X^T dS^T,  G2^T += Y^T P^T
      if constexpr (kF32) {
        typedef float vecE __attribute__((ext_vector_type(EB)));
        const float* xbase = (const float*)Xs + (32 * jb + 4 * h) * ST + EB * r;
        const float* ybase = (const float*)Ys + (32 * jb + 4 * h) * ST + EB * r;
        vecE xv = *reinterpret_cast<const vecE*>(xbase), yv = xv;
        if constexpr (KEYS) yv = *reinterpret_cast<const vecE*>(ybase);
#pragma unroll
        for (int v = 0; v < 16; v++) {
          vecE xn = xv, yn = yv;
          if (v + 1 < 16) {
            const int jn = (8 * ((v + 1) / 4) + ((v + 1) % 4)) * ST;
            xn = *reinterpret_cast<const vecE*>(xbase + jn);
            if constexpr (KEYS) yn = *reinterpret_cast<const vecE*>(ybase + jn);
          }
#pragma unroll
          for (int eb = 0; eb < EB; eb++) {
            g1[eb] = __builtin_amdgcn_mfma_f32_32x32x2f32(xv[eb], dp[v], g1[eb], 0, 0, 0);
            if constexpr (KEYS) g2[eb] = __builtin_amdgcn_mfma_f32_32x32x2f32(yv[eb], s[v], g2[eb], 0, 0, 0);
          }
          xv = xn;
          yv = yn;
        }
      } else {
        typedef short s16x4 __attribute__((ext_vector_type(4)));
        typedef short s16x8 __attribute__((ext_vector_type(8)));
        typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
#pragma unroll
        for (int sl = 0; sl < 2; sl++) {
          uint4v dsb, pb;
#pragma unroll
          for (int x = 0; x < 4; x++) {
            dsb[x] = pack2<T>(dp[8 * sl + 2 * x], dp[8 * sl + 2 * x + 1]);
            pb[x] = pack2<T>(s[8 * sl + 2 * x], s[8 * sl + 2 * x + 1]);
          }
          const T* xt = Xs + (32 * jb + 16 * sl) * ST + tadr;
          const T* yt = Ys + (32 * jb + 16 * sl) * ST + tadr;
#pragma unroll
          for (int eb = 0; eb < EB; eb++) {
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(xt + 32 * eb));
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(xt + 32 * eb + 8 * ST));
            const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            g1[eb] = mfma16<T>(__builtin_bit_cast(uint4v, both), dsb, g1[eb]);
            if constexpr (KEYS) {
              const s16x4 lo2 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(yt + 32 * eb));
              const s16x4 hi2 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(yt + 32 * eb + 8 * ST));
              const s16x8 both2 = {lo2[0], lo2[1], lo2[2], lo2[3], hi2[0], hi2[1], hi2[2], hi2[3]};
              g2[eb] = mfma16<T>(__builtin_bit_cast(uint4v, both2), pb, g2[eb]);
            }
          }
        }
      }
    }
  }

  // ---- add into the owner's gradient rows.  g[eb][v] is element 32*eb + i of the row for the half
  // types and (D/32)*i + eb for fp32, i = 8*(v/4) + 4*h + v%4: four registers of one block, or of
  // all blocks, are four adjacent elements
  if (!own_ok) return;
  float* out1 = (KEYS ? g.d_k : g.d_q) + own_row * dr;
  float* out2 = KEYS ? g.d_v + own_row * dr : nullptr;
#pragma unroll
  for (int oc = 0; oc < EB; oc++)
#pragma unroll
    for (int g4 = 0; g4 < 4; g4++) {
      const int e = kF32 ? EB * (8 * g4 + 4 * h) + 4 * oc : 32 * oc + 8 * g4 + 4 * h;
      float4v x, y = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int eb = kF32 ? (4 * oc + u) % EB : oc;
        const int v = kF32 ? 4 * g4 + (4 * oc + u) / EB : 4 * g4 + u;
        x[u] = g1[eb][v] * scale;
        if constexpr (KEYS) y[u] = g2[eb][v];
      }
      if constexpr (MODE == kTileGlobalRows) {
        // partial sums of this split (and half): [problem][split][half][which][listed token][D]
        const int64_t slot0 = ((part_bb * a.n_split + part_split) * 2 + (wave_k > 0 ? 1 : 0)) * (KEYS ? 2 : 1);
        // (rows of the real length: elements from dr on are padding)
        float* p1 = a.pacc + (slot0 * a.n_globs + tq) * dr + e;
        if (!PAD || e < dr) {
          *reinterpret_cast<float4v*>(p1) = x;
          if constexpr (KEYS) *reinterpret_cast<float4v*>(p1 + a.n_globs * dr) = y;
        }
      } else if (!PAD || e < dr) {
        float4v x0 = *reinterpret_cast<const float4v*>(out1 + e);
#pragma unroll
        for (int u = 0; u < 4; u++) x0[u] += x[u];
        *reinterpret_cast<float4v*>(out1 + e) = x0;
        if constexpr (KEYS) {
          float4v y0 = *reinterpret_cast<const float4v*>(out2 + e);
#pragma unroll
          for (int u = 0; u < 4; u++) y0[u] += y[u];
          *reinterpret_cast<float4v*>(out2 + e) = y0;
        }
      }
    }
}

// ---------------------------------------------------------------------------------------
// Band / block masks, bf16 / fp16: the streamed tiles go from global memory straight into LDS
// ---------------------------------------------------------------------------------------
// tile_grad_kernel's band problem with the plumbing of band_dma_kernel: the X and Y tiles of 64
// streamed rows are written into a ring of LDS stages by the loads themselves
// (global_load_lds_dwordx4, row-major, unpadded), one barrier per tile, a tile asked for
// NBUF - 1 steps before it is used.  A tile is read by rows (16-byte reads, first two products)
// and transposed (ds_read_b64_tr_b16, last two), so one chunk permutation has to serve both:
// chunk c of row j is stored at chunk position c ^ perm(j) with
//   d = 128 (16 chunks, a row is a bank cycle):  perm = the two low bit pairs of j swapped - 16
//            consecutive rows take 16 different positions (row reads), and the four rows a
//            transposing read touches (j = 4a .. 4a+3) put their 4-chunk groups in four different
//            quarters of the bank cycle;
//   d = 64  (8 chunks, two rows to a bank cycle): with t = (j >> 1) mod 8, perm = t rotated left
//            by two bits of three - rows of the same parity take 8 different positions, and rows
//            4a, 4a+2 (4a+1, 4a+3) put their groups in different halves.
// The key pass also needs lse and delta of the streamed rows: 64 + 64 floats per stage, loaded
// the same way (4 bytes per lane; every wavefront issues them, so that all wavefronts have the
// same number of loads in flight and one wait count serves all).
// PART (key pass): 0 both gradients in one launch, 1 dK only, 2 dV only.  At d = 128 the two
// accumulators and two owner vectors of the combined pass need more than 256 registers: one
// workgroup per CU, every matrix result in an AccVGPR and copied out for the vector work (a
// third of the pass's vector instructions).  As two launches (dK: S, dP and one accumulator, the
// query pass's shape; dV: S and one accumulator) both run two workgroups per CU from plain
// registers, for a quarter more matrix instructions.
template <typename T, int D, bool KEYS, int PART = 0>
struct BandGradDmaCfg {
  static constexpr int BM = 128, BN = 64, NB = 2;
  static constexpr int ROWB = D * 2, CH = D / 8;
  static constexpr int TILE_B = BN * ROWB, BUF_B = 2 * TILE_B;  // X tile then Y tile
  static constexpr int NI = TILE_B / 4096, RPI = 4096 / ROWB;
  // the key pass at d = 128 holds two accumulators and two owner vectors (one workgroup per CU
  // for its registers): four stages; otherwise what fits 64 KB
  static constexpr int NBUF = (KEYS && D == 128 && PART == 0) ? 4 : (65536 / BUF_B < 4 ? 65536 / BUF_B : 4);
  static constexpr int STAT_B = KEYS ? 2 * BN * 4 : 0;          // lse then delta of a stage
  static constexpr int LDS_BYTES = NBUF * (BUF_B + STAT_B);
  static constexpr int LOADS = 2 * NI + (KEYS ? 2 : 0);         // load instructions per wavefront and tile
  static constexpr int EB = D / 32, AREGS = D / 16;
  static_assert(D == 64 || D == 128, "d = 64 or 128");
  static_assert(RPI % 16 == 0, "the permutation must repeat per load instruction");
  __device__ static constexpr int perm(int j) {
    if (D == 128) return ((j & 3) << 2) | ((j >> 2) & 3);
    const int t = (j >> 1) & 7;
    return ((t & 1) << 2) | (t >> 1);
  }
};

template <typename T, int D, bool KEYS, int PART>
__global__ __launch_bounds__(256, (KEYS && D == 128 && PART == 0) ? 1 : 2) void band_grad_dma_kernel(TileArgs a, GradArgs g) {
  using C = BandGradDmaCfg<T, D, KEYS, PART>;
  static_assert(KEYS || PART == 0, "the query pass has one gradient");
  constexpr bool kG1 = PART != 2;           // dQ / dK: needs S, dP and the first accumulator
  constexpr bool kG2 = KEYS && PART != 1;   // dV: needs S and the second accumulator
  constexpr int BM = C::BM, BN = C::BN, NB = C::NB, EB = C::EB, ROWB = C::ROWB, CH = C::CH;
  constexpr int TILE_B = C::TILE_B, BUF_B = C::BUF_B, NI = C::NI, RPI = C::RPI, NBUF = C::NBUF, AR = C::AREGS;
  constexpr int LOADS = C::LOADS;
  static_assert(sizeof(T) == 2, "half types");
  static_assert(LOADS * (NBUF - 1) < 64, "outstanding tile loads must fit the vmcnt field");
  extern __shared__ __attribute__((aligned(1024))) char lds_dyn[];
  char* const lds = lds_dyn;
  char* const stat = lds + NBUF * BUF_B;  // [stage][lse 64 floats, delta 64 floats]

  // the tile list of the forward band kernels (32-bit arithmetic; the launcher checks the sizes)
  auto uni = [](int x) { return __builtin_amdgcn_readfirstlane(x); };
  const uint32_t n_tiles = (uint32_t)a.n_tiles, tiles_per_sub = (uint32_t)a.tiles_per_sub;
  const uint32_t n_all = n_tiles * (uint32_t)a.t.n_batch;
  const uint32_t per_xcd = (n_all + 7u) / 8u;
  uint32_t lt = (blockIdx.x % 8u) * per_xcd + blockIdx.x / 8u;
  if (lt >= n_all) return;
  const uint32_t pb_ = lt / n_tiles;
  lt -= pb_ * n_tiles;
  const uint32_t sub = lt / tiles_per_sub;
  const int tile = uni((int)(lt - sub * tiles_per_sub));
  int64_t base;
  int len;
  if (a.block > 0) {
    base = (int64_t)sub * a.block + (int64_t)pb_ * a.n;
    len = (int)a.cnt;
  } else {
    base = (int64_t)sub + (int64_t)pb_ * a.n;
    len = uni((int)(((uint32_t)a.n - sub + (uint32_t)a.s - 1u) / (uint32_t)a.s));
  }
  const int wlim = (int)(a.w < (int64_t)0x3fffffff ? a.w : (int64_t)0x3fffffff);
  const int t0 = tile * BM;
  if (t0 >= len) return;
  const int u_lo = t0 > wlim ? t0 - wlim : 0;
  const int u_hi = (len - BM - wlim > t0) ? t0 + BM + wlim : len;
  // The streamed tiles are visited in a rotated order, as in band_dma_kernel: visit number `it`
  // is the tile whose number along the subsequence is `it` modulo the tile count, so that the
  // workgroups of neighbouring owner tiles (resident at the same time, in the same XCD) ask for
  // the same tile at about the same time.  (The sums do not care about the order.)
  const int nk = (u_hi - u_lo + BN - 1) / BN;
  const int rot0 = uni((nk - (int)(((uint32_t)tile * (uint32_t)(BM / BN)) % (uint32_t)nk)) % nk);
  auto tile_start = [&](int it) __attribute__((always_inline)) {
    int j = rot0 + it;
    j = j >= nk ? j - nk : j;
    return u_lo + j * BN;
  };

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, h = lane >> 5;
  const T* Ap = (const T*)(KEYS ? g.k : g.q);            // owner vectors
  const T* Bp = (const T*)(KEYS ? g.v : g.d_out);
  const char* Xp = (const char*)(KEYS ? g.q : g.k);      // streamed rows
  const char* Yp = (const char*)(KEYS ? g.d_out : g.v);
  const float scale = 1.0f / sqrtf((float)D);
  const float sc = 1.4426950408889634f * scale;

  // ---- tile loads (band_dma_kernel's scheme: two lane offsets, the rest in the scalar base)
  const uint32_t row_step = (uint32_t)a.s * (uint32_t)ROWB;
  const int j0 = (wave * 1024 + lane * 16) / ROWB, p0 = ((wave * 1024 + lane * 16) % ROWB) / 16;
  const uint32_t xoff = (uint32_t)j0 * row_step + (uint32_t)((p0 ^ C::perm(j0)) * 16);
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  auto request = [&](int ut, int stage) __attribute__((always_inline)) {
    const int64_t tile_byte = (base + (int64_t)ut * a.s) * (int64_t)ROWB;  // scalar
    const bool whole = ut + BN <= u_hi;
#pragma unroll
    for (int it = 0; it < NI; it++) {
      uint32_t xo = xoff;
      int64_t it_byte = tile_byte + (int64_t)it * RPI * (int64_t)row_step;  // scalar
      if (!whole) {
        // last tile of a subsequence: rows past the last position are replaced by the last one
        // (finite values; they are masked out)
        int last = u_hi - 1 - ut;
        asm volatile("" : "+s"(last));
        const int j = j0 + it * RPI;
        xo = xoff + (uint32_t)((j > last ? last : j) - j0) * row_step;
        it_byte = tile_byte;
      }
      const uint32_t lds_x = lds_base + (uint32_t)(stage * BUF_B + (4 * it + wave) * 1024);
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :: "v"(xo), "s"(Xp + it_byte), "s"(lds_x) : "memory", "m0");
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :: "v"(xo), "s"(Yp + it_byte), "s"(lds_x + (uint32_t)TILE_B) : "memory", "m0");
    }
    if constexpr (KEYS) {
      // lse and delta of the tile's rows: lane l takes row ut + l (past the end: the last row)
      int last = u_hi - 1 - ut;
      asm volatile("" : "+s"(last));
      const uint32_t so = (uint32_t)(lane > last ? last : lane) * (uint32_t)a.s * 4u;
      const int64_t st_byte = (base + (int64_t)ut * a.s) * 4;
      const uint32_t lds_s = lds_base + (uint32_t)(NBUF * BUF_B + stage * C::STAT_B);
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
                   :: "v"(so), "s"((const char*)g.lse + st_byte), "s"(lds_s) : "memory", "m0");
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
                   :: "v"(so), "s"((const char*)g.delta + st_byte), "s"(lds_s + (uint32_t)(BN * 4)) : "memory", "m0");
    }
  };
#pragma unroll
  for (int i = 0; i < NBUF - 1; i++)
    if (i < nk) request(tile_start(i), i);

  const int tw0 = t0 + 32 * wave;  // first owner of this wavefront
  const int tq = tw0 + r;          // this lane's owner position
  const bool own_ok = tq < len;
  const int64_t own_row = base + (int64_t)(own_ok ? tq : len - 1) * a.s;

  // ---- the owner's two vectors as B operands, kept in registers
  uint4v ah[AR], bh[kG1 ? AR : 1];
  {
    const T* arow = Ap + own_row * D;
    const T* brow = Bp + own_row * D;
#pragma unroll
    for (int ks = 0; ks < AR; ks++) {
      ah[ks] = *reinterpret_cast<const uint4v*>(arow + 16 * ks + 8 * h);
      if constexpr (kG1) bh[ks] = *reinterpret_cast<const uint4v*>(brow + 16 * ks + 8 * h);
    }
  }
  float lse_o = 0.f, delta_o = 0.f;
  if constexpr (!KEYS) {
    lse_o = g.lse[own_row] * 1.4426950408889634f;
    delta_o = g.delta[own_row];
  }
  SPFA_WAIT_VMCNT(0);  // (the owner's vectors and the first tiles, once; see band_dma_kernel)

  // ---- operand addresses inside a stage (bytes)
  // by rows: row 32*jb + r, chunk 2*ks + h
  int radr[AR];
#pragma unroll
  for (int ks = 0; ks < AR; ks++) radr[ks] = r * ROWB + (((2 * ks + h) ^ C::perm(r)) * 16);
  // transposed: lane 4*x + y of a group of 16 points at row 4*h + x (+ 8 for the second half of
  // an operand), columns 32*eb + 16*r_hi + 4*y .. +3, i.e. chunk 4*eb + 2*r_hi + y/2, half y & 1
  int tadr_lo[EB], tadr_hi[EB];
  {
    const int x = (lane & 15) >> 2, y = lane & 3, r_hi = (lane >> 4) & 1;
    const int key = 4 * h + x;
#pragma unroll
    for (int eb = 0; eb < EB; eb++) {
      const int c = 4 * eb + 2 * r_hi + (y >> 1);
      tadr_lo[eb] = key * ROWB + ((c ^ C::perm(key)) * 16) + (y & 1) * 8;
      tadr_hi[eb] = (key + 8) * ROWB + ((c ^ C::perm(key + 8)) * 16) + (y & 1) * 8;
    }
  }

  f32x16 g1[kG1 ? EB : 1], g2[kG2 ? EB : 1];
#pragma unroll
  for (int eb = 0; eb < EB; eb++)
#pragma unroll
    for (int v = 0; v < 16; v++) {
      if constexpr (kG1) g1[eb][v] = 0.f;
      if constexpr (kG2) g2[eb][v] = 0.f;
    }

  typedef short s16x4 __attribute__((ext_vector_type(4)));
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const uint32_t w32 = (uint32_t)wlim, w2 = 2u * (uint32_t)wlim;
  // the end of the subsequence folded into the band test (see tile_grad_kernel)
  const uint32_t end_hi = (uint32_t)(u_hi - 1 - tq) + w32;
  const uint32_t band_hi = own_ok && end_hi < w2 ? end_hi : w2;

  auto step = [&](int it, int stage) __attribute__((always_inline)) {
    const int ut = tile_start(it);
    const char* xs = lds + stage * BUF_B;
    const char* ys = xs + TILE_B;
    const float* lse_s = reinterpret_cast<const float*>(stat + stage * C::STAT_B);
    const float* delta_s = lse_s + BN;
    if constexpr (NBUF > 2) {
      const int after = nk - 1 - it;  // tiles behind this one
      if (after >= 2) SPFA_WAIT_VMCNT(2 * LOADS);
      else if (after == 1) SPFA_WAIT_VMCNT(LOADS);
      else SPFA_WAIT_VMCNT(0);
    } else {
      SPFA_WAIT_VMCNT(0);
    }
    __syncthreads();  // the tile has landed for everyone, and everyone is done with the stage before it
    if (it + NBUF - 1 < nk) request(tile_start(it + NBUF - 1), (stage + NBUF - 1) % NBUF);

    const uint32_t d0 = (uint32_t)(ut - tq) + w32;
#pragma unroll
    for (int jb = 0; jb < NB; jb++) {
      const int ub = ut + 32 * jb;
      const bool need = (tw0 < len) && (ub < u_hi) && (ub <= tw0 + 31 + wlim) && (ub + 31 + wlim >= tw0);
      if (!need) continue;
      f32x16 s = zero16, dp = zero16;
      if constexpr (kG1) {
#pragma unroll
        for (int v = 0; v < 16; v++) {
          if constexpr (KEYS) dp[v] = -delta_s[32 * jb + 8 * (v / 4) + 4 * h + (v % 4)];
          else dp[v] = -delta_o;
        }
      }
#pragma unroll
      for (int ks = 0; ks < AR; ks++) {
        s = mfma16<T>(*reinterpret_cast<const uint4v*>(xs + 32 * jb * ROWB + radr[ks]), ah[ks], s);
        if constexpr (kG1)
          dp = mfma16<T>(*reinterpret_cast<const uint4v*>(ys + 32 * jb * ROWB + radr[ks]), bh[ks], dp);
      }
      const bool full = (ub + 31 < u_hi) && (ub + wlim >= tw0 + 31) && (ub + 31 <= tw0 + wlim);
      if (!full) {
#pragma unroll
        for (int v = 0; v < 16; v++) {
          const int j = 32 * jb + 8 * (v / 4) + 4 * h + (v % 4);
          s[v] = (d0 + (uint32_t)j <= band_hi) ? s[v] : kNegInf;  // exp2(-inf) = 0
        }
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int v = 0; v < 16; v++) {
        float ls = lse_o;
        if constexpr (KEYS) ls = lse_s[32 * jb + 8 * (v / 4) + 4 * h + (v % 4)] * 1.4426950408889634f;
        const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], sc, -ls));
        s[v] = p;
        if constexpr (kG1) dp[v] *= p;  // dS without its 1/sqrt(d), which the write-out applies
      }
#pragma unroll
      for (int sl = 0; sl < 2; sl++) {
        uint4v dsb = {0u, 0u, 0u, 0u}, pb = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int x = 0; x < 4; x++) {
          if constexpr (kG1) dsb[x] = pack2<T>(dp[8 * sl + 2 * x], dp[8 * sl + 2 * x + 1]);
          if constexpr (kG2) pb[x] = pack2<T>(s[8 * sl + 2 * x], s[8 * sl + 2 * x + 1]);
        }
        const char* xt = xs + (32 * jb + 16 * sl) * ROWB;
        const char* yt = ys + (32 * jb + 16 * sl) * ROWB;
#pragma unroll
        for (int eb = 0; eb < EB; eb++) {
          if constexpr (kG1) {
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(xt + tadr_lo[eb]));
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(xt + tadr_hi[eb]));
            const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            g1[eb] = mfma16<T>(__builtin_bit_cast(uint4v, both), dsb, g1[eb]);
          }
          if constexpr (kG2) {
            const s16x4 lo2 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(yt + tadr_lo[eb]));
            const s16x4 hi2 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(yt + tadr_hi[eb]));
            const s16x8 both2 = {lo2[0], lo2[1], lo2[2], lo2[3], hi2[0], hi2[1], hi2[2], hi2[3]};
            g2[eb] = mfma16<T>(__builtin_bit_cast(uint4v, both2), pb, g2[eb]);
          }
        }
      }
    }
  };

  for (int it = 0; it < nk; it += NBUF) {
#pragma unroll
    for (int sg = 0; sg < NBUF; sg++)
      if (it + sg < nk) step(it + sg, sg);
  }

  // ---- add into the owner's gradient rows (g[eb][v] is element 32*eb + 8*(v/4) + 4*h + v%4)
  if (!own_ok) return;
  float* out1 = (KEYS ? g.d_k : g.d_q) + own_row * D;
  float* out2 = KEYS ? g.d_v + own_row * D : nullptr;
#pragma unroll
  for (int oc = 0; oc < EB; oc++)
#pragma unroll
    for (int g4 = 0; g4 < 4; g4++) {
      const int e = 32 * oc + 8 * g4 + 4 * h;
      if constexpr (kG1) {
        float4v x0 = *reinterpret_cast<const float4v*>(out1 + e);
#pragma unroll
        for (int u = 0; u < 4; u++) x0[u] += g1[oc][4 * g4 + u] * scale;
        *reinterpret_cast<float4v*>(out1 + e) = x0;
      }
      if constexpr (kG2) {
        float4v y0 = *reinterpret_cast<const float4v*>(out2 + e);
#pragma unroll
        for (int u = 0; u < 4; u++) y0[u] += g2[oc][4 * g4 + u];
        *reinterpret_cast<float4v*>(out2 + e) = y0;
      }
    }
}

// One pass of band_grad_dma_kernel (its LDS stages are dynamic LDS; the kernel's limit is raised
// once per device).  False: not launched.
template <typename T, int D, bool KEYS, int PART = 0>
bool launch_band_grad_dma(const TileArgs& a, const GradArgs& g, dim3 grid, hipStream_t stream) {
  using C = BandGradDmaCfg<T, D, KEYS, PART>;
  static std::atomic<bool> raised[kLdsLimitDevices];
  if (!raise_lds_limit(reinterpret_cast<const void*>(&band_grad_dma_kernel<T, D, KEYS, PART>), C::LDS_BYTES, raised))
    return false;
  hipLaunchKernelGGL((band_grad_dma_kernel<T, D, KEYS, PART>), grid, dim3(256), C::LDS_BYTES, stream, a, g);
  return true;
}

// Both passes of a band / block mask described by `a` (as the forward tile kernels take it).
template <typename T, int D>
int launch_band_grad(const TileArgs& a, const GradArgs& g, hipStream_t stream) {
  const int64_t rows = g.n_q * g.n_batch;
  if (rows == 0 || a.n_tiles == 0) return 0;
  hipLaunchKernelGGL((grad_prologue_kernel<T>), dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, stream,
                     a.t, g);
  const int64_t grid = (a.n_tiles * a.t.n_batch + 7) / 8 * 8;
  if constexpr (sizeof(T) == 2 && (D == 64 || D == 128)) {
    // the direct-to-LDS kernels address a tile's rows with 32-bit offsets, and tile numbers,
    // windows and positions with 32-bit arithmetic (the forward kernel's conditions)
    const int64_t max_len = a.block > 0 ? a.cnt : (a.n + a.s - 1) / a.s;
    const bool dma = a.s * (int64_t)(2 * D) * 64 < ((int64_t)1 << 31) && a.n < ((int64_t)1 << 31) &&
                     a.n_tiles * a.t.n_batch < ((int64_t)1 << 31) &&
                     (a.w <= (int64_t)0x3fffffff || max_len <= (int64_t)0x3fffffff);
#ifndef SPFA_GRAD_KEY_SPLIT
#define SPFA_GRAD_KEY_SPLIT 1
#endif
    if (dma && launch_band_grad_dma<T, D, false>(a, g, dim3((unsigned)grid), stream)) {
      bool ok;
      if constexpr (D == 128 && SPFA_GRAD_KEY_SPLIT)
        ok = launch_band_grad_dma<T, D, true, 1>(a, g, dim3((unsigned)grid), stream) &&
             launch_band_grad_dma<T, D, true, 2>(a, g, dim3((unsigned)grid), stream);
      else
        ok = launch_band_grad_dma<T, D, true, 0>(a, g, dim3((unsigned)grid), stream);
      return ok && hipGetLastError() == hipSuccess ? 0 : 4;
    }
  }
  hipLaunchKernelGGL((tile_grad_kernel<T, D, false, kTileBand>), dim3((unsigned)grid), dim3(256), 0, stream,
                     a, g);
  hipLaunchKernelGGL((tile_grad_kernel<T, D, true, kTileBand>), dim3((unsigned)grid), dim3(256), 0, stream,
                     a, g);
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

// Rows of a.t.d < D elements, D the next multiple of 32 the tile kernel is built for: the
// register-staged kernel with zero-filled operands (the forward tiles' rule).
template <typename T, int D>
int launch_band_grad_padded(const TileArgs& a, const GradArgs& g, hipStream_t stream) {
  const int64_t rows = g.n_q * g.n_batch;
  if (rows == 0 || a.n_tiles == 0) return 0;
  hipLaunchKernelGGL((grad_prologue_kernel<T>), dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, stream,
                     a.t, g);
  const int64_t grid = (a.n_tiles * a.t.n_batch + 7) / 8 * 8;
  hipLaunchKernelGGL((tile_grad_kernel<T, D, false, kTileBand, true>), dim3((unsigned)grid), dim3(256), 0,
                     stream, a, g);
  hipLaunchKernelGGL((tile_grad_kernel<T, D, true, kTileBand, true>), dim3((unsigned)grid), dim3(256), 0,
                     stream, a, g);
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

// Adds the partial sums of the GlobalRows passes into the gradient rows of the listed tokens.
// Grid: x = (problem, listed token), y = a chunk of the splits; a thread per element of (g1, g2)
// sums its chunk and adds it to the row with one atomic (gridDim.y adds per address).
template <typename T, int D, bool PAD = false>
__global__ __launch_bounds__(2 * D) void global_grad_merge_kernel(TileArgs a, GradArgs g, int keys) {
  const int64_t n_uq = (int64_t)*a.n_uq;
  const int64_t bb = blockIdx.x / a.n_globs;
  const int64_t t = blockIdx.x - bb * a.n_globs;
  if (t >= n_uq) return;
  const int dd = PAD ? (int)a.t.d : D;  // (PAD: rows of a.t.d < D elements)
  const int which = threadIdx.x / D, e = threadIdx.x % D;
  const int n_which = keys ? 2 : 1;
  if (which >= n_which || e >= dd) return;
  const int halves = (GradTileCfg<T, D>::NB == 2 && n_uq <= 64) ? 2 : 1;  // the tile kernel's pair split
  const int64_t per = (a.n_split + gridDim.y - 1) / gridDim.y;
  const int64_t sp0 = (int64_t)blockIdx.y * per;
  const int64_t sp1 = sp0 + per < a.n_split ? sp0 + per : a.n_split;
  float acc = 0.f;
  for (int64_t sp = sp0; sp < sp1; sp++)
    for (int hf = 0; hf < halves; hf++) {
      const int64_t slot = (((bb * a.n_split + sp) * 2 + hf) * n_which + which) * a.n_globs + t;
      acc += a.pacc[slot * dd + e];
    }
  if (sp0 >= sp1) return;
  const int64_t row = (int64_t)a.uq[t] + bb * a.n;
  float* out = (keys ? (which ? g.d_v : g.d_k) : g.d_q) + row * dd + e;
  unsafeAtomicAdd(out, acc);
}

// Both passes of the global-minus-local mask: the ordinary tokens against the listed ones, then
// the listed ones against everything (a: globs, n_globs, gbits, uq, n_uq, key_run, n_split set).
template <typename T, int D, bool PAD = false>
int launch_global_grad(const TileArgs& a, const GradArgs& g, hipStream_t stream) {
  const int64_t rows = g.n_q * g.n_batch;
  if (rows == 0) return 0;
  hipLaunchKernelGGL((grad_prologue_kernel<T>), dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, stream,
                     a.t, g);
  const unsigned nb = (unsigned)a.t.n_batch;
  const dim3 grid_cols((unsigned)((a.n + 127) / 128), nb);
  hipLaunchKernelGGL((tile_grad_kernel<T, D, false, kTileGlobalCols, PAD>), grid_cols, dim3(256), 0, stream, a, g);
  hipLaunchKernelGGL((tile_grad_kernel<T, D, true, kTileGlobalCols, PAD>), grid_cols, dim3(256), 0, stream, a, g);
  const int64_t q_tiles = (a.n_globs + 127) / 128;
  const dim3 grid_rows((unsigned)(q_tiles * a.n_split * nb));
  // enough workgroups to fill the device, at least 8 splits each
  int64_t chunks = 4096 / (a.n_globs * nb);
  if (chunks > a.n_split / 8) chunks = a.n_split / 8;
  if (chunks < 1) chunks = 1;
  const dim3 grid_merge((unsigned)(a.n_globs * nb), (unsigned)chunks);
  hipLaunchKernelGGL((tile_grad_kernel<T, D, false, kTileGlobalRows, PAD>), grid_rows, dim3(256), 0, stream, a, g);
  hipLaunchKernelGGL((global_grad_merge_kernel<T, D, PAD>), grid_merge, dim3(2 * D), 0, stream, a, g, 0);
  hipLaunchKernelGGL((tile_grad_kernel<T, D, true, kTileGlobalRows, PAD>), grid_rows, dim3(256), 0, stream, a, g);
  hipLaunchKernelGGL((global_grad_merge_kernel<T, D, PAD>), grid_merge, dim3(2 * D), 0, stream, a, g, 1);
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

// Returns -1 when the shape is not covered (the caller then runs the gather passes).
template <typename T>
int run_band_grad_tiles(const TileArgs& a, const GradArgs& g, hipStream_t stream) {
  if (((uintptr_t)g.d_out | (uintptr_t)g.d_q | (uintptr_t)g.d_k | (uintptr_t)g.d_v) & 15) return -1;
  if (a.t.d % 32 != 0) {
    // rows of whole 16-byte pieces: the tiles of the next multiple of 32 that is built
    if (!tile_shape_padded_ok<T>(a.t)) return -1;
    const int64_t dp = (a.t.d + 31) / 32 * 32;
    if (dp == 32) return launch_band_grad_padded<T, 32>(a, g, stream);
    if (dp == 64) return launch_band_grad_padded<T, 64>(a, g, stream);
    if (dp == 96) return launch_band_grad_padded<T, 96>(a, g, stream);
    if (dp == 128) return launch_band_grad_padded<T, 128>(a, g, stream);
    if constexpr (sizeof(T) == 2) {
      if (dp == 160) return launch_band_grad_padded<T, 160>(a, g, stream);
      if (dp == 192) return launch_band_grad_padded<T, 192>(a, g, stream);
    }
    return -1;
  }
  if (!tile_shape_ok(a.t, sizeof(T))) return -1;
  if (a.t.d == 64) return launch_band_grad<T, 64>(a, g, stream);
  if (a.t.d == 128) return launch_band_grad<T, 128>(a, g, stream);
  if (a.t.d == 32) return launch_band_grad<T, 32>(a, g, stream);
  if (a.t.d == 96) return launch_band_grad<T, 96>(a, g, stream);
  // (fp32 beyond d = 128: the key pass no longer fits 512 registers)
  if constexpr (sizeof(T) == 2) {
    if (a.t.d == 160) return launch_band_grad<T, 160>(a, g, stream);
    if (a.t.d == 192) return launch_band_grad<T, 192>(a, g, stream);
  }
  return -1;
}

template <typename T>
int run_global_grad_tiles(const TileArgs& a, const GradArgs& g, hipStream_t stream) {
  if (((uintptr_t)g.d_out | (uintptr_t)g.d_q | (uintptr_t)g.d_k | (uintptr_t)g.d_v) & 15) return -1;
  if (a.t.d % 32 != 0) {
    if (!tile_shape_padded_ok<T>(a.t)) return -1;
    const int64_t dp = (a.t.d + 31) / 32 * 32;
    if (dp == 32) return launch_global_grad<T, 32, true>(a, g, stream);
    if (dp == 64) return launch_global_grad<T, 64, true>(a, g, stream);
    if (dp == 96) return launch_global_grad<T, 96, true>(a, g, stream);
    if (dp == 128) return launch_global_grad<T, 128, true>(a, g, stream);
    return -1;
  }
  if (!tile_shape_ok(a.t, sizeof(T))) return -1;
  if (a.t.d == 64) return launch_global_grad<T, 64>(a, g, stream);
  if (a.t.d == 128) return launch_global_grad<T, 128>(a, g, stream);
  if (a.t.d == 32) return launch_global_grad<T, 32>(a, g, stream);
  if (a.t.d == 96) return launch_global_grad<T, 96>(a, g, stream);
  return -1;
}

}  // namespace spfa
