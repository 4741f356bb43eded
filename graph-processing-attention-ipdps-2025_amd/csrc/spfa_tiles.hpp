// Dense-tile attention for band and block masks on the gfx950 matrix cores.
//
// A band / block mask is a set of independent *subsequences*: position t of a subsequence is
// token base + t*s, and query t attends keys u with |t - u| <= w inside the subsequence.
//   Local                 one subsequence (base 0, s = 1)
//   Local 1D dilated      s subsequences, one per residue class mod s
//   Local 2D dilated      one subsequence per block (base b*B, cnt live tokens, w = everything)
// so all three are the same tile problem.  One workgroup (4 wavefronts) owns 128 consecutive
// query positions, one wavefront 32 of them; keys are streamed in tiles of 64 (32 for fp32 at
// d = 128) through LDS and shared by the four wavefronts.  tile_kernel stages the tiles through
// registers (every type of the global mask; band masks only when a tile's rows are too far apart
// for 32-bit offsets); band_dma_kernel (bf16 / fp16) and band_dma_f32_kernel let the loads write
// LDS directly.
//
// Everything is computed transposed, S^T = K Q^T and O^T = V^T P^T, with 32x32 MFMA tiles.  In
// the 32x32 result layout lane (r, h) = (lane % 32, lane / 32) holds column r, rows
// 8*(v/4) + 4*h + v%4 for register v.  With queries on the columns
//   - a query's running max / sum live in one lane pair (r,0),(r,1): the row reductions of the
//     softmax are in-register plus one exchange across the two halves of the wavefront;
//   - the P^T registers are already the B operand of the second product (the summation index of
//     that product is the key, and any key order works as long as V^T uses the same one).
// Half types use v_mfma_f32_32x32x16 (8 consecutive k per lane), fp32 uses v_mfma_f32_32x32x2
// (no down-cast of fp32 inputs).
//
// fp32 operands come out of LDS 16 bytes at a time, one read for four (K) or D/32 (V) matrix
// instructions, which takes two free choices of index order:
//   - first product: the instruction sums over two k, one per half of the wavefront.  Half h
//     takes k = 8g + 4h + i in instruction 4g + i, so its four values of a group g are adjacent
//     in the K row (and in the Q row, which is loaded into registers the same way);
//   - second product: row i of result block eb is element e = (D/32) * i + eb of the output
//     row, so the D/32 values a lane feeds to the blocks for one key are adjacent in the V row.
//     tile_write_row and the partial results of the global rows undo that order when they write.
// (With one 4-byte read per instruction the compiler, short of registers, ran read - wait - two
// instructions in strict sequence and the matrix pipe idled through every LDS round trip.)
#pragma once

#include "spfa_engine.hpp"

namespace spfa {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

// What a tile problem looks like.  Band: queries and keys are the positions of one subsequence.
// GlobalRows: queries are the (distinct) global rows, keys are all tokens outside the query's
// window; the key range is split over workgroups and each writes a partial (m, l, acc).
// GlobalCols: queries are all non-global tokens, keys are the listed global tokens outside the
// query's window (Sparse_FlashAttention_Global_No_Local/sp_flatt_global_no_local_kernel.cu:38-64).
enum { kTileBand = 0, kTileGlobalRows = 1, kTileGlobalCols = 2 };

struct TileArgs {
  Tensors t;
  int64_t n;              // tokens
  int64_t w;              // window half-width (band: subsequence positions; global: tokens)
  int64_t s;              // token stride of a subsequence
  int64_t block;          // 0: band mode, else block size
  int64_t cnt;            // block mode: live positions per block
  int64_t tiles_per_sub;  // query tiles per subsequence (of the longest subsequence)
  int64_t n_tiles;
  int64_t n_tail;         // band: the last n_tail tiles (over all problems) are each shared by four
                          // workgroups of 32 queries whose wavefronts deal the key blocks among
                          // themselves; they fill the last, partly empty round of the grid
  // global modes
  const int32_t* globs;   // listed global tokens (keys of GlobalCols)
  int64_t n_globs;
  const uint32_t* gbits;  // bit i set <=> token i is a global row
  const int32_t* uq;      // distinct global rows (queries of GlobalRows)
  const uint32_t* n_uq;   // how many
  int32_t persist;        // GlobalCols: all keys fit one LDS tile; workgroups keep it and walk
                          // over query tiles (grid-stride)
  int32_t pair_split;     // GlobalRows with at most 64 global rows: wavefronts 0,1 take the first
                          // 32 keys of every tile, wavefronts 2,3 the second 32, for the same two
                          // query blocks; the pairs are folded through LDS at the end
  int64_t key_run;        // GlobalRows: keys per split (multiple of 64)
  int64_t n_split;
  float* pm;              // GlobalRows partials, slot = query * n_split + split
  float* pl;
  float* pacc;
};

template <typename T, int D>
struct TileCfg {
  static constexpr bool kF32 = sizeof(T) == 4;
  static constexpr int BM = 128;  // queries per workgroup
  // keys per LDS tile (fp32 above d = 64 and the half types at d = 256 take half tiles to stay
  // inside 64 KB of LDS)
  static constexpr int BN = (kF32 ? D > 64 : D >= 256) ? 32 : 64;
  static constexpr int NB = BN / 32;  // 32-key blocks per tile
  // K tile: [key][k] rows padded so that the 32 keys read by one operand fetch spread over the
  // banks.  V tile: half types are stored transposed [e][key'] (16-byte operand reads), fp32
  // row-major [key][e].
  static constexpr int K_STRIDE = kF32 ? D + 4 : D + 8;
  static constexpr int V_STRIDE = kF32 ? D + 8 : BN + 8;
  static constexpr int K_ELEMS = BN * K_STRIDE;
  static constexpr int V_ELEMS = kF32 ? BN * V_STRIDE : D * V_STRIDE;
  static constexpr int LDS_BYTES = (K_ELEMS + V_ELEMS) * (int)sizeof(T);
  // more than the 64 KB a kernel can declare (fp32 at d = 256: 66 KB): the tile buffers are then
  // dynamic LDS, sized at the launch
  static constexpr bool kDynLds = LDS_BYTES + BN * 4 > 65536;
  static constexpr int EB = D / 32;                 // 32-row blocks of O^T
  static constexpr int QREGS = kF32 ? D / 2 : D / 16;
};

// key order inside a 64-key tile for the transposed V tile of the half types: swap bits 2 and 3
__device__ __forceinline__ int key_slot(int j) {
  return (j & ~12) | ((j & 4) << 1) | ((j & 8) >> 1);
}

template <typename T>
__device__ __forceinline__ f32x16 mfma16(const uint4v& a, const uint4v& b, f32x16 c) {
  if constexpr (__is_same(T, bf16)) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
}

template <typename T>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  typedef T t2 __attribute__((ext_vector_type(2)));
  t2 x = {(T)lo, (T)hi};
  return __builtin_bit_cast(uint32_t, x);
}

template <bool B>
struct BoolConst {
  static constexpr bool value = B;
};

// N adjacent floats of an LDS row, read as one piece where N is a power of two (8 or 16 bytes,
// aligned as such), as single floats otherwise (d = 96, 160, 192, 224: 3, 5, 6, 7 floats)
template <int N>
struct alignas((N & (N - 1)) == 0 ? 4 * N : 4) RowPiece {
  float x[N];
  __device__ __forceinline__ float operator[](int i) const { return x[i]; }
};

// Fold the incoming state of row `row` into a finished tile result and write the row back.
// o holds O^T in the 32x32 result layout: o[eb][v] is element e = 32*eb + i of the row for the
// half types and e = (D/32)*i + eb for fp32, i = 8*(v/4) + 4*h + v%4; m is the running max in log2 units, l the row sum (already summed over both halves
// of the wavefront); o * o_scale is the accumulator that goes with (m, l).
// dr: length of a row of `out` in elements (a multiple of 16 bytes, at most D; the accumulator's
// elements from dr on belong to zero padding and are not written).
template <typename T, int D>
__device__ __forceinline__ void tile_write_row(const Tensors& t, int64_t row, int h, float m, float l,
                                               const f32x16 (&o)[D / 32], float o_scale = 1.f,
                                               bool have_in = false, float l_pre = 0.f, float m_pre = 0.f,
                                               int dr = D) {
  constexpr bool kF32 = sizeof(T) == 4;
  const bool sf = t.state_f32 != 0;
  const float m_nat = m * 0.6931471805599453f;
  float m_out = m_nat, l_out = l;
  float wa = 0.f, wb = 1.f;
  // (have_in: the caller has read the incoming state already, while it worked on the tile)
  const float l_in = have_in ? l_pre : load_state<T>(t.l, row, sf);
  if (l_in != 0.f) {
    const float m_in = have_in ? m_pre : load_state<T>(t.m, row, sf);
    m_out = fmaxf(m_nat, m_in);
    wa = l_in * __expf(m_in - m_out);
    wb = __expf(m_nat - m_out);
    l_out = wa + l * wb;
  }
  const float inv = 1.f / l_out;
  wb *= inv * o_scale;  // o_scale: o was accumulated against a reference below the maximum m
  wa *= inv;
  T* orow = (T*)t.out + row * dr;
  if constexpr (kF32) {
    // registers 4*g4 .. 4*g4+3 of all blocks: 4*EB consecutive elements from EB * (8*g4 + 4*h)
    constexpr int EB = D / 32;
#pragma unroll
    for (int g4 = 0; g4 < 4; g4++) {
#pragma unroll
      for (int c = 0; c < EB; c++) {
        const int e = EB * (8 * g4 + 4 * h) + 4 * c;
        if (e >= dr) continue;
        float x[4];
#pragma unroll
        for (int u = 0; u < 4; u++) x[u] = o[(4 * c + u) % EB][4 * g4 + (4 * c + u) / EB] * wb;
        if (wa != 0.f) {
          float4v oi = *reinterpret_cast<const float4v*>(orow + e);
#pragma unroll
          for (int u = 0; u < 4; u++) x[u] += wa * oi[u];
        }
        float4v y = {x[0], x[1], x[2], x[3]};
        *reinterpret_cast<float4v*>(orow + e) = y;
      }
    }
  } else {
    // A lane holds 4 consecutive elements (8 bytes) of each group of 8; the other 4 are in the
    // lane of the other half of the wavefront that works on the same row.  The two trade
    // halves so that each writes whole 16-byte pieces (groups 0, 1 of every 32 elements stay
    // with the lower lane, 2, 3 with the upper one).
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const int partner = (int)((__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)) ^ 32u) << 2);
#pragma unroll
    for (int eb = 0; eb < D / 32; eb++) {
      u32x2 y[4];
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++) {
        const int e = 32 * eb + 8 * g4 + 4 * h;
        float x[4];
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] = o[eb][4 * g4 + i] * wb;
        if (wa != 0.f && e < dr) {
          typedef T t4 __attribute__((ext_vector_type(4)));
          t4 oi = *reinterpret_cast<const t4*>(orow + e);
#pragma unroll
          for (int i = 0; i < 4; i++) x[i] += wa * (float)oi[i];
        }
        y[g4][0] = pack2<T>(x[0], x[1]);
        y[g4][1] = pack2<T>(x[2], x[3]);
      }
#pragma unroll
      for (int k = 0; k < 2; k++) {
        const u32x2 give = h ? y[k] : y[2 + k];
        const u32x2 keep = h ? y[2 + k] : y[k];
        u32x2 got;
        got[0] = (uint32_t)__builtin_amdgcn_ds_bpermute(partner, (int)give[0]);
        got[1] = (uint32_t)__builtin_amdgcn_ds_bpermute(partner, (int)give[1]);
        const uint4v piece = h ? uint4v{got[0], got[1], keep[0], keep[1]}
                               : uint4v{keep[0], keep[1], got[0], got[1]};
        if (32 * eb + 8 * (2 * h + k) < dr) *reinterpret_cast<uint4v*>(orow + 32 * eb + 8 * (2 * h + k)) = piece;
      }
    }
  }
  if (h == 0) {
    store_state<T>(t.m, row, m_out, sf);
    store_state<T>(t.l, row, l_out, sf);
  }
}

template <typename T, int D, int MODE, bool PAD = false>
__global__ __launch_bounds__(256, D > 128 ? 1 : 2) void tile_kernel(TileArgs a) {
  using C = TileCfg<T, D>;
  constexpr bool kF32 = C::kF32;
  constexpr int BM = C::BM, BN = C::BN, EB = C::EB, NB = C::NB;
  __shared__ __attribute__((aligned(16))) T lds_fixed[C::kDynLds ? 4 : C::K_ELEMS + C::V_ELEMS];
  extern __shared__ __attribute__((aligned(16))) char lds_dyn[];
  T* const lds = C::kDynLds ? reinterpret_cast<T*>(lds_dyn) : lds_fixed;
  __shared__ int ktok_s[BN];  // GlobalCols: token of every key of the tile
  T* Ks = lds;
  T* Vs = lds + C::K_ELEMS;

  // base/len: token of position 0 and number of positions (band); qlen/klen: query and key
  // position counts; [u_lo, u_hi): key positions this workgroup walks
  int64_t base = 0, qlen, klen, t0, u_lo, u_hi, split = 0;
  int64_t bb = 0;  // problem of the batch (global modes; band mode folds it into base)
  int quarter = -1;  // band: which 32 queries of a shared tail tile (-1: a whole tile)
  if constexpr (MODE == kTileBand) {
    // workgroups are dealt round-robin to the 8 XCDs: give each XCD a contiguous run of tiles
    // so that neighbouring query tiles (which share most of their keys) meet in one L2
    // (the tiles of all problems of a batch form one list; problem pb starts at token pb * n)
    const int64_t n_all = a.n_tiles * a.t.n_batch;
    const int64_t n_main = n_all - a.n_tail;
    const int64_t per_xcd = (n_main + 7) / 8;
    int64_t lt;
    if ((int64_t)blockIdx.x < 8 * per_xcd) {
      lt = (int64_t)(blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
      if (lt >= n_main) return;
    } else {
      const int64_t qid = (int64_t)blockIdx.x - 8 * per_xcd;
      lt = n_main + qid / 4;
      quarter = (int)(qid & 3);
    }
    const int64_t pb = lt / a.n_tiles;
    lt -= pb * a.n_tiles;
    const int64_t sub = lt / a.tiles_per_sub;
    const int64_t tile = lt - sub * a.tiles_per_sub;
    if (a.block > 0) {
      base = sub * a.block + pb * a.n;
      qlen = a.cnt;
    } else {
      base = sub + pb * a.n;
      qlen = (a.n - sub + a.s - 1) / a.s;
    }
    klen = qlen;
    t0 = tile * BM + (quarter >= 0 ? 32 * quarter : 0);
    if (t0 >= qlen) return;
    u_lo = t0 - a.w;
    if (u_lo < 0) u_lo = 0;
    u_hi = t0 + (quarter >= 0 ? 32 : BM) + a.w;
    if (u_hi > klen || u_hi < 0) u_hi = klen;
  } else if constexpr (MODE == kTileGlobalRows) {
    // grid: [problem][query tile][key split]
    const int64_t per_problem = (int64_t)gridDim.x / a.t.n_batch;
    bb = blockIdx.x / per_problem;
    const int64_t in_problem = blockIdx.x - bb * per_problem;
    const int64_t qt = in_problem / a.n_split;
    split = in_problem - qt * a.n_split;
    qlen = (int64_t)*a.n_uq;
    klen = a.n;
    t0 = qt * BM;
    if (t0 >= qlen) return;
    u_lo = split * a.key_run;
    u_hi = u_lo + a.key_run;
    if (u_hi > klen) u_hi = klen;
  } else {
    bb = blockIdx.y;  // one grid row per problem
    qlen = a.n;
    klen = a.n_globs;
    t0 = (int64_t)blockIdx.x * BM;
    if (t0 >= qlen) return;
    u_lo = 0;
    u_hi = klen;
  }

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  // the wavefront index as a scalar: everything derived from it (which key blocks this
  // wavefront needs) then branches on scalars instead of lane masks
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, h = lane >> 5;
  const T* Qp = (const T*)a.t.q;
  const T* Kp = (const T*)a.t.k;
  const T* Vp = (const T*)a.t.v;
  // PAD: rows of Q, K, V and out are dr < D elements long (a multiple of 16 bytes); the operands
  // are filled up with zeros, which change neither the scores nor the elements below dr
  const int dr = PAD ? (int)a.t.d : D;
  const float sc = 1.4426950408889634f / sqrtf((float)dr);
  const bool persist = (MODE == kTileGlobalCols) && a.persist != 0;
  // global modes: tokens of problem bb are rows bb * n + token of the stacked tensors (masks work
  // on the tokens, only addresses take the offset)
  const int64_t tok_off = (MODE == kTileBand) ? 0 : bb * a.n;
  bool staged = false;  // persist: the key tile is already in LDS

  // Q^T operand of a query tile, kept in registers.  A persistent workgroup asks for the rows of
  // its next query tile before it works on the current one (where the registers allow it).
  constexpr bool kNextQ = (MODE == kTileGlobalCols) && D <= 64;
  uint4v qh[kF32 ? 1 : C::QREGS], qh_next[(kNextQ && !kF32) ? C::QREGS : 1];
  float qf[kF32 ? C::QREGS : 1], qf_next[(kNextQ && kF32) ? C::QREGS : 1];
  auto load_q = [&](const T* qrow, uint4v* dh, float* df) {
    if constexpr (kF32) {
#pragma unroll
      for (int g = 0; g < D / 8; g++) {
        float4v x = {0.f, 0.f, 0.f, 0.f};
        if (!PAD || 8 * g + 4 * h < dr) x = *reinterpret_cast<const float4v*>(qrow + 8 * g + 4 * h);
        df[4 * g] = x[0];
        df[4 * g + 1] = x[1];
        df[4 * g + 2] = x[2];
        df[4 * g + 3] = x[3];
      }
    } else {
#pragma unroll
      for (int ks = 0; ks < C::QREGS; ks++) {
        dh[ks] = uint4v{0u, 0u, 0u, 0u};
        if (!PAD || 16 * ks + 8 * h < dr) dh[ks] = *reinterpret_cast<const uint4v*>(qrow + 16 * ks + 8 * h);
      }
    }
  };
  bool have_q = false;  // the rows of this trip were asked for during the previous one

  // One trip per query tile.  Only a persistent GlobalCols workgroup makes more than one.
  for (;; t0 += (int64_t)gridDim.x * BM) {
  if (t0 >= qlen) break;
  const bool pair_split = (MODE == kTileGlobalRows) && NB == 2 && a.pair_split != 0;
  const bool quad_split = (MODE == kTileBand) && quarter >= 0;
  // query block of this wavefront, and the share of the key blocks it is restricted to (-1: all)
  const int wave_q = quad_split ? 0 : pair_split ? (wave & 1) : wave;
  const int wave_k = quad_split ? wave : pair_split ? (wave >> 1) : -1;
  const int64_t tw0 = t0 + 32 * wave_q;  // first query of this wavefront
  const int64_t tq = tw0 + r;          // this lane's query position
  bool q_ok = tq < qlen;
  int64_t q_tok;                       // its token (row of Q / out)
  if constexpr (MODE == kTileBand) {
    q_tok = base + (q_ok ? tq : qlen - 1) * a.s;
  } else if constexpr (MODE == kTileGlobalRows) {
    q_tok = a.uq[q_ok ? tq : qlen - 1];
  } else {
    q_tok = q_ok ? tq : qlen - 1;
    if (q_ok && bit_is_set(a.gbits, q_tok)) q_ok = false;  // global rows belong to GlobalRows
  }

  if (!have_q) load_q(Qp + (q_tok + tok_off) * dr, qh, qf);
  // a persistent workgroup finishes a row every few microseconds: its incoming state is read
  // here, long before the write-back needs it
  float l_pre = 0.f, m_pre = 0.f;
  if constexpr (MODE == kTileGlobalCols) {
    l_pre = load_state<T>(a.t.l, q_tok + tok_off, a.t.state_f32 != 0);
    m_pre = load_state<T>(a.t.m, q_tok + tok_off, a.t.state_f32 != 0);
  }
  if constexpr (kNextQ) {
    const int64_t t0n = t0 + (int64_t)gridDim.x * BM;
    have_q = persist && t0n < qlen;
    if (have_q) {
      const int64_t tqn = t0n + 32 * wave_q + r;
      load_q(Qp + ((tqn < qlen ? tqn : qlen - 1) + tok_off) * dr, qh_next, qf_next);
    }
  }

  f32x16 o[EB];
#pragma unroll
  for (int eb = 0; eb < EB; eb++)
#pragma unroll
    for (int v = 0; v < 16; v++) o[eb][v] = 0.f;
  float m = kNegInf;  // running max in log2 units
  float l = 0.f;      // running sum over this lane's half of the keys


  // Tiles are fetched one ahead: the global loads of tile n+1 are issued before tile n is
  // consumed and land in registers; they are written to LDS once tile n has been consumed.
  auto key_tok = [&](int64_t u) -> int64_t {
    if constexpr (MODE == kTileBand) return base + u * a.s;
    else if constexpr (MODE == kTileGlobalRows) return u + tok_off;
    else {
      const int g = listed_token(a.globs[u], a.n);  // (an out-of-range entry reads row 0, masked below)
      return (int64_t)(g < 0 ? 0 : g) + tok_off;
    }
  };
  constexpr int CH = kF32 ? D / 4 : D / 8;       // 16-byte chunks per row
  constexpr int KIT = BN * CH / 256;             // chunks of K per thread and tile
  // half types, V: a lane stages the key pair jp = lane % (BN / 2) and 8 columns; the 64 / (BN / 2)
  // lanes of a pair times four wavefronts take VCOLS chunks of 8 columns per trip (d = 32: half
  // of the lanes have no columns to stage)
  constexpr int PAIRS = BN / 2, LPP = kWave / PAIRS, VCOLS = 4 * LPP;
  constexpr int VIT = kF32 ? KIT : (CH + VCOLS - 1) / VCOLS;
  static_assert(KIT >= 1 && C::LDS_BYTES + BN * 4 <= 160 * 1024, "tile shape does not fit");
  uint4v kreg[KIT], vreg[kF32 ? KIT : 2 * VIT];
  int ktok_reg = 0;

  auto fetch = [&](int64_t ut) {
#pragma unroll
    for (int it = 0; it < KIT; it++) {
      const int idx = it * 256 + tid;
      const int j = idx / CH, c = idx % CH;
      const int64_t u = ut + j;
      uint4v kx = {0u, 0u, 0u, 0u}, vx = {0u, 0u, 0u, 0u};
      if (u < u_hi && (!PAD || (16 / (int)sizeof(T)) * c < dr)) {
        const int64_t off = key_tok(u) * dr + (16 / (int)sizeof(T)) * c;
        kx = *reinterpret_cast<const uint4v*>(Kp + off);
        if constexpr (kF32) vx = *reinterpret_cast<const uint4v*>(Vp + off);
      }
      kreg[it] = kx;
      if constexpr (kF32) vreg[it] = vx;
    }
    if constexpr (!kF32) {
      // V: a lane takes the key pair (2*jp, 2*jp+1) and 8 columns e
#pragma unroll
      for (int it = 0; it < VIT; it++) {
        const int jp = lane % PAIRS;
        const int c = lane / PAIRS + LPP * (wave + 4 * it);
        const int64_t u = ut + 2 * jp;
        uint4v v0 = {0u, 0u, 0u, 0u}, v1 = {0u, 0u, 0u, 0u};
        const bool c_ok = c < CH && (!PAD || 8 * c < dr);
        if (u < u_hi && c_ok) v0 = *reinterpret_cast<const uint4v*>(Vp + key_tok(u) * dr + 8 * c);
        if (u + 1 < u_hi && c_ok) v1 = *reinterpret_cast<const uint4v*>(Vp + key_tok(u + 1) * dr + 8 * c);
        vreg[2 * it] = v0;
        vreg[2 * it + 1] = v1;
      }
    }
    if constexpr (MODE == kTileGlobalCols) {
      if (tid < BN) ktok_reg = (ut + tid < u_hi) ? listed_token(a.globs[ut + tid], a.n) : 0;
    }
  };

  auto stash = [&]() {
#pragma unroll
    for (int it = 0; it < KIT; it++) {
      const int idx = it * 256 + tid;
      const int j = idx / CH, c = idx % CH;
      if constexpr (kF32) {
        *reinterpret_cast<uint4v*>((float*)Ks + j * C::K_STRIDE + 4 * c) = kreg[it];
        *reinterpret_cast<uint4v*>((float*)Vs + j * C::V_STRIDE + 4 * c) = vreg[it];
      } else {
        *reinterpret_cast<uint4v*>(Ks + j * C::K_STRIDE + 8 * c) = kreg[it];
      }
    }
    if constexpr (!kF32) {
      // the 8 packed key pairs go down a column of the transposed tile
#pragma unroll
      for (int it = 0; it < VIT; it++) {
        const int jp = lane % PAIRS;
        const int c = lane / PAIRS + LPP * (wave + 4 * it);
        const uint4v v0 = vreg[2 * it], v1 = vreg[2 * it + 1];
        const int slot = key_slot(2 * jp);
        uint32_t* col = reinterpret_cast<uint32_t*>(Vs + (8 * c) * C::V_STRIDE + slot);
        if (c < CH) {
#pragma unroll
        for (int x = 0; x < 4; x++) {
          // dword x of v0/v1 holds columns 2x, 2x+1
          col[(2 * x) * (C::V_STRIDE / 2)] = __builtin_amdgcn_perm(v1[x], v0[x], 0x05040100u);
          col[(2 * x + 1) * (C::V_STRIDE / 2)] = __builtin_amdgcn_perm(v1[x], v0[x], 0x07060302u);
        }
        }
      }
    }
    if constexpr (MODE == kTileGlobalCols) {
      if (tid < BN) ktok_s[tid] = ktok_reg;
    }
  };

  if (u_lo < u_hi && !staged) fetch(u_lo);
  for (int64_t ut = u_lo; ut < u_hi; ut += BN) {
    if (!staged) {
      __syncthreads();  // the previous tile has been consumed
      stash();
      __syncthreads();
      if (ut + BN < u_hi) fetch(ut + BN);
    }
    if (persist) staged = true;

    // ---- this wavefront's share of the tile: up to two 32-key blocks
    // block jb holds keys ut + 32*jb .. +31; it matters iff it overlaps the wavefront's band
    bool need[NB];
    bool any_need = false;
#pragma unroll
    for (int jb = 0; jb < NB; jb++) {
      const int64_t ub = ut + 32 * jb;
      if constexpr (MODE == kTileBand)
        need[jb] = (tw0 < qlen) && (ub < u_hi) && (ub <= tw0 + 31 + a.w) && (ub + 31 + a.w >= tw0) &&
                   (wave_k < 0 || (int)(((ub - u_lo) >> 5) & 3) == wave_k);
      else
        need[jb] = (tw0 < qlen) && (ub < u_hi) && (wave_k < 0 || wave_k == jb);
      any_need = any_need || need[jb];
    }
    if (!any_need) continue;

    f32x16 sreg[NB];
    const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int jb = 0; jb < NB; jb++) {
      if (!need[jb]) continue;  // (filled with -inf below)
      if constexpr (kF32) {
        // operand reads run two groups of four instructions ahead (order pinned: left to
        // itself the compiler issues a read, waits for it and only then starts the four)
        const float* krow = (const float*)Ks + (32 * jb + r) * C::K_STRIDE + 4 * h;
        float4v kx[3];
        kx[0] = *reinterpret_cast<const float4v*>(krow);
        kx[1] = *reinterpret_cast<const float4v*>(krow + 8);
        sreg[jb] = zero16;
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
        for (int g = 0; g < D / 8; g++) {
          if (g + 2 < D / 8) {
            kx[(g + 2) % 3] = *reinterpret_cast<const float4v*>(krow + 8 * (g + 2));
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          }
#pragma unroll
          for (int i = 0; i < 4; i++)
            sreg[jb] = __builtin_amdgcn_mfma_f32_32x32x2f32(kx[g % 3][i], qf[4 * g + i], sreg[jb], 0, 0, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        }
      } else {
        const T* krow = Ks + (32 * jb + r) * C::K_STRIDE + 8 * h;
        sreg[jb] = mfma16<T>(*reinterpret_cast<const uint4v*>(krow), qh[0], zero16);
#pragma unroll
        for (int ks = 1; ks < D / 16; ks++) {
          uint4v kx = *reinterpret_cast<const uint4v*>(krow + 16 * ks);
          sreg[jb] = mfma16<T>(kx, qh[ks], sreg[jb]);
        }
      }
    }

    // ---- mask, running max, exponentials.  Scores stay un-scaled in the registers; the
    // 1/sqrt(d) * log2(e) factor is folded into the exponent's fma (it is positive, so the max
    // can be taken first).  Masks are 32-bit: a key is live iff (unsigned)(delta + w) <= 2w
    // (band; delta = key position - query position) or > 2w (global; delta in tokens).
    const uint32_t w32 = (uint32_t)a.w, w2 = 2u * (uint32_t)a.w;
    const int rem = (int)((u_hi - ut) < BN ? (u_hi - ut) : BN);  // live key slots of this tile
    uint32_t d0;
    if constexpr (MODE == kTileBand) d0 = (uint32_t)(int32_t)(ut - tq) + w32;
    else if constexpr (MODE == kTileGlobalRows) d0 = (uint32_t)(int32_t)(ut - q_tok) + w32;
    else d0 = w32 - (uint32_t)(int32_t)q_tok;
    float mx = kNegInf;
#pragma unroll
    for (int jb = 0; jb < NB; jb++) {
      if (!need[jb]) {
#pragma unroll
        for (int v = 0; v < 16; v++) sreg[jb][v] = kNegInf;
        continue;
      }
      bool full = false;  // every (query, key) pair of the block is live: no per-element test
      if constexpr (MODE == kTileBand) {
        const int64_t ub = ut + 32 * jb;
        full = (ub + 31 < u_hi) && (ub + a.w >= tw0 + 31) && (ub + 31 <= tw0 + a.w);
      } else if constexpr (MODE == kTileGlobalRows) {
        // keys are the tokens ub .. ub+31: live for every query unless the block touches the
        // window of one of this wavefront's query tokens
        const int64_t ub = ut + 32 * jb;
        const bool hit = (ub + 31 + a.w >= q_tok) && (ub <= q_tok + a.w);
        full = (ub + 31 < u_hi) && (__builtin_amdgcn_ballot_w64(hit) == 0);
      } else {
        // keys are listed tokens, queries the tokens tw0 .. tw0+31: live unless one of the
        // block's keys lies in the window of one of them
        const int64_t kt = (int64_t)ktok_s[32 * jb + r];
        const bool hit = kt < 0 || ((kt + a.w >= tw0) && (kt <= tw0 + 31 + a.w));
        full = (32 * jb + 31 < rem) && (__builtin_amdgcn_ballot_w64(hit) == 0);
      }
      if (!full) {
#pragma unroll
        for (int v = 0; v < 16; v++) {
          const int j = 32 * jb + 8 * (v / 4) + 4 * h + (v % 4);
          bool ok;
          if constexpr (MODE == kTileBand) ok = (d0 + (uint32_t)j <= w2);
          else if constexpr (MODE == kTileGlobalRows) ok = (d0 + (uint32_t)j > w2);
          else ok = (d0 + (uint32_t)ktok_s[j] > w2) && ktok_s[j] >= 0;
          if (!(ok && j < rem)) sreg[jb][v] = kNegInf;
        }
      }
#pragma unroll
      for (int v = 0; v < 16; v++) mx = fmaxf(mx, sreg[jb][v]);
    }
    mx = fmaxf(mx, shfl_xor_f32(mx, 32)) * sc;
    const float m_new = fmaxf(m, mx);
    const bool live = m_new > kNegInf;
    const float alpha = live ? __builtin_amdgcn_exp2f(m - m_new) : 1.f;
    const float neg_m = live ? -m_new : 0.f;
    float lsum = 0.f;
#pragma unroll
    for (int jb = 0; jb < NB; jb++)
#pragma unroll
      for (int v = 0; v < 16; v++) {
        // exp2(-inf) = 0 for masked entries
        const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sreg[jb][v], sc, neg_m));
        sreg[jb][v] = p;
        lsum += p;
      }
    l = l * alpha + lsum;
    m = m_new;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
      for (int eb = 0; eb < EB; eb++)
#pragma unroll
        for (int v = 0; v < 16; v++) o[eb][v] *= alpha;
    }

    // ---- O^T += V^T P^T
#pragma unroll
    for (int jb = 0; jb < NB; jb++) {
      if (!need[jb]) continue;
      if constexpr (kF32) {
        typedef RowPiece<EB> vecE;
        const float* vbase = (const float*)Vs + (32 * jb + 4 * h) * C::V_STRIDE + EB * r;
        // reads run PD keys ahead of the instructions that use them (order pinned, as above)
        constexpr int PD = 8 / EB;
        vecE vx[PD + 1];
#pragma unroll
        for (int v = 0; v < PD; v++)
          vx[v] = *reinterpret_cast<const vecE*>(vbase + (8 * (v / 4) + (v % 4)) * C::V_STRIDE);
        __builtin_amdgcn_sched_group_barrier(0x100, PD, 0);
#pragma unroll
        for (int v = 0; v < 16; v++) {
          if (v + PD < 16) {
            vx[(v + PD) % (PD + 1)] =
                *reinterpret_cast<const vecE*>(vbase + (8 * ((v + PD) / 4) + ((v + PD) % 4)) * C::V_STRIDE);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          }
#pragma unroll
          for (int eb = 0; eb < EB; eb++)
            o[eb] = __builtin_amdgcn_mfma_f32_32x32x2f32(vx[v % (PD + 1)][eb], sreg[jb][v], o[eb], 0, 0, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, EB, 0);
        }
      } else {
#pragma unroll
        for (int sl = 0; sl < 2; sl++) {
          uint4v pb;
#pragma unroll
          for (int x = 0; x < 4; x++)
            pb[x] = pack2<T>(sreg[jb][8 * sl + 2 * x], sreg[jb][8 * sl + 2 * x + 1]);
          const T* vcol = Vs + r * C::V_STRIDE + 32 * jb + 16 * sl + 8 * h;
#pragma unroll
          for (int eb = 0; eb < EB; eb++) {
            uint4v va = *reinterpret_cast<const uint4v*>(vcol + 32 * eb * C::V_STRIDE);
            o[eb] = mfma16<T>(va, pb, o[eb]);
          }
        }
      }
    }
  }

  // ---- finish: combine the two key halves, fold the incoming state in, write back
  l += shfl_xor_f32(l, 32);
  if constexpr ((MODE == kTileGlobalRows && NB == 2) || MODE == kTileBand) {
    if (pair_split || quad_split) {
      // fold the wavefronts that share a query block, upper half into lower half, through LDS
      // (the tiles are no longer needed): (q, 1) into (q, 0) for the pairs; 2, 3 into 0, 1 and
      // then 1 into 0 for the four wavefronts of a shared tail tile
      // (a shape whose exchange area does not fit the tile buffers is never launched with shared
      // query blocks: d = 256 has one key block per tile and no shared tail tiles)
      constexpr int XR = EB * 16 + 2;
      if constexpr (2 * XR * kWave * 4 <= C::LDS_BYTES) {
      const int nq = quad_split ? 1 : 2;
      for (int step = quad_split ? 2 : 1; step >= 1; step >>= 1) {
        const bool gives = wave_k >= step && wave_k < 2 * step;
        const bool takes = wave_k < step;
        float* xs = reinterpret_cast<float*>(lds) +
                    (size_t)(wave_q + nq * (gives ? wave_k - step : wave_k)) * XR * kWave + lane;
        __syncthreads();
        if (gives) {
#pragma unroll
          for (int eb = 0; eb < EB; eb++)
#pragma unroll
            for (int v = 0; v < 16; v++) xs[(eb * 16 + v) * kWave] = o[eb][v];
          xs[(EB * 16) * kWave] = m;
          xs[(EB * 16 + 1) * kWave] = l;
        }
        __syncthreads();
        if (takes) {
          const float m2 = xs[(EB * 16) * kWave], l2 = xs[(EB * 16 + 1) * kWave];
          const float m_new = fmaxf(m, m2);
          if (m_new > kNegInf) {
            const float fa = __builtin_amdgcn_exp2f(m - m_new), fb = __builtin_amdgcn_exp2f(m2 - m_new);
            l = l * fa + l2 * fb;
#pragma unroll
            for (int eb = 0; eb < EB; eb++)
#pragma unroll
              for (int v = 0; v < 16; v++) o[eb][v] = o[eb][v] * fa + xs[(eb * 16 + v) * kWave] * fb;
            m = m_new;
          }
        }
      }
      }
      if (wave_k != 0) return;  // (both modes make a single trip)
    }
  }
  if constexpr (MODE == kTileGlobalRows) {
    // partial result of this key split; an empty one is (m, l, acc) = (-inf, 0, 0)
    if (!q_ok) return;  // (this mode makes a single trip)
    const int64_t slot = (bb * a.n_globs + tq) * a.n_split + split;
    const bool any = l > 0.f;
    float* prow = a.pacc + slot * dr;  // (rows of the real length; elements from dr on are padding)
    if constexpr (kF32) {
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++)
#pragma unroll
        for (int c = 0; c < EB; c++) {
          float4v y = {0.f, 0.f, 0.f, 0.f};
          if (any) {
#pragma unroll
            for (int u = 0; u < 4; u++) y[u] = o[(4 * c + u) % EB][4 * g4 + (4 * c + u) / EB];
          }
          const int e = EB * (8 * g4 + 4 * h) + 4 * c;
          if (!PAD || e < dr) *reinterpret_cast<float4v*>(prow + e) = y;
        }
    } else {
#pragma unroll
      for (int eb = 0; eb < EB; eb++)
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
          float4v y = {0.f, 0.f, 0.f, 0.f};
          if (any) {
            y[0] = o[eb][4 * g4]; y[1] = o[eb][4 * g4 + 1]; y[2] = o[eb][4 * g4 + 2]; y[3] = o[eb][4 * g4 + 3];
          }
          const int e = 32 * eb + 8 * g4 + 4 * h;
          if (!PAD || e < dr) *reinterpret_cast<float4v*>(prow + e) = y;
        }
    }
    if (h == 0) {
      a.pm[slot] = any ? m * 0.6931471805599453f : kNegInf;
      a.pl[slot] = any ? l : 0.f;
    }
    return;
  }
  if (q_ok && l > 0.f && wave_k <= 0)
    tile_write_row<T, D>(a.t, q_tok + tok_off, h, m, l, o, 1.f, MODE == kTileGlobalCols, l_pre, m_pre, dr);
  if (!persist) break;
  if constexpr (kNextQ) {
    if (have_q) {
      if constexpr (kF32) {
#pragma unroll
        for (int i = 0; i < C::QREGS; i++) qf[i] = qf_next[i];
      } else {
#pragma unroll
        for (int i = 0; i < C::QREGS; i++) qh[i] = qh_next[i];
      }
    }
  }
  }  // query tiles
}

// ---------------------------------------------------------------------------------------
// Band masks, half types: tiles go from global memory straight into LDS
// ---------------------------------------------------------------------------------------
// Same tile problem and register layouts as tile_kernel<T, D, kTileBand>, different plumbing:
//   - K and V tiles are written to LDS by the load instructions themselves (16 bytes per lane,
//     64 lanes = 1 KB of consecutive LDS per instruction), row-major and unpadded; no staging
//     registers, no LDS store instructions.  A ring of NBUF tile buffers, one barrier per tile:
//     tile n + NBUF - 1 is requested right after the barrier that publishes tile n, into the
//     buffer that tile n - 1 has left.
//   - Rows are 128 or 256 bytes, a multiple of the bank cycle, so bank conflicts are avoided by
//     permuting the 16-byte chunks inside a row instead of padding: chunk c of row j is stored at
//     chunk position c ^ f(j).  K is read with 16-byte operand fetches by 8 consecutive rows at a
//     time (f = j mod chunks per row).  V is read with the transposing 8-byte load: a group of
//     16 lanes reads 4 keys x 16 columns (4 lanes per key, 4 columns per lane) and lane i
//     receives column i of the 4 keys, which is the V^T operand; f = 4 * (bank-cycle index mod
//     chunks/4) keeps the keys read by one instruction apart.
//   - The softmax runs per 32-key block; both S products of a tile are issued before the first
//     softmax step, so the matrix pipe works on the second block while the vector ALU is busy
//     with the first.
template <typename T, int D, int BN_>
struct BandDmaCfg {
  static constexpr int BM = 128, BN = BN_;      // queries per workgroup, keys per tile
  static constexpr int NB = BN / 32;            // 32-key blocks per tile
  static constexpr int ROWB = D * 2;            // bytes per K / V row
  static constexpr int CH = D / 8;              // 16-byte chunks per row
  static constexpr int RPC = ROWB < 256 ? 256 / ROWB : 1;  // rows per 256-byte bank cycle
  static constexpr int TILE_B = BN * ROWB;      // bytes of one K (or V) tile
  static constexpr int BUF_B = 2 * TILE_B;      // K tile then V tile
  static constexpr int NI = TILE_B / 4096;      // load instructions per wavefront, tile and matrix
  static constexpr int EB = D / 32, QREGS = D / 16;
  // Tile buffers.  A tile is requested NBUF - 1 steps before it is consumed.  A request takes
  // about 3500 clocks to land when the whole device streams tiles (measured with the cycle
  // counter), a 64-key step of the tile loop about 3300 at d = 128: with two buffers every step
  // waits for its data.  Four buffers fit 64 KB (two workgroups per CU) with 64-key tiles at
  // d = 64 and with 32-key tiles at d = 128.
  static constexpr int NBUF = 65536 / BUF_B < 4 ? 65536 / BUF_B : 4;
  static_assert(BN == 32 || BN == 64, "one or two 32-key blocks per tile");
  static_assert(NI >= 1 && NBUF >= 2, "tile too small or too large");
  // K rows: chunk c of row j is stored at chunk position c ^ kperm(j).  A K operand fetch reads
  // one 16-byte chunk of 16 consecutive rows; they cover the 16 chunk positions of a 256-byte
  // bank cycle once when the rows that start at the same place in the cycle (every 16 / CH-th
  // row for rows shorter than the cycle) get different positions.
  static constexpr int KSHIFT = CH >= 16 ? 0 : (CH == 8 ? 1 : 2);
  static constexpr int KMASK = (CH < 16 ? CH : 16) - 1;
  __device__ static constexpr int kperm(int j) { return (j >> KSHIFT) & KMASK; }
};

// keys per tile of band_dma_kernel (d = 256: two 32-KB buffers of 32 keys)
#ifndef SPFA_BAND_BN
#define SPFA_BAND_BN(D) ((D) > 128 ? 32 : 64)
#endif

// s_waitcnt vmcnt(N) alone (the other counters at their maximum), gfx9 encoding
#define SPFA_WAIT_VMCNT(N) __builtin_amdgcn_s_waitcnt(((N) & 15) | (((N) >> 4) << 14) | 0x0f70)

template <typename T, int D, int BN_>
__global__ __launch_bounds__(256, D > 128 ? 1 : 2) void band_dma_kernel(TileArgs a) {
  using C = BandDmaCfg<T, D, BN_>;
  constexpr int BM = C::BM, BN = C::BN, NB = C::NB, EB = C::EB, ROWB = C::ROWB, CH = C::CH, RPC = C::RPC;
  constexpr int TILE_B = C::TILE_B, BUF_B = C::BUF_B, NI = C::NI, NBUF = C::NBUF;
  static_assert(sizeof(T) == 2 && (D == 32 || D == 64 || D == 128 || D == 256), "half types, d = 32 ... 256");
  static_assert(2 * NI * (NBUF - 1) < 64, "outstanding tile loads must fit the vmcnt field");
  __shared__ __attribute__((aligned(1024))) char lds[NBUF * BUF_B];

  // workgroups are dealt round-robin to the 8 XCDs: give each XCD a contiguous run of tiles.
  // Tile numbers and positions inside a subsequence fit 32 bits (the launcher checks); everything
  // that is the same for the whole workgroup is moved to scalar registers.
  auto uni = [](int x) { return __builtin_amdgcn_readfirstlane(x); };
  // (the tiles of all problems of a batch form one list; problem bb starts at token bb * n)
  // Whole tiles first, then four workgroups for each of the last a.n_tail tiles (the tiles of a
  // sparsely filled last round): such a workgroup has 32 of the tile's queries, all four
  // wavefronts work on them and take the key tiles in turn (folded through LDS at the end).
  const uint32_t n_tiles = (uint32_t)a.n_tiles, tiles_per_sub = (uint32_t)a.tiles_per_sub;
  const uint32_t n_all = n_tiles * (uint32_t)a.t.n_batch;
  const uint32_t n_main = n_all - (uint32_t)a.n_tail;
  const uint32_t per_xcd = (n_main + 7u) / 8u;
  uint32_t lt;
  int quarter = -1;  // which 32 queries of a shared tail tile (-1: a whole tile)
  if (blockIdx.x < 8u * per_xcd) {
    lt = (blockIdx.x % 8u) * per_xcd + blockIdx.x / 8u;
    if (lt >= n_main) return;
  } else {
    const uint32_t qid = blockIdx.x - 8u * per_xcd;
    lt = n_main + qid / 4u;
    quarter = uni((int)(qid & 3u));
  }
  const bool quad = quarter >= 0;
  const uint32_t bb = lt / n_tiles;
  lt -= bb * n_tiles;
  const uint32_t sub = lt / tiles_per_sub;
  const int tile = uni((int)(lt - sub * tiles_per_sub));
  int64_t base;
  int qlen;
  if (a.block > 0) {
    base = (int64_t)sub * a.block + (int64_t)bb * a.n;
    qlen = (int)a.cnt;
  } else {
    base = (int64_t)sub + (int64_t)bb * a.n;
    qlen = uni((int)(((uint32_t)a.n - sub + (uint32_t)a.s - 1u) / (uint32_t)a.s));
  }
  const int wlim = (int)(a.w < (int64_t)0x3fffffff ? a.w : (int64_t)0x3fffffff);  // window, clamped
  const int t0 = tile * BM + (quad ? 32 * quarter : 0);
  const int qspan = quad ? 32 : BM;
  if (t0 >= qlen) return;
  const int u_lo = t0 > wlim ? t0 - wlim : 0;
  const int u_hi = (qlen - qspan - wlim > t0) ? t0 + qspan + wlim : qlen;
  // Key tiles are visited in a rotated order: the workgroups of neighbouring query tiles (the
  // same XCD has them, at the same time) walk ranges that overlap in all but BM / BN tiles, and
  // started at their own first tile they would ask for any one tile BM / BN steps apart, after
  // the L2 has seen a whole round of other tiles.  Visit number `it` is therefore the tile whose
  // number, counted along the subsequence, is it modulo the tile count, so that all of them ask
  // for the same tile at about the same time.  (The online softmax does not care about order.)
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
  const char* Kp = (const char*)a.t.k;
  const char* Vp = (const char*)a.t.v;
  const float sc = 1.4426950408889634f / sqrtf((float)D);

  // ---- tile loads: instruction `it` of this wavefront fills the 1-KB segment 4*it + wave of a
  // tile; this lane's 16 bytes are row j0 + it * RPI, chunk position p0 of it.  The chunk
  // permutation repeats every CH rows and an instruction covers a multiple of CH rows, so the
  // lane's offset for instruction `it` is that of instruction 0 plus whole rows, which go into
  // the scalar base: two offset registers serve every load.
  constexpr int RPI = 4096 / ROWB;  // rows per load instruction of the workgroup's four wavefronts
  // (d = 256: an instruction covers 8 rows, half a period of the K permutation; the other half
  // differs by one bit of the chunk position, KXOR below)
  static_assert((RPI % 16 == 0 || RPI == 8) && (RPI / RPC) % (CH / 4 > 0 ? CH / 4 : 1) == 0,
                "chunk permutation must repeat per instruction");
  const uint32_t row_step = (uint32_t)a.s * (uint32_t)ROWB;  // bytes between consecutive keys
  const int j0 = (wave * 1024 + lane * 16) / ROWB, p0 = ((wave * 1024 + lane * 16) % ROWB) / 16;
  constexpr int VPER = CH / 4 > 0 ? CH / 4 : 1;  // period of the V permutation (in bank cycles)
  const uint32_t koff = (uint32_t)j0 * row_step + (uint32_t)((p0 ^ C::kperm(j0)) * 16);
  const uint32_t voff = (uint32_t)j0 * row_step + (uint32_t)((p0 ^ (4 * ((j0 / RPC) % VPER))) * 16);
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  // The loads are written as instructions: scalar base + 32-bit lane offset, LDS address in M0.
  // (Through the builtin the compiler forms a 64-bit address per lane and load, and it orders the
  // loads against LDS reads it cannot tell apart from them; the waits for the tiles are explicit
  // below, the compiler does not know of these loads.)
  // The lane offsets of all NI instructions are kept in registers where there is room (up to
  // d = 128): a whole tile then costs one 64-bit scalar address per matrix and nothing per
  // instruction; only the last, partly filled tile of a subsequence computes clamped offsets.
  constexpr bool kOffRegs = D <= 128;
  uint32_t koffs[kOffRegs ? NI : 1], voffs[kOffRegs ? NI : 1];
  if constexpr (kOffRegs) {
#pragma unroll
    for (int it = 0; it < NI; it++) {
      koffs[it] = koff + (uint32_t)(it * RPI) * row_step;
      voffs[it] = voff + (uint32_t)(it * RPI) * row_step;
      if constexpr (RPI < 16) koffs[it] ^= (uint32_t)(C::kperm(it * RPI) * 16);
    }
  }
  const int64_t base_byte = base * (int64_t)ROWB;  // scalar
  auto request = [&](int ut, int stage) __attribute__((always_inline)) {
    const int64_t tile_byte = base_byte + (int64_t)ut * (int64_t)row_step;  // scalar
    const bool whole = ut + BN <= u_hi;
    if constexpr (kOffRegs) {
      if (whole) {
        const char* kp = Kp + tile_byte;
        const char* vp = Vp + tile_byte;
#pragma unroll
        for (int it = 0; it < NI; it++) {
          const uint32_t lds_k = lds_base + (uint32_t)(stage * BUF_B + (4 * it + wave) * 1024);
          asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                       :: "v"(koffs[it]), "s"(kp), "s"(lds_k) : "memory", "m0");
          asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                       :: "v"(voffs[it]), "s"(vp), "s"(lds_k + (uint32_t)TILE_B) : "memory", "m0");
        }
        return;
      }
    }
#pragma unroll
    for (int it = 0; it < NI; it++) {
      // whole tile: this instruction's rows are added to the scalar base; last tile of a
      // subsequence: they stay in the lane offset, where rows past the last key are replaced by
      // the last key (finite values; they are masked out)
      uint32_t ko = koff, vo = voff;
      int64_t it_byte = tile_byte + (int64_t)it * RPI * (int64_t)row_step;  // scalar
      if (!whole) {
        // (the opaque copy keeps the compiler from precomputing these products for every
        // instruction outside the tile loop, where they would hold registers all the time)
        int last = u_hi - 1 - ut;
        asm volatile("" : "+s"(last));
        const int j = j0 + it * RPI;
        // source row min(j, last), relative to the row j0 that koff / voff stand for (the sum is
        // non-negative; the unsigned arithmetic wraps to it when last < j0)
        const uint32_t rel = (uint32_t)((j > last ? last : j) - j0) * row_step;
        ko = koff + rel;
        vo = voff + rel;
        it_byte = tile_byte;
      }
      const uint32_t lds_k = lds_base + (uint32_t)(stage * BUF_B + (4 * it + wave) * 1024);
      if constexpr (RPI < 16) ko ^= (uint32_t)(C::kperm(it * RPI) * 16);  // (j0 < RPI: the bits do not overlap)
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :: "v"(ko), "s"(Kp + it_byte), "s"(lds_k) : "memory", "m0");
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :: "v"(vo), "s"(Vp + it_byte), "s"(lds_k + (uint32_t)TILE_B) : "memory", "m0");
    }
  };
  // the first NBUF - 1 tiles are on their way before anything else is loaded
#pragma unroll
  for (int i = 0; i < NBUF - 1; i++)
    if (i < nk) request(tile_start(i), i);

  const int tw0 = t0 + (quad ? 0 : 32 * wave);  // first query of this wavefront
  const int tq = tw0 + r;                       // this lane's query position
  const bool q_ok = tq < qlen;
  const int64_t q_tok = base + (int64_t)(q_ok ? tq : qlen - 1) * a.s;

  // ---- Q^T operand, kept in registers; the row's incoming state is asked for here as well, long
  // before the write-back needs it
  uint4v qh[C::QREGS];
  {
    const T* qrow = (const T*)a.t.q + q_tok * D;
#pragma unroll
    for (int ks = 0; ks < C::QREGS; ks++)
      qh[ks] = *reinterpret_cast<const uint4v*>(qrow + 16 * ks + 8 * h);
  }
  const uint32_t l_raw = load_state_raw<T>(a.t.l, q_tok, a.t.state_f32 != 0);
  const uint32_t m_raw = load_state_raw<T>(a.t.m, q_tok, a.t.state_f32 != 0);
  // Everything asked for so far is waited for here, once: the compiler keeps count of the loads
  // it knows (Q, the state) and would otherwise wait for them inside the tile loop with counts
  // that make the tile requests it does not know of complete as well.
  SPFA_WAIT_VMCNT(0);

  // ---- operand addresses inside a tile buffer (bytes)
  // K block jb, step ks: row 32*jb + r, chunk 2*ks + h
  int kadr[C::QREGS];
#pragma unroll
  for (int ks = 0; ks < C::QREGS; ks++) kadr[ks] = r * ROWB + (((2 * ks + h) ^ C::kperm(r)) * 16);
  // V: group of 16 lanes = (column half r_hi, key half h); lane 4*x + y of the group points at
  // key 4*h + x (+ 8 for the second half of an operand), columns 32*eb + 16*r_hi + 4*y .. +3,
  // i.e. chunk 4*eb + 2*r_hi + y/2, stored at that chunk ^ g with g = 4 * gx a whole number of
  // eb steps: the row's eb order is permuted, the chunk inside an eb is not
  int vadr[EB];
  {
    const int x = (lane & 15) >> 2, y = lane & 3, r_hi = (lane >> 4) & 1;
    const int key = 4 * h + x;
    const int gx = (key / RPC) % VPER;
    const int common = TILE_B + key * ROWB + (2 * r_hi + (y >> 1)) * 16 + (y & 1) * 8;
#pragma unroll
    for (int eb = 0; eb < EB; eb++) vadr[eb] = common + 64 * (eb ^ gx);
  }

  f32x16 o[EB];
#pragma unroll
  for (int eb = 0; eb < EB; eb++)
#pragma unroll
    for (int v = 0; v < 16; v++) o[eb][v] = 0.f;
  constexpr float kSlack = 8.f;
  float m = kNegInf;        // reference maximum of the exponentials, log2 units
  float neg_m = 0.f;        // -m (0 while m is -inf), the addend of the exponent
  float thr_raw = kNegInf;  // (m + kSlack) / sc: a raw score above it moves the reference
  float mt_raw = kNegInf;   // true running maximum of this lane's raw scores (its half of the keys)
  // Row sums of P: one more result block of the second product whose A operand is all ones, so
  // every row of it is the sum over all keys (both halves of the wavefront) of the ROUNDED
  // weights, the ones the numerator is built from; only lsum[0] is ever read.  (Not at d = 256,
  // where the registers are all taken: there the sum is a chain of additions, l_add, over this
  // lane's half of the keys.)
#ifndef SPFA_BAND_MFMA_SUM
#define SPFA_BAND_MFMA_SUM(D) ((D) <= 64)
#endif
  constexpr bool kMfmaSum = SPFA_BAND_MFMA_SUM(D);
  float l_add = 0.f;
  f32x16 lsum;
#pragma unroll
  for (int v = 0; v < 16; v++) lsum[v] = 0.f;
  const uint32_t one2 = sizeof(T) == 2 && __is_same(T, bf16) ? 0x3f803f80u : 0x3c003c00u;
  const uint4v ones = {one2, one2, one2, one2};
  const float inv_sc = sqrtf((float)D) * 0.6931471805599453f;

  typedef short s16x4 __attribute__((ext_vector_type(4)));
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  constexpr int QR = C::QREGS;
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  // One online-softmax step over a 32-key block whose dead entries are -inf already; leaves the
  // exponentials in s.  The exponentials are taken against a reference maximum m that is only
  // moved (and the accumulators rescaled) when a row's maximum has grown by more than kSlack
  // (log2 units) since the reference was set: the weights then stay below 2^kSlack, the final
  // division by the row sum cancels the reference, and the rescale is rare instead of happening
  // on every block while the maxima are still settling.  The common path is 8 three-input
  // maxima, one compare, and a multiply-add + exponential per score: the running maximum stays
  // per lane and in raw units (the two lanes of a query only meet when the reference moves, and
  // once at the end for the row statistics), and the row sum comes out of the matrix pipe.
  auto soft_max = [&](const f32x16& s) __attribute__((always_inline)) {
    float mx = mt_raw;
#pragma unroll
    for (int v = 0; v < 16; v += 2) mx = fmaxf(fmaxf(mx, s[v]), s[v + 1]);
    mt_raw = mx;
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(mx > thr_raw) != 0, 0)) {
      // (m = -inf: first live block of a row, nothing accumulated yet - for the whole wavefront
      // when this is its first live block, and then there is nothing to rescale)
      const bool fresh = __builtin_amdgcn_ballot_w64(m > kNegInf) == 0;
      const float mp = fmaxf(mx, shfl_xor_f32(mx, 32)) * sc;
      const float m_new = (mp > m + kSlack) ? mp : m;
      const float alpha = (m > kNegInf) ? __builtin_amdgcn_exp2f(m - m_new) : 0.f;
      m = m_new;
      neg_m = (m > kNegInf) ? -m : 0.f;
      thr_raw = (m + kSlack) * inv_sc;
      if (!fresh) {
        lsum[0] *= alpha;
        l_add *= alpha;
#pragma unroll
        for (int eb = 0; eb < EB; eb++)
#pragma unroll
          for (int v = 0; v < 16; v++) o[eb][v] *= alpha;
      }
    }
  };
  // ... and its second half: the exponentials, packed as the B operands of the second product
  auto soft_exp = [&](f32x16& s, uint4v (&pb)[2]) __attribute__((always_inline)) {
#pragma unroll
    for (int v = 0; v < 16; v++)
      s[v] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], sc, neg_m));  // exp2(-inf) = 0
    if constexpr (!kMfmaSum) {
      float part = 0.f;
#pragma unroll
      for (int v = 0; v < 16; v++) part += s[v];
      l_add += part;
    }
#pragma unroll
    for (int sl = 0; sl < 2; sl++)
#pragma unroll
      for (int x = 0; x < 4; x++) pb[sl][x] = pack2<T>(s[8 * sl + 2 * x], s[8 * sl + 2 * x + 1]);
  };
  auto soft_core = [&](f32x16& s, uint4v (&pb)[2]) __attribute__((always_inline)) {
    soft_max(s);
    soft_exp(s, pb);
  };
  // V^T operands of block jb of the tile at tb: [sl][eb], two transposing 8-byte reads each
  auto v_fetch = [&](const char* tb, int jb, uint4v (&va)[2 * EB]) __attribute__((always_inline)) {
#pragma unroll
    for (int sl = 0; sl < 2; sl++)
#pragma unroll
      for (int eb = 0; eb < EB; eb++) {
        const char* va_p = tb + (32 * jb + 16 * sl) * ROWB + vadr[eb];
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)va_p);
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(va_p + 8 * ROWB));
        const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        va[sl * EB + eb] = __builtin_bit_cast(uint4v, both);
      }
  };
  // O^T += V_block^T P_block^T
  auto pv = [&](const uint4v (&pb)[2], const uint4v (&va)[2 * EB]) __attribute__((always_inline)) {
#pragma unroll
    for (int sl = 0; sl < 2; sl++) {
#pragma unroll
      for (int eb = 0; eb < EB; eb++) o[eb] = mfma16<T>(va[sl * EB + eb], pb[sl], o[eb]);
      if constexpr (kMfmaSum) lsum = mfma16<T>(ones, pb[sl], lsum);
    }
  };

  // What a 32-key block that starts at key ub is to this wavefront's 32 queries: dead when
  // ub < blk_dead_lo or ub > blk_dead_hi (no live pair: before every window, after every window
  // or past the last key), full when blk_full_lo <= ub <= blk_full_hi (every pair live: inside
  // every query's window and whole).  Positions and the clamped window are below 2^30.
  const bool wave_live = tw0 < qlen;
  const int blk_dead_lo = tw0 - wlim - 31;
  const int blk_dead_hi = (tw0 + 31 + wlim < u_hi - 1) ? tw0 + 31 + wlim : u_hi - 1;
  const int blk_full_lo = tw0 + 31 - wlim;
  const int blk_full_hi = (tw0 - 31 + wlim < u_hi - 32) ? tw0 - 31 + wlim : u_hi - 32;

  // one tile: wait for it, publish it, request the tile NBUF - 1 steps ahead into the buffer the
  // previous step has freed, consume it
  auto step = [&](int it, int stage) __attribute__((always_inline)) {
    const int ut = tile_start(it);
    const char* tb = lds + stage * BUF_B;
    // this wavefront's part of the tile has landed: the loads complete in order, and the tiles
    // requested after this one (at most NBUF - 2) may still be under way
    if constexpr (NBUF > 2) {
      const int after = nk - 1 - it;  // tiles behind this one
      if (after >= 2) SPFA_WAIT_VMCNT(2 * 2 * NI);
      else if (after == 1) SPFA_WAIT_VMCNT(2 * NI);
      else SPFA_WAIT_VMCNT(0);
      static_assert(NBUF <= 4, "one more case per buffer");
    } else {
      SPFA_WAIT_VMCNT(0);
    }
    __syncthreads();  // everyone's has, and everyone is done with the buffer of the previous step

    // What the 32-key blocks of the tile are to this wavefront's 32 queries (all of it the same
    // for the whole wavefront, so the code below branches on scalars).  A block is dead when no
    // (query, key) pair of it is live; a live block needs a per-element test when some query's
    // window starts after the block's first key, or some query's window (or the subsequence)
    // ends before its last key.  A dead block beside a live one is computed and masked out.
    // (positions and the clamped window are below 2^30, so the sums stay inside 32 bits)
    // (the four bounds of a block's first key are set up once per wavefront, before the loop)
    bool test[NB];
    bool none = true;
#pragma unroll
    for (int jb = 0; jb < NB; jb++) {
      const int ub = ut + 32 * jb;
      const bool dead = !wave_live || ub < blk_dead_lo || ub > blk_dead_hi;
      test[jb] = !(ub >= blk_full_lo && ub <= blk_full_hi);  // (a dead block is never full)
      none = none && dead;
    }
    // (a shared tail tile: the wavefronts take the key tiles in turn)
    if (quad && (it & 3) != wave) none = true;

    // The K operands of the first block are asked for before the next tile is requested:
    // the four wavefronts issue their tile loads in one burst right after the barrier, and the
    // operand reads come back while that burst drains.
    uint4v ka[QR];
    if (!none) {
#pragma unroll
      for (int ks = 0; ks < QR; ks++) ka[ks] = *reinterpret_cast<const uint4v*>(tb + kadr[ks]);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (it + NBUF - 1 < nk) request(tile_start(it + NBUF - 1), (stage + NBUF - 1) % NBUF);
    __builtin_amdgcn_sched_barrier(0);
    if (none) return;

    // the band test of a block (a compare and a select per element); its per-lane bounds are
    // only worked out for a block that needs them (the opaque copy keeps the compiler from
    // moving that work in front of the branch, into every step)
    auto band_test = [&](f32x16& s, int jb, bool test) __attribute__((always_inline)) {
      if (test) {
        int ut_o = ut;
        asm volatile("" : "+s"(ut_o));
        // key slot j of the tile is live for this lane's query iff jlo <= j <= jhi; the slots
        // this lane holds are c + 4*h for compile-time c, so the bounds are shifted by 4*h once
        const int live_slots = (u_hi - ut_o) < BN ? (u_hi - ut_o) : BN;
        const int jlo = (tq - wlim - ut_o) - 4 * h;
        const int jhi_band = tq + wlim - ut_o;
        const int jhi = (jhi_band < live_slots - 1 ? jhi_band : live_slots - 1) - 4 * h;
        // both ends at once: (unsigned)(c - jlo) <= jhi - jlo; a query without a live key in the
        // tile (jhi < jlo) gets bounds that no c meets
        const int jlo_both = jhi >= jlo ? jlo : 0x40000000;
        const uint32_t span = jhi >= jlo ? (uint32_t)(jhi - jlo) : 0u;
#pragma unroll
        for (int v = 0; v < 16; v++) {
          const int c = 32 * jb + 8 * (v / 4) + (v % 4);
          s[v] = ((uint32_t)(c - jlo_both) <= span) ? s[v] : kNegInf;
        }
      }
    };

    uint4v va[2 * EB];
    // Operands are fetched from LDS well ahead of the products that use them, in an order the
    // scheduler is told to keep.
    if constexpr (NB == 2) {
      // the K operands of block 1 while the S product of block 0 runs, the V operands of a block
      // before its softmax step
      uint4v kb[QR];
      f32x16 s0 = zero16, s1 = zero16;
#pragma unroll
      for (int ks = 0; ks < QR; ks++) {
        kb[ks] = *reinterpret_cast<const uint4v*>(tb + 32 * ROWB + kadr[ks]);
        s0 = mfma16<T>(ka[ks], qh[ks], s0);
      }
      // one LDS read behind every matrix instruction
#pragma unroll
      for (int ks = 0; ks < QR; ks++) {
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < QR; ks++) s1 = mfma16<T>(kb[ks], qh[ks], s1);
      v_fetch(tb, 0, va);
      __builtin_amdgcn_sched_barrier(0);
      uint4v pb[2];
      band_test(s0, 0, test[0]);
      soft_core(s0, pb);
      pv(pb, va);
      __builtin_amdgcn_sched_barrier(0);
      v_fetch(tb, 1, va);
      __builtin_amdgcn_sched_barrier(0);
      band_test(s1, 1, test[1]);
      soft_core(s1, pb);
      pv(pb, va);
    } else {
      // one block: its V operands are read while the S product runs
      f32x16 s0 = zero16;
      v_fetch(tb, 0, va);
#pragma unroll
      for (int ks = 0; ks < QR; ks++) s0 = mfma16<T>(ka[ks], qh[ks], s0);
      __builtin_amdgcn_sched_barrier(0);
      uint4v pb[2];
      band_test(s0, 0, test[0]);
      soft_core(s0, pb);
      pv(pb, va);
    }
  };

  // (unrolled over the buffers, so that every LDS address is a register plus a constant)
  for (int it = 0; it < nk; it += NBUF) {
#pragma unroll
    for (int sg = 0; sg < NBUF; sg++)
      if (it + sg < nk) step(it + sg, sg);
  }

  // ---- listed global tokens as further keys (the window + global composite): a query that is
  // not a listed token itself attends the listed tokens outside its window
  // (Sparse_FlashAttention_Global_No_Local/sp_flatt_global_no_local_kernel.cu:38-64); the rows
  // of the listed tokens are not touched here.  The listed tokens' K and V rows are gathered
  // into the first tile buffer, BN of them at a time; a list entry counts every time it is
  // listed, an entry outside [0, n) not at all.
  if (a.globs != nullptr) {
    __shared__ int gtok_s[BN];  // token of every key of the gathered tile (-1: no key)
    const int64_t tok_base = (int64_t)bb * a.n;             // first row of this problem
    const int64_t tq_tok = q_tok - tok_base;                // this lane's query token
    const bool q_plain = q_ok && !bit_is_set(a.gbits, tq_tok);
    const uint32_t w32 = (uint32_t)wlim, w2 = 2u * (uint32_t)wlim;
    const uint32_t d0 = w32 - (uint32_t)(int32_t)tq_tok;    // key token + d0 > 2w: outside the window
    const int ng = (int)a.n_globs;
    for (int gt = 0; gt < ng; gt += BN) {
      __syncthreads();  // everyone is done with the buffer (band tiles, or the previous gathered tile)
#pragma unroll
      for (int it = 0; it < NI; it++) {
        const int j = j0 + it * RPI;  // key slot of the tile this lane loads a chunk of
        int g = -1;
        if (gt + j < ng) g = listed_token(a.globs[gt + j], a.n);
        if (p0 == 0) gtok_s[j] = g;
        const uint32_t row_byte = (uint32_t)((tok_base + (g < 0 ? 0 : g)) * (int64_t)ROWB);
        const uint32_t ko = row_byte + (uint32_t)((p0 ^ C::kperm(j)) * 16);
        const uint32_t vo = row_byte + (uint32_t)((p0 ^ (4 * ((j / RPC) % VPER))) * 16);
        const uint32_t lds_k = lds_base + (uint32_t)((4 * it + wave) * 1024);
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :: "v"(ko), "s"(Kp), "s"(lds_k) : "memory", "m0");
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :: "v"(vo), "s"(Vp), "s"(lds_k + (uint32_t)TILE_B) : "memory", "m0");
      }
      SPFA_WAIT_VMCNT(0);
      __syncthreads();
      if (tw0 >= qlen) continue;
      const char* tb = lds;
#pragma unroll
      for (int jb = 0; jb < NB; jb++) {
        if (gt + 32 * jb >= ng) break;
        uint4v ka[QR], va[2 * EB];
#pragma unroll
        for (int ks = 0; ks < QR; ks++) ka[ks] = *reinterpret_cast<const uint4v*>(tb + 32 * jb * ROWB + kadr[ks]);
        v_fetch(tb, jb, va);
        f32x16 s0 = zero16;
#pragma unroll
        for (int ks = 0; ks < QR; ks++) s0 = mfma16<T>(ka[ks], qh[ks], s0);
#pragma unroll
        for (int v = 0; v < 16; v++) {
          const int tok = gtok_s[32 * jb + 8 * (v / 4) + 4 * h + (v % 4)];
          const bool ok = q_plain && tok >= 0 && ((uint32_t)tok + d0 > w2);
          s0[v] = ok ? s0[v] : kNegInf;
        }
        uint4v pb[2];
        soft_core(s0, pb);
        pv(pb, va);
      }
    }
  }

  // (the matrix product has summed over both halves of the wavefront)
  float l = kMfmaSum ? lsum[0] : l_add + shfl_xor_f32(l_add, 32);
  float mt = fmaxf(mt_raw, shfl_xor_f32(mt_raw, 32)) * sc;  // true maximum, log2 units
  if (quad) {
    // fold the four wavefronts (same queries, different key tiles) through LDS, 2, 3 into 0, 1
    // and then 1 into 0; the tile buffers are no longer needed
    constexpr int XR = EB * 16 + 3;
    if constexpr (2 * XR * kWave * 4 <= NBUF * BUF_B) {
      for (int fs = 2; fs >= 1; fs >>= 1) {
        const bool gives = wave >= fs && wave < 2 * fs;
        const bool takes = wave < fs;
        float* xs = reinterpret_cast<float*>(lds) + (size_t)(gives ? wave - fs : wave) * XR * kWave + lane;
        __syncthreads();
        if (gives) {
#pragma unroll
          for (int eb = 0; eb < EB; eb++)
#pragma unroll
            for (int v = 0; v < 16; v++) xs[(eb * 16 + v) * kWave] = o[eb][v];
          xs[(EB * 16) * kWave] = m;
          xs[(EB * 16 + 1) * kWave] = l;
          xs[(EB * 16 + 2) * kWave] = mt;
        }
        __syncthreads();
        if (takes) {
          const float m2 = xs[(EB * 16) * kWave], l2 = xs[(EB * 16 + 1) * kWave];
          mt = fmaxf(mt, xs[(EB * 16 + 2) * kWave]);
          const float m_new = fmaxf(m, m2);
          if (m_new > kNegInf) {
            const float fa = __builtin_amdgcn_exp2f(m - m_new), fb = __builtin_amdgcn_exp2f(m2 - m_new);
            l = l * fa + l2 * fb;
#pragma unroll
            for (int eb = 0; eb < EB; eb++)
#pragma unroll
              for (int v = 0; v < 16; v++) o[eb][v] = o[eb][v] * fa + xs[(eb * 16 + v) * kWave] * fb;
            m = m_new;
          }
        }
      }
    }
    if (wave != 0) return;
  }
  if (q_ok && l > 0.f) {
    // hand the row over relative to its true maximum: (m, l, o) -> (mt, l * 2^(m - mt), o)
    // (o is divided by l later, so only l changes)
    const float shrink = __builtin_amdgcn_exp2f(m - mt);
    tile_write_row<T, D>(a.t, q_tok, h, mt, l * shrink, o, shrink, true,
                         state_from_raw<T>(l_raw, a.t.state_f32 != 0), state_from_raw<T>(m_raw, a.t.state_f32 != 0));
  }
}

// ---------------------------------------------------------------------------------------
// Band masks, fp32: tiles go from global memory straight into LDS
// ---------------------------------------------------------------------------------------
// The fp32 counterpart of band_dma_kernel: the same plumbing (two 32-KB tile buffers filled by the
// load instructions, one barrier per tile, reference maximum with slack) around the fp32
// products of tile_kernel (k pairing and permuted output rows, 16-byte operand reads).  A tile is
// 4096 floats of K and of V: 64 keys at d = 64, 32 keys at d = 128.  Rows are 256 or 512 bytes,
// so chunk c of row j sits at chunk position c ^ (j mod 16): the 16 rows read by a quarter of a
// wavefront for one K operand, and the 16 consecutive chunks of one row read for a V operand,
// then cover every bank once.
template <int D>
struct BandDmaF32Cfg {
  static constexpr int BM = 128;
  static constexpr int BN = 4096 / D;           // keys per tile
  static constexpr int NB = BN / 32;            // 32-key blocks per tile
  static constexpr int ROWB = D * 4;            // bytes per K / V row
  static constexpr int TILE_B = BN * ROWB;      // bytes of one K (or V) tile: 16 KB
  static constexpr int BUF_B = 2 * TILE_B;      // K tile then V tile
  static constexpr int NI = TILE_B / 4096;      // load instructions per wavefront, tile and matrix
  static constexpr int EB = D / 32, QREGS = D / 2;
};

template <int D>
__global__ __launch_bounds__(256, 2) void band_dma_f32_kernel(TileArgs a) {
  using C = BandDmaF32Cfg<D>;
  constexpr int BM = C::BM, BN = C::BN, NB = C::NB, EB = C::EB, ROWB = C::ROWB;
  constexpr int TILE_B = C::TILE_B, BUF_B = C::BUF_B, NI = C::NI;
  static_assert(D == 64 || D == 128, "d = 64 or 128");
  __shared__ __attribute__((aligned(1024))) char lds_even[BUF_B];
  __shared__ __attribute__((aligned(1024))) char lds_odd[BUF_B];

  auto uni = [](int x) { return __builtin_amdgcn_readfirstlane(x); };
  // whole tiles first (a contiguous run per XCD), then four workgroups for each shared tail tile
  const int64_t n_main = a.n_tiles * a.t.n_batch - a.n_tail;
  const int64_t per_xcd = (n_main + 7) / 8;
  int64_t lt;
  int quarter = -1;  // which 32 queries of a shared tail tile (-1: a whole tile)
  if ((int64_t)blockIdx.x < 8 * per_xcd) {
    lt = (int64_t)(blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (lt >= n_main) return;
  } else {
    const int64_t qid = (int64_t)blockIdx.x - 8 * per_xcd;
    lt = n_main + qid / 4;
    quarter = uni((int)(qid & 3));
  }
  const bool quad = quarter >= 0;
  const int64_t bb = lt / a.n_tiles;
  lt -= bb * a.n_tiles;
  const int64_t sub = lt / a.tiles_per_sub;
  const int tile = uni((int)(lt - sub * a.tiles_per_sub));
  int64_t base;
  int qlen;
  if (a.block > 0) {
    base = sub * a.block + bb * a.n;
    qlen = (int)a.cnt;
  } else {
    base = sub + bb * a.n;
    qlen = uni((int)((a.n - sub + a.s - 1) / a.s));
  }
  const int wlim = (int)(a.w < (int64_t)0x3fffffff ? a.w : (int64_t)0x3fffffff);  // window, clamped
  // a shared tail tile: this workgroup has 32 of its queries, all four wavefronts work on them
  // and take the key tiles in turn
  const int t0 = tile * BM + (quad ? 32 * quarter : 0);
  const int qspan = quad ? 32 : BM;
  if (t0 >= qlen) return;
  const int u_lo = t0 > wlim ? t0 - wlim : 0;
  const int u_hi = (qlen - qspan - wlim > t0) ? t0 + qspan + wlim : qlen;
  // key tiles are visited in a rotated order, so that the workgroups of neighbouring query tiles
  // ask for the same tile at about the same time (see band_dma_kernel)
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
  const char* Kp = (const char*)a.t.k;
  const char* Vp = (const char*)a.t.v;
  const float sc = 1.4426950408889634f / sqrtf((float)D);

  const int tw0 = t0 + (quad ? 0 : 32 * wave);  // first query of this wavefront
  const int tq = tw0 + r;          // this lane's query position
  const bool q_ok = tq < qlen;
  const int64_t q_tok = base + (int64_t)(q_ok ? tq : qlen - 1) * a.s;

  // ---- Q^T operand, kept in registers: half h holds k = 8g + 4h + i in qf[4g + i]
  float qf[C::QREGS];
  {
    const float* qrow = (const float*)a.t.q + q_tok * D;
#pragma unroll
    for (int g = 0; g < D / 8; g++) {
      const float4v x = *reinterpret_cast<const float4v*>(qrow + 8 * g + 4 * h);
      qf[4 * g] = x[0];
      qf[4 * g + 1] = x[1];
      qf[4 * g + 2] = x[2];
      qf[4 * g + 3] = x[3];
    }
  }

  // ---- tile loads: instruction `it` of this wavefront fills the 1-KB segment 4*it + wave of a
  // tile; this lane's 16 bytes are row j, chunk position p of it (K and V alike)
  uint32_t toff[NI];  // byte offset of the lane's source chunk from the tile's first row
  const uint32_t row_step = (uint32_t)a.s * (uint32_t)ROWB;  // bytes between consecutive keys
#pragma unroll
  for (int it = 0; it < NI; it++) {
    const int at = (4 * it + wave) * 1024 + lane * 16;
    const int j = at / ROWB, p = (at % ROWB) / 16;
    toff[it] = (uint32_t)j * row_step + (uint32_t)((p ^ (j & 15)) * 16);
  }
  auto request = [&](int ut, char* dst_buf) {
    const int64_t tile_byte = (base + (int64_t)ut * a.s) * (int64_t)ROWB;  // scalar
    const bool whole = ut + BN <= u_hi;
#pragma unroll
    for (int it = 0; it < NI; it++) {
      uint32_t off = toff[it];
      if (!whole) {
        // rows past the last key repeat the last key (finite values; they are masked out)
        const int last = u_hi - 1 - ut;
        const int j = ((4 * it + wave) * 1024 + lane * 16) / ROWB;
        if (j > last) {
          // (the chunk permutation depends on the row's slot in the tile, not on the key)
          off -= (uint32_t)(j - last) * row_step;
        }
      }
      char* dst = dst_buf + (4 * it + wave) * 1024;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(Kp + tile_byte + off),
                                       (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(Vp + tile_byte + off),
                                       (__attribute__((address_space(3))) void*)(dst + TILE_B), 16, 0, 0);
    }
  };

  // ---- operand addresses inside a tile buffer (bytes).  A chunk index is compile-time bits
  // XOR a per-lane value, so eight addresses (the low three variable bits) serve every operand
  // and the rest is a constant offset.
  // K, block jb, group g: row 32*jb + r, chunk 2*g + h, at position (2*g) ^ (h ^ (r mod 16))
  int kadr[8];
#pragma unroll
  for (int gl = 0; gl < 8; gl++) kadr[gl] = r * ROWB + (((2 * gl) ^ (h ^ (r & 15))) * 16);
  // V, register v: row 8*(v/4) + 4*h + v%4 (+ 32*jb), the lane's EB floats from element EB*r:
  // chunk (EB*r)/4, at position that ^ (row mod 16) = ((EB*r)/4 ^ 4*h) ^ cv, cv = 8*((v/4)%2) + v%4
  int vadr[8];
#pragma unroll
  for (int x = 0; x < 8; x++) {
    const int cv = 8 * (x / 4) + (x % 4);
    vadr[x] = TILE_B + (4 * h + cv) * ROWB + (((((EB * r) / 4) ^ (4 * h)) ^ cv) * 16) + ((EB * r) % 4) * 4;
  }

  f32x16 o[EB];
#pragma unroll
  for (int eb = 0; eb < EB; eb++)
#pragma unroll
    for (int v = 0; v < 16; v++) o[eb][v] = 0.f;
  constexpr float kSlack = 8.f;
  float m = kNegInf;   // reference maximum of the exponentials, log2 units
  float mt = kNegInf;  // true running maximum
  float l = 0.f;       // running sum (relative to m) over this lane's half of the keys

  // one online-softmax step over a 32-key block whose dead entries are -inf already (reference
  // maximum with slack, as in band_dma_kernel); leaves the exponentials in s
  auto soft_core = [&](f32x16& s) __attribute__((always_inline)) {
    float mx = s[0];
#pragma unroll
    for (int v = 1; v < 16; v++) mx = fmaxf(mx, s[v]);
    mx = fmaxf(mx, shfl_xor_f32(mx, 32)) * sc;
    mt = fmaxf(mt, mx);
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(mx > m + kSlack) != 0, 0)) {
      const float m_new = (mx > m + kSlack) ? mx : m;
      const float alpha = (m > kNegInf) ? __builtin_amdgcn_exp2f(m - m_new) : 0.f;
      m = m_new;
      l *= alpha;
#pragma unroll
      for (int eb = 0; eb < EB; eb++)
#pragma unroll
        for (int v = 0; v < 16; v++) o[eb][v] *= alpha;
    }
    const float neg_m = (m > kNegInf) ? -m : 0.f;
    float lsum = 0.f;
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], sc, neg_m));  // exp2(-inf) = 0
      s[v] = p;
      lsum += p;
    }
    l += lsum;
  };
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  // S^T = K Q^T of the 32-key block at kb, operand reads two groups of four instructions ahead
  // (order pinned)
  auto s_product = [&](const char* kb) __attribute__((always_inline)) -> f32x16 {
    float4v kx[3];
    kx[0] = *reinterpret_cast<const float4v*>(kb + kadr[0]);
    kx[1] = *reinterpret_cast<const float4v*>(kb + kadr[1]);
    f32x16 sb = zero16;
    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
    for (int g = 0; g < D / 8; g++) {
      if (g + 2 < D / 8) {
        kx[(g + 2) % 3] = *reinterpret_cast<const float4v*>(kb + kadr[(g + 2) % 8] + 256 * ((g + 2) / 8));
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; i++)
        sb = __builtin_amdgcn_mfma_f32_32x32x2f32(kx[g % 3][i], qf[4 * g + i], sb, 0, 0, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
    }
    return sb;
  };
  // O^T += V^T P^T of the 32-key block at vb, V reads PD keys ahead (order pinned)
  auto pv_product = [&](const char* vb, const f32x16& sb) __attribute__((always_inline)) {
    typedef float vecE __attribute__((ext_vector_type(EB)));
    constexpr int PD = 8 / EB;
    vecE vx[PD + 1];
#pragma unroll
    for (int v = 0; v < PD; v++)
      vx[v] = *reinterpret_cast<const vecE*>(vb + vadr[v % 8] + 16 * ROWB * (v / 8));
    __builtin_amdgcn_sched_group_barrier(0x100, PD, 0);
#pragma unroll
    for (int v = 0; v < 16; v++) {
      if (v + PD < 16) {
        vx[(v + PD) % (PD + 1)] =
            *reinterpret_cast<const vecE*>(vb + vadr[(v + PD) % 8] + 16 * ROWB * ((v + PD) / 8));
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
#pragma unroll
      for (int eb = 0; eb < EB; eb++)
        o[eb] = __builtin_amdgcn_mfma_f32_32x32x2f32(vx[v % (PD + 1)][eb], sb[v], o[eb], 0, 0, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, EB, 0);
    }
  };

  auto step = [&](int it, const char* tb, char* other) __attribute__((always_inline)) {
    const int ut = tile_start(it);
    __builtin_amdgcn_s_waitcnt(0);  // this wavefront's part of the tile has landed
    __syncthreads();                // everyone's has, and everyone is done with the other buffer
    if (it + 1 < nk) request(tile_start(it + 1), other);

    const bool all_full = (ut + BN <= u_hi) && (ut >= tw0 + 31 - wlim) && (ut + BN - 1 - wlim <= tw0);
    const bool none = (tw0 >= qlen) || (ut - wlim > tw0 + 31) || (ut + BN - 1 < tw0 - wlim) ||
                      (quad && (it & 3) != wave);
    if (none) return;

    // key slot j of the tile is live for this lane's query iff jlo <= j <= jhi; the slots this
    // lane holds are c + 4*h for compile-time c, so the bounds are shifted by 4*h once
    const int live_slots = (u_hi - ut) < BN ? (u_hi - ut) : BN;
    const int jlo = (tq - wlim - ut) - 4 * h;
    const int jhi_band = tq + wlim - ut;
    const int jhi = (jhi_band < live_slots - 1 ? jhi_band : live_slots - 1) - 4 * h;
    const uint32_t span = (uint32_t)(jhi - jlo);  // jhi < jlo: wraps to a huge value, handled below
    const bool any_live = jhi >= jlo;

    // the band test of a block, then the softmax step
    auto soft = [&](f32x16& s, int jb) {
      if (!all_full) {
#pragma unroll
        for (int v = 0; v < 16; v++) {
          const int c = 32 * jb + 8 * (v / 4) + (v % 4);
          const bool ok = any_live && ((uint32_t)(c - jlo) <= span);
          s[v] = ok ? s[v] : kNegInf;
        }
      }
      soft_core(s);
    };

    // a 32-key block without a live pair beside a live one (the first and the last tile of a
    // wavefront's band) is left out: here the matrix instructions are the time
    bool live[NB];
#pragma unroll
    for (int jb = 0; jb < NB; jb++) {
      const int ub = ut + 32 * jb;
      live[jb] = NB == 1 || !((ub >= u_hi) || (ub - wlim > tw0 + 31) || (ub + 31 < tw0 - wlim));
    }
    f32x16 s[NB];
#pragma unroll
    for (int jb = 0; jb < NB; jb++)
      if (live[jb]) s[jb] = s_product(tb + 32 * jb * ROWB);
    // ---- softmax and O^T += V^T P^T per block
#pragma unroll
    for (int jb = 0; jb < NB; jb++) {
      if (!live[jb]) continue;
      soft(s[jb], jb);
      __builtin_amdgcn_sched_barrier(0);
      pv_product(tb + 32 * jb * ROWB, s[jb]);
    }
  };

  request(tile_start(0), lds_even);
  for (int it = 0; it < nk; it += 2) {
    step(it, lds_even, lds_odd);
    if (it + 1 < nk) step(it + 1, lds_odd, lds_even);
  }

  // ---- listed global tokens as further keys (the window + global composite), as in
  // band_dma_kernel: a query that is not a listed token itself attends the listed tokens outside
  // its window; their K and V rows are gathered into the first tile buffer, BN at a time.  (Never
  // together with shared tail tiles: the launcher makes none for such a call.)
  if (a.globs != nullptr) {
    __shared__ int gtok_s[BN];  // token of every key of the gathered tile (-1: no key)
    const int64_t tok_base = bb * a.n;        // first row of this problem
    const int64_t tq_tok = q_tok - tok_base;  // this lane's query token
    const bool q_plain = q_ok && !bit_is_set(a.gbits, tq_tok);
    const uint32_t w32 = (uint32_t)wlim, w2 = 2u * (uint32_t)wlim;
    const uint32_t d0 = w32 - (uint32_t)(int32_t)tq_tok;  // key token + d0 > 2w: outside the window
    const int ng = (int)a.n_globs;
    for (int gt = 0; gt < ng; gt += BN) {
      __builtin_amdgcn_s_waitcnt(0);
      __syncthreads();  // everyone is done with the buffer (band tiles, or the previous gathered tile)
#pragma unroll
      for (int it = 0; it < NI; it++) {
        const int at = (4 * it + wave) * 1024 + lane * 16;
        const int j = at / ROWB, p = (at % ROWB) / 16;  // key slot and chunk position this lane fills
        int g = -1;
        if (gt + j < ng) g = listed_token(a.globs[gt + j], a.n);
        if (p == 0) gtok_s[j] = g;
        const int64_t src = (tok_base + (g < 0 ? 0 : g)) * (int64_t)ROWB + (int64_t)((p ^ (j & 15)) * 16);
        char* dst = lds_even + (4 * it + wave) * 1024;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(Kp + src),
                                         (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(Vp + src),
                                         (__attribute__((address_space(3))) void*)(dst + TILE_B), 16, 0, 0);
      }
      __builtin_amdgcn_s_waitcnt(0);
      __syncthreads();
      if (tw0 >= qlen) continue;
#pragma unroll
      for (int jb = 0; jb < NB; jb++) {
        if (gt + 32 * jb >= ng) break;
        f32x16 sg = s_product(lds_even + 32 * jb * ROWB);
#pragma unroll
        for (int v = 0; v < 16; v++) {
          const int tok = gtok_s[32 * jb + 8 * (v / 4) + 4 * h + (v % 4)];
          const bool ok = q_plain && tok >= 0 && ((uint32_t)tok + d0 > w2);
          sg[v] = ok ? sg[v] : kNegInf;
        }
        soft_core(sg);
        __builtin_amdgcn_sched_barrier(0);
        pv_product(lds_even + 32 * jb * ROWB, sg);
      }
    }
  }

  l += shfl_xor_f32(l, 32);
  if (quad) {
    // fold the four wavefronts (same queries, different key tiles) through LDS, 2, 3 into 0, 1
    // and then 1 into 0; the tile buffers are no longer needed
    constexpr int XR = EB * 16 + 3;
    static_assert(XR * kWave * 4 <= BUF_B, "exchange area does not fit a tile buffer");
    for (int step = 2; step >= 1; step >>= 1) {
      const bool gives = wave >= step && wave < 2 * step;
      const bool takes = wave < step;
      // (one exchange slot in each of the two buffers)
      float* xs = reinterpret_cast<float*>((gives ? wave - step : wave) ? lds_odd : lds_even) + lane;
      __builtin_amdgcn_s_waitcnt(0);
      __syncthreads();
      if (gives) {
#pragma unroll
        for (int eb = 0; eb < EB; eb++)
#pragma unroll
          for (int v = 0; v < 16; v++) xs[(eb * 16 + v) * kWave] = o[eb][v];
        xs[(EB * 16) * kWave] = m;
        xs[(EB * 16 + 1) * kWave] = l;
        xs[(EB * 16 + 2) * kWave] = mt;
      }
      __syncthreads();
      if (takes) {
        const float m2 = xs[(EB * 16) * kWave], l2 = xs[(EB * 16 + 1) * kWave];
        mt = fmaxf(mt, xs[(EB * 16 + 2) * kWave]);
        const float m_new = fmaxf(m, m2);
        if (m_new > kNegInf) {
          const float fa = __builtin_amdgcn_exp2f(m - m_new), fb = __builtin_amdgcn_exp2f(m2 - m_new);
          l = l * fa + l2 * fb;
#pragma unroll
          for (int eb = 0; eb < EB; eb++)
#pragma unroll
            for (int v = 0; v < 16; v++) o[eb][v] = o[eb][v] * fa + xs[(eb * 16 + v) * kWave] * fb;
          m = m_new;
        }
      }
    }
    if (wave != 0) return;
  }
  if (q_ok && l > 0.f) {
    // hand the row over relative to its true maximum: (m, l, o) -> (mt, l * 2^(m - mt), o)
    const float shrink = __builtin_amdgcn_exp2f(m - mt);
    tile_write_row<float, D>(a.t, q_tok, h, mt, l * shrink, o, shrink);
  }
}

// ---------------------------------------------------------------------------------------
// Global mask, half types, at most 64 listed tokens: every other token against the listed ones
// ---------------------------------------------------------------------------------------
// The column pass of the global mask (queries = the tokens that are not listed, keys = the listed
// tokens outside the query's window, Sparse_FlashAttention_Global_No_Local/
// sp_flatt_global_no_local_kernel.cu:38-64,146-162) when all keys fit one 64-key tile: there is no
// running state across key tiles, so a query tile is one S product, one softmax and one P V
// product, and everything that does not depend on the query tile is set up once per workgroup:
//   - the listed tokens' K and V rows are gathered into LDS (band_dma_kernel's layout and loads)
//     and read from there ONCE, into registers: both matrix operands (K rows; V^T through the
//     transposing read) stay in registers for every query tile of the workgroup, as do the listed
//     tokens themselves in the order of the score registers;
//   - a wavefront's 32 consecutive Q rows are one contiguous piece of memory: the load
//     instructions write it straight into the wavefront's own LDS buffer (1 KB per instruction,
//     every cache line whole), two buffers, the next tile's rows asked for before the current
//     tile is worked on; no barrier in the tile loop;
//   - almost no wavefront has a listed token within reach of its 32 queries (64 tokens among a
//     million): one compare per lane (lane = key slot) and a ballot tell, and only then are the
//     window and "query is listed itself" tests made per score;
//   - the row sums come out of the matrix pipe (an all-ones operand), which idles here;
//   - finished rows leave through the wavefront's LDS buffer as whole rows, 1 KB per store
//     instruction (76 -> 61 us for 1 M tokens at d = 64 without this, 51 us with it: the rate of
//     a plain device copy of the same bytes); rows with an incoming state, and wavefronts near a
//     listed token, take the general write-back.
// A persistent grid; a workgroup walks query tiles blockIdx.x, blockIdx.x + gridDim.x, ...
template <typename T, int D>
__global__ __launch_bounds__(256, 2) void global_cols_dma_kernel(TileArgs a) {
  using C = BandDmaCfg<T, D, 64>;
  constexpr int BN = 64, EB = C::EB, ROWB = C::ROWB, RPC = C::RPC, CH = C::CH, TILE_B = C::TILE_B;
  constexpr int QR = C::QREGS, NI = C::NI;
  constexpr int QB = 32 * ROWB;       // bytes of a wavefront's 32 Q rows
  constexpr int QNI = QB / 1024;      // load instructions for them
  constexpr int QROWS = 1024 / ROWB;  // rows per load instruction
  static_assert(sizeof(T) == 2 && (D == 32 || D == 64), "half types, d = 32 or 64");
  __shared__ __attribute__((aligned(1024))) char lds[2 * TILE_B + 4 * 2 * QB];
  __shared__ int gtok_s[BN];  // token of every key slot (-1: no key)

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, h = lane >> 5;
  const int64_t bb = blockIdx.y;             // one grid row per problem
  const int64_t tok_base = bb * a.n;          // first row of this problem
  const char* Qp = (const char*)a.t.q + tok_base * ROWB;
  const char* Kp = (const char*)a.t.k;
  const char* Vp = (const char*)a.t.v;
  const float sc = 1.4426950408889634f / sqrtf((float)D);
  const int n = (int)a.n, ng = (int)a.n_globs;
  const int wlim = (int)(a.w < (int64_t)0x3fffffff ? a.w : (int64_t)0x3fffffff);
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  constexpr int VPER = CH / 4 > 0 ? CH / 4 : 1;

  // ---- the key tile, once: gathered by token, band_dma_kernel's chunk permutations
  {
    constexpr int RPI = 4096 / ROWB;
    const int j0 = (wave * 1024 + lane * 16) / ROWB, p0 = ((wave * 1024 + lane * 16) % ROWB) / 16;
#pragma unroll
    for (int it = 0; it < NI; it++) {
      const int j = j0 + it * RPI;
      int g = -1;
      if (j < ng) g = listed_token(a.globs[j], a.n);
      if (p0 == 0) gtok_s[j] = g;
      const uint32_t row_byte = (uint32_t)((tok_base + (g < 0 ? 0 : g)) * (int64_t)ROWB);
      const uint32_t ko = row_byte + (uint32_t)((p0 ^ C::kperm(j)) * 16);
      const uint32_t vo = row_byte + (uint32_t)((p0 ^ (4 * ((j / RPC) % VPER))) * 16);
      const uint32_t lds_k = lds_base + (uint32_t)((4 * it + wave) * 1024);
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :: "v"(ko), "s"(Kp), "s"(lds_k) : "memory", "m0");
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :: "v"(vo), "s"(Vp), "s"(lds_k + (uint32_t)TILE_B) : "memory", "m0");
    }
  }

  // ---- Q rows of a query tile: instruction i of this wavefront fills rows QROWS*i .. of its
  // buffer; this lane's 16 bytes are row jq, chunk position pq, i.e. source chunk pq ^ kperm(row)
  // (the layout of a K tile: the B operand reads below are the A operand reads of band_dma_kernel)
  const int jq = lane * 16 / ROWB, pq = (lane * 16 % ROWB) / 16;
  char* const qbuf = lds + 2 * TILE_B + wave * 2 * QB;
  const uint32_t qbuf_lds = lds_base + (uint32_t)(2 * TILE_B + wave * 2 * QB);
  const int n_tiles = (n + 127) / 128;
  auto request_q = [&](int qt, int buf) __attribute__((always_inline)) {
    const int tw0 = qt * 128 + 32 * wave;
    const char* src = Qp + (int64_t)tw0 * ROWB;  // scalar
#pragma unroll
    for (int i = 0; i < QNI; i++) {
      const int j = QROWS * i + jq;
      // rows past the last token repeat the last token (their lanes never write)
      int row = j;
      if (tw0 + 31 >= n) row = tw0 + j < n ? j : n - 1 - tw0;
      const uint32_t off = (uint32_t)(row * ROWB + ((pq ^ C::kperm(j)) * 16));
      const uint32_t dst = qbuf_lds + (uint32_t)(buf * QB + i * 1024);
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :: "v"(off), "s"(src), "s"(dst) : "memory", "m0");
    }
  };
  int qt = (int)blockIdx.x;
  if (qt < n_tiles && qt * 128 + 32 * wave < n) request_q(qt, 0);
  SPFA_WAIT_VMCNT(0);
  __syncthreads();  // the key tile and the token table are complete

  // ---- operands that do not depend on the query tile, read once
  uint4v ka[2][QR], va[2][2 * EB];
  int tokv[2][16];
  {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    const int x = (lane & 15) >> 2, y = lane & 3, r_hi = (lane >> 4) & 1;
    const int key = 4 * h + x;
    const int gx = (key / RPC) % VPER;
    const int common = TILE_B + key * ROWB + (2 * r_hi + (y >> 1)) * 16 + (y & 1) * 8;
#pragma unroll
    for (int jb = 0; jb < 2; jb++) {
#pragma unroll
      for (int ks = 0; ks < QR; ks++)
        ka[jb][ks] = *reinterpret_cast<const uint4v*>(lds + (32 * jb + r) * ROWB +
                                                     (((2 * ks + h) ^ C::kperm(32 * jb + r)) * 16));
#pragma unroll
      for (int sl = 0; sl < 2; sl++)
#pragma unroll
        for (int eb = 0; eb < EB; eb++) {
          const char* va_p = lds + (32 * jb + 16 * sl) * ROWB + common + 64 * (eb ^ gx);
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)va_p);
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(va_p + 8 * ROWB));
          const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          va[jb][sl * EB + eb] = __builtin_bit_cast(uint4v, both);
        }
#pragma unroll
      for (int v = 0; v < 16; v++) tokv[jb][v] = gtok_s[32 * jb + 8 * (v / 4) + 4 * h + (v % 4)];
    }
  }
  const int tok_lane = gtok_s[lane];  // lane = key slot
  const bool all_keys = __builtin_amdgcn_ballot_w64(tok_lane < 0) == 0;
  const uint32_t one2 = __is_same(T, bf16) ? 0x3f803f80u : 0x3c003c00u;
  const uint4v ones = {one2, one2, one2, one2};
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const bool sf = a.t.state_f32 != 0;
  const int kq_adr = r * ROWB;  // B operand of step ks: row r, chunk (2*ks + h) ^ kperm(r)

  int buf = 0;
  for (; qt < n_tiles; qt += (int)gridDim.x, buf ^= 1) {
    const int tw0 = qt * 128 + 32 * wave;
    const int qn = qt + (int)gridDim.x;
    // this tile's rows have landed (asked for a whole tile ago); the next tile's are asked for now
    SPFA_WAIT_VMCNT(0);
    asm volatile("" ::: "memory");  // (the reads of the buffer below stay behind the wait)
    if (qn < n_tiles && qn * 128 + 32 * wave < n) request_q(qn, buf ^ 1);
    if (tw0 >= n) continue;  // (a wavefront past the end: its workgroup has no barrier to keep)
    const int tq = tw0 + r;
    const bool q_ok = tq < n;
    const int64_t q_row = tok_base + (q_ok ? tq : n - 1);
    // the row's incoming state, long before the write-back needs it
    const uint32_t l_raw = load_state_raw<T>(a.t.l, q_row, sf);
    const uint32_t m_raw = load_state_raw<T>(a.t.m, q_row, sf);

    uint4v qh[QR];
    char* qb = qbuf + buf * QB;
#pragma unroll
    for (int ks = 0; ks < QR; ks++)
      qh[ks] = *reinterpret_cast<const uint4v*>(qb + kq_adr + (((2 * ks + h) ^ C::kperm(r)) * 16));
    f32x16 s[2];
#pragma unroll
    for (int jb = 0; jb < 2; jb++) {
      s[jb] = zero16;
#pragma unroll
      for (int ks = 0; ks < QR; ks++) s[jb] = mfma16<T>(ka[jb][ks], qh[ks], s[jb]);
    }
    // Is any listed token within reach of one of this wavefront's queries (inside a window, or
    // a query itself)?  Else every pair of the tile is live.
    const bool near = (uint32_t)(tok_lane - tw0 + wlim) <= (uint32_t)(31 + 2 * wlim) && tok_lane >= 0;
    bool q_plain = q_ok;
    if (__builtin_expect(!all_keys || __builtin_amdgcn_ballot_w64(near) != 0, 0)) {
      q_plain = q_ok && !bit_is_set(a.gbits, tq);
      const uint32_t d0 = (uint32_t)wlim - (uint32_t)tq, w2 = 2u * (uint32_t)wlim;
#pragma unroll
      for (int jb = 0; jb < 2; jb++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
          const int tok = tokv[jb][v];
          const bool ok = q_plain && tok >= 0 && ((uint32_t)tok + d0 > w2);
          s[jb][v] = ok ? s[jb][v] : kNegInf;
        }
    }
    float mx = s[0][0];
#pragma unroll
    for (int jb = 0; jb < 2; jb++)
#pragma unroll
      for (int v = jb == 0 ? 1 : 0; v < 16; v++) mx = fmaxf(mx, s[jb][v]);
    const float m2 = fmaxf(mx, shfl_xor_f32(mx, 32)) * sc;  // row maximum, log2 units
    const float neg_m = (m2 > kNegInf) ? -m2 : 0.f;
    f32x16 o[EB], lsum = zero16;
#pragma unroll
    for (int eb = 0; eb < EB; eb++) o[eb] = zero16;
#pragma unroll
    for (int jb = 0; jb < 2; jb++) {
#pragma unroll
      for (int v = 0; v < 16; v++)
        s[jb][v] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[jb][v], sc, neg_m));  // exp2(-inf) = 0
#pragma unroll
      for (int sl = 0; sl < 2; sl++) {
        uint4v pb;
#pragma unroll
        for (int x = 0; x < 4; x++) pb[x] = pack2<T>(s[jb][8 * sl + 2 * x], s[jb][8 * sl + 2 * x + 1]);
#pragma unroll
        for (int eb = 0; eb < EB; eb++) o[eb] = mfma16<T>(va[jb][sl * EB + eb], pb, o[eb]);
        lsum = mfma16<T>(ones, pb, lsum);
      }
    }
    const float l = lsum[0];  // (summed over both halves of the wavefront by the product)
    const float l_in = state_from_raw<T>(l_raw, sf);
    // Every row of the wavefront is written and none has an incoming state (the common case):
    // the rows go through the wavefront's LDS buffer (its Q rows are in registers by now) and
    // leave as whole rows, 1 KB per store instruction, instead of 32-byte pieces of 32 rows.
    const bool plain_rows = q_plain == q_ok && l > 0.f && l_in == 0.f;
    if (__builtin_amdgcn_ballot_w64(!plain_rows) == 0) {
      const float inv = 1.f / l;
      typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
#pragma unroll
      for (int eb = 0; eb < EB; eb++)
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
          u32x2 y;
          y[0] = pack2<T>(o[eb][4 * g4] * inv, o[eb][4 * g4 + 1] * inv);
          y[1] = pack2<T>(o[eb][4 * g4 + 2] * inv, o[eb][4 * g4 + 3] * inv);
          // element 32*eb + 8*g4 + 4*h: chunk 4*eb + g4 of the row (stored at that ^ row mod 8 ... CH), half h
          const int pos = (4 * eb + g4) ^ (r & (CH - 1));
          *reinterpret_cast<u32x2*>(qb + r * ROWB + pos * 16 + 8 * h) = y;
        }
      if (h == 0 && q_ok) {
        store_state<T>(a.t.m, q_row, m2 * 0.6931471805599453f, sf);
        store_state<T>(a.t.l, q_row, l, sf);
      }
      char* orow0 = (char*)a.t.out + (tok_base + tw0) * (int64_t)ROWB;
#pragma unroll
      for (int i = 0; i < QNI; i++) {
        const int row = QROWS * i + jq;
        const uint4v piece = *reinterpret_cast<const uint4v*>(qb + row * ROWB + ((pq ^ (row & (CH - 1))) * 16));
        if (tw0 + row < n) *reinterpret_cast<uint4v*>(orow0 + row * ROWB + pq * 16) = piece;
      }
      continue;
    }
    if (q_plain && l > 0.f)
      tile_write_row<T, D>(a.t, q_row, h, m2, l, o, 1.f, true, l_in, state_from_raw<T>(m_raw, sf));
  }
}

// ---------------------------------------------------------------------------------------
// Global mask, half types, at most 64 listed tokens: the listed tokens' rows against everything
// ---------------------------------------------------------------------------------------
// The row pass of the global mask (queries = the distinct listed tokens, keys = every token
// outside the query's window) is a stream of K and V read once against queries that fit in
// registers, with next to no arithmetic per byte, so it is written as independent wavefronts
// instead of workgroups in step: a workgroup owns one split of the key range (as in
// tile_kernel<.., kTileGlobalRows>), its four wavefronts take 32-key blocks in turn, and each
// wavefront has its own two LDS buffers that the load instructions fill (a block is 32
// consecutive rows: one contiguous piece of K and one of V, 1 KB per instruction); no barrier in
// the loop, the next block is asked for before the current one is worked on.  Both 32-query
// blocks are computed from one read of a block's operands.  The running maximum is a reference
// with slack as in band_dma_kernel; row sums come out of the matrix pipe.  At the end the four
// wavefronts are folded through LDS and the workgroup writes one partial (m, l, acc) per query
// for global_rows_merge_kernel.
template <typename T, int D>
__global__ __launch_bounds__(256, 2) void global_rows_dma_kernel(TileArgs a) {
  using C = BandDmaCfg<T, D, 64>;
  constexpr int EB = C::EB, ROWB = C::ROWB, RPC = C::RPC, CH = C::CH, QR = C::QREGS;
  constexpr int BB = 32 * ROWB;       // bytes of a 32-row block of K (or V)
  constexpr int BNI = BB / 1024;      // load instructions per block and matrix
  constexpr int BROWS = 1024 / ROWB;  // rows per load instruction
  constexpr int VPER = CH / 4 > 0 ? CH / 4 : 1;
  constexpr int STAGE_B = 2 * BB;     // K block then V block
  constexpr int XR = EB * 16 + 3;     // floats per lane of a folded state
  static_assert(sizeof(T) == 2 && (D == 32 || D == 64), "half types, d = 32 or 64");
  static_assert(2 * XR * kWave * 4 <= 4 * 2 * STAGE_B, "the fold does not fit the block buffers");
  __shared__ __attribute__((aligned(1024))) char lds[4 * 2 * STAGE_B];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, h = lane >> 5;
  // grid: [problem][key split]
  const int64_t per_problem = (int64_t)gridDim.x / a.t.n_batch;
  const int64_t bb = blockIdx.x / per_problem;
  const int64_t split = blockIdx.x - bb * per_problem;
  const int nq = (int)*a.n_uq;
  const int n = (int)a.n;
  const int u_lo = (int)(split * a.key_run);
  const int u_hi = u_lo + (int)a.key_run < n ? u_lo + (int)a.key_run : n;
  if (u_lo >= u_hi || nq <= 0) return;
  const int64_t tok_base = bb * a.n;
  const char* Kp = (const char*)a.t.k + tok_base * ROWB;
  const char* Vp = (const char*)a.t.v + tok_base * ROWB;
  const float sc = 1.4426950408889634f / sqrtf((float)D);
  const float inv_sc = sqrtf((float)D) * 0.6931471805599453f;
  const int wlim = (int)(a.w < (int64_t)0x3fffffff ? a.w : (int64_t)0x3fffffff);
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  char* const wbuf = lds + wave * 2 * STAGE_B;
  const uint32_t wbuf_lds = lds_base + (uint32_t)(wave * 2 * STAGE_B);
  const bool two = nq > 32;  // a second block of queries

  // ---- block loads: instruction i fills rows BROWS*i .. of the block; this lane's 16 bytes are
  // row jl, chunk position pl of it (K and V with band_dma_kernel's chunk permutations)
  const int jl = lane * 16 / ROWB, pl = (lane * 16 % ROWB) / 16;
  auto request = [&](int ub, int stage) __attribute__((always_inline)) {
    const char* ksrc = Kp + (int64_t)ub * ROWB;  // scalar
    const char* vsrc = Vp + (int64_t)ub * ROWB;
#pragma unroll
    for (int i = 0; i < BNI; i++) {
      const int j = BROWS * i + jl;
      // rows past the last token repeat the last token (finite values; they are masked out)
      int row = j;
      if (ub + 31 >= n) row = ub + j < n ? j : n - 1 - ub;
      const uint32_t ko = (uint32_t)(row * ROWB + ((pl ^ C::kperm(j)) * 16));
      const uint32_t vo = (uint32_t)(row * ROWB + ((pl ^ (4 * ((j / RPC) % VPER))) * 16));
      const uint32_t dst = wbuf_lds + (uint32_t)(stage * STAGE_B + i * 1024);
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :: "v"(ko), "s"(ksrc), "s"(dst) : "memory", "m0");
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :: "v"(vo), "s"(vsrc), "s"(dst + (uint32_t)BB) : "memory", "m0");
    }
  };
  const int n_blk = (u_hi - u_lo + 31) / 32;
  if (wave < n_blk) request(u_lo + 32 * wave, 0);

  // ---- the queries: Q^T operands of both 32-query blocks, kept in registers
  int q_tok[2];
  bool q_ok[2];
  uint4v qh[2][QR];
#pragma unroll
  for (int qb = 0; qb < 2; qb++) {
    const int tq = 32 * qb + r;
    q_ok[qb] = tq < nq;
    q_tok[qb] = a.uq[q_ok[qb] ? tq : nq - 1];
    const T* qrow = (const T*)a.t.q + (tok_base + q_tok[qb]) * D;
#pragma unroll
    for (int ks = 0; ks < QR; ks++) qh[qb][ks] = *reinterpret_cast<const uint4v*>(qrow + 16 * ks + 8 * h);
  }

  // ---- operand addresses inside a stage (bytes): K block row r, chunk 2*ks + h; V as in
  // band_dma_kernel (a group of 16 lanes reads 4 keys x 16 columns transposed)
  int kadr[QR], vadr[EB];
#pragma unroll
  for (int ks = 0; ks < QR; ks++) kadr[ks] = r * ROWB + (((2 * ks + h) ^ C::kperm(r)) * 16);
  {
    const int x = (lane & 15) >> 2, y = lane & 3, r_hi = (lane >> 4) & 1;
    const int key = 4 * h + x;
    const int gx = (key / RPC) % VPER;
    const int common = BB + key * ROWB + (2 * r_hi + (y >> 1)) * 16 + (y & 1) * 8;
#pragma unroll
    for (int eb = 0; eb < EB; eb++) vadr[eb] = common + 64 * (eb ^ gx);
  }

  constexpr float kSlack = 8.f;
  f32x16 o[2][EB], lsum[2];
  float m[2], neg_m[2], thr_raw[2], mt_raw[2];
#pragma unroll
  for (int qb = 0; qb < 2; qb++) {
#pragma unroll
    for (int eb = 0; eb < EB; eb++)
#pragma unroll
      for (int v = 0; v < 16; v++) o[qb][eb][v] = 0.f;
#pragma unroll
    for (int v = 0; v < 16; v++) lsum[qb][v] = 0.f;
    m[qb] = kNegInf;
    neg_m[qb] = 0.f;
    thr_raw[qb] = kNegInf;
    mt_raw[qb] = kNegInf;
  }
  const uint32_t one2 = __is_same(T, bf16) ? 0x3f803f80u : 0x3c003c00u;
  const uint4v ones = {one2, one2, one2, one2};
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

  int stage = 0;
  for (int blk = wave; blk < n_blk; blk += 4, stage ^= 1) {
    const int ub = u_lo + 32 * blk;
    // this block has landed (asked for a block ago); the next one is asked for now, into the
    // buffer the previous block has left
    SPFA_WAIT_VMCNT(0);
    asm volatile("" ::: "memory");
    if (blk + 4 < n_blk) request(ub + 128, stage ^ 1);
    const char* tb = wbuf + stage * STAGE_B;
    uint4v ka[QR], va[2 * EB];
#pragma unroll
    for (int ks = 0; ks < QR; ks++) ka[ks] = *reinterpret_cast<const uint4v*>(tb + kadr[ks]);
#pragma unroll
    for (int sl = 0; sl < 2; sl++)
#pragma unroll
      for (int eb = 0; eb < EB; eb++) {
        const char* va_p = tb + 16 * sl * ROWB + vadr[eb];
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)va_p);
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(va_p + 8 * ROWB));
        const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        va[sl * EB + eb] = __builtin_bit_cast(uint4v, both);
      }
    const bool partial = ub + 32 > u_hi;
#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
      if (qb == 1 && !two) break;
      f32x16 s = zero16;
#pragma unroll
      for (int ks = 0; ks < QR; ks++) s = mfma16<T>(ka[ks], qh[qb][ks], s);
      // keys are the tokens ub .. ub+31: live for every query unless the block touches the window
      // of one of this block's query tokens, runs past the last key, or the query does not exist
      const bool hit = !q_ok[qb] || ((ub + 31 + wlim >= q_tok[qb]) && (ub <= q_tok[qb] + wlim));
      if (__builtin_expect(partial || __builtin_amdgcn_ballot_w64(hit) != 0, 0)) {
        const uint32_t d0 = (uint32_t)(ub - q_tok[qb]) + (uint32_t)wlim, w2 = 2u * (uint32_t)wlim;
        const int rem = u_hi - ub;
#pragma unroll
        for (int v = 0; v < 16; v++) {
          const int j = 8 * (v / 4) + 4 * h + (v % 4);
          const bool ok = q_ok[qb] && (d0 + (uint32_t)j > w2) && j < rem;
          s[v] = ok ? s[v] : kNegInf;
        }
      }
      float mx = mt_raw[qb];
#pragma unroll
      for (int v = 0; v < 16; v += 2) mx = fmaxf(fmaxf(mx, s[v]), s[v + 1]);
      mt_raw[qb] = mx;
      if (__builtin_expect(__builtin_amdgcn_ballot_w64(mx > thr_raw[qb]) != 0, 0)) {
        const float mp = fmaxf(mx, shfl_xor_f32(mx, 32)) * sc;
        const float m_new = (mp > m[qb] + kSlack) ? mp : m[qb];
        const float alpha = (m[qb] > kNegInf) ? __builtin_amdgcn_exp2f(m[qb] - m_new) : 0.f;
        m[qb] = m_new;
        neg_m[qb] = (m_new > kNegInf) ? -m_new : 0.f;
        thr_raw[qb] = (m_new + kSlack) * inv_sc;
        lsum[qb][0] *= alpha;
#pragma unroll
        for (int eb = 0; eb < EB; eb++)
#pragma unroll
          for (int v = 0; v < 16; v++) o[qb][eb][v] *= alpha;
      }
#pragma unroll
      for (int v = 0; v < 16; v++)
        s[v] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], sc, neg_m[qb]));  // exp2(-inf) = 0
#pragma unroll
      for (int sl = 0; sl < 2; sl++) {
        uint4v pb;
#pragma unroll
        for (int x = 0; x < 4; x++) pb[x] = pack2<T>(s[8 * sl + 2 * x], s[8 * sl + 2 * x + 1]);
#pragma unroll
        for (int eb = 0; eb < EB; eb++) o[qb][eb] = mfma16<T>(va[sl * EB + eb], pb, o[qb][eb]);
        lsum[qb] = mfma16<T>(ones, pb, lsum[qb]);
      }
    }
  }

  // ---- fold the four wavefronts (same queries, different key blocks) through LDS, 2, 3 into
  // 0, 1 and then 1 into 0, one block of queries at a time; then the partial result of this split
  SPFA_WAIT_VMCNT(0);
#pragma unroll
  for (int qb = 0; qb < 2; qb++) {
    if (qb == 1 && !two) break;
    float l = lsum[qb][0];
    float mt = fmaxf(mt_raw[qb], shfl_xor_f32(mt_raw[qb], 32)) * sc;  // true maximum, log2 units
    float mq = m[qb];
    for (int fs = 2; fs >= 1; fs >>= 1) {
      const bool gives = wave >= fs && wave < 2 * fs;
      const bool takes = wave < fs;
      float* xs = reinterpret_cast<float*>(lds) + (size_t)(gives ? wave - fs : wave) * XR * kWave + lane;
      __syncthreads();
      if (gives) {
#pragma unroll
        for (int eb = 0; eb < EB; eb++)
#pragma unroll
          for (int v = 0; v < 16; v++) xs[(eb * 16 + v) * kWave] = o[qb][eb][v];
        xs[(EB * 16) * kWave] = mq;
        xs[(EB * 16 + 1) * kWave] = l;
        xs[(EB * 16 + 2) * kWave] = mt;
      }
      __syncthreads();
      if (takes) {
        const float m2 = xs[(EB * 16) * kWave], l2 = xs[(EB * 16 + 1) * kWave];
        mt = fmaxf(mt, xs[(EB * 16 + 2) * kWave]);
        const float m_new = fmaxf(mq, m2);
        if (m_new > kNegInf) {
          const float fa = __builtin_amdgcn_exp2f(mq - m_new), fb = __builtin_amdgcn_exp2f(m2 - m_new);
          l = l * fa + l2 * fb;
#pragma unroll
          for (int eb = 0; eb < EB; eb++)
#pragma unroll
            for (int v = 0; v < 16; v++) o[qb][eb][v] = o[qb][eb][v] * fa + xs[(eb * 16 + v) * kWave] * fb;
          mq = m_new;
        }
      }
    }
    if (wave == 0 && q_ok[qb]) {
      // relative to the true maximum: (m, l, o) -> (mt, l * 2^(m - mt), o * 2^(m - mt)); an empty
      // split is (-inf, 0, 0)
      const int64_t slot = (bb * a.n_globs + (32 * qb + r)) * a.n_split + split;
      const bool any = l > 0.f;
      const float shrink = any ? __builtin_amdgcn_exp2f(mq - mt) : 0.f;
      float* prow = a.pacc + slot * D;
#pragma unroll
      for (int eb = 0; eb < EB; eb++)
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
          float4v y = {0.f, 0.f, 0.f, 0.f};
          if (any) {
#pragma unroll
            for (int i = 0; i < 4; i++) y[i] = o[qb][eb][4 * g4 + i] * shrink;
          }
          *reinterpret_cast<float4v*>(prow + 32 * eb + 8 * g4 + 4 * h) = y;
        }
      if (h == 0) {
        a.pm[slot] = any ? mt * 0.6931471805599453f : kNegInf;
        a.pl[slot] = any ? l * shrink : 0.f;
      }
    }
    __syncthreads();  // (the exchange area is used again by the second block of queries)
  }
}

// rows of a block mask that have no live column: out := NaN (m, l untouched)
template <typename T>
__global__ void band_dead_rows_kernel(T* out, int64_t n, int d, int64_t block, int64_t s) {
  // (n: rows of all problems of a batch; the block size divides the rows of one problem)
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t row = idx / d;
  if (row >= n) return;
  if (((row % block) % s) != 0) out[idx] = from_f32<T>(__builtin_nanf(""));
}

// One workgroup per distinct global row: fold the key-split partials (two passes: overall max,
// then weighted sums with the splits spread over the threads), fold the incoming state in,
// write the row.
template <typename T, int D, bool PAD = false>
__global__ __launch_bounds__(256) void global_rows_merge_kernel(TileArgs a) {
  // (PAD: rows of a.t.d < D elements, the tile kernels ran with zero-filled operands)
  const int dd = PAD ? (int)a.t.d : D;
  __shared__ float red[4];
  __shared__ float4v part[256];
  // grid: [problem][listed global]; the first n_uq of a problem's slots are its distinct rows
  const int64_t bb = blockIdx.x / a.n_globs;
  const int64_t g = blockIdx.x - bb * a.n_globs;
  if (g >= (int64_t)*a.n_uq) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t s0 = (bb * a.n_globs + g) * a.n_split;

  float mx = kNegInf;
  for (int64_t k = tid; k < a.n_split; k += 256) mx = fmaxf(mx, a.pm[s0 + k]);
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) mx = fmaxf(mx, shfl_xor_f32(mx, off));
  if (lane == 0) red[wave] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  if (mx == kNegInf) return;  // no live column at all: row untouched (same answer in every thread)

  float lsum = 0.f;
  for (int64_t k = tid; k < a.n_split; k += 256) lsum += a.pl[s0 + k] * __expf(a.pm[s0 + k] - mx);
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) lsum += shfl_xor_f32(lsum, off);
  if (lane == 0) red[wave] = lsum;
  __syncthreads();
  lsum = (red[0] + red[1]) + (red[2] + red[3]);

  // A thread sums one 16-byte piece of the row over every nsub-th partial result (rows are whole
  // 16-byte pieces; where the pieces do not divide 256 the last threads have none).
  const int c4 = dd / 4, nsub = 256 / c4;
  const int e4 = tid % c4, sub = tid / c4;
  float4v acc = {0.f, 0.f, 0.f, 0.f};
  int64_t k = sub < nsub ? sub : a.n_split;
  for (; k + 3 * nsub < a.n_split; k += 4 * nsub) {
    float4v x[4];
    float wgt[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
      x[u] = *reinterpret_cast<const float4v*>(a.pacc + (s0 + k + u * nsub) * dd + 4 * e4);
      wgt[u] = a.pm[s0 + k + u * nsub];
    }
#pragma unroll
    for (int u = 0; u < 4; u++) {
      const float wk = __expf(wgt[u] - mx);
#pragma unroll
      for (int i = 0; i < 4; i++) acc[i] += wk * x[u][i];
    }
  }
  for (; k < a.n_split; k += nsub) {
    const float wk = __expf(a.pm[s0 + k] - mx);
    const float4v x = *reinterpret_cast<const float4v*>(a.pacc + (s0 + k) * dd + 4 * e4);
#pragma unroll
    for (int i = 0; i < 4; i++) acc[i] += wk * x[i];
  }
  part[tid] = acc;
  __syncthreads();
  if (sub != 0) return;
  for (int u = 1; u < nsub; u++) {
    const float4v x = part[u * c4 + e4];
#pragma unroll
    for (int i = 0; i < 4; i++) acc[i] += x[i];
  }

  const int64_t row = a.uq[g] + bb * a.n;
  const bool sf = a.t.state_f32 != 0;
  float m_out = mx, l_out = lsum, wa = 0.f, wb = 1.f;
  const float l_in = load_state<T>(a.t.l, row, sf);
  if (l_in != 0.f) {
    const float m_in = load_state<T>(a.t.m, row, sf);
    m_out = fmaxf(mx, m_in);
    wa = l_in * __expf(m_in - m_out);
    wb = __expf(mx - m_out);
    l_out = wa + lsum * wb;
  }
  const float inv = 1.f / l_out;
  typedef T t4 __attribute__((ext_vector_type(4)));
  t4* opiece = reinterpret_cast<t4*>((T*)a.t.out + row * dd + 4 * e4);
  float x[4];
#pragma unroll
  for (int i = 0; i < 4; i++) x[i] = acc[i] * wb;
  if (wa != 0.f) {
    const t4 oi = *opiece;
#pragma unroll
    for (int i = 0; i < 4; i++) x[i] += wa * (float)oi[i];
  }
  t4 y;
#pragma unroll
  for (int i = 0; i < 4; i++) y[i] = (T)(x[i] * inv);
  *opiece = y;
  if (e4 == 0) {
    store_state<T>(a.t.m, row, m_out, sf);
    store_state<T>(a.t.l, row, l_out, sf);
  }
}

// most listed tokens band_dma_kernel takes as further keys (they are gathered one tile at a time,
// without prefetch)
constexpr int64_t kFusedMaxGlobals = 256;

// tile_kernel's launch: shapes whose tile buffers exceed 64 KB get them as dynamic LDS (the limit
// of the kernel is raised once per device)
// (tile_kernel_ready: false when the runtime refuses the limit; the callers ask before they
// launch anything and leave the call to the row-gather engine then)
template <typename T, int D, int MODE, bool PAD = false>
bool tile_kernel_ready() {
  using C = TileCfg<T, D>;
  if constexpr (C::kDynLds) {
    static std::atomic<bool> raised[kLdsLimitDevices];
    return raise_lds_limit(reinterpret_cast<const void*>(&tile_kernel<T, D, MODE, PAD>), C::LDS_BYTES, raised);
  }
  return true;
}

template <typename T, int D, int MODE, bool PAD = false>
void launch_tile_kernel(const KernelEvents& ev, dim3 grid, hipStream_t stream, const TileArgs& a) {
  using C = TileCfg<T, D>;
  if constexpr (C::kDynLds) {
    if (!tile_kernel_ready<T, D, MODE, PAD>()) return;  // (asked before; a refusal surfaces as a launch error)
    if (ev.start != nullptr && ev.stop != nullptr)
      hipExtLaunchKernelGGL((tile_kernel<T, D, MODE, PAD>), grid, dim3(256), C::LDS_BYTES, stream, ev.start, ev.stop, 0, a);
    else
      hipLaunchKernelGGL((tile_kernel<T, D, MODE, PAD>), grid, dim3(256), C::LDS_BYTES, stream, a);
  } else {
    launch_maybe_timed(ev, tile_kernel<T, D, MODE, PAD>, grid, dim3(256), stream, a);
  }
}

template <typename T, int D>
int launch_band_tiles(const TileArgs& a, int use_nan, hipStream_t stream) {
  const KernelEvents ev = kernel_events();
  if (a.n_tiles > 0) {
    const int64_t grid = (a.n_tiles * a.t.n_batch + 7) / 8 * 8;
    if constexpr (sizeof(T) == 2) {
      // the direct-to-LDS kernel addresses a tile's rows with 32-bit offsets, and tile numbers,
      // windows and positions with 32-bit arithmetic
      const int64_t max_len = a.block > 0 ? a.cnt : (a.n + a.s - 1) / a.s;
      constexpr bool kDmaShape = D == 32 || D == 64 || D == 128 || D == 256;  // (rows a power of two long)
      const bool dma = kDmaShape && a.s * (int64_t)(2 * D) * 64 < ((int64_t)1 << 31) && a.n < ((int64_t)1 << 31) &&
                       a.n_tiles * a.t.n_batch < ((int64_t)1 << 31) &&
                       (a.w <= (int64_t)0x3fffffff || max_len <= (int64_t)0x3fffffff);
      // listed global tokens as further keys: only the direct-to-LDS kernel takes them, and it
      // gathers their rows with 32-bit byte offsets
      if (a.globs != nullptr &&
          !(dma && a.n * a.t.n_batch * (int64_t)(2 * D) < ((int64_t)1 << 31) && a.n_globs <= kFusedMaxGlobals))
        return -1;
      if constexpr (kDmaShape) if (dma) {
        // the tiles of a sparsely filled last round are shared out to four workgroups each (see
        // the fp32 branch below); not with listed tokens, and not where the fold does not fit
        TileArgs at = a;
        using BC = BandDmaCfg<T, D, SPFA_BAND_BN(D)>;
        const int64_t n_all = a.n_tiles * a.t.n_batch;
        const int64_t resident = (int64_t)device_cu_count() * (D > 128 ? 1 : 2);
        const int64_t rem = n_all % resident;
        constexpr bool kFoldFits = 2 * (BC::EB * 16 + 3) * kWave * 4 <= BC::NBUF * BC::BUF_B;
        // (a problem of at most an eighth of a round: every such workgroup has a CU to itself)
        const bool few = n_all > resident ? 4 * rem <= resident : 8 * rem <= resident;
        at.n_tail = (kFoldFits && a.globs == nullptr && few) ? rem : 0;
        const int64_t grid_d = (n_all - at.n_tail + 7) / 8 * 8 + 4 * at.n_tail;
        launch_maybe_timed(ev, band_dma_kernel<T, D, SPFA_BAND_BN(D)>, dim3((unsigned)grid_d), dim3(256), stream, at);
      }
      if (!dma) {
        if (!tile_kernel_ready<T, D, kTileBand>()) return -1;
        launch_tile_kernel<T, D, kTileBand>(ev, dim3((unsigned)grid), stream, a);
      }
    } else {
      // listed global tokens as further keys: only the direct-to-LDS kernel takes them
      if (a.globs != nullptr && !((D == 64 || D == 128) && a.n_globs <= kFusedMaxGlobals)) return -1;
      // Two workgroups fit a CU, and tiles take about the same time, so the grid runs in rounds
      // of `resident` tiles and the tiles of a last, sparsely filled round keep the chip
      // waiting for a whole round (0.14 ms for a single tile left over at d = 128, window 256).
      // When four workgroups for each of those tiles still fit one round, the tiles are shared
      // out that way: such a workgroup takes two thirds of the time of a whole tile (its
      // wavefronts take turns, one key block per LDS tile), and all of them together cost about
      // twice the time per tile, hence not for fuller rounds.
      TileArgs at = a;
      const int64_t n_all = a.n_tiles * a.t.n_batch;
      const int64_t resident = (int64_t)device_cu_count() * 2;
      const int64_t rem = n_all % resident;
      // (a problem of less than a round: only while every such workgroup gets a CU to itself -
      // 64 tiles, i.e. N = 8192, took 30 / 48 us instead of 33 / 58 at d = 64 / 128, but 128 tiles
      // 44 / 201 us instead of 33 / 152 at d = 64, w = 128 / 1024)
      const bool few = n_all > resident ? 4 * rem <= resident : 8 * rem <= resident;
      at.n_tail = (few && a.globs == nullptr) ? rem : 0;
      // loads write LDS directly where a tile's rows can be addressed with 32-bit offsets and
      // positions fit 32-bit arithmetic
      const int64_t max_len = a.block > 0 ? a.cnt : (a.n + a.s - 1) / a.s;
      bool dma = false;
      if constexpr (D == 64 || D == 128)
        dma = a.s * (int64_t)(4 * D) * BandDmaF32Cfg<D>::BN < ((int64_t)1 << 31) &&
              (a.w <= (int64_t)0x3fffffff || max_len <= (int64_t)0x3fffffff);
      const int64_t n_main = n_all - at.n_tail;
      if (dma) {
        if constexpr (D == 64 || D == 128) {
          const int64_t grid_d = (n_main + 7) / 8 * 8 + 4 * at.n_tail;
          launch_maybe_timed(ev, band_dma_f32_kernel<D>, dim3((unsigned)grid_d), dim3(256), stream, at);
        }
      } else if (a.globs != nullptr) {
        return -1;
      } else {
        const int64_t grid_t = (n_main + 7) / 8 * 8 + 4 * at.n_tail;
        if (!tile_kernel_ready<T, D, kTileBand>()) return -1;
        launch_tile_kernel<T, D, kTileBand>(ev, dim3((unsigned)grid_t), stream, at);
      }
    }
  }
  if (a.block > 0 && use_nan && a.s > 1) {
    const int64_t rows = a.n * a.t.n_batch;
    const int64_t total = rows * D;
    hipLaunchKernelGGL((band_dead_rows_kernel<T>), dim3((unsigned)((total + 255) / 256)), dim3(256),
                       0, stream, (T*)a.t.out, rows, D, a.block, a.s);
  }
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

// Rows of a.t.d < D elements, D the next multiple of 32 (d = 40, 80, 100 ...): the register-staged
// kernel with its operands filled up with zeros.  One workgroup per tile; no listed tokens.
template <typename T, int D>
int launch_band_tiles_padded(const TileArgs& a, int use_nan, hipStream_t stream) {
  if (a.globs != nullptr) return -1;
  const KernelEvents ev = kernel_events();
  if (a.n_tiles > 0) {
    const int64_t grid = (a.n_tiles * a.t.n_batch + 7) / 8 * 8;
    if (!tile_kernel_ready<T, D, kTileBand, true>()) return -1;
    TileArgs at = a;
    at.n_tail = 0;
    launch_tile_kernel<T, D, kTileBand, true>(ev, dim3((unsigned)grid), stream, at);
  }
  if (a.block > 0 && use_nan && a.s > 1) {
    const int64_t rows = a.n * a.t.n_batch;
    const int64_t total = rows * a.t.d;
    hipLaunchKernelGGL((band_dead_rows_kernel<T>), dim3((unsigned)((total + 255) / 256)), dim3(256),
                       0, stream, (T*)a.t.out, rows, (int)a.t.d, a.block, a.s);
  }
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

// Global minus local: non-global rows against the listed globals, then the global rows against
// everything (key range split over workgroups), then the fold of the splits.
// rows_only: the listed tokens' own rows only (the other rows have had the listed tokens as keys
// already, inside band_dma_kernel)
template <typename T, int D>
int launch_global_tiles(const TileArgs& a, hipStream_t stream, bool rows_only) {
  const KernelEvents ev = kernel_events();
  if (!tile_kernel_ready<T, D, kTileGlobalCols>() || !tile_kernel_ready<T, D, kTileGlobalRows>()) return -1;
  int64_t grid_cols = (a.n + 127) / 128;
  TileArgs ac = a;
  ac.persist = (a.n_globs <= TileCfg<T, D>::BN) ? 1 : 0;
  if (ac.persist) {
    const int64_t resident = (int64_t)device_cu_count() * 2;  // two workgroups fit a CU
    if (grid_cols > resident) grid_cols = resident;
  }
  const unsigned nb = (unsigned)a.t.n_batch;
  if (ac.persist && nb > 1) {  // the resident workgroups are shared out over the problems
    grid_cols = grid_cols / nb;
    if (grid_cols < 1) grid_cols = 1;
  }
  if (!rows_only) {
    // all keys in one tile, half types, rows addressed with 32-bit offsets: the single-tile kernel
    bool single = false;
    if constexpr (sizeof(T) == 2 && (D == 32 || D == 64))
      single = ac.persist && a.n * (int64_t)nb * (int64_t)(2 * D) < ((int64_t)1 << 31) &&
               a.w <= (int64_t)0x3fffffff;
    if (single) {
      if constexpr (sizeof(T) == 2 && (D == 32 || D == 64))
        hipLaunchKernelGGL((global_cols_dma_kernel<T, D>), dim3((unsigned)grid_cols, nb), dim3(256), 0, stream, ac);
    } else {
      launch_tile_kernel<T, D, kTileGlobalCols>(KernelEvents{}, dim3((unsigned)grid_cols, nb), stream, ac);
    }
  }
  const int64_t q_tiles = (a.n_globs + 127) / 128;
  TileArgs ar = a;
  ar.pair_split = (a.n_globs <= 64 && TileCfg<T, D>::NB == 2) ? 1 : 0;
  // at most 64 listed tokens, half types: independent wavefronts streaming K and V
  bool streamed = false;
  if constexpr (sizeof(T) == 2 && (D == 32 || D == 64))
    streamed = a.n_globs <= 64 && a.n < ((int64_t)1 << 31) - 64 && a.w <= (int64_t)0x3fffffff;
  if (streamed) {
    if constexpr (sizeof(T) == 2 && (D == 32 || D == 64))
      launch_maybe_timed(ev, global_rows_dma_kernel<T, D>, dim3((unsigned)(a.n_split * nb)), dim3(256), stream, ar);
  } else {
    launch_tile_kernel<T, D, kTileGlobalRows>(ev, dim3((unsigned)(q_tiles * a.n_split * nb)), stream, ar);
  }
  hipLaunchKernelGGL((global_rows_merge_kernel<T, D>), dim3((unsigned)(a.n_globs * nb)), dim3(256), 0,
                     stream, a);
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

// The global mask with rows of a.t.d < D elements, D the next multiple of 32: the register-staged
// kernels with zero-filled operands; the partial results and the merge keep the real row length.
template <typename T, int D>
int launch_global_tiles_padded(const TileArgs& a, hipStream_t stream, bool rows_only) {
  const KernelEvents ev = kernel_events();
  if (!tile_kernel_ready<T, D, kTileGlobalCols, true>() || !tile_kernel_ready<T, D, kTileGlobalRows, true>()) return -1;
  int64_t grid_cols = (a.n + 127) / 128;
  TileArgs ac = a;
  ac.persist = (a.n_globs <= TileCfg<T, D>::BN) ? 1 : 0;
  const unsigned nb = (unsigned)a.t.n_batch;
  if (ac.persist) {
    const int64_t resident = (int64_t)device_cu_count() * 2;  // two workgroups fit a CU
    if (grid_cols > resident) grid_cols = resident;
    if (nb > 1) grid_cols = grid_cols / nb > 0 ? grid_cols / nb : 1;
  }
  if (!rows_only)
    launch_tile_kernel<T, D, kTileGlobalCols, true>(KernelEvents{}, dim3((unsigned)grid_cols, nb), stream, ac);
  const int64_t q_tiles = (a.n_globs + 127) / 128;
  TileArgs ar = a;
  ar.pair_split = (a.n_globs <= 64 && TileCfg<T, D>::NB == 2) ? 1 : 0;
  launch_tile_kernel<T, D, kTileGlobalRows, true>(ev, dim3((unsigned)(q_tiles * a.n_split * nb)), stream, ar);
  hipLaunchKernelGGL((global_rows_merge_kernel<T, D, true>), dim3((unsigned)(a.n_globs * nb)), dim3(256), 0,
                     stream, a);
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

// rows of whole 16-byte pieces that are no multiple of 32 elements, up to 256
template <typename T>
inline bool tile_shape_padded_ok(const Tensors& t) {
  constexpr int64_t kPiece = 16 / (int64_t)sizeof(T);
  if (!aligned16(t.q) || !aligned16(t.k) || !aligned16(t.v) || !aligned16(t.out)) return false;
  return t.d % 32 != 0 && t.d % kPiece == 0 && t.d >= kPiece && t.d <= 256;
}

inline bool tile_shape_ok(const Tensors& t, size_t elem_bytes) {
  if (!aligned16(t.q) || !aligned16(t.k) || !aligned16(t.v) || !aligned16(t.out)) return false;
  (void)elem_bytes;
  return t.d % 32 == 0 && t.d >= 32 && t.d <= 256;
}

// Returns -1 when the shape is not covered (caller falls back to the row-gather engine).
template <typename T>
int run_band_tiles(const TileArgs& a, int use_nan, hipStream_t stream) {
  if (a.t.d % 32 != 0) {
    // rows of whole 16-byte pieces: the tiles of the next multiple of 32, filled up with zeros
    if (!tile_shape_padded_ok<T>(a.t)) return -1;
    switch ((a.t.d + 31) / 32) {
      case 1: return launch_band_tiles_padded<T, 32>(a, use_nan, stream);
      case 2: return launch_band_tiles_padded<T, 64>(a, use_nan, stream);
      case 3: return launch_band_tiles_padded<T, 96>(a, use_nan, stream);
      case 4: return launch_band_tiles_padded<T, 128>(a, use_nan, stream);
      case 5: return launch_band_tiles_padded<T, 160>(a, use_nan, stream);
      case 6: return launch_band_tiles_padded<T, 192>(a, use_nan, stream);
      case 7: return launch_band_tiles_padded<T, 224>(a, use_nan, stream);
      default: return launch_band_tiles_padded<T, 256>(a, use_nan, stream);
    }
  }
  if (!tile_shape_ok(a.t, sizeof(T))) return -1;
  if (a.t.d == 64) return launch_band_tiles<T, 64>(a, use_nan, stream);
  if (a.t.d == 128) return launch_band_tiles<T, 128>(a, use_nan, stream);
  if (a.t.d == 32) return launch_band_tiles<T, 32>(a, use_nan, stream);
  if (a.t.d == 256) return launch_band_tiles<T, 256>(a, use_nan, stream);
  if (a.t.d == 96) return launch_band_tiles<T, 96>(a, use_nan, stream);
  if (a.t.d == 160) return launch_band_tiles<T, 160>(a, use_nan, stream);
  if (a.t.d == 192) return launch_band_tiles<T, 192>(a, use_nan, stream);
  if (a.t.d == 224) return launch_band_tiles<T, 224>(a, use_nan, stream);
  return -1;
}

template <typename T>
int run_global_tiles(const TileArgs& a, hipStream_t stream, bool rows_only = false) {
  if (a.t.d % 32 != 0) {
    if (!tile_shape_padded_ok<T>(a.t)) return -1;
    switch ((a.t.d + 31) / 32) {
      case 1: return launch_global_tiles_padded<T, 32>(a, stream, rows_only);
      case 2: return launch_global_tiles_padded<T, 64>(a, stream, rows_only);
      case 3: return launch_global_tiles_padded<T, 96>(a, stream, rows_only);
      case 4: return launch_global_tiles_padded<T, 128>(a, stream, rows_only);
      case 5: return launch_global_tiles_padded<T, 160>(a, stream, rows_only);
      case 6: return launch_global_tiles_padded<T, 192>(a, stream, rows_only);
      case 7: return launch_global_tiles_padded<T, 224>(a, stream, rows_only);
      default: return launch_global_tiles_padded<T, 256>(a, stream, rows_only);
    }
  }
  if (!tile_shape_ok(a.t, sizeof(T))) return -1;
  if (a.t.d == 64) return launch_global_tiles<T, 64>(a, stream, rows_only);
  if (a.t.d == 128) return launch_global_tiles<T, 128>(a, stream, rows_only);
  if (a.t.d == 32) return launch_global_tiles<T, 32>(a, stream, rows_only);
  if (a.t.d == 256) return launch_global_tiles<T, 256>(a, stream, rows_only);
  if (a.t.d == 96) return launch_global_tiles<T, 96>(a, stream, rows_only);
  if (a.t.d == 160) return launch_global_tiles<T, 160>(a, stream, rows_only);
  if (a.t.d == 192) return launch_global_tiles<T, 192>(a, stream, rows_only);
  if (a.t.d == 224) return launch_global_tiles<T, 224>(a, stream, rows_only);
  return -1;
}

}  // namespace spfa
