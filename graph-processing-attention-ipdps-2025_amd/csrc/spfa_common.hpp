// Shared device helpers for the gfx950 sparse-attention kernels: element conversions,
// wave64 lane layouts and cross-lane reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace spfa {

constexpr int kWave = 64;
constexpr float kNegInf = -__builtin_inff();

using f16 = _Float16;
using bf16 = __bf16;

typedef float float4v __attribute__((ext_vector_type(4)));
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef __bf16 bhalf8v __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef __bf16 bhalf2v __attribute__((ext_vector_type(2)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

template <typename T>
__device__ __forceinline__ float to_f32(T x) { return (float)x; }
template <typename T>
__device__ __forceinline__ T from_f32(float x) { return (T)x; }

// m and l may be stored in the element type (reference behaviour) or in fp32.
template <typename T>
__device__ __forceinline__ float load_state(const void* p, int64_t i, bool state_f32) {
  return state_f32 ? ((const float*)p)[i] : to_f32(((const T*)p)[i]);
}
// The same load in two parts, for a value that is asked for long before it is needed: the raw
// bits stay in a register and are only turned into a float where the value is used (a load that
// is converted at once is waited for at once).
template <typename T>
__device__ __forceinline__ uint32_t load_state_raw(const void* p, int64_t i, bool state_f32) {
  uint32_t raw;
  if (state_f32) raw = ((const uint32_t*)p)[i];
  else raw = ((const uint16_t*)p)[i];
  return raw;
}
template <typename T>
__device__ __forceinline__ float state_from_raw(uint32_t raw, bool state_f32) {
  static_assert(sizeof(T) == 2, "two-byte state types");
  const uint16_t lo = (uint16_t)raw;
  return state_f32 ? __builtin_bit_cast(float, raw) : to_f32(__builtin_bit_cast(T, lo));
}
template <typename T>
__device__ __forceinline__ void store_state(void* p, int64_t i, float x, bool state_f32) {
  if (state_f32) ((float*)p)[i] = x;
  else ((T*)p)[i] = from_f32<T>(x);
}

// ---------------------------------------------------------------------------------------
// cross-lane moves
// ---------------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float x) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}

__device__ __forceinline__ float shfl_xor_f32(float x, int mask) {
  int lane = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
  return __builtin_bit_cast(
      float, __builtin_amdgcn_ds_bpermute((lane ^ mask) << 2, __builtin_bit_cast(int, x)));
}
__device__ __forceinline__ int shfl_i32(int x, int src_lane) {
  return __builtin_amdgcn_ds_bpermute(src_lane << 2, x);
}
__device__ __forceinline__ float shfl_f32(float x, int src_lane) {
  return __builtin_bit_cast(float,
                            __builtin_amdgcn_ds_bpermute(src_lane << 2, __builtin_bit_cast(int, x)));
}

// Sum over aligned groups of LPR consecutive lanes; every lane of the group gets the total.
// 4 lanes: two quad permutes; 8: half-row mirror; 16: row mirror (all DPP, no LDS traffic);
// 32: ds_swizzle xor 16; 64: bpermute xor 32.
template <int LPR>
__device__ __forceinline__ float group_sum(float x) {
  static_assert(LPR == 1 || LPR == 2 || LPR == 4 || LPR == 8 || LPR == 16 || LPR == 32 || LPR == 64,
                "lanes per row must be a power of two");
  if constexpr (LPR >= 2) x += dpp_f32<0xB1>(x);   // quad_perm [1,0,3,2]
  if constexpr (LPR >= 4) x += dpp_f32<0x4E>(x);   // quad_perm [2,3,0,1]
  if constexpr (LPR >= 8) x += dpp_f32<0x141>(x);  // row_half_mirror
  if constexpr (LPR >= 16) x += dpp_f32<0x140>(x); // row_mirror
  if constexpr (LPR >= 32)
    x += __builtin_bit_cast(float,
                            __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, x), 0x401F));
  if constexpr (LPR >= 64) x += shfl_xor_f32(x, 32);
  return x;
}

// ---------------------------------------------------------------------------------------
// lane layouts: how the d elements of one K/V/Q/O row are spread over lanes
// ---------------------------------------------------------------------------------------
// VecLay: d * sizeof(T) == LPR * 16 bytes.  Lane c of a group owns 16 contiguous bytes of the
// row, so one wave-wide load instruction fetches 64/LPR whole rows with full 16-byte lanes.
// PAD: rows of any multiple of 16 bytes up to LPR * 16 - the lanes past the end of a row hold
// zeros and neither load nor store (a row of 96 floats takes 24 of a group's 32 lanes).
template <typename T, int LPR_, bool PAD_ = false>
struct VecLay {
  using elem = T;
  static constexpr int LPR = LPR_;
  static constexpr bool PAD = PAD_;
  static constexpr int GROUPS = kWave / LPR;
  static constexpr int NE = 16 / (int)sizeof(T);  // floats held per lane
  static constexpr int D = LPR * NE;
  static constexpr int U = 16;       // neighbours in flight per group in the segment kernel
  static constexpr int U_SHORT = 4;  // ... in the row kernel
  static constexpr int U_MEDIUM = 8; // ... in the medium-row kernel
  using raw = uint4v;
  // which element of the row lane c holds in slot e (may lie past the end of a padded row)
  __device__ static __forceinline__ int elem_index(int c, int e) { return c * NE + e; }

  __device__ static __forceinline__ raw load(const T* row_ptr, int c, int d) {
    if constexpr (PAD) {
      if (c * NE >= d) return raw{0u, 0u, 0u, 0u};
    }
    return *reinterpret_cast<const raw*>(reinterpret_cast<const char*>(row_ptr) + c * 16);
  }
  // gathered K / V rows
  __device__ static __forceinline__ raw load_gather(const T* row_ptr, int c, int d) {
    return load(row_ptr, c, d);
  }
  __device__ static __forceinline__ void unpack(const raw& r, float (&f)[NE]) {
    if constexpr (sizeof(T) == 4) {
      float4v x = __builtin_bit_cast(float4v, r);
#pragma unroll
      for (int e = 0; e < 4; e++) f[e] = x[e];
    } else if constexpr (__is_same(T, f16)) {
      half8v x = __builtin_bit_cast(half8v, r);
#pragma unroll
      for (int e = 0; e < 8; e++) f[e] = (float)x[e];
    } else {
      // bf16 -> f32 is a 16-bit left shift
#pragma unroll
      for (int e = 0; e < 4; e++) {
        f[2 * e] = __builtin_bit_cast(float, r[e] << 16);
        f[2 * e + 1] = __builtin_bit_cast(float, r[e] & 0xffff0000u);
      }
    }
  }
  // The dot product of a gathered piece with the owner's piece.  For the two-byte types the
  // owner's floats came out of that type, so they pack again exactly and two products at a time
  // go through the dot instructions (fp32 sums of exact products): 4 instructions a piece where
  // unpacking and multiplying takes 16.
  static constexpr bool kPackedDot = sizeof(T) == 2;
  __device__ static __forceinline__ raw pack_exact(const float (&f)[NE]) {
    raw r{0u, 0u, 0u, 0u};
    if constexpr (__is_same(T, f16)) {
      half8v x;
#pragma unroll
      for (int e = 0; e < 8; e++) x[e] = (f16)f[e];
      r = __builtin_bit_cast(raw, x);
    } else if constexpr (sizeof(T) == 2) {
#pragma unroll
      for (int e = 0; e < 4; e++)
        r[e] = (__builtin_bit_cast(uint32_t, f[2 * e]) >> 16) |
               (__builtin_bit_cast(uint32_t, f[2 * e + 1]) & 0xffff0000u);
    }
    return r;
  }
  __device__ static __forceinline__ float packed_dot(const raw& x, const raw& y) {
    float acc = 0.f;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      // (copies first: a bit cast applied to an element of a vector reads the vector's first
      // element whichever one is named)
      const uint32_t xe = x[e], ye = y[e];
      if constexpr (__is_same(T, f16))
        acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, xe), __builtin_bit_cast(half2v, ye), acc, false);
      else if constexpr (sizeof(T) == 2)
        acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bhalf2v, xe), __builtin_bit_cast(bhalf2v, ye), acc,
                                              false);
    }
    return acc;
  }
  __device__ static __forceinline__ void store(T* row_ptr, int c, int d, const float (&f)[NE]) {
    if constexpr (PAD) {
      if (c * NE >= d) return;
    }
    raw r;
    if constexpr (sizeof(T) == 4) {
      float4v x;
#pragma unroll
      for (int e = 0; e < 4; e++) x[e] = f[e];
      r = __builtin_bit_cast(raw, x);
    } else if constexpr (__is_same(T, f16)) {
      half8v x;
#pragma unroll
      for (int e = 0; e < 8; e++) x[e] = (f16)f[e];
      r = __builtin_bit_cast(raw, x);
    } else {
      bhalf8v x;
#pragma unroll
      for (int e = 0; e < 8; e++) x[e] = (bf16)f[e];
      r = __builtin_bit_cast(raw, x);
    }
    *reinterpret_cast<raw*>(reinterpret_cast<char*>(row_ptr) + c * 16) = r;
  }
  // fp32 partial rows in the workspace: element e of lane c is at c*NE + e
  __device__ static __forceinline__ void load_f32(const float* row_ptr, int c, int d, float (&f)[NE]) {
    if constexpr (PAD) {
      if (c * NE >= d) {
#pragma unroll
        for (int e = 0; e < NE; e++) f[e] = 0.f;
        return;
      }
    }
#pragma unroll
    for (int e = 0; e < NE; e += 4) {
      float4v x = *reinterpret_cast<const float4v*>(row_ptr + c * NE + e);
      f[e] = x[0]; f[e + 1] = x[1]; f[e + 2] = x[2]; f[e + 3] = x[3];
    }
  }
  __device__ static __forceinline__ void store_f32(float* row_ptr, int c, int d, const float (&f)[NE]) {
    if constexpr (PAD) {
      if (c * NE >= d) return;
    }
#pragma unroll
    for (int e = 0; e < NE; e += 4) {
      float4v x = {f[e], f[e + 1], f[e + 2], f[e + 3]};
      *reinterpret_cast<float4v*>(row_ptr + c * NE + e) = x;
    }
  }
};

// WideLay: rows of more than 512 bytes, up to NCH * 512 (a multiple of 16).  Half a wavefront per
// row; lane c owns the 16-byte chunks c, c + 32, ... of it (NCH load instructions per row, each
// 512 contiguous bytes), lanes past the end of a row hold zeros.
template <typename T, int NCH_>
struct WideLay {
  using elem = T;
  static constexpr int LPR = 32;
  static constexpr int NCH = NCH_;
  static constexpr bool PAD = true;
  static constexpr int GROUPS = kWave / LPR;
  static constexpr int NC = 16 / (int)sizeof(T);  // elements per chunk
  static constexpr int NE = NCH * NC;             // floats held per lane
  static constexpr int U = 16 / NCH;  // (the bytes in flight per lane of VecLay)
  static constexpr int U_SHORT = U >= 4 ? U / 4 : 1;
  static constexpr int U_MEDIUM = U >= 2 ? U / 2 : 1;
  static constexpr bool kPackedDot = false;
  static_assert(NCH == 2 || NCH == 4 || NCH == 8, "two to eight chunks per lane");
  struct raw { uint4v x[NCH]; };
  __device__ static __forceinline__ int elem_index(int c, int e) { return (c + 32 * (e / NC)) * NC + e % NC; }

  __device__ static __forceinline__ raw load(const T* row_ptr, int c, int d) {
    raw r;
#pragma unroll
    for (int j = 0; j < NCH; j++) {
      const int ch = c + 32 * j;
      r.x[j] = uint4v{0u, 0u, 0u, 0u};
      if (ch * NC < d) r.x[j] = *reinterpret_cast<const uint4v*>(reinterpret_cast<const char*>(row_ptr) + ch * 16);
    }
    return r;
  }
  __device__ static __forceinline__ raw load_gather(const T* row_ptr, int c, int d) { return load(row_ptr, c, d); }
  __device__ static __forceinline__ void unpack(const raw& r, float (&f)[NE]) {
#pragma unroll
    for (int j = 0; j < NCH; j++) {
      float g[NC];
      VecLay<T, 32>::unpack(r.x[j], g);
#pragma unroll
      for (int e = 0; e < NC; e++) f[j * NC + e] = g[e];
    }
  }
  __device__ static __forceinline__ void store(T* row_ptr, int c, int d, const float (&f)[NE]) {
#pragma unroll
    for (int j = 0; j < NCH; j++) {
      float g[NC];
#pragma unroll
      for (int e = 0; e < NC; e++) g[e] = f[j * NC + e];
      VecLay<T, 64, true>::store(row_ptr, c + 32 * j, d, g);
    }
  }
  // fp32 partial rows in the workspace: the row's own element order
  __device__ static __forceinline__ void load_f32(const float* row_ptr, int c, int d, float (&f)[NE]) {
#pragma unroll
    for (int j = 0; j < NCH; j++)
#pragma unroll
      for (int e = 0; e < NC; e += 4) {
        const int idx = (c + 32 * j) * NC + e;
        float4v x = {0.f, 0.f, 0.f, 0.f};
        if (idx < d) x = *reinterpret_cast<const float4v*>(row_ptr + idx);
        f[j * NC + e] = x[0]; f[j * NC + e + 1] = x[1]; f[j * NC + e + 2] = x[2]; f[j * NC + e + 3] = x[3];
      }
  }
  __device__ static __forceinline__ void store_f32(float* row_ptr, int c, int d, const float (&f)[NE]) {
#pragma unroll
    for (int j = 0; j < NCH; j++)
#pragma unroll
      for (int e = 0; e < NC; e += 4) {
        const int idx = (c + 32 * j) * NC + e;
        float4v x = {f[j * NC + e], f[j * NC + e + 1], f[j * NC + e + 2], f[j * NC + e + 3]};
        if (idx < d) *reinterpret_cast<float4v*>(row_ptr + idx) = x;
      }
  }
};

// GenLay: any d <= 64*EPL.  One row per wave-wide load; lane c owns elements c, c+64, ...
// Slower (scalar loads) but complete: the fallback for sizes VecLay does not cover.
template <typename T, int EPL>
struct GenLay {
  using elem = T;
  static constexpr int LPR = kWave;
  static constexpr int GROUPS = 1;
  static constexpr int NE = EPL;
  static constexpr int U = (EPL <= 2) ? 8 : 2;
  static constexpr int U_SHORT = U;
  static constexpr int U_MEDIUM = U;
  static constexpr bool kPackedDot = false;
  struct raw { T x[EPL]; };
  __device__ static __forceinline__ int elem_index(int c, int e) { return c + e * kWave; }

  __device__ static __forceinline__ raw load(const T* row_ptr, int c, int d) {
    raw r;
#pragma unroll
    for (int e = 0; e < EPL; e++) {
      int idx = c + e * kWave;
      r.x[e] = idx < d ? row_ptr[idx] : from_f32<T>(0.f);
    }
    return r;
  }
  __device__ static __forceinline__ raw load_gather(const T* row_ptr, int c, int d) {
    return load(row_ptr, c, d);
  }
  __device__ static __forceinline__ void unpack(const raw& r, float (&f)[NE]) {
#pragma unroll
    for (int e = 0; e < EPL; e++) f[e] = to_f32(r.x[e]);
  }
  __device__ static __forceinline__ void store(T* row_ptr, int c, int d, const float (&f)[NE]) {
#pragma unroll
    for (int e = 0; e < EPL; e++) {
      int idx = c + e * kWave;
      if (idx < d) row_ptr[idx] = from_f32<T>(f[e]);
    }
  }
  __device__ static __forceinline__ void load_f32(const float* row_ptr, int c, int d, float (&f)[NE]) {
#pragma unroll
    for (int e = 0; e < EPL; e++) {
      int idx = c + e * kWave;
      f[e] = idx < d ? row_ptr[idx] : 0.f;
    }
  }
  __device__ static __forceinline__ void store_f32(float* row_ptr, int c, int d, const float (&f)[NE]) {
#pragma unroll
    for (int e = 0; e < EPL; e++) {
      int idx = c + e * kWave;
      if (idx < d) row_ptr[idx] = f[e];
    }
  }
};

__device__ __forceinline__ bool bit_is_set(const uint32_t* bits, int64_t i) {
  return (bits[i >> 5] >> (i & 31)) & 1u;
}

// A listed (global) token as the kernels use it: itself when it names a row of the problem, else
// -1 (such an entry is masked for every query and never used as an address).
__device__ __forceinline__ int listed_token(int g, int64_t n) {
  return ((int64_t)g >= 0 && (int64_t)g < n) ? g : -1;
}

__device__ __forceinline__ int lane_id() {
  return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

}  // namespace spfa
