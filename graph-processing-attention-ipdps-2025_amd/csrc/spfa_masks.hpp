// Mask functors for the row-gather engine.  Each answers, for query row i,
//   row(i)        -> the row's candidate count (deg) plus whatever col() needs, and
//   col(rc, t, v) -> the column of candidate t (v := false if that candidate is masked).
#pragma once

#include "spfa_common.hpp"

namespace spfa {

// Explicit CSR adjacency: row i owns col_ind[row_off[i] .. row_off[i+1])
// (reference: Sparse_FlashAttention_CSR/sp_flatt_csr_kernel.cu:29-33,117).
struct CsrMask {
  static constexpr bool kWeighted = false;  // every candidate counts once
  static constexpr bool kExplicit = true;   // the mask lives in arrays that can be inconsistent
  const void* row_off;
  const uint32_t* cols;
  int32_t off64;  // row_off entries are 8 bytes wide (else 4)
  // COO only: when *use_alt != 0 the columns are read from alt_cols (the bucketed copy) instead
  const uint32_t* alt_cols;
  const uint32_t* use_alt;
  // Bounds the arrays are held to, so that inconsistent mask arrays cannot send a load outside
  // the tensors: a row's range is cut to [0, nnz) and a column >= n_cols is masked.
  int64_t nnz;
  int64_t n_cols;
  struct Row {
    int64_t start;
    int64_t deg;
    const uint32_t* cols;
  };
  __device__ __forceinline__ Row row(int64_t i) const {
    int64_t a, b;
    if (off64) {
      const uint64_t* p = (const uint64_t*)row_off;
      a = (int64_t)p[i];
      b = (int64_t)p[i + 1];
    } else {
      const uint32_t* p = (const uint32_t*)row_off;
      a = (int64_t)p[i];
      b = (int64_t)p[i + 1];
    }
    const uint32_t* cp = cols;
    if (use_alt != nullptr && *use_alt != 0u) cp = alt_cols;
    if (b > nnz) b = nnz;
    if (a < 0) a = 0;  // (an offset of 2^63 or more)
    if (a > b) a = b;
    return Row{a, b - a, cp};
  }
  __device__ __forceinline__ int64_t col(const Row& r, int64_t t, bool& valid) const {
    const int64_t c = (int64_t)r.cols[r.start + t];
    valid = c < n_cols;
    return c;
  }
  // The same in two steps, for loops that ask for a column long before they use it: testing the
  // column where it is loaded would make the loop wait for the load (and for every load issued
  // before it) on the spot.
  __device__ __forceinline__ int64_t col_unchecked(const Row& r, int64_t t) const {
    return (int64_t)r.cols[r.start + t];
  }
  __device__ __forceinline__ bool in_range(int c) const { return c >= 0 && (int64_t)c < n_cols; }
  // the row's offsets as stored, for consistency checks: 0 <= start <= end <= nnz
  __device__ __forceinline__ bool consistent(int64_t i) const {
    int64_t a, b;
    if (off64) {
      const uint64_t* p = (const uint64_t*)row_off;
      a = (int64_t)p[i];
      b = (int64_t)p[i + 1];
    } else {
      const uint32_t* p = (const uint32_t*)row_off;
      a = (int64_t)p[i];
      b = (int64_t)p[i + 1];
    }
    return a >= 0 && a <= b && b <= nnz;
  }
};

// Strided runs: candidate t of row i is low(i) + t*s.
//   block == 0: band.  low = max(i - w*s, i mod s), up = min(i + w*s, n-1), deg = (up-low)/s + 1
//               (Sparse_FlashAttention_Local_1D_Dilated/sp_flatt_local_1d_dilated_kernel.cu:25-29,102;
//               with s == 1 this is Sparse_FlashAttention_Local/sp_flatt_local_kernel.cu:24-28,101).
//   block  > 0: block-diagonal with 2-D dilation.  low = (i / block) * block; the row is live
//               only when (i - low) mod s == 0, then deg = cnt = min(block, (block-1)/s + 1)
//               (Sparse_FlashAttention_Local_2D_Dilated/sp_flatt_local_2d_dilated_kernel.cu:26-39,123).
struct StrideMask {
  static constexpr bool kWeighted = false;
  static constexpr bool kExplicit = false;
  int64_t n;
  int64_t w;
  int64_t s;
  int64_t block;
  int64_t cnt;
  struct Row {
    int64_t low;
    int64_t deg;
  };
  __device__ __forceinline__ Row row(int64_t i) const {
    if (block > 0) {
      int64_t low = (i / block) * block;
      return Row{low, ((i - low) % s == 0) ? cnt : 0};
    }
    int64_t low = i - w * s;
    int64_t r = i % s;
    if (low < r) low = r;
    int64_t up = i + w * s;
    if (up > n - 1) up = n - 1;
    return Row{low, (up - low) / s + 1};
  }
  __device__ __forceinline__ int64_t col(const Row& r, int64_t t, bool&) const {
    return r.low + t * s;
  }
};

// Global minus local window [low, up) = [max(0, i-w), min(n, i+w+1)):
//   global row: candidates are all n - (up-low) columns outside the window;
//   other rows: candidates are the n_globs listed indices, those inside the window are masked
//   (Sparse_FlashAttention_Global_No_Local/sp_flatt_global_no_local_kernel.cu:38-64,134-162).
// Bit i of gbits marks the listed rows.
struct GlobalMask {
  static constexpr bool kWeighted = false;
  static constexpr bool kExplicit = false;
  int64_t n;
  int64_t w;
  const int32_t* globs;
  int64_t n_globs;
  const uint32_t* gbits;
  struct Row {
    int64_t low;
    int64_t up;
    int64_t deg;
    bool glob;
  };
  __device__ __forceinline__ Row row(int64_t i) const {
    int64_t low = i - w;
    if (low < 0) low = 0;
    int64_t up = i + w + 1;
    if (up > n) up = n;
    bool glob = bit_is_set(gbits, i);
    return Row{low, up, glob ? n - (up - low) : n_globs, glob};
  }
  __device__ __forceinline__ int64_t col(const Row& r, int64_t t, bool& valid) const {
    if (r.glob) return t < r.low ? t : t + (r.up - r.low);
    int64_t c = (int64_t)globs[t];
    valid = c >= 0 && c < n && ((c < r.low) || (c >= r.up));  // (an out-of-range entry is masked)
    return c;
  }
};

// The global-minus-local mask read by COLUMN (the gradient's key-side pass): which query rows
// attend column j, and how often.  The window test is symmetric, so
//   listed column j:  every row outside the window; a listed row attends j once, any other row
//                     once per occurrence of j in the list (it walks the list, duplicates and all);
//   other columns:    the distinct listed rows outside the window, once each.
struct GlobalColMask {
  static constexpr bool kWeighted = true;
  static constexpr bool kExplicit = false;
  int64_t n;
  int64_t w;
  const int32_t* globs;   // the list as given (duplicates allowed)
  int64_t n_globs;
  const uint32_t* gbits;
  const int32_t* uq;      // distinct listed rows
  const uint32_t* n_uq;   // how many
  struct Row {
    int64_t low;
    int64_t up;
    int64_t deg;
    bool glob;
    float mult;  // occurrences of this column in the list
  };
  __device__ __forceinline__ Row row(int64_t j) const {
    int64_t low = j - w;
    if (low < 0) low = 0;
    int64_t up = j + w + 1;
    if (up > n) up = n;
    const bool glob = bit_is_set(gbits, j);
    float mult = 1.f;
    if (glob) {
      int cnt = 0;
      for (int64_t t = 0; t < n_globs; t++) cnt += (globs[t] == (int32_t)j) ? 1 : 0;
      mult = (float)cnt;
    }
    return Row{low, up, glob ? n - (up - low) : (int64_t)*n_uq, glob, mult};
  }
  __device__ __forceinline__ int64_t col(const Row& r, int64_t t, bool& valid) const {
    if (r.glob) return t < r.low ? t : t + (r.up - r.low);
    int64_t c = (int64_t)uq[t];
    valid = (c < r.low) || (c >= r.up);
    return c;
  }
  __device__ __forceinline__ float weight(const Row& r, int64_t c) const {
    return (r.glob && !bit_is_set(gbits, c)) ? r.mult : 1.f;
  }
};

}  // namespace spfa
