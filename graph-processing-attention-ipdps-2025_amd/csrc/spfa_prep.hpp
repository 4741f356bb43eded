// Host entry points of the mask pre-passes (spfa_prep.hip).
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace spfa {

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

struct CooWorkspace {
  size_t off_counts, off_row_off, off_cursor, off_tiles, off_cols, total;
};

CooWorkspace coo_workspace(int64_t n_rows, int64_t nnz);

// Buckets COO entries by row into 32-bit CSR arrays placed in `ws` (coo_workspace().total bytes).
// Entries with a row outside [0, n_rows) are dropped.  Columns keep no particular order inside
// a row.
int coo_bucket_by_row(const void* row_ind, int row_wide, const uint32_t* col_ind, int64_t nnz,
                      int64_t n_rows, void* ws, hipStream_t stream, const uint32_t** row_off_out,
                      const uint32_t** cols_out);

// flags[i] = 1 for every listed i in [0, n), 0 elsewhere.  flags holds (n+3)/4*4 bytes.
int mark_global_rows(const int32_t* globs, int64_t n_globs, int64_t n, uint8_t* flags,
                     hipStream_t stream);

}  // namespace spfa
