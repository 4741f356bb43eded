// Host entry points of the mask pre-passes (spfa_prep.hip).
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace spfa {

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

struct CooWorkspace {
  // what the attention kernels read afterwards: offsets, bucketed columns, the "unsorted" flag
  size_t off_row_off, off_cols, off_flag, keep_total;
  // scratch of the conversion itself (follows the part above)
  size_t off_counts, off_cursor, off_tiles;
  // two-pass partition (used when the row index fits 22 bits)
  size_t off_hist, off_tmp_pairs, total;
  int partition;       // 1: two-pass LDS partition, 0: per-entry global atomics
  int lo_bits;         // low digit width; high digit = row >> lo_bits
  int64_t n_hi;        // high-digit buckets
  int64_t n_tiles1;    // entry tiles of pass 1
};

CooWorkspace coo_workspace(int64_t n_rows, int64_t nnz);

struct CooCsr {
  const uint32_t* row_off;    // n_rows + 1 offsets (32-bit)
  const uint32_t* cols;       // bucketed columns, valid when *unsorted != 0
  const uint32_t* unsorted;   // device flag: 0 = the entries came sorted by row, use the
                              // caller's column array as it is
};

// Turns COO entries into 32-bit CSR offsets (coo_workspace() sizes the two buffers).
// Entries that already come sorted by row (the reference's contract) only need the offsets;
// otherwise they are bucketed by row and the columns copied, in no particular order inside a
// row: a two-pass partition with LDS-private histograms (high digit of the row, then low digit
// inside each high bucket) when the row index fits 22 bits, per-entry global atomics otherwise.  The choice is made on the device (no host synchronisation):
// both sets of kernels are enqueued and the ones that are not needed return at once.
// Entries with a row outside [0, n_rows) are dropped (and force the bucketing path).
// `keep` receives the result (keep_total bytes), `scratch` is total - keep_total bytes.
// n_cols: columns >= n_cols mean nothing to the caller (they may come back as n_cols); 0 when the
// columns must come back exactly as given.
int coo_to_csr(const void* row_ind, int row_wide, const uint32_t* col_ind, int64_t nnz,
               int64_t n_rows, int64_t n_cols, void* keep, void* scratch, hipStream_t stream, CooCsr* out);

// The entry list of a CSR mask: rows[e], cols[e] for every entry e of row_off / col_ind (cols
// from alt_cols when *use_alt != 0, as CsrMask reads them).  Feeding (cols, rows) back into
// coo_to_csr gives the transposed mask.
int csr_entry_list(const void* row_off, int off64, const uint32_t* cols, const uint32_t* alt_cols,
                   const uint32_t* use_alt, int64_t n_rows, int64_t nnz, uint32_t* rows_out,
                   uint32_t* cols_out, hipStream_t stream);

// A CooCsr result as two plain arrays: row_off_out[0..n_rows] and cols_out[0..nnz) (the bucketed
// columns, or `given_cols` unchanged when the entries came sorted).
int coo_csr_export(const CooCsr& csr, const uint32_t* given_cols, int64_t n_rows, int64_t nnz,
                   uint32_t* row_off_out, uint32_t* cols_out, hipStream_t stream);

// Global-row bookkeeping for the global-minus-local mask.  `bits` holds (n+31)/32 bitmap words
// followed by one counter word; afterwards bit i is set for every listed i in [0, n), `uq` holds
// the distinct listed rows (any order) and the counter word their number.
inline size_t global_bits_words(int64_t n) { return (size_t)((n + 31) / 32) + 1; }
int prepare_global_rows(const int32_t* globs, int64_t n_globs, int64_t n, uint32_t* bits,
                        int32_t* uq, hipStream_t stream);

}  // namespace spfa
