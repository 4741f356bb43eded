/*
 * spfa_hip.h - C ABI of libspfa_hip.so: masked single-head attention on gfx950 (MI355X)
 * that does work only on un-masked positions.
 *
 * One entry point per mask kind.  Each replaces the host dispatcher + device kernel pair of
 * one reference extension (paths relative to the reference tree):
 *
 *   spfa_csr_forward               Sparse_FlashAttention_CSR/sp_flatt_csr_kernel.cu:14-288
 *   spfa_coo_forward               Sparse_FlashAttention_COO/sp_flatt_coo_kernel.cu:14-327
 *   spfa_local_forward             Sparse_FlashAttention_Local/sp_flatt_local_kernel.cu:12-272
 *   spfa_local_1d_dilated_forward  Sparse_FlashAttention_Local_1D_Dilated/sp_flatt_local_1d_dilated_kernel.cu:12-280
 *   spfa_local_2d_dilated_forward  Sparse_FlashAttention_Local_2D_Dilated/sp_flatt_local_2d_dilated_kernel.cu:12-306
 *   spfa_global_no_local_forward   Sparse_FlashAttention_Global_No_Local/sp_flatt_global_no_local_kernel.cu:12-353
 *
 * Contract shared by all entry points
 *   - Every pointer is a device pointer on the current device; q, k, v, out are row-major
 *     contiguous [n, d]; m and l are [n].  Nothing is allocated, retained or synchronised by
 *     the library: work is enqueued on `stream` (a hipStream_t passed as void*, NULL = the
 *     default stream) and the call returns.
 *   - (m, l, out) is in/out state exactly as in the reference (sp_flatt_csr_kernel.cu:79-92,
 *     162-201, 208-218): out is kept normalised, m is the running maximum score, l the running
 *     sum of exp(score - m).  A fresh state is m = -inf, l = 0, out = anything (an incoming
 *     row with l == 0 carries no weight and its out row is not read).  Masks handed to
 *     successive calls on one state must be disjoint.
 *   - A row without any live column: out row := NaN when use_nan != 0 (CSR, COO, 2D-dilated),
 *     otherwise untouched; m and l of such a row are never touched
 *     (sp_flatt_csr_kernel.cu:45-54).
 *   - Scores are q.k / sqrt(d) (sp_flatt_csr_kernel.cu:137).  Accumulation is fp32 for every
 *     element type.
 *   - `workspace` is scratch device memory of at least *_workspace_bytes(...) bytes, 256-byte
 *     aligned, owned by the caller, and may be reused by the next call on the same stream.
 *   - Return value: SPFA_OK or one of the codes below; spfa_status_string() gives the text
 *     (for the parameter checks it is the text of the reference's std::invalid_argument).
 *     Parameter checks run in the reference's order before anything is enqueued.
 */
#ifndef SPFA_HIP_H
#define SPFA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element type of q, k, v, out */
/* F64 (the reference dispatches double too, sp_flatt_csr_kernel.cu:270) runs a plain kernel
 * with double arithmetic, for parity rather than speed; m and l must then be F64 as well. */
enum { SPFA_DTYPE_F32 = 0, SPFA_DTYPE_F16 = 1, SPFA_DTYPE_BF16 = 2, SPFA_DTYPE_F64 = 3 };

enum {
  SPFA_OK = 0,
  SPFA_ERR_BAD_ARG = 1,       /* null pointer, negative size, bad enum, index width not 4/8 */
  SPFA_ERR_UNSUPPORTED = 2,   /* element type / size combination not built */
  SPFA_ERR_WORKSPACE = 3,     /* workspace missing, misaligned or too small */
  SPFA_ERR_LAUNCH = 4,        /* the HIP runtime refused a launch (hipGetLastError) */
  SPFA_ERR_EMB_TOO_LARGE = 5, /* sp_flatt_csr_kernel.cu:264-266; here: d > 1024 or d < 1 */
  SPFA_ERR_LOCAL_SIZE = 6,    /* sp_flatt_local_kernel.cu:252-254 */
  SPFA_ERR_DILATION_NEG = 7,  /* sp_flatt_local_1d_dilated_kernel.cu:259-261 */
  SPFA_ERR_BLOCK_DIVISOR = 8, /* sp_flatt_local_2d_dilated_kernel.cu:274-276 */
  SPFA_ERR_BLOCK_DILATION = 9,/* sp_flatt_local_2d_dilated_kernel.cu:284-286 */
  SPFA_ERR_GLOBAL_COUNT = 10, /* sp_flatt_global_no_local_kernel.cu:325-327 */
  SPFA_ERR_STATIC_LIMIT = 11  /* spfa_csr_forward_static: the mask needs more scratch than
                                 SPFA_STATIC_SCRATCH_BYTES */
};

typedef struct spfa_problem {
  const void* q;       /* [n_q, d] */
  const void* k;       /* [n_k, d] */
  const void* v;       /* [n_k, d] */
  void* m;             /* [n_q] running max, in/out */
  void* l;             /* [n_q] running sum, in/out */
  void* out;           /* [n_q, d] normalised output, in/out */
  int64_t n_q;
  int64_t n_k;         /* implicit masks use n_q for both, as the reference does */
  int64_t d;           /* 1 <= d <= 1024 */
  int32_t dtype;       /* SPFA_DTYPE_* of q, k, v, out */
  int32_t state_dtype; /* SPFA_DTYPE_* of m, l: the same as dtype (reference), or F32 */
  /* Independent problems that share the mask (batch x heads; the reference is limited to one,
   * README.md:10).  0 or 1: a single problem.  With n_batch > 1 the tensors are stacked:
   * q, out [n_batch, n_q, d], k, v [n_batch, n_k, d], m, l [n_batch, n_q], all contiguous; the
   * workspace must hold n_batch times the bytes *_workspace_bytes(...) reports. */
  int64_t n_batch;
} spfa_problem_t;

int spfa_version(void);
const char* spfa_status_string(int status);

/* What the kernels found wrong with mask arrays they can only look at on the device.  The
 * reference checks nothing there (sp_flatt_csr_kernel.cu:271-287 launches on whatever row_off and
 * col_ind hold, and reads out of bounds when they disagree).  Here the explicit-mask kernels hold
 * the arrays to the sizes the call states - a row's range is cut to [0, nnz), a column >= n_k is
 * masked, COO entries with a row >= n_q are dropped, listed global tokens outside [0, n) are
 * masked - so inconsistent arrays cannot send a load outside the tensors; rows hit by an
 * inconsistency are computed on what is left of them or left untouched, and the call still
 * returns SPFA_OK because the host never sees device data.  Each device keeps a sticky word that
 * the CSR / COO kernels OR these bits into (only calls with nnz > 32 look):
 *   SPFA_STATUS_WORK_LIST_OVERFLOW  the row offsets describe more long-row entries than the nnz
 *                                   passed; every long row of that call was left untouched
 *   SPFA_STATUS_ROW_OFFSETS         some row's offsets decrease or end beyond nnz
 * spfa_device_status returns the current device's word (>= 0; reset != 0 clears it), or -1 when it
 * cannot be read.  It copies from the device: synchronise the streams of the calls in question
 * first. */
enum { SPFA_STATUS_WORK_LIST_OVERFLOW = 1, SPFA_STATUS_ROW_OFFSETS = 2 };
int spfa_device_status(int reset);

/* Measurement aid; no counterpart in the reference.  While both handles are non-NULL
 * (hipEvent_t passed as void*), every forward call MADE BY THE CALLING HOST THREAD attaches
 * `start` and `stop` to the dispatch of the kernel that does the bulk of the call's attention
 * work (the segment kernel when a mask has long rows, else the row kernel; the band kernel; the
 * global rows' tile kernel), so a benchmark can time that one kernel with hipEventElapsedTime.
 * The pair is kept per host thread (other threads' calls are not affected and do not race on
 * it): set it, run, read the events, reset it with NULLs. */
void spfa_set_kernel_events(void* start, void* stop);

/* Rows of an explicit mask with at most this many entries are finished by the row kernels (a
 * lane group or a wavefront per row); longer rows go through the segment kernel.  Exposed so a
 * benchmark can attribute bytes to kernels. */
int64_t spfa_explicit_inline_row_limit(void);

/* 1 when a CSR / COO call with n_k keys of d elements of `dtype` walks the segments of its long
 * rows with an ordinary grid (items_grid_kernel) instead of the persistent segments_kernel: K and V
 * of one problem small enough to stay in the caches (48 MiB; 96 MiB for rows of at most 128 bytes).  Exposed so a benchmark can name the kernel
 * it times. */
int spfa_explicit_long_rows_on_grid(int64_t n_k, int64_t d, int dtype);

/* Such a call of at most this many rows (over all problems) runs its three row kernels - long
 * rows' items, medium rows, short rows - as one launch, so no single kernel of it can be timed. */
int64_t spfa_explicit_one_launch_row_limit(void);

/* CSR: row i attends col_ind[row_off[i] .. row_off[i+1]).  row_off has n_q+1 entries of
 * row_off_bytes (4 or 8) bytes each, col_ind has nnz 4-byte entries; signed and unsigned
 * index tensors are bit-identical in range.  The reference's value vector is never read
 * (sp_flatt_csr_kernel.cu:21) and is not part of this interface. */
size_t spfa_csr_workspace_bytes(int64_t n_q, int64_t nnz, int64_t d, int dtype);
/* ... of a call with p->n_batch == n_batch: the exact size (the work list is shared by the
 * problems of a batch, only the partial results are per problem); n_batch times the
 * single-problem size is always enough too. */
size_t spfa_csr_workspace_bytes_batched(int64_t n_q, int64_t nnz, int64_t d, int dtype, int64_t n_batch);
int spfa_csr_forward(const spfa_problem_t* p, const void* row_off, int row_off_bytes,
                     const void* col_ind, int64_t nnz, int use_nan, void* workspace,
                     size_t workspace_bytes, void* stream);

/* spfa_csr_forward without a workspace argument and without any allocation.  No counterpart in
 * the reference (its kernel needs no scratch, sp_flatt_csr_kernel.cu:271-287); it is for callers
 * that cannot allocate device memory: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  Same arguments, checks, kernels and results as
 * spfa_csr_forward; the scratch is a device array of SPFA_STATIC_SCRATCH_BYTES bytes inside the
 * library (one per device, held until the process ends), and a call calls neither hipMalloc nor
 * hipFree nor any allocating routine.
 *   - Limit: spfa_csr_workspace_bytes_batched(n_q, nnz, d, dtype, n_batch) <=
 *     SPFA_STATIC_SCRATCH_BYTES, else SPFA_ERR_STATIC_LIMIT and nothing is enqueued (16 MiB holds
 *     a mask of 131072 rows and 12.8 M entries at d = 64; SPFA_DTYPE_F64 problems use no scratch
 *     and have no limit).
 *   - The first call on a device looks the array's address up (hipGetSymbolAddress, under a
 *     mutex); make one call on each device before capturing the entry point in a HIP graph.
 *   - All calls on one device share that device's array: calls that overlap in time on one
 *     device (two streams, two host threads) race; calls in stream order do not.  Nothing needs
 *     clearing between calls. */
#define SPFA_STATIC_SCRATCH_BYTES (16u << 20)
int spfa_csr_forward_static(const spfa_problem_t* p, const void* row_off, int row_off_bytes,
                            const void* col_ind, int64_t nnz, int use_nan, void* stream);

/* COO: row i attends {col_ind[e] : row_ind[e] == i}.  Entries may come in any order (the
 * reference needs them sorted by row, sp_flatt_coo_kernel.cu:47-79); they are bucketed by
 * row on the device first.  row_ind entries are row_ind_bytes (4 or 8) bytes wide. */
size_t spfa_coo_workspace_bytes(int64_t n_q, int64_t nnz, int64_t d, int dtype);
/* ... of a batched call (the conversion's scratch is needed once, not per problem) */
size_t spfa_coo_workspace_bytes_batched(int64_t n_q, int64_t nnz, int64_t d, int dtype, int64_t n_batch);
int spfa_coo_forward(const spfa_problem_t* p, const void* row_ind, int row_ind_bytes,
                     const void* col_ind, int64_t nnz, int use_nan, void* workspace,
                     size_t workspace_bytes, void* stream);

/* Mask plans for the explicit masks.  The reference rebuilds nothing between calls because its
 * kernel reads the mask directly; its callers build a mask once and reuse it for many calls
 * (verification/verify.py:68-71,95-98 build the CSR / COO tensors once; 337-352 chain calls on
 * them).  Here the mask pre-pass (the work list of long rows; for COO also the row offsets and, for
 * unsorted entries, the bucketed columns) does not depend on Q, K, V or their type, so it can be
 * built once into a caller-owned device buffer and reused:
 *
 *   plan = device buffer of spfa_*_plan_bytes(...) bytes, 256-byte aligned
 *   spfa_*_plan(...)              fills it (asynchronous on `stream`)
 *   spfa_*_forward_planned(...)   same result as spfa_*_forward with the same mask arrays, without
 *                                 the pre-pass; reads the plan, writes only `workspace`
 *                                 (spfa_*_workspace_bytes(...) bytes as for the plain call).
 *
 * The mask arrays passed to forward_planned must be the ones the plan was built from (CSR: both;
 * COO: col_ind - it is read in place when the entries were sorted by row).  Calls that share a
 * plan but use different workspaces are independent.  spfa_coo_plan also needs a scratch buffer
 * of spfa_coo_plan_workspace_bytes(...) bytes that is free again when the call has run. */
size_t spfa_csr_plan_bytes(int64_t n_q, int64_t nnz);
int spfa_csr_plan(int64_t n_q, const void* row_off, int row_off_bytes, const void* col_ind,
                  int64_t nnz, void* plan, size_t plan_bytes, void* stream);
int spfa_csr_forward_planned(const spfa_problem_t* p, const void* row_off, int row_off_bytes,
                             const void* col_ind, int64_t nnz, int use_nan, const void* plan,
                             size_t plan_bytes, void* workspace, size_t workspace_bytes,
                             void* stream);
size_t spfa_coo_plan_bytes(int64_t n_q, int64_t nnz);
size_t spfa_coo_plan_workspace_bytes(int64_t n_q, int64_t nnz);
int spfa_coo_plan(int64_t n_q, const void* row_ind, int row_ind_bytes, const void* col_ind,
                  int64_t nnz, void* plan, size_t plan_bytes, void* workspace,
                  size_t workspace_bytes, void* stream);
int spfa_coo_forward_planned(const spfa_problem_t* p, const void* col_ind, int64_t nnz, int use_nan,
                             const void* plan, size_t plan_bytes, void* workspace,
                             size_t workspace_bytes, void* stream);

/* Window + global + CSR in one call (the "BigBird" / "Longformer" pattern).  The reference's
 * callers get it by chaining three calls on one (m, l, out) state: Local, Global-no-local with the
 * same window, CSR with the random part (verification/verify.py:337-352); this entry point is that
 * chain: row i attends its window [i-w, i+w], the listed global tokens outside it (a listed row
 * attends every token), and the columns of the CSR rows.  The three parts must not overlap (a
 * column present twice counts twice, exactly as in the chain); n_globals == 0 or nnz == 0 leave
 * that part out.  n_k must equal n_q.  No row is ever empty (the window holds the diagonal). */
size_t spfa_window_global_csr_workspace_bytes(int64_t n, int64_t d, int dtype, int64_t local_size,
                                              int64_t n_globals, int64_t nnz);
int spfa_window_global_csr_forward(const spfa_problem_t* p, int64_t local_size,
                                   const int32_t* global_inds, int64_t n_globals,
                                   const void* row_off, int row_off_bytes, const void* col_ind,
                                   int64_t nnz, void* workspace, size_t workspace_bytes,
                                   void* stream);

/* Local: row i attends columns max(0, i-w) .. min(n-1, i+w)  (sp_flatt_local_kernel.cu:24-28). */
size_t spfa_local_workspace_bytes(int64_t n, int64_t d, int dtype, int64_t local_size);
int spfa_local_forward(const spfa_problem_t* p, int64_t local_size, void* workspace,
                       size_t workspace_bytes, void* stream);

/* Local 1D dilated, s = dil_factor+1: columns low, low+s, ... <= up with
 * low = max(i - w*s, i mod s), up = min(i + w*s, n-1)
 * (sp_flatt_local_1d_dilated_kernel.cu:25-29,102). */
size_t spfa_local_1d_dilated_workspace_bytes(int64_t n, int64_t d, int dtype, int64_t local_size,
                                             int64_t dil_factor);
int spfa_local_1d_dilated_forward(const spfa_problem_t* p, int64_t local_size, int64_t dil_factor,
                                  void* workspace, size_t workspace_bytes, void* stream);

/* Local 2D dilated: inside each block of block_size rows only rows and columns at multiples
 * of s = dil_factor+1 from the block start are live; other rows are empty
 * (sp_flatt_local_2d_dilated_kernel.cu:26-39,123). */
size_t spfa_local_2d_dilated_workspace_bytes(int64_t n, int64_t d, int dtype, int64_t block_size,
                                             int64_t dil_factor);
int spfa_local_2d_dilated_forward(const spfa_problem_t* p, int64_t block_size, int64_t dil_factor,
                                  int use_nan, void* workspace, size_t workspace_bytes,
                                  void* stream);

/* Global minus local: with window [max(0,i-w), min(n-1,i+w)], a row listed in global_inds
 * attends every column outside its window, any other row attends the global_inds outside its
 * window (sp_flatt_global_no_local_kernel.cu:38-64,134-162).  global_inds: n_globals int32. */
size_t spfa_global_no_local_workspace_bytes(int64_t n, int64_t d, int dtype, int64_t n_globals,
                                            int64_t local_size);
int spfa_global_no_local_forward(const spfa_problem_t* p, const int32_t* global_inds,
                                 int64_t n_globals, int64_t local_size, void* workspace,
                                 size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Gradients.  The reference has no backward pass (its extensions bind `forward` only,
 * Sparse_FlashAttention_CSR/sp_flatt_csr.cpp:57-59); these entry points have no counterpart there.
 * They differentiate the attention the matching *_forward computes: with (m, l, out) the FINISHED
 * forward state of `p` and d_out the gradient of the loss with respect to out, they ADD
 *     d_q[i] += sum_j dS_ij k_j / sqrt(d),  d_k[j] += sum_i dS_ij q_i / sqrt(d),
 *     d_v[j] += sum_i P_ij d_out[i],
 * where P_ij = exp(q_i.k_j / sqrt(d) - m_i - log l_i) on the live positions of the mask and
 * dS_ij = P_ij (d_out[i].v_j - d_out[i].out[i]).  A state built by several chained forward calls is
 * differentiated by one backward call per mask on the same gradient tensors.  Rows with l == 0
 * (never any live column) carry no gradient.
 *   d_out        [n_batch * n_q, d], element type of the problem
 *   d_q          [n_batch * n_q, d]  fp32 (fp64 for F64 problems); the caller zeroes it
 *   d_k, d_v     [n_batch * n_k, d]  likewise.  Rows with more than 1024 live positions are
 *                                    split and their pieces added with floating-point atomics, so
 *                                    two runs may differ in the last bits there (F64: everywhere)
 * Parameter checks and their codes are those of the matching forward call. */
typedef struct spfa_grads {
  const void* d_out;
  void* d_q;
  void* d_k;
  void* d_v;
} spfa_grads_t;

/* workspace: scratch of at least *_backward_workspace_bytes(...) bytes, 256-byte aligned (the
 * softmax statistics of every row, the work list of long rows and, for explicit masks, the mask
 * transposed); n_batch as in spfa_problem_t. */
size_t spfa_csr_backward_workspace_bytes(int64_t n_q, int64_t n_k, int64_t nnz, int64_t d, int dtype,
                                         int64_t n_batch);
/* t_row_off / t_col_ind: the mask read by key row, as spfa_csr_transpose writes it, or both NULL
 * (it is then built inside the call; *_backward_workspace_bytes covers both cases). */
int spfa_csr_backward(const spfa_problem_t* p, const spfa_grads_t* g, const void* row_off,
                      int row_off_bytes, const void* col_ind, int64_t nnz, const uint32_t* t_row_off,
                      const uint32_t* t_col_ind, void* workspace, size_t workspace_bytes, void* stream);
/* A CSR mask of n_q rows over n_k columns read by column: afterwards
 * t_col_ind[t_row_off[j] .. t_row_off[j+1]) are the rows whose CSR row holds column j, in no
 * particular order (t_row_off: n_k + 1 entries, t_col_ind: nnz).  A mask that is used for many
 * backward calls is transposed once with this. */
size_t spfa_csr_transpose_workspace_bytes(int64_t n_q, int64_t n_k, int64_t nnz);
int spfa_csr_transpose(int64_t n_q, int64_t n_k, const void* row_off, int row_off_bytes,
                       const void* col_ind, int64_t nnz, uint32_t* t_row_off, uint32_t* t_col_ind,
                       void* workspace, size_t workspace_bytes, void* stream);
/* COO entries in any order as a CSR mask: row_off (n_rows + 1 entries) and csr_col_ind (nnz; the
 * columns of a row in no particular order), both uint32 - the conversion every spfa_coo_* call does
 * internally (Sparse_FlashAttention_COO/sp_flatt_coo_kernel.cu:47-84 locates a row's range by a
 * scan instead), for callers that keep a mask for many calls and want the CSR entry points, their
 * plans and spfa_csr_transpose. */
size_t spfa_coo_to_csr_workspace_bytes(int64_t n_rows, int64_t nnz);
int spfa_coo_to_csr(int64_t n_rows, const void* row_ind, int row_ind_bytes, const void* col_ind, int64_t nnz,
                    uint32_t* row_off, uint32_t* csr_col_ind, void* workspace, size_t workspace_bytes,
                    void* stream);
size_t spfa_coo_backward_workspace_bytes(int64_t n_q, int64_t n_k, int64_t nnz, int64_t d, int dtype,
                                         int64_t n_batch);
int spfa_coo_backward(const spfa_problem_t* p, const spfa_grads_t* g, const void* row_ind,
                      int row_ind_bytes, const void* col_ind, int64_t nnz, void* workspace,
                      size_t workspace_bytes, void* stream);
size_t spfa_local_backward_workspace_bytes(int64_t n, int64_t d, int dtype, int64_t local_size,
                                           int64_t n_batch);
int spfa_local_backward(const spfa_problem_t* p, const spfa_grads_t* g, int64_t local_size,
                        void* workspace, size_t workspace_bytes, void* stream);
size_t spfa_local_1d_dilated_backward_workspace_bytes(int64_t n, int64_t d, int dtype,
                                                      int64_t local_size, int64_t dil_factor,
                                                      int64_t n_batch);
int spfa_local_1d_dilated_backward(const spfa_problem_t* p, const spfa_grads_t* g,
                                   int64_t local_size, int64_t dil_factor, void* workspace,
                                   size_t workspace_bytes, void* stream);
size_t spfa_local_2d_dilated_backward_workspace_bytes(int64_t n, int64_t d, int dtype,
                                                      int64_t block_size, int64_t dil_factor,
                                                      int64_t n_batch);
int spfa_local_2d_dilated_backward(const spfa_problem_t* p, const spfa_grads_t* g,
                                   int64_t block_size, int64_t dil_factor, void* workspace,
                                   size_t workspace_bytes, void* stream);
size_t spfa_global_no_local_backward_workspace_bytes(int64_t n, int64_t d, int dtype,
                                                     int64_t n_globals, int64_t local_size,
                                                     int64_t n_batch);
int spfa_global_no_local_backward(const spfa_problem_t* p, const spfa_grads_t* g,
                                  const int32_t* global_inds, int64_t n_globals,
                                  int64_t local_size, void* workspace, size_t workspace_bytes,
                                  void* stream);

/* The gradients of spfa_window_global_csr_forward: the three parts' gradient calls in sequence on
 * one workspace (t_row_off / t_col_ind as in spfa_csr_backward, may be NULL). */
size_t spfa_window_global_csr_backward_workspace_bytes(int64_t n, int64_t d, int dtype,
                                                       int64_t local_size, int64_t n_globals,
                                                       int64_t nnz, int64_t n_batch);
int spfa_window_global_csr_backward(const spfa_problem_t* p, const spfa_grads_t* g, int64_t local_size,
                                    const int32_t* global_inds, int64_t n_globals, const void* row_off,
                                    int row_off_bytes, const void* col_ind, int64_t nnz,
                                    const uint32_t* t_row_off, const uint32_t* t_col_ind, void* workspace,
                                    size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SPFA_HIP_H */
