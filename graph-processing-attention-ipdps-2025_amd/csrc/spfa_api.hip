// extern "C" surface of libspfa_hip.so: argument checks, work sizing, workspace carving and the
// dispatch on element type.  Declarations and the contract live in include/spfa_hip.h.
#include "spfa_hip.h"

#include <limits>
#include <mutex>

#include "spfa_backward.hpp"
#include "spfa_grad.hpp"
#include "spfa_f64.hpp"
#include "spfa_kernels.hpp"

using namespace spfa;

namespace {

constexpr int64_t kInlineAll = std::numeric_limits<int64_t>::max();
constexpr int64_t kAnyColumn = std::numeric_limits<int64_t>::max();  // a mask used for its row lengths only



inline bool dtype_ok(int dtype) {
  return dtype == SPFA_DTYPE_F32 || dtype == SPFA_DTYPE_F16 || dtype == SPFA_DTYPE_BF16;
}

// Segment length for long rows: long enough to amortise the pipeline fill and the partial
// result of a segment (1024 candidates: 64 per lane group at d*s = 256 bytes), short enough
// that the work list holds several items per persistent wavefront (about 2048 of them) - but
// never below 512: small masks are walked by an ordinary grid, which does not need the items
// for its balance and pays for every one of them (the Zipf mask at 8192 / 16384 tokens, 128 ->
// 512: 0.139 -> 0.121 / 0.172 -> 0.146 ms fp32, 0.108 -> 0.083 / 0.132 -> 0.097 ms bf16).
inline int64_t pick_segment(int64_t nnz_long) {
  int64_t seg = 512;
  while (seg < 1024 && seg * 2 * 8192 <= nnz_long) seg *= 2;
  return seg;
}

// Rows of up to this many entries are finished by the lane group that looks at them (rows_kernel).
// 8 / 12 / 16 / 24 / 32 / 64 on the Zipf mask: 0.661 / 0.659 / 0.659 / 0.669 / 0.665 / 0.686 ms
// fp32, 0.393 / 0.390 / 0.392 / 0.396 / 0.399 / 0.417 ms bf16; the 1 M-row COO mask and the 4 M-row
// Zipf mask do not care.
constexpr int64_t kExplicitInlineRowLimit = 16;
// Rows between the two limits get a wavefront of their own (medium_rows_kernel).  Measured with
// the limit at 64 / 128 / 256 / 512: the Zipf mask (12.8 M positions) does not care (0.867-0.873
// ms); 64 heads of the 2 % Bernoulli mask (rows of ~83) need it above their row length (3.03 ms
// without, 0.65 with).
constexpr int64_t kExplicitMediumRowLimit = 256;
// ... and rows of up to this many in the masks described below.  (A rule that took 1024 for
// every mask whose K and V stay in the caches, from when the work list was walked row by row by
// persistent wavefronts only, costs the Zipf mask 19 - 27 % at 8192 ... 32768 tokens now: its
// rows of 257 ... 1024 entries, each of another length, are better off as items of the ordered
// work list than as wavefronts of their own.)
constexpr int64_t kExplicitMediumRowLimitDense = 1024;
// K + V up to which the medium-row kernel takes smaller batches (explicit_medium_batch)
constexpr int64_t kCachedKvBytes = (int64_t)24 << 20;

// A mask whose rows hold 128 entries or more on average mostly has rows of about that length (a
// power-law mask of that density being the exception), and rows of one length with sorted columns
// are what a wavefront per row does best: launched together they walk K and V from low to high
// columns in step and find each other's rows in the caches.  Uniform rows of 300 / 600 / 1000
// sorted columns, fp32 d = 64, segment kernel against a wavefront per row: K + V of 16 MiB 8.9 /
// 8.9 / 13.6 against 18.1 / 22.5 / 24.9 TB/s of gathered rows, 64 MiB 7.6 / 6.9 / 8.8 against 8.8 /
// 11.7 / 13.5, 256 MiB 7.3 / 6.4 / 7.5 against 7.2 / 7.6 / 8.2; bf16 at 128 MiB 5.1 / 4.6 / 6.3
// against 7.5 / 8.4 / 8.3.
int64_t medium_limit_of_mask(int64_t n_q, int64_t nnz) {
  return n_q > 0 && nnz / n_q >= 128 ? kExplicitMediumRowLimitDense : kExplicitMediumRowLimit;
}

EngineSizing size_csr(int64_t n_q, int64_t nnz) {
  EngineSizing s{};
  s.nnz_bound = nnz;
  s.max_deg = nnz;
  s.short_max = kExplicitInlineRowLimit;
  s.medium_max = medium_limit_of_mask(n_q, nnz);
  s.seg = pick_segment(nnz);
  s.n_long_bound = n_q;
  return s;
}

// whether the long rows' work list is walked by an ordinary grid (items_grid_kernel, see there)
// (rows of at most 128 bytes keep the advantage longer: bf16 d = 64 at K + V = 64 MiB - 8 %, even at 128 MiB)
constexpr int64_t kItemsGridKvBytes = (int64_t)48 << 20;
constexpr int64_t kItemsGridKvBytesShortRows = (int64_t)96 << 20;
bool explicit_items_on_grid(int64_t n_k, int64_t d, int dtype) {
  const int64_t es = dtype == SPFA_DTYPE_F32 ? 4 : dtype == SPFA_DTYPE_F64 ? 8 : 2;
  return 2 * n_k * d * es <= (d * es <= 128 ? kItemsGridKvBytesShortRows : kItemsGridKvBytes);
}

// ... and whether the list is walked as plan_kernel appended it.  The order it is handed out in
// otherwise keeps the wavefronts at work to one part of K and V at a time, which is worth nothing
// while K and V of a problem fit the L2s anyway; order_kernel's launch then only adds its 4 - 5 us
// to a short call (Zipf mask, d = 64, fp32 / bf16: 8192 tokens 0.063 -> 0.058 / 0.050 -> 0.043 ms,
// 16384 tokens 0.088 -> 0.084 / 0.072 -> 0.065, 32768 tokens 0.154 -> 0.170 / 0.105 -> 0.103: K + V
// of 4, 8 and 16 MiB in fp32).
constexpr int64_t kItemsAsListedKvBytes = (int64_t)8 << 20;
bool explicit_items_as_listed(int64_t n_k, int64_t d, int dtype) {
  const int64_t es = dtype == SPFA_DTYPE_F32 ? 4 : dtype == SPFA_DTYPE_F64 ? 8 : 2;
  return 2 * n_k * d * es <= kItemsAsListedKvBytes;
}

// ... and its batch size in the medium-row kernel (see there): smaller while K and V are not much
// larger than the caches and the rows are long enough on average for the wavefronts to fall in
// step (measured on uniform rows of sorted columns; the Zipf headline - 97 entries per row on
// average, most of them in few long rows - loses 5 % of that kernel with 4, which does not show
// in the call; 64 heads of the 2 % Bernoulli mask of 4096 tokens, rows of ~83: 0.595 -> 0.510 ms
// fp32, 0.440 -> 0.396 ms bf16 with 2).  From 128 entries per row on average; from 64 when K and V
// of a problem fit an L2.  CSR calls only:
// the rows that the COO pre-pass builds keep their entries in the order they came in, and on
// unsorted columns the smaller batches lose up to 10 %.
int explicit_medium_batch(const spfa_problem_t* p, int64_t nnz) {
  if (p->n_q <= 0 || nnz / p->n_q < 64) return 0;
  const int64_t es = p->dtype == SPFA_DTYPE_F32 ? 4 : p->dtype == SPFA_DTYPE_F64 ? 8 : 2;
  // (K and V of one problem: the problems of a batch are walked one after the other)
  const int64_t kv = 2 * p->n_k * p->d * es;
  // 64 ... 127 entries per row: only while K and V fit an L2 (the Zipf mask, ~100 per row, loses
  // 13 % at 16384 tokens - 8 MiB - with 2 or 4, and nothing at 8192)
  if (nnz / p->n_q < 128) return kv <= ((int64_t)4 << 20) ? 2 : 0;
  return kv <= kCachedKvBytes ? 2 : kv <= 4 * kCachedKvBytes ? 4 : 0;
}

// Band / block masks are uniform: every row has about the same number of candidates, so rows
// are finished in place unless there are too few rows to fill the device and they are long.
EngineSizing size_stride(int64_t n, int64_t max_deg) {
  EngineSizing s{};
  s.max_deg = max_deg;
  s.nnz_bound = n * max_deg;
  s.n_long_bound = n;
  if (n < 16384 && max_deg > 1024) {
    s.short_max = 256;
    s.seg = 256;
  } else {
    s.short_max = kInlineAll;
    s.seg = 256;
  }
  return s;
}

EngineSizing size_global(int64_t n, int64_t n_globs) {
  EngineSizing s{};
  const int64_t g = n_globs < n ? n_globs : n;
  s.max_deg = n;
  if (n_globs <= 4096) {
    // ordinary rows (n_globs candidates each) are finished in place, global rows are split
    s.short_max = n_globs < 32 ? 32 : n_globs;
    s.n_long_bound = g;
    s.nnz_bound = g * n;
  } else {
    s.short_max = 256;
    s.n_long_bound = n;
    s.nnz_bound = g * n + n * n_globs;
  }
  s.seg = pick_segment(s.nnz_bound);
  return s;
}

int check_problem(const spfa_problem_t* p) {
  if (p == nullptr) return SPFA_ERR_BAD_ARG;
  if (p->n_q < 0 || p->n_k < 0 || p->n_batch < 0) return SPFA_ERR_BAD_ARG;
  if (p->n_q >= (int64_t)1 << 31 || p->n_k >= (int64_t)1 << 31) return SPFA_ERR_BAD_ARG;
  if (p->d < 1 || p->d > 1024) return SPFA_ERR_EMB_TOO_LARGE;
  return SPFA_OK;
}

bool is_f64(const spfa_problem_t* p) { return p->dtype == SPFA_DTYPE_F64; }

int check_pointers(const spfa_problem_t* p) {
  if (is_f64(p)) {
    if (p->state_dtype != SPFA_DTYPE_F64) return SPFA_ERR_UNSUPPORTED;
  } else {
    if (!dtype_ok(p->dtype)) return SPFA_ERR_UNSUPPORTED;
    if (p->state_dtype != p->dtype && p->state_dtype != SPFA_DTYPE_F32) return SPFA_ERR_UNSUPPORTED;
  }
  if (p->n_q == 0) return SPFA_OK;
  if (!p->q || !p->k || !p->v || !p->m || !p->l || !p->out) return SPFA_ERR_BAD_ARG;
  return SPFA_OK;
}

int check_workspace(const void* ws, size_t have, size_t need) {
  if (need == 0) return SPFA_OK;
  if (ws == nullptr || ((uintptr_t)ws & 255u) != 0 || have < need) return SPFA_ERR_WORKSPACE;
  return SPFA_OK;
}

Tensors make_tensors(const spfa_problem_t* p) {
  Tensors t{};
  t.q = p->q;
  t.k = p->k;
  t.v = p->v;
  t.m = p->m;
  t.l = p->l;
  t.out = p->out;
  t.n_q = p->n_q;
  t.d = (int32_t)p->d;
  t.state_f32 = (p->state_dtype == SPFA_DTYPE_F32) ? 1 : 0;
  t.n_batch = p->n_batch > 1 ? p->n_batch : 1;
  t.kv_stride = p->n_k * p->d;
  return t;
}

int64_t batch_of(const spfa_problem_t* p) { return p->n_batch > 1 ? p->n_batch : 1; }

size_t elem_bytes(int dtype) {
  return dtype == SPFA_DTYPE_F64 ? 8 : dtype == SPFA_DTYPE_F32 ? 4 : 2;
}

// Problem b of a batch as a problem of its own (the paths without batched kernels walk the batch
// on the host, one problem after the other on the same stream and workspace).
spfa_problem_t batch_slice(const spfa_problem_t* p, int64_t b) {
  spfa_problem_t s = *p;
  const size_t es = elem_bytes(p->dtype), ss = elem_bytes(p->state_dtype);
  s.q = (const char*)p->q + (size_t)b * p->n_q * p->d * es;
  s.k = (const char*)p->k + (size_t)b * p->n_k * p->d * es;
  s.v = (const char*)p->v + (size_t)b * p->n_k * p->d * es;
  s.out = (char*)p->out + (size_t)b * p->n_q * p->d * es;
  s.m = (char*)p->m + (size_t)b * p->n_q * ss;
  s.l = (char*)p->l + (size_t)b * p->n_q * ss;
  s.n_batch = 1;
  return s;
}

int dispatch_csr(const spfa_problem_t* p, const CsrMask& mask, const EngineSizing& s, int use_nan,
                 void* ws, hipStream_t stream, int phase = kEngineAll, const void* plan_buf = nullptr) {
  Tensors t = make_tensors(p);
  switch (p->dtype) {
    case SPFA_DTYPE_F32: return run_csr<float>(t, mask, s, use_nan, ws, stream, phase, plan_buf);
    case SPFA_DTYPE_F16: return run_csr<f16>(t, mask, s, use_nan, ws, stream, phase, plan_buf);
    case SPFA_DTYPE_BF16: return run_csr<bf16>(t, mask, s, use_nan, ws, stream, phase, plan_buf);
  }
  return SPFA_ERR_UNSUPPORTED;
}

// The work list of an explicit mask does not depend on Q, K, V or their type: it is built with a
// problem that only carries the row count.
int build_work_list(int64_t n_q, const CsrMask& mask, const EngineSizing& s, void* plan_buf,
                    hipStream_t stream) {
  Tensors t{};
  t.n_q = n_q;
  t.d = 64;
  t.n_batch = 1;
  return run_csr<float>(t, mask, s, 0, plan_buf, stream, kEnginePlanOnly, nullptr);
}

// The batched engine counts work items of all problems in one 32-bit cursor.
bool batch_fits_engine(const EngineSizing& s, const spfa_problem_t* p) {
  const int64_t b = batch_of(p);
  if (b == 1) return true;
  const WorkspaceLayout w = engine_workspace(s, p->n_q, p->d, 1);
  return (int64_t)w.cap_items * b < ((int64_t)1 << 32) - 1 && p->n_q * b < ((int64_t)1 << 40);
}

size_t work_list_bytes(int64_t n_q, int64_t nnz) {
  return engine_workspace(size_csr(n_q, nnz), n_q, 64).off_pm;
}

int dispatch_stride(const spfa_problem_t* p, const StrideMask& mask, const EngineSizing& s,
                    int use_nan, void* ws, hipStream_t stream) {
  Tensors t = make_tensors(p);
  switch (p->dtype) {
    case SPFA_DTYPE_F32: return run_stride<float>(t, mask, s, use_nan, ws, stream);
    case SPFA_DTYPE_F16: return run_stride<f16>(t, mask, s, use_nan, ws, stream);
    case SPFA_DTYPE_BF16: return run_stride<bf16>(t, mask, s, use_nan, ws, stream);
  }
  return SPFA_ERR_UNSUPPORTED;
}

// Band / block masks whose rows are long enough go to the dense-tile kernel.
// The tile problem of a band / block mask; false when it does not fit the tile kernels' index
// arithmetic.
bool band_tile_args(const spfa_problem_t* p, int64_t w, int64_t stride, int64_t block, int64_t cnt,
                    TileArgs* out) {
  TileArgs a{};
  a.t = make_tensors(p);
  a.n = p->n_q;
  a.s = stride;
  a.block = block;
  a.cnt = cnt;
  int64_t n_sub, len_max;
  if (block > 0) {
    n_sub = p->n_q / block;
    len_max = cnt;
    a.w = cnt;
  } else {
    n_sub = stride < p->n_q ? stride : p->n_q;
    len_max = (p->n_q + stride - 1) / stride;
    a.w = w < len_max ? w : len_max;
  }
  a.tiles_per_sub = (len_max + 127) / 128;
  a.n_tiles = n_sub * a.tiles_per_sub;
  if (a.n_tiles * a.t.n_batch + 8 >= ((int64_t)1 << 31)) return false;
  if (p->n_q * a.t.n_batch * p->d >= ((int64_t)1 << 40)) return false;
  *out = a;
  return true;
}

int dispatch_band(const spfa_problem_t* p, int64_t w, int64_t stride, int64_t block, int64_t cnt,
                  int use_nan, hipStream_t stream) {
  TileArgs a{};
  if (!band_tile_args(p, w, stride, block, cnt, &a)) return -1;
  switch (p->dtype) {
    case SPFA_DTYPE_F32: return run_band<float>(a, use_nan, stream);
    case SPFA_DTYPE_F16: return run_band<f16>(a, use_nan, stream);
    case SPFA_DTYPE_BF16: return run_band<bf16>(a, use_nan, stream);
  }
  return -1;
}

// rows shorter than this are cheaper on the row-gather engine than on 32x32 tiles
constexpr int64_t kBandTileMinRow = 32;
// the tile kernels test windows in 32-bit arithmetic: (unsigned)(delta + w) <= 2w
constexpr int64_t kTileMaxWindow = (int64_t)1 << 30;

// Shortest row (candidates per query, 2w + 1) of a window mask that goes to the tiles.  A tile
// costs the same whatever part of it is live, a gathered row costs by the candidate.  Measured
// crossovers of the window kernels (N = 32768 ... 262144, d = 32 ... 256): forward 5 - 7
// candidates per row for the half types and 11 - 27 for fp32 (whose matrix instructions are
// sixteen times slower); the gradient call, whose gather passes cost more per candidate, below
// 3 for the half types and for fp32 at d = 32, 11 at d = 64, 27 at d = 128.  A call of fewer rows
// is bound by its launches either way and stays on the gather engine up to the general limit.
int64_t window_tile_min_row(const spfa_problem_t* p, bool gradient) {
  if (p->n_q * batch_of(p) < 32768) return kBandTileMinRow;
  const bool f32 = p->dtype == SPFA_DTYPE_F32;
  if (gradient) {
    if (!f32 || p->d <= 32) return 3;
    return p->d <= 64 ? 13 : p->d <= 128 ? 27 : kBandTileMinRow;
  }
  if (!f32) return 7;
  return p->d <= 32 ? 13 : p->d <= 64 ? 21 : p->d <= 128 ? 13 : 27;
}

int dispatch_global(const spfa_problem_t* p, const GlobalMask& mask, const EngineSizing& s,
                    void* ws, hipStream_t stream) {
  Tensors t = make_tensors(p);
  switch (p->dtype) {
    case SPFA_DTYPE_F32: return run_global<float>(t, mask, s, 0, ws, stream);
    case SPFA_DTYPE_F16: return run_global<f16>(t, mask, s, 0, ws, stream);
    case SPFA_DTYPE_BF16: return run_global<bf16>(t, mask, s, 0, ws, stream);
  }
  return SPFA_ERR_UNSUPPORTED;
}

int64_t band_max_deg(int64_t n, int64_t w) {
  int64_t deg = 2 * w + 1;
  return deg < n ? deg : n;
}

int64_t block_live_count(int64_t block, int64_t s) {
  int64_t cnt = (block - 1) / s + 1;
  return cnt < block ? cnt : block;
}

// workspace of the global-minus-local path: [bitmap + counter][distinct rows][engine][partials]
struct GlobalLayout {
  size_t off_bits, off_uq, off_engine, off_pm, off_pl, off_pacc, total;
  int64_t key_run, n_split;
};

GlobalLayout global_layout(int64_t n, int64_t n_globs, int64_t d, int64_t n_batch = 1) {
  GlobalLayout g{};
  const int64_t q_tiles = (n_globs + 127) / 128;
  // one key split per workgroup slot of the device (two workgroups fit a CU): more splits only
  // add partial results for the merge to read; none shorter than 512 keys for long sequences,
  // down to 128 for short ones (a workgroup walks its keys one tile after the other: with 512
  // for every length, as first written, 30000 tokens used 59 of the 512 slots and 1000 tokens
  // spent 60 us in two workgroups at d = 128 fp32)
  int64_t want = 2 * (int64_t)device_cu_count() / q_tiles;
  if (want < 1) want = 1;
  int64_t run = (n + want - 1) / want;
  int64_t min_run = (n / 128 + 63) / 64 * 64;
  min_run = min_run < 128 ? 128 : min_run > 512 ? 512 : min_run;
  if (run < min_run) run = min_run;
  run = (run + 63) / 64 * 64;
  g.key_run = run;
  g.n_split = (n + run - 1) / run;
  const size_t slots = (size_t)n_globs * (size_t)g.n_split * (size_t)(n_batch > 1 ? n_batch : 1);
  size_t off = 0;
  g.off_bits = off;   off = align_up(off + global_bits_words(n) * 4, 256);
  g.off_uq = off;     off = align_up(off + (size_t)n_globs * 4, 256);
  g.off_engine = off; off = align_up(off + engine_workspace(size_global(n, n_globs), n, d, n_batch).total, 256);
  g.off_pm = off;     off = align_up(off + slots * 4, 256);
  g.off_pl = off;     off = align_up(off + slots * 4, 256);
  g.off_pacc = off;   off = align_up(off + slots * (size_t)d * 4, 256);
  g.total = off;
  return g;
}

}  // namespace

// One word per device that kernels OR bits into when mask arrays turn out inconsistent (see
// spfa_device_status).  Its name is only a host-side handle: the device address comes from the
// runtime, once per device.
static __device__ uint32_t spfa_status_word;

namespace spfa {
KernelEvents& kernel_events() {
  static thread_local KernelEvents ev;  // (per host thread: the caller's own calls only)
  return ev;
}

uint32_t* device_status_word() {
  constexpr int kMaxDevices = 64;
  static uint32_t* ptrs[kMaxDevices];
  static bool tried[kMaxDevices];
  static std::mutex mu;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lock(mu);
  if (!tried[dev]) {
    tried[dev] = true;
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(spfa_status_word)) == hipSuccess) ptrs[dev] = (uint32_t*)ptr;
    else (void)hipGetLastError();
  }
  return ptrs[dev];
}
}  // namespace spfa

extern "C" {

int spfa_version(void) { return 1; }

int64_t spfa_explicit_inline_row_limit(void) { return kExplicitMediumRowLimit; }

int spfa_explicit_long_rows_on_grid(int64_t n_k, int64_t d, int dtype) {
  return explicit_items_on_grid(n_k, d, dtype) ? 1 : 0;
}

int64_t spfa_explicit_one_launch_row_limit(void) { return kFusedRowsMax; }

int spfa_device_status(int reset) {
  uint32_t* word = device_status_word();
  if (word == nullptr) return -1;
  uint32_t bits = 0;
  if (hipMemcpy(&bits, word, sizeof(bits), hipMemcpyDeviceToHost) != hipSuccess) return -1;
  if (reset && bits != 0) {
    const uint32_t zero = 0;
    if (hipMemcpy(word, &zero, sizeof(zero), hipMemcpyHostToDevice) != hipSuccess) return -1;
  }
  return (int)bits;
}

void spfa_set_kernel_events(void* start, void* stop) {
  kernel_events().start = (hipEvent_t)start;
  kernel_events().stop = (hipEvent_t)stop;
}

const char* spfa_status_string(int status) {
  switch (status) {
    case SPFA_OK: return "ok";
    case SPFA_ERR_BAD_ARG: return "spfa: bad argument (null pointer, negative size or index width not 4/8)";
    case SPFA_ERR_UNSUPPORTED: return "spfa: unsupported element type";
    case SPFA_ERR_WORKSPACE: return "spfa: workspace missing, misaligned or too small";
    case SPFA_ERR_LAUNCH: return "spfa: kernel launch failed";
    case SPFA_ERR_EMB_TOO_LARGE:
      return "The embedded dimension is too large for the amount of shared memory on your GPU.";
    case SPFA_ERR_LOCAL_SIZE:
      return "The local size specified is either negative or greater than/equal to (1 - Sequence Length).";
    case SPFA_ERR_DILATION_NEG: return "The dilation factor must be atleast 0.";
    case SPFA_ERR_BLOCK_DIVISOR:
      return "The block/window size must be a divisor of the whole tensor's size.";
    case SPFA_ERR_BLOCK_DILATION: return "The dilation factor must be less than the block/window size.";
    case SPFA_ERR_GLOBAL_COUNT:
      return "There are either no global tokens provided or there are more than the sequence length given.";
    case SPFA_ERR_STATIC_LIMIT:
      return "spfa: the mask needs more scratch than the library's static buffer "
             "(SPFA_STATIC_SCRATCH_BYTES) holds; use spfa_csr_forward with a workspace";
  }
  return "spfa: unknown status";
}

/* ------------------------------------------------------------------------------ CSR */
size_t spfa_csr_workspace_bytes(int64_t n_q, int64_t nnz, int64_t d, int dtype) {
  (void)dtype;
  if (n_q < 0 || nnz < 0 || d < 1) return 0;
  return engine_workspace(size_csr(n_q, nnz), n_q, d).total;
}

size_t spfa_csr_workspace_bytes_batched(int64_t n_q, int64_t nnz, int64_t d, int dtype, int64_t n_batch) {
  (void)dtype;
  if (n_q < 0 || nnz < 0 || d < 1) return 0;
  const EngineSizing s = size_csr(n_q, nnz);
  spfa_problem_t p{};
  p.n_q = n_q;
  p.d = d;
  p.n_batch = n_batch;
  // (a batch too large for the engine's 32-bit work cursor is walked problem by problem)
  return engine_workspace(s, n_q, d, batch_fits_engine(s, &p) ? batch_of(&p) : 1).total;
}

int spfa_csr_forward(const spfa_problem_t* p, const void* row_off, int row_off_bytes,
                     const void* col_ind, int64_t nnz, int use_nan, void* workspace,
                     size_t workspace_bytes, void* stream) {
  int rc = check_problem(p);
  if (rc) return rc;
  if (nnz < 0 || (row_off_bytes != 4 && row_off_bytes != 8)) return SPFA_ERR_BAD_ARG;
  rc = check_pointers(p);
  if (rc) return rc;
  if (p->n_q == 0) return SPFA_OK;
  if (!row_off || (nnz > 0 && !col_ind)) return SPFA_ERR_BAD_ARG;
  if (is_f64(p)) {
    CsrMask mask{row_off, (const uint32_t*)col_ind, row_off_bytes == 8 ? 1 : 0, nullptr, nullptr, nnz, p->n_k};
    return run_f64(make_tensors(p), mask, use_nan ? 1 : 0, (hipStream_t)stream);
  }
  EngineSizing s = size_csr(p->n_q, nnz);
  s.items_on_grid = explicit_items_on_grid(p->n_k, p->d, p->dtype);
  s.items_as_listed = explicit_items_as_listed(p->n_k, p->d, p->dtype);
  s.medium_batch = explicit_medium_batch(p, nnz);
  if (!batch_fits_engine(s, p)) {
    for (int64_t b = 0; b < batch_of(p); b++) {
      const spfa_problem_t one = batch_slice(p, b);
      rc = spfa_csr_forward(&one, row_off, row_off_bytes, col_ind, nnz, use_nan, workspace,
                            workspace_bytes, stream);
      if (rc) return rc;
    }
    return SPFA_OK;
  }
  rc = check_workspace(workspace, workspace_bytes,
                       engine_workspace(s, p->n_q, p->d, batch_of(p)).total);
  if (rc) return rc;
  CsrMask mask{row_off, (const uint32_t*)col_ind, row_off_bytes == 8 ? 1 : 0, nullptr, nullptr, nnz, p->n_k};
  return dispatch_csr(p, mask, s, use_nan ? 1 : 0, workspace, (hipStream_t)stream);
}

size_t spfa_csr_plan_bytes(int64_t n_q, int64_t nnz) {
  if (n_q < 0 || nnz < 0) return 0;
  return work_list_bytes(n_q, nnz);
}

int spfa_csr_plan(int64_t n_q, const void* row_off, int row_off_bytes, const void* col_ind,
                  int64_t nnz, void* plan, size_t plan_bytes, void* stream) {
  if (n_q < 0 || n_q >= (int64_t)1 << 31 || nnz < 0 || (row_off_bytes != 4 && row_off_bytes != 8))
    return SPFA_ERR_BAD_ARG;
  if (n_q == 0) return SPFA_OK;
  if (!row_off || (nnz > 0 && !col_ind)) return SPFA_ERR_BAD_ARG;
  int rc = check_workspace(plan, plan_bytes, work_list_bytes(n_q, nnz));
  if (rc) return rc;
  CsrMask mask{row_off, (const uint32_t*)col_ind, row_off_bytes == 8 ? 1 : 0, nullptr, nullptr, nnz, kAnyColumn};
  return build_work_list(n_q, mask, size_csr(n_q, nnz), plan, (hipStream_t)stream);
}

int spfa_csr_forward_planned(const spfa_problem_t* p, const void* row_off, int row_off_bytes,
                             const void* col_ind, int64_t nnz, int use_nan, const void* plan,
                             size_t plan_bytes, void* workspace, size_t workspace_bytes,
                             void* stream) {
  int rc = check_problem(p);
  if (rc) return rc;
  if (nnz < 0 || (row_off_bytes != 4 && row_off_bytes != 8)) return SPFA_ERR_BAD_ARG;
  rc = check_pointers(p);
  if (rc) return rc;
  if (p->n_q == 0) return SPFA_OK;
  if (!row_off || (nnz > 0 && !col_ind)) return SPFA_ERR_BAD_ARG;
  if (is_f64(p)) {  // (the fp64 kernel needs no work list)
    CsrMask mask{row_off, (const uint32_t*)col_ind, row_off_bytes == 8 ? 1 : 0, nullptr, nullptr, nnz, p->n_k};
    return run_f64(make_tensors(p), mask, use_nan ? 1 : 0, (hipStream_t)stream);
  }
  EngineSizing s = size_csr(p->n_q, nnz);
  s.items_on_grid = explicit_items_on_grid(p->n_k, p->d, p->dtype);
  s.items_as_listed = explicit_items_as_listed(p->n_k, p->d, p->dtype);
  s.medium_batch = explicit_medium_batch(p, nnz);  // (a launch-time choice: the plan does not depend on it)
  rc = check_workspace(plan, plan_bytes, work_list_bytes(p->n_q, nnz));
  if (rc) return rc;
  if (!batch_fits_engine(s, p)) {
    for (int64_t b = 0; b < batch_of(p); b++) {
      const spfa_problem_t one = batch_slice(p, b);
      rc = spfa_csr_forward_planned(&one, row_off, row_off_bytes, col_ind, nnz, use_nan, plan,
                                    plan_bytes, workspace, workspace_bytes, stream);
      if (rc) return rc;
    }
    return SPFA_OK;
  }
  rc = check_workspace(workspace, workspace_bytes,
                       engine_workspace(s, p->n_q, p->d, batch_of(p)).total);
  if (rc) return rc;
  CsrMask mask{row_off, (const uint32_t*)col_ind, row_off_bytes == 8 ? 1 : 0, nullptr, nullptr, nnz, p->n_k};
  return dispatch_csr(p, mask, s, use_nan ? 1 : 0, workspace, (hipStream_t)stream, kEngineRunOnly,
                      plan);
}

/* ------------------------------------------------------------------------------ COO */
size_t spfa_coo_workspace_bytes(int64_t n_q, int64_t nnz, int64_t d, int dtype) {
  (void)dtype;
  if (n_q < 0 || nnz < 0 || d < 1) return 0;
  return coo_workspace(n_q, nnz).total + engine_workspace(size_csr(n_q, nnz), n_q, d).total;
}

size_t spfa_coo_workspace_bytes_batched(int64_t n_q, int64_t nnz, int64_t d, int dtype, int64_t n_batch) {
  if (n_q < 0 || nnz < 0 || d < 1) return 0;
  return coo_workspace(n_q, nnz).total + spfa_csr_workspace_bytes_batched(n_q, nnz, d, dtype, n_batch);
}

int spfa_coo_forward(const spfa_problem_t* p, const void* row_ind, int row_ind_bytes,
                     const void* col_ind, int64_t nnz, int use_nan, void* workspace,
                     size_t workspace_bytes, void* stream) {
  int rc = check_problem(p);
  if (rc) return rc;
  if (nnz < 0 || nnz >= (int64_t)1 << 31 || (row_ind_bytes != 4 && row_ind_bytes != 8))
    return SPFA_ERR_BAD_ARG;
  rc = check_pointers(p);
  if (rc) return rc;
  if (p->n_q == 0) return SPFA_OK;
  if (nnz > 0 && (!row_ind || !col_ind)) return SPFA_ERR_BAD_ARG;
  EngineSizing s = size_csr(p->n_q, nnz);
  s.items_on_grid = explicit_items_on_grid(p->n_k, p->d, p->dtype);
  s.items_as_listed = explicit_items_as_listed(p->n_k, p->d, p->dtype);
  const size_t coo_bytes = coo_workspace(p->n_q, nnz).total;
  const bool batched = batch_fits_engine(s, p);
  rc = check_workspace(workspace, workspace_bytes,
                       coo_bytes + engine_workspace(s, p->n_q, p->d, batched ? batch_of(p) : 1).total);
  if (rc) return rc;
  CooCsr csr{};
  const CooWorkspace cw = coo_workspace(p->n_q, nnz);
  rc = coo_to_csr(row_ind, row_ind_bytes == 8 ? 1 : 0, (const uint32_t*)col_ind, nnz, p->n_q, p->n_k,
                  workspace, (char*)workspace + cw.keep_total, (hipStream_t)stream, &csr);
  if (rc) return rc;
  CsrMask mask{csr.row_off, (const uint32_t*)col_ind, 0, csr.cols, csr.unsorted, nnz, p->n_k};
  if (is_f64(p)) return run_f64(make_tensors(p), mask, use_nan ? 1 : 0, (hipStream_t)stream);
  if (!batched) {  // one conversion, then problem after problem
    for (int64_t b = 0; b < batch_of(p); b++) {
      const spfa_problem_t one = batch_slice(p, b);
      rc = dispatch_csr(&one, mask, s, use_nan ? 1 : 0, (char*)workspace + coo_bytes,
                        (hipStream_t)stream);
      if (rc) return rc;
    }
    return SPFA_OK;
  }
  return dispatch_csr(p, mask, s, use_nan ? 1 : 0, (char*)workspace + coo_bytes,
                      (hipStream_t)stream);
}

size_t spfa_coo_plan_bytes(int64_t n_q, int64_t nnz) {
  if (n_q < 0 || nnz < 0) return 0;
  return coo_workspace(n_q, nnz).keep_total + work_list_bytes(n_q, nnz);
}

size_t spfa_coo_plan_workspace_bytes(int64_t n_q, int64_t nnz) {
  if (n_q < 0 || nnz < 0) return 0;
  const CooWorkspace w = coo_workspace(n_q, nnz);
  return w.total - w.keep_total;
}

int spfa_coo_plan(int64_t n_q, const void* row_ind, int row_ind_bytes, const void* col_ind,
                  int64_t nnz, void* plan, size_t plan_bytes, void* workspace,
                  size_t workspace_bytes, void* stream) {
  if (n_q < 0 || n_q >= (int64_t)1 << 31 || nnz < 0 || nnz >= (int64_t)1 << 31 ||
      (row_ind_bytes != 4 && row_ind_bytes != 8))
    return SPFA_ERR_BAD_ARG;
  if (n_q == 0) return SPFA_OK;
  if (nnz > 0 && (!row_ind || !col_ind)) return SPFA_ERR_BAD_ARG;
  const CooWorkspace w = coo_workspace(n_q, nnz);
  int rc = check_workspace(plan, plan_bytes, w.keep_total + work_list_bytes(n_q, nnz));
  if (rc) return rc;
  rc = check_workspace(workspace, workspace_bytes, w.total - w.keep_total);
  if (rc) return rc;
  CooCsr csr{};
  rc = coo_to_csr(row_ind, row_ind_bytes == 8 ? 1 : 0, (const uint32_t*)col_ind, nnz, n_q, 0, plan,
                  workspace, (hipStream_t)stream, &csr);
  if (rc) return rc;
  CsrMask mask{csr.row_off, (const uint32_t*)col_ind, 0, csr.cols, csr.unsorted, nnz, kAnyColumn};
  return build_work_list(n_q, mask, size_csr(n_q, nnz), (char*)plan + w.keep_total,
                         (hipStream_t)stream);
}

int spfa_coo_forward_planned(const spfa_problem_t* p, const void* col_ind, int64_t nnz, int use_nan,
                             const void* plan, size_t plan_bytes, void* workspace,
                             size_t workspace_bytes, void* stream) {
  int rc = check_problem(p);
  if (rc) return rc;
  if (nnz < 0 || nnz >= (int64_t)1 << 31) return SPFA_ERR_BAD_ARG;
  rc = check_pointers(p);
  if (rc) return rc;
  if (p->n_q == 0) return SPFA_OK;
  if (nnz > 0 && !col_ind) return SPFA_ERR_BAD_ARG;
  EngineSizing s = size_csr(p->n_q, nnz);
  s.items_on_grid = explicit_items_on_grid(p->n_k, p->d, p->dtype);
  s.items_as_listed = explicit_items_as_listed(p->n_k, p->d, p->dtype);
  const CooWorkspace w = coo_workspace(p->n_q, nnz);
  rc = check_workspace(plan, plan_bytes, w.keep_total + work_list_bytes(p->n_q, nnz));
  if (rc) return rc;
  if (!batch_fits_engine(s, p)) {
    for (int64_t b = 0; b < batch_of(p); b++) {
      const spfa_problem_t one = batch_slice(p, b);
      rc = spfa_coo_forward_planned(&one, col_ind, nnz, use_nan, plan, plan_bytes, workspace,
                                    workspace_bytes, stream);
      if (rc) return rc;
    }
    return SPFA_OK;
  }
  rc = check_workspace(workspace, workspace_bytes,
                       engine_workspace(s, p->n_q, p->d, batch_of(p)).total);
  if (rc) return rc;
  const char* pb = (const char*)plan;
  CsrMask mask{pb + w.off_row_off, (const uint32_t*)col_ind, 0, (const uint32_t*)(pb + w.off_cols),
               (const uint32_t*)(pb + w.off_flag), nnz, p->n_k};
  if (is_f64(p)) return run_f64(make_tensors(p), mask, use_nan ? 1 : 0, (hipStream_t)stream);
  return dispatch_csr(p, mask, s, use_nan ? 1 : 0, workspace, (hipStream_t)stream, kEngineRunOnly,
                      pb + w.keep_total);
}

/* ------------------------------------------------------------------------------ Local */
size_t spfa_local_workspace_bytes(int64_t n, int64_t d, int dtype, int64_t local_size) {
  (void)dtype;
  if (n < 1 || d < 1 || local_size < 0) return 0;
  return engine_workspace(size_stride(n, band_max_deg(n, local_size)), n, d).total;
}

int spfa_local_forward(const spfa_problem_t* p, int64_t local_size, void* workspace,
                       size_t workspace_bytes, void* stream) {
  return spfa_local_1d_dilated_forward(p, local_size, 0, workspace, workspace_bytes, stream);
}

/* ------------------------------------------------------------------------------ Local 1D dilated */
size_t spfa_local_1d_dilated_workspace_bytes(int64_t n, int64_t d, int dtype, int64_t local_size,
                                             int64_t dil_factor) {
  (void)dil_factor;
  return spfa_local_workspace_bytes(n, d, dtype, local_size);
}

int spfa_local_1d_dilated_forward(const spfa_problem_t* p, int64_t local_size, int64_t dil_factor,
                                  void* workspace, size_t workspace_bytes, void* stream) {
  int rc = check_problem(p);
  if (rc) return rc;
  if (local_size < 0 || local_size > p->n_q - 1) return SPFA_ERR_LOCAL_SIZE;
  if (dil_factor < 0) return SPFA_ERR_DILATION_NEG;
  if (dil_factor >= (int64_t)1 << 31 || p->n_k != p->n_q) return SPFA_ERR_BAD_ARG;
  rc = check_pointers(p);
  if (rc) return rc;
  const int64_t n = p->n_q;
  EngineSizing s = size_stride(n, band_max_deg(n, local_size));
  rc = check_workspace(workspace, workspace_bytes, engine_workspace(s, n, p->d, batch_of(p)).total);
  if (rc) return rc;
  {
    const int64_t len_max = (n + dil_factor) / (dil_factor + 1);
    const int64_t span = 2 * local_size + 1 < len_max ? 2 * local_size + 1 : len_max;
    if (span >= window_tile_min_row(p, false) && dtype_ok(p->dtype) && local_size <= kTileMaxWindow) {
      rc = dispatch_band(p, local_size, dil_factor + 1, 0, 0, 0, (hipStream_t)stream);
      if (rc >= 0) return rc;
    }
  }
  StrideMask mask{n, local_size, dil_factor + 1, 0, 0};
  if (is_f64(p)) return run_f64(make_tensors(p), mask, 0, (hipStream_t)stream);
  return dispatch_stride(p, mask, s, 0, workspace, (hipStream_t)stream);
}

/* ------------------------------------------------------------------------------ Local 2D dilated */
size_t spfa_local_2d_dilated_workspace_bytes(int64_t n, int64_t d, int dtype, int64_t block_size,
                                             int64_t dil_factor) {
  (void)dtype;
  if (n < 1 || d < 1 || block_size < 1 || dil_factor < 0) return 0;
  return engine_workspace(size_stride(n, block_live_count(block_size, dil_factor + 1)), n, d).total;
}

int spfa_local_2d_dilated_forward(const spfa_problem_t* p, int64_t block_size, int64_t dil_factor,
                                  int use_nan, void* workspace, size_t workspace_bytes,
                                  void* stream) {
  int rc = check_problem(p);
  if (rc) return rc;
  if (block_size <= 0 || p->n_q % block_size != 0) return SPFA_ERR_BLOCK_DIVISOR;
  if (dil_factor < 0) return SPFA_ERR_DILATION_NEG;
  if (block_size / (dil_factor + 1) < 1) return SPFA_ERR_BLOCK_DILATION;
  if (p->n_k != p->n_q) return SPFA_ERR_BAD_ARG;
  rc = check_pointers(p);
  if (rc) return rc;
  const int64_t n = p->n_q;
  if (n == 0) return SPFA_OK;
  const int64_t cnt = block_live_count(block_size, dil_factor + 1);
  EngineSizing s = size_stride(n, cnt);
  rc = check_workspace(workspace, workspace_bytes, engine_workspace(s, n, p->d, batch_of(p)).total);
  if (rc) return rc;
  if (cnt >= kBandTileMinRow && dtype_ok(p->dtype)) {
    rc = dispatch_band(p, 0, dil_factor + 1, block_size, cnt, use_nan ? 1 : 0, (hipStream_t)stream);
    if (rc >= 0) return rc;
  }
  StrideMask mask{n, 0, dil_factor + 1, block_size, cnt};
  if (is_f64(p)) return run_f64(make_tensors(p), mask, use_nan ? 1 : 0, (hipStream_t)stream);
  return dispatch_stride(p, mask, s, use_nan ? 1 : 0, workspace, (hipStream_t)stream);
}

/* ------------------------------------------------------------------------------ Global minus local */
size_t spfa_global_no_local_workspace_bytes(int64_t n, int64_t d, int dtype, int64_t n_globals,
                                            int64_t local_size) {
  (void)dtype;
  (void)local_size;
  if (n < 1 || d < 1 || n_globals < 1) return 0;
  return global_layout(n, n_globals, d).total;
}

namespace {

// The dense-tile problem of the global-minus-local mask over a workspace laid out by
// global_layout; false when it does not fit the tile kernels' index arithmetic.
bool global_tile_args(const spfa_problem_t* p, const int32_t* global_inds, int64_t n_globals,
                      int64_t local_size, const GlobalLayout& lay, char* base, TileArgs* out) {
  const int64_t n = p->n_q;
  uint32_t* bits = (uint32_t*)(base + lay.off_bits);
  TileArgs a{};
  a.t = make_tensors(p);
  a.n = n;
  a.w = local_size;
  a.s = 1;
  a.globs = global_inds;
  a.n_globs = n_globals;
  a.gbits = bits;
  a.uq = (int32_t*)(base + lay.off_uq);
  a.n_uq = bits + (global_bits_words(n) - 1);
  a.key_run = lay.key_run;
  a.n_split = lay.n_split;
  a.pm = (float*)(base + lay.off_pm);
  a.pl = (float*)(base + lay.off_pl);
  a.pacc = (float*)(base + lay.off_pacc);
  *out = a;
  const int64_t q_tiles = (n_globals + 127) / 128;
  return q_tiles * lay.n_split * batch_of(p) < ((int64_t)1 << 31) &&
         n_globals * batch_of(p) < ((int64_t)1 << 31) && batch_of(p) < 65536 &&
         local_size <= kTileMaxWindow;
}

}  // namespace

int spfa_global_no_local_forward(const spfa_problem_t* p, const int32_t* global_inds,
                                 int64_t n_globals, int64_t local_size, void* workspace,
                                 size_t workspace_bytes, void* stream) {
  int rc = check_problem(p);
  if (rc) return rc;
  if (n_globals <= 0 || n_globals > p->n_q) return SPFA_ERR_GLOBAL_COUNT;
  if (local_size < 0 || local_size > p->n_q - 1) return SPFA_ERR_LOCAL_SIZE;
  if (p->n_k != p->n_q) return SPFA_ERR_BAD_ARG;
  rc = check_pointers(p);
  if (rc) return rc;
  if (!global_inds) return SPFA_ERR_BAD_ARG;
  const int64_t n = p->n_q;
  const GlobalLayout lay = global_layout(n, n_globals, p->d, batch_of(p));
  rc = check_workspace(workspace, workspace_bytes, lay.total);
  if (rc) return rc;
  char* base = (char*)workspace;
  uint32_t* bits = (uint32_t*)(base + lay.off_bits);
  int32_t* uq = (int32_t*)(base + lay.off_uq);
  rc = prepare_global_rows(global_inds, n_globals, n, bits, uq, (hipStream_t)stream);
  if (rc) return rc;
  if (is_f64(p)) {
    GlobalMask mask{n, local_size, global_inds, n_globals, bits};
    return run_f64(make_tensors(p), mask, 0, (hipStream_t)stream);
  }

  // dense tiles when the shape allows it
  TileArgs a{};
  if (global_tile_args(p, global_inds, n_globals, local_size, lay, base, &a)) {
    rc = -1;
    switch (p->dtype) {
      case SPFA_DTYPE_F32: rc = run_global_dense<float>(a, (hipStream_t)stream); break;
      case SPFA_DTYPE_F16: rc = run_global_dense<f16>(a, (hipStream_t)stream); break;
      case SPFA_DTYPE_BF16: rc = run_global_dense<bf16>(a, (hipStream_t)stream); break;
    }
    if (rc >= 0) return rc;
  }

  EngineSizing s = size_global(n, n_globals);
  GlobalMask mask{n, local_size, global_inds, n_globals, bits};
  return dispatch_global(p, mask, s, base + lay.off_engine, (hipStream_t)stream);
}

namespace {

// The listed tokens' rows of a window + global call whose other rows have had the listed tokens as
// keys inside the band kernel already.
int global_rows_only(const spfa_problem_t* p, const TileArgs& a, hipStream_t stream) {
  switch (p->dtype) {
    case SPFA_DTYPE_F16: return run_global_dense<f16>(a, stream, true);
    case SPFA_DTYPE_BF16: return run_global_dense<bf16>(a, stream, true);
    case SPFA_DTYPE_F32: return run_global_dense<float>(a, stream, true);
  }
  return -1;
}

}  // namespace

/* ------------------------------------------------------------------------------ window + global + CSR */
size_t spfa_window_global_csr_workspace_bytes(int64_t n, int64_t d, int dtype, int64_t local_size,
                                              int64_t n_globals, int64_t nnz) {
  // the three parts run one after the other on the stream and may share the bytes
  size_t need = spfa_local_workspace_bytes(n, d, dtype, local_size);
  if (n_globals > 0) {
    const size_t g = spfa_global_no_local_workspace_bytes(n, d, dtype, n_globals, local_size);
    if (g > need) need = g;
  }
  if (nnz > 0) {
    const size_t c = spfa_csr_workspace_bytes(n, nnz, d, dtype);
    if (c > need) need = c;
  }
  return need;
}

int spfa_window_global_csr_forward(const spfa_problem_t* p, int64_t local_size,
                                   const int32_t* global_inds, int64_t n_globals,
                                   const void* row_off, int row_off_bytes, const void* col_ind,
                                   int64_t nnz, void* workspace, size_t workspace_bytes,
                                   void* stream) {
  // every parameter check of the three parts, before anything is enqueued
  int rc = check_problem(p);
  if (rc) return rc;
  if (p->n_k != p->n_q) return SPFA_ERR_BAD_ARG;
  if (local_size < 0 || local_size > p->n_q - 1) return SPFA_ERR_LOCAL_SIZE;
  if (n_globals < 0 || n_globals > p->n_q) return SPFA_ERR_GLOBAL_COUNT;
  if (nnz < 0 || (nnz > 0 && row_off_bytes != 4 && row_off_bytes != 8)) return SPFA_ERR_BAD_ARG;
  rc = check_pointers(p);
  if (rc) return rc;
  if (p->n_q == 0) return SPFA_OK;
  if ((n_globals > 0 && !global_inds) || (nnz > 0 && (!row_off || !col_ind))) return SPFA_ERR_BAD_ARG;
  const size_t scale = (size_t)batch_of(p);
  rc = check_workspace(workspace, workspace_bytes,
                       scale * spfa_window_global_csr_workspace_bytes(p->n_q, p->d, p->dtype, local_size,
                                                                      n_globals, nnz));
  if (rc) return rc;

  // On the direct-to-LDS tile kernels the band kernel takes the listed tokens as further keys of
  // the rows that are not listed themselves, so those rows' state makes one round trip instead
  // of two and Q is read once; the listed tokens' own rows follow.
  bool fused = false;
  if (n_globals > 0 &&
      (p->dtype == SPFA_DTYPE_F16 || p->dtype == SPFA_DTYPE_BF16 || p->dtype == SPFA_DTYPE_F32) &&
      2 * local_size + 1 >= kBandTileMinRow && p->n_q >= kBandTileMinRow && local_size <= kTileMaxWindow) {
    const GlobalLayout lay = global_layout(p->n_q, n_globals, p->d, batch_of(p));
    char* base = (char*)workspace;
    TileArgs ag{}, ab{};
    if (global_tile_args(p, global_inds, n_globals, local_size, lay, base, &ag) &&
        tile_shape_ok(ag.t, p->dtype == SPFA_DTYPE_F32 ? 4 : 2) && band_tile_args(p, local_size, 1, 0, 0, &ab)) {
      rc = prepare_global_rows(global_inds, n_globals, p->n_q, (uint32_t*)ag.gbits, (int32_t*)ag.uq,
                               (hipStream_t)stream);
      if (rc) return rc;
      ab.globs = global_inds;
      ab.n_globs = n_globals;
      ab.gbits = ag.gbits;
      rc = p->dtype == SPFA_DTYPE_F16    ? run_band<f16>(ab, 0, (hipStream_t)stream)
           : p->dtype == SPFA_DTYPE_BF16 ? run_band<bf16>(ab, 0, (hipStream_t)stream)
                                         : run_band<float>(ab, 0, (hipStream_t)stream);
      if (rc > 0) return rc;
      if (rc == 0) {
        rc = global_rows_only(p, ag, (hipStream_t)stream);
        if (rc != 0) return rc < 0 ? SPFA_ERR_LAUNCH : rc;
        fused = true;
      }
    }
  }
  if (!fused) {
    rc = spfa_local_forward(p, local_size, workspace, workspace_bytes, stream);
    if (rc) return rc;
    if (n_globals > 0) {
      rc = spfa_global_no_local_forward(p, global_inds, n_globals, local_size, workspace, workspace_bytes,
                                        stream);
      if (rc) return rc;
    }
  }
  if (nnz > 0)
    rc = spfa_csr_forward(p, row_off, row_off_bytes, col_ind, nnz, 0, workspace, workspace_bytes, stream);
  return rc;
}

/* ------------------------------------------------------------------------------ Gradients */
namespace {

constexpr int64_t kGradSegment = 1024;  // candidates one wavefront takes of an owner row

// q, k, v, m, l, out of a finished forward state plus the four gradient tensors.
int check_grads(const spfa_problem_t* p, const spfa_grads_t* g) {
  if (g == nullptr) return SPFA_ERR_BAD_ARG;
  int rc = check_pointers(p);
  if (rc) return rc;
  if (p->n_q == 0) return SPFA_OK;
  if (!g->d_out || !g->d_q || !g->d_k || !g->d_v) return SPFA_ERR_BAD_ARG;
  return SPFA_OK;
}

Grads make_grads(const spfa_grads_t* g) { return Grads{g->d_out, g->d_q, g->d_k, g->d_v}; }

// Owners (query rows in the query pass, key rows in the key pass) with more candidates than this
// leave their segments on the work list of the pass instead of walking them with their own
// wavefront.  Explicit masks, whole gradient call with 128 / 256 / 512 / 1024: the Zipf mask of
// 131 K rows 1.43 / 1.34 / 1.36 / 1.40 ms fp32 and 1.06 / 1.00 / 1.00 / 1.02 ms bf16, the COO mask
// of 1 M rows 9.40 / 9.09 / 8.90 / 8.80 ms.  The implicit masks' rows are all about equally long,
// so a wavefront per row keeps the device busy whatever their length: only what is longer than a
// segment is shared out.
constexpr int64_t kGradOwnExplicit = 512;
constexpr int64_t kGradOwnImplicit = kGradSegment;

// Most work items one pass can leave behind, per problem, and the limit that goes with the count.
struct ItemsBound {
  int64_t items;
  int64_t own_max;
  int64_t seg;
};
// Segments of an explicit mask: half as long below 32 M entries, where a call is short enough for
// the length of one wavefront's walk to show (whole gradient call of the Zipf mask at 8192 /
// 16384 / 65536 / 131072 tokens with 1024 -> 512: 0.275 -> 0.237, 0.307 -> 0.262, 0.715 -> 0.672,
// 1.332 -> 1.324 ms fp32; 256: 0.219, 0.263, 0.656, 1.459; the COO mask of 50 M entries 9.21 -> 9.35
// -> 9.64 ms).
constexpr int64_t kGradSegmentShort = 512;
int64_t explicit_grad_segment(int64_t nnz) { return nnz < ((int64_t)1 << 25) ? kGradSegmentShort : kGradSegment; }
int64_t grad_items_of(int64_t deg, int64_t own_max) {
  return deg > own_max ? (deg + kGradSegment - 1) / kGradSegment : 0;
}
ItemsBound explicit_items_bound(int64_t nnz) {
  // every owner of more than own_max candidates: deg / seg + 1 items at most, nnz / (own_max + 1) such owners
  const int64_t seg = explicit_grad_segment(nnz);
  return ItemsBound{nnz / seg + nnz / (kGradOwnExplicit + 1), kGradOwnExplicit, seg};
}
ItemsBound uniform_items_bound(int64_t n_rows, int64_t max_deg) {
  return ItemsBound{n_rows * grad_items_of(max_deg, kGradOwnImplicit), kGradOwnImplicit, kGradSegment};
}
ItemsBound global_items_bound(int64_t n, int64_t n_globals) {
  return ItemsBound{n_globals * grad_items_of(n, kGradOwnImplicit) + n * grad_items_of(n_globals, kGradOwnImplicit),
                    kGradOwnImplicit, kGradSegment};
}

// Workspace of a gradient call: lse and delta of every query row (apart and side by side), the counters and the
// work lists of the two passes (as appended and in hand-out order), then whatever the mask needs (`mask_bytes`).
struct GradLayout {
  size_t off_lse, off_delta, off_stat, off_cnt, off_phases, off_items, off_mask, total;
  uint32_t cap_items;
  int32_t own_max;
  int32_t seg;
  bool ok;
};

GradLayout grad_layout(int64_t n_q, int64_t n_batch, ItemsBound bound, size_t mask_bytes) {
  GradLayout g{};
  const int64_t b = n_batch > 1 ? n_batch : 1;
  const int64_t cap = bound.items * b + 1;
  g.ok = cap < ((int64_t)1 << 31);
  g.cap_items = (uint32_t)(g.ok ? cap : 1);
  g.own_max = (int32_t)bound.own_max;
  g.seg = (int32_t)bound.seg;
  size_t off = 0;
  g.off_lse = off;    off = align_up(off + (size_t)(n_q * b) * 4, 256);
  g.off_delta = off;  off = align_up(off + (size_t)(n_q * b) * 4, 256);
  g.off_stat = off;   off = align_up(off + (size_t)(n_q * b) * 8, 256);
  g.off_cnt = off;    off += 2 * 256;                                  // Counters of the two passes
  g.off_phases = off; off += 2 * align_up(sizeof(Phases), 256);
  // (a call that leaves no items - cap_items == 1 - never touches the lists)
  g.off_items = off;  off = align_up(off + 4 * align_up((size_t)g.cap_items * sizeof(Item), 256), 256);
  g.off_mask = off;   off = align_up(off + mask_bytes, 256);
  g.total = off;
  return g;
}

// what the transposed explicit mask needs: the entry list (rows, columns) and the conversion
struct TransposeLayout {
  size_t off_rows, off_cols, off_coo, total;
};
TransposeLayout transpose_layout(int64_t n_k, int64_t nnz) {
  TransposeLayout t{};
  size_t off = 0;
  t.off_rows = off; off = align_up(off + (size_t)nnz * 4, 256);
  t.off_cols = off; off = align_up(off + (size_t)nnz * 4, 256);
  t.off_coo = off;  off = align_up(off + coo_workspace(n_k, nnz).total, 256);
  t.total = off;
  return t;
}

GradArgs make_grad_args(const spfa_problem_t* p, const spfa_grads_t* g, const GradLayout& lay,
                        void* workspace) {
  char* base = (char*)workspace;
  GradArgs a{};
  a.q = p->q;
  a.k = p->k;
  a.v = p->v;
  a.d_out = g->d_out;
  a.lse = (float*)(base + lay.off_lse);
  a.delta = (float*)(base + lay.off_delta);
  a.stat = (float2*)(base + lay.off_stat);
  a.d_q = (float*)g->d_q;
  a.d_k = (float*)g->d_k;
  a.d_v = (float*)g->d_v;
  a.n_q = p->n_q;
  a.n_k = p->n_k;
  a.n_batch = batch_of(p);
  a.d = (int32_t)p->d;
  a.seg = lay.seg;
  a.own_max = lay.own_max;
  const size_t list_bytes = align_up((size_t)lay.cap_items * sizeof(Item), 256);
  for (int pass = 0; pass < 2; pass++) {
    a.cnt[pass] = (Counters*)(base + lay.off_cnt + (size_t)pass * 256);
    a.phases[pass] = (Phases*)(base + lay.off_phases + (size_t)pass * align_up(sizeof(Phases), 256));
    a.listed[pass] = (Item*)(base + lay.off_items + (size_t)(2 * pass) * list_bytes);
    a.ordered[pass] = (Item*)(base + lay.off_items + (size_t)(2 * pass + 1) * list_bytes);
  }
  a.cap_items = lay.cap_items;
  a.status = device_status_word();
  // (explicit masks whose gathered tensors - K, V in the query pass, Q, dO in the key pass - stay in the caches)
  a.items_on_grid = lay.own_max == kGradOwnExplicit &&
                    explicit_items_on_grid(p->n_k > p->n_q ? p->n_k : p->n_q, p->d, p->dtype) ? 1 : 0;
  // (Zipf mask, d = 64, gradient call with and without the two order_kernel launches, fp32 / bf16:
  // 8192 tokens 0.197 -> 0.191 / 0.148 -> 0.140 ms, 16384 tokens 0.226 -> 0.220 / 0.188 -> 0.182,
  // 32768 tokens 0.347 -> 0.352 / 0.273 -> 0.278)
  a.items_as_listed = lay.own_max == kGradOwnExplicit &&
                      explicit_items_as_listed(p->n_k > p->n_q ? p->n_k : p->n_q, p->d, p->dtype) ? 1 : 0;
  return a;
}

// The transposed mask of `rows` (a CsrMask over n_q query rows) built in `mbase`
// (transpose_layout() bytes): on return `out` reads it by key row.
int transpose_mask(const CsrMask& rows, int64_t n_q, int64_t n_k, int64_t nnz, char* mbase,
                   hipStream_t stream, CooCsr* tr, const uint32_t** entry_rows) {
  const TransposeLayout tl = transpose_layout(n_k, nnz);
  uint32_t* e_rows = (uint32_t*)(mbase + tl.off_rows);
  uint32_t* e_cols = (uint32_t*)(mbase + tl.off_cols);
  int rc = csr_entry_list(rows.row_off, rows.off64, rows.cols, rows.alt_cols, rows.use_alt, n_q, nnz, e_rows,
                          e_cols, stream);
  if (rc) return rc;
  const CooWorkspace cw = coo_workspace(n_k, nnz);
  *entry_rows = e_rows;
  return coo_to_csr(e_cols, 0, e_rows, nnz, n_k, n_q, mbase + tl.off_coo, mbase + tl.off_coo + cw.keep_total,
                    stream, tr);
}

// Gradients through an explicit mask given as a CsrMask over the query rows: the two passes, the
// key pass over `given_cols` when the caller brought the transposed mask, else over one built here.
int explicit_backward(const spfa_problem_t* p, const spfa_grads_t* g, const CsrMask& rows, int64_t nnz,
                      const CsrMask* given_cols, const GradLayout& lay, void* workspace,
                      hipStream_t stream) {
  if (is_f64(p)) return run_backward_csr(p->dtype, make_tensors(p), rows, make_grads(g), stream);
  CsrMask cols{};
  if (given_cols != nullptr) {
    cols = *given_cols;
  } else {
    CooCsr tr{};
    const uint32_t* e_rows = nullptr;
    int rc = transpose_mask(rows, p->n_q, p->n_k, nnz, (char*)workspace + lay.off_mask, stream, &tr, &e_rows);
    if (rc) return rc;
    cols = CsrMask{tr.row_off, e_rows, 0, tr.cols, tr.unsorted, nnz, p->n_q};
  }
  const GradArgs a = make_grad_args(p, g, lay, workspace);
  const Tensors t = make_tensors(p);
  switch (p->dtype) {
    case SPFA_DTYPE_F32: return run_grad_csr<float>(t, a, rows, cols, stream);
    case SPFA_DTYPE_F16: return run_grad_csr<f16>(t, a, rows, cols, stream);
    case SPFA_DTYPE_BF16: return run_grad_csr<bf16>(t, a, rows, cols, stream);
  }
  return SPFA_ERR_UNSUPPORTED;
}

// tiles: whether the rows are long enough for the dense-tile kernels (the forward call's rule)
int stride_backward(const spfa_problem_t* p, const spfa_grads_t* g, const StrideMask& mask, bool tiles,
                    const GradLayout& lay, void* workspace, hipStream_t stream) {
  if (is_f64(p)) return run_backward_stride(p->dtype, make_tensors(p), mask, make_grads(g), stream);
  const GradArgs a = make_grad_args(p, g, lay, workspace);
  const Tensors t = make_tensors(p);
  TileArgs ta{};
  if (tiles && band_tile_args(p, mask.w, mask.s, mask.block, mask.cnt, &ta)) {
    int rc = -1;
    switch (p->dtype) {
      case SPFA_DTYPE_F32: rc = run_band_grad<float>(ta, a, stream); break;
      case SPFA_DTYPE_F16: rc = run_band_grad<f16>(ta, a, stream); break;
      case SPFA_DTYPE_BF16: rc = run_band_grad<bf16>(ta, a, stream); break;
    }
    if (rc >= 0) return rc;
  }
  switch (p->dtype) {
    case SPFA_DTYPE_F32: return run_grad_stride<float>(t, a, mask, stream);
    case SPFA_DTYPE_F16: return run_grad_stride<f16>(t, a, mask, stream);
    case SPFA_DTYPE_BF16: return run_grad_stride<bf16>(t, a, mask, stream);
  }
  return SPFA_ERR_UNSUPPORTED;
}

// bit map of listed tokens, their distinct list, and the partial sums of the listed tokens'
// passes: [problem][split][half][dK or dV][listed token][d] floats
size_t global_grad_partial_bytes(int64_t n, int64_t n_globals, int64_t d, int64_t n_batch) {
  const GlobalLayout fl = global_layout(n, n_globals, d, 1);
  return (size_t)(n_batch > 1 ? n_batch : 1) * (size_t)fl.n_split * 4 * (size_t)n_globals * (size_t)d * 4;
}
size_t global_mask_bytes(int64_t n, int64_t n_globals, int64_t d, int64_t n_batch) {
  return align_up(global_bits_words(n) * 4, 256) + align_up((size_t)n_globals * 4, 256) +
         align_up(global_grad_partial_bytes(n, n_globals, d, n_batch), 256);
}

}  // namespace

size_t spfa_csr_backward_workspace_bytes(int64_t n_q, int64_t n_k, int64_t nnz, int64_t d, int dtype,
                                         int64_t n_batch) {
  (void)d;
  (void)dtype;
  if (n_q < 0 || n_k < 0 || nnz < 0) return 0;
  return grad_layout(n_q, n_batch, explicit_items_bound(nnz), transpose_layout(n_k, nnz).total).total;
}

int spfa_csr_backward(const spfa_problem_t* p, const spfa_grads_t* g, const void* row_off,
                      int row_off_bytes, const void* col_ind, int64_t nnz, const uint32_t* t_row_off,
                      const uint32_t* t_col_ind, void* workspace, size_t workspace_bytes, void* stream) {
  int rc = check_problem(p);
  if (rc) return rc;
  if (nnz < 0 || nnz >= (int64_t)1 << 31 || (row_off_bytes != 4 && row_off_bytes != 8))
    return SPFA_ERR_BAD_ARG;
  if ((t_row_off == nullptr) != (t_col_ind == nullptr)) return SPFA_ERR_BAD_ARG;
  rc = check_grads(p, g);
  if (rc) return rc;
  if (p->n_q == 0 || nnz == 0) return SPFA_OK;
  if (!row_off || !col_ind) return SPFA_ERR_BAD_ARG;
  const bool given = t_row_off != nullptr;
  const GradLayout lay = grad_layout(p->n_q, batch_of(p), explicit_items_bound(nnz),
                                     given ? 0 : transpose_layout(p->n_k, nnz).total);
  if (!lay.ok) return SPFA_ERR_BAD_ARG;
  rc = check_workspace(workspace, workspace_bytes, lay.total);
  if (rc) return rc;
  CsrMask rows{row_off, (const uint32_t*)col_ind, row_off_bytes == 8 ? 1 : 0, nullptr, nullptr, nnz, p->n_k};
  CsrMask cols{t_row_off, t_col_ind, 0, nullptr, nullptr, nnz, p->n_q};
  return explicit_backward(p, g, rows, nnz, given ? &cols : nullptr, lay, workspace,
                           (hipStream_t)stream);
}

size_t spfa_csr_transpose_workspace_bytes(int64_t n_q, int64_t n_k, int64_t nnz) {
  if (n_q < 0 || n_k < 0 || nnz < 0) return 0;
  return transpose_layout(n_k, nnz).total;
}

int spfa_csr_transpose(int64_t n_q, int64_t n_k, const void* row_off, int row_off_bytes,
                       const void* col_ind, int64_t nnz, uint32_t* t_row_off, uint32_t* t_col_ind,
                       void* workspace, size_t workspace_bytes, void* stream) {
  if (n_q < 0 || n_k < 0 || n_k >= (int64_t)1 << 31 || n_q >= (int64_t)1 << 31 || nnz < 0 ||
      nnz >= (int64_t)1 << 31 || (row_off_bytes != 4 && row_off_bytes != 8))
    return SPFA_ERR_BAD_ARG;
  if (!t_row_off || (nnz > 0 && (!row_off || !col_ind || !t_col_ind))) return SPFA_ERR_BAD_ARG;
  int rc = check_workspace(workspace, workspace_bytes, transpose_layout(n_k, nnz).total);
  if (rc) return rc;
  CsrMask rows{row_off, (const uint32_t*)col_ind, row_off_bytes == 8 ? 1 : 0, nullptr, nullptr, nnz, n_k};
  CooCsr tr{};
  const uint32_t* e_rows = nullptr;
  rc = transpose_mask(rows, n_q, n_k, nnz, (char*)workspace, (hipStream_t)stream, &tr, &e_rows);
  if (rc) return rc;
  return coo_csr_export(tr, e_rows, n_k, nnz, t_row_off, t_col_ind, (hipStream_t)stream);
}

size_t spfa_coo_to_csr_workspace_bytes(int64_t n_rows, int64_t nnz) {
  if (n_rows < 0 || nnz < 0) return 0;
  return coo_workspace(n_rows, nnz).total;
}

int spfa_coo_to_csr(int64_t n_rows, const void* row_ind, int row_ind_bytes, const void* col_ind, int64_t nnz,
                    uint32_t* row_off, uint32_t* csr_col_ind, void* workspace, size_t workspace_bytes,
                    void* stream) {
  if (n_rows < 0 || n_rows >= (int64_t)1 << 31 || nnz < 0 || nnz >= (int64_t)1 << 31 ||
      (row_ind_bytes != 4 && row_ind_bytes != 8))
    return SPFA_ERR_BAD_ARG;
  if (!row_off || (nnz > 0 && (!row_ind || !col_ind || !csr_col_ind))) return SPFA_ERR_BAD_ARG;
  const CooWorkspace cw = coo_workspace(n_rows, nnz);
  int rc = check_workspace(workspace, workspace_bytes, cw.total);
  if (rc) return rc;
  CooCsr csr{};
  rc = coo_to_csr(row_ind, row_ind_bytes == 8 ? 1 : 0, (const uint32_t*)col_ind, nnz, n_rows, 0, workspace,
                  (char*)workspace + cw.keep_total, (hipStream_t)stream, &csr);
  if (rc) return rc;
  return coo_csr_export(csr, (const uint32_t*)col_ind, n_rows, nnz, row_off, csr_col_ind, (hipStream_t)stream);
}

size_t spfa_coo_backward_workspace_bytes(int64_t n_q, int64_t n_k, int64_t nnz, int64_t d, int dtype,
                                         int64_t n_batch) {
  (void)d;
  (void)dtype;
  if (n_q < 0 || n_k < 0 || nnz < 0) return 0;
  const size_t mask_bytes = align_up(coo_workspace(n_q, nnz).total, 256) + transpose_layout(n_k, nnz).total;
  return grad_layout(n_q, n_batch, explicit_items_bound(nnz), mask_bytes).total;
}

int spfa_coo_backward(const spfa_problem_t* p, const spfa_grads_t* g, const void* row_ind,
                      int row_ind_bytes, const void* col_ind, int64_t nnz, void* workspace,
                      size_t workspace_bytes, void* stream) {
  int rc = check_problem(p);
  if (rc) return rc;
  if (nnz < 0 || nnz >= (int64_t)1 << 31 || (row_ind_bytes != 4 && row_ind_bytes != 8))
    return SPFA_ERR_BAD_ARG;
  rc = check_grads(p, g);
  if (rc) return rc;
  if (p->n_q == 0 || nnz == 0) return SPFA_OK;
  if (!row_ind || !col_ind) return SPFA_ERR_BAD_ARG;
  const CooWorkspace cw = coo_workspace(p->n_q, nnz);
  const size_t fwd_bytes = align_up(cw.total, 256);
  GradLayout lay = grad_layout(p->n_q, batch_of(p), explicit_items_bound(nnz),
                               fwd_bytes + transpose_layout(p->n_k, nnz).total);
  if (!lay.ok) return SPFA_ERR_BAD_ARG;
  rc = check_workspace(workspace, workspace_bytes, lay.total);
  if (rc) return rc;
  // the mask by query row first (as the forward call does), then as an explicit CSR mask
  char* fwd = (char*)workspace + lay.off_mask;
  CooCsr csr{};
  rc = coo_to_csr(row_ind, row_ind_bytes == 8 ? 1 : 0, (const uint32_t*)col_ind, nnz, p->n_q, p->n_k, fwd,
                  fwd + cw.keep_total, (hipStream_t)stream, &csr);
  if (rc) return rc;
  CsrMask rows{csr.row_off, (const uint32_t*)col_ind, 0, csr.cols, csr.unsorted, nnz, p->n_k};
  lay.off_mask += fwd_bytes;
  return explicit_backward(p, g, rows, nnz, nullptr, lay, workspace, (hipStream_t)stream);
}

size_t spfa_local_backward_workspace_bytes(int64_t n, int64_t d, int dtype, int64_t local_size,
                                           int64_t n_batch) {
  (void)d;
  (void)dtype;
  if (n < 1 || local_size < 0) return 0;
  return grad_layout(n, n_batch, uniform_items_bound(n, band_max_deg(n, local_size)), 0).total;
}

int spfa_local_backward(const spfa_problem_t* p, const spfa_grads_t* g, int64_t local_size,
                        void* workspace, size_t workspace_bytes, void* stream) {
  return spfa_local_1d_dilated_backward(p, g, local_size, 0, workspace, workspace_bytes, stream);
}

size_t spfa_local_1d_dilated_backward_workspace_bytes(int64_t n, int64_t d, int dtype,
                                                      int64_t local_size, int64_t dil_factor,
                                                      int64_t n_batch) {
  (void)dil_factor;
  return spfa_local_backward_workspace_bytes(n, d, dtype, local_size, n_batch);
}

int spfa_local_1d_dilated_backward(const spfa_problem_t* p, const spfa_grads_t* g,
                                   int64_t local_size, int64_t dil_factor, void* workspace,
                                   size_t workspace_bytes, void* stream) {
  int rc = check_problem(p);
  if (rc) return rc;
  if (local_size < 0 || local_size > p->n_q - 1) return SPFA_ERR_LOCAL_SIZE;
  if (dil_factor < 0) return SPFA_ERR_DILATION_NEG;
  if (dil_factor >= (int64_t)1 << 31) return SPFA_ERR_BAD_ARG;
  rc = check_grads(p, g);
  if (rc) return rc;
  if (p->n_k != p->n_q) return SPFA_ERR_BAD_ARG;
  const int64_t n = p->n_q;
  const GradLayout lay =
      grad_layout(n, batch_of(p), uniform_items_bound(n, band_max_deg(n, local_size)), 0);
  if (!lay.ok) return SPFA_ERR_BAD_ARG;
  rc = check_workspace(workspace, workspace_bytes, lay.total);
  if (rc) return rc;
  StrideMask mask{n, local_size, dil_factor + 1, 0, 0};
  const int64_t len_max = (n + dil_factor) / (dil_factor + 1);
  const int64_t span = 2 * local_size + 1 < len_max ? 2 * local_size + 1 : len_max;
  const bool tiles = span >= window_tile_min_row(p, true) && local_size <= kTileMaxWindow;
  return stride_backward(p, g, mask, tiles, lay, workspace, (hipStream_t)stream);
}

size_t spfa_local_2d_dilated_backward_workspace_bytes(int64_t n, int64_t d, int dtype,
                                                      int64_t block_size, int64_t dil_factor,
                                                      int64_t n_batch) {
  (void)d;
  (void)dtype;
  if (n < 1 || block_size < 1 || dil_factor < 0) return 0;
  return grad_layout(n, n_batch, uniform_items_bound(n, block_live_count(block_size, dil_factor + 1)), 0)
      .total;
}

int spfa_local_2d_dilated_backward(const spfa_problem_t* p, const spfa_grads_t* g,
                                   int64_t block_size, int64_t dil_factor, void* workspace,
                                   size_t workspace_bytes, void* stream) {
  int rc = check_problem(p);
  if (rc) return rc;
  if (block_size <= 0 || p->n_q % block_size != 0) return SPFA_ERR_BLOCK_DIVISOR;
  if (dil_factor < 0) return SPFA_ERR_DILATION_NEG;
  if (block_size / (dil_factor + 1) < 1) return SPFA_ERR_BLOCK_DILATION;
  rc = check_grads(p, g);
  if (rc) return rc;
  if (p->n_k != p->n_q) return SPFA_ERR_BAD_ARG;
  const int64_t n = p->n_q;
  if (n == 0) return SPFA_OK;
  const int64_t cnt = block_live_count(block_size, dil_factor + 1);
  const GradLayout lay = grad_layout(n, batch_of(p), uniform_items_bound(n, cnt), 0);
  if (!lay.ok) return SPFA_ERR_BAD_ARG;
  rc = check_workspace(workspace, workspace_bytes, lay.total);
  if (rc) return rc;
  StrideMask mask{n, 0, dil_factor + 1, block_size, cnt};
  return stride_backward(p, g, mask, cnt >= kBandTileMinRow, lay, workspace, (hipStream_t)stream);
}

size_t spfa_global_no_local_backward_workspace_bytes(int64_t n, int64_t d, int dtype,
                                                     int64_t n_globals, int64_t local_size,
                                                     int64_t n_batch) {
  (void)dtype;
  (void)local_size;
  if (n < 1 || n_globals < 1 || d < 1) return 0;
  return grad_layout(n, n_batch, global_items_bound(n, n_globals), global_mask_bytes(n, n_globals, d, n_batch))
      .total;
}

int spfa_global_no_local_backward(const spfa_problem_t* p, const spfa_grads_t* g,
                                  const int32_t* global_inds, int64_t n_globals,
                                  int64_t local_size, void* workspace, size_t workspace_bytes,
                                  void* stream) {
  int rc = check_problem(p);
  if (rc) return rc;
  if (n_globals <= 0 || n_globals > p->n_q) return SPFA_ERR_GLOBAL_COUNT;
  if (local_size < 0 || local_size > p->n_q - 1) return SPFA_ERR_LOCAL_SIZE;
  rc = check_grads(p, g);
  if (rc) return rc;
  if (!global_inds || p->n_k != p->n_q) return SPFA_ERR_BAD_ARG;
  const int64_t n = p->n_q;
  const GradLayout lay = grad_layout(n, batch_of(p), global_items_bound(n, n_globals),
                                     global_mask_bytes(n, n_globals, p->d, batch_of(p)));
  if (!lay.ok) return SPFA_ERR_BAD_ARG;
  rc = check_workspace(workspace, workspace_bytes, lay.total);
  if (rc) return rc;
  char* mbase = (char*)workspace + lay.off_mask;
  uint32_t* bits = (uint32_t*)mbase;
  int32_t* uq = (int32_t*)(mbase + align_up(global_bits_words(n) * 4, 256));
  rc = prepare_global_rows(global_inds, n_globals, n, bits, uq, (hipStream_t)stream);
  if (rc) return rc;
  GlobalMask rows{n, local_size, global_inds, n_globals, bits};
  if (is_f64(p))
    return run_backward_global(p->dtype, make_tensors(p), rows, make_grads(g), (hipStream_t)stream);
  GlobalColMask cols{n, local_size, global_inds, n_globals, bits, uq, bits + (global_bits_words(n) - 1)};
  const GradArgs a = make_grad_args(p, g, lay, workspace);
  const Tensors t = make_tensors(p);
  {
    // dense tiles when the shape allows it (the forward call's rule); the streamed range of the
    // listed tokens' pass is split as in the forward pass
    const GlobalLayout fl = global_layout(n, n_globals, p->d, 1);
    TileArgs ta{};
    ta.t = t;
    ta.n = n;
    ta.w = local_size;
    ta.s = 1;
    ta.globs = global_inds;
    ta.n_globs = n_globals;
    ta.gbits = bits;
    ta.uq = uq;
    ta.n_uq = bits + (global_bits_words(n) - 1);
    ta.key_run = fl.key_run;
    ta.n_split = fl.n_split;
    ta.pacc = (float*)(mbase + align_up(global_bits_words(n) * 4, 256) + align_up((size_t)n_globals * 4, 256));
    const int64_t q_tiles = (n_globals + 127) / 128;
    if (q_tiles * fl.n_split * batch_of(p) < ((int64_t)1 << 31) && batch_of(p) < 65536 &&
        local_size <= kTileMaxWindow && n * batch_of(p) * p->d < ((int64_t)1 << 40)) {
      rc = -1;
      switch (p->dtype) {
        case SPFA_DTYPE_F32: rc = run_global_grad_dense<float>(ta, a, (hipStream_t)stream); break;
        case SPFA_DTYPE_F16: rc = run_global_grad_dense<f16>(ta, a, (hipStream_t)stream); break;
        case SPFA_DTYPE_BF16: rc = run_global_grad_dense<bf16>(ta, a, (hipStream_t)stream); break;
      }
      if (rc >= 0) return rc;
    }
  }
  switch (p->dtype) {
    case SPFA_DTYPE_F32: return run_grad_global<float>(t, a, rows, cols, (hipStream_t)stream);
    case SPFA_DTYPE_F16: return run_grad_global<f16>(t, a, rows, cols, (hipStream_t)stream);
    case SPFA_DTYPE_BF16: return run_grad_global<bf16>(t, a, rows, cols, (hipStream_t)stream);
  }
  return SPFA_ERR_UNSUPPORTED;
}

/* window + global + CSR: the three gradient calls behind one entry point, like the forward one */
size_t spfa_window_global_csr_backward_workspace_bytes(int64_t n, int64_t d, int dtype,
                                                       int64_t local_size, int64_t n_globals,
                                                       int64_t nnz, int64_t n_batch) {
  size_t need = spfa_local_backward_workspace_bytes(n, d, dtype, local_size, n_batch);
  if (n_globals > 0) {
    const size_t g = spfa_global_no_local_backward_workspace_bytes(n, d, dtype, n_globals, local_size, n_batch);
    if (g > need) need = g;
  }
  if (nnz > 0) {
    const size_t c = spfa_csr_backward_workspace_bytes(n, n, nnz, d, dtype, n_batch);
    if (c > need) need = c;
  }
  return need;
}

int spfa_window_global_csr_backward(const spfa_problem_t* p, const spfa_grads_t* g, int64_t local_size,
                                    const int32_t* global_inds, int64_t n_globals, const void* row_off,
                                    int row_off_bytes, const void* col_ind, int64_t nnz,
                                    const uint32_t* t_row_off, const uint32_t* t_col_ind, void* workspace,
                                    size_t workspace_bytes, void* stream) {
  // every parameter check of the three parts, before anything is enqueued
  int rc = check_problem(p);
  if (rc) return rc;
  if (p->n_k != p->n_q) return SPFA_ERR_BAD_ARG;
  if (local_size < 0 || local_size > p->n_q - 1) return SPFA_ERR_LOCAL_SIZE;
  if (n_globals < 0 || n_globals > p->n_q) return SPFA_ERR_GLOBAL_COUNT;
  if (nnz < 0 || (nnz > 0 && row_off_bytes != 4 && row_off_bytes != 8)) return SPFA_ERR_BAD_ARG;
  if ((t_row_off == nullptr) != (t_col_ind == nullptr)) return SPFA_ERR_BAD_ARG;
  rc = check_grads(p, g);
  if (rc) return rc;
  if (p->n_q == 0) return SPFA_OK;
  if ((n_globals > 0 && !global_inds) || (nnz > 0 && (!row_off || !col_ind))) return SPFA_ERR_BAD_ARG;
  rc = check_workspace(workspace, workspace_bytes,
                       spfa_window_global_csr_backward_workspace_bytes(p->n_q, p->d, p->dtype, local_size,
                                                                       n_globals, nnz, batch_of(p)));
  if (rc) return rc;
  rc = spfa_local_backward(p, g, local_size, workspace, workspace_bytes, stream);
  if (rc) return rc;
  if (n_globals > 0) {
    rc = spfa_global_no_local_backward(p, g, global_inds, n_globals, local_size, workspace, workspace_bytes,
                                       stream);
    if (rc) return rc;
  }
  if (nnz > 0)
    rc = spfa_csr_backward(p, g, row_off, row_off_bytes, col_ind, nnz, t_row_off, t_col_ind, workspace,
                           workspace_bytes, stream);
  return rc;
}

}  // extern "C"
