// spfa_csr_forward_static: the CSR call for callers that cannot allocate device memory (code
// under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  The scratch
// the attention kernels need - work list, counters and partial results, what spfa_csr_forward
// takes as its `workspace` argument - lives in a file-scope device array of this library instead.
//
// One array per device, held until the process ends.  Every call on a device shares that
// device's array, so two calls that overlap in time on one device (different streams, or
// different host threads) race on it; calls that follow each other on one stream do not.
// Nothing has to be cleared between calls: the kernels reset the counters they use and read
// only what the same call wrote.
#include "spfa_hip.h"

#include <hip/hip_runtime.h>

#include <mutex>

namespace {

static __device__ __align__(256) unsigned char scratch[SPFA_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
void* scratch_ptr[kMaxDevices];  // device address of `scratch` on each device, once looked up
std::mutex scratch_mutex;

// The address of this device's copy of the array.  `scratch` itself is only a host-side handle
// for the symbol; the device address comes from the runtime, once per device, with that device
// current.
int device_scratch(void** out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return SPFA_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) {
      (void)hipGetLastError();
      return SPFA_ERR_LAUNCH;
    }
    scratch_ptr[dev] = ptr;
  }
  *out = scratch_ptr[dev];
  return SPFA_OK;
}

}  // namespace

extern "C" int spfa_csr_forward_static(const spfa_problem_t* p, const void* row_off, int row_off_bytes,
                                       const void* col_ind, int64_t nnz, int use_nan, void* stream) {
  if (p == nullptr || nnz < 0) return SPFA_ERR_BAD_ARG;
  // The limit is what the call below asks of its workspace: the work list once, the partial
  // results once per problem of a batch (a batch too large for one work cursor is walked problem
  // by problem on one problem's worth).  Sizes that are not a valid problem give 0 here and are
  // rejected by the call's own checks; fp64 problems use no scratch at all.
  if (p->dtype != SPFA_DTYPE_F64) {
    const size_t need = spfa_csr_workspace_bytes_batched(p->n_q, nnz, p->d, p->dtype, p->n_batch > 1 ? p->n_batch : 1);
    if (need > (size_t)SPFA_STATIC_SCRATCH_BYTES) return SPFA_ERR_STATIC_LIMIT;
  }
  void* ptr = nullptr;
  const int rc = device_scratch(&ptr);
  if (rc) return rc;
  return spfa_csr_forward(p, row_off, row_off_bytes, col_ind, nnz, use_nan, ptr,
                          (size_t)SPFA_STATIC_SCRATCH_BYTES, stream);
}
