// Shared host-side glue of the six spfa_* Python modules: the reference bindings' tensor checks,
// the translation torch tensor -> C-ABI problem description, workspace allocation through torch's
// allocator, the current HIP stream, and status -> exception mapping.  No device code here.
#pragma once

#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/extension.h>

#include <stdexcept>

#include "spfa_hip.h"

// Same checks and texts as the reference bindings (sp_flatt_csr.cpp:7-9).
#define CHECK_CUDA(x) TORCH_CHECK(x.device().is_cuda(), #x " must be a CUDA tensor")
#define CHECK_CONTIGUOUS(x) TORCH_CHECK(x.is_contiguous(), #x " must be contiguous")
#define CHECK_INPUT(x) \
  CHECK_CUDA(x);       \
  CHECK_CONTIGUOUS(x)

namespace spfa_ext {

inline int elem_dtype(const torch::Tensor& t) {
  switch (t.scalar_type()) {
    case torch::kFloat32: return SPFA_DTYPE_F32;
    case torch::kFloat16: return SPFA_DTYPE_F16;
    case torch::kBFloat16: return SPFA_DTYPE_BF16;
    case torch::kFloat64: return SPFA_DTYPE_F64;
    default: return -1;  // reported by the library after the parameter checks
  }
}

// Width in bytes of an integer index tensor; signed and unsigned are bit-identical in range.
inline int index_bytes(const torch::Tensor& t, const char* name, bool allow_wide) {
  switch (t.scalar_type()) {
    case torch::kInt32:
    case torch::kUInt32: return 4;
    case torch::kInt64:
    case torch::kUInt64:
      TORCH_CHECK(allow_wide, name, " must be a 32-bit integer tensor");
      return 8;
    default: TORCH_CHECK(false, name, " must be an integer index tensor (got ", t.scalar_type(), ")");
  }
  return 0;
}

// Q, K, V, O are [tokens, embedding] as in the reference, or carry leading batch dimensions
// ([batch, tokens, embedding], [batch, heads, tokens, embedding], ...) with m and l shaped like
// Q without its last dimension: independent problems that share the mask.
inline spfa_problem_t make_problem(const torch::Tensor& Q, const torch::Tensor& K,
                                   const torch::Tensor& V, const torch::Tensor& m,
                                   const torch::Tensor& l, const torch::Tensor& O) {
  const int64_t nd = Q.dim();
  TORCH_CHECK(nd >= 2 && K.dim() == nd && V.dim() == nd && O.dim() == nd,
              "Q, K, V and O must be [tokens, embedding], optionally with the same leading batch dimensions");
  TORCH_CHECK(m.dim() == nd - 1 && l.dim() == nd - 1, "m and l must be shaped like Q without its last dimension");
  for (int64_t i = 0; i + 2 < nd; i++)
    TORCH_CHECK(K.size(i) == Q.size(i) && V.size(i) == Q.size(i) && O.size(i) == Q.size(i) &&
                    m.size(i) == Q.size(i) && l.size(i) == Q.size(i),
                "all tensors must share the leading batch dimensions");
  const int64_t rq = nd - 2, rd = nd - 1;
  TORCH_CHECK(K.size(rd) == Q.size(rd) && V.size(rd) == Q.size(rd) && O.size(rd) == Q.size(rd),
              "Q, K, V and O must share the embedding dimension");
  TORCH_CHECK(K.size(rq) == V.size(rq), "K and V must have the same number of rows");
  TORCH_CHECK(O.size(rq) == Q.size(rq) && m.size(rq) == Q.size(rq) && l.size(rq) == Q.size(rq),
              "O, m and l must have one row per row of Q");
  TORCH_CHECK(K.scalar_type() == Q.scalar_type() && V.scalar_type() == Q.scalar_type() &&
                  O.scalar_type() == Q.scalar_type(),
              "Q, K, V and O must have the same dtype");
  TORCH_CHECK(m.scalar_type() == l.scalar_type() &&
                  (m.scalar_type() == Q.scalar_type() || m.scalar_type() == torch::kFloat32),
              "m and l must have the dtype of Q (or float32)");
  TORCH_CHECK(K.device() == Q.device() && V.device() == Q.device() && O.device() == Q.device() &&
                  m.device() == Q.device() && l.device() == Q.device(),
              "all tensors must be on the same device");
  int64_t batch = 1;
  for (int64_t i = 0; i + 2 < nd; i++) batch *= Q.size(i);
  spfa_problem_t p;
  p.q = Q.data_ptr();
  p.k = K.data_ptr();
  p.v = V.data_ptr();
  p.m = m.data_ptr();
  p.l = l.data_ptr();
  p.out = O.data_ptr();
  p.n_q = Q.size(rq);
  p.n_k = K.size(rq);
  p.d = Q.size(rd);
  p.dtype = elem_dtype(Q);
  p.state_dtype = (m.scalar_type() == Q.scalar_type()) ? p.dtype : SPFA_DTYPE_F32;
  p.n_batch = batch;
  return p;
}

// The gradient tensors of a backward call: d_out shaped and typed like Q; d_q like Q, d_k and d_v
// like K, all three float32 (float64 when Q is float64).  They are added to.
inline spfa_grads_t make_grads(const torch::Tensor& Q, const torch::Tensor& K, const torch::Tensor& dO,
                               const torch::Tensor& dQ, const torch::Tensor& dK,
                               const torch::Tensor& dV) {
  const auto acc = Q.scalar_type() == torch::kFloat64 ? torch::kFloat64 : torch::kFloat32;
  TORCH_CHECK(dO.sizes() == Q.sizes() && dO.scalar_type() == Q.scalar_type(),
              "dO must have the shape and dtype of Q");
  TORCH_CHECK(dQ.sizes() == Q.sizes() && dK.sizes() == K.sizes() && dV.sizes() == K.sizes(),
              "dQ must be shaped like Q, dK and dV like K");
  TORCH_CHECK(dQ.scalar_type() == acc && dK.scalar_type() == acc && dV.scalar_type() == acc,
              "dQ, dK and dV must be float32 (float64 for float64 inputs)");
  TORCH_CHECK(dO.device() == Q.device() && dQ.device() == Q.device() && dK.device() == Q.device() &&
                  dV.device() == Q.device(),
              "all tensors must be on the same device");
  spfa_grads_t g;
  g.d_out = dO.data_ptr();
  g.d_q = dQ.data_ptr();
  g.d_k = dK.data_ptr();
  g.d_v = dV.data_ptr();
  return g;
}

#define SPFA_CHECK_GRAD_INPUTS() \
  CHECK_INPUT(dO);               \
  CHECK_INPUT(dQ);               \
  CHECK_INPUT(dK);               \
  CHECK_INPUT(dV)

// Entry i of an integer index tensor on the device, read back to the host (synchronises).
inline int64_t index_value(const torch::Tensor& t, int64_t i) {
  const torch::Tensor x = t.narrow(0, i, 1).cpu();
  switch (x.scalar_type()) {
    case torch::kInt32: return (int64_t)*x.data_ptr<int32_t>();
    case torch::kUInt32: return (int64_t)*(const uint32_t*)x.data_ptr();
    case torch::kInt64: return *x.data_ptr<int64_t>();
    default: return (int64_t)*(const uint64_t*)x.data_ptr();
  }
}

// the status word of the current device (spfa_device_status)
inline int64_t device_status(bool reset) {
  const int bits = spfa_device_status(reset ? 1 : 0);
  TORCH_CHECK(bits >= 0, "the device status word cannot be read");
  return bits;
}

// workspace of a (possibly batched) call: the single-problem size times the batch count
inline size_t batched(size_t bytes, const spfa_problem_t& p) {
  return bytes * (size_t)(p.n_batch > 1 ? p.n_batch : 1);
}

inline torch::Tensor make_workspace(size_t bytes, const torch::Tensor& like) {
  if (bytes < 256) bytes = 256;
  return torch::empty({(int64_t)bytes}, torch::TensorOptions().dtype(torch::kUInt8).device(like.device()));
}

inline void* current_stream(const torch::Tensor& like) {
  return (void*)c10::hip::getCurrentHIPStream(like.device().index()).stream();
}

// Parameter errors keep the reference's exception type (std::invalid_argument -> ValueError) and
// text; everything else is a RuntimeError.
inline void raise_on_error(int status) {
  if (status == SPFA_OK) return;
  if (status >= SPFA_ERR_EMB_TOO_LARGE && status <= SPFA_ERR_GLOBAL_COUNT)
    throw std::invalid_argument(spfa_status_string(status));
  TORCH_CHECK(false, spfa_status_string(status), " (status ", status, ")");
}

}  // namespace spfa_ext
