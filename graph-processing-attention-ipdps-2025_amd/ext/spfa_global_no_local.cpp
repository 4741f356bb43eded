// Python module spfa_global_no_local: forward(q, k, v, m, l, out, globs, LOCAL_SIZE).
// Host wrapper with the reference binding's signature and checks
// (Sparse_FlashAttention_Global_No_Local/sp_flatt_global_no_local.cpp:26-53); the work is done by
// spfa_global_no_local_forward in libspfa_hip.so.
#include "spfa_ext_common.h"

torch::Tensor spfa_global_no_local_forward_py(torch::Tensor Q, torch::Tensor K, torch::Tensor V,
                                              torch::Tensor m, torch::Tensor l, torch::Tensor O,
                                              torch::Tensor global_inds, int local_size_each_dir) {
  CHECK_INPUT(Q);
  CHECK_INPUT(K);
  CHECK_INPUT(V);
  CHECK_INPUT(m);
  CHECK_INPUT(l);
  CHECK_INPUT(O);
  CHECK_INPUT(global_inds);

  c10::DeviceGuard guard(Q.device());
  spfa_problem_t p = spfa_ext::make_problem(Q, K, V, m, l, O);
  TORCH_CHECK(p.n_k == p.n_q, "Q, K and V must have the same number of rows");
  TORCH_CHECK(global_inds.dim() == 1, "global_inds must be 1-D");
  // the reference reads the list through an int accessor (sp_flatt_global_no_local_kernel.cu:345)
  TORCH_CHECK(global_inds.scalar_type() == torch::kInt32, "global_inds must be an int32 tensor");
  const int64_t n_globs = global_inds.size(0);
  const size_t ws_bytes =
      spfa_ext::batched(spfa_global_no_local_workspace_bytes(p.n_q, p.d, p.dtype, n_globs, local_size_each_dir), p);
  torch::Tensor ws = spfa_ext::make_workspace(ws_bytes, Q);
  spfa_ext::raise_on_error(spfa_global_no_local_forward(
      &p, (const int32_t*)global_inds.data_ptr(), n_globs, local_size_each_dir, ws.data_ptr(),
      (size_t)ws.numel(), spfa_ext::current_stream(Q)));
  return O;
}

// backward(<the arguments of forward, without use_nan>, dO, dQ, dK, dV) -> (dQ, dK, dV): adds the
// gradients of the attention this module's forward computes to dQ, dK, dV (float32; float64 for
// float64 inputs).  m, l, O are the finished forward state.  The reference binds no backward.
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> spfa_global_no_local_backward_py(
    torch::Tensor Q, torch::Tensor K, torch::Tensor V, torch::Tensor m, torch::Tensor l, torch::Tensor O,
    torch::Tensor global_inds, int local_size_each_dir, torch::Tensor dO, torch::Tensor dQ, torch::Tensor dK, torch::Tensor dV) {
  CHECK_INPUT(Q);
  CHECK_INPUT(K);
  CHECK_INPUT(V);
  CHECK_INPUT(m);
  CHECK_INPUT(l);
  CHECK_INPUT(O);
  SPFA_CHECK_GRAD_INPUTS();
  CHECK_INPUT(global_inds);
  c10::DeviceGuard guard(Q.device());
  spfa_problem_t p = spfa_ext::make_problem(Q, K, V, m, l, O);
  spfa_grads_t g = spfa_ext::make_grads(Q, K, dO, dQ, dK, dV);
  TORCH_CHECK(p.n_k == p.n_q, "Q, K and V must have the same number of rows");
  TORCH_CHECK(global_inds.dim() == 1, "global_inds must be 1-D");
  TORCH_CHECK(global_inds.scalar_type() == torch::kInt32, "global_inds must be an int32 tensor");
  const int64_t n_globs = global_inds.size(0);
  torch::Tensor ws = spfa_ext::make_workspace(
      spfa_global_no_local_backward_workspace_bytes(p.n_q, p.d, p.dtype, n_globs, local_size_each_dir,
                                                    p.n_batch), Q);
  spfa_ext::raise_on_error(spfa_global_no_local_backward(
      &p, &g, (const int32_t*)global_inds.data_ptr(), n_globs, local_size_each_dir, ws.data_ptr(),
      (size_t)ws.numel(), spfa_ext::current_stream(Q)));
  return std::make_tuple(dQ, dK, dV);
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, mod) {
  mod.def("forward", &spfa_global_no_local_forward_py,
          "Sparse-FlashAttention forward, global-minus-local mask (HIP, gfx950)");
  mod.def("backward", &spfa_global_no_local_backward_py, "Gradients of forward(...), added to dQ, dK, dV");
}
