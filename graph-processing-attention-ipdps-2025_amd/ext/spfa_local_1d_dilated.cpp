// Python module spfa_local_1d_dilated: forward(q, k, v, m, l, out, LOCAL_SIZE, DILATE_FACTOR).
// Host wrapper with the reference binding's signature and checks
// (Sparse_FlashAttention_Local_1D_Dilated/sp_flatt_local_1d_dilated.cpp:26-52); the work is done
// by spfa_local_1d_dilated_forward in libspfa_hip.so.
#include "spfa_ext_common.h"

torch::Tensor spfa_local_1d_dilated_forward_py(torch::Tensor Q, torch::Tensor K, torch::Tensor V,
                                               torch::Tensor m, torch::Tensor l, torch::Tensor O,
                                               int local_size_each_dir, int dil_factor) {
  CHECK_INPUT(Q);
  CHECK_INPUT(K);
  CHECK_INPUT(V);
  CHECK_INPUT(m);
  CHECK_INPUT(l);
  CHECK_INPUT(O);

  c10::DeviceGuard guard(Q.device());
  spfa_problem_t p = spfa_ext::make_problem(Q, K, V, m, l, O);
  TORCH_CHECK(p.n_k == p.n_q, "Q, K and V must have the same number of rows");
  const size_t ws_bytes =
      spfa_ext::batched(spfa_local_1d_dilated_workspace_bytes(p.n_q, p.d, p.dtype, local_size_each_dir, dil_factor), p);
  torch::Tensor ws = spfa_ext::make_workspace(ws_bytes, Q);
  spfa_ext::raise_on_error(spfa_local_1d_dilated_forward(&p, local_size_each_dir, dil_factor,
                                                         ws.data_ptr(), (size_t)ws.numel(),
                                                         spfa_ext::current_stream(Q)));
  return O;
}

// backward(<the arguments of forward, without use_nan>, dO, dQ, dK, dV) -> (dQ, dK, dV): adds the
// gradients of the attention this module's forward computes to dQ, dK, dV (float32; float64 for
// float64 inputs).  m, l, O are the finished forward state.  The reference binds no backward.
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> spfa_local_1d_dilated_backward_py(
    torch::Tensor Q, torch::Tensor K, torch::Tensor V, torch::Tensor m, torch::Tensor l, torch::Tensor O,
    int local_size_each_dir, int dil_factor, torch::Tensor dO, torch::Tensor dQ, torch::Tensor dK, torch::Tensor dV) {
  CHECK_INPUT(Q);
  CHECK_INPUT(K);
  CHECK_INPUT(V);
  CHECK_INPUT(m);
  CHECK_INPUT(l);
  CHECK_INPUT(O);
  SPFA_CHECK_GRAD_INPUTS();
  c10::DeviceGuard guard(Q.device());
  spfa_problem_t p = spfa_ext::make_problem(Q, K, V, m, l, O);
  spfa_grads_t g = spfa_ext::make_grads(Q, K, dO, dQ, dK, dV);
  TORCH_CHECK(p.n_k == p.n_q, "Q, K and V must have the same number of rows");
  torch::Tensor ws = spfa_ext::make_workspace(
      spfa_local_1d_dilated_backward_workspace_bytes(p.n_q, p.d, p.dtype, local_size_each_dir, dil_factor,
                                                     p.n_batch), Q);
  spfa_ext::raise_on_error(spfa_local_1d_dilated_backward(&p, &g, local_size_each_dir, dil_factor,
                                                          ws.data_ptr(), (size_t)ws.numel(),
                                                          spfa_ext::current_stream(Q)));
  return std::make_tuple(dQ, dK, dV);
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, mod) {
  mod.def("forward", &spfa_local_1d_dilated_forward_py,
          "Sparse-FlashAttention forward, 1D-dilated local mask (HIP, gfx950)");
  mod.def("backward", &spfa_local_1d_dilated_backward_py, "Gradients of forward(...), added to dQ, dK, dV");
}
