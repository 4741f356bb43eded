// Python module spfa_csr: forward(q, k, v, w_row_off, w_col_ind, w_val, m, l, out, use_nan).
// Host wrapper with the reference binding's signature and checks
// (Sparse_FlashAttention_CSR/sp_flatt_csr.cpp:28-59); the work is done by spfa_csr_forward in
// libspfa_hip.so.
#include "spfa_ext_common.h"

torch::Tensor spfa_csr_forward_py(torch::Tensor Q, torch::Tensor K, torch::Tensor V,
                                  torch::Tensor W_row_off, torch::Tensor W_col_ind,
                                  torch::Tensor W_val, torch::Tensor m, torch::Tensor l,
                                  torch::Tensor O, bool use_nan) {
  CHECK_INPUT(Q);
  CHECK_INPUT(K);
  CHECK_INPUT(V);
  CHECK_INPUT(W_row_off);
  CHECK_INPUT(W_col_ind);
  CHECK_INPUT(W_val);
  CHECK_INPUT(m);
  CHECK_INPUT(l);
  CHECK_INPUT(O);

  c10::DeviceGuard guard(Q.device());
  spfa_problem_t p = spfa_ext::make_problem(Q, K, V, m, l, O);
  TORCH_CHECK(W_row_off.dim() == 1 && W_row_off.size(0) == p.n_q + 1,
              "W_row_off must hold rows+1 offsets");
  TORCH_CHECK(W_col_ind.dim() == 1, "W_col_ind must be 1-D");
  // the value vector is type-checked and otherwise unused, as in the reference kernel
  TORCH_CHECK(W_val.scalar_type() == Q.scalar_type(), "W_val must have the dtype of Q");
  const int off_bytes = spfa_ext::index_bytes(W_row_off, "W_row_off", true);
  spfa_ext::index_bytes(W_col_ind, "W_col_ind", false);
  const int64_t nnz = W_col_ind.size(0);

  const size_t ws_bytes = spfa_ext::batched(spfa_csr_workspace_bytes(p.n_q, nnz, p.d, p.dtype), p);
  torch::Tensor ws = spfa_ext::make_workspace(ws_bytes, Q);
  spfa_ext::raise_on_error(spfa_csr_forward(&p, W_row_off.data_ptr(), off_bytes, W_col_ind.data_ptr(),
                                            nnz, use_nan ? 1 : 0, ws.data_ptr(), (size_t)ws.numel(),
                                            spfa_ext::current_stream(Q)));
  return O;
}

// plan(w_row_off, w_col_ind) -> uint8 device tensor: the mask pre-pass, reusable by
// forward_planned for any number of calls with the same two mask tensors (masks are built once
// and reused by the reference's callers, verification/verify.py:68-71).
torch::Tensor spfa_csr_plan_py(torch::Tensor W_row_off, torch::Tensor W_col_ind) {
  CHECK_INPUT(W_row_off);
  CHECK_INPUT(W_col_ind);
  c10::DeviceGuard guard(W_row_off.device());
  TORCH_CHECK(W_row_off.dim() == 1 && W_row_off.size(0) >= 1, "W_row_off must hold rows+1 offsets");
  TORCH_CHECK(W_col_ind.dim() == 1, "W_col_ind must be 1-D");
  const int off_bytes = spfa_ext::index_bytes(W_row_off, "W_row_off", true);
  spfa_ext::index_bytes(W_col_ind, "W_col_ind", false);
  const int64_t n_q = W_row_off.size(0) - 1, nnz = W_col_ind.size(0);
  torch::Tensor plan = spfa_ext::make_workspace(spfa_csr_plan_bytes(n_q, nnz), W_row_off);
  spfa_ext::raise_on_error(spfa_csr_plan(n_q, W_row_off.data_ptr(), off_bytes, W_col_ind.data_ptr(), nnz,
                                         plan.data_ptr(), (size_t)plan.numel(),
                                         spfa_ext::current_stream(W_row_off)));
  return plan;
}

torch::Tensor spfa_csr_forward_planned_py(torch::Tensor Q, torch::Tensor K, torch::Tensor V,
                                          torch::Tensor W_row_off, torch::Tensor W_col_ind,
                                          torch::Tensor W_val, torch::Tensor m, torch::Tensor l,
                                          torch::Tensor O, bool use_nan, torch::Tensor plan) {
  CHECK_INPUT(Q);
  CHECK_INPUT(K);
  CHECK_INPUT(V);
  CHECK_INPUT(W_row_off);
  CHECK_INPUT(W_col_ind);
  CHECK_INPUT(W_val);
  CHECK_INPUT(m);
  CHECK_INPUT(l);
  CHECK_INPUT(O);
  CHECK_INPUT(plan);

  c10::DeviceGuard guard(Q.device());
  spfa_problem_t p = spfa_ext::make_problem(Q, K, V, m, l, O);
  TORCH_CHECK(W_row_off.dim() == 1 && W_row_off.size(0) == p.n_q + 1,
              "W_row_off must hold rows+1 offsets");
  TORCH_CHECK(W_col_ind.dim() == 1, "W_col_ind must be 1-D");
  TORCH_CHECK(W_val.scalar_type() == Q.scalar_type(), "W_val must have the dtype of Q");
  TORCH_CHECK(plan.scalar_type() == torch::kUInt8 && plan.dim() == 1, "plan must come from plan()");
  const int off_bytes = spfa_ext::index_bytes(W_row_off, "W_row_off", true);
  spfa_ext::index_bytes(W_col_ind, "W_col_ind", false);
  const int64_t nnz = W_col_ind.size(0);

  const size_t ws_bytes = spfa_ext::batched(spfa_csr_workspace_bytes(p.n_q, nnz, p.d, p.dtype), p);
  torch::Tensor ws = spfa_ext::make_workspace(ws_bytes, Q);
  spfa_ext::raise_on_error(spfa_csr_forward_planned(
      &p, W_row_off.data_ptr(), off_bytes, W_col_ind.data_ptr(), nnz, use_nan ? 1 : 0, plan.data_ptr(),
      (size_t)plan.numel(), ws.data_ptr(), (size_t)ws.numel(), spfa_ext::current_stream(Q)));
  return O;
}

// backward(<the arguments of forward, without use_nan>, dO, dQ, dK, dV) -> (dQ, dK, dV): adds the
// gradients of the attention this module's forward computes to dQ, dK, dV (float32; float64 for
// float64 inputs).  m, l, O are the finished forward state.  The reference binds no backward.
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> spfa_csr_backward_py(torch::Tensor Q, torch::Tensor K, torch::Tensor V,
                                                                   torch::Tensor W_row_off, torch::Tensor W_col_ind,
                                                                   torch::Tensor W_val, torch::Tensor m, torch::Tensor l,
                                                                   torch::Tensor O, torch::Tensor dO, torch::Tensor dQ, torch::Tensor dK, torch::Tensor dV) {
  CHECK_INPUT(Q);
  CHECK_INPUT(K);
  CHECK_INPUT(V);
  CHECK_INPUT(m);
  CHECK_INPUT(l);
  CHECK_INPUT(O);
  SPFA_CHECK_GRAD_INPUTS();
  CHECK_INPUT(W_row_off);
  CHECK_INPUT(W_col_ind);
  c10::DeviceGuard guard(Q.device());
  spfa_problem_t p = spfa_ext::make_problem(Q, K, V, m, l, O);
  spfa_grads_t g = spfa_ext::make_grads(Q, K, dO, dQ, dK, dV);
  TORCH_CHECK(W_row_off.dim() == 1 && W_row_off.size(0) == p.n_q + 1,
              "W_row_off must hold rows+1 offsets");
  TORCH_CHECK(W_col_ind.dim() == 1, "W_col_ind must be 1-D");
  (void)W_val;
  const int off_bytes = spfa_ext::index_bytes(W_row_off, "W_row_off", true);
  spfa_ext::index_bytes(W_col_ind, "W_col_ind", false);
  const int64_t nnz = W_col_ind.size(0);
  torch::Tensor ws = spfa_ext::make_workspace(
      spfa_csr_backward_workspace_bytes(p.n_q, p.n_k, nnz, p.d, p.dtype, p.n_batch), Q);
  spfa_ext::raise_on_error(spfa_csr_backward(&p, &g, W_row_off.data_ptr(), off_bytes, W_col_ind.data_ptr(),
                                             nnz, ws.data_ptr(), (size_t)ws.numel(),
                                             spfa_ext::current_stream(Q)));
  return std::make_tuple(dQ, dK, dV);
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, mod) {
  mod.def("forward", &spfa_csr_forward_py, "Sparse-FlashAttention forward, CSR mask (HIP, gfx950)");
  mod.def("plan", &spfa_csr_plan_py, "Mask pre-pass of a CSR mask, for forward_planned");
  mod.def("forward_planned", &spfa_csr_forward_planned_py,
          "forward(...) with the mask pre-pass taken from plan(...)");
  mod.def("backward", &spfa_csr_backward_py, "Gradients of forward(...), added to dQ, dK, dV");
}
