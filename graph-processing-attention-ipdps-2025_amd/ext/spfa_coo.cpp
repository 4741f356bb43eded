// Python module spfa_coo: forward(q, k, v, w_row_ind, w_col_ind, w_val, m, l, out, use_nan).
// Host wrapper with the reference binding's signature and checks
// (Sparse_FlashAttention_COO/sp_flatt_coo.cpp:28-59); the work is done by spfa_coo_forward in
// libspfa_hip.so.  Entries may be in any order.
#include "spfa_ext_common.h"

torch::Tensor spfa_coo_forward_py(torch::Tensor Q, torch::Tensor K, torch::Tensor V,
                                  torch::Tensor W_row_ind, torch::Tensor W_col_ind,
                                  torch::Tensor W_val, torch::Tensor m, torch::Tensor l,
                                  torch::Tensor O, bool use_nan) {
  CHECK_INPUT(Q);
  CHECK_INPUT(K);
  CHECK_INPUT(V);
  CHECK_INPUT(W_row_ind);
  CHECK_INPUT(W_col_ind);
  CHECK_INPUT(W_val);
  CHECK_INPUT(m);
  CHECK_INPUT(l);
  CHECK_INPUT(O);

  c10::DeviceGuard guard(Q.device());
  spfa_problem_t p = spfa_ext::make_problem(Q, K, V, m, l, O);
  TORCH_CHECK(W_row_ind.dim() == 1 && W_col_ind.dim() == 1 &&
                  W_row_ind.size(0) == W_col_ind.size(0),
              "W_row_ind and W_col_ind must be 1-D and of equal length");
  TORCH_CHECK(W_val.scalar_type() == Q.scalar_type(), "W_val must have the dtype of Q");
  const int row_bytes = spfa_ext::index_bytes(W_row_ind, "W_row_ind", true);
  spfa_ext::index_bytes(W_col_ind, "W_col_ind", false);
  const int64_t nnz = W_col_ind.size(0);

  const size_t ws_bytes = spfa_coo_workspace_bytes_batched(p.n_q, nnz, p.d, p.dtype, p.n_batch);
  torch::Tensor ws = spfa_ext::make_workspace(ws_bytes, Q);
  spfa_ext::raise_on_error(spfa_coo_forward(&p, W_row_ind.data_ptr(), row_bytes, W_col_ind.data_ptr(),
                                            nnz, use_nan ? 1 : 0, ws.data_ptr(), (size_t)ws.numel(),
                                            spfa_ext::current_stream(Q)));
  return O;
}

// plan(w_row_ind, w_col_ind, n_rows) -> uint8 device tensor: row offsets, bucketed columns (when
// the entries are not sorted by row) and the work list, reusable by forward_planned for any
// number of calls with the same w_col_ind (masks are built once and reused by the reference's
// callers, verification/verify.py:95-98).
torch::Tensor spfa_coo_plan_py(torch::Tensor W_row_ind, torch::Tensor W_col_ind, int64_t n_rows) {
  CHECK_INPUT(W_row_ind);
  CHECK_INPUT(W_col_ind);
  c10::DeviceGuard guard(W_row_ind.device());
  TORCH_CHECK(W_row_ind.dim() == 1 && W_col_ind.dim() == 1 &&
                  W_row_ind.size(0) == W_col_ind.size(0),
              "W_row_ind and W_col_ind must be 1-D and of equal length");
  TORCH_CHECK(n_rows >= 0, "n_rows must not be negative");
  const int row_bytes = spfa_ext::index_bytes(W_row_ind, "W_row_ind", true);
  spfa_ext::index_bytes(W_col_ind, "W_col_ind", false);
  const int64_t nnz = W_col_ind.size(0);
  torch::Tensor plan = spfa_ext::make_workspace(spfa_coo_plan_bytes(n_rows, nnz), W_row_ind);
  torch::Tensor ws = spfa_ext::make_workspace(spfa_coo_plan_workspace_bytes(n_rows, nnz), W_row_ind);
  spfa_ext::raise_on_error(spfa_coo_plan(n_rows, W_row_ind.data_ptr(), row_bytes, W_col_ind.data_ptr(),
                                         nnz, plan.data_ptr(), (size_t)plan.numel(), ws.data_ptr(),
                                         (size_t)ws.numel(), spfa_ext::current_stream(W_row_ind)));
  return plan;
}

torch::Tensor spfa_coo_forward_planned_py(torch::Tensor Q, torch::Tensor K, torch::Tensor V,
                                          torch::Tensor W_row_ind, torch::Tensor W_col_ind,
                                          torch::Tensor W_val, torch::Tensor m, torch::Tensor l,
                                          torch::Tensor O, bool use_nan, torch::Tensor plan) {
  CHECK_INPUT(Q);
  CHECK_INPUT(K);
  CHECK_INPUT(V);
  CHECK_INPUT(W_row_ind);
  CHECK_INPUT(W_col_ind);
  CHECK_INPUT(W_val);
  CHECK_INPUT(m);
  CHECK_INPUT(l);
  CHECK_INPUT(O);
  CHECK_INPUT(plan);

  c10::DeviceGuard guard(Q.device());
  spfa_problem_t p = spfa_ext::make_problem(Q, K, V, m, l, O);
  TORCH_CHECK(W_row_ind.dim() == 1 && W_col_ind.dim() == 1 &&
                  W_row_ind.size(0) == W_col_ind.size(0),
              "W_row_ind and W_col_ind must be 1-D and of equal length");
  TORCH_CHECK(W_val.scalar_type() == Q.scalar_type(), "W_val must have the dtype of Q");
  TORCH_CHECK(plan.scalar_type() == torch::kUInt8 && plan.dim() == 1, "plan must come from plan()");
  spfa_ext::index_bytes(W_col_ind, "W_col_ind", false);
  const int64_t nnz = W_col_ind.size(0);

  // (the attention part of the plain call's workspace would do; the plain size is simply enough)
  const size_t ws_bytes = spfa_csr_workspace_bytes_batched(p.n_q, nnz, p.d, p.dtype, p.n_batch);
  torch::Tensor ws = spfa_ext::make_workspace(ws_bytes, Q);
  spfa_ext::raise_on_error(spfa_coo_forward_planned(
      &p, W_col_ind.data_ptr(), nnz, use_nan ? 1 : 0, plan.data_ptr(), (size_t)plan.numel(),
      ws.data_ptr(), (size_t)ws.numel(), spfa_ext::current_stream(Q)));
  return O;
}

// backward(<the arguments of forward, without use_nan>, dO, dQ, dK, dV) -> (dQ, dK, dV): adds the
// gradients of the attention this module's forward computes to dQ, dK, dV (float32; float64 for
// float64 inputs).  m, l, O are the finished forward state.  The reference binds no backward.
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> spfa_coo_backward_py(torch::Tensor Q, torch::Tensor K, torch::Tensor V,
                                                                   torch::Tensor W_row_ind, torch::Tensor W_col_ind,
                                                                   torch::Tensor W_val, torch::Tensor m, torch::Tensor l,
                                                                   torch::Tensor O, torch::Tensor dO, torch::Tensor dQ, torch::Tensor dK, torch::Tensor dV) {
  CHECK_INPUT(Q);
  CHECK_INPUT(K);
  CHECK_INPUT(V);
  CHECK_INPUT(m);
  CHECK_INPUT(l);
  CHECK_INPUT(O);
  SPFA_CHECK_GRAD_INPUTS();
  CHECK_INPUT(W_row_ind);
  CHECK_INPUT(W_col_ind);
  c10::DeviceGuard guard(Q.device());
  spfa_problem_t p = spfa_ext::make_problem(Q, K, V, m, l, O);
  spfa_grads_t g = spfa_ext::make_grads(Q, K, dO, dQ, dK, dV);
  TORCH_CHECK(W_row_ind.dim() == 1 && W_col_ind.dim() == 1 &&
                  W_row_ind.size(0) == W_col_ind.size(0),
              "W_row_ind and W_col_ind must be 1-D and of equal length");
  (void)W_val;
  const int row_bytes = spfa_ext::index_bytes(W_row_ind, "W_row_ind", true);
  spfa_ext::index_bytes(W_col_ind, "W_col_ind", false);
  const int64_t nnz = W_col_ind.size(0);
  torch::Tensor ws = spfa_ext::make_workspace(
      spfa_coo_backward_workspace_bytes(p.n_q, p.n_k, nnz, p.d, p.dtype, p.n_batch), Q);
  spfa_ext::raise_on_error(spfa_coo_backward(&p, &g, W_row_ind.data_ptr(), row_bytes, W_col_ind.data_ptr(),
                                             nnz, ws.data_ptr(), (size_t)ws.numel(),
                                             spfa_ext::current_stream(Q)));
  return std::make_tuple(dQ, dK, dV);
}

// to_csr(w_row_ind, w_col_ind, n_rows) -> (row_off, col_ind), uint32: the entries as a CSR mask (columns
// of a row in no particular order), for the spfa_csr entry points (plans, transpose, backward).
std::tuple<torch::Tensor, torch::Tensor> spfa_coo_to_csr_py(torch::Tensor W_row_ind, torch::Tensor W_col_ind,
                                                            int64_t n_rows) {
  CHECK_INPUT(W_row_ind);
  CHECK_INPUT(W_col_ind);
  c10::DeviceGuard guard(W_row_ind.device());
  TORCH_CHECK(W_row_ind.dim() == 1 && W_col_ind.dim() == 1 && W_row_ind.size(0) == W_col_ind.size(0),
              "W_row_ind and W_col_ind must be 1-D and of equal length");
  TORCH_CHECK(n_rows >= 0, "n_rows must not be negative");
  const int row_bytes = spfa_ext::index_bytes(W_row_ind, "W_row_ind", true);
  spfa_ext::index_bytes(W_col_ind, "W_col_ind", false);
  const int64_t nnz = W_col_ind.size(0);
  auto opt = torch::TensorOptions().dtype(torch::kUInt32).device(W_row_ind.device());
  torch::Tensor row_off = torch::empty({n_rows + 1}, opt);
  torch::Tensor cols = torch::empty({nnz}, opt);
  torch::Tensor ws = spfa_ext::make_workspace(spfa_coo_to_csr_workspace_bytes(n_rows, nnz), W_row_ind);
  spfa_ext::raise_on_error(spfa_coo_to_csr(n_rows, W_row_ind.data_ptr(), row_bytes, W_col_ind.data_ptr(), nnz,
                                           (uint32_t*)row_off.data_ptr(), (uint32_t*)cols.data_ptr(),
                                           ws.data_ptr(), (size_t)ws.numel(),
                                           spfa_ext::current_stream(W_row_ind)));
  return std::make_tuple(row_off, cols);
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, mod) {
  mod.def("forward", &spfa_coo_forward_py, "Sparse-FlashAttention forward, COO mask (HIP, gfx950)");
  mod.def("plan", &spfa_coo_plan_py, "Mask pre-pass of a COO mask, for forward_planned");
  mod.def("forward_planned", &spfa_coo_forward_planned_py,
          "forward(...) with the mask pre-pass taken from plan(...)");
  mod.def("backward", &spfa_coo_backward_py, "Gradients of forward(...), added to dQ, dK, dV");
  mod.def("to_csr", &spfa_coo_to_csr_py, "The COO entries as a CSR mask (uint32 offsets and columns)");
}
