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

  const size_t ws_bytes = spfa_csr_workspace_bytes_batched(p.n_q, nnz, p.d, p.dtype, p.n_batch);
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
  // a plan is built once and used many times: worth one look at the data (this synchronises)
  TORCH_CHECK(spfa_ext::index_value(W_row_off, n_q) == nnz,
              "W_row_off must end at the number of entries of W_col_ind");
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

  const size_t ws_bytes = spfa_csr_workspace_bytes_batched(p.n_q, nnz, p.d, p.dtype, p.n_batch);
  torch::Tensor ws = spfa_ext::make_workspace(ws_bytes, Q);
  spfa_ext::raise_on_error(spfa_csr_forward_planned(
      &p, W_row_off.data_ptr(), off_bytes, W_col_ind.data_ptr(), nnz, use_nan ? 1 : 0, plan.data_ptr(),
      (size_t)plan.numel(), ws.data_ptr(), (size_t)ws.numel(), spfa_ext::current_stream(Q)));
  return O;
}

// backward(<the arguments of forward, without use_nan>, dO, dQ, dK, dV, t_row_off=None,
// t_col_ind=None) -> (dQ, dK, dV): adds the gradients of the attention forward computes to dQ, dK,
// dV (float32; float64 for float64 inputs).  m, l, O are the finished forward state.  t_row_off /
// t_col_ind are the mask by key row from transpose(); without them it is rebuilt in every call.
// The reference binds no backward.
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> spfa_csr_backward_py(
    torch::Tensor Q, torch::Tensor K, torch::Tensor V, torch::Tensor W_row_off, torch::Tensor W_col_ind,
    torch::Tensor W_val, torch::Tensor m, torch::Tensor l, torch::Tensor O, torch::Tensor dO,
    torch::Tensor dQ, torch::Tensor dK, torch::Tensor dV, c10::optional<torch::Tensor> t_row_off,
    c10::optional<torch::Tensor> t_col_ind) {
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
  const uint32_t* tro = nullptr;
  const uint32_t* tci = nullptr;
  TORCH_CHECK(t_row_off.has_value() == t_col_ind.has_value(), "t_row_off and t_col_ind go together");
  if (t_row_off.has_value()) {
    const torch::Tensor& a = *t_row_off;
    const torch::Tensor& b = *t_col_ind;
    CHECK_INPUT(a);
    CHECK_INPUT(b);
    TORCH_CHECK(a.dim() == 1 && a.size(0) == p.n_k + 1 && b.dim() == 1 && b.size(0) == nnz &&
                    spfa_ext::index_bytes(a, "t_row_off", false) == 4 &&
                    spfa_ext::index_bytes(b, "t_col_ind", false) == 4,
                "t_row_off / t_col_ind must be the 32-bit tensors transpose() returned for this mask");
    tro = (const uint32_t*)a.data_ptr();
    tci = (const uint32_t*)b.data_ptr();
  }
  torch::Tensor ws = spfa_ext::make_workspace(
      spfa_csr_backward_workspace_bytes(p.n_q, p.n_k, nnz, p.d, p.dtype, p.n_batch), Q);
  spfa_ext::raise_on_error(spfa_csr_backward(&p, &g, W_row_off.data_ptr(), off_bytes, W_col_ind.data_ptr(),
                                             nnz, tro, tci, ws.data_ptr(), (size_t)ws.numel(),
                                             spfa_ext::current_stream(Q)));
  return std::make_tuple(dQ, dK, dV);
}

// transpose(w_row_off, w_col_ind, n_cols) -> (t_row_off, t_col_ind), uint32: the mask read by
// column, for backward(..., t_row_off, t_col_ind).  A mask reused over many steps is transposed once.
std::tuple<torch::Tensor, torch::Tensor> spfa_csr_transpose_py(torch::Tensor W_row_off,
                                                               torch::Tensor W_col_ind, int64_t n_cols) {
  CHECK_INPUT(W_row_off);
  CHECK_INPUT(W_col_ind);
  c10::DeviceGuard guard(W_row_off.device());
  TORCH_CHECK(W_row_off.dim() == 1 && W_row_off.size(0) >= 1, "W_row_off must hold rows+1 offsets");
  TORCH_CHECK(W_col_ind.dim() == 1, "W_col_ind must be 1-D");
  TORCH_CHECK(n_cols >= 0, "n_cols must not be negative");
  const int off_bytes = spfa_ext::index_bytes(W_row_off, "W_row_off", true);
  spfa_ext::index_bytes(W_col_ind, "W_col_ind", false);
  const int64_t n_q = W_row_off.size(0) - 1, nnz = W_col_ind.size(0);
  auto opt = torch::TensorOptions().dtype(torch::kUInt32).device(W_row_off.device());
  torch::Tensor t_row_off = torch::empty({n_cols + 1}, opt);
  torch::Tensor t_col_ind = torch::empty({nnz}, opt);
  torch::Tensor ws = spfa_ext::make_workspace(spfa_csr_transpose_workspace_bytes(n_q, n_cols, nnz), W_row_off);
  spfa_ext::raise_on_error(spfa_csr_transpose(n_q, n_cols, W_row_off.data_ptr(), off_bytes,
                                              W_col_ind.data_ptr(), nnz, (uint32_t*)t_row_off.data_ptr(),
                                              (uint32_t*)t_col_ind.data_ptr(), ws.data_ptr(),
                                              (size_t)ws.numel(), spfa_ext::current_stream(W_row_off)));
  return std::make_tuple(t_row_off, t_col_ind);
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, mod) {
  namespace py = pybind11;
  mod.def("forward", &spfa_csr_forward_py, "Sparse-FlashAttention forward, CSR mask (HIP, gfx950)");
  mod.def("plan", &spfa_csr_plan_py, "Mask pre-pass of a CSR mask, for forward_planned");
  mod.def("forward_planned", &spfa_csr_forward_planned_py,
          "forward(...) with the mask pre-pass taken from plan(...)");
  mod.def("backward", &spfa_csr_backward_py, "Gradients of forward(...), added to dQ, dK, dV", py::arg("Q"),
          py::arg("K"), py::arg("V"), py::arg("W_row_off"), py::arg("W_col_ind"), py::arg("W_val"),
          py::arg("m"), py::arg("l"), py::arg("O"), py::arg("dO"), py::arg("dQ"), py::arg("dK"),
          py::arg("dV"), py::arg("t_row_off") = py::none(), py::arg("t_col_ind") = py::none());
  mod.def("transpose", &spfa_csr_transpose_py, "The CSR mask read by column, for backward(...)");
  mod.def("device_status", &spfa_ext::device_status,
          "Bits the kernels set on the current device when mask arrays were inconsistent "
          "(1: more long-row entries than W_col_ind holds, 2: row offsets decreasing or beyond its "
          "size); synchronise first",
          py::arg("reset") = false);
}
