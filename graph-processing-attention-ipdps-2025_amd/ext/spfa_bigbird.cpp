// Python module spfa_bigbird:
//   forward(q, k, v, m, l, out, LOCAL_SIZE, global_inds, w_row_off, w_col_ind, w_val)
//   backward(the same, dO, dQ, dK, dV[, t_row_off, t_col_ind])
// Window + global + CSR mask in one call: the chain Local -> Global-no-local -> CSR that the
// reference's callers write by hand (verification/verify.py:337-352).  global_inds and the CSR
// tensors may be empty.  The work is done by spfa_window_global_csr_forward in libspfa_hip.so.
#include "spfa_ext_common.h"

torch::Tensor spfa_bigbird_forward_py(torch::Tensor Q, torch::Tensor K, torch::Tensor V, torch::Tensor m,
                                      torch::Tensor l, torch::Tensor O, int64_t local_size_each_dir,
                                      torch::Tensor global_inds, torch::Tensor W_row_off,
                                      torch::Tensor W_col_ind, torch::Tensor W_val) {
  CHECK_INPUT(Q);
  CHECK_INPUT(K);
  CHECK_INPUT(V);
  CHECK_INPUT(m);
  CHECK_INPUT(l);
  CHECK_INPUT(O);
  CHECK_INPUT(global_inds);
  CHECK_INPUT(W_row_off);
  CHECK_INPUT(W_col_ind);
  CHECK_INPUT(W_val);

  c10::DeviceGuard guard(Q.device());
  spfa_problem_t p = spfa_ext::make_problem(Q, K, V, m, l, O);
  TORCH_CHECK(p.n_k == p.n_q, "Q, K and V must have the same number of rows");
  TORCH_CHECK(global_inds.dim() == 1, "global_inds must be 1-D");
  TORCH_CHECK(global_inds.numel() == 0 || global_inds.scalar_type() == torch::kInt32,
              "global_inds must be an int32 tensor");
  TORCH_CHECK(W_col_ind.dim() == 1, "W_col_ind must be 1-D");
  const int64_t nnz = W_col_ind.size(0);
  int off_bytes = 8;
  if (nnz > 0) {
    TORCH_CHECK(W_row_off.dim() == 1 && W_row_off.size(0) == p.n_q + 1, "W_row_off must hold rows+1 offsets");
    TORCH_CHECK(W_val.scalar_type() == Q.scalar_type(), "W_val must have the dtype of Q");
    off_bytes = spfa_ext::index_bytes(W_row_off, "W_row_off", true);
    spfa_ext::index_bytes(W_col_ind, "W_col_ind", false);
  }
  const int64_t n_globs = global_inds.size(0);
  const size_t ws_bytes = spfa_ext::batched(
      spfa_window_global_csr_workspace_bytes(p.n_q, p.d, p.dtype, local_size_each_dir, n_globs, nnz), p);
  torch::Tensor ws = spfa_ext::make_workspace(ws_bytes, Q);
  spfa_ext::raise_on_error(spfa_window_global_csr_forward(
      &p, local_size_each_dir, n_globs ? (const int32_t*)global_inds.data_ptr() : nullptr, n_globs,
      nnz ? W_row_off.data_ptr() : nullptr, off_bytes, nnz ? W_col_ind.data_ptr() : nullptr, nnz,
      ws.data_ptr(), (size_t)ws.numel(), spfa_ext::current_stream(Q)));
  return O;
}

// backward(q, k, v, m, l, out, LOCAL_SIZE, global_inds, w_row_off, w_col_ind, w_val, dO, dQ, dK, dV,
//          t_row_off=None, t_col_ind=None) -> (dQ, dK, dV): the gradients of forward(...), added to
// dQ, dK, dV; t_row_off / t_col_ind as in spfa_csr.backward.
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> spfa_bigbird_backward_py(
    torch::Tensor Q, torch::Tensor K, torch::Tensor V, torch::Tensor m, torch::Tensor l, torch::Tensor O,
    int64_t local_size_each_dir, torch::Tensor global_inds, torch::Tensor W_row_off, torch::Tensor W_col_ind,
    torch::Tensor W_val, torch::Tensor dO, torch::Tensor dQ, torch::Tensor dK, torch::Tensor dV,
    c10::optional<torch::Tensor> t_row_off, c10::optional<torch::Tensor> t_col_ind) {
  CHECK_INPUT(Q);
  CHECK_INPUT(K);
  CHECK_INPUT(V);
  CHECK_INPUT(m);
  CHECK_INPUT(l);
  CHECK_INPUT(O);
  CHECK_INPUT(global_inds);
  CHECK_INPUT(W_row_off);
  CHECK_INPUT(W_col_ind);
  SPFA_CHECK_GRAD_INPUTS();
  (void)W_val;
  c10::DeviceGuard guard(Q.device());
  spfa_problem_t p = spfa_ext::make_problem(Q, K, V, m, l, O);
  spfa_grads_t g = spfa_ext::make_grads(Q, K, dO, dQ, dK, dV);
  TORCH_CHECK(p.n_k == p.n_q, "Q, K and V must have the same number of rows");
  TORCH_CHECK(global_inds.dim() == 1, "global_inds must be 1-D");
  TORCH_CHECK(global_inds.numel() == 0 || global_inds.scalar_type() == torch::kInt32,
              "global_inds must be an int32 tensor");
  TORCH_CHECK(W_col_ind.dim() == 1, "W_col_ind must be 1-D");
  const int64_t nnz = W_col_ind.size(0);
  int off_bytes = 8;
  if (nnz > 0) {
    TORCH_CHECK(W_row_off.dim() == 1 && W_row_off.size(0) == p.n_q + 1, "W_row_off must hold rows+1 offsets");
    off_bytes = spfa_ext::index_bytes(W_row_off, "W_row_off", true);
    spfa_ext::index_bytes(W_col_ind, "W_col_ind", false);
  }
  const uint32_t* tro = nullptr;
  const uint32_t* tci = nullptr;
  TORCH_CHECK(t_row_off.has_value() == t_col_ind.has_value(), "t_row_off and t_col_ind go together");
  if (t_row_off.has_value() && nnz > 0) {
    const torch::Tensor& a = *t_row_off;
    const torch::Tensor& b = *t_col_ind;
    CHECK_INPUT(a);
    CHECK_INPUT(b);
    TORCH_CHECK(a.dim() == 1 && a.size(0) == p.n_k + 1 && b.dim() == 1 && b.size(0) == nnz &&
                    spfa_ext::index_bytes(a, "t_row_off", false) == 4 &&
                    spfa_ext::index_bytes(b, "t_col_ind", false) == 4,
                "t_row_off / t_col_ind must be the 32-bit tensors spfa_csr.transpose() returned for this mask");
    tro = (const uint32_t*)a.data_ptr();
    tci = (const uint32_t*)b.data_ptr();
  }
  const int64_t n_globs = global_inds.size(0);
  torch::Tensor ws = spfa_ext::make_workspace(
      spfa_window_global_csr_backward_workspace_bytes(p.n_q, p.d, p.dtype, local_size_each_dir, n_globs, nnz,
                                                      p.n_batch), Q);
  spfa_ext::raise_on_error(spfa_window_global_csr_backward(
      &p, &g, local_size_each_dir, n_globs ? (const int32_t*)global_inds.data_ptr() : nullptr, n_globs,
      nnz ? W_row_off.data_ptr() : nullptr, off_bytes, nnz ? W_col_ind.data_ptr() : nullptr, nnz, tro, tci,
      ws.data_ptr(), (size_t)ws.numel(), spfa_ext::current_stream(Q)));
  return std::make_tuple(dQ, dK, dV);
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, mod) {
  namespace py = pybind11;
  mod.def("forward", &spfa_bigbird_forward_py,
          "Window + global + CSR mask in one call (HIP, gfx950)");
  mod.def("backward", &spfa_bigbird_backward_py, "Gradients of forward(...), added to dQ, dK, dV", py::arg("Q"),
          py::arg("K"), py::arg("V"), py::arg("m"), py::arg("l"), py::arg("O"), py::arg("LOCAL_SIZE"),
          py::arg("global_inds"), py::arg("W_row_off"), py::arg("W_col_ind"), py::arg("W_val"), py::arg("dO"),
          py::arg("dQ"), py::arg("dK"), py::arg("dV"), py::arg("t_row_off") = py::none(),
          py::arg("t_col_ind") = py::none());
}
