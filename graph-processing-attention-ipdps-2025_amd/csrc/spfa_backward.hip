// The gradient kernels, one instantiation per mask functor (every element type in each).
#include "spfa_backward.hpp"
#include "spfa_kernels.hpp"

namespace spfa {

int run_backward_csr(int dtype, const Tensors& t, const CsrMask& mask, const Grads& g,
                     hipStream_t stream) {
  return run_backward_any(dtype, t, mask, g, stream);
}
int run_backward_stride(int dtype, const Tensors& t, const StrideMask& mask, const Grads& g,
                        hipStream_t stream) {
  return run_backward_any(dtype, t, mask, g, stream);
}
int run_backward_global(int dtype, const Tensors& t, const GlobalMask& mask, const Grads& g,
                        hipStream_t stream) {
  return run_backward_any(dtype, t, mask, g, stream);
}

}  // namespace spfa
