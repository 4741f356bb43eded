// One (mask kind, element type) instantiation of the gradient passes per object file:
// compiled with -DSPFA_INST_MASK={0,1,2} -DSPFA_INST_T={float,spfa::f16,spfa::bf16}.
#include "spfa_grad.hpp"
#include "spfa_grad_tiles.hpp"
#include "spfa_kernels.hpp"

namespace spfa {

#if SPFA_INST_MASK == 0
template <>
int run_grad_csr<SPFA_INST_T>(const Tensors& t, const GradArgs& g, const CsrMask& rows,
                              const CsrMask& cols, hipStream_t stream) {
  return run_grad<SPFA_INST_T>(t, g, rows, cols, stream);
}
#elif SPFA_INST_MASK == 1
template <>
int run_grad_stride<SPFA_INST_T>(const Tensors& t, const GradArgs& g, const StrideMask& mask,
                                 hipStream_t stream) {
  return run_grad<SPFA_INST_T>(t, g, mask, mask, stream);  // symmetric: rows and columns alike
}
template <>
int run_band_grad<SPFA_INST_T>(const TileArgs& a, const GradArgs& g, hipStream_t stream) {
  return run_band_grad_tiles<SPFA_INST_T>(a, g, stream);
}
#elif SPFA_INST_MASK == 2
template <>
int run_grad_global<SPFA_INST_T>(const Tensors& t, const GradArgs& g, const GlobalMask& rows,
                                 const GlobalColMask& cols, hipStream_t stream) {
  return run_grad<SPFA_INST_T>(t, g, rows, cols, stream);
}
template <>
int run_global_grad_dense<SPFA_INST_T>(const TileArgs& a, const GradArgs& g, hipStream_t stream) {
  return run_global_grad_tiles<SPFA_INST_T>(a, g, stream);
}
#else
#error "SPFA_INST_MASK must be 0 (csr), 1 (stride) or 2 (global)"
#endif

}  // namespace spfa
