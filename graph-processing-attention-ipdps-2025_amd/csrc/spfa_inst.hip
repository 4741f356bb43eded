// One (mask kind, element type) instantiation of the row-gather engine per object file:
// compiled with -DSPFA_INST_MASK={0,1,2} -DSPFA_INST_T={float,spfa::f16,spfa::bf16}.
#include "spfa_kernels.hpp"

namespace spfa {

#if SPFA_INST_MASK == 0
template <>
int run_csr<SPFA_INST_T>(const Tensors& t, const CsrMask& mask, const EngineSizing& s, int use_nan,
                         void* ws, hipStream_t stream, int phase, const void* plan_buf) {
  return run_engine<SPFA_INST_T, CsrMask>(t, mask, s, use_nan, ws, stream, phase, plan_buf);
}
#elif SPFA_INST_MASK == 1
template <>
int run_stride<SPFA_INST_T>(const Tensors& t, const StrideMask& mask, const EngineSizing& s,
                            int use_nan, void* ws, hipStream_t stream) {
  return run_engine<SPFA_INST_T, StrideMask>(t, mask, s, use_nan, ws, stream);
}
template <>
int run_band<SPFA_INST_T>(const TileArgs& a, int use_nan, hipStream_t stream) {
  return run_band_tiles<SPFA_INST_T>(a, use_nan, stream);
}
#elif SPFA_INST_MASK == 2
template <>
int run_global<SPFA_INST_T>(const Tensors& t, const GlobalMask& mask, const EngineSizing& s,
                            int use_nan, void* ws, hipStream_t stream) {
  return run_engine<SPFA_INST_T, GlobalMask>(t, mask, s, use_nan, ws, stream);
}
template <>
int run_global_dense<SPFA_INST_T>(const TileArgs& a, hipStream_t stream, bool rows_only) {
  return run_global_tiles<SPFA_INST_T>(a, stream, rows_only);
}
#else
#error "SPFA_INST_MASK must be 0 (csr), 1 (stride) or 2 (global)"
#endif

}  // namespace spfa
