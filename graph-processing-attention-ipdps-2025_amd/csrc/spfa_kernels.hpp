// Entry points of the per-(mask, element type) translation units.
#pragma once

#include "spfa_tiles.hpp"
#include "spfa_engine.hpp"
#include "spfa_masks.hpp"

namespace spfa {

// phase / plan_buf: see launch_engine (whole call, work list only, or attention against a work
// list built earlier)
template <typename T>
int run_csr(const Tensors& t, const CsrMask& mask, const EngineSizing& s, int use_nan, void* ws,
            hipStream_t stream, int phase = kEngineAll, const void* plan_buf = nullptr);
template <typename T>
int run_stride(const Tensors& t, const StrideMask& mask, const EngineSizing& s, int use_nan,
               void* ws, hipStream_t stream);
// Dense-tile (MFMA) path for band / block masks; -1 when the shape is not covered.
template <typename T>
int run_band(const TileArgs& a, int use_nan, hipStream_t stream);
// Dense-tile path for the global-minus-local mask; -1 when the shape is not covered.
// (rows_only: see launch_global_tiles)
template <typename T>
int run_global_dense(const TileArgs& a, hipStream_t stream, bool rows_only = false);
template <typename T>
int run_global(const Tensors& t, const GlobalMask& mask, const EngineSizing& s, int use_nan,
               void* ws, hipStream_t stream);

// Gradients by two gather passes (spfa_grad.hpp): `rows` walks the mask by query row, `cols` by
// key row.
struct GradArgs;
template <typename T>
int run_grad_csr(const Tensors& t, const GradArgs& g, const CsrMask& rows, const CsrMask& cols,
                 hipStream_t stream);
template <typename T>
int run_grad_stride(const Tensors& t, const GradArgs& g, const StrideMask& mask, hipStream_t stream);
// Dense-tile gradients of band / block masks; -1 when the shape is not covered.
template <typename T>
int run_band_grad(const TileArgs& a, const GradArgs& g, hipStream_t stream);
// ... of the global-minus-local mask
template <typename T>
int run_global_grad_dense(const TileArgs& a, const GradArgs& g, hipStream_t stream);
template <typename T>
int run_grad_global(const Tensors& t, const GradArgs& g, const GlobalMask& rows,
                    const GlobalColMask& cols, hipStream_t stream);

// fp64 gradients: one plain kernel with atomics (spfa_backward.hpp); dtype is the C enum.
struct Grads;
int run_backward_csr(int dtype, const Tensors& t, const CsrMask& mask, const Grads& g,
                     hipStream_t stream);
int run_backward_stride(int dtype, const Tensors& t, const StrideMask& mask, const Grads& g,
                        hipStream_t stream);
int run_backward_global(int dtype, const Tensors& t, const GlobalMask& mask, const Grads& g,
                        hipStream_t stream);

}  // namespace spfa
