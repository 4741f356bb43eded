// fp64 inputs (the reference dispatches double as well, sp_flatt_csr_kernel.cu:270): one plain
// kernel for every mask functor, double arithmetic throughout, not tuned.  One wavefront per query
// row; candidates are taken 64 at a time: lane j scores candidate j (a full dot product per lane),
// the chunk's maximum and sum are wave reductions, and the V rows of the chunk are then added up
// with lane e owning output elements e, e + 64, ...
#pragma once

#include "spfa_engine.hpp"

namespace spfa {

__device__ __forceinline__ double wave_max_f64(double x) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) x = fmax(x, __shfl_xor(x, off, kWave));
  return x;
}
__device__ __forceinline__ double wave_sum_f64(double x) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off, kWave);
  return x;
}

constexpr int kF64MaxEpl = 16;  // d <= 1024

template <class Mask>
__global__ __launch_bounds__(256) void rows_f64_kernel(Tensors t, Mask mask, int use_nan) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int64_t row = (int64_t)blockIdx.x * 4 + wave;  // among all problems of the batch
  if (row >= t.n_q * t.n_batch) return;
  int64_t b, ri;
  split_row(t, row, b, ri);
  const int d = t.d;
  const double* q = (const double*)t.q + row * d;
  const double* K = (const double*)t.k + b * t.kv_stride;
  const double* V = (const double*)t.v + b * t.kv_stride;
  double* out = (double*)t.out + row * d;
  const double kInf = __builtin_inf();

  const typename Mask::Row rc = mask.row(ri);
  const int64_t deg = rc.deg;
  const double scale = 1.0 / sqrt((double)d);
  double m = -kInf, l = 0.0;
  double acc[kF64MaxEpl];
#pragma unroll
  for (int e = 0; e < kF64MaxEpl; e++) acc[e] = 0.0;

  for (int64_t t0 = 0; t0 < deg; t0 += kWave) {
    const int64_t tt = t0 + lane;
    bool valid = tt < deg;
    int64_t col = 0;
    if (valid) col = mask.col(rc, tt, valid);
    double s = -kInf;
    if (valid) {
      const double* kr = K + col * d;
      double dot = 0.0;
      for (int e = 0; e < d; e++) dot += q[e] * kr[e];
      s = dot * scale;
    }
    const double cm = wave_max_f64(s);
    if (cm == -kInf) continue;  // (the same for every lane)
    const double m_new = fmax(m, cm);
    const double corr = (m == -kInf) ? 0.0 : exp(m - m_new);
    const double p = valid ? exp(s - m_new) : 0.0;
    l = l * corr + wave_sum_f64(p);
#pragma unroll
    for (int e = 0; e < kF64MaxEpl; e++) acc[e] *= corr;
    const int live = (int)((deg - t0) < kWave ? (deg - t0) : kWave);
    for (int j = 0; j < live; j++) {
      const double pj = __shfl(p, j, kWave);
      const int64_t cj = __shfl(col, j, kWave);
      if (pj == 0.0) continue;  // masked candidate (uniform: every lane reads the same lane j)
      const double* vr = V + cj * d;
#pragma unroll
      for (int e = 0; e < kF64MaxEpl; e++) {
        const int idx = lane + e * kWave;
        if (idx < d) acc[e] += pj * vr[idx];
      }
    }
    m = m_new;
  }

  if (!(l > 0.0)) {  // no live column: m, l untouched, out untouched or NaN
    if (use_nan) {
      for (int idx = lane; idx < d; idx += kWave) out[idx] = __builtin_nan("");
    }
    return;
  }
  // fold the incoming state in (sp_flatt_csr_kernel.cu:171-193)
  double* mp = (double*)t.m + row;
  double* lp = (double*)t.l + row;
  const double m_in = *mp, l_in = *lp;
  double m_out = m, l_out = l, wa = 0.0, wb = 1.0;
  if (l_in != 0.0) {
    m_out = fmax(m, m_in);
    wa = l_in * exp(m_in - m_out);
    wb = exp(m - m_out);
    l_out = wa + l * wb;
  }
  const double inv = 1.0 / l_out;
#pragma unroll
  for (int e = 0; e < kF64MaxEpl; e++) {
    const int idx = lane + e * kWave;
    if (idx < d) {
      double x = acc[e] * wb;
      if (wa != 0.0) x += wa * out[idx];
      out[idx] = x * inv;
    }
  }
  if (lane == 0) {  // (every lane has read m_in, l_in above, in the same instruction)
    *mp = m_out;
    *lp = l_out;
  }
}

template <class Mask>
int run_f64(const Tensors& t, const Mask& mask, int use_nan, hipStream_t stream) {
  if (t.d > kF64MaxEpl * kWave) return 5;
  const int64_t rows = t.n_q * t.n_batch;
  if (rows == 0) return 0;
  if ((rows + 3) / 4 >= ((int64_t)1 << 31)) return 1;
  hipLaunchKernelGGL((rows_f64_kernel<Mask>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, t,
                     mask, use_nan);
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

}  // namespace spfa
