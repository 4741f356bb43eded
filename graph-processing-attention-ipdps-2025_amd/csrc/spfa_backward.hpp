// fp64 gradients of masked attention: one plain kernel for every mask functor, double arithmetic,
// for parity checks (torch.autograd.gradcheck) rather than speed.  The fp32 / half problems go
// through the two gather passes of spfa_grad.hpp and the tile kernels of spfa_grad_tiles.hpp.
//
// With lse_i = m_i + log l_i, p_ij = exp(q_i.k_j / sqrt(d) - lse_i) on live positions and
// delta_i = dO_i . O_i:
//     dV_j += p_ij dO_i
//     dS_ij = p_ij (dO_i . v_j - delta_i)
//     dQ_i += dS_ij k_j / sqrt(d)          dK_j += dS_ij q_i / sqrt(d)
// (m, l, O) are those of the FINISHED forward state, so a state built by several chained calls on
// disjoint masks is differentiated by one backward call per mask, all adding into the same
// gradients.
//
// One wavefront per query row.  Candidates are taken 64 at a time: lane j holds candidate j and
// computes both of its dot products (q_i.k_j and dO_i.v_j) from the row's q and dO kept in LDS;
// then, candidate after candidate, lane e adds to dQ in registers and to dK_j, dV_j with
// hardware floating-point atomics (consecutive lanes, consecutive addresses).  (The same kernel
// in fp32 spent its time in those atomics - 7.8 ms at 12.8 M positions - which is why the fp32
// path walks the mask twice instead.)
#pragma once

#include "spfa_engine.hpp"
#include "spfa_masks.hpp"

namespace spfa {

struct Grads {
  const void* d_out;  // [n_batch * n_q, d], element type of the problem
  void* d_q;          // gradients: fp32 (fp64 for fp64 problems), added to
  void* d_k;
  void* d_v;
};

constexpr int kBwdMaxEpl = 16;  // d <= 1024
constexpr int kBwdWaves = 4;

template <typename A>
__device__ __forceinline__ A wave_sum_any(A x) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off, kWave);
  return x;
}

template <typename T, typename A>
__device__ __forceinline__ A load_state_any(const void* p, int64_t i, bool state_f32) {
  if constexpr (sizeof(A) == 8) return ((const double*)p)[i];
  else return load_state<T>(p, i, state_f32);
}

// Both dot products of one candidate: s = q . k_row, dp = dO . v_row (q, dO in LDS as A).
template <typename T, typename A>
__device__ __forceinline__ void two_dots(const A* q, const A* dout, const T* kr, const T* vr, int d,
                                         A& s, A& dp) {
  constexpr int V = 16 / (int)sizeof(T);  // elements per 16-byte load
  A s0 = 0, s1 = 0, p0 = 0, p1 = 0;
  int e = 0;
  if ((d % V) == 0) {  // rows are 16-byte aligned then
    typedef T vec __attribute__((ext_vector_type(V)));
    for (; e < d; e += V) {
      const vec kk = *reinterpret_cast<const vec*>(kr + e);
      const vec vv = *reinterpret_cast<const vec*>(vr + e);
#pragma unroll
      for (int x = 0; x < V; x += 2) {
        s0 += q[e + x] * (A)kk[x];
        s1 += q[e + x + 1] * (A)kk[x + 1];
        p0 += dout[e + x] * (A)vv[x];
        p1 += dout[e + x + 1] * (A)vv[x + 1];
      }
    }
  } else {
    for (; e < d; e++) {
      s0 += q[e] * (A)kr[e];
      p0 += dout[e] * (A)vr[e];
    }
  }
  s = s0 + s1;
  dp = p0 + p1;
}

template <typename T, typename A, class Mask>
__global__ __launch_bounds__(kBwdWaves* kWave) void rows_backward_kernel(Tensors t, Mask mask, Grads g) {
  extern __shared__ __align__(16) unsigned char bwd_lds[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int d = t.d;
  const int64_t total = t.n_q * t.n_batch;
  int64_t row = (int64_t)blockIdx.x * kBwdWaves + wave;  // among all problems of the batch
  const bool active = row < total;
  if (!active) row = total - 1;
  int64_t b, ri;
  split_row(t, row, b, ri);

  A* qs = reinterpret_cast<A*>(bwd_lds) + (size_t)wave * 2 * d;
  A* ds = qs + d;
  const T* qrow = (const T*)t.q + row * d;
  const T* dorow = (const T*)g.d_out + row * d;
  const T* orow = (const T*)t.out + row * d;
  A qreg[kBwdMaxEpl], doreg[kBwdMaxEpl], dq[kBwdMaxEpl];
  A delta = 0;
#pragma unroll
  for (int e = 0; e < kBwdMaxEpl; e++) {
    const int idx = lane + e * kWave;
    qreg[e] = 0;
    doreg[e] = 0;
    dq[e] = 0;
    if (idx < d) {
      qreg[e] = (A)qrow[idx];
      doreg[e] = (A)dorow[idx];
      qs[idx] = qreg[e];
      ds[idx] = doreg[e];
      delta += doreg[e] * (A)orow[idx];
    }
  }
  __syncthreads();
  if (!active) return;

  const A m_i = load_state_any<T, A>(t.m, row, t.state_f32 != 0);
  const A l_i = load_state_any<T, A>(t.l, row, t.state_f32 != 0);
  if (!(l_i > (A)0)) return;  // the row never saw a live column: no gradient flows through it
  const A lse = m_i + log(l_i);
  delta = wave_sum_any(delta);
  const A scale = (A)1 / sqrt((A)d);

  const T* K = (const T*)t.k + b * t.kv_stride;
  const T* V = (const T*)t.v + b * t.kv_stride;
  A* dK = (A*)g.d_k + b * t.kv_stride;
  A* dV = (A*)g.d_v + b * t.kv_stride;
  const int epl = (d + kWave - 1) / kWave;

  const typename Mask::Row rc = mask.row(ri);
  const int64_t deg = rc.deg;
  for (int64_t t0 = 0; t0 < deg; t0 += kWave) {
    const int64_t tt = t0 + lane;
    bool valid = tt < deg;
    int64_t col = 0;
    if (valid) col = mask.col(rc, tt, valid);
    A p = 0, dsc = 0;
    if (valid) {
      A s, dp;
      two_dots<T, A>(qs, ds, K + col * d, V + col * d, d, s, dp);
      p = exp(s * scale - lse);
      dsc = p * (dp - delta) * scale;
    }
    const int live = (int)((deg - t0) < kWave ? (deg - t0) : kWave);
    for (int j = 0; j < live; j++) {
      const A pj = __shfl(p, j, kWave);
      const A dj = __shfl(dsc, j, kWave);
      const int64_t cj = __shfl(col, j, kWave);
      if (pj == (A)0) continue;  // masked candidate (uniform: every lane reads lane j)
      const T* kr = K + cj * d;
      A* dkr = dK + cj * d;
      A* dvr = dV + cj * d;
#pragma unroll
      for (int e = 0; e < kBwdMaxEpl; e++) {
        if (e < epl) {
          const int idx = lane + e * kWave;
          if (idx < d) {
            dq[e] += dj * (A)kr[idx];
            unsafeAtomicAdd(dkr + idx, dj * qreg[e]);
            unsafeAtomicAdd(dvr + idx, pj * doreg[e]);
          }
        }
      }
    }
  }
  A* dqrow = (A*)g.d_q + row * d;
#pragma unroll
  for (int e = 0; e < kBwdMaxEpl; e++) {
    const int idx = lane + e * kWave;
    if (idx < d) dqrow[idx] += dq[e];  // (the row belongs to this wavefront alone)
  }
}

template <typename T, typename A, class Mask>
int run_backward(const Tensors& t, const Mask& mask, const Grads& g, hipStream_t stream) {
  if (t.d > kBwdMaxEpl * kWave) return 5;
  const int64_t rows = t.n_q * t.n_batch;
  if (rows == 0) return 0;
  const int64_t blocks = (rows + kBwdWaves - 1) / kBwdWaves;
  if (blocks >= ((int64_t)1 << 31)) return 1;
  const size_t lds = (size_t)kBwdWaves * 2 * t.d * sizeof(A);
  hipLaunchKernelGGL((rows_backward_kernel<T, A, Mask>), dim3((unsigned)blocks),
                     dim3(kBwdWaves * kWave), lds, stream, t, mask, g);
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

// dtype: the C enum of the element type (3 = fp64, the only one served here)
template <class Mask>
int run_backward_any(int dtype, const Tensors& t, const Mask& mask, const Grads& g,
                     hipStream_t stream) {
  if (dtype == 3) return run_backward<double, double, Mask>(t, mask, g, stream);
  return 2;  // the other element types have kernels of their own
}

}  // namespace spfa
