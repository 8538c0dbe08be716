// Chunk merge (reference SMVecMatMul, universal_attention_autograd.py:278-297):
//   result[row, dd] = sum_i softmax_i(vec[row, :]) * mat[row, dd, i]
// and its backward.  Pure streaming kernels (HBM bound): one wave per row, weights in LDS.
#pragma once
#include "ua_common.hpp"

namespace ua {

struct ChunkedView { void* p; long sz, st, sd, si; };

constexpr int kMergeMaxN = 1024;   // chunks per row supported by the merge kernels

template <class T>
__device__ __forceinline__ void row_softmax(const T* __restrict__ vec, int n, float* __restrict__ wts, int lane) {
  float mx = -3.0e38f;
  for (int i = lane; i < n; i += 64) mx = fmaxf(mx, (float)vec[i]);
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m, 64));
  float sum = 0.f;
  for (int i = lane; i < n; i += 64) { float e = __expf((float)vec[i] - mx); wts[i] = e; sum += e; }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) sum += __shfl_xor(sum, m, 64);
  const float inv = 1.0f / sum;
  for (int i = lane; i < n; i += 64) wts[i] *= inv;
}

template <class T>
__global__ void __launch_bounds__(256) k_merge_fwd(ChunkedView mat, const T* __restrict__ vec, T* __restrict__ res,
                                                   long rows, int L, int d, int n) {
  extern __shared__ __align__(16) char smem[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float* wts = reinterpret_cast<float*>(smem) + wave * n;
  const long row = (long)blockIdx.x * 4 + wave;
  if (row >= rows) return;
  row_softmax(vec + row * n, n, wts, lane);
  __builtin_amdgcn_wave_barrier();
  const T* m = reinterpret_cast<const T*>(mat.p) + (row / L) * mat.sz + (row % L) * mat.st;
  for (int dd = lane; dd < d; dd += 64) {
    float acc = 0.f;
    for (int i = 0; i < n; ++i) acc += wts[i] * (float)m[dd * mat.sd + i * mat.si];
    res[row * d + dd] = cvt<T>(acc);
  }
}

template <class T>
__global__ void __launch_bounds__(256) k_merge_bwd(ChunkedView mat, const T* __restrict__ vec, const T* __restrict__ g,
                                                   ChunkedView dmat, T* __restrict__ dvec, long rows, int L, int d, int n) {
  extern __shared__ __align__(16) char smem[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float* wts = reinterpret_cast<float*>(smem) + wave * 2 * n;
  float* dw = wts + n;
  const long row = (long)blockIdx.x * 4 + wave;
  if (row >= rows) return;
  row_softmax(vec + row * n, n, wts, lane);
  __builtin_amdgcn_wave_barrier();
  const T* m = reinterpret_cast<const T*>(mat.p) + (row / L) * mat.sz + (row % L) * mat.st;
  T* dm = reinterpret_cast<T*>(dmat.p) + (row / L) * dmat.sz + (row % L) * dmat.st;
  const T* gr = g + row * d;
  // d_mat[dd, i] = g[dd] * w[i]
  for (int dd = lane; dd < d; dd += 64) {
    const float gv = (float)gr[dd];
    for (int i = 0; i < n; ++i) dm[dd * dmat.sd + i * dmat.si] = cvt<T>(gv * wts[i]);
  }
  // d_w[i] = sum_dd g[dd] * mat[dd, i]
  for (int i = 0; i < n; ++i) {
    float acc = 0.f;
    for (int dd = lane; dd < d; dd += 64) acc += (float)gr[dd] * (float)m[dd * mat.sd + i * mat.si];
#pragma unroll
    for (int k = 32; k >= 1; k >>= 1) acc += __shfl_xor(acc, k, 64);
    if (lane == 0) dw[i] = acc;
  }
  __builtin_amdgcn_wave_barrier();
  float dot = 0.f;
  for (int i = lane; i < n; i += 64) dot += dw[i] * wts[i];
#pragma unroll
  for (int k = 32; k >= 1; k >>= 1) dot += __shfl_xor(dot, k, 64);
  for (int i = lane; i < n; i += 64) dvec[row * n + i] = cvt<T>((dw[i] - dot) * wts[i]);
}

}  // namespace ua
