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

// VEC: unit feature stride, every (row, chunk) slice 16-byte aligned and d / V (V = elements per 16 bytes) a power of
// two of at most 64 (host-checked): lpr = d / V lanes read one slice with 16-byte loads and the 64 / lpr lane groups
// of a wave take chunks i = group, group + 64 / lpr, ...
template <class T, bool VEC>
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
  if constexpr (VEC) {
    constexpr int V = 16 / (int)sizeof(T);
    const int lpr = d / V, sub = lane & (lpr - 1), grp = lane / lpr, ng = 64 / lpr;
    float acc[V];
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = 0.f;
    for (int i = grp; i < n; i += ng) {
      const float wi = wts[i];
      // a chunk whose normaliser is the reference's fill value (-1e12: no key of it is visible to this query) has a
      // weight of exactly zero: its slice is not read (half of the tensor after the chunked operator)
      if (wi == 0.f) continue;
      T x[V];
      *reinterpret_cast<uint4*>(x) = *reinterpret_cast<const uint4*>(m + sub * V + i * mat.si);
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] += wi * (float)x[e];
    }
    for (int k = lpr; k < 64; k <<= 1) {
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] += __shfl_xor(acc[e], k, 64);
    }
    if (grp == 0) {
      T y[V];
#pragma unroll
      for (int e = 0; e < V; ++e) y[e] = cvt<T>(acc[e]);
      *reinterpret_cast<uint4*>(res + row * d + sub * V) = *reinterpret_cast<const uint4*>(y);
    }
    return;
  }
  for (int dd = lane; dd < d; dd += 64) {
    float acc = 0.f;
    for (int i = 0; i < n; ++i)
      if (wts[i] != 0.f) acc += wts[i] * (float)m[dd * mat.sd + i * mat.si];
    res[row * d + dd] = cvt<T>(acc);
  }
}

template <class T, bool VEC>
// delta (optional): [rows / L][n][Lp] float receives sum_dd mat[dd, i] d_mat[dd, i] - d_vec[i] = w_i (g . result), what
// the chunked operator's backward needs first from exactly these gradients (rows of length Lp, written for t < L)
__global__ void __launch_bounds__(256) k_merge_bwd(ChunkedView mat, const T* __restrict__ vec, const T* __restrict__ g,
                                                   ChunkedView dmat, T* __restrict__ dvec, long rows, int L, int d, int n,
                                                   float* __restrict__ delta, int Lp) {
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
  if constexpr (VEC) {
    constexpr int V = 16 / (int)sizeof(T);
    const int lpr = d / V, sub = lane & (lpr - 1), grp = lane / lpr, ng = 64 / lpr;
    T gx[V];
    *reinterpret_cast<uint4*>(gx) = *reinterpret_cast<const uint4*>(gr + sub * V);
    float gf[V];
#pragma unroll
    for (int e = 0; e < V; ++e) gf[e] = (float)gx[e];
    for (int i0 = 0; i0 < n; i0 += ng) {          // uniform trip count: the shuffles below involve every lane
      const int i = i0 + grp;
      float acc = 0.f;
      if (i < n) {
        T x[V], y[V];
        const float wi = wts[i];
        // zero weight (see k_merge_fwd): the slice's gradient is zero whatever it holds, and so is its share of d_vec
        if (wi != 0.f) {
          *reinterpret_cast<uint4*>(x) = *reinterpret_cast<const uint4*>(m + sub * V + i * mat.si);
#pragma unroll
          for (int e = 0; e < V; ++e) acc += gf[e] * (float)x[e];
        }
#pragma unroll
        for (int e = 0; e < V; ++e) y[e] = cvt<T>(gf[e] * wi);
        *reinterpret_cast<uint4*>(dm + sub * V + i * dmat.si) = *reinterpret_cast<const uint4*>(y);
      }
      for (int k = 1; k < lpr; k <<= 1) acc += __shfl_xor(acc, k, 64);
      if (sub == 0 && i < n) dw[i] = acc;
    }
  } else {
  // d_mat[dd, i] = g[dd] * w[i]
  for (int dd = lane; dd < d; dd += 64) {
    const float gv = (float)gr[dd];
    for (int i = 0; i < n; ++i) dm[dd * dmat.sd + i * dmat.si] = cvt<T>(gv * wts[i]);
  }
  // d_w[i] = sum_dd g[dd] * mat[dd, i]
  for (int i = 0; i < n; ++i) {
    float acc = 0.f;
    if (wts[i] != 0.f)
      for (int dd = lane; dd < d; dd += 64) acc += (float)gr[dd] * (float)m[dd * mat.sd + i * mat.si];
#pragma unroll
    for (int k = 32; k >= 1; k >>= 1) acc += __shfl_xor(acc, k, 64);
    if (lane == 0) dw[i] = acc;
  }
  }
  __builtin_amdgcn_wave_barrier();
  float dot = 0.f;
  for (int i = lane; i < n; i += 64) dot += dw[i] * wts[i];
#pragma unroll
  for (int k = 32; k >= 1; k >>= 1) dot += __shfl_xor(dot, k, 64);
  for (int i = lane; i < n; i += 64) dvec[row * n + i] = cvt<T>((dw[i] - dot) * wts[i]);
  if (delta) {
    float* dl = delta + (row / L) * (long)n * Lp + (row % L);
    for (int i = lane; i < n; i += 64) dl[(long)i * Lp] = wts[i] * dot;
  }
}

}  // namespace ua
