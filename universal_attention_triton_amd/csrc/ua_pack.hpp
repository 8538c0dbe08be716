// Layout kernels: bring user tensors (arbitrary strides, head dim d) into the padded,
// contiguous working layouts the matrix-core kernels read, plus small row reductions.
#pragma once
#include "ua_common.hpp"

namespace ua {

// A tensor addressed as (z, row, col) with z = ((b*H + h)*R + r)*N + i; element offset
//   b*sb + h*sh + r*sr + i*sn + (row / inner)*so + (row % inner)*si + col*sc
struct RowsView {
  const void* p;
  long sb, sh, sr, sn, so, si, sc;
  int inner, H, R, N;
};
__device__ __forceinline__ long rows_offset(const RowsView& v, int z, int row) {
  int i = z % v.N; z /= v.N;
  int r = z % v.R; z /= v.R;
  int h = z % v.H, b = z / v.H;
  return (long)b * v.sb + (long)h * v.sh + (long)r * v.sr + (long)i * v.sn + (long)(row / v.inner) * v.so +
         (long)(row % v.inner) * v.si;
}

// x (dtype T) -> nat and/or tr working tensors, zero padded (rows >= L, cols >= d).
//   tiled == 0: nat [Z][Lp][D] row-major, tr [Z][D][Lp] row-major       (chunked-mode kernels)
//   tiled != 0: both in tiles of 32 positions, k-group-major (nat_off / tr_off)   (fused kernels)
// tr stores position t at column perm16(t) (tr_mode 0), perm32(t) (1) or t (2) of its group of 32.
template <class T, int D>
__global__ void __launch_bounds__(256) k_pack(RowsView x, T* __restrict__ nat, T* __restrict__ tr, int d, int L, int Lp,
                                              int tr_mode, int tiled) {
  __shared__ float tile[32][D + 1];
  const int z = blockIdx.y, row0 = blockIdx.x * 32, tid = threadIdx.x;
  const T* xp = reinterpret_cast<const T*>(x.p);
  for (int i = tid; i < 32 * D; i += 256) {
    int rr = i / D, col = i - rr * D, row = row0 + rr;
    float val = 0.f;
    if (row < L && col < d) val = (float)xp[rows_offset(x, z, row) + (long)col * x.sc];
    tile[rr][col] = val;
    if (nat && !tiled) nat[((long)z * Lp + row) * D + col] = cvt<T>(val);
  }
  if (!tr && !(nat && tiled)) return;
  __syncthreads();
  if (nat && tiled) {
    // consecutive threads write consecutive elements of the tiled order: (k-group, row, e)
    for (int i = tid; i < 32 * D; i += 256) {
      const int e = i & 7, rr = (i >> 3) & 31, kg = i >> 8;
      nat[nat_off<D>(z, Lp, row0 + rr, 8 * kg + e)] = cvt<T>(tile[rr][8 * kg + e]);
    }
  }
  if (!tr) return;
  for (int i = tid; i < 32 * D; i += 256) {
    // perm16 and perm32 are bijections of 0..31: column p holds the position that maps onto it
    if (tiled) {
      const int e = i & 7, dd = (i >> 3) % D, kg = i / (8 * D), p = 8 * kg + e;
      const int src = tr_mode == 0 ? perm16(p) : (tr_mode == 1 ? (((p >> 3) & 3) << 2 | ((p >> 2) & 1) << 4 | (p & 3)) : p);
      tr[tr_off<D>(z, Lp, dd, blockIdx.x, p)] = cvt<T>(tile[src][dd]);
    } else {
      const int dd = i >> 5, rr = i & 31;
      const int src = tr_mode == 0 ? perm16(rr) : (tr_mode == 1 ? (((rr >> 3) & 3) << 2 | ((rr >> 2) & 1) << 4 | (rr & 3)) : rr);
      tr[((long)z * D + dd) * Lp + row0 + rr] = cvt<T>(tile[src][dd]);
    }
  }
}

// delta[z][t] = sum_dd O[z][t][dd] * dO[z][t][dd] - sub[z][t]   (fp32; padded rows -> 0)
// O, dO, sub are views (sub optional, float); one wave per row.
// lse_in (optional, natural log, float view) is rewritten in log2 units into lse2 [Z][Lp].
template <class T>
__global__ void __launch_bounds__(256) k_delta(RowsView O, RowsView dO, RowsView sub, RowsView lse_in,
                                               float* __restrict__ delta, float* __restrict__ lse2, int d, int L, int Lp) {
  const int z = blockIdx.y, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + wave;
  if (t >= Lp) return;
  float s = 0.f;
  if (t < L) {
    const T* o = reinterpret_cast<const T*>(O.p) + rows_offset(O, z, t);
    const T* g = reinterpret_cast<const T*>(dO.p) + rows_offset(dO, z, t);
    for (int c = lane; c < d; c += 64) s += (float)o[(long)c * O.sc] * (float)g[(long)c * dO.sc];
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) s += __shfl_xor(s, m, 64);
  if (lane == 0) {
    if (sub.p && t < L) s -= reinterpret_cast<const float*>(sub.p)[rows_offset(sub, z, t)];
    delta[(long)z * Lp + t] = s;
    if (lse_in.p) lse2[(long)z * Lp + t] = (t < L) ? reinterpret_cast<const float*>(lse_in.p)[rows_offset(lse_in, z, t)] * kLog2e : 0.f;
  }
}

// log-gates: out[z][t] = log2(gate[z][t]) / 3 for t < L, kGatePad beyond (gate contiguous [Z][L], dtype T)
template <class T>
__global__ void __launch_bounds__(256) k_gates(const T* __restrict__ src, const T* __restrict__ dest, float* __restrict__ lsrc,
                                               float* __restrict__ ldest, int L, int Lp) {
  const int z = blockIdx.y, t = blockIdx.x * 256 + threadIdx.x;
  if (t >= Lp) return;
  float a = kGatePad, b = kGatePad;
  if (t < L) {
    a = __builtin_amdgcn_logf((float)src[(long)z * L + t]) * (1.0f / 3.0f);
    b = __builtin_amdgcn_logf((float)dest[(long)z * L + t]) * (1.0f / 3.0f);
  }
  lsrc[(long)z * Lp + t] = a;
  ldest[(long)z * Lp + t] = b;
}

// plain fill (kept as a kernel so that callers may capture the sequence in a HIP graph)
__global__ void __launch_bounds__(256) k_zero(float4* __restrict__ p, size_t n16) {
  for (size_t i = blockIdx.x * (size_t)256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256) p[i] = make_float4(0.f, 0.f, 0.f, 0.f);
}

}  // namespace ua
