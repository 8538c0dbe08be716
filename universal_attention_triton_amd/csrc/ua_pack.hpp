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

// the same offset split into its z part and its row part (the row part without divisions when row < inner)
__device__ __forceinline__ long rows_base(const RowsView& v, int z) {
  int i = z % v.N; z /= v.N;
  int r = z % v.R; z /= v.R;
  int h = z % v.H, b = z / v.H;
  return (long)b * v.sb + (long)h * v.sh + (long)r * v.sr + (long)i * v.sn;
}
__device__ __forceinline__ long rows_row(const RowsView& v, int row) {
  if (row < v.inner) return (long)row * v.si;
  return (long)(row / v.inner) * v.so + (long)(row % v.inner) * v.si;
}

// x (dtype T) -> nat and/or tr working tensors, zero padded (rows >= L, cols >= d).
//   tiled == 0: nat [Z][Lp][D] row-major, tr [Z][D][Lp] row-major       (chunked-mode kernels)
//   tiled != 0: both in tiles of 32 positions, k-group-major (nat_off / tr_off)   (fused kernels)
// tr stores position t at column perm16(t) (tr_mode 0), perm32(t) (1) or t (2) of its group of 32.
// vec != 0: every row start of x is 16-byte aligned and d is a multiple of the 16-byte vector (host-checked), so
// rows are read with 16-byte loads.
// masked_nz (optional; chunked operator, z = zq*N + chunk, chunk size c): blocks of rows before their chunk are left
// untouched while *masked_nz is 0 (k_delta has found every such row of x to be zero, and no kernel reads them then).
template <class T, int D>
__global__ void __launch_bounds__(256) k_pack(RowsView x, T* __restrict__ nat, T* __restrict__ tr, int d, int L, int Lp,
                                              int tr_mode, int tiled, int vec, float* __restrict__ norm2,
                                              const int* __restrict__ masked_nz, int c) {
  constexpr int V = 16 / (int)sizeof(T);
  __shared__ float tile[32][D + 1];
  const int z = blockIdx.y, row0 = blockIdx.x * 32, tid = threadIdx.x;
  if (masked_nz && row0 + 32 <= (z % x.N) * c && *masked_nz == 0) return;
  const T* xp = reinterpret_cast<const T*>(x.p);
  if (vec) {
    for (int i = tid; i < 32 * (D / V); i += 256) {
      const int rr = i / (D / V), col = (i - rr * (D / V)) * V, row = row0 + rr;
      T v[V];
      if (row < L && col < d) {
        *reinterpret_cast<uint4*>(v) = *reinterpret_cast<const uint4*>(xp + rows_offset(x, z, row) + col);
      } else {
#pragma unroll
        for (int e = 0; e < V; ++e) v[e] = cvt<T>(0.f);
      }
#pragma unroll
      for (int e = 0; e < V; ++e) tile[rr][col + e] = (float)v[e];
      if (nat && !tiled) *reinterpret_cast<uint4*>(nat + ((long)z * Lp + row) * D + col) = *reinterpret_cast<const uint4*>(v);
    }
  } else {
    for (int i = tid; i < 32 * D; i += 256) {
      int rr = i / D, col = i - rr * D, row = row0 + rr;
      float val = 0.f;
      if (row < L && col < d) val = (float)xp[rows_offset(x, z, row) + (long)col * x.sc];
      tile[rr][col] = val;
      if (nat && !tiled) nat[((long)z * Lp + row) * D + col] = cvt<T>(val);
    }
  }
  if (!tr && !(nat && tiled) && !norm2) return;
  __syncthreads();
  if (norm2) {
    // largest squared row norm of the block's (dtype-rounded) rows -> norm2[z][block]: 8 threads per row, then the
    // maximum over the block
    __shared__ float wmax[4];
    const int rr = tid >> 3;
    float s2 = 0.f;
    for (int c = tid & 7; c < D; c += 8) s2 += tile[rr][c] * tile[rr][c];
#pragma unroll
    for (int m = 1; m <= 4; m <<= 1) s2 += __shfl_xor(s2, m, 64);             // the 8 threads of a row
#pragma unroll
    for (int m = 8; m <= 32; m <<= 1) s2 = fmaxf(s2, __shfl_xor(s2, m, 64));   // the 8 rows of a wave
    if ((tid & 63) == 0) wmax[tid >> 6] = s2;
    __syncthreads();
    if (tid == 0) norm2[(long)z * gridDim.x + blockIdx.x] = fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3]));
  }
  if (nat && tiled) {
    // one (k-group, row) cell of 8 elements per thread; consecutive threads write consecutive cells
    for (int i = tid; i < 4 * D; i += 256) {
      const int rr = i & 31, kg = i >> 5;
      T v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = cvt<T>(tile[rr][8 * kg + e]);
      T* dst = nat + nat_off<D>(z, Lp, row0 + rr, 8 * kg);
#pragma unroll
      for (int u = 0; u < 8 / V; ++u) reinterpret_cast<uint4*>(dst)[u] = reinterpret_cast<const uint4*>(v)[u];
    }
  }
  if (!tr) return;
  // perm16 and perm32 are bijections of 0..31: column p holds the position that maps onto it
  if (tiled) {
    for (int i = tid; i < 4 * D; i += 256) {
      const int dd = i % D, kg = i / D;
      T v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int p = 8 * kg + e;
        const int src = tr_mode == 0 ? perm16(p) : (tr_mode == 1 ? (((p >> 3) & 3) << 2 | ((p >> 2) & 1) << 4 | (p & 3)) : p);
        v[e] = cvt<T>(tile[src][dd]);
      }
      T* dst = tr + tr_off<D>(z, Lp, dd, blockIdx.x, 8 * kg);
#pragma unroll
      for (int u = 0; u < 8 / V; ++u) reinterpret_cast<uint4*>(dst)[u] = reinterpret_cast<const uint4*>(v)[u];
    }
  } else {
    for (int i = tid; i < 32 * D; i += 256) {
      const int dd = i >> 5, rr = i & 31;
      const int src = tr_mode == 0 ? perm16(rr) : (tr_mode == 1 ? (((rr >> 3) & 3) << 2 | ((rr >> 2) & 1) << 4 | (rr & 3)) : rr);
      tr[((long)z * D + dd) * Lp + row0 + rr] = cvt<T>(tile[src][dd]);
    }
  }
}

// delta[z][t] = sum_dd O[z][t][dd] * dO[z][t][dd] - sub[z][t]   (fp32; padded rows -> 0)
// O, dO, sub are views (sub optional, float); 16 lanes per row, 128 rows per block (grid (Lp/128, Z)).
// lse_in (optional, natural log, float view) is rewritten in log2 units into lse2 [Z][Lp].
// vec != 0: rows of O and dO start 16-byte aligned, have unit feature stride and d is a multiple of the vector.
// masked_nz (optional; chunked operator, z = zq*N + chunk, chunk size c): set to 1 when a row of dO or sub that lies
// before its chunk (t < chunk*c, a query that sees no key of the chunk) holds a non-zero.
template <class T>
__global__ void __launch_bounds__(256) k_delta(RowsView O, RowsView dO, RowsView sub, RowsView lse_in,
                                               float* __restrict__ delta, float* __restrict__ lse2, int d, int L, int Lp, int vec,
                                               int* __restrict__ masked_nz, int c) {
  constexpr int V = 16 / (int)sizeof(T), IT = 8;
  const int z = blockIdx.y, sub16 = threadIdx.x & 15;
  const int t0 = blockIdx.x * (16 * IT) + (threadIdx.x >> 4);
  const int chunk_start = masked_nz ? (z % dO.N) * c : 0;
  const T* Oz = reinterpret_cast<const T*>(O.p) + rows_base(O, z);
  const T* Gz = reinterpret_cast<const T*>(dO.p) + rows_base(dO, z);
  const float* Sz = sub.p ? reinterpret_cast<const float*>(sub.p) + rows_base(sub, z) : nullptr;
  const float* Lz = lse_in.p ? reinterpret_cast<const float*>(lse_in.p) + rows_base(lse_in, z) : nullptr;
  bool flag = false;
#pragma unroll
  for (int it = 0; it < IT; ++it) {
    const int t = t0 + 16 * it;
    float s = 0.f;
    bool nz = false;
    if (t < L) {
      const T* o = Oz + rows_row(O, t);
      const T* g = Gz + rows_row(dO, t);
      if (vec) {
        // a row before its chunk normally holds zeros: its product with O is then not needed
        const bool before_chunk = t < chunk_start;
        for (int cc = sub16 * V; cc < d; cc += 16 * V) {
          T a[V], b[V];
          *reinterpret_cast<uint4*>(b) = *reinterpret_cast<const uint4*>(g + cc);
          if (before_chunk) {
            bool any = false;
#pragma unroll
            for (int e = 0; e < V; ++e) any |= ((float)b[e] != 0.f);
            if (!any) continue;
          }
          *reinterpret_cast<uint4*>(a) = *reinterpret_cast<const uint4*>(o + cc);
#pragma unroll
          for (int e = 0; e < V; ++e) { s += (float)a[e] * (float)b[e]; nz |= ((float)b[e] != 0.f); }
        }
      } else {
        for (int cc = sub16; cc < d; cc += 16) {
          const float b = (float)g[(long)cc * dO.sc];
          s += (float)o[(long)cc * O.sc] * b;
          nz |= (b != 0.f);
        }
      }
    }
#pragma unroll
    for (int m = 8; m >= 1; m >>= 1) s += __shfl_xor(s, m, 64);
    if (sub16 == 0 && t < Lp) {
      if (Sz && t < L) {
        const float sv = Sz[rows_row(sub, t)];
        s -= sv;
        nz |= (sv != 0.f);
      }
      delta[(long)z * Lp + t] = s;
      if (Lz) lse2[(long)z * Lp + t] = (t < L) ? Lz[rows_row(lse_in, t)] * kLog2e : 0.f;
    }
    flag |= nz && t < chunk_start;
  }
  if (masked_nz && __any(flag)) {
    if ((threadIdx.x & 63) == 0 && *reinterpret_cast<volatile int*>(masked_nz) == 0) atomicOr(masked_nz, 1);
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
