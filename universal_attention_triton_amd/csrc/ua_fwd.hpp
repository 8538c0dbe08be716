// Chunked forward kernel.
//   k_fwd_chunked  key-chunk-stationary kernel producing the per-chunk partial outputs and
//                  normalisers of the reference operator (universal_attention_autograd.py:9-38).
#pragma once
#include "ua_common.hpp"

namespace ua {

constexpr float kLseMasked = kNoKeyLse;
constexpr float kNegBig = -1.0e30f;

// ---------------------------------------------------------------------------------------------
// Chunked forward (reference operator semantics).  grid (n_chunks, Z_kv); NW = ceil(c/32) waves.
// Wave w owns keys i*c + 32w .. (valid while < (i+1)*c).  For every query block and every query
// group r: softmax over the keys of the chunk only, out[t,:,i] = P^T V_i, denom[t,i] = lse.
// Queries before the chunk see no key: reference gives the uniform softmax there
// (out = mean of the chunk's values through a dtype-rounded 1/c, denom = float32(-1e12)).
// out element (zq, t, dd, i) is written at  zq*o_sz + t*o_st + dd*o_sd + i*o_si.
// ---------------------------------------------------------------------------------------------
template <class T, int D, int NW>
__global__ void __launch_bounds__(64 * NW) k_fwd_chunked(const T* __restrict__ Qp, const T* __restrict__ Kp,
                                                         const T* __restrict__ VT, const float* __restrict__ lsrc,
                                                         const float* __restrict__ ldest, T* __restrict__ out,
                                                         T* __restrict__ denom, float* __restrict__ lse2,
                                                         long o_sz, long o_st, long o_sd, long o_si,
                                                         int R, int L, int Lp, int d, int c, int nch) {
  extern __shared__ __align__(16) char smem[];
  constexpr int NQ = D / 16, NB = D / 32, LS = lds_stride<T>(D), CP = 32 * NW, PS = lds_stride<T>(CP);
  constexpr int NBW = (NB + NW - 1) / NW, NKQ = CP / 16, NT = 64 * NW;
  T* sKd = reinterpret_cast<T*>(smem);
  T* sQ = sKd + 32 * LS;
  T* sP = sQ + 32 * LS;
  float* sM = reinterpret_cast<float*>(sP + 32 * PS);   // [NW][32]
  float* sMean = sM + NW * 32;                          // [D]
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, col = lane & 31, hi = lane >> 5;
  const int i = blockIdx.x, zk = blockIdx.y;
  const int kbase = i * c + 32 * w;
  const bool valid = (32 * w + col) < c;
  const int spos = kbase + col;
  const int nTr = (L + 31) / 32, tb0 = (i * c) / 32;
  const float kFill2 = kNegFill * kLog2e;

  Frag<T> kp[NQ];
  {
    const T* b = Kp + ((long)zk * Lp + spos) * D + 8 * hi;
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      if (valid) kp[q] = ld8(b + 16 * q);
      else {
#pragma unroll
        for (int e = 0; e < 8; ++e) kp[q].v[e] = cvt<T>(0.f);
      }
    }
  }
  const float la = valid ? lsrc[(long)zk * Lp + spos] : kGatePad;
  // V^T operands of this wave's output column blocks: lane <-> dd, k <-> key inside the chunk
  Frag<T> vt[NBW][NKQ];
  Frag<T> ones;
#pragma unroll
  for (int e = 0; e < 8; ++e) ones.v[e] = cvt<T>(1.f);
#pragma unroll
  for (int nb = 0; nb < NBW; ++nb) {
    const int n = w + nb * NW;
#pragma unroll
    for (int kq = 0; kq < NKQ; ++kq) {
      const int s0 = i * c + 16 * kq + 8 * hi;
      if (n < NB && s0 + 8 <= Lp) vt[nb][kq] = ld8(VT + ((long)zk * D + 32 * n + col) * Lp + s0);
      else {
#pragma unroll
        for (int e = 0; e < 8; ++e) vt[nb][kq].v[e] = cvt<T>(0.f);
      }
    }
  }
  // ---- queries before the chunk: uniform softmax over the c keys
  if (tb0 > 0) {
    const T pu = cvt<T>(1.0f / (float)c);
    for (int dd = tid; dd < D; dd += NT) {
      float acc = 0.f;
      for (int s = 0; s < c; ++s) acc += (float)pu * (float)VT[((long)zk * D + dd) * Lp + i * c + s];
      sMean[dd] = acc;
    }
    __syncthreads();
    const int rows = 32 * tb0;
    for (int r = 0; r < R; ++r) {
      const long zq = (long)zk * R + r;
      if (out) {
        for (int idx = tid; idx < rows * d; idx += NT) {
          int t = idx / d, dd = idx - t * d;
          out[zq * o_sz + t * o_st + dd * o_sd + i * o_si] = cvt<T>(sMean[dd]);
        }
      }
      for (int t = tid; t < rows; t += NT) {
        if (denom) denom[(zq * L + t) * nch + i] = cvt<T>(kNegFill);
        lse2[(zq * nch + i) * Lp + t] = kLseMasked;
      }
    }
  }
  float carry = 0.f;
  for (int tb = tb0; tb < nTr; ++tb) {
    __syncthreads();
    stage_tile(sKd, Kp + ((long)zk * Lp + 32 * tb) * D, 32, D, D, LS, tid, NT);
    __syncthreads();
    f32x16 bias;
    {
      f32x16 g = {0};
#pragma unroll
      for (int q = 0; q < NQ; ++q) mma(g, ld8(sKd + col * LS + 16 * q + 8 * hi), kp[q]);
      float lb[16];
      load_t16(ldest + (long)zk * Lp + 32 * tb, hi, lb);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int tpos = 32 * tb + t_of(v, hi);
        float l2 = log2_one_minus(affinity(log2_relu(g[v]), la + lb[v]));
        g[v] = (valid && tpos > spos) ? l2 : 0.f;
      }
      const float tot = block_prefix(g, hi);
#pragma unroll
      for (int v = 0; v < 16; ++v) bias[v] = g[v] + carry;
      carry += tot;
    }
    for (int r = 0; r < R; ++r) {
      const long zq = (long)zk * R + r;
      __syncthreads();
      stage_tile(sQ, Qp + (zq * Lp + 32 * tb) * D, 32, D, D, LS, tid, NT);
      __syncthreads();
      f32x16 sc = {0};
#pragma unroll
      for (int q = 0; q < NQ; ++q) mma(sc, ld8(sQ + col * LS + 16 * q + 8 * hi), kp[q]);
      float s2[16];
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int tpos = 32 * tb + t_of(v, hi);
        float x = __builtin_fmaf(sc[v], kLog2e, bias[v]);
        x = (tpos >= spos) ? x : kFill2;
        s2[v] = valid ? x : -3.0e38f;
        const float mw = allmax32(s2[v]);
        if (col == 0) sM[w * 32 + t_of(v, hi)] = mw;
      }
      __syncthreads();
      float m[16];
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        float mm = sM[t_of(v, hi)];
#pragma unroll
        for (int ww = 1; ww < NW; ++ww) mm = fmaxf(mm, sM[ww * 32 + t_of(v, hi)]);
        m[v] = mm;
        sP[t_of(v, hi) * PS + 32 * w + perm16(col)] = cvt<T>(__builtin_amdgcn_exp2f(s2[v] - mm));
      }
      __syncthreads();
      f32x16 osum = {0};
      f32x16 o[NBW];
#pragma unroll
      for (int nb = 0; nb < NBW; ++nb) o[nb] = (f32x16){0};
#pragma unroll
      for (int kq = 0; kq < NKQ; ++kq) {
        Frag<T> a = ld8(sP + col * PS + 16 * kq + 8 * hi);
        mma(osum, a, ones);
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb) mma(o[nb], a, vt[nb][kq]);
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int t = 32 * tb + t_of(v, hi);
        if (t >= L) {   // padded query rows: keep the normaliser buffer finite
          if (w == 0 && col == 0) lse2[(zq * nch + i) * Lp + t] = 0.f;
          continue;
        }
        const float inv = 1.0f / osum[v];
        if (out) {
#pragma unroll
          for (int nb = 0; nb < NBW; ++nb) {
            const int n = w + nb * NW, dd = 32 * n + col;
            if (n < NB && dd < d) out[zq * o_sz + t * o_st + dd * o_sd + i * o_si] = cvt<T>(o[nb][v] * inv);
          }
        }
        if (w == 0 && col == 0) {
          const bool none = m[v] < -1.0e11f;
          const float l2v = m[v] + __builtin_amdgcn_logf(osum[v]);
          if (denom) denom[(zq * L + t) * nch + i] = cvt<T>(none ? kNegFill : l2v * kLn2);
          lse2[(zq * nch + i) * Lp + t] = none ? kLseMasked : l2v;
        }
      }
    }
  }
}

}  // namespace ua
