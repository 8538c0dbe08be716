// Forward kernels.
//   k_carry        key-stationary pre-pass: per key s and per 32-query block tb the decay bias
//                  accumulated over all queries before the block (log2 units).
//   k_fwd_fused    query-stationary fused kernel: bias rebuilt per tile from the carries,
//                  online softmax across key tiles, O and log-sum-exp written once.
//   k_fwd_chunked  key-chunk-stationary kernel producing the per-chunk partial outputs and
//                  normalisers of the reference operator (universal_attention_autograd.py:9-38).
#pragma once
#include "ua_common.hpp"

namespace ua {

// marker stored in the log2-unit normaliser buffer for a (query, chunk) pair with no visible key
constexpr float kLseMasked = 3.0e38f;
constexpr float kNegBig = -1.0e30f;

// ---------------------------------------------------------------------------------------------
// C[z][tb][s] = sum_{u < 32*tb, u > s} log2(1 - A[s,u])      for tb >= s/32
// grid (Lp/128, Z_kv); 4 waves, wave w owns keys 32*(4*bx+w) .. +31 and sweeps query blocks.
// ---------------------------------------------------------------------------------------------
template <class T, int D>
__global__ void __launch_bounds__(256) k_carry(const T* __restrict__ Kp, const float* __restrict__ lsrc,
                                               const float* __restrict__ ldest, float* __restrict__ C, int Lp) {
  extern __shared__ __align__(16) char smem[];
  T* sKd = reinterpret_cast<T*>(smem);
  constexpr int NQ = D / 16, LS = lds_stride<T>(D);
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, col = lane & 31, hi = lane >> 5;
  const int z = blockIdx.y, nT = Lp / 32, sb = 4 * blockIdx.x + w;
  Frag<T> ks[NQ];
  {
    const T* krow = Kp + ((long)z * Lp + 32 * sb + col) * D + 8 * hi;
#pragma unroll
    for (int q = 0; q < NQ; ++q) ks[q] = ld8(krow + 16 * q);
  }
  const float la = lsrc[(long)z * Lp + 32 * sb + col];
  float carry = 0.f;
  float* Cz = C + (long)z * nT * Lp;
  for (int tb = 4 * blockIdx.x; tb < nT; ++tb) {
    __syncthreads();
    stage_tile(sKd, Kp + ((long)z * Lp + 32 * tb) * D, 32, D, D, LS, tid, 256);
    __syncthreads();
    if (tb >= sb) {
      f32x16 g = {0};
#pragma unroll
      for (int q = 0; q < NQ; ++q) mma(g, ld8(sKd + col * LS + 16 * q + 8 * hi), ks[q]);
      float lb[16];
      load_t16(ldest + (long)z * Lp + 32 * tb, hi, lb);
      float tot = 0.f;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        float l2 = log2_one_minus(affinity(log2_relu(g[v]), la + lb[v]));
        if (tb == sb && t_of(v, hi) <= col) l2 = 0.f;
        tot += l2;
      }
      tot += xor_lane(tot, 32);
      if (hi == 0) Cz[(long)tb * Lp + 32 * sb + col] = carry;
      carry += tot;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Fused forward.  grid (Lp/128, Z_q) ; 4 waves ; wave w owns queries 32*(4*jt+w) .. +31.
// Per key tile of BS keys: G = K_t.K_s -> A -> log2(1-A) -> in-lane prefix + carry = bias,
// S = Q_t.K_s, online softmax over keys, P^T through LDS, O += P^T V.
// ---------------------------------------------------------------------------------------------
template <class T, int D, int BS>
__global__ void __launch_bounds__(256) k_fwd_fused(const T* __restrict__ Qp, const T* __restrict__ Kp,
                                                   const T* __restrict__ VT, const float* __restrict__ lsrc,
                                                   const float* __restrict__ ldest, const float* __restrict__ C,
                                                   T* __restrict__ O, float* __restrict__ lse, float* __restrict__ lse2,
                                                   int R, int L, int Lp, int d) {
  extern __shared__ __align__(16) char smem[];
  constexpr int NQ = D / 16, NB = D / 32, NSB = BS / 32, LS = lds_stride<T>(D), PS = lds_stride<T>(BS);
  T* sKp = reinterpret_cast<T*>(smem);
  T* sVT = sKp + BS * LS;
  T* sP = sVT + D * PS;
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, col = lane & 31, hi = lane >> 5;
  const int zq = blockIdx.y, zk = zq / R, nT = Lp / 32;
  const int jt = gridDim.x - 1 - blockIdx.x, tb = 4 * jt + w;
  T* sPw = sP + w * 32 * PS;

  Frag<T> qf[NQ], kdf[NQ];
  {
    const T* qrow = Qp + ((long)zq * Lp + 32 * tb + col) * D + 8 * hi;
    const T* krow = Kp + ((long)zk * Lp + 32 * tb + col) * D + 8 * hi;
#pragma unroll
    for (int q = 0; q < NQ; ++q) { qf[q] = ld8(qrow + 16 * q); kdf[q] = ld8(krow + 16 * q); }
  }
  float lb[16];
  load_t16(ldest + (long)zk * Lp + 32 * tb, hi, lb);
  f32x16 o[NB];
#pragma unroll
  for (int n = 0; n < NB; ++n) o[n] = (f32x16){0};
  float m[16], ls[16];
#pragma unroll
  for (int v = 0; v < 16; ++v) { m[v] = kNegBig; ls[v] = 0.f; }
  const float* Crow = C + ((long)zk * nT + tb) * Lp;

  const int n_kt = (128 * jt + 128) / BS;
  for (int kt = 0; kt < n_kt; ++kt) {
    __syncthreads();
    stage_tile(sKp, Kp + ((long)zk * Lp + BS * kt) * D, BS, D, D, LS, tid, 256);
    stage_tile(sVT, VT + (long)zk * D * Lp + BS * kt, D, BS, Lp, PS, tid, 256);
    __syncthreads();
    f32x16 s2[NSB];
#pragma unroll
    for (int j = 0; j < NSB; ++j) {
      const int sbk = NSB * kt + j;
      if (sbk <= tb) {
        f32x16 g = {0};
#pragma unroll
        for (int q = 0; q < NQ; ++q) mma(g, kdf[q], ld8(sKp + (32 * j + col) * LS + 16 * q + 8 * hi));
        const bool diag = (sbk == tb);
        const float la = lsrc[(long)zk * Lp + 32 * sbk + col];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          float l2 = log2_one_minus(affinity(log2_relu(g[v]), la + lb[v]));
          g[v] = (diag && t_of(v, hi) <= col) ? 0.f : l2;
        }
        block_prefix(g, hi);
        const float c = Crow[32 * sbk + col];
        f32x16 sc = {0};
#pragma unroll
        for (int q = 0; q < NQ; ++q) mma(sc, qf[q], ld8(sKp + (32 * j + col) * LS + 16 * q + 8 * hi));
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          float x = __builtin_fmaf(sc[v], kLog2e, g[v] + c);
          s2[j][v] = (diag && t_of(v, hi) < col) ? kNegBig : x;
        }
      } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) s2[j][v] = kNegBig;
      }
    }
    // online softmax over this tile's keys
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      float mx = s2[0][v];
#pragma unroll
      for (int j = 1; j < NSB; ++j) mx = fmaxf(mx, s2[j][v]);
      mx = allmax32(mx);
      const float mn = fmaxf(m[v], mx);
      const float alpha = __builtin_amdgcn_exp2f(m[v] - mn);
      m[v] = mn;
      ls[v] *= alpha;
#pragma unroll
      for (int n = 0; n < NB; ++n) o[n][v] *= alpha;
#pragma unroll
      for (int j = 0; j < NSB; ++j) {
        float p = __builtin_amdgcn_exp2f(s2[j][v] - mn);
        ls[v] += p;
        sPw[t_of(v, hi) * PS + 32 * j + col] = cvt<T>(p);
      }
    }
    __syncthreads();
#pragma unroll
    for (int kq = 0; kq < BS / 16; ++kq) {
      if (NSB * kt + kq / 2 <= tb) {
        Frag<T> a = ld8(sPw + col * PS + 16 * kq + 8 * hi);
#pragma unroll
        for (int n = 0; n < NB; ++n) mma(o[n], a, ld8(sVT + (32 * n + col) * PS + 16 * kq + 8 * hi));
      }
    }
  }
  // epilogue
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const float tot = allsum32(ls[v]);
    const float inv = 1.0f / tot;
    const int t = 32 * tb + t_of(v, hi);
    if (t < L) {
#pragma unroll
      for (int n = 0; n < NB; ++n) {
        const int dd = 32 * n + col;
        if (dd < d) O[((long)zq * L + t) * d + dd] = cvt<T>(o[n][v] * inv);
      }
    }
    if (col == 0) {
      const float l2v = m[v] + __builtin_amdgcn_logf(tot);
      lse2[(long)zq * Lp + t] = (t < L) ? l2v : 0.f;
      if (t < L) lse[(long)zq * L + t] = l2v * kLn2;
    }
  }
}

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
        sP[t_of(v, hi) * PS + 32 * w + col] = cvt<T>(__builtin_amdgcn_exp2f(s2[v] - mm));
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
