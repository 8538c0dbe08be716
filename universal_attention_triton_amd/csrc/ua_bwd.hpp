// Backward kernels.
//   k_bwd_keys   key-stationary reverse sweep over query blocks.  A wave owns 32 keys and keeps
//                dV^T, dK^T (score part + row side of the affinity part) and the source-gate
//                gradient in registers; the suffix sum of dBias over queries is an in-lane scan
//                plus a per-key carry.  Query-side sums (dQ and the gradient w.r.t. the
//                destination-scaled key) leave the workgroup through fp32 atomics.
//   k_bwd_finish combines the partial gradients into the caller's tensors.
//
// Math per (key s, query t), see reference universal_attention_autograd.py:47-99:
//   P = exp(S - lse_t)            dS = P (V_s.dO_t - delta_t)           (delta carries -g_denom in chunked mode)
//   dBias = sum_r dS              dlog[s,u] = sum_{t>=u} dBias[s,t]  (u > s)
//   dA = dlog / (clamp(A,1e-6,1-1e-6) - 1) [A <= 1-1e-6]
// With g = k_s.k_u and A = relu(g)^(2/3) (src_s dest_u)^(1/3):
//   dg = dA (2/3) g^(-1/3) (src_s dest_u)^(1/3)   (g > 0)         [= (2/3) dA A / g]
//   dk_s += sum_u dg k_u   (row side, here)        dkcol_u = sum_s dg k_s   (column side, atomics)
//   dsrc_s = sum_u dA A / (3 src_s)
//   ddest_u = sum_s dA A / (3 dest_u) = (k_u . dkcol_u) / (2 dest_u)          (k_bwd_finish)
#pragma once
#include "ua_common.hpp"
#include "ua_fwd.hpp"

namespace ua {

template <class T>
struct BwdArgs {
  const int *reach, *minkey;    // pruning state of the fused mode: [Zk][Lp/16], [Zk][Lp/32]
  const int* masked_nz;         // chunked mode: non-zero when an upstream gradient of a (query, later chunk) pair is non-zero
  const T *Kp, *Vp;             // [Zk][Lp][D]
  const T *KT;                  // [Zk][D][Lp]
  const float *lsrc, *ldest;    // [Zk][Lp]  log2(gate)/3
  const T *Qp, *QT;             // [Zq][Lp][D], [Zq][D][Lp]
  const T *dOp, *dOT;           // [Zq*nch][Lp][D], [Zq*nch][D][Lp]
  const float *lse2, *delta;    // [Zq*nch][Lp]
  const float* C;               // [Zk][Lp/32][Lp]
  float *dQacc;                 // [Zq][Lp][D]  atomics (COLS only)
  float *dKdacc;                // [Zk][Lp][D]  atomics (COLS) / plain stores of k_bwd_queries
  float *Dsuf;                  // [Zk][Lp/32][Lp]  suffix carry of dBias entering each query block (!COLS)
  float *dKrow, *dVrow;         // [Zk][Lp][D]
  float* dsrc_raw;              // [Zk][Lp]
  // optional (16-bit dtypes, fused mode): k_bwd_keys2 leaves the score gradient dS [Zq] and the decay gradient dG [Zk]
  // of every visited (16 keys, 32 queries) tile, in operand precision, as [z][causal triangle of (16-query tile, 32-key half)
  // pairs, grouped by eight query tiles, see grp_tile] tiles of 1 KB laid out like StageT (32 keys x 16 queries); k_bwd_queries3 turns them into dQ and the column side of dK
  T *dS_st, *dG_st;
  const _Float16* Bt;           // with dS_st: fp16 bias tiles of k_carry2<BO>, [Zk][triangle, see tri_bias_row][1 KB]
  int R, L, Lp, c, nch, chunked, skip_masked;
  int split_r;                  // k_bwd_queries2: one workgroup per (kv head, query group); dKdacc is then [Zq][Lp][D]
  int key_parts;                // k_bwd_keys2: sweeps per kv head (1 .. R, a divisor of R); dKrow, dVrow, dsrc_raw and dG_st hold one slice per (kv head, part)
  // direct (tile exchange, r = 1): the two kernels write the caller's gradients themselves and k_bwd_finish is not run:
  // k_bwd_keys2 dv and dsrc, k_bwd_queries3 dk (row side from dKrow + its own column side) and ddest.
  // dk_out, dv_out [Z][L][d_out]; dsrc_out, ddest_out and the caller's gates src_in, dest_in [Z][L].
  int direct, d_out;
  T *dk_out, *dv_out, *dsrc_out, *ddest_out;
  const T *src_in, *dest_in;
  // chunked operator with tile exchange: dOp is not the packed copy but the caller's upstream gradient itself, stored
  // chunk-major as rows of exactly D elements, [Zq*nch][L][D] with L a multiple of 32 (k_bwd_keys2 gathers its tiles)
  int dO_rows;
};

// grid (key groups, Zk).  chunked == 0: key group = 128 consecutive keys, 4 waves.
// chunked == 1: key group = min(c, 32*NW) keys of ONE chunk (gridDim.x = nch * ceil(c / (32*NW))).
// Chunked mode (COLS = true): also produces the query-side sums (dQ, dkcol) through atomics.  The fused
// mode uses k_bwd_keys2 / k_bwd_queries2 (ua_fused.hpp) instead.
template <class T, int D, int NW, bool COLS>
__global__ void __launch_bounds__(64 * NW) k_bwd_keys(BwdArgs<T> a) {
  extern __shared__ __align__(16) char smem[];
  constexpr int NQ = D / 16, NB = D / 32, LS = lds_stride<T>(D), TS = lds_stride<T>(32), CP = 32 * NW,
                SS = lds_stride<T>(CP), NT = 64 * NW, NBW = (NB + NW - 1) / NW, NKQ = CP / 16;
  T* sKd = reinterpret_cast<T*>(smem);
  T* sQ = sKd + 32 * LS;
  T* sdO = sQ + 32 * LS;
  T* sKdT = sdO + 32 * LS;
  T* sQT = sKdT + D * TS;
  T* sdOT = sQT + D * TS;
  T* sX = sdOT + D * TS;                                  // [32 t][SS]  transposed dS / dg staging
  float* sStat = reinterpret_cast<float*>(sX + 32 * SS);  // lse2[32], delta[32]
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, col = lane & 31, hi = lane >> 5;
  const int zk = blockIdx.y, Lp = a.Lp, L = a.L, nT = Lp / 32;

  int chunk_i = 0, wg_key0, wg_keys;
  if (a.chunked) {
    const int gpc = (a.c + CP - 1) / CP;                  // key groups per chunk
    chunk_i = blockIdx.x / gpc;
    const int sub = blockIdx.x - chunk_i * gpc;
    wg_key0 = chunk_i * a.c + sub * CP;
    wg_keys = min(CP, a.c - sub * CP);
  } else {
    wg_key0 = (gridDim.x - 1 - blockIdx.x) * CP;          // light (late) key groups last
    wg_keys = CP;
  }
  const int kbase = wg_key0 + 32 * w;
  const bool valid = (32 * w + col) < wg_keys;
  const int spos = kbase + col;
  const int tb_first = kbase / 32;                        // query block holding this wave's first key
  const bool wave_live = (32 * w) < wg_keys;
  const float inv_c = 1.0f / (float)a.c;

  Frag<T> kp[NQ], vf[NQ];
  {
    const long ro = ((long)zk * Lp + spos) * D + 8 * hi;
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      if (valid) { kp[q] = ld8(a.Kp + ro + 16 * q); vf[q] = ld8(a.Vp + ro + 16 * q); }
      else {
#pragma unroll
        for (int e = 0; e < 8; ++e) { kp[q].v[e] = cvt<T>(0.f); vf[q].v[e] = cvt<T>(0.f); }
      }
    }
  }
  const float la = valid ? a.lsrc[(long)zk * Lp + min(spos, Lp - 1)] : kGatePad;

  f32x16 dVt[NB], dKt[NB];
#pragma unroll
  for (int n = 0; n < NB; ++n) { dVt[n] = (f32x16){0}; dKt[n] = (f32x16){0}; }
  float dsrc_acc = 0.f, dcar = 0.f;

  const int nTr = (L + 31) / 32;
  const int tb_lo = (a.chunked && !a.skip_masked) ? 0 : wg_key0 / 32;
  for (int tb = nTr - 1; tb >= tb_lo; --tb) {
    // mode of this wave for this query block: 2 = has decay part, 1 = score part only (no visible key), 0 = idle
    const int mode = !wave_live ? 0 : (tb >= tb_first ? 2 : ((a.chunked && !a.skip_masked) ? 1 : 0));
    __syncthreads();
    stage_tile(sKd, a.Kp + ((long)zk * Lp + 32 * tb) * D, 32, D, D, LS, tid, NT);
    stage_tile(sKdT, a.KT + (long)zk * D * Lp + 32 * tb, D, 32, Lp, TS, tid, NT);
    __syncthreads();
    f32x16 aff, bias, gk;      // gk holds log2(relu(k_s.k_t)) after the forward recompute
    float lab[16];
    if (mode == 2) {
      gk = (f32x16){0};
#pragma unroll
      for (int q = 0; q < NQ; ++q) mma(gk, ld8(sKd + col * LS + 16 * q + 8 * hi), kp[q]);
      load_t16(a.ldest + (long)zk * Lp + 32 * tb, hi, lab);
      f32x16 x;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int tpos = 32 * tb + t_of(v, hi);
        lab[v] += la;
        gk[v] = log2_relu(gk[v]);
        aff[v] = affinity(gk[v], lab[v]);
        const float l2 = log2_one_minus(aff[v]);
        x[v] = (valid && tpos > spos) ? l2 : 0.f;
      }
      block_prefix(x, hi);
      const float cin = a.C[((long)zk * (Lp / 16) + 2 * tb) * Lp + min(spos, Lp - 1)];   // carries are kept per 16-query tile
#pragma unroll
      for (int v = 0; v < 16; ++v) bias[v] = x[v] + cin;
    }
    f32x16 dB = {0};
    for (int r = 0; r < a.R; ++r) {
      const long zq = (long)zk * a.R + r;
      const long zi = a.chunked ? zq * a.nch + chunk_i : zq;
      __syncthreads();
      stage_tile(sQ, a.Qp + (zq * Lp + 32 * tb) * D, 32, D, D, LS, tid, NT);
      stage_tile(sdO, a.dOp + (zi * Lp + 32 * tb) * D, 32, D, D, LS, tid, NT);
      stage_tile(sQT, a.QT + zq * D * Lp + 32 * tb, D, 32, Lp, TS, tid, NT);
      stage_tile(sdOT, a.dOT + zi * D * Lp + 32 * tb, D, 32, Lp, TS, tid, NT);
      if (tid < 32) sStat[tid] = a.lse2[zi * Lp + 32 * tb + tid];
      else if (tid < 64) sStat[tid] = a.delta[zi * Lp + 32 * tb + tid - 32];
      __syncthreads();
      f32x16 dS;
      if (mode != 0) {
        f32x16 sc = {0}, dP = {0};
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
          mma(sc, ld8(sQ + col * LS + 16 * q + 8 * hi), kp[q]);
          mma(dP, ld8(sdO + col * LS + 16 * q + 8 * hi), vf[q]);
        }
        f32x16 P;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int tl = t_of(v, hi), tpos = 32 * tb + tl;
          const float l2t = sStat[tl], dlt = sStat[32 + tl];
          float p;
          if (l2t >= 1.0e38f) p = valid ? inv_c : 0.f;                 // query sees no key of the chunk: uniform
          else if (mode == 2 && valid && tpos >= spos) p = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[v], kLog2e, bias[v]) - l2t);
          else p = 0.f;
          P[v] = p;
          dS[v] = p * (dP[v] - dlt);
          dB[v] += dS[v];
        }
#pragma unroll
        for (int q2 = 0; q2 < 2; ++q2) {
          const Frag<T> bp = as_operand<T>(P, q2), bs = as_operand<T>(dS, q2);
#pragma unroll
          for (int n = 0; n < NB; ++n) {
            mma(dVt[n], ld8(sdOT + (32 * n + col) * TS + 16 * q2 + 8 * hi), bp);
            mma(dKt[n], ld8(sQT + (32 * n + col) * TS + 16 * q2 + 8 * hi), bs);
          }
        }
      } else {
        dS = (f32x16){0};
      }
      // ---- query side: dQ[t,:] += sum_s dS[s,t] k_s   (all keys of the workgroup, then atomics)
      if constexpr (COLS) {
#pragma unroll
      for (int v = 0; v < 16; ++v) sX[t_of(v, hi) * SS + 32 * w + perm16(col)] = cvt<T>(dS[v]);
      __syncthreads();
#pragma unroll
      for (int nb = 0; nb < NBW; ++nb) {
        const int n = w + nb * NW;
        if (n < NB) {
          f32x16 acc = {0};
#pragma unroll
          for (int kq = 0; kq < NKQ; ++kq) {
            const int s0 = wg_key0 + 16 * kq + 8 * hi;
            if (s0 + 8 <= Lp)
              mma(acc, ld8(sX + col * SS + 16 * kq + 8 * hi), ld8(a.KT + ((long)zk * D + 32 * n + col) * Lp + s0));
          }
#pragma unroll
          for (int v = 0; v < 16; ++v)
            atomicAdd(a.dQacc + (zq * Lp + 32 * tb + t_of(v, hi)) * D + 32 * n + col, acc[v]);
        }
      }
      }
    }
    // ---- decay part
    f32x16 dg;
    if (mode == 2) {
      if constexpr (!COLS) {
        if (valid && hi == 0) a.Dsuf[((long)zk * nT + tb) * Lp + spos] = dcar;
      }
      const float tot = block_suffix(dB, hi);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int tpos = 32 * tb + t_of(v, hi);
        const float dl = (valid && tpos > spos) ? dB[v] + dcar : 0.f;
        const float av = aff[v];
        const float den = fmaxf(fminf(av, kAMax), kAMinBwd) - 1.0f;
        const float dA = (av <= kAMax) ? dl * __builtin_amdgcn_rcpf(den) : 0.f;
        dsrc_acc += dA * av;
        // (2/3) g^(-1/3) (src dest)^(1/3); g <= 0 (log2 = -inf) contributes nothing
        const float f = (2.0f / 3.0f) * __builtin_amdgcn_exp2f(__builtin_fmaf(gk[v], -1.0f / 3.0f, lab[v]));
        dg[v] = (gk[v] > -1.0e30f) ? dA * f : 0.f;
      }
      dcar += tot;
#pragma unroll
      for (int q2 = 0; q2 < 2; ++q2) {
        const Frag<T> b = as_operand<T>(dg, q2);
#pragma unroll
        for (int n = 0; n < NB; ++n) mma(dKt[n], ld8(sKdT + (32 * n + col) * TS + 16 * q2 + 8 * hi), b);
      }
    } else {
      dg = (f32x16){0};
    }
    if constexpr (COLS) {
    __syncthreads();
#pragma unroll
    for (int v = 0; v < 16; ++v) sX[t_of(v, hi) * SS + 32 * w + perm16(col)] = cvt<T>(dg[v]);
    __syncthreads();
    if (tb >= wg_key0 / 32) {
#pragma unroll
      for (int nb = 0; nb < NBW; ++nb) {
        const int n = w + nb * NW;
        if (n < NB) {
          f32x16 acc = {0};
#pragma unroll
          for (int kq = 0; kq < NKQ; ++kq) {
            const int s0 = wg_key0 + 16 * kq + 8 * hi;
            if (s0 + 8 <= Lp)
              mma(acc, ld8(sX + col * SS + 16 * kq + 8 * hi), ld8(a.KT + ((long)zk * D + 32 * n + col) * Lp + s0));
          }
#pragma unroll
          for (int v = 0; v < 16; ++v)
            atomicAdd(a.dKdacc + ((long)zk * Lp + 32 * tb + t_of(v, hi)) * D + 32 * n + col, acc[v]);
        }
      }
    }
    }
  }
  // ---- epilogue: key-side results
  dsrc_acc += xor_lane(dsrc_acc, 32);
  if (valid && spos < Lp) {
    if (hi == 0) a.dsrc_raw[(long)zk * Lp + spos] = dsrc_acc;
#pragma unroll
    for (int n = 0; n < NB; ++n) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const long o = ((long)zk * Lp + spos) * D + 32 * n + 8 * g + 4 * hi;
        *reinterpret_cast<float4*>(a.dVrow + o) = make_float4(dVt[n][4 * g], dVt[n][4 * g + 1], dVt[n][4 * g + 2], dVt[n][4 * g + 3]);
        *reinterpret_cast<float4*>(a.dKrow + o) = make_float4(dKt[n][4 * g], dKt[n][4 * g + 1], dKt[n][4 * g + 2], dKt[n][4 * g + 3]);
      }
    }
  }
}

// Combine partial gradients into the caller's contiguous tensors:
//   dk [Zk][L][d], dv [Zk][L][d], dq [Zq][L][d], dsrc [Zk][L], ddest [Zk][L]
// grid (ceil(L/4), max(Zk, Zq)); one wave per row.  The fp32 partial gradients are row-major [Z][Lp][D].
// TG: dtype of the gates and of their gradients (the reference allocates dstatic_src in static_src.dtype,
// Universal_Attention/triton/universal_attention_kernel.py:828)
template <class T, class TG = T>
__global__ void __launch_bounds__(256) k_bwd_finish(const float* __restrict__ dKrow, const float* __restrict__ dVrow,
                                                    const float* __restrict__ dKdacc, const float* __restrict__ dQacc,
                                                    const float* __restrict__ dsrc_raw, const T* __restrict__ Kp,
                                                    const TG* __restrict__ src, const TG* __restrict__ dest,
                                                    T* __restrict__ dk, T* __restrict__ dv, T* __restrict__ dq,
                                                    TG* __restrict__ dsrc, TG* __restrict__ ddest, int Zk, int Zq, int L,
                                                    int Lp, int D, int d, int tiled, int RS, int RK) {
  const int z = blockIdx.y, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + wave;
  if (t >= L) return;
  if (z < Zq && dQacc) {
    for (int c = lane; c < d; c += 64) dq[((long)z * L + t) * d + c] = cvt<T>(dQacc[((long)z * Lp + t) * D + c]);
  }
  if (z < Zk) {
    const float sd = (float)dest[(long)z * L + t];
    float dot = 0.f;
    for (int c = lane; c < d; c += 64) {
      const long i = ((long)z * Lp + t) * D + c;
      // RS > 1: the column side comes in one slice per query group of the head
      float kd = 0.f;
      for (int r = 0; r < RS; ++r) kd += dKdacc[(((long)z * RS + r) * Lp + t) * D + c];
      // the packed keys are row-major in chunked mode and tiled (nat_off) in fused mode
      const long ik = !tiled ? i : (D == 64 ? nat_off<64>(z, Lp, t, c) : (D == 128 ? nat_off<128>(z, Lp, t, c) : nat_off<256>(z, Lp, t, c)));
      dot += kd * (float)Kp[ik];
      // RK > 1: so does the row side, and dV
      float kr = 0.f, vr = 0.f;
      for (int r = 0; r < RK; ++r) {
        const long ir = (((long)z * RK + r) * Lp + t) * D + c;
        kr += dKrow[ir];
        vr += dVrow[ir];
      }
      dk[((long)z * L + t) * d + c] = cvt<T>(kr + kd);
      dv[((long)z * L + t) * d + c] = cvt<T>(vr);
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) dot += __shfl_xor(dot, m, 64);
    if (lane == 0) {
      ddest[(long)z * L + t] = cvt<TG>(dot / (2.0f * sd));
      float sr = 0.f;
      for (int r = 0; r < RK; ++r) sr += dsrc_raw[((long)z * RK + r) * Lp + t];
      dsrc[(long)z * L + t] = cvt<TG>(sr / (3.0f * (float)src[(long)z * L + t]));
    }
  }
}

}  // namespace ua
