// Stand-alone decay bias ("affinity scores") of the second-generation reference interface
// (Universal_Attention/triton/affinity_kernel_opt.py:100-127 forward, :425-450 autograd wrapper, :457-462 torch form):
//
//   aff[b,h,t,s] = sum_{s<u<=t} ln(1 - min(A[s,u], 1-1e-6))   for s < t,   0 for s == t,   -1e12 for s > t
//   A[s,u] = relu(k_s.k_u)^(2/3) (src_s dest_u)^(1/3)
//
// i.e. the L x L matrix users hand to a generic attention as an additive mask; [query t][key s], dtype of k.
// The backward takes d aff and returns dk, dsrc, ddest.  With DL[u][s] = sum_{t>=u} daff[t][s] (one reverse running
// sum down every column) the gradient of the key-key product is W[s,u] = DL[u][s] F[s,u] for u > s (F = decay_grad
// with dl = 1), and
//   dk_s = sum_{u>s} W[s,u] k_u + sum_{u<s} W[u,s] k_u,   dsrc_s = sum_u W[s,u] G[s,u] / (2 src_s),
//   ddest_u = sum_s W[s,u] G[s,u] / (2 dest_u).
// Both sums are the same kernel with the roles of the two indices exchanged (k_aff_bwd_side<COL>).
#pragma once
#include "ua_common.hpp"
#include "ua_fused.hpp"

namespace ua {

// The pipeline macros of ua_fused.hpp are private to that header; these kernels use a plain two-stage loop.
// grid (Lp/128, Z), 8 waves; wave w owns keys 16*(8*bx+w)..+15 and sweeps the 32-query blocks from its own on.
template <class T, int D>
__global__ void __launch_bounds__(512) k_aff_fwd(const T* __restrict__ Kp, const float* __restrict__ lsrc,
                                                 const float* __restrict__ ldest, T* __restrict__ aff, int L, int Lp) {
  using TN = Tile<T, 32, D>;
  constexpr int NK = D / 32, SB = TN::BYTES + 1024;
  __shared__ __attribute__((aligned(1024))) char stage[2][SB];
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, col = lane & 15, g = lane >> 4;
  const int bx = blockIdx.x, z = blockIdx.y;
  const int nT = Lp / 32, sb16 = 8 * bx + w, first = 4 * bx, own = sb16 >> 1;
  const int spos = 16 * sb16 + col;
  const GroupMasks gm = group_masks(lane);
  Stager<TN, 8> st;
  st.init(w, lane, D * (long)sizeof(T), 32);
  Frag<T> ks[NK];
#pragma unroll
  for (int q = 0; q < NK; ++q) ks[q] = ld8(Kp + nat_off<D>(z, Lp, spos, 32 * q + 8 * g));
  const float la = lsrc[(long)z * Lp + spos];
  const T* Kz = Kp + (long)z * Lp * D;
  T* az = aff + (long)z * L * L;
  const T fill = cvt<T>(kNegFill);
  // queries before the wave's own block see none of its keys
  if (spos < L)
    for (int t = g; t < min(32 * own, L); t += 4) az[(long)t * L + spos] = fill;
  float carry = 0.f;
  const int total = nT - first;
  auto issue = [&] __device__ (int s, char* base) __attribute__((always_inline)) {
    st.issue(base, Kz + (long)32 * (first + s) * D, w);
    if (w == 0) issue_row(base + TN::BYTES, ldest + (long)z * Lp + 32 * (first + s) + 4 * (lane & 7));
  };
  issue(0, stage[0]);
  for (int s = 0; s < total; ++s) {
    wait_async_loads();
    __syncthreads();
    if (s + 1 < total) issue(s + 1, stage[(s + 1) & 1]);
    const int tb = first + s;
    if (tb < own) continue;
    const char* base = stage[s & 1];
    const T* sK = reinterpret_cast<const T*>(base);
    const float* stats = reinterpret_cast<const float*>(base + TN::BYTES);
    f32x4 x[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      f32x4 acc = {0, 0, 0, 0};
#pragma unroll
      for (int q = 0; q < NK; ++q) mma16(acc, ld8(sK + TN::at(i, col, q, g)), ks[q]);
      const f32x4 lb = load_t4(stats + 16 * i, g);
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const float l2 = log2_one_minus(affinity(log2_relu(acc[v]), la + lb[v]));
        x[i][v] = (32 * tb + 16 * i + 4 * g + v <= spos) ? 0.f : l2;
      }
    }
    const float tot = prefix32(x[0], x[1], gm);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int t = 32 * tb + 16 * i + 4 * g + v;
        if (t < L && spos < L) az[(long)t * L + spos] = (t < spos) ? fill : cvt<T>((x[i][v] + carry) * kLn2);
      }
    carry += tot;
  }
}

// DL[z][u][s] = sum_{t >= u} daff[z][t][s]   (float32); one thread per column s
template <class T>
__global__ void __launch_bounds__(256) k_aff_revcumsum(const T* __restrict__ daff, float* __restrict__ DL, int L) {
  const int s = blockIdx.x * 256 + threadIdx.x, z = blockIdx.y;
  if (s >= L) return;
  const T* p = daff + (long)z * L * L + s;
  float* q = DL + (long)z * L * L + s;
  float acc = 0.f;
  for (int t = L - 1; t >= 0; --t) {
    acc += (float)p[(long)t * L];
    q[(long)t * L] = acc;
  }
}

// One side of the key gradient.  grid (Lp/128, Z), 8 waves; wave w owns the 16 positions i = 16*(8*bx+w)..+15 and
// sweeps the blocks of 32 positions j on its side of the diagonal.
//   COL = false (i = key s, j = later key u):   W = DL[j][i] F(G, src_i dest_j),  j > i
//   COL = true  (i = later key u, j = key s):   W = DL[i][j] F(G, src_j dest_i),  j < i
//   out[z][i][:] = sum_j W k_j          gsum[z][i] = sum_j W relu(G)
template <class T, int D, bool COL>
__global__ void __launch_bounds__(512) k_aff_bwd_side(const T* __restrict__ Kp, const T* __restrict__ KT,
                                                      const float* __restrict__ lsrc, const float* __restrict__ ldest,
                                                      const float* __restrict__ DL, float* __restrict__ out,
                                                      float* __restrict__ gsum, int L, int Lp) {
  using TN = Tile<T, 32, D>;
  using TT = Tile<T, D, 32>;
  constexpr int NK = D / 32, ND = D / 16, SB = TN::BYTES + TT::BYTES + 1024;
  __shared__ __attribute__((aligned(1024))) char stage[2][SB];
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, col = lane & 15, g = lane >> 4;
  const int bx = blockIdx.x, z = blockIdx.y;
  const int nT = Lp / 32, ib16 = 8 * bx + w, own = ib16 >> 1;
  const int ipos = 16 * ib16 + col;
  Stager<TN, 8> stN;
  Stager<TT, 8> stT;
  stN.init(w, lane, D * (long)sizeof(T), 32);
  stT.init(w, lane, Lp * (long)sizeof(T), D);
  Frag<T> ki[NK];
#pragma unroll
  for (int q = 0; q < NK; ++q) ki[q] = ld8(Kp + nat_off<D>(z, Lp, ipos, 32 * q + 8 * g));
  // log-gate of the stationary position and of the swept ones
  const float* gate_i = COL ? ldest : lsrc;
  const float* gate_j = COL ? lsrc : ldest;
  const float li = gate_i[(long)z * Lp + ipos];
  const T* Kz = Kp + (long)z * Lp * D;
  const T* KTz = KT + (long)z * D * Lp;
  const float* DLz = DL + (long)z * L * L;
  f32x4 acc_o[ND];
#pragma unroll
  for (int n = 0; n < ND; ++n) acc_o[n] = (f32x4){0, 0, 0, 0};
  float gs = 0.f;
  // blocks swept by the workgroup: its own four and everything after (rows) or before (columns)
  const int jb0 = COL ? 0 : 4 * bx, jb1 = COL ? min(4 * bx + 4, nT) : nT, total = jb1 - jb0;
  auto issue = [&] __device__ (int s, char* base) __attribute__((always_inline)) {
    const int jb = jb0 + s;
    stN.issue(base, Kz + (long)(32 * jb) * D, w);
    stT.issue(base + TN::BYTES, KTz + (long)(32 * jb) * D, w);
    if (w == 0) issue_row(base + TN::BYTES + TT::BYTES, gate_j + (long)z * Lp + 32 * jb + 4 * (lane & 7));
  };
  issue(0, stage[0]);
  for (int s = 0; s < total; ++s) {
    wait_async_loads();
    __syncthreads();
    if (s + 1 < total) issue(s + 1, stage[(s + 1) & 1]);
    const int jb = jb0 + s;
    if (COL ? jb > own : jb < own) continue;
    const char* base = stage[s & 1];
    const T* sK = reinterpret_cast<const T*>(base);
    const T* sKT = reinterpret_cast<const T*>(base + TN::BYTES);
    const float* stats = reinterpret_cast<const float*>(base + TN::BYTES + TT::BYTES);
    f32x4 W[2];
#pragma unroll
    for (int i2 = 0; i2 < 2; ++i2) {
      f32x4 acc = {0, 0, 0, 0};
#pragma unroll
      for (int q = 0; q < NK; ++q) mma16(acc, ld8(sK + TN::at(i2, col, q, g)), ki[q]);
      const f32x4 lj = load_t4(stats + 16 * i2, g);
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int jpos = 32 * jb + 16 * i2 + 4 * g + v;
        const bool valid = (COL ? jpos < ipos : jpos > ipos) && jpos < L && ipos < L;
        const float gk = fmaxf(acc[v], 0.f);
        const float a = affinity(__builtin_amdgcn_logf(gk), li + lj[v]);
        float wv = 0.f;
        if (valid) wv = DLz[COL ? (long)ipos * L + jpos : (long)jpos * L + ipos] * decay_grad(1.0f, a, gk);
        W[i2][v] = wv;
        gs = __builtin_fmaf(wv, gk, gs);
      }
    }
    const Frag<T> b = as_operand16<T>(W[0], W[1]);
#pragma unroll
    for (int n = 0; n < ND; ++n) mma16(acc_o[n], ld8(sKT + TT::at(n, col, 0, g)), b);
  }
  {
    const GroupMasks gm = group_masks(lane);
    float b, af, tot;
    group_scan(gs, gm, b, af, tot);
    if (g == 0) gsum[(long)z * Lp + ipos] = tot;
  }
#pragma unroll
  for (int n = 0; n < ND; ++n) {
    const long o = ((long)z * Lp + ipos) * D + 16 * n + 4 * g;
    *reinterpret_cast<float4*>(out + o) = make_float4(acc_o[n][0], acc_o[n][1], acc_o[n][2], acc_o[n][3]);
  }
}

// dk = row side + column side; dsrc = gsum_row / (2 src); ddest = gsum_col / (2 dest)   (sum W G = 3/2 sum dA A)
template <class T>
__global__ void __launch_bounds__(256) k_aff_finish(const float* __restrict__ row, const float* __restrict__ colp,
                                                    const float* __restrict__ gs_row, const float* __restrict__ gs_col,
                                                    const T* __restrict__ src, const T* __restrict__ dest, T* __restrict__ dk,
                                                    T* __restrict__ dsrc, T* __restrict__ ddest, int L, int Lp, int D, int d) {
  const int z = blockIdx.y, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + wave;
  if (t >= L) return;
  for (int c = lane; c < d; c += 64) {
    const long i = ((long)z * Lp + t) * D + c;
    dk[((long)z * L + t) * d + c] = cvt<T>(row[i] + colp[i]);
  }
  if (lane == 0) {
    dsrc[(long)z * L + t] = cvt<T>(gs_row[(long)z * Lp + t] / (2.0f * (float)src[(long)z * L + t]));
    ddest[(long)z * L + t] = cvt<T>(gs_col[(long)z * Lp + t] / (2.0f * (float)dest[(long)z * L + t]));
  }
}

}  // namespace ua
