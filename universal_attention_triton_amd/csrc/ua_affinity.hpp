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

// The pipeline macros of ua_fused.hpp are private to that header; these kernels use a two-stage loop of their own,
// unrolled by two over two distinct LDS objects, and take one key group per workgroup or two of complementary length.
// grid (Lp/128 or half of it, Z), 8 waves; wave w owns keys 16*(8*bx+w)..+15 and sweeps the 32-query blocks from its own on.
// The (32 queries, 128 keys) block of a step goes through LDS so that it leaves as whole rows of 256 (bf16) or 512
// bytes, 16 bytes per lane (vec: rows of aff start 16-byte aligned); the block of step s is written out during step
// s + 1.  The rows above the workgroup's first block (queries before all of its keys) are filled the same way.
template <class T, int D>
__global__ void __launch_bounds__(512) k_aff_fwd(const T* __restrict__ Kp, const float* __restrict__ lsrc,
                                                 const float* __restrict__ ldest, T* __restrict__ aff, int L, int Lp, int vec) {
  using TN = Tile<T, 32, D>;
  constexpr int NK = D / 32, SB = TN::BYTES + 1024;
  constexpr int EPV = 16 / (int)sizeof(T);            // elements per 16-byte vector
  constexpr int ROWB = 128 * (int)sizeof(T) + 16;     // bytes per row of the block in LDS (padded: no bank conflicts)
  constexpr int TPR = 128 / EPV, RPP = 512 / TPR;     // threads per row, rows per pass of the workgroup
  // distinct objects per stage: the compiler then knows that the asynchronous loads filling one stage do not alias
  // the reads of the other and does not wait for them
  __shared__ __attribute__((aligned(1024))) char stage0[SB];
  __shared__ __attribute__((aligned(1024))) char stage1[SB];
  __shared__ __attribute__((aligned(16))) char oblk0[32 * ROWB];
  __shared__ __attribute__((aligned(16))) char oblk1[32 * ROWB];
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, col = lane & 15, g = lane >> 4;
  const int bx0 = blockIdx.x, z = blockIdx.y, n_kg = Lp / 128;
  const GroupMasks gm = group_masks(lane);
  auto sweep = [&](const int bx) __attribute__((always_inline)) {
  const int nT = Lp / 32, sb16 = 8 * bx + w, first = 4 * bx, own = sb16 >> 1;
  const int spos = 16 * sb16 + col;
  Stager<TN, 8> st;
  st.init(w, lane, D * (long)sizeof(T), 32);
  Frag<T> ks[NK];
#pragma unroll
  for (int q = 0; q < NK; ++q) ks[q] = ld8(Kp + nat_off<D>(z, Lp, spos, 32 * q + 8 * g));
  const float la = lsrc[(long)z * Lp + spos];
  const T* Kz = Kp + (long)z * Lp * D;
  T* az = aff + (long)z * L * L;
  const T fill = cvt<T>(kNegFill);
  // this thread's piece of a row of the workgroup's 128 columns
  const int prow = tid / TPR, s0 = 128 * bx + EPV * (tid % TPR);
  // stores this thread's 16 bytes of row t (handed over in registers: a pointer to them would send them through scratch
  // memory, and every store would wait for the one before it)
  auto put_piece = [&] __device__ (int t, const uint4 val) __attribute__((always_inline)) {
    if (t < L && s0 < L) {
      T* dst = az + (long)t * L + s0;
      if (vec) {       // L is a multiple of EPV, so the piece lies inside the row
        *reinterpret_cast<uint4*>(dst) = val;
      } else {
        const unsigned wd[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
          T x;
          if constexpr (sizeof(T) == 2) {
            const unsigned short h = (unsigned short)(wd[e / 2] >> (16 * (e % 2)));
            __builtin_memcpy(&x, &h, 2);
          } else {
            __builtin_memcpy(&x, &wd[e], 4);
          }
          if (s0 + e < L) dst[e] = x;
        }
      }
    }
  };
  // queries before the workgroup's first block see none of its keys
  {
    uint4 fills;
#pragma unroll
    for (int e = 0; e < EPV; ++e) reinterpret_cast<T*>(&fills)[e] = fill;
    for (int t = prow; t < min(32 * first, L); t += RPP) put_piece(t, fills);
  }
  auto flush = [&] __device__ (int tb, const char* blk) __attribute__((always_inline)) {
#pragma unroll
    for (int r0 = 0; r0 < 32; r0 += RPP)
      put_piece(32 * tb + r0 + prow, *reinterpret_cast<const uint4*>(blk + (r0 + prow) * ROWB + 16 * (tid % TPR)));
  };
  float carry = 0.f;
  const int total = nT - first;
  auto issue = [&] __device__ (int s, char* base) __attribute__((always_inline)) {
    st.issue(base, Kz + (long)32 * (first + s) * D, w);
    if (w == 0) issue_row(base + TN::BYTES, ldest + (long)z * Lp + 32 * (first + s) + 4 * (lane & 7));
  };
  issue(0, stage0);
  auto step = [&] __device__ (const int s, char* cur, char* nxt, char* ob_cur, char* ob_prev) __attribute__((always_inline)) {
    wait_async_loads();
    __syncthreads();
    if (s > 0) flush(first + s - 1, ob_prev);
    if (s + 1 < total) issue(s + 1, nxt);
    const int tb = first + s;
    if (32 * tb >= L) return;                        // padding rows only: nothing to write
    char* mine = ob_cur + (16 * w + col) * (int)sizeof(T);
    if (tb < own) {                  // the wave's keys come after every query of the block
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v) *reinterpret_cast<T*>(mine + (16 * i + 4 * g + v) * ROWB) = fill;
      return;
    }
    const T* sK = reinterpret_cast<const T*>(cur);
    const float* stats = reinterpret_cast<const float*>(cur + TN::BYTES);
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
        *reinterpret_cast<T*>(mine + (16 * i + 4 * g + v) * ROWB) = (t < spos) ? fill : cvt<T>((x[i][v] + carry) * kLn2);
      }
    carry += tot;
  };
  int s = 0;
  for (; s + 1 < total; s += 2) {
    step(s, stage0, stage1, oblk0, oblk1);
    step(s + 1, stage1, stage0, oblk1, oblk0);
  }
  if (s < total) step(s, stage0, stage1, oblk0, oblk1);
  __syncthreads();
  if (32 * (first + total - 1) < L) flush(first + total - 1, ((total - 1) & 1) ? oblk1 : oblk0);
  };
  // a launch of half as many workgroups as key groups: each takes two of complementary length (every workgroup then
  // computes the same number of blocks and writes the same number of bytes)
  sweep(bx0);
  if ((int)gridDim.x != n_kg && n_kg - 1 - bx0 != bx0) {
    __syncthreads();
    sweep(n_kg - 1 - bx0);
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

// ---------------------------------------------------------------------------------------------
// 16-bit dtypes, rows of daff 16-byte aligned: the backward without the L x L float32 tensor DL.
// k_aff_bwd_keys is key-stationary like k_aff_bwd_side<false> but sweeps the query blocks from the last one down to
// its own, carrying the reverse running sum per key (dcar), and reads the (32 queries, 128 keys) block of daff of a step
// through LDS (rows of 256 bytes, 16 bytes per lane).  It leaves W = dl F as bf16 tiles of 1 KB — (32 keys, 16
// queries) in the LDS image of StageT, row after row of the causal triangle (tri_grad_row) — and k_aff_bwd_cols, one
// wave per 16 positions u, turns its row of tiles into the column side sum_s W[s,u] k_s with nothing but matrix products.
//   grid (Lp/128, Z), 8 waves each.
// ---------------------------------------------------------------------------------------------
template <class T, int D>
__global__ void __launch_bounds__(512) k_aff_bwd_keys(const T* __restrict__ Kp, const T* __restrict__ KT,
                                                      const float* __restrict__ lsrc, const float* __restrict__ ldest,
                                                      const T* __restrict__ daff, T* __restrict__ Wst, float* __restrict__ row,
                                                      float* __restrict__ gsum, int L, int Lp) {
  static_assert(sizeof(T) == 2, "tiles are exchanged in 16-bit operand precision");
  using TN = Tile<T, 32, D>;
  using TT = Tile<T, D, 32>;
  constexpr int NK = D / 32, ND = D / 16, DB = 32 * 128 * (int)sizeof(T), SB = TN::BYTES + TT::BYTES + DB + 1024;
  // distinct objects per stage (see k_aff_fwd)
  __shared__ __attribute__((aligned(1024))) char stage0[SB];
  __shared__ __attribute__((aligned(1024))) char stage1[SB];
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, col = lane & 15, g = lane >> 4;
  const int bx0 = blockIdx.x, z = blockIdx.y, n_kg = Lp / 128;
  const int nTr = (L + 31) / 32;
  const GroupMasks gm = group_masks(lane);
  auto sweep = [&](const int bx) __attribute__((always_inline)) {
    const int first = 4 * bx;
    if (first >= nTr) return;                      // every key of this group is padding
    const int sb16 = 8 * bx + w, own = sb16 >> 1, spos = 16 * sb16 + col;
    Stager<TN, 8> stN;
    Stager<TT, 8> stT;
    stN.init(w, lane, D * (long)sizeof(T), 32);
    stT.init(w, lane, Lp * (long)sizeof(T), D);
    Frag<T> ki[NK];
#pragma unroll
    for (int q = 0; q < NK; ++q) ki[q] = ld8(Kp + nat_off<D>(z, Lp, spos, 32 * q + 8 * g));
    const float li = lsrc[(long)z * Lp + spos];
    const T* Kz = Kp + (long)z * Lp * D;
    const T* KTz = KT + (long)z * D * Lp;
    const T* dz = daff + (long)z * L * L;
    f32x4 acc_o[ND];
#pragma unroll
    for (int n = 0; n < ND; ++n) acc_o[n] = (f32x4){0, 0, 0, 0};
    float gs = 0.f, dcar = 0.f;
    // where this lane's four values of a (16 keys, 16 queries) tile go inside the 1 KB tile of its 32-key half
    char* wz = reinterpret_cast<char*>(Wst) + (long)z * (tri_tiles(Lp >> 5) << 10) + ((long)(sb16 >> 1) << 10) +
               StageT<bf16>::addr(perm32(16 * (sb16 & 1) + col), 8 * g);
    // this lane's 16 bytes of the daff block of a step: row 4 w + g, keys 128 bx + 8 col ..
    const int drow = 4 * w + g, dcol = 128 * bx + 8 * col;
    const int total = nTr - first;
    auto issue = [&] __device__ (int s, char* base) __attribute__((always_inline)) {
      const int tb = nTr - 1 - s;
      stN.issue(base, Kz + (long)(32 * tb) * D, w);
      stT.issue(base + TN::BYTES, KTz + (long)(32 * tb) * D, w);
      if (32 * tb + drow < L && dcol < L)          // L is a multiple of 8: the piece lies inside the row
        issue_row_nt(base + TN::BYTES + TT::BYTES + w * 1024, dz + (long)(32 * tb + drow) * L + dcol);
      if (w == 0) issue_row(base + TN::BYTES + TT::BYTES + DB, ldest + (long)z * Lp + 32 * tb + 4 * (lane & 7));
    };
    issue(0, stage0);
    auto step = [&] __device__ (const int s, const char* base, char* nxt) __attribute__((always_inline)) {
      wait_async_loads();
      __syncthreads();
      if (s + 1 < total) issue(s + 1, nxt);
      const int tb = nTr - 1 - s;
      if (tb < own) return;                        // the block's queries all precede this wave's keys
      const T* sK = reinterpret_cast<const T*>(base);
      const T* sKT = reinterpret_cast<const T*>(base + TN::BYTES);
      const unsigned short* sD = reinterpret_cast<const unsigned short*>(base + TN::BYTES + TT::BYTES) + 16 * w + col;
      const float* stats = reinterpret_cast<const float*>(base + TN::BYTES + TT::BYTES + DB);
      f32x4 aff[2], gk[2], W[2];
#pragma unroll
      for (int i2 = 0; i2 < 2; ++i2) {
        f32x4 acc = {0, 0, 0, 0};
#pragma unroll
        for (int q = 0; q < NK; ++q) mma16(acc, ld8(sK + TN::at(i2, col, q, g)), ki[q]);
        const f32x4 lj = load_t4(stats + 16 * i2, g);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int r = 16 * i2 + 4 * g + v, t = 32 * tb + r;
          gk[i2][v] = fmaxf(acc[v], 0.f);
          aff[i2][v] = affinity(__builtin_amdgcn_logf(gk[i2][v]), li + lj[v]);
          // aff[t][s] depends on the inputs only for t > s (it is a constant elsewhere)
          const bool valid = t > spos && t < L && spos < L;
          W[i2][v] = valid ? __uint_as_float((unsigned)sD[r * 128] << 16) : 0.f;
        }
      }
      float t1;
      const float tot = suffix32(W[0], W[1], gm, t1);
#pragma unroll
      for (int i2 = 0; i2 < 2; ++i2)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int t = 32 * tb + 16 * i2 + 4 * g + v;
          const float wv = (t > spos && t < L && spos < L) ? decay_grad(W[i2][v] + dcar, aff[i2][v], gk[i2][v]) : 0.f;
          W[i2][v] = wv;
          gs = __builtin_fmaf(wv, gk[i2][v], gs);
        }
      dcar += tot;
      const Frag<T> b = as_operand16<T>(W[0], W[1]);
      {   // query tiles 2 tb and 2 tb + 1: their rows of tiles start tb + 1 tiles apart
        char* p = wz + (tri_grad_row(2 * tb) << 10);
        __builtin_nontemporal_store(reinterpret_cast<const u32x2*>(&b)[0], reinterpret_cast<u32x2*>(p));
        __builtin_nontemporal_store(reinterpret_cast<const u32x2*>(&b)[1], reinterpret_cast<u32x2*>(p + ((long)(tb + 1) << 10)));
      }
#pragma unroll
      for (int n = 0; n < ND; ++n) mma16(acc_o[n], ld8(sKT + TT::at(n, col, 0, g)), b);
    };
    int s = 0;
    for (; s + 1 < total; s += 2) {
      step(s, stage0, stage1);
      step(s + 1, stage1, stage0);
    }
    if (s < total) step(s, stage0, stage1);
    {
      float b, af, tot;
      group_scan(gs, gm, b, af, tot);
      if (g == 0) gsum[(long)z * Lp + spos] = tot;
    }
#pragma unroll
    for (int n = 0; n < ND; ++n) {
      const long o = ((long)z * Lp + spos) * D + 16 * n + 4 * g;
      *reinterpret_cast<float4*>(row + o) = make_float4(acc_o[n][0], acc_o[n][1], acc_o[n][2], acc_o[n][3]);
    }
  };
  // a launch of half as many workgroups as key groups: each sweeps two of complementary length
  sweep(bx0);
  if ((int)gridDim.x != n_kg && n_kg - 1 - bx0 != bx0) {
    __syncthreads();
    sweep(n_kg - 1 - bx0);
  }
}

// colp[z][u][:] = sum_{s<u} W[s,u] k_s from the tiles of k_aff_bwd_keys; wave w owns positions 16*(8*jt+w)..+15 and
// streams its own row of tiles (two 32-key halves per step of 64 keys) straight into LDS.
template <class T, int D>
__global__ void __launch_bounds__(512) k_aff_bwd_cols(const T* __restrict__ KT, const T* __restrict__ Wst, float* __restrict__ colp,
                                                      int L, int Lp) {
  static_assert(sizeof(T) == 2, "tiles are exchanged in 16-bit operand precision");
  using TT = Tile<T, D, 32>;
  using ST = StageT<T>;
  constexpr int ND = D / 16, TILES = 2 * TT::BYTES, WAVE = 2 * ST::BYTES, SB = TILES + 8 * WAVE;
  // distinct objects per stage (see k_aff_fwd)
  __shared__ __attribute__((aligned(1024))) char stage0[SB];
  __shared__ __attribute__((aligned(1024))) char stage1[SB];
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, col = lane & 15, g = lane >> 4;
  const int z = blockIdx.y, n_blk = Lp / 128, bx0 = blockIdx.x;
  auto sweep = [&](const int jt) __attribute__((always_inline)) {
    const int tq = 8 * jt + w;
    if (128 * jt >= L) return;                     // padding positions only
    Stager<TT, 8> stT;
    stT.init(w, lane, Lp * (long)sizeof(T), D);
    f32x4 dKc[ND];
#pragma unroll
    for (int n = 0; n < ND; ++n) dKc[n] = (f32x4){0, 0, 0, 0};
    const T* KTz = KT + (long)z * D * Lp;
    const char* pW = reinterpret_cast<const char*>(Wst) + (long)z * (tri_tiles(Lp >> 5) << 10) + (tri_grad_row(tq) << 10) + 16 * lane;
    const int n_kt = 2 * jt + 2;
    auto issue = [&] __device__ (int s, char* base) __attribute__((always_inline)) {
      stT.issue(base, KTz + (long)(64 * s) * D, w);
      stT.issue(base + TT::BYTES, KTz + (long)(64 * s + 32) * D, w);
      char* mine = base + TILES + w * WAVE;
      // halves 2 s and 2 s + 1 of this wave's row; a row has (tq >> 1) + 1 of them
      if (2 * s <= (tq >> 1)) issue_row_nt(mine, pW + ((long)(2 * s) << 10));
      if (2 * s + 1 <= (tq >> 1)) issue_row_nt(mine + ST::BYTES, pW + ((long)(2 * s + 1) << 10));
    };
    issue(0, stage0);
    auto step = [&] __device__ (const int s, char* base, char* nxt) __attribute__((always_inline)) {
      wait_async_loads();
      __syncthreads();
      if (s + 1 < n_kt) issue(s + 1, nxt);
      char* mine = base + TILES + w * WAVE;
#pragma unroll
      for (int kq = 0; kq < 2; ++kq) {
        // the half's two 16-key tiles were written iff their keys do not come after this wave's positions
        const int sbk = 4 * s + 2 * kq;
        const bool live0 = sbk <= tq && 16 * tq < L, live1 = sbk + 1 <= tq;      // (a wave of padding positions has no tiles)
        if (!live0) continue;
        Frag<T> ag = ST::get(mine + kq * ST::BYTES, lane);
        // elements 0-3 of an operand are keys of the first tile, 4-7 of the second (perm32)
        if (!live1) reinterpret_cast<uint2*>(&ag)[1] = make_uint2(0, 0);
        const T* sKT = reinterpret_cast<const T*>(base + kq * TT::BYTES);
#pragma unroll
        for (int n = 0; n < ND; ++n) mma16(dKc[n], ag, ld8(sKT + TT::at(n, col, 0, g)));
      }
    };
    int s = 0;
    for (; s + 1 < n_kt; s += 2) {
      step(s, stage0, stage1);
      step(s + 1, stage1, stage0);
    }
    if (s < n_kt) step(s, stage0, stage1);
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int t = 16 * tq + 4 * g + v;
#pragma unroll
      for (int n = 0; n < ND; ++n) colp[((long)z * Lp + t) * D + 16 * n + col] = dKc[n][v];
    }
  };
  // the longest rows first; a launch of half as many workgroups as blocks: each takes two of complementary length
  sweep(n_blk - 1 - bx0);
  if ((int)gridDim.x != n_blk && n_blk - 1 - bx0 != bx0) {
    __syncthreads();
    sweep(bx0);
  }
}

// dk = row side + column side; dsrc = gsum_row / (2 src); ddest = gsum_col / (2 dest)   (sum W G = 3/2 sum dA A)
template <class T>
__global__ void __launch_bounds__(256) k_aff_finish(const float* __restrict__ row, const float* __restrict__ colp,
                                                    const float* __restrict__ gs_row, const float* __restrict__ gs_col,
                                                    const T* __restrict__ src, const T* __restrict__ dest, T* __restrict__ dk,
                                                    T* __restrict__ dsrc, T* __restrict__ ddest, int L, int Lp, int D, int d,
                                                    const T* __restrict__ Kp) {
  const int z = blockIdx.y, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + wave;
  if (t >= L) return;
  // without gs_col: sum_s W[s,u] G[s,u] = k_u . colp_u (W vanishes where the key-key product is not positive)
  float dot = 0.f;
  for (int c = lane; c < d; c += 64) {
    const long i = ((long)z * Lp + t) * D + c;
    dk[((long)z * L + t) * d + c] = cvt<T>(row[i] + colp[i]);
    if (!gs_col) dot += colp[i] * (float)Kp[D == 64 ? nat_off<64>(z, Lp, t, c) : nat_off<128>(z, Lp, t, c)];
  }
  if (!gs_col) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) dot += __shfl_xor(dot, m, 64);
  }
  if (lane == 0) {
    dsrc[(long)z * L + t] = cvt<T>(gs_row[(long)z * Lp + t] / (2.0f * (float)src[(long)z * L + t]));
    ddest[(long)z * L + t] = cvt<T>((gs_col ? gs_col[(long)z * Lp + t] : dot) / (2.0f * (float)dest[(long)z * L + t]));
  }
}

}  // namespace ua
