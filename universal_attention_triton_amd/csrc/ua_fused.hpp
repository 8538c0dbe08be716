// Kernels of the fused path (ua_fused_fwd / ua_fused_bwd), software pipelined: the tiles of step k+1
// are fetched global -> LDS by asynchronous 16-byte loads while step k computes; one workgroup
// barrier per step.  NST = number of LDS stages (2: overlap; 1: no overlap, for the fp32 footprint).
//
//   k_carry2        key-stationary pre-pass: decay bias accumulated before each 32-query block
//   k_fwd_fused2    query-stationary forward with online softmax (key tiles visited from the
//                   diagonal backwards, so the running maximum settles in the first tile)
//   k_bwd_keys2     key-stationary reverse sweep: dV, dK (score + row side of the decay), dsrc,
//                   and the suffix carries of dBias for k_bwd_queries2
//   k_bwd_queries2  query-stationary: dQ and the column side of dK
// Tile math and conventions: see ua_common.hpp (orientation) and ua_bwd.hpp (formulas).
#pragma once
#include "ua_bwd.hpp"
#include "ua_common.hpp"

namespace ua {

// One asynchronous instruction (1 KB, issued by one wave): lane l copies 16 bytes from src to base + 16*l.
__device__ __forceinline__ void issue_row(void* lds_base, const void* src_lane) {
  __builtin_amdgcn_global_load_lds(src_lane, (lds_ptr_t)lds_base, 16, 0, 0);
}

// Pipeline skeleton.  Every kernel declares two STATIC LDS arrays stage0 / stage1 (distinct objects, so the
// compiler can prove that the asynchronous loads filling one stage do not alias the reads of the other and
// does not wait for them) and provides ISSUE(step, stage) and COMPUTE(step, stage).
// UA_PIPE_RANGE runs steps [S0, S1) of a pipeline of NSTEPS steps whose step S0 has already been issued
// (by UA_PIPE_START or by the previous range), so that consecutive ranges may use different COMPUTE bodies.
#define UA_PIPE_START(NSTEPS, ISSUE)                                                       \
  do {                                                                                     \
    if ((NSTEPS) > 0) ISSUE(0, stage0);                                                    \
  } while (0)
#define UA_STEP2_(STEP, NSTEPS, CUR, NXT, ISSUE, COMPUTE)                                  \
  {                                                                                        \
    wait_async_loads();                                                                    \
    __syncthreads();                                                                       \
    if ((STEP) + 1 < (NSTEPS)) ISSUE((STEP) + 1, NXT);                                     \
    COMPUTE((STEP), CUR);                                                                  \
  }
// With two stages S0 must be even (even steps live in stage0); the loop is unrolled by two so that both
// stage roles are compile-time constants on a straight-line path.
#define UA_PIPE_RANGE(S0, S1, NSTEPS, ISSUE, COMPUTE)                                      \
  do {                                                                                     \
    const int nsteps_ = (NSTEPS), s1_ = (S1);                                              \
    int step_ = (S0);                                                                      \
    if constexpr (NST == 2) {                                                              \
      for (; step_ + 1 < s1_; step_ += 2) {                                                \
        UA_STEP2_(step_, nsteps_, stage0, stage1, ISSUE, COMPUTE)                          \
        UA_STEP2_(step_ + 1, nsteps_, stage1, stage0, ISSUE, COMPUTE)                      \
      }                                                                                    \
      if (step_ < s1_) UA_STEP2_(step_, nsteps_, stage0, stage1, ISSUE, COMPUTE)           \
    } else {                                                                               \
      for (; step_ < s1_; ++step_) {                                                       \
        wait_async_loads();                                                                \
        __syncthreads();                                                                   \
        COMPUTE(step_, stage0);                                                            \
        __syncthreads();                                                                   \
        if (step_ + 1 < nsteps_) ISSUE(step_ + 1, stage0);                                 \
      }                                                                                    \
    }                                                                                      \
  } while (0)
#define UA_PIPELINE(NSTEPS, ISSUE, COMPUTE)                                                \
  do {                                                                                     \
    UA_PIPE_START(NSTEPS, ISSUE);                                                          \
    UA_PIPE_RANGE(0, NSTEPS, NSTEPS, ISSUE, COMPUTE);                                      \
  } while (0)
#define UA_STAGES(BYTES)                                                                   \
  __shared__ __attribute__((aligned(1024))) char stage0[BYTES];                            \
  __shared__ __attribute__((aligned(1024))) char stage1[NST == 2 ? (BYTES) : 1024]

// ---------------------------------------------------------------------------------------------
// C[z][tb][s] = sum_{u < 32*tb, u > s} log2(1 - A[s,u])   (tb >= s/32).  grid (Lp/128, Zk), 4 waves.
// ---------------------------------------------------------------------------------------------
template <class T, int D, int NST>
__global__ void __launch_bounds__(256) k_carry2(const T* __restrict__ Kp, const float* __restrict__ lsrc,
                                                const float* __restrict__ ldest, float* __restrict__ C, int Lp) {
  using TN = Tile<T, 32, D>;
  constexpr int NQ = D / 16, LS = TN::STRIDE, SB = TN::BYTES + 1024;   // tile + [ldest of the block: 32 floats]
  UA_STAGES(SB);
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, col = lane & 31, hi = lane >> 5;
  const int z = blockIdx.y, nT = Lp / 32, sb = 4 * blockIdx.x + w, first = 4 * blockIdx.x;
  Stager<TN, 4> st;
  st.init(w, lane, D * (long)sizeof(T), 32);
  Frag<T> ks[NQ];
  {
    const T* krow = Kp + ((long)z * Lp + 32 * sb + col) * D + 8 * hi;
#pragma unroll
    for (int q = 0; q < NQ; ++q) ks[q] = ld8(krow + 16 * q);
  }
  const float la = lsrc[(long)z * Lp + 32 * sb + col];
  float carry = 0.f;
  float* Cz = C + (long)z * nT * Lp;
  const T* Kz = Kp + (long)z * Lp * D;
#define UA_ISSUE(s, base)                                                                   \
  {                                                                                         \
    st.issue((base), Kz + (long)32 * (first + (s)) * D, w);                                 \
    if (w == 0) issue_row((base) + TN::BYTES, ldest + (long)z * Lp + 32 * (first + (s)) + 4 * (lane & 7)); \
  }
#define UA_COMPUTE(s, base)                                                                 \
  {                                                                                         \
    const int tb = first + (s);                                                             \
    const T* sK = reinterpret_cast<const T*>(base);                                         \
    if (tb >= sb) {                                                                         \
      float lb[16];                                                                         \
      load_t16(reinterpret_cast<const float*>((base) + TN::BYTES), hi, lb);                 \
      f32x16 g = {0};                                                                       \
      _Pragma("unroll") for (int q = 0; q < NQ; ++q) mma(g, ld8(sK + col * LS + 16 * q + 8 * hi), ks[q]); \
      float tot = 0.f;                                                                      \
      _Pragma("unroll") for (int v = 0; v < 16; ++v) {                                      \
        float l2 = log2_one_minus(affinity(log2_relu(g[v]), la + lb[v]));                   \
        if (tb == sb && t_of(v, hi) <= col) l2 = 0.f;                                       \
        tot += l2;                                                                          \
      }                                                                                     \
      float lo, up;                                                                         \
      swap32(tot, lo, up);                                                                  \
      if (hi == 0) Cz[(long)tb * Lp + 32 * sb + col] = carry;                               \
      carry += lo + up;                                                                     \
    }                                                                                       \
  }
  UA_PIPELINE(nT - first, UA_ISSUE, UA_COMPUTE);
#undef UA_ISSUE
#undef UA_COMPUTE
}

// ---------------------------------------------------------------------------------------------
// Fused forward.  grid (Lp/128, Zq); 4 waves; wave w owns queries 32*(4*jt+w)..+31; 64 keys per step.
// ---------------------------------------------------------------------------------------------
template <class T, int D, int NST>
__global__ void __launch_bounds__(256) k_fwd_fused2(const T* __restrict__ Qp, const T* __restrict__ Kp,
                                                    const T* __restrict__ VT, const float* __restrict__ lsrc,
                                                    const float* __restrict__ ldest, const float* __restrict__ C,
                                                    T* __restrict__ O, float* __restrict__ lse, float* __restrict__ lse2,
                                                    int R, int L, int Lp, int d) {
  using TN = Tile<T, 32, D>;
  using TT = Tile<T, D, 32>;
  constexpr int NQ = D / 16, NB = D / 32, LS = TN::STRIDE, TS = TT::STRIDE, PS = lds_stride<T>(64);
  constexpr int TILES = 2 * TN::BYTES + 2 * TT::BYTES, SB = TILES + 4 * 1024;   // + per wave [C row: 64f][lsrc: 64f]
  UA_STAGES(SB);
  __shared__ __attribute__((aligned(16))) T sPbuf[4 * 32 * PS];
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, col = lane & 31, hi = lane >> 5;
  const int zq = blockIdx.y, zk = zq / R, nT = Lp / 32;
  const int jt = gridDim.x - 1 - blockIdx.x, tb = 4 * jt + w;
  T* sPw = sPbuf + w * 32 * PS;
  const int pcol = perm16(col);
  Stager<TN, 4> stN;
  Stager<TT, 4> stT;
  stN.init(w, lane, D * (long)sizeof(T), 32);
  stT.init(w, lane, Lp * (long)sizeof(T), D);

  Frag<T> qf[NQ], kf[NQ];
  {
    const T* qrow = Qp + ((long)zq * Lp + 32 * tb + col) * D + 8 * hi;
    const T* krow = Kp + ((long)zk * Lp + 32 * tb + col) * D + 8 * hi;
#pragma unroll
    for (int q = 0; q < NQ; ++q) { qf[q] = ld8(qrow + 16 * q); kf[q] = ld8(krow + 16 * q); }
  }
  float lb[16];
  load_t16(ldest + (long)zk * Lp + 32 * tb, hi, lb);
  f32x16 o[NB];
#pragma unroll
  for (int n = 0; n < NB; ++n) o[n] = (f32x16){0};
  float m[16], ls[16];
#pragma unroll
  for (int v = 0; v < 16; ++v) { m[v] = -1.0e30f; ls[v] = 0.f; }
  const float* Crow = C + ((long)zk * nT + tb) * Lp;
  const float* lsz = lsrc + (long)zk * Lp;
  const T* Kz = Kp + (long)zk * Lp * D;
  const T* Vz = VT + (long)zk * D * Lp;
  const int n_kt = 2 * jt + 2;   // key tiles of 64 covering s <= last query of the workgroup

#define UA_ISSUE(s, base)                                                                   \
  {                                                                                         \
    const int kt_ = n_kt - 1 - (s);                                                         \
    stN.issue((base), Kz + (long)(64 * kt_) * D, w);                                        \
    stN.issue((base) + TN::BYTES, Kz + (long)(64 * kt_ + 32) * D, w);                       \
    stT.issue((base) + 2 * TN::BYTES, Vz + 64 * kt_, w);                                    \
    stT.issue((base) + 2 * TN::BYTES + TT::BYTES, Vz + 64 * kt_ + 32, w);                   \
    issue_row((base) + TILES + w * 1024, ((lane & 16) ? lsz : Crow) + 64 * kt_ + 4 * (lane & 15)); \
  }
#define UA_COMPUTE(s, base)                                                                 \
  {                                                                                         \
    const int kt_ = n_kt - 1 - (s);                                                         \
    fwd_tile(kt_, base);                                                                    \
  }
  auto fwd_tile = [&] __device__ (int kt, const char* base) {
    f32x16 s2[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int sbk = 2 * kt + j;
      const T* sK = reinterpret_cast<const T*>(base + j * TN::BYTES);
      if (sbk <= tb) {
        const float* stats = reinterpret_cast<const float*>(base + TILES + w * 1024);
        const float c = stats[32 * j + col];
        const float la = stats[64 + 32 * j + col];
        f32x16 g = {0}, sc = {0};
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
          const Frag<T> kb = ld8(sK + col * LS + 16 * q + 8 * hi);
          mma(g, kf[q], kb);
          mma(sc, qf[q], kb);
        }
        const bool diag = (sbk == tb);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float l2 = log2_one_minus(affinity(log2_relu(g[v]), la + lb[v]));
          g[v] = (diag && t_of(v, hi) <= col) ? 0.f : l2;
        }
        block_prefix(g, hi);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float x = __builtin_fmaf(sc[v], kLog2e, g[v] + c);
          s2[j][v] = (diag && t_of(v, hi) < col) ? -1.0e30f : x;
        }
      } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) s2[j][v] = -1.0e30f;
      }
    }
    // online softmax: rescale only when some query of this wave raises its maximum
    float mx[16];
    bool grow = false;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      mx[v] = allmax32(fmaxf(s2[0][v], s2[1][v]));
      grow |= (mx[v] > m[v]);
    }
    if (__builtin_amdgcn_ballot_w64(grow) != 0) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float mn = fmaxf(m[v], mx[v]);
        const float alpha = __builtin_amdgcn_exp2f(m[v] - mn);
        m[v] = mn;
        ls[v] *= alpha;
#pragma unroll
        for (int n = 0; n < NB; ++n) o[n][v] *= alpha;
      }
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const float p = __builtin_amdgcn_exp2f(s2[j][v] - m[v]);
        ls[v] += p;
        sPw[t_of(v, hi) * PS + 32 * j + pcol] = cvt<T>(p);
      }
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      if (2 * kt + j <= tb) {
        const T* sV = reinterpret_cast<const T*>(base + 2 * TN::BYTES + j * TT::BYTES);
#pragma unroll
        for (int kq = 0; kq < 2; ++kq) {
          const Frag<T> pa = ld8(sPw + col * PS + 32 * j + 16 * kq + 8 * hi);
#pragma unroll
          for (int n = 0; n < NB; ++n) mma(o[n], pa, ld8(sV + (32 * n + col) * TS + 16 * kq + 8 * hi));
        }
      }
    }
  };
  UA_PIPELINE(n_kt, UA_ISSUE, UA_COMPUTE);
#undef UA_ISSUE
#undef UA_COMPUTE
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
// Key-stationary backward (fused mode).  grid (Lp/128, Zk); 4 waves; wave w owns keys 128g+32w..+31,
// sweeps query blocks from the last one down to its own; one (query block, query group) per step.
// MR = more than one query group per kv head (the decay state of a query block then lives across steps).
// ---------------------------------------------------------------------------------------------
struct TrueC { static constexpr bool value = true; };
struct FalseC { static constexpr bool value = false; };

template <class T, int D, int NST, bool MR>
__global__ void __launch_bounds__(256) k_bwd_keys2(BwdArgs<T> a) {
  using TN = Tile<T, 32, D>;
  using TT = Tile<T, D, 32>;
  constexpr int NQ = D / 16, NB = D / 32, LS = TN::STRIDE, TS = TT::STRIDE;
  constexpr int TILES = 3 * TN::BYTES + 3 * TT::BYTES, SB = TILES + 1024;
  UA_STAGES(SB);
  // stats row of a stage: [lse2: 32f][delta: 32f][ldest: 32f][unused: 32f][forward carries of the 128 keys: 128f]
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, col = lane & 31, hi = lane >> 5;
  const int zk = blockIdx.y, Lp = a.Lp, L = a.L, nT = Lp / 32, R = MR ? a.R : 1;
  const int g = gridDim.x - 1 - blockIdx.x, sb = 4 * g + w, spos = 32 * sb + col;
  const int nTr = (L + 31) / 32, first = 4 * g;
  if (first >= nTr) return;                      // every key of this workgroup is padding
  Stager<TN, 4> stN;
  Stager<TT, 4> stT;
  stN.init(w, lane, D * (long)sizeof(T), 32);
  stT.init(w, lane, Lp * (long)sizeof(T), D);

  Frag<T> kp[NQ], vf[NQ];
  {
    const long ro = ((long)zk * Lp + spos) * D + 8 * hi;
#pragma unroll
    for (int q = 0; q < NQ; ++q) { kp[q] = ld8(a.Kp + ro + 16 * q); vf[q] = ld8(a.Vp + ro + 16 * q); }
  }
  const float la = a.lsrc[(long)zk * Lp + spos];
  f32x16 dVt[NB], dKt[NB];
#pragma unroll
  for (int n = 0; n < NB; ++n) { dVt[n] = (f32x16){0}; dKt[n] = (f32x16){0}; }
  float dsrc_acc = 0.f, dcar = 0.f;
  f32x16 aff_s, bias_s, gk_s, dB_s;              // state of the current query block (used when MR)
  float lab_s[16];
  const T* Kz = a.Kp + (long)zk * Lp * D;
  const T* KTz = a.KT + (long)zk * D * Lp;
  const float* ldz = a.ldest + (long)zk * Lp;
  const float* Cz = a.C + (long)zk * nT * Lp + 128 * g;
  float* Dz = a.Dsuf + (long)zk * nT * Lp + spos;

#define UA_ISSUE(s, base)                                                                   \
  {                                                                                         \
    const int tb_ = nTr - 1 - (s) / R;                                                      \
    const long zq_ = (long)zk * R + (s) % R;                                                \
    const long qo_ = (zq_ * Lp + 32 * tb_) * D, to_ = zq_ * D * Lp + 32 * tb_;              \
    stN.issue((base), Kz + (long)(32 * tb_) * D, w);                                        \
    stN.issue((base) + TN::BYTES, a.Qp + qo_, w);                                           \
    stN.issue((base) + 2 * TN::BYTES, a.dOp + qo_, w);                                      \
    stT.issue((base) + 3 * TN::BYTES, KTz + 32 * tb_, w);                                   \
    stT.issue((base) + 3 * TN::BYTES + TT::BYTES, a.QT + to_, w);                           \
    stT.issue((base) + 3 * TN::BYTES + 2 * TT::BYTES, a.dOT + to_, w);                      \
    if (w == 0) {                                                                           \
      const float* src_;                                                                    \
      if (lane < 8) src_ = a.lse2 + zq_ * Lp + 32 * tb_ + 4 * lane;                         \
      else if (lane < 16) src_ = a.delta + zq_ * Lp + 32 * tb_ + 4 * (lane - 8);            \
      else if (lane < 32) src_ = ldz + 32 * tb_ + 4 * (lane & 7);                           \
      else src_ = Cz + (long)tb_ * Lp + 4 * (lane - 32);                                    \
      issue_row((base) + TILES, src_);                                                      \
    }                                                                                       \
  }
#define UA_COMPUTE_FAST(s, base) bwd_step((s), (base), FalseC(), false)
#define UA_COMPUTE_SLOW(s, base)                                                            \
  {                                                                                         \
    const int tb_ = nTr - 1 - (s) / R;                                                      \
    if (tb_ >= sb) bwd_step((s), (base), TrueC(), tb_ == sb);                               \
  }
  // MASKED: the step may be this wave's diagonal block (run-time flag diag); otherwise every pair is visible
  auto bwd_step = [&] __device__ (int s, const char* base, auto masked_c, const bool diag) {
    constexpr bool DIAG = decltype(masked_c)::value;
    const int tb = nTr - 1 - s / R, r = s % R;
    const T* sKt = reinterpret_cast<const T*>(base);
    const T* sQ = reinterpret_cast<const T*>(base + TN::BYTES);
    const T* sdO = reinterpret_cast<const T*>(base + 2 * TN::BYTES);
    const T* sKT = reinterpret_cast<const T*>(base + 3 * TN::BYTES);
    const T* sQT = reinterpret_cast<const T*>(base + 3 * TN::BYTES + TT::BYTES);
    const T* sdOT = reinterpret_cast<const T*>(base + 3 * TN::BYTES + 2 * TT::BYTES);
    const float* stats = reinterpret_cast<const float*>(base + TILES);
    f32x16 aff_l, bias_l, gk_l, dB_l;
    float lab_l[16];
    f32x16& aff = MR ? aff_s : aff_l;
    f32x16& bias = MR ? bias_s : bias_l;
    f32x16& gk = MR ? gk_s : gk_l;
    f32x16& dB = MR ? dB_s : dB_l;
    float (&lab)[16] = MR ? lab_s : lab_l;
    if (!MR || r == 0) {
      const float cin = stats[128 + 32 * w + col];
      load_t16(stats + 64, hi, lab);
      f32x16 acc = {0};
#pragma unroll
      for (int q = 0; q < NQ; ++q) mma(acc, ld8(sKt + col * LS + 16 * q + 8 * hi), kp[q]);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        lab[v] += la;
        gk[v] = log2_relu(acc[v]);
        aff[v] = affinity(gk[v], lab[v]);
        const float l2 = log2_one_minus(aff[v]);
        bias[v] = (DIAG && diag && t_of(v, hi) <= col) ? 0.f : l2;
      }
      block_prefix(bias, hi);
#pragma unroll
      for (int v = 0; v < 16; ++v) { bias[v] += cin; if (MR) dB[v] = 0.f; }
    }
    {
      f32x16 sc = {0}, dP = {0};
#pragma unroll
      for (int q = 0; q < NQ; ++q) mma(sc, ld8(sQ + col * LS + 16 * q + 8 * hi), kp[q]);
#pragma unroll
      for (int q = 0; q < NQ; ++q) mma(dP, ld8(sdO + col * LS + 16 * q + 8 * hi), vf[q]);
      float l2t[16], dlt[16];
      load_t16(stats, hi, l2t);
      load_t16(stats + 32, hi, dlt);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[v], kLog2e, bias[v]) - l2t[v]);
        if (DIAG) p = (diag && t_of(v, hi) < col) ? 0.f : p;
        sc[v] = p;
        dP[v] = p * (dP[v] - dlt[v]);
      }
#pragma unroll
      for (int q2 = 0; q2 < 2; ++q2) {
        const Frag<T> bp = as_operand<T>(sc, q2);
#pragma unroll
        for (int n = 0; n < NB; ++n) mma(dVt[n], ld8(sdOT + (32 * n + col) * TS + 16 * q2 + 8 * hi), bp);
      }
#pragma unroll
      for (int q2 = 0; q2 < 2; ++q2) {
        const Frag<T> bs = as_operand<T>(dP, q2);
#pragma unroll
        for (int n = 0; n < NB; ++n) mma(dKt[n], ld8(sQT + (32 * n + col) * TS + 16 * q2 + 8 * hi), bs);
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) dB[v] = MR ? dB[v] + dP[v] : dP[v];
    }
    if (!MR || r == R - 1) {
      if (hi == 0) Dz[(long)tb * Lp] = dcar;
      const float tot = block_suffix(dB, hi);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        float dl = dB[v] + dcar;
        if (DIAG) dl = (diag && t_of(v, hi) <= col) ? 0.f : dl;
        const float av = aff[v];
        const float den = __builtin_amdgcn_fmed3f(av, kAMinBwd, kAMax) - 1.0f;
        const float dA = (av <= kAMax) ? dl * __builtin_amdgcn_rcpf(den) : 0.f;
        dsrc_acc = __builtin_fmaf(dA, av, dsrc_acc);
        const float f = (2.0f / 3.0f) * __builtin_amdgcn_exp2f(__builtin_fmaf(gk[v], -1.0f / 3.0f, lab[v]));
        dB[v] = (gk[v] > -1.0e30f) ? dA * f : 0.f;
      }
      dcar += tot;
#pragma unroll
      for (int q2 = 0; q2 < 2; ++q2) {
        const Frag<T> b = as_operand<T>(dB, q2);
#pragma unroll
        for (int n = 0; n < NB; ++n) mma(dKt[n], ld8(sKT + (32 * n + col) * TS + 16 * q2 + 8 * hi), b);
      }
    }
  };
  {
    // the last four query blocks of the sweep hold the diagonal blocks of the four waves
    const int nblk = nTr - first, total = nblk * R, nfast = ((nblk > 4 ? nblk - 4 : 0) * R) & ~1;
    UA_PIPE_START(total, UA_ISSUE);
    UA_PIPE_RANGE(0, nfast, total, UA_ISSUE, UA_COMPUTE_FAST);
    UA_PIPE_RANGE(nfast, total, total, UA_ISSUE, UA_COMPUTE_SLOW);
  }
#undef UA_ISSUE
#undef UA_COMPUTE_FAST
#undef UA_COMPUTE_SLOW
  // epilogue
  float lo, up;
  swap32(dsrc_acc, lo, up);
  if (hi == 0) a.dsrc_raw[(long)zk * Lp + spos] = lo + up;
#pragma unroll
  for (int n = 0; n < NB; ++n) {
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      const long o = ((long)zk * Lp + spos) * D + 32 * n + 8 * gq + 4 * hi;
      *reinterpret_cast<float4*>(a.dVrow + o) = make_float4(dVt[n][4 * gq], dVt[n][4 * gq + 1], dVt[n][4 * gq + 2], dVt[n][4 * gq + 3]);
      *reinterpret_cast<float4*>(a.dKrow + o) = make_float4(dKt[n][4 * gq], dKt[n][4 * gq + 1], dKt[n][4 * gq + 2], dKt[n][4 * gq + 3]);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Query-stationary backward (fused mode): dQ and the column side of dK, no atomics.
// grid (Lp/128, Zk); 4 waves; wave w owns queries 32*(4*jt+w)..+31; 64 keys per step.
// ---------------------------------------------------------------------------------------------
template <class T, int D, int NST>
__global__ void __launch_bounds__(256) k_bwd_queries2(BwdArgs<T> a, T* __restrict__ dq, int d) {
  using TN = Tile<T, 32, D>;
  using TT = Tile<T, D, 32>;
  constexpr int NQ = D / 16, NB = D / 32, LS = TN::STRIDE, TS = TT::STRIDE, SS = lds_stride<T>(32);
  constexpr int TILES = 4 * TN::BYTES + 2 * TT::BYTES, SB = TILES + 4 * 1024;   // + per wave [C: 64f][lsrc: 64f][Dsuf: 64f]
  UA_STAGES(SB);
  __shared__ __attribute__((aligned(16))) T sXbuf[4 * 2 * 32 * SS];
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, col = lane & 31, hi = lane >> 5;
  const int zk = blockIdx.y, Lp = a.Lp, L = a.L, nT = Lp / 32, R = a.R;
  const int jt = gridDim.x - 1 - blockIdx.x, tb = 4 * jt + w;
  T* sXs = sXbuf + w * 2 * 32 * SS;
  T* sXg = sXs + 32 * SS;
  const int pcol = perm16(col);
  Stager<TN, 4> stN;
  Stager<TT, 4> stT;
  stN.init(w, lane, D * (long)sizeof(T), 32);
  stT.init(w, lane, Lp * (long)sizeof(T), D);

  Frag<T> kt[NQ];
  {
    const T* krow = a.Kp + ((long)zk * Lp + 32 * tb + col) * D + 8 * hi;
#pragma unroll
    for (int q = 0; q < NQ; ++q) kt[q] = ld8(krow + 16 * q);
  }
  float lb[16];
  load_t16(a.ldest + (long)zk * Lp + 32 * tb, hi, lb);
  f32x16 dKc[NB];
#pragma unroll
  for (int n = 0; n < NB; ++n) dKc[n] = (f32x16){0};
  const float* Crow = a.C + ((long)zk * nT + tb) * Lp;
  const float* Drow = a.Dsuf + ((long)zk * nT + tb) * Lp;
  const float* lsz = a.lsrc + (long)zk * Lp;
  const T* Kz = a.Kp + (long)zk * Lp * D;
  const T* Vz = a.Vp + (long)zk * Lp * D;
  const T* KTz = a.KT + (long)zk * D * Lp;
  const int n_kt = 2 * jt + 2;

  for (int r = 0; r < R; ++r) {
    const long zq = (long)zk * R + r;
    Frag<T> qt[NQ], gt[NQ];
    {
      const T* qrow = a.Qp + (zq * Lp + 32 * tb + col) * D + 8 * hi;
      const T* grow = a.dOp + (zq * Lp + 32 * tb + col) * D + 8 * hi;
#pragma unroll
      for (int q = 0; q < NQ; ++q) { qt[q] = ld8(qrow + 16 * q); gt[q] = ld8(grow + 16 * q); }
    }
    float l2t[16], dlt[16];
    load_t16(a.lse2 + zq * Lp + 32 * tb, hi, l2t);
    load_t16(a.delta + zq * Lp + 32 * tb, hi, dlt);
    f32x16 dQ[NB];
#pragma unroll
    for (int n = 0; n < NB; ++n) dQ[n] = (f32x16){0};

#define UA_ISSUE(s, base)                                                                   \
  {                                                                                         \
    const int k0_ = 64 * (s);                                                               \
    stN.issue((base), Kz + (long)k0_ * D, w);                                               \
    stN.issue((base) + TN::BYTES, Kz + (long)(k0_ + 32) * D, w);                            \
    stN.issue((base) + 2 * TN::BYTES, Vz + (long)k0_ * D, w);                               \
    stN.issue((base) + 3 * TN::BYTES, Vz + (long)(k0_ + 32) * D, w);                        \
    stT.issue((base) + 4 * TN::BYTES, KTz + k0_, w);                                        \
    stT.issue((base) + 4 * TN::BYTES + TT::BYTES, KTz + k0_ + 32, w);                       \
    issue_row((base) + TILES + w * 1024,                                                    \
              (lane < 16 ? Crow : (lane < 32 ? lsz : Drow)) + k0_ + 4 * (lane & 15));       \
  }
#define UA_COMPUTE(s, base) bq_step((s), (base))
    auto bq_step = [&] __device__ (int kti, const char* base) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int sbk = 2 * kti + j;
        if (sbk > tb) continue;
        const T* sK = reinterpret_cast<const T*>(base + j * TN::BYTES);
        const T* sV = reinterpret_cast<const T*>(base + (2 + j) * TN::BYTES);
        const T* sKT = reinterpret_cast<const T*>(base + 4 * TN::BYTES + j * TT::BYTES);
        const bool diag = (sbk == tb);
        const float* stats = reinterpret_cast<const float*>(base + TILES + w * 1024);
        const float cin = stats[32 * j + col];
        const float la = stats[64 + 32 * j + col];
        const float din = (r == 0) ? stats[128 + 32 * j + col] : 0.f;
        f32x16 gk = {0}, sc = {0}, dP = {0};
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
          const Frag<T> kb = ld8(sK + col * LS + 16 * q + 8 * hi);
          mma(gk, kt[q], kb);
          mma(sc, qt[q], kb);
          mma(dP, gt[q], ld8(sV + col * LS + 16 * q + 8 * hi));
        }
        f32x16 aff, x;
        float lab[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          lab[v] = la + lb[v];
          gk[v] = log2_relu(gk[v]);
          aff[v] = affinity(gk[v], lab[v]);
          const float l2 = log2_one_minus(aff[v]);
          x[v] = (diag && t_of(v, hi) <= col) ? 0.f : l2;
        }
        block_prefix(x, hi);
        f32x16 dS;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[v], kLog2e, x[v] + cin) - l2t[v]);
          p = (diag && t_of(v, hi) < col) ? 0.f : p;
          dS[v] = p * (dP[v] - dlt[v]);
          sXs[t_of(v, hi) * SS + pcol] = cvt<T>(dS[v]);
        }
        block_suffix(dS, hi);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float dl = (diag && t_of(v, hi) <= col) ? 0.f : dS[v] + din;
          const float av = aff[v];
          const float den = fmaxf(fminf(av, kAMax), kAMinBwd) - 1.0f;
          const float dA = (av <= kAMax) ? dl * __builtin_amdgcn_rcpf(den) : 0.f;
          const float f = (2.0f / 3.0f) * __builtin_amdgcn_exp2f(__builtin_fmaf(gk[v], -1.0f / 3.0f, lab[v]));
          const float dg = (gk[v] > -1.0e30f) ? dA * f : 0.f;
          sXg[t_of(v, hi) * SS + pcol] = cvt<T>(dg);
        }
#pragma unroll
        for (int kq = 0; kq < 2; ++kq) {
          const Frag<T> as = ld8(sXs + col * SS + 16 * kq + 8 * hi), ag = ld8(sXg + col * SS + 16 * kq + 8 * hi);
#pragma unroll
          for (int n = 0; n < NB; ++n) {
            const Frag<T> kb = ld8(sKT + (32 * n + col) * TS + 16 * kq + 8 * hi);
            mma(dQ[n], as, kb);
            mma(dKc[n], ag, kb);
          }
        }
      }
    };
    UA_PIPELINE(n_kt, UA_ISSUE, UA_COMPUTE);
#undef UA_ISSUE
#undef UA_COMPUTE
    __syncthreads();   // the next group's prologue reuses stage 0
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int t = 32 * tb + t_of(v, hi);
      if (t < L) {
#pragma unroll
        for (int n = 0; n < NB; ++n) {
          const int dd = 32 * n + col;
          if (dd < d) dq[(zq * L + t) * d + dd] = cvt<T>(dQ[n][v]);
        }
      }
    }
  }
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int t = 32 * tb + t_of(v, hi);
#pragma unroll
    for (int n = 0; n < NB; ++n) a.dKdacc[((long)zk * Lp + t) * D + 32 * n + col] = dKc[n][v];
  }
}

#undef UA_PIPELINE
#undef UA_PIPE_RANGE
#undef UA_PIPE_START
#undef UA_STEP2_
#undef UA_STAGES

}  // namespace ua
