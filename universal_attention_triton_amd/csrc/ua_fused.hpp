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
// The same for data that is read exactly once (the exchanged tiles): non-temporal, so that it does not displace the
// operand tiles the workgroups of a head share in L2.
__device__ __forceinline__ void issue_row_nt(void* lds_base, const void* src_lane) {
  __builtin_amdgcn_global_load_lds(src_lane, (lds_ptr_t)lds_base, 16, 0, 2);
}

// Pipeline skeleton.  Every kernel declares two STATIC LDS arrays stage0 / stage1 (distinct objects, so the
// compiler can prove that the asynchronous loads filling one stage do not alias the reads of the other and
// does not wait for them) and provides ISSUE(step, stage) and COMPUTE(step, stage).
// UA_PIPE_RANGE runs steps [S0, S1) of a pipeline of NSTEPS steps whose step S0 has already been issued
// (by UA_PIPE_START or by the previous range), so that consecutive ranges may use different COMPUTE bodies.
#define UA_PIPE_START_AT(S0, NSTEPS, ISSUE)                                                \
  do {                                                                                     \
    if ((S0) < (NSTEPS)) ISSUE((S0), stage0);                                              \
  } while (0)
#define UA_PIPE_START(NSTEPS, ISSUE) UA_PIPE_START_AT(0, NSTEPS, ISSUE)
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
// The fused-path kernels tile with v_mfma_f32_16x16x32: a wave owns 16 stationary rows (keys in the
// key-stationary kernels, queries in the query-stationary ones), which halves its operand strips and
// accumulators so that two waves fit per SIMD; workgroups have 8 waves and share the staged tiles.
// Carries are kept per 16-query tile:
//   C[z][t16][s]    = sum_{u < 16*t16, u > s} log2(1 - A[s,u])        (t16 >= s/16 ... any t16 with 16*t16+15 >= s)
//   Dsuf[z][t16][s] = sum_{t >= 16*(t16+1)} dBias[s,t]
// ---------------------------------------------------------------------------------------------
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
struct TrueC { static constexpr bool value = true; };
struct FalseC { static constexpr bool value = false; };

// grid (Lp/128, Zk), 8 waves; wave w owns keys 16*(8*bx+w)..+15 and sweeps the 32-query blocks from its own on.
// CM: the key tensor is stored in tiled k-group-major order (fused mode) rather than row-major (chunked mode).
// Pruning (knorm2 != null; knorm2 [Zk][Lp/32] and qnorm2 [Zk*R][Lp/32] hold the largest squared row norm of every
// block of 32 keys / queries): a key whose accumulated bias has fallen below -(kPruneLog2 + 2 max|k| max|q| log2 e)
// cannot contribute a softmax weight above 2^-kPruneLog2 to any later query (the bias only decreases, a score
// is at most max|k| max|q|, and a query's normaliser is at least its own score); a wave stops once all its 16
// keys are there and records the last 32-query block it reached in reach[z][key tile].
// BO: instead of the carries C, leave the bias of every visited (16 keys, 32 queries) tile itself, as fp16, in
// Bt[z][causal triangle of (32-query block, 16-key tile) pairs, see tri_bias_row][1 KB]: lane l of the key tile's wave owns
// bytes 16 l .. 16 l + 15 = its
// key's bias towards queries 4g..4g+3 of the block's first 16-query tile, then of the second (g = l / 16).  The
// 16-bit forward and backward kernels then read the bias instead of recomputing the affinity chain; fp16 resolves
// the bias of every pair that carries weight (|bias| < 16: 2^-7 at worst) to better than the bf16 rounding of the
// softmax weight itself.
// NW: waves per workgroup (8, or 4 for launches of few workgroups: twice as many, half as long in LDS and registers).
template <class T, int D, int NST, bool CM, bool BO, int NW = 8>
__global__ void __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(2))) k_carry2(const T* __restrict__ Kp, const float* __restrict__ lsrc,
                                                const float* __restrict__ ldest, float* __restrict__ C, int Lp,
                                                const float* __restrict__ knorm2, const float* __restrict__ qnorm2, int R,
                                                int* __restrict__ reach, _Float16* __restrict__ Bt) {
  using TN = Tile<T, 32, D, CM>;
  constexpr int NK = D / 32, SB = TN::BYTES + 1024;   // tile + [ldest of the block: 32 floats]
  UA_STAGES(SB);
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, col = lane & 15, g = lane >> 4;
  // A launch of half as many workgroups has each sweep two key groups, bx and (number of key groups - 1 - bx), one after
  // the other with the body expanded once per key group (see k_bwd_keys2).  It pays in small launches (b = 2, h = 16,
  // L = 2048, d = 64: 0.074 -> 0.056 ms) and costs in large ones (b = 1, h = 32, L = 8192: 0.70 -> 0.83 ms), so it is a
  // variant of the tuning slot.
  int bx0, z;
  xcd_map(bx0, z);
  const int n_kg = Lp / (16 * NW);
  __shared__ int n_dead;
  __shared__ float red[2][NW];
  auto sweep = [&](const int bx) __attribute__((always_inline)) {
  const int nT = Lp / 32, nT16 = Lp / 16, sb16 = NW * bx + w, first = (NW / 2) * bx;
  const int spos = 16 * sb16 + col;
  const GroupMasks gm = group_masks(lane);
  Stager<TN, NW> st;
  st.init(w, lane, D * (long)sizeof(T), 32);
  Frag<T> ks[NK];
  {
#pragma unroll
    for (int q = 0; q < NK; ++q)
      ks[q] = ld8(Kp + (CM ? nat_off<D>(z, Lp, spos, 32 * q + 8 * g) : ((long)z * Lp + spos) * D + 32 * q + 8 * g));
  }
  const float la = lsrc[(long)z * Lp + spos];
  float carry = 0.f;
  // bias tiles: the running sum over the block's queries runs on the matrix core (see scan32_mma); carry4 replaces carry
  ScanOps sc_ops;
  f32x4 carry4 = {0, 0, 0, 0};
  if constexpr (BO) sc_ops = scan_operands<false>(lane);
  float* Cz = C + (long)z * nT16 * Lp + spos;
  const T* Kz = Kp + (long)z * Lp * D;
  bool dead = false;
  int last = sb16 >> 1;
  float thr = -3.0e38f;
  if (tid == 0) n_dead = 0;
  if (knorm2) {
    float km = 0.f, qm = 0.f;
    for (int i = tid; i < nT; i += 64 * NW) km = fmaxf(km, knorm2[(long)z * nT + i]);
    for (int i = tid; i < R * nT; i += 64 * NW) qm = fmaxf(qm, qnorm2[(long)z * R * nT + i]);
#pragma unroll
    for (int m = 1; m <= 32; m <<= 1) { km = fmaxf(km, __shfl_xor(km, m, 64)); qm = fmaxf(qm, __shfl_xor(qm, m, 64)); }
    if (lane == 0) { red[0][w] = km; red[1][w] = qm; }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NW; ++i) { km = fmaxf(km, red[0][i]); qm = fmaxf(qm, red[1][i]); }
    thr = -(kPruneLog2 + 2.0f * kLog2e * sqrtf(km * qm));
  }
  __syncthreads();
#define UA_ISSUE(s, base)                                                                   \
  {                                                                                         \
    st.issue((base), Kz + (long)32 * (first + (s)) * D, w);                                 \
    if (w == 0) issue_row((base) + TN::BYTES, ldest + (long)z * Lp + 32 * (first + (s)) + 4 * (lane & 7)); \
  }
#define UA_COMPUTE_FAST(s, base) carry_step((s), (base), FalseC())
#define UA_COMPUTE_SLOW(s, base)                                                            \
  {                                                                                         \
    if (first + (s) >= (sb16 >> 1)) carry_step((s), (base), TrueC());                       \
  }
  auto carry_step = [&] __device__ (int s, const char* base, auto masked_c) {
    constexpr bool MASKED = decltype(masked_c)::value;
    const int tb = first + s;
    if (dead) return;
    if (__builtin_amdgcn_ballot_w64((BO ? carry4[0] : carry) > thr) == 0) {        // every key of this wave is out of reach from here on
      dead = true;
      if (lane == 0) atomicAdd(&n_dead, 1);
      return;
    }
    last = tb;
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
        float l2 = log2_one_minus(affinity(log2_relu(acc[v]), la + lb[v]));
        if (MASKED) l2 = (32 * tb + 16 * i + 4 * g + v <= spos) ? 0.f : l2;
        x[i][v] = l2;
      }
    }
    if constexpr (BO) {
      f32x4 y[2];
      scan32_mma(sc_ops, as_operand16<bf16>(x[0], x[1]), carry4, y);
      typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
      f16x8 hb;
#pragma unroll
      for (int v = 0; v < 4; ++v) { hb[v] = (_Float16)y[0][v]; hb[4 + v] = (_Float16)y[1][v]; }
      char* dst = reinterpret_cast<char*>(Bt) + (((long)z * tri_tiles(nT) + tri_bias_row(tb) + sb16) << 10) + 16 * lane;
      __builtin_nontemporal_store(hb, reinterpret_cast<f16x8*>(dst));
    } else {
      float b0, a0, t0, b1, a1, t1;
      group_scan((x[0][0] + x[0][1]) + (x[0][2] + x[0][3]), gm, b0, a0, t0);
      group_scan((x[1][0] + x[1][1]) + (x[1][2] + x[1][3]), gm, b1, a1, t1);
      if (g == 0) {
        Cz[(long)(2 * tb) * Lp] = carry;
        Cz[(long)(2 * tb + 1) * Lp] = carry + t0;
      }
      carry += t0 + t1;
    }
  };
  {
    // segments of 16 blocks, so that the workgroup can leave once all its waves have stopped
    const int total = nT - first;
    for (int s0 = 0; s0 < total; s0 += 16) {
      const int s1 = min(total, s0 + 16);
      UA_PIPE_START_AT(s0, s1, UA_ISSUE);
      if (s0 == 0) {
        const int nslow = s1 < NW / 2 ? s1 : NW / 2;               // the first NW / 2 blocks hold the diagonals
        UA_PIPE_RANGE(0, nslow, s1, UA_ISSUE, UA_COMPUTE_SLOW);
        UA_PIPE_RANGE(nslow, s1, s1, UA_ISSUE, UA_COMPUTE_FAST);
      } else {
        UA_PIPE_RANGE(s0, s1, s1, UA_ISSUE, UA_COMPUTE_FAST);
      }
      __syncthreads();
      if (n_dead == NW) break;
    }
  }
#undef UA_ISSUE
#undef UA_COMPUTE_FAST
#undef UA_COMPUTE_SLOW
  if (reach && lane == 0) reach[z * nT16 + sb16] = last;
  };
  sweep(bx0);
  if ((int)gridDim.x != n_kg && n_kg - 1 - bx0 != bx0) {
    __syncthreads();       // the stages, n_dead and red are free
    sweep(n_kg - 1 - bx0);
  }
}

// minkey[z][tb] = first key tile (of 16) that reaches query block tb; it never decreases with tb.
template <class Unused = void>
__global__ void __launch_bounds__(256) k_minkey(const int* __restrict__ reach, int* __restrict__ minkey, int nT16) {
  const int z = blockIdx.y, tb = blockIdx.x * 256 + threadIdx.x, nT32 = nT16 / 2;
  if (tb >= nT32) return;
  int sb = 0;
  while (sb < 2 * tb && reach[z * nT16 + sb] < tb) ++sb;          // tiles 2 tb and 2 tb + 1 hold the block's own keys
  minkey[z * nT32 + tb] = sb;
}

// Destination of the per-chunk results of the chunked operator (reference universal_attention_autograd.py:9-38):
// out element (zq, t, dd, i) at zq*sz + t*st + dd*sd + i*si, denom [Zq][L][nch]; either may be null.
template <class T> struct ChunkOut {
  T* out;
  T* denom;
  long sz, st, sd, si;
  int c, nch;
  int vec;      // rows of out[.., i] are contiguous in dd (sd == 1), 16-byte aligned, and d is a multiple of the vector
};

// Queries that precede a whole chunk see none of its keys; the reference's softmax over a row of equal fill values
// is uniform there: out = mean of the chunk's values (through a dtype-rounded 1/c), denom = float32(-1e12).
// grid (ceil(max rows / kMaskedSlab), nch, Zq), 256 threads: slab x of chunk i writes rows [x kMaskedSlab, (x + 1) kMaskedSlab)
// ∩ [0, i*c) of out[.., i].  vec: rows of out[.., i] are contiguous in dd, 16-byte aligned and d is a multiple of the vector.
constexpr int kMaskedSlab = 4096;
template <class T, int D>
__global__ void __launch_bounds__(256) k_chunk_masked_out(const T* __restrict__ Vp, ChunkOut<T> co, int R, int L, int Lp, int d,
                                                          int vec) {
  constexpr int V = 16 / (int)sizeof(T), NKG = D / 8, NRG = 256 / NKG;
  __shared__ __attribute__((aligned(16))) T mean[D];
  __shared__ float part[NRG][D];
  const int i = blockIdx.y, zq = blockIdx.z, zk = zq / R, tid = threadIdx.x;
  const int rows = min(i * co.c, L), r0 = blockIdx.x * kMaskedSlab, r1 = min(rows, r0 + kMaskedSlab);
  if (r0 >= rows) return;
  const float pu = (float)cvt<T>(1.0f / (float)co.c);
  {
    // thread (k-group kg, row group rg) adds up the 8-element cells of rows rg, rg + NRG, ... of the chunk
    const int kg = tid % NKG, rg = tid / NKG;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    for (int s = rg; s < co.c; s += NRG) {
      const Frag<T> x = ld8(Vp + nat_off<D>(zk, Lp, i * co.c + s, 8 * kg));
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += pu * (float)x.v[e];
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) part[rg][8 * kg + e] = acc[e];
  }
  __syncthreads();
  for (int dd = tid; dd < D; dd += 256) {
    float acc = 0.f;
#pragma unroll
    for (int rg = 0; rg < NRG; ++rg) acc += part[rg][dd];
    mean[dd] = cvt<T>(acc);
  }
  __syncthreads();
  T* base = co.out + (long)zq * co.sz + (long)i * co.si;
  if (vec) {
    const int vpr = d / V;                                      // vectors per row
    if (256 % vpr == 0) {
      // a thread keeps its piece of the row in registers and walks down the rows: nothing but stores in the loop (plain
      // ones: 6 % faster here than non-temporal ones; slabs of 4096 rows instead of 1024: the mean is computed a quarter
      // as often; together 0.55 -> 0.43 ms for the 2.15 GB of the headline shape with chunk 128)
      const int cv = tid % vpr, rstep = 256 / vpr;
      const u32x4 val = *reinterpret_cast<const u32x4*>(mean + cv * V);
      T* p = base + (long)(r0 + tid / vpr) * co.st + cv * V;
      const long pstep = (long)rstep * co.st;
#pragma unroll 8
      for (int t = r0 + tid / vpr; t < r1; t += rstep, p += pstep) *reinterpret_cast<u32x4*>(p) = val;
    } else
    for (int idx = tid; idx < (r1 - r0) * vpr; idx += 256) {
      const int t = r0 + idx / vpr, cv = idx % vpr;
      // written once and read by nobody in the reference's call sequence (the merge skips slices of zero weight)
      __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(mean + cv * V), reinterpret_cast<u32x4*>(base + (long)t * co.st + cv * V));
    }
  } else {
    for (int idx = tid; idx < (r1 - r0) * d; idx += 256) {
      const int t = r0 + idx / d, dd = idx % d;
      base[(long)t * co.st + (long)dd * co.sd] = mean[dd];
    }
  }
}
// denom[zq][t][i] = -1e12 and lse2[zq*nch + i][t] = "no visible key" for the chunks i after the one holding query t.
// grid (ceil(Lp/256), Zq); denom may be null.
template <class T>
__global__ void __launch_bounds__(256) k_chunk_masked_denom(T* __restrict__ denom, float* __restrict__ lse2, int L, int Lp,
                                                            int c, int nch) {
  const int t = blockIdx.x * 256 + threadIdx.x, zq = blockIdx.y;
  if (t >= Lp) return;
  const T fill = cvt<T>(kNegFill);
  for (int i = t / c + 1; i < nch; ++i) {
    if (denom && t < L) denom[((long)zq * L + t) * nch + i] = fill;
    lse2[((long)zq * nch + i) * Lp + t] = kNoKeyLse;
  }
}

// ---------------------------------------------------------------------------------------------
// Fused forward.  grid (ceil(Lp/16/NW), Zq); NW waves; wave w owns queries 16*(NW*jt+w)..+15; 64 keys per step,
// key tiles visited from the diagonal backwards.
// ---------------------------------------------------------------------------------------------
// CHUNKED: the reference's chunked operator instead of the merged one: the softmax restarts at every chunk of
// co.c keys (a multiple of 64) and each chunk's result goes to out[.., i] / denom[.., i] / lse2[zq*nch + i][t].
// BI (4 or 8 waves): the decay bias comes from the fp16 tiles k_carry2<BO> left in Bt instead of being recomputed (no key-key
// product, no affinity chain, no scan).  The two waves that share a 32-query block copy its four key tiles (two each)
// into one LDS region per step.
// RB (bias tiles, 8 waves): query groups of one kv head per workgroup.  With grouped queries the RB groups' waves of a
// 32-query block share the block's key, value and bias tiles: the workgroup then covers 4 / RB blocks of RB heads
// (grid (Lp / (128 / RB), Zk * R / RB)) instead of 4 blocks of one head.
template <class T, int D, int NST, int NW, bool CHUNKED, bool BI = false, int RB = 1>
__global__ void __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(NW >= 8 ? (BI && NST == 1 ? (D > 128 ? 2 : 4) : NW / 4) : (BI ? 3 : 2), NW >= 8 ? (BI && NST == 1 ? (D > 128 ? 2 : 4) : NW / 4) : (BI ? 3 : 2)))) k_fwd_fused2(const T* __restrict__ Qp, const T* __restrict__ Kp,
                                                    const T* __restrict__ VT, const float* __restrict__ lsrc,
                                                    const float* __restrict__ ldest, const float* __restrict__ C,
                                                    T* __restrict__ O, float* __restrict__ lse, float* __restrict__ lse2,
                                                    const int* __restrict__ reach, const int* __restrict__ minkey,
                                                    int R, int L, int Lp, int d, ChunkOut<T> co,
                                                    const _Float16* __restrict__ Bt = nullptr) {
  static_assert(!BI || ((NW == 8 || NW == 4) && !CHUNKED), "bias tiles: 4 or 8 waves, merged operator");
  static_assert(RB == 1 || (BI && NW == 8 && (RB == 2 || RB == 4)), "shared blocks: bias tiles, 8 waves, 2 or 4 query groups");
  using TN = Tile<T, 32, D>;
  using TT = Tile<T, D, 32>;
  constexpr int NK = D / 32, ND = D / 16;
  using ST = StageT<T>;
  // + per wave [C row: 64f][lsrc: 64f][reach], or (BI) per pair of waves 4 bias tiles of 1 KB, then one reach row
  constexpr int TILES = 2 * TN::BYTES + 2 * TT::BYTES, SB = TILES + (BI ? NW * 2048 + 1024 : NW * 1024);
  UA_STAGES(SB);
  __shared__ __attribute__((aligned(256))) char sPbuf[NW * 2 * ST::BYTES];
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, col = lane & 15, g = lane >> 4;
  int bx, zy;
  xcd_map(bx, zy);
  constexpr int NB = NW / (2 * RB);                          // 32-query blocks per workgroup
  // wave w: block w / (2 RB) of the workgroup, query group (w / 2) % RB of the workgroup's RB, half w % 2 of the block
  const int zq = RB == 1 ? zy : (zy / (R / RB)) * R + (zy % (R / RB)) * RB + (w >> 1) % RB;
  const int zk = zq / R, nT16 = Lp / 16;
  // chunked operator, 16-bit outputs: per-wave [16 queries][D + 8] tile through which a chunk's result is transposed
  __shared__ __attribute__((aligned(16))) T sObuf[(CHUNKED && sizeof(T) == 2) ? NW * 16 * (D + 8) : 8];
  const int n_blk = (nT16 + NW - 1) / NW;                    // workgroup blocks of 16 NW queries
  // chunked operator: a workgroup may handle two blocks of complementary length, jt and n_blk - 1 - jt, the body
  // expanded once per block (see k_bwd_keys2)
  auto sweep = [&](const int jt) __attribute__((always_inline)) {
  const int blk = w / (2 * RB), wb = w % (2 * RB), tq_raw = 2 * (NB * jt + blk) + (w & 1);
  const bool live = tq_raw < nT16;                           // the last workgroup may hold waves past the end
  const int tq = live ? tq_raw : nT16 - 1;                   // 16-query tile of this wave
  char* sPw = sPbuf + w * 2 * ST::BYTES;     // P of the two 32-key halves of a step
  T* sOw = sObuf + ((CHUNKED && sizeof(T) == 2) ? w * 16 * (D + 8) : 0);
  const GroupMasks gm = group_masks(lane);
  Stager<TN, NW> stN;
  Stager<TT, NW> stT;
  stN.init(w, lane, D * (long)sizeof(T), 32);
  stT.init(w, lane, Lp * (long)sizeof(T), D);

  Frag<T> qf[NK], kf[NK];
  {
#pragma unroll
    for (int q = 0; q < NK; ++q) {
      qf[q] = ld8(Qp + nat_off<D>(zq, Lp, 16 * tq + col, 32 * q + 8 * g));
      if (!BI) kf[q] = ld8(Kp + nat_off<D>(zk, Lp, 16 * tq + col, 32 * q + 8 * g));
    }
  }
  f32x4 lb = {0, 0, 0, 0};
  if (!BI) lb = load_t4(ldest + (long)zk * Lp + 16 * tq, g);
  f32x4 o[ND];
#pragma unroll
  for (int n = 0; n < ND; ++n) o[n] = (f32x4){0, 0, 0, 0};
  f32x4 m = {-1.0e30f, -1.0e30f, -1.0e30f, -1.0e30f}, ls = {0, 0, 0, 0};
  const T* Kz = Kp + (long)zk * Lp * D;
  const T* Vz = VT + (long)zk * D * Lp;
  const int tq_end = min(2 * NB * (jt + 1), nT16);
  const int n_kt = (tq_end + 3) / 4;   // key tiles of 64 covering s <= last query of the workgroup
  // key tiles that cannot reach this workgroup's first query block (see k_carry2) are not visited at all; inside
  // the visited range a tile that does not reach this wave's block gets a carry of -1e30 (its weights become 0)
  const int tbq = tq >> 1;
  const int kt_min = minkey[zk * (nT16 >> 1) + NB * jt] >> 2;
  const int n_steps = n_kt - kt_min;
  // per-wave stats row of a step: [C row: 64f][lsrc: 64f][reach of the 4 key tiles: 4 ints]; source of each lane's
  // 16 bytes as base + step * stride (in 4-byte units)
  const float* row_base;
  int row_step = 64;
  if (lane < 16) row_base = C + ((long)zk * nT16 + tq) * Lp + 4 * lane;
  else if (lane < 32) row_base = lsrc + (long)zk * Lp + 4 * (lane - 16);
  else { row_base = reinterpret_cast<const float*>(reach + zk * nT16); row_step = 4; }
  // BI: this lane's 16 bytes of key tile 0 of the wave's query block
  const char* bt_src = reinterpret_cast<const char*>(Bt) + (((long)zk * tri_tiles(Lp >> 5) + tri_bias_row(tbq)) << 10) + 16 * lane;

#define UA_ISSUE(s, base)                                                                   \
  {                                                                                         \
    const int kt_ = n_kt - 1 - (s);                                                         \
    stN.issue((base), Kz + (long)(64 * kt_) * D, w);                                        \
    stN.issue((base) + TN::BYTES, Kz + (long)(64 * kt_ + 32) * D, w);                       \
    stT.issue((base) + 2 * TN::BYTES, Vz + (long)(2 * kt_) * (32 * D), w);                  \
    stT.issue((base) + 2 * TN::BYTES + TT::BYTES, Vz + (long)(2 * kt_ + 1) * (32 * D), w);  \
    if (BI) {                                                                               \
      /* the 2 RB waves of a block fetch its four bias tiles: two each, or one each (the first four waves) */ \
      if (RB == 1) {                                                                        \
        const char* src_ = bt_src + ((long)(4 * kt_ + 2 * wb) << 10);                       \
        char* dst_ = (base) + TILES + blk * 4096 + wb * 2048;                               \
        issue_row_nt(dst_, src_);                                                           \
        issue_row_nt(dst_ + 1024, src_ + 1024);                                             \
      } else if (wb < 4) {                                                                  \
        issue_row_nt((base) + TILES + blk * 4096 + wb * 1024, bt_src + ((long)(4 * kt_ + wb) << 10)); \
      }                                                                                     \
      if (w == 0) issue_row((base) + TILES + NW * 2048, reach + zk * nT16 + 4 * kt_);        \
    } else {                                                                                \
      issue_row((base) + TILES + w * 1024, row_base + (long)kt_ * row_step);                \
    }                                                                                       \
  }
#define UA_COMPUTE_FAST(s, base) fwd_tile(n_kt - 1 - (s), (base), FalseC())
#define UA_COMPUTE_SLOW(s, base) fwd_tile(n_kt - 1 - (s), (base), TrueC())
  // chunked operator: chunk i is complete, write its normalised result and restart the softmax
  auto flush_chunk = [&] __device__ (int i) __attribute__((always_inline)) {
    // chunks after this wave's queries are written by k_chunk_masked_*; a key tile of padding beyond the last chunk
    // (L a multiple of 64 but not of 128) belongs to no chunk
    if (live && i < co.nch && i <= (16 * tq) / co.c) {
      const bool via_lds = sizeof(T) == 2 && co.vec && co.out;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const float tot = allsum16(ls[v]);
        const float inv = 1.0f / tot;
        const int t = 16 * tq + 4 * g + v;
        if (via_lds) {
          // transpose through the wave's LDS tile [16 queries][D] so that rows leave as 16-byte vectors
#pragma unroll
          for (int n = 0; n < ND; ++n) sOw[(4 * g + v) * (D + 8) + 16 * n + col] = cvt<T>(o[n][v] * inv);
        } else if (t < L && co.out) {
#pragma unroll
          for (int n = 0; n < ND; ++n) {
            const int dd = 16 * n + col;
            if (dd < d) co.out[(long)zq * co.sz + (long)t * co.st + (long)dd * co.sd + (long)i * co.si] = cvt<T>(o[n][v] * inv);
          }
        }
        if (col == 0) {
          const float l2v = m[v] + __builtin_amdgcn_logf(tot);
          lse2[((long)zq * co.nch + i) * Lp + t] = (t < L) ? l2v : 0.f;
          if (t < L && co.denom) co.denom[((long)zq * L + t) * co.nch + i] = cvt<T>(l2v * kLn2);
        }
      }
      if (via_lds) {
        constexpr int VPR = D / 8;                               // 16-byte vectors per row
        T* dst = co.out + (long)zq * co.sz + (long)i * co.si;
#pragma unroll
        for (int k = 0; k < 16 * VPR / 64; ++k) {
          const int idx = 64 * k + lane, row = idx / VPR, cv = idx % VPR, t = 16 * tq + row;
          if (t < L && 8 * cv < d)
            *reinterpret_cast<uint4*>(dst + (long)t * co.st + 8 * cv) = *reinterpret_cast<const uint4*>(sOw + row * (D + 8) + 8 * cv);
        }
      }
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) { m[v] = -1.0e30f; ls[v] = 0.f; }
#pragma unroll
    for (int n = 0; n < ND; ++n) o[n] = (f32x4){0, 0, 0, 0};
  };
  auto fwd_tile = [&] __device__ (int kt, const char* base, auto masked_c) {
    constexpr bool MASKED = decltype(masked_c)::value;
    const float* stats = reinterpret_cast<const float*>(base + TILES + w * 1024);
    f32x4 s2[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int sbk = 4 * kt + j;                      // 16-key tile
      const T* sK = reinterpret_cast<const T*>(base + (j >> 1) * TN::BYTES);
      if constexpr (BI) {
        if (!MASKED || sbk <= tq) {
          f32x4 sc = {0, 0, 0, 0};
#pragma unroll
          for (int q = 0; q < NK; ++q) mma16(sc, qf[q], ld8(sK + TN::at(j & 1, col, q, g)));
          typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
          const f16x4 hb = *reinterpret_cast<const f16x4*>(base + TILES + blk * 4096 + j * 1024 + 16 * lane + 8 * (w & 1));
          const bool in_reach = reinterpret_cast<const int*>(base + TILES + NW * 2048)[j] >= tbq;
          const bool diag = MASKED && (sbk == tq);
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const float x = in_reach ? __builtin_fmaf(sc[v], kLog2e, (float)hb[v]) : -1.0e30f;
            s2[j][v] = (MASKED && diag && 4 * g + v < col) ? -1.0e30f : x;
          }
        } else {
          s2[j] = (f32x4){-1.0e30f, -1.0e30f, -1.0e30f, -1.0e30f};
        }
      } else if (!MASKED || sbk <= tq) {
        const float c = reinterpret_cast<const int*>(stats)[128 + j] >= tbq ? stats[16 * j + col] : -1.0e30f;
        const float la = stats[64 + 16 * j + col];
        f32x4 gt = {0, 0, 0, 0}, sc = {0, 0, 0, 0};
#pragma unroll
        for (int q = 0; q < NK; ++q) {
          const Frag<T> kb = ld8(sK + TN::at(j & 1, col, q, g));
          mma16(gt, kf[q], kb);
          mma16(sc, qf[q], kb);
        }
        const bool diag = MASKED && (sbk == tq);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const float l2 = log2_one_minus(affinity(log2_relu(gt[v]), la + lb[v]));
          gt[v] = (MASKED && diag && 4 * g + v <= col) ? 0.f : l2;
        }
        // inclusive prefix over the 16 queries of this wave
        gt[1] += gt[0]; gt[2] += gt[1]; gt[3] += gt[2];
        float before, after, tot;
        group_scan(gt[3], gm, before, after, tot);
        before += c;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const float x = __builtin_fmaf(sc[v], kLog2e, gt[v] + before);
          s2[j][v] = (MASKED && diag && 4 * g + v < col) ? -1.0e30f : x;
        }
      } else {
        s2[j] = (f32x4){-1.0e30f, -1.0e30f, -1.0e30f, -1.0e30f};
      }
    }
    // online softmax: rescale only when some query of this wave raises its maximum
    f32x4 mx;
    bool grow = false;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      mx[v] = allmax16(fmaxf(fmaxf(s2[0][v], s2[1][v]), fmaxf(s2[2][v], s2[3][v])));
      grow |= (mx[v] > m[v]);
    }
    if (__builtin_amdgcn_ballot_w64(grow) != 0) {
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const float mn = fmaxf(m[v], mx[v]);
        const float alpha = __builtin_amdgcn_exp2f(m[v] - mn);
        m[v] = mn;
        ls[v] *= alpha;
#pragma unroll
        for (int n = 0; n < ND; ++n) o[n][v] *= alpha;
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f32x4 p;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        p[v] = __builtin_amdgcn_exp2f(s2[j][v] - m[v]);
        ls[v] += p[v];
      }
      ST::put(sPw + (j >> 1) * ST::BYTES, 16 * (j & 1) + col, g, p);
    }
#pragma unroll
    for (int kq = 0; kq < 2; ++kq) {                   // 32 keys per k-step
      if (!MASKED || 4 * kt + 2 * kq <= tq) {
        const T* sV = reinterpret_cast<const T*>(base + 2 * TN::BYTES + kq * TT::BYTES);
        const Frag<T> pa = ST::get(sPw + kq * ST::BYTES, lane);
#pragma unroll
        for (int n = 0; n < ND; ++n) mma16(o[n], pa, ld8(sV + TT::at(n, col, 0, g)));
      }
    }
    if constexpr (CHUNKED) {
      if ((64 * kt) % co.c == 0) flush_chunk(64 * kt / co.c);
    }
  };
  {
    // the key tiles visited first hold the diagonal blocks of the waves
    const int nslow = min(n_steps, (n_kt - (2 * NB * jt) / 4 + 1) & ~1);
    UA_PIPE_START(n_steps, UA_ISSUE);
    UA_PIPE_RANGE(0, nslow, n_steps, UA_ISSUE, UA_COMPUTE_SLOW);
    UA_PIPE_RANGE(nslow, n_steps, n_steps, UA_ISSUE, UA_COMPUTE_FAST);
  }
#undef UA_ISSUE
#undef UA_COMPUTE_FAST
#undef UA_COMPUTE_SLOW
  // epilogue
  if (CHUNKED || !live) return;
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const float tot = allsum16(ls[v]);
    const float inv = 1.0f / tot;
    const int t = 16 * tq + 4 * g + v;
    if (t < L) {
#pragma unroll
      for (int n = 0; n < ND; ++n) {
        const int dd = 16 * n + col;
        if (dd < d) O[((long)zq * L + t) * d + dd] = cvt<T>(o[n][v] * inv);
      }
    }
    if (col == 0) {
      const float l2v = m[v] + __builtin_amdgcn_logf(tot);
      lse2[(long)zq * Lp + t] = (t < L) ? l2v : 0.f;
      if (t < L) lse[(long)zq * L + t] = l2v * kLn2;
    }
  }
  };
  if constexpr (CHUNKED) {
    sweep(n_blk - 1 - bx);                                   // heaviest first
    if ((int)gridDim.x != n_blk && n_blk - 1 - bx != bx) {
      __syncthreads();       // the stages are free
      sweep(bx);
    }
  } else {
    sweep((int)gridDim.x - 1 - bx);
  }
}

// ---------------------------------------------------------------------------------------------
// Fused forward of the 16-bit operator with bias tiles, one 32-query block per wave.
// grid (n or ceil(n / 2), Zk * R / RB) with n = ceil(Lp/32 / NB) workgroup blocks jt (the second form: blocks jt and
// n - 1 - jt one after the other, see the body), 8 waves, NB = 8 / RB 32-query blocks per workgroup block; wave w owns block NB jt + w / RB of
// query group w % RB of the workgroup's RB groups (grouped queries share the key and value tiles of a step).
// Against k_fwd_fused2<BI> (16 queries per wave): every key / value operand read from LDS feeds two matrix
// instructions (the two 16-query tiles of the block), the staged tiles serve 256 queries instead of 128, and a bias
// tile of k_carry2<BO> -- (16 keys, 32 queries), lane l owning bytes 16 l .. 16 l + 15 -- is exactly what a lane of
// this kernel needs for a key tile, so it is loaded straight into registers one step ahead and never touches LDS.
// 64 keys per step, key tiles visited from the diagonal backwards, two LDS stages.
// ---------------------------------------------------------------------------------------------
template <int D, int RB>
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
k_fwd_fused3(const bf16* __restrict__ Qp, const bf16* __restrict__ Kp, const bf16* __restrict__ VT, bf16* __restrict__ O,
             float* __restrict__ lse, float* __restrict__ lse2, const int* __restrict__ reach, const int* __restrict__ minkey,
             int R, int L, int Lp, int d, const _Float16* __restrict__ Bt) {
  using T = bf16;
  using TN = Tile<T, 32, D>;
  using TT = Tile<T, D, 32>;
  using ST = StageT<T>;
  static_assert(RB == 1 || RB == 2 || RB == 4, "1, 2 or 4 query groups per workgroup");
  constexpr int NK = D / 32, ND = D / 16, NST = 2, NB = 8 / RB;
  constexpr int TILES = 2 * TN::BYTES + 2 * TT::BYTES, SB = TILES + 1024;     // + reach of the step's four key tiles
  UA_STAGES(SB);
  __shared__ __attribute__((aligned(256))) char sPbuf[8 * 4 * ST::BYTES];     // per wave: P of (query tile, 32-key half)
  typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, col = lane & 15, g = lane >> 4;
  // A workgroup handles two blocks of 32 NB queries one after the other, jt and (number of blocks - 1 - jt): every pair
  // visits the same number of key tiles, so the launch is a whole number of equal rounds with half the workgroup changes
  // (see k_bwd_keys2).  The body is expanded once per block.
  int bx0, zy;
  xcd_map(bx0, zy);
  const int n_blk = (Lp / 32 + NB - 1) / NB;
  auto sweep = [&](const int jt) __attribute__((always_inline)) {
  const int zq = RB == 1 ? zy : (zy / (R / RB)) * R + (zy % (R / RB)) * RB + w % RB;
  const int zk = zq / R, nT16 = Lp / 16, nT32 = Lp / 32;
  const int qb_raw = NB * jt + w / RB;
  const bool live = qb_raw < nT32;                            // the last workgroup may hold waves past the end
  const int qb = live ? qb_raw : nT32 - 1;                    // 32-query block of this wave
  char* sPw = sPbuf + w * 4 * ST::BYTES;
  Stager<TN, 8> stN;
  Stager<TT, 8> stT;
  stN.init(w, lane, D * (long)sizeof(T), 32);
  stT.init(w, lane, Lp * (long)sizeof(T), D);

  Frag<T> qf[2][NK];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int q = 0; q < NK; ++q) qf[i][q] = ld8(Qp + nat_off<D>(zq, Lp, 32 * qb + 16 * i + col, 32 * q + 8 * g));
  f32x4 o[2][ND], m[2], ls[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int n = 0; n < ND; ++n) o[i][n] = (f32x4){0, 0, 0, 0};
    m[i] = (f32x4){-1.0e30f, -1.0e30f, -1.0e30f, -1.0e30f};
    ls[i] = (f32x4){0, 0, 0, 0};
  }
  const T* Kz = Kp + (long)zk * Lp * D;
  const T* Vz = VT + (long)zk * D * Lp;
  const int qb_end = min(NB * (jt + 1), nT32);
  const int n_kt = (qb_end + 1) / 2;                          // key tiles of 64 covering s <= last query of the workgroup
  // key tiles that cannot reach this workgroup's first query block (see k_carry2) are not visited
  const int kt_min = minkey[zk * nT32 + NB * jt] >> 2;
  const int n_steps = n_kt - kt_min;
  // this lane's 16 bytes of key tile 0 of the wave's query block
  const char* bt_src = reinterpret_cast<const char*>(Bt) + (((long)zk * tri_tiles(nT32) + tri_bias_row(qb)) << 10) + 16 * lane;
  f16x8 hb_next[4];
  auto load_bias = [&] __device__ (int kt) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      hb_next[j] = __builtin_nontemporal_load(reinterpret_cast<const f16x8*>(bt_src + ((long)(4 * kt + j) << 10)));
  };

#define UA_ISSUE(s, base)                                                                   \
  {                                                                                         \
    const int kt_ = n_kt - 1 - (s);                                                         \
    stN.issue((base), Kz + (long)(64 * kt_) * D, w);                                        \
    stN.issue((base) + TN::BYTES, Kz + (long)(64 * kt_ + 32) * D, w);                       \
    stT.issue((base) + 2 * TN::BYTES, Vz + (long)(2 * kt_) * (32 * D), w);                  \
    stT.issue((base) + 2 * TN::BYTES + TT::BYTES, Vz + (long)(2 * kt_ + 1) * (32 * D), w);  \
    if (w == 0) issue_row((base) + TILES, reach + zk * nT16 + 4 * kt_);                      \
  }
#define UA_COMPUTE_FAST(s, base) fwd_tile(n_kt - 1 - (s), (base), FalseC())
#define UA_COMPUTE_SLOW(s, base) fwd_tile(n_kt - 1 - (s), (base), TrueC())
  auto fwd_tile = [&] __device__ (int kt, const char* base, auto masked_c) {
    constexpr bool MASKED = decltype(masked_c)::value;
    // the bias tiles of this step arrived during the previous one; fetch the next step's (a tile row is followed by
    // the next rows and the tensor by slack, so the loads of the last step stay inside the tensor)
    f16x8 hb[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) hb[j] = hb_next[j];
    if (kt > 0) load_bias(kt - 1);
    if (MASKED && 4 * kt > 2 * qb + 1) return;         // the whole step lies after this wave's queries
    const int* rch = reinterpret_cast<const int*>(base + TILES);
    f32x4 s2[2][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int sbk = 4 * kt + j;                      // 16-key tile
      const T* sK = reinterpret_cast<const T*>(base + (j >> 1) * TN::BYTES);
      if (!MASKED || sbk <= 2 * qb + 1) {
        f32x4 sc[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
#pragma unroll
        for (int q = 0; q < NK; ++q) {
          const Frag<T> kb = ld8(sK + TN::at(j & 1, col, q, g));
          mma16(sc[0], qf[0][q], kb);
          mma16(sc[1], qf[1][q], kb);
        }
        const bool in_reach = rch[j] >= qb;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const int tq = 2 * qb + i;
          const bool diag = MASKED && sbk == tq, after = MASKED && sbk > tq;
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const float x = in_reach ? __builtin_fmaf(sc[i][v], kLog2e, (float)hb[j][4 * i + v]) : -1.0e30f;
            s2[i][j][v] = (MASKED && (after || (diag && 4 * g + v < col))) ? -1.0e30f : x;
          }
        }
      } else {
        s2[0][j] = (f32x4){-1.0e30f, -1.0e30f, -1.0e30f, -1.0e30f};
        s2[1][j] = s2[0][j];
      }
    }
    // online softmax: rescale only when some query of this wave raises its maximum
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      f32x4 mx;
      bool grow = false;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        mx[v] = allmax16(fmaxf(fmaxf(s2[i][0][v], s2[i][1][v]), fmaxf(s2[i][2][v], s2[i][3][v])));
        grow |= (mx[v] > m[i][v]);
      }
      if (__builtin_amdgcn_ballot_w64(grow) != 0) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const float mn = fmaxf(m[i][v], mx[v]);
          const float alpha = __builtin_amdgcn_exp2f(m[i][v] - mn);
          m[i][v] = mn;
          ls[i][v] *= alpha;
#pragma unroll
          for (int n = 0; n < ND; ++n) o[i][n][v] *= alpha;
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        f32x4 p;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          p[v] = __builtin_amdgcn_exp2f(s2[i][j][v] - m[i][v]);
          ls[i][v] += p[v];
        }
        ST::put(sPw + (2 * i + (j >> 1)) * ST::BYTES, 16 * (j & 1) + col, g, p);
      }
    }
    // the 32 independent matrix instructions of P V issue back to back while the SIMD's other wave fills the gaps
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int kq = 0; kq < 2; ++kq) {                   // 32 keys per k-step
      if (!MASKED || 4 * kt + 2 * kq <= 2 * qb + 1) {
        const T* sV = reinterpret_cast<const T*>(base + 2 * TN::BYTES + kq * TT::BYTES);
        const Frag<T> pa0 = ST::get(sPw + kq * ST::BYTES, lane), pa1 = ST::get(sPw + (2 + kq) * ST::BYTES, lane);
#pragma unroll
        for (int n = 0; n < ND; ++n) {
          const Frag<T> vb = ld8(sV + TT::at(n, col, 0, g));
          mma16(o[0][n], pa0, vb);
          mma16(o[1][n], pa1, vb);
        }
      }
    }
    __builtin_amdgcn_s_setprio(0);
  };
  {
    // the key tiles visited first hold the diagonal blocks of the waves: those with keys of the workgroup's own blocks
    const int nslow = min(n_steps, (n_kt - (NB * jt) / 2 + 1) & ~1);
    if (n_steps > 0) load_bias(n_kt - 1);
    UA_PIPE_START(n_steps, UA_ISSUE);
    UA_PIPE_RANGE(0, nslow, n_steps, UA_ISSUE, UA_COMPUTE_SLOW);
    UA_PIPE_RANGE(nslow, n_steps, n_steps, UA_ISSUE, UA_COMPUTE_FAST);
  }
#undef UA_ISSUE
#undef UA_COMPUTE_FAST
#undef UA_COMPUTE_SLOW
  if (!live) return;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const float tot = allsum16(ls[i][v]);
      const float inv = 1.0f / tot;
      const int t = 32 * qb + 16 * i + 4 * g + v;
      if (t < L) {
#pragma unroll
        for (int n = 0; n < ND; ++n) {
          const int dd = 16 * n + col;
          if (dd < d) O[((long)zq * L + t) * d + dd] = cvt<T>(o[i][n][v] * inv);
        }
      }
      if (col == 0) {
        const float l2v = m[i][v] + __builtin_amdgcn_logf(tot);
        lse2[(long)zq * Lp + t] = (t < L) ? l2v : 0.f;
        if (t < L) lse[(long)zq * L + t] = l2v * kLn2;
      }
    }
  };
  sweep(n_blk - 1 - bx0);
  if (gridDim.x != n_blk && n_blk - 1 - bx0 != bx0) {     // (launches of few workgroups keep one block each)
    __syncthreads();       // the stages are free
    sweep(bx0);
  }
}

// The A operand [16 features 16n.. x 32 positions] of a "transposed" product out of the NATURAL tile [32 positions][D]
// (k-group-major, see Tile): two transposing reads, each turning a block of 4 positions x 16 features (8 bytes per lane:
// lane i of a 16-lane group supplies position i/4 of the block and features 4(i%4)..+3) into 4 positions of feature i
// per lane.  The k index follows as_operand16: elements 0-3 are positions 4G..4G+3, elements 4-7 positions 16+4G..+3
// (G = lane / 16).  The 64 lanes of one read touch 2 x 256 contiguous bytes; the LDS pipe takes 32 lanes at a time and
// the first 32 touch the first half of both pieces, i.e. half of the banks twice: 4.1 cycles of the pipe per read where
// 2.5 are possible.  A layout without that conflict was built and measured (feature tiles made of k-groups n and
// n + D/16, positions p and p ^ 8 exchanged in the upper k-groups on the source side of the copy; the exchange has to be
// the same for the four k-groups of a 16-byte operand read, which takes lane groups in pairs and costs 8 cycles
// instead of 4 when their patterns differ): k_bwd_keys2 was 1-2 % slower with it, so the LDS pipe is not what its
// waves wait for, and the plain layout stays.
template <class T>
__device__ __forceinline__ Frag<T> ld8_tr(const T* tile, int n, int lane) {
  static_assert(sizeof(T) == 2, "transposing LDS reads are 16-bit");
  const int i = lane & 15, G = lane >> 4;
  const char* p = reinterpret_cast<const char*>(tile) + (((2 * n + ((i & 3) >> 1)) * 32 + 4 * G + (i >> 2)) << 4) + 8 * (i & 1);
  Frag<T> f;
  reinterpret_cast<v4s16*>(&f)[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s16_t)p);
  reinterpret_cast<v4s16*>(&f)[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s16_t)(p + 256));
  return f;
}

// ---------------------------------------------------------------------------------------------
// Key-stationary backward (fused mode).  grid (n or ceil(n / 2), Zk) with n = Lp/128 key groups g (the second form: groups
// g and n - 1 - g one after the other, see the body); 8 waves; wave w owns keys 128g+16w..+15 and
// sweeps the 32-query blocks from the last one down to its own; one (query block, query group) per step.
// MR = more than one query group per kv head (the decay state of a query block then lives across steps).
// ---------------------------------------------------------------------------------------------
// CH: chunked operator (a.c a multiple of 64): the upstream gradient, delta and the normaliser depend on the key's chunk
// (z index zq*nch + chunk); the 128 keys of a workgroup lie in at most two chunks, whose dO tiles are both staged.
// TO (16-bit dtypes): leave the score gradient dS and the decay gradient dG of every visited tile, in operand precision,
// in a.dS_st / a.dG_st for k_bwd_queries3 (which then needs no suffix carries Dsuf).
template <class T, int D, int NST, bool MR, bool CH, bool TO>
__global__ void __launch_bounds__(512) k_bwd_keys2(BwdArgs<T> a) {
  using TN = Tile<T, 32, D>;
  using TT = Tile<T, D, 32>;
  constexpr int NK = D / 32, ND = D / 16;
  // merged operator with tile exchange: the bias comes from the fp16 tiles of k_carry2<BO> (a.Bt), one 1 KB tile per wave
  // and step after the stats row (the chunked operator keeps the carries C, and Dsuf for the recomputing query side)
  constexpr bool BI = TO && !CH;
  // With the tile exchange the operands of the three products that contract over the block's positions are read out of
  // the natural tiles with transposing LDS reads (ld8_tr), so the transposed copies are neither staged nor fetched
  constexpr bool TR = TO;
  constexpr int TILES = TR ? (CH ? 4 : 3) * TN::BYTES : (CH ? 4 : 3) * (TN::BYTES + TT::BYTES);
  // offsets of the second chunk's upstream tile (CH), natural and transposed
  constexpr int DO2 = TR ? 3 * TN::BYTES : 3 * TN::BYTES + 3 * TT::BYTES, DO2T = 4 * TN::BYTES + 3 * TT::BYTES;
  constexpr int SB = TILES + (CH ? 2048 : 1024) + (BI ? 8 * 1024 : 0);
  // tiles of a stage: Kt, Q, dO | (!TR) KT, QT, dOT | (CH) dO, dOT of the workgroup's second chunk
  // stats row of a stage: [lse2: 32f][delta: 32f][ldest: 32f][unused: 32f][forward carries of the 128 keys: 128f]
  // (CH) followed by [lse2: 32f][delta: 32f] of the second chunk
  UA_STAGES(SB);
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, col = lane & 15, g = lane >> 4;
  // grid y: (kv head, part).  The r query groups of a kv head are divided into a.key_parts parts; a workgroup sweeps
  // the groups of its part one after the other (MR: more than one, sharing the key-key part of a step) and its
  // key-side sums land in slice zo of dKrow / dVrow / dsrc_raw / dG_st (k_bwd_finish and k_bwd_queries3 add the parts
  // up).  More parts repeat the key-key part of a step but shorten the longest workgroup of the launch, which is
  // what bounds it when there are few kv heads.
  // A workgroup sweeps two key groups one after the other, kg and (number of key groups - 1 - kg): their sweeps add up to
  // the same length for every pair, so that the launch is a whole number of equal rounds and has half the workgroup
  // changes (a CU slot idles for about 16 us between the end of a workgroup and the start of its successor): 2.44 -> 2.36 ms at
  // b = 1, h = 32, L = 8192, d = 128.  The body is expanded once per key group: inside a loop (two pairs per workgroup, or
  // workgroups that draw their key groups from a queue) the same step is scheduled with nearly twice the LDS waits and the
  // kernel is slower than with a workgroup per key group.
  int bx0, zo;
  xcd_map(bx0, zo);
  const int n_kg = a.Lp / 128;
  auto sweep = [&](const int bx) __attribute__((always_inline)) {
  const int zk = zo / a.key_parts;
  const int Lp = a.Lp, L = a.L, nT16 = Lp / 16, R = MR ? a.R / a.key_parts : 1;
  const long zq0 = (long)zk * a.R + (zo % a.key_parts) * (a.R / a.key_parts);      // first query head of the part
  const int kg = bx, sb16 = 8 * kg + w, spos = 16 * sb16 + col;      // key group 0 sweeps the most query blocks: first
  const int nTr = (L + 31) / 32, first = 4 * kg;
  if (first >= nTr) return;                      // every key of this workgroup is padding
  // chunked operator: chunk of the workgroup's first key, whether the workgroup reaches into the next one, and which
  // of the two this wave's keys belong to
  const int nch = CH ? a.nch : 1;
  const int ch0 = CH ? min((128 * kg) / a.c, nch - 1) : 0;
  const bool two = CH && min((128 * kg + 127) / a.c, nch - 1) != ch0;
  const int csel = CH ? min((16 * sb16) / a.c, nch - 1) - ch0 : 0;
  const int cstart32 = CH ? ((ch0 + csel) * a.c) >> 5 : 0;      // first query block of this wave's chunk
  const float inv_c = CH ? 1.0f / (float)a.c : 0.f;
  // the blocks before the chunk are swept only when some upstream gradient there is non-zero (flag set by k_delta)
  const bool uniform_part = CH && !a.skip_masked && *a.masked_nz != 0;
  // query blocks beyond the reach of a key tile (see k_carry2) are not visited: the sweep starts at the farthest
  // block any of the 8 waves reaches, and a wave joins in at its own
  const int* reach_z = a.reach + zk * nT16 + 8 * kg;
  int top = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) top = max(top, reach_z[i]);
  top = min(top, nTr - 1);
  const int myreach = reach_z[w];
  const GroupMasks gm = group_masks(lane);
  Stager<TN, 8> stN;
  Stager<TT, 8> stT;
  stN.init(w, lane, D * (long)sizeof(T), 32);
  stT.init(w, lane, Lp * (long)sizeof(T), D);
  // Upstream-gradient tiles.  Normally the packed copy (tiles like those of K and Q).  Chunked operator with a.dO_rows:
  // the caller's own tensor, rows of D elements: lane l of copy instruction i fetches the 16 bytes that belong at LDS
  // unit 64 i + l = (k-group, position) from row `position`, so that the LDS image is the same (32 rows of 16 bytes
  // per instruction instead of 1 KB in one piece).
  const bool dO_in_place = CH && TR && a.dO_rows;
  const long dO_len = dO_in_place ? L : Lp;             // rows per (query head, chunk)
  Stager<TN, 8> stG = stN;
  if (dO_in_place) {
#pragma unroll
    for (int k = 0; k < Stager<TN, 8>::PER; ++k) {
      const int n = (w + k * 8) * 64 + lane;
      stG.off[k] = (n & 31) * (D * (int)sizeof(T)) + (n >> 5) * 16;
    }
  }

  Frag<T> kp[NK], vf[NK];
  {
#pragma unroll
    for (int q = 0; q < NK; ++q) {
      const long ro = nat_off<D>(zk, Lp, spos, 32 * q + 8 * g);
      kp[q] = ld8(a.Kp + ro);
      vf[q] = ld8(a.Vp + ro);
    }
  }
  const float la = a.lsrc[(long)zk * Lp + spos];
  f32x4 dVt[ND], dKt[ND];
#pragma unroll
  for (int n = 0; n < ND; ++n) { dVt[n] = (f32x4){0, 0, 0, 0}; dKt[n] = (f32x4){0, 0, 0, 0}; }
  float dsrc_acc = 0.f, dcar = 0.f;
  // 16-bit operands: the reverse running sum of dS over the block's queries runs on the matrix core (scan32_mma); dcar4
  // replaces dcar, and with several query groups (MR) the groups' sums accumulate in dB through the same products
  constexpr bool MS = sizeof(T) == 2;
  ScanOps sc_ops;
  f32x4 dcar4 = {0, 0, 0, 0}, dtot4 = {0, 0, 0, 0};
  if constexpr (MS) sc_ops = scan_operands<true>(lane);
  f32x4 aff_s[2], bias_s[2], gk_s[2], dB_s[2];     // state of the current query block (used when MR); gk = relu(G)
  const T* Kz = a.Kp + (long)zk * Lp * D;
  const T* KTz = a.KT + (long)zk * D * Lp;
  const float* ldz = a.ldest + (long)zk * Lp;
  const float* Cz = a.C + (long)zk * nT16 * Lp + 128 * kg;
  float* Dz = a.Dsuf + (long)zk * nT16 * Lp + spos;
  // where this lane's four values of a (16 keys, 16 queries) tile go inside the 1 KB tile of its 32-key half
  static_assert(!TO || sizeof(T) == 2, "tiles are exchanged in 16-bit operand precision");
  // this lane's 16 bytes of the wave's bias tile of query block 0
  const char* bt_src = reinterpret_cast<const char*>(a.Bt) + (((long)zk * tri_tiles(Lp >> 5) + sb16) << 10) + 16 * lane;
  const long st_head = grp_tiles(Lp >> 5) << 10;                   // bytes of gradient tiles per head
  const long st_lane = StageT<bf16>::addr(perm32(16 * (sb16 & 1) + col), 8 * g);

#define UA_ISSUE(s, base)                                                                   \
  {                                                                                         \
    const int tb_ = top - (s) / R;                                                          \
    const long zq_ = zq0 + (MR ? (s) % R : 0);                                              \
    const long qo_ = (zq_ * Lp + 32 * tb_) * D;   /* tile base, natural and transposed */      \
    const long zg_ = zq_ * nch + ch0;             /* z index of dO, delta, lse2 */             \
    const long go_ = (zg_ * dO_len + 32 * tb_) * D;                                         \
    stN.issue((base), Kz + (long)(32 * tb_) * D, w);                                        \
    stN.issue((base) + TN::BYTES, a.Qp + qo_, w);                                           \
    stG.issue((base) + 2 * TN::BYTES, a.dOp + go_, w);                                      \
    if (!TR) {                                                                              \
      stT.issue((base) + 3 * TN::BYTES, KTz + (long)(32 * tb_) * D, w);                     \
      stT.issue((base) + 3 * TN::BYTES + TT::BYTES, a.QT + qo_, w);                         \
      stT.issue((base) + 3 * TN::BYTES + 2 * TT::BYTES, a.dOT + go_, w);                    \
    }                                                                                       \
    if (w == 0) {                                                                           \
      const float* src_;                                                                    \
      if (lane < 8) src_ = a.lse2 + zg_ * Lp + 32 * tb_ + 4 * lane;                         \
      else if (lane < 16) src_ = a.delta + zg_ * Lp + 32 * tb_ + 4 * (lane - 8);            \
      else if (lane < 32) src_ = ldz + 32 * tb_ + 4 * (lane & 7);                           \
      else src_ = BI ? ldz + 32 * tb_ + 4 * (lane & 7)   /* no carries with bias tiles */      \
                     : Cz + (long)(2 * tb_) * Lp + 4 * (lane - 32);                         \
      issue_row((base) + TILES, src_);                                                      \
    }                                                                                       \
    if (BI) issue_row_nt((base) + TILES + 1024 + w * 1024, bt_src + (tri_bias_row(tb_) << 10)); \
    if (CH && two) {                                                                        \
      stG.issue((base) + DO2, a.dOp + go_ + dO_len * D, w);                                 \
      if (!TR) stT.issue((base) + DO2T, a.dOT + go_ + (long)Lp * D, w);                     \
      if (w == 1) {                                                                         \
        const float* src_ = ((lane & 8) ? a.delta : a.lse2) + (zg_ + 1) * Lp + 32 * tb_ + 4 * (lane & 7); \
        issue_row((base) + TILES + 1024, src_);                                             \
      }                                                                                     \
    }                                                                                       \
  }
#define UA_COMPUTE_FAST(s, base)                                                            \
  {                                                                                         \
    if (top - (s) / R <= myreach) bwd_step((s), (base), FalseC(), false);                   \
  }
#define UA_COMPUTE_SLOW(s, base)                                                            \
  {                                                                                         \
    const int tb_ = top - (s) / R;                                                          \
    if (tb_ >= (sb16 >> 1)) {                                                               \
      if (tb_ <= myreach) bwd_step((s), (base), TrueC(), tb_ == (sb16 >> 1));               \
    } else if (CH && uniform_part && tb_ < cstart32) {                                      \
      uniform_step((s), (base));                                                            \
    }                                                                                       \
  }
  // Chunked operator, query block entirely before this wave's chunk: the reference fills the bias of such a
  // (key, query) pair with -1e12, which swamps the score, so the softmax over the chunk's keys is uniform
  // (universal_attention_autograd.py:27-33) while the gradient still flows through the score:
  //   P = 1/c,  dS = (dP - delta) / c,  no decay part.
  auto uniform_step = [&] __device__ (int s, const char* base) __attribute__((always_inline)) {
    const T* sdO = reinterpret_cast<const T*>(base + (csel ? DO2 : 2 * TN::BYTES));
    const T* sQT = reinterpret_cast<const T*>(base + 3 * TN::BYTES + TT::BYTES);
    const T* sdOT = reinterpret_cast<const T*>(base + (csel ? DO2T : 3 * TN::BYTES + 2 * TT::BYTES));
    const T* sQ = reinterpret_cast<const T*>(base + TN::BYTES);
    const float* qstats = reinterpret_cast<const float*>(base + TILES) + (csel ? 256 : 0);
    f32x4 P[2], dS[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      f32x4 dP = {0, 0, 0, 0};
#pragma unroll
      for (int q = 0; q < NK; ++q) mma16(dP, ld8(sdO + TN::at(i, col, q, g)), vf[q]);
      const f32x4 dlt = load_t4(qstats + 32 + 16 * i, g);
#pragma unroll
      for (int v = 0; v < 4; ++v) { P[i][v] = inv_c; dS[i][v] = inv_c * (dP[v] - dlt[v]); }
    }
    const Frag<T> bp = as_operand16<T>(P[0], P[1]), bs = as_operand16<T>(dS[0], dS[1]);
#pragma unroll
    for (int n = 0; n < ND; ++n) {
      if constexpr (TR) mma16(dVt[n], ld8_tr<T>(sdO, n, lane), bp);
      else mma16(dVt[n], ld8(sdOT + TT::at(n, col, 0, g)), bp);
    }
#pragma unroll
    for (int n = 0; n < ND; ++n) {
      if constexpr (TR) mma16(dKt[n], ld8_tr<T>(sQ, n, lane), bs);
      else mma16(dKt[n], ld8(sQT + TT::at(n, col, 0, g)), bs);
    }
  };
  // MASKED: the step may be the query block that holds this wave's own keys (run-time flag diag)
  auto bwd_step = [&] __device__ (int s, const char* base, auto masked_c, const bool diag) {
    constexpr bool MASKED = decltype(masked_c)::value;
    const int tb = top - s / R, r = s % R;
    const T* sKt = reinterpret_cast<const T*>(base);
    const T* sQ = reinterpret_cast<const T*>(base + TN::BYTES);
    const T* sdO = reinterpret_cast<const T*>(base + (csel ? DO2 : 2 * TN::BYTES));
    const T* sKT = reinterpret_cast<const T*>(base + 3 * TN::BYTES);
    const T* sQT = reinterpret_cast<const T*>(base + 3 * TN::BYTES + TT::BYTES);
    const T* sdOT = reinterpret_cast<const T*>(base + (csel ? DO2T : 3 * TN::BYTES + 2 * TT::BYTES));
    const float* stats = reinterpret_cast<const float*>(base + TILES);
    const float* qstats = stats + (csel ? 256 : 0);       // lse2 / delta of this wave's chunk
    f32x4 aff_l[2], bias_l[2], gk_l[2], dB_l[2];
    f32x4 (&aff)[2] = MR ? aff_s : aff_l;
    f32x4 (&bias)[2] = MR ? bias_s : bias_l;
    f32x4 (&gk)[2] = MR ? gk_s : gk_l;
    f32x4 (&dB)[2] = MR ? dB_s : dB_l;
    const int tl0 = 32 * tb + 4 * g - spos;        // query position minus key position for (tile 0, v = 0)
    if (!MR || r == 0) {
      typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
      f16x8 hb;
      if constexpr (BI) hb = *reinterpret_cast<const f16x8*>(base + TILES + 1024 + w * 1024 + 16 * lane);
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        f32x4 acc = {0, 0, 0, 0};
#pragma unroll
        for (int q = 0; q < NK; ++q) mma16(acc, ld8(sKt + TN::at(i, col, q, g)), kp[q]);
        const f32x4 lab = load_t4(stats + 64 + 16 * i, g);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          gk[i][v] = fmaxf(acc[v], 0.f);
          aff[i][v] = affinity(__builtin_amdgcn_logf(gk[i][v]), lab[v] + la);
          if constexpr (BI) {
            bias[i][v] = (float)hb[4 * i + v];
          } else {
            const float l2 = log2_one_minus(aff[i][v]);
            bias[i][v] = (MASKED && diag && tl0 + 16 * i + v <= 0) ? 0.f : l2;
          }
          if (MR) dB[i][v] = 0.f;
        }
      }
      if constexpr (!BI) {
        const float cin = stats[128 + 16 * w + col];
        prefix32(bias[0], bias[1], gm);
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int v = 0; v < 4; ++v) bias[i][v] += cin;
      }
    }
    {
      f32x4 P[2], dS[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        f32x4 sc = {0, 0, 0, 0}, dP = {0, 0, 0, 0};
#pragma unroll
        for (int q = 0; q < NK; ++q) mma16(sc, ld8(sQ + TN::at(i, col, q, g)), kp[q]);
#pragma unroll
        for (int q = 0; q < NK; ++q) mma16(dP, ld8(sdO + TN::at(i, col, q, g)), vf[q]);
        const f32x4 l2t = load_t4(qstats + 16 * i, g), dlt = load_t4(qstats + 32 + 16 * i, g);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[v], kLog2e, bias[i][v]) - l2t[v]);
          if (MASKED) p = (diag && tl0 + 16 * i + v < 0) ? 0.f : p;
          P[i][v] = p;
          dS[i][v] = p * (dP[v] - dlt[v]);
        }
      }
      const Frag<T> bp = as_operand16<T>(P[0], P[1]), bs = as_operand16<T>(dS[0], dS[1]);
      if constexpr (TO) {     // the two halves of the operand are the two query tiles of the block
        // query tiles 2 tb and 2 tb + 1: their rows start tb + 1 tiles apart
        char* p = reinterpret_cast<char*>(a.dS_st) + (zq0 + r) * st_head + (grp_tile(2 * tb, sb16 >> 1) << 10) + st_lane;
        __builtin_nontemporal_store(reinterpret_cast<const u32x2*>(&bs)[0], reinterpret_cast<u32x2*>(p));
        __builtin_nontemporal_store(reinterpret_cast<const u32x2*>(&bs)[1], reinterpret_cast<u32x2*>(p + 1024));
      }
      // The two waves of a SIMD are rarely in the same phase of a step; the one that reaches its long run of independent
      // matrix instructions goes first, and the other one's vector work fills the gaps (k_bwd_keys2<TO>: -6 %; raising
      // the priority around the short dependent chains of the input products as well gives the gain back).
      __builtin_amdgcn_s_setprio(1);
#pragma unroll
      for (int n = 0; n < ND; ++n) {
        if constexpr (TR) mma16(dVt[n], ld8_tr<T>(sdO, n, lane), bp);
        else mma16(dVt[n], ld8(sdOT + TT::at(n, col, 0, g)), bp);
      }
#pragma unroll
      for (int n = 0; n < ND; ++n) {
        if constexpr (TR) mma16(dKt[n], ld8_tr<T>(sQ, n, lane), bs);
        else mma16(dKt[n], ld8(sQT + TT::at(n, col, 0, g)), bs);
      }
      if constexpr (MS) {
        // dB (+)= reverse running sums of this group's dS; the block totals of the groups add up in dtot4
        if (!MR || r == 0) { dB[0] = dcar4; dB[1] = dcar4; if (MR) dtot4 = dcar4; }
        mma16(dB[0], sc_ops.tri[0], bs);
        mma16(dB[1], sc_ops.tri[1], bs);
        mma16(MR ? dtot4 : dcar4, sc_ops.ones, bs);
      }
      __builtin_amdgcn_s_setprio(0);
      if constexpr (!MS) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int v = 0; v < 4; ++v) dB[i][v] = MR ? dB[i][v] + dS[i][v] : dS[i][v];
      }
    }
    if (!MR || r == R - 1) {
      float t1 = 0.f, tot = 0.f;
      if constexpr (MS) {
        // suffix carries for the recomputing query side: before the block's second tile, before its first
        if (!BI && g == 0) {
          Dz[(long)(2 * tb + 1) * Lp] = dcar;
          Dz[(long)(2 * tb) * Lp] = dB[1][0];
        }
        if (MR) dcar4 = dtot4;
      } else {
        tot = suffix32(dB[0], dB[1], gm, t1);
        if (!BI && g == 0) {
          Dz[(long)(2 * tb + 1) * Lp] = dcar;
          Dz[(long)(2 * tb) * Lp] = dcar + t1;
        }
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          float dl = MS ? dB[i][v] : dB[i][v] + dcar;
          if (MASKED) dl = (diag && tl0 + 16 * i + v <= 0) ? 0.f : dl;
          dB[i][v] = decay_grad(dl, aff[i][v], gk[i][v]);
          dsrc_acc = __builtin_fmaf(dB[i][v], gk[i][v], dsrc_acc);
        }
      }
      if constexpr (MS) dcar = dcar4[0];
      else dcar += tot;
      const Frag<T> b = as_operand16<T>(dB[0], dB[1]);
      if constexpr (TO) {
        char* p = reinterpret_cast<char*>(a.dG_st) + (long)zo * st_head + (grp_tile(2 * tb, sb16 >> 1) << 10) + st_lane;
        __builtin_nontemporal_store(reinterpret_cast<const u32x2*>(&b)[0], reinterpret_cast<u32x2*>(p));
        __builtin_nontemporal_store(reinterpret_cast<const u32x2*>(&b)[1], reinterpret_cast<u32x2*>(p + 1024));
      }
      __builtin_amdgcn_s_setprio(1);
#pragma unroll
      for (int n = 0; n < ND; ++n) {
        if constexpr (TR) mma16(dKt[n], ld8_tr<T>(sKt, n, lane), b);
        else mma16(dKt[n], ld8(sKT + TT::at(n, col, 0, g)), b);
      }
      __builtin_amdgcn_s_setprio(0);
    }
  };
  {
    // the last four query blocks of the sweep hold the diagonal blocks of the eight waves
    const int nblk = top + 1 - first, nfast = ((nblk > 4 ? nblk - 4 : 0) * R) & ~1;
    const int total = (uniform_part ? top + 1 : nblk) * R;
    UA_PIPE_START(total, UA_ISSUE);
    UA_PIPE_RANGE(0, nfast, total, UA_ISSUE, UA_COMPUTE_FAST);
    UA_PIPE_RANGE(nfast, total, total, UA_ISSUE, UA_COMPUTE_SLOW);
  }
#undef UA_ISSUE
#undef UA_COMPUTE_FAST
#undef UA_COMPUTE_SLOW
  // epilogue
  {
    float b, af, tot;
    group_scan(dsrc_acc, gm, b, af, tot);
    if (TO && !MR && a.direct) {      // straight into the caller's tensor: dsrc = sum dA A / (3 src)
      if (g == 0 && spos < L) a.dsrc_out[(long)zo * L + spos] = cvt<T>(1.5f * tot / (3.0f * (float)a.src_in[(long)zo * L + spos]));
    } else if (g == 0) {
      a.dsrc_raw[(long)zo * Lp + spos] = 1.5f * tot;    // sum dA A = 3/2 sum dG G
    }
  }
  const bool direct = TO && !MR && a.direct;
#pragma unroll
  for (int n = 0; n < ND; ++n) {
    const long o = ((long)zo * Lp + spos) * D + 16 * n + 4 * g;
    *reinterpret_cast<float4*>(a.dKrow + o) = make_float4(dKt[n][0], dKt[n][1], dKt[n][2], dKt[n][3]);
    if (!direct) {
      *reinterpret_cast<float4*>(a.dVrow + o) = make_float4(dVt[n][0], dVt[n][1], dVt[n][2], dVt[n][3]);
    } else if (spos < L) {
      T* dst = a.dv_out + ((long)zo * L + spos) * a.d_out + 16 * n + 4 * g;
#pragma unroll
      for (int v = 0; v < 4; ++v)
        if (16 * n + 4 * g + v < a.d_out) dst[v] = cvt<T>(dVt[n][v]);
    }
  }
  };
  sweep(bx0);
  if (gridDim.x != n_kg && n_kg - 1 - bx0 != bx0) {       // (launches of few workgroups keep one key group each)
    __syncthreads();       // the stages are free
    sweep(n_kg - 1 - bx0);
  }
}

// ---------------------------------------------------------------------------------------------
// Query-stationary backward (fused mode): dQ and the column side of dK, no atomics.
// grid (Lp/128, Zk); 8 waves; wave w owns queries 16*(8*jt+w)..+15; 64 keys per step.
//   dQ[t,:] += sum_s dS[s,t] k_s        dkcol[u,:] += sum_s dg[s,u] k_s
// dS^T and dg^T pass through a wave-private LDS tile to become A operands.  With r query groups the sweep is
// repeated per group; dg is linear in dBias, so the groups' contributions to dkcol add up (the cross-tile
// suffix carry is added in the first group only).
// ---------------------------------------------------------------------------------------------
// CH: chunked operator (a.c a multiple of 64): the upstream gradient, delta and the normaliser are those of the chunk
// the step's 64 keys belong to (z index zq*nch + chunk) and are reloaded when the chunk changes.
template <class T, int D, int NST, bool CH>
__global__ void __launch_bounds__(512) k_bwd_queries2(BwdArgs<T> a, T* __restrict__ dq, int d) {
  using TN = Tile<T, 32, D>;
  using TT = Tile<T, D, 32>;
  constexpr int NK = D / 32, ND = D / 16;
  using ST = StageT<T>;
  constexpr int TILES = 4 * TN::BYTES + 2 * TT::BYTES, SB = TILES + 8 * 1024;   // + per wave [C: 64f][lsrc: 64f][Dsuf: 64f]
  UA_STAGES(SB);
  __shared__ __attribute__((aligned(256))) char sXbuf[8 * 2 * ST::BYTES];
  // Chunked operator: the stationary upstream rows of the NEXT chunk are copied asynchronously into a wave-private
  // LDS region one step ahead (where the 160 KB of LDS allow it), so that entering a chunk costs an LDS read instead
  // of a round trip to memory; lse2 and delta of the step's chunk travel in the stats row.
  constexpr int GBYTES = 16 * D * (int)sizeof(T), GH = (int)sizeof(Frag<T>) / 16;
  constexpr bool PRE = CH && (NST == 2 ? 2 * SB : SB + 1024) + 8 * 2 * ST::BYTES + 8 * GBYTES <= 163840;
  __shared__ __attribute__((aligned(1024))) char sGbuf[PRE ? 8 * GBYTES : 1024];
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, col = lane & 15, g = lane >> 4;
  // grid y: kv heads (the query groups of a head are then swept one after the other), or, when gridDim.y is the number
  // of query heads, one (kv head, query group) per workgroup: more, smaller workgroups; the column-side key gradient
  // is then written per query head and added up by k_bwd_finish
  int bx, zy;
  xcd_map(bx, zy);
  const int Lp = a.Lp, L = a.L, nT16 = Lp / 16, R = a.R;
  const bool split_r = a.split_r != 0;
  const int zk = split_r ? zy / R : zy, r_begin = split_r ? zy % R : 0, r_end = split_r ? r_begin + 1 : R;
  const int jt = gridDim.x - 1 - bx, tq = 8 * jt + w;
  char* sX = sXbuf + w * 2 * ST::BYTES;      // [dS of a 32-key half][dg of that half]
  const GroupMasks gm = group_masks(lane);
  Stager<TN, 8> stN;
  Stager<TT, 8> stT;
  stN.init(w, lane, D * (long)sizeof(T), 32);
  stT.init(w, lane, Lp * (long)sizeof(T), D);

  Frag<T> kt[NK];
  {
#pragma unroll
    for (int q = 0; q < NK; ++q) kt[q] = ld8(a.Kp + nat_off<D>(zk, Lp, 16 * tq + col, 32 * q + 8 * g));
  }
  const f32x4 lb = load_t4(a.ldest + (long)zk * Lp + 16 * tq, g);
  f32x4 dKc[ND];
#pragma unroll
  for (int n = 0; n < ND; ++n) dKc[n] = (f32x4){0, 0, 0, 0};
  const T* Kz = a.Kp + (long)zk * Lp * D;
  const T* Vz = a.Vp + (long)zk * Lp * D;
  const T* KTz = a.KT + (long)zk * D * Lp;
  const int n_kt = 2 * jt + 2;
  // key tiles out of reach of this workgroup's first query block are not visited (see k_carry2); inside the range
  // a tile that does not reach this wave's block gets a carry of -1e30, which zeroes its dS and dG
  const int tbq = tq >> 1;
  const int kt_min = (a.minkey[zk * (nT16 >> 1) + 4 * jt] >> 2) & ~1;
  // per-wave stats row of a step: [C row: 64f][lsrc: 64f][Dsuf row: 64f][reach of the 4 key tiles: 4 ints] and, with
  // the chunked operator, [lse2: 16f][delta: 16f] of this wave's queries in the step's chunk at floats 208 and 224; source of
  // each lane's 16 bytes as base + step * stride (in 4-byte units)
  const float* row_base;
  int row_step = 64;
  if (lane < 16) row_base = a.C + ((long)zk * nT16 + tq) * Lp + 4 * lane;
  else if (lane < 32) row_base = a.lsrc + (long)zk * Lp + 4 * (lane - 16);
  else if (lane < 48) row_base = a.Dsuf + ((long)zk * nT16 + tq) * Lp + 4 * (lane - 32);
  else { row_base = reinterpret_cast<const float*>(a.reach + zk * nT16); row_step = 4; }
  // column of key (16*(j&1) + col) inside its 32-key group of the transposed key tile
  const int pc0 = perm32(col), pc1 = perm32(16 + col);
  // chunked operator: key tiles [uk0, uk1) belong to chunks after the workgroup's first query (uk0_w: after this
  // wave's queries); they are swept only when some upstream gradient there is non-zero (flag set by k_delta)
  const float inv_c = CH ? 1.0f / (float)a.c : 0.f;
  const bool uniform_part = CH && !a.skip_masked && *a.masked_nz != 0;
  if (CH && a.dS_st && !uniform_part) return;      // k_bwd_queries3 does the query side from the tiles
  const int uk0 = CH ? ((min((128 * jt) / a.c, a.nch - 1) + 1) * a.c) >> 6 : 0;
  const int uk0_w = CH ? ((min((16 * tq) / a.c, a.nch - 1) + 1) * a.c) >> 6 : 0;
  const int uk1 = uniform_part ? max(uk0, L >> 6) : uk0;

  for (int r = r_begin; r < r_end; ++r) {
    const long zq = (long)zk * R + r;
    Frag<T> qt[NK], gt[NK];
    f32x4 l2t, dlt;
    int cur_chunk = -1;      // chunk whose upstream rows gt holds
    int in_lds = -1;         // chunk whose upstream rows are (being) copied into this wave's LDS region
    char* sG = sGbuf + (PRE ? w * GBYTES : 0);
    // upstream operands of chunk ch (chunked operator) or of the merged operator (ch = 0, nch = 1), straight from memory
    auto load_upstream = [&] __device__ (int ch) __attribute__((always_inline)) {
      const long zg = CH ? zq * a.nch + ch : zq;
#pragma unroll
      for (int q = 0; q < NK; ++q) gt[q] = ld8(a.dOp + nat_off<D>(zg, Lp, 16 * tq + col, 32 * q + 8 * g));
      if (!PRE) {
        l2t = load_t4(a.lse2 + zg * Lp + 16 * tq, g);
        dlt = load_t4(a.delta + zg * Lp + 16 * tq, g);
      }
      cur_chunk = ch;
    };
    // PRE: every lane copies the 16-byte pieces of its own operand fragments; the copy is complete after the next
    // step's wait_async_loads()
    auto prefetch_upstream = [&] __device__ (int ch) __attribute__((always_inline)) {
      if (ch == in_lds) return;
      const long zg = zq * a.nch + ch;
#pragma unroll
      for (int q = 0; q < NK; ++q)
#pragma unroll
        for (int hh = 0; hh < GH; ++hh)
          issue_row(sG + (q * GH + hh) * 1024,
                    reinterpret_cast<const char*>(a.dOp + nat_off<D>(zg, Lp, 16 * tq + col, 32 * q + 8 * g)) + 16 * hh);
      in_lds = ch;
    };
    // PRE: fragments of chunk ch out of the LDS region (which must hold them, completely)
    auto take_upstream = [&] __device__ (int ch) __attribute__((always_inline)) {
      if (ch == cur_chunk) return;
#pragma unroll
      for (int q = 0; q < NK; ++q)
#pragma unroll
        for (int hh = 0; hh < GH; ++hh)
          reinterpret_cast<uint4*>(&gt[q])[hh] = *reinterpret_cast<const uint4*>(sG + (q * GH + hh) * 1024 + 16 * lane);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // before the region may be refilled
      cur_chunk = ch;
    };
    {
#pragma unroll
      for (int q = 0; q < NK; ++q) qt[q] = ld8(a.Qp + nat_off<D>(zq, Lp, 16 * tq + col, 32 * q + 8 * g));
    }
    if (!CH) load_upstream(0);
    f32x4 dQ[ND];
#pragma unroll
    for (int n = 0; n < ND; ++n) dQ[n] = (f32x4){0, 0, 0, 0};

#define UA_ISSUE(s, base)                                                                   \
  {                                                                                         \
    const int k0_ = 64 * ((s) < n_kt ? (s) : (s) - n_kt + uk0);                             \
    const int ch_ = CH ? min(k0_ / a.c, a.nch - 1) : 0;                                     \
    if (PRE && in_lds >= 0) take_upstream(in_lds);   /* rows of the step computed next */    \
    stN.issue((base), Kz + (long)k0_ * D, w);                                               \
    stN.issue((base) + TN::BYTES, Kz + (long)(k0_ + 32) * D, w);                            \
    stN.issue((base) + 2 * TN::BYTES, Vz + (long)k0_ * D, w);                               \
    stN.issue((base) + 3 * TN::BYTES, Vz + (long)(k0_ + 32) * D, w);                        \
    stT.issue((base) + 4 * TN::BYTES, KTz + (long)k0_ * D, w);                              \
    stT.issue((base) + 4 * TN::BYTES + TT::BYTES, KTz + (long)(k0_ + 32) * D, w);           \
    {                                                                                       \
      const float* src_ = row_base + (long)(k0_ >> 6) * row_step;                           \
      if (PRE && lane >= 52 && lane < 60)                                                   \
        src_ = (lane < 56 ? a.lse2 : a.delta) + (zq * a.nch + ch_) * Lp + 16 * tq + 4 * (lane & 3); \
      issue_row((base) + TILES + w * 1024, src_);                                           \
    }                                                                                       \
    if (PRE) prefetch_upstream(ch_);                                                        \
  }
#define UA_COMPUTE_FAST(s, base) bq_step((s), (base), FalseC())
#define UA_COMPUTE_SLOW(s, base)                                                            \
  {                                                                                         \
    if ((s) < n_kt) bq_step((s), (base), TrueC());                                          \
    else if (CH && (s) - n_kt + uk0 >= uk0_w) uniform_step((s) - n_kt + uk0, (base));       \
  }
    // Chunked operator, key tile of a chunk after this wave's queries: uniform softmax over the chunk's keys,
    // dS = (dP - delta) / c (see k_bwd_keys2), no decay part.
    auto uniform_step = [&] __device__ (int kti, const char* base) __attribute__((always_inline)) {
      const int ch = min((64 * kti) / a.c, a.nch - 1);
      if (PRE) {
        take_upstream(ch);
        dlt = load_t4(reinterpret_cast<const float*>(base + TILES + w * 1024) + 224, g);
      } else if (ch != cur_chunk) {
        load_upstream(ch);
      }
#pragma unroll
      for (int kq = 0; kq < 2; ++kq) {
        const T* sV = reinterpret_cast<const T*>(base + (2 + kq) * TN::BYTES);
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
          f32x4 dP = {0, 0, 0, 0}, dS;
#pragma unroll
          for (int q = 0; q < NK; ++q) mma16(dP, gt[q], ld8(sV + TN::at(jj, col, q, g)));
#pragma unroll
          for (int v = 0; v < 4; ++v) dS[v] = inv_c * (dP[v] - dlt[v]);
          ST::put(sX, jj ? pc1 : pc0, g, dS);
        }
        const T* sKT = reinterpret_cast<const T*>(base + 4 * TN::BYTES + kq * TT::BYTES);
        const Frag<T> as = ST::get(sX, lane);
#pragma unroll
        for (int n = 0; n < ND; ++n) mma16(dQ[n], as, ld8(sKT + TT::at(n, col, 0, g)));
      }
    };
    auto bq_step = [&] __device__ (int kti, const char* base, auto masked_c) {
      constexpr bool MASKED = decltype(masked_c)::value;
      const float* stats = reinterpret_cast<const float*>(base + TILES + w * 1024);
      if constexpr (CH) {
        const int ch = min((64 * kti) / a.c, a.nch - 1);
        if (PRE) {
          take_upstream(ch);
          l2t = load_t4(stats + 208, g);
          dlt = load_t4(stats + 224, g);
        } else if (ch != cur_chunk) {
          load_upstream(ch);
        }
      }
      // the 64 keys of the step are handled as two halves of 32 (= one contraction step of the column products);
#pragma unroll
      for (int kq = 0; kq < 2; ++kq) {
        if (MASKED && 4 * kti + 2 * kq > tq) continue;     // wave-uniform: the whole half lies after this wave's queries
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
          const int j = 2 * kq + jj, sbk = 4 * kti + j;
          const bool live = !MASKED || sbk <= tq;
          const bool diag = MASKED && (sbk == tq);
          f32x4 dS = {0, 0, 0, 0}, dg = {0, 0, 0, 0};
          if (live) {
            const T* sK = reinterpret_cast<const T*>(base + kq * TN::BYTES);
            const T* sV = reinterpret_cast<const T*>(base + (2 + kq) * TN::BYTES);
            const bool in_reach = reinterpret_cast<const int*>(stats)[192 + j] >= tbq;
            const float cin = in_reach ? stats[16 * j + col] : -1.0e30f;
            const float la = stats[64 + 16 * j + col];
            const float din = (r == 0 && in_reach) ? stats[128 + 16 * j + col] : 0.f;
            f32x4 acc = {0, 0, 0, 0}, sc = {0, 0, 0, 0}, dP = {0, 0, 0, 0};
#pragma unroll
            for (int q = 0; q < NK; ++q) {
              const int o = TN::at(jj, col, q, g);
              const Frag<T> kb = ld8(sK + o);
              mma16(acc, kt[q], kb);
              mma16(sc, qt[q], kb);
              mma16(dP, gt[q], ld8(sV + o));
            }
            f32x4 x, gk, aff;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
              gk[v] = fmaxf(acc[v], 0.f);
              aff[v] = affinity(__builtin_amdgcn_logf(gk[v]), la + lb[v]);
              const float l2 = log2_one_minus(aff[v]);
              x[v] = (MASKED && diag && 4 * g + v <= col) ? 0.f : l2;
            }
            x[1] += x[0]; x[2] += x[1]; x[3] += x[2];
            float before, after, tot;
            group_scan(x[3], gm, before, after, tot);
            before += cin;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
              float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[v], kLog2e, x[v] + before) - l2t[v]);
              if (MASKED) p = (diag && 4 * g + v < col) ? 0.f : p;
              dS[v] = p * (dP[v] - dlt[v]);
            }
            // decay part: suffix over this wave's 16 queries + carry of the later tiles
            f32x4 y = dS;
            y[2] += y[3]; y[1] += y[2]; y[0] += y[1];
            group_scan(y[0], gm, before, after, tot);
            after += din;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
              float dl = y[v] + after;
              if (MASKED) dl = (diag && 4 * g + v <= col) ? 0.f : dl;
              dg[v] = decay_grad(dl, aff[v], gk[v]);
            }
          }
          ST::put(sX, jj ? pc1 : pc0, g, dS);
          ST::put(sX + ST::BYTES, jj ? pc1 : pc0, g, dg);
        }
        // dQ += dS^T K,  dkcol += dg^T K   (contraction over the 32 keys of the half)
        const T* sKT = reinterpret_cast<const T*>(base + 4 * TN::BYTES + kq * TT::BYTES);
        const Frag<T> as = ST::get(sX, lane), ag = ST::get(sX + ST::BYTES, lane);
#pragma unroll
        for (int n = 0; n < ND; ++n) {
          const Frag<T> kb = ld8(sKT + TT::at(n, col, 0, g));
          mma16(dQ[n], as, kb);
          mma16(dKc[n], ag, kb);
        }
      }
    };
    {
      // the last two key tiles hold the diagonal blocks of the eight waves
      const int nfast = max(n_kt - 2, kt_min), n_all = n_kt + uk1 - uk0;
      UA_PIPE_START_AT(kt_min, n_all, UA_ISSUE);
      UA_PIPE_RANGE(kt_min, nfast, n_all, UA_ISSUE, UA_COMPUTE_FAST);
      UA_PIPE_RANGE(nfast, n_all, n_all, UA_ISSUE, UA_COMPUTE_SLOW);
    }
#undef UA_ISSUE
#undef UA_COMPUTE_FAST
#undef UA_COMPUTE_SLOW
    __syncthreads();   // the next group's prologue refills stage 0
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int t = 16 * tq + 4 * g + v;
      if (t < L) {
#pragma unroll
        for (int n = 0; n < ND; ++n) {
          const int dd = 16 * n + col;
          if (dd < d) dq[(zq * L + t) * d + dd] = cvt<T>(dQ[n][v]);
        }
      }
    }
  }
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const int t = 16 * tq + 4 * g + v;
#pragma unroll
    for (int n = 0; n < ND; ++n) a.dKdacc[((long)zy * Lp + t) * D + 16 * n + col] = dKc[n][v];
  }
}

// ---------------------------------------------------------------------------------------------
// Query side of the backward from the tiles k_bwd_keys2 left (16-bit dtypes, fused mode): pure matrix work.
//   dQ[t,:] = sum_s dS[s,t] k_s        dkcol[u,:] = sum_s dG[s,u] k_s
// grid (Lp/128, Zq); 8 waves; wave w owns queries 16*(8*jt+w)..+15 and streams its own row of 1 KB tiles (HV
// 32-key halves of dS and of dG per step of 32 HV keys) straight into LDS, where they are read transposed as A
// operands; the transposed key tiles are shared by the workgroup.  dG belongs to the kv head: with r query groups
// per head swept together (a part, see k_bwd_keys2: Rl groups share one dG), group r accumulates the feature tiles
// n = r % Rl, r % Rl + Rl, ... of dkcol (its slice of dKdacc holds zeros elsewhere; k_bwd_finish adds the slices).
// ---------------------------------------------------------------------------------------------
// HV: 32-key halves per step.  With one half a stage is 25 KB and two workgroups share a CU (the kernel only moves
// bytes: more of them in flight, and one workgroup's prologue and epilogue under the other's stream).
template <class T, int D, int NST, int HV>
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(HV == 1 ? 4 : 2, HV == 1 ? 4 : 2)))
k_bwd_queries3(BwdArgs<T> a, T* __restrict__ dq, int d) {
  static_assert(sizeof(T) == 2, "tiles are exchanged in 16-bit operand precision");
  static_assert(HV == 1 || HV == 2, "one or two key halves per step");
  using TT = Tile<T, D, 32>;
  using ST = StageT<T>;
  constexpr int ND = D / 16;
  // stage: [KT half 0]([KT half 1])[per wave: dS half 0, (dS half 1,) dG half 0(, dG half 1)][reach of 4 key tiles]
  constexpr int TILES = HV * TT::BYTES, WAVE = 2 * HV * ST::BYTES, SB = TILES + 8 * WAVE + 1024;
  UA_STAGES(SB);
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, col = lane & 15, g = lane >> 4;
  int bx0, zq;
  xcd_map(bx0, zq);
  const int Lp = a.Lp, L = a.L, nT16 = Lp / 16, R = a.R, zk = zq / R, r = zq % R;
  // chunked operator with live (query, later chunk) pairs: their tiles are not exchanged, k_bwd_queries2 runs instead
  if (a.chunked && !a.skip_masked && *a.masked_nz != 0) return;
  const int n_blk = Lp / 128;
  // two query blocks of complementary length per workgroup, the body expanded once per block (see k_bwd_keys2)
  auto sweep = [&](const int jt) __attribute__((always_inline)) {
  const int tq = 8 * jt + w, tbq = tq >> 1;
  Stager<TT, 8> stT;
  stT.init(w, lane, Lp * (long)sizeof(T), D);
  f32x4 dQ[ND], dKc[ND];
#pragma unroll
  for (int n = 0; n < ND; ++n) { dQ[n] = (f32x4){0, 0, 0, 0}; dKc[n] = (f32x4){0, 0, 0, 0}; }
  const T* KTz = a.KT + (long)zk * D * Lp;
  const int n_kt = (4 * jt + 4) / HV;                  // steps of 32 HV keys
  const int kt_min = (a.minkey[zk * (nT16 >> 1) + 4 * jt] >> (HV == 2 ? 2 : 1)) & ~1;
  // this lane's 16 bytes of the wave's tiles of key half h: base + h * 1024
  const long st_head = grp_tiles(Lp >> 5) << 10;
  const char* pS = reinterpret_cast<const char*>(a.dS_st) + (long)zq * st_head + (grp_tile(tq, 0) << 10) + 16 * lane;
  // dG belongs to the part of the kv head's query groups that was swept together (see k_bwd_keys2): Rl groups
  const int Rl = R / a.key_parts;
  const char* pG = reinterpret_cast<const char*>(a.dG_st) + ((long)zk * a.key_parts + r / Rl) * st_head + (grp_tile(tq, 0) << 10) + 16 * lane;
  const int* reach_z = a.reach + zk * nT16;

#define UA_ISSUE(s, base)                                                                   \
  {                                                                                         \
    const int k0_ = 32 * HV * (s);                                                          \
    stT.issue((base), KTz + (long)k0_ * D, w);                                              \
    if (HV == 2) stT.issue((base) + TT::BYTES, KTz + (long)(k0_ + 32) * D, w);              \
    char* mine_ = (base) + TILES + w * WAVE;                                                \
    const long h_ = (long)(HV * (s)) << 13;      /* half h of the group: 8 tiles on */         \
    issue_row_nt(mine_, pS + h_);                                                                             \
    if (HV == 2) issue_row_nt(mine_ + ST::BYTES, pS + h_ + 8192);                                        \
    issue_row_nt(mine_ + HV * ST::BYTES, pG + h_);                                                               \
    if (HV == 2) issue_row_nt(mine_ + 3 * ST::BYTES, pG + h_ + 8192);                                    \
    if (w == 0) issue_row((base) + TILES + 8 * WAVE, reach_z + 4 * (HV == 2 ? (s) : (s) >> 1));                  \
  }
#define UA_COMPUTE(s, base) bq_step((s), (base))
  auto bq_step = [&] __device__ (int kti, char* base) {
    char* mine = base + TILES + w * WAVE;
    const int* rch = reinterpret_cast<const int*>(base + TILES + 8 * WAVE);
#pragma unroll
    for (int kq = 0; kq < HV; ++kq) {
      // the half's two 16-key tiles: visited by k_bwd_keys2 (hence written) iff not after the queries and in reach
      const int sbk = 2 * (HV * kti + kq), ri = HV == 2 ? 2 * kq : 2 * (kti & 1);
      const bool live0 = sbk <= tq && rch[ri] >= tbq, live1 = sbk + 1 <= tq && rch[ri + 1] >= tbq;
      if (!live0 && !live1) continue;
      Frag<T> as = ST::get(mine + kq * ST::BYTES, lane), ag = ST::get(mine + (HV + kq) * ST::BYTES, lane);
      // elements 0-3 of an operand are keys of the first tile, 4-7 of the second (perm32)
      if (!live0) { reinterpret_cast<uint2*>(&as)[0] = make_uint2(0, 0); reinterpret_cast<uint2*>(&ag)[0] = make_uint2(0, 0); }
      if (!live1) { reinterpret_cast<uint2*>(&as)[1] = make_uint2(0, 0); reinterpret_cast<uint2*>(&ag)[1] = make_uint2(0, 0); }
      const T* sKT = reinterpret_cast<const T*>(base + kq * TT::BYTES);
#pragma unroll
      for (int n = 0; n < ND; ++n) {
        const Frag<T> kb = ld8(sKT + TT::at(n, col, 0, g));
        mma16(dQ[n], as, kb);
        if (n % Rl == r % Rl) mma16(dKc[n], ag, kb);
      }
    }
  };
  UA_PIPE_START_AT(kt_min, n_kt, UA_ISSUE);
  UA_PIPE_RANGE(kt_min, n_kt, n_kt, UA_ISSUE, UA_COMPUTE);
#undef UA_ISSUE
#undef UA_COMPUTE
  // Epilogue.  A result tile holds (query 4g + v, feature 16n + col) in lane (g, col); stored from there, a wave moves
  // 32-byte pieces with one instruction per (v, n) and fetches the row side of dk the same way.  The tiles go through the
  // wave's share of the (now idle) stages instead, 64 features at a time, and leave as pieces of rows: lane (g, col) then
  // holds features 4 col .. 4 col + 3 of queries 4i + g, i = 0..3, so that 16 lanes move 128 contiguous bytes of dq / dk
  // and 256 of the row side of dk.
  static_assert(NST == 2, "the epilogue stages its tiles in both stage buffers");
  __syncthreads();                      // every wave is done with the stages
  constexpr int RS = 64 + 4;            // floats per staged row: the four row groups of a store hit different banks
  static_assert(4 * 16 * RS * 4 <= SB, "staging area");
  float* xs = reinterpret_cast<float*>((w < 4 ? stage0 : stage1) + (w & 3) * (16 * RS * 4));
  const bool vec_ok = (d & 3) == 0 && ((reinterpret_cast<uintptr_t>(dq) | reinterpret_cast<uintptr_t>(a.dk_out)) & 7) == 0;
  auto stage_half = [&] __device__ (const f32x4 (&X)[ND], int hf, f32x4 (&out)[4]) {
#pragma unroll
    for (int nn = 0; nn < 4; ++nn)
#pragma unroll
      for (int v = 0; v < 4; ++v) xs[(4 * g + v) * RS + 16 * nn + col] = X[4 * hf + nn][v];
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < 4; ++i) out[i] = *reinterpret_cast<const f32x4*>(xs + (4 * i + g) * RS + 4 * col);
    __builtin_amdgcn_wave_barrier();
  };
  auto store4 = [&] __device__ (T* dst, long row, int f0, const f32x4& x) {      // 4 consecutive features of a row of d
    if (vec_ok) {
      if (f0 < d) {
        union { T h[4]; u32x2 u; } pk;
#pragma unroll
        for (int e = 0; e < 4; ++e) pk.h[e] = cvt<T>(x[e]);
        __builtin_nontemporal_store(pk.u, reinterpret_cast<u32x2*>(dst + row * d + f0));
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (f0 + e < d) dst[row * d + f0 + e] = cvt<T>(x[e]);
    }
  };
  float dot[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int hf = 0; hf < D / 64; ++hf) {
    const int f0 = 64 * hf + 4 * col;
    // the row side of dk and the keys themselves, fetched before the tiles are staged
    f32x4 krow[4];
    u32x2 kraw[4];
    if (a.direct) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int t = 16 * tq + 4 * i + g;        // < Lp: both tensors are padded
        krow[i] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(a.dKrow + ((long)zq * Lp + t) * D + f0));
        kraw[i] = *reinterpret_cast<const u32x2*>(a.Kp + nat_off<D>(zq, Lp, t, f0));
      }
    }
    f32x4 x[4];
    stage_half(dQ, hf, x);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int t = 16 * tq + 4 * i + g;
      if (t < L) store4(dq, (long)zq * L + t, f0, x[i]);
    }
    stage_half(dKc, hf, x);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int t = 16 * tq + 4 * i + g;
      if (a.direct) {       // r = 1: dk = row side (k_bwd_keys2) + column side, ddest = (k_u . dkcol_u) / (2 dest_u)
        const T* kk = reinterpret_cast<const T*>(&kraw[i]);
#pragma unroll
        for (int e = 0; e < 4; ++e) dot[i] = __builtin_fmaf(x[i][e], (float)kk[e], dot[i]);      // padded features: k = 0
        if (t < L) store4(a.dk_out, (long)zq * L + t, f0, x[i] + krow[i]);
      } else {
        *reinterpret_cast<f32x4*>(a.dKdacc + ((long)zq * Lp + t) * D + f0) = x[i];
      }
    }
  }
  if (a.direct) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int t = 16 * tq + 4 * i + g;
      const float sum = allsum16(dot[i]);
      if (col == 0 && t < L) a.ddest_out[(long)zq * L + t] = cvt<T>(sum / (2.0f * (float)a.dest_in[(long)zq * L + t]));
    }
  }
  };
  // Several blocks per workgroup, the body expanded once per block (steps of 32 keys only: with steps of 64 the
  // expanded kernel is scheduled worse even for a single block).  Blocks of complementary length, heaviest first: all
  // workgroups are equally long, the launch is a whole number of rounds, and the epilogues - whose traffic slows the
  // stream of every other workgroup far beyond its bytes - fall together instead of spreading over the
  // launch.  Four blocks j, n/2 - 1 - j, n/2 + j, n - 1 - j when the grid says so, else two, else one.
  if constexpr (HV == 2) {
    sweep(n_blk - 1 - bx0);
  } else if (gridDim.x * 4 == n_blk) {
    sweep(n_blk - 1 - bx0);
    __syncthreads();       // the stages and the staging area are free
    sweep(n_blk / 2 + bx0);
    __syncthreads();
    sweep(n_blk / 2 - 1 - bx0);
    __syncthreads();
    sweep(bx0);
  } else {
    sweep(n_blk - 1 - bx0);
    if (gridDim.x != n_blk && n_blk - 1 - bx0 != bx0) {
      __syncthreads();
      sweep(bx0);
    }
  }
}

#undef UA_PIPELINE
#undef UA_PIPE_RANGE
#undef UA_PIPE_START
#undef UA_PIPE_START_AT
#undef UA_STEP2_
#undef UA_STAGES

}  // namespace ua
