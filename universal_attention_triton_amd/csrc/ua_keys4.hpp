// Key-stationary backward of the bf16 fused operator on 32x32 tiles, one wave per SIMD, software pipelined.
//
//   k_bwd_keys4   same inputs, outputs and tile formats as k_bwd_keys2<TO> (ua_fused.hpp): bias from the fp16 tiles of
//                 k_carry2<BO>, dS / dG tiles for k_bwd_queries3, dV, the row side of dK and dsrc.
//
// Why another tiling.  Measured on this part (instruction streams without memory traffic): a v_mfma_f32_16x16x32_bf16 keeps
// the matrix pipe for 16 cycles but also takes two of the SIMD's four-cycle issue slots, a v_mfma_f32_32x32x16_bf16 does twice
// the work in 32 cycles and takes one, and every LDS operand of 1 KB feeds twice the work.  With 16 keys per wave the
// products of a step are bound by operand delivery from LDS (1 KB per 16-cycle instruction is the whole LDS bandwidth of
// a CU) and the elementwise chain by instruction issue, one after the other.  Here a wave owns 32 keys: half the LDS
// operand bytes and a quarter of the issue slots per product, at the price of 128 accumulator registers per wave for
// dK and dV (head dim 128), i.e. one wave per SIMD with the accumulators in the second half of the register file.
// A single wave per SIMD has nobody to hide its latencies behind, so a step is laid out by hand as 48 slots of one matrix
// instruction, the LDS reads of a later one and a share of the vector work each (see `body`).
//
// Orientation (v_mfma_f32_32x32x16): a result tile is [32 queries][32 keys]; lane l holds key l % 32 and the 16 queries
// t = 8 (v / 4) + 4 (l / 32) + v % 4 of the block in register v (t_of).  as_operand(tile, q) turns registers 8q..8q+7
// into the B operand of a product that contracts over the block's queries 16q..16q+15.
#pragma once
#include <type_traits>

#include "ua_bwd.hpp"
#include "ua_common.hpp"
#include "ua_fused.hpp"

namespace ua {

// Natural [32 positions][D features] tiles in LDS, k-group-major (16-byte unit u = kgroup * 32 + row, see Tile), with the
// row of a unit exchanged inside its k-group: row ^ swz(kgroup).  The 16-byte operand reads of the input products (one
// k-group, 32 rows per half wave) stay contiguous; the transposing 8-byte reads of the output products, whose 32 lanes of
// a half wave touch (4 rows) x (4 k-groups) x (8 bytes), then fall on 32 different banks instead of 8 (measured without
// the exchange: 8 cycles of the LDS pipe per read instead of 2, which made the LDS pipe the longest resource of a step).
__host__ __device__ __forceinline__ constexpr int k4_swz(int kgroup) { return ((kgroup & 1) << 3) | (((kgroup >> 1) & 1) << 2); }

// Ties a value to this point of the program: the compiler may neither compute it later nor use it earlier than here
// (arithmetic is otherwise free to move across the scheduling fences of a slot).
__device__ __forceinline__ void pin(float& x) { asm volatile("" : "+v"(x)); }
#define UA_PINV(vec, idx) { float t_ = (vec)[idx]; pin(t_); (vec)[idx] = t_; }      // the same for an element of a register tile
// Asynchronous 16-byte-per-lane copies global -> LDS (lane l lands at lds_addr + 16 l), written as assembly.  As a builtin
// the copy counts as a flat-address instruction that is outstanding on both memory counters, and while one is in flight
// the compiler turns every wait for an LDS read into a wait for all of them (lgkmcnt(0)), i.e. for the operand requested
// a few instructions earlier instead of the one requested four slots ago.  Invisible to the compiler, the copies need no
// distinct stage objects either; the kernel orders them against the LDS reads itself (memory counter wait + barrier at
// the top of a step).
__device__ __forceinline__ void dma16(const void* src_lane, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(src_lane), "s"(lds_addr) : "memory");
}
__device__ __forceinline__ void dma16_nt(const void* src_lane, unsigned lds_addr) {      // read-once data
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt" :: "v"(src_lane), "s"(lds_addr) : "memory");
}
// Matrix instructions whose result the vector unit reads: written as assembly so that accumulator and result live in
// vector registers (with 512 registers per lane the compiler places every result of the matrix builtins in the
// accumulation half of the file and copies it out, one instruction per register) and the stationary operand in the
// accumulation half.  The compiler does not know their latency: a result is only read several slots (each longer than
// the 11 wait states an 8-pass instruction needs) after its last instruction, and dependent instructions on one
// accumulator are at least a slot apart.
typedef __attribute__((ext_vector_type(8))) __bf16 k4_bf16x8;
__device__ __forceinline__ void mma_v(f32x16& c, const Frag<bf16>& a, const k4_bf16x8& b) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(__builtin_bit_cast(k4_bf16x8, a)), "a"(b));
}
__device__ __forceinline__ void mma_v0(f32x16& c, const Frag<bf16>& a, const k4_bf16x8& b) {      // c = a b
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(__builtin_bit_cast(k4_bf16x8, a)), "a"(b));
}
// compile-time loop: f(std::integral_constant<int, B>()), ..., f(std::integral_constant<int, E - 1>())
template <int B, int E, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (B < E) {
    f(std::integral_constant<int, B>());
    static_for<B + 1, E>(f);
  }
}

// grid (Lp / 128, Zk); 4 waves; wave w owns keys 128 g + 32 w .. + 31 and sweeps the 32-query blocks from the last one it
// reaches down to its own.  One query group per kv head, merged operator, head dim (padded) 128.
template <int D>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) k_bwd_keys4(BwdArgs<bf16> a) {
  static_assert(D == 128, "the slot layout of a step is written for eight k-steps per input product");
  using T = bf16;
  using TN = Tile<T, 32, D>;
  constexpr int NQ = D / 16, NB = D / 32;
  // stage: [K of the query block][Q][dO][stats: -lse (natural log) 32f, -delta 32f, ldest 32f][bias: 2 KB per wave]
  constexpr int TILES = 3 * TN::BYTES, SB = TILES + 1024 + 4 * 2048;
  // four stages in a ring: during step s the tiles of blocks s - 1 and s are read, the first operands of block s + 1 are
  // fetched at its end, and the tiles of block s + 2 arrive
  __shared__ __attribute__((aligned(1024))) char lds[4 * SB];
  const unsigned lds0 = (unsigned)(size_t)lds;
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, col = lane & 31, hi = lane >> 5;
  int kg0, zo;
  xcd_map(kg0, zo);
  const int zk = zo;
  const int Lp = a.Lp, L = a.L, nT16 = Lp / 16;
  // a grid of half as many workgroups as key groups: this one sweeps group kg0 and then group (last - kg0), which
  // together are as long as every other pair (equal workgroups, half as many workgroup changes)
  const int n_kg = Lp / 128, n_items = (int)gridDim.x < n_kg ? 2 : 1;
  for (int item = 0; item < n_items; ++item) {
  const int kg = item == 0 ? kg0 : n_kg - 1 - kg0;
  if (item == 1) {
    if (kg == kg0) break;                        // odd number of groups: the middle one has no partner
    __syncthreads();                             // the stages of the first sweep are free
  }
  const int sb32 = 4 * kg + w, spos = 32 * sb32 + col;
  const int nTr = (L + 31) / 32, first = 4 * kg;
  if (first >= nTr) continue;                    // every key of this group is padding
  const int* reach_z = a.reach + zk * nT16 + 8 * kg;
  int top = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) top = max(top, reach_z[i]);
  top = min(top, nTr - 1);
  const int myreach = min(max(reach_z[2 * w], reach_z[2 * w + 1]), top);
  // the wave sweeps as far as the farther-reaching of its two 16-key tiles; the pre-pass wrote no bias tiles for the other
  // one beyond that tile's own reach, so this lane's weights are zero in the blocks after `lane_reach`
  const int lane_reach = reach_z[2 * w + (col >> 4)];
  const int total = top + 1 - first;
  // this wave takes part in steps s_lo .. s_hi (query blocks top - s): from the last block it reaches to its own
  const int s_lo = top - myreach, s_hi = top - sb32;
  // source offsets of this wave's two copy instructions per tile: unit u of the LDS image holds row (u & 31) ^ swz(u >> 5)
  int cp_off[2];
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    const int u = (w + 4 * k) * 64 + lane;
    cp_off[k] = ((u & ~31) | ((u & 31) ^ k4_swz(u >> 5))) * 16;
  }

  k4_bf16x8 kp[NQ], vf[NQ];
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const long ro = nat_off<D>(zk, Lp, spos, 16 * q + 8 * hi);
    kp[q] = __builtin_bit_cast(k4_bf16x8, ld8(a.Kp + ro));
    vf[q] = __builtin_bit_cast(k4_bf16x8, ld8(a.Vp + ro));
  }
  const float la = a.lsrc[(long)zk * Lp + spos];
  f32x16 dVt[NB], dKt[NB];
#pragma unroll
  for (int n = 0; n < NB; ++n) { dVt[n] = (f32x16){0}; dKt[n] = (f32x16){0}; }
  float dsrc_acc = 0.f;
  // reverse running sum of dS over the block's queries on the matrix core: row u of the 0/1 operand sums the queries >= u;
  // a second product with an operand of ones keeps the sum over all queries swept so far in every row of `run`
  k4_bf16x8 tri[2], ones;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
#pragma unroll
    for (int q = 0; q < 2; ++q) tri[q][e] = (__bf16)((16 * q + 8 * (e >> 2) + 4 * hi + (e & 3)) >= col ? 1.0f : 0.0f);
    ones[e] = (__bf16)1.0f;
  }
  const T* Kz = a.Kp + (long)zk * Lp * D;
  const T* Qz = a.Qp + (long)zk * Lp * D;
  const T* Gz = a.dOp + (long)zk * Lp * D;
  const float* ldz = a.ldest + (long)zk * Lp;
  // wave 0 fetches the block's normalisers and deltas through registers and stores them negated (lse in natural units), so
  // that they can start the accumulators of the score and dP products
  const float* st_src = (lane < 32 ? a.lse2 : a.delta) + (long)zk * Lp + (lane & 31);
  const float st_mul = lane < 32 ? -kLn2 : -1.0f;
  float st_pre = 0.f;
  // this lane's 16 bytes of the wave's two bias tiles (16 keys each) of query block 0
  const char* bt_src = reinterpret_cast<const char*>(a.Bt) + (((long)zk * tri_tiles(Lp >> 5) + 2 * sb32) << 10) + 16 * lane;
  const long st_head = grp_tiles(Lp >> 5) << 10;                   // bytes of gradient tiles per head
  // tile indices inside a head in 32 bits (the scalar unit multiplies 64-bit values in several instructions, and a lone
  // wave pays for every one of them); widened once for the byte offset
  auto grp32 = [] __device__ (int tq, int h) __attribute__((always_inline)) -> long {
    return (long)(unsigned)(16 * (tq >> 3) * ((tq >> 3) + 1) + 8 * h + (tq & 7)) << 10;
  };
  // a lane's 8-byte pieces inside a (32 keys, 16 queries) gradient tile: queries 8 (j & 1) + 4 hi .. + 3 of the tile
  const int st_lane0 = StageT<bf16>::addr(perm32(col), 8 * hi), st_lane1 = StageT<bf16>::addr(perm32(col), 8 * (2 + hi));
  char* dS_base = reinterpret_cast<char*>(a.dS_st) + (long)zk * st_head;
  char* dG_base = reinterpret_cast<char*>(a.dG_st) + (long)zo * st_head;
  // A operand of an input product: lane (row col, half hi) takes the 16 bytes of k-group 2 q + hi of its row
  const int nat_even = hi * 512 + ((col ^ (hi << 3)) << 4), nat_odd = hi * 512 + ((col ^ (hi << 3) ^ 4) << 4);
  // A operand of an output product (row = feature 32 n + l % 32, k = the 16 queries of half q of the block in as_operand
  // order) out of a natural tile with two transposing 8-byte reads: the 16 lanes of a lane group fetch a (4 positions,
  // 16 features) block and receive it transposed.  Lane (i, fh, hi) fetches k-group 4 n + 2 fh + kbit, position
  // 16 q + 4 hi + i / 4 (+ 8 in the second read), bytes 8 (i & 1) ..
  int tr_a, tr_b;
  {
    const int i = lane & 15, fh = (lane >> 4) & 1, kbit = (i & 3) >> 1, kgrp = 2 * fh + kbit;
    tr_a = kgrp * 512 + (((4 * hi + (i >> 2)) ^ k4_swz(kgrp)) << 4) + 8 * (i & 1);
    tr_b = tr_a ^ 128;
  }
  const int bias_lane = TILES + 1024 + w * 2048 + (col >> 4) * 1024 + 16 * (col & 15) + 256 * hi;

  // ---- state carried from step to step
  f32x16 F, Gk, dB, run;        // of the block worked on last: dG / dl, relu(G), reverse running sum of dS; sum of dS so far
  Frag<T> bp[2], bs[2];         // its P and dS as operands
  constexpr int PF = 4;         // operands in flight
  Frag<T> ring[PF];             // the first operands of the coming step
  f32x16 S, dP;                 // accumulators of its score and dP products, started from -lse and -delta of its queries
#pragma unroll
  for (int v = 0; v < 16; ++v) { F[v] = 0.f; Gk[v] = 0.f; dB[v] = 0.f; run[v] = 0.f; }
#pragma unroll
  for (int q = 0; q < 2; ++q)
#pragma unroll
    for (int e = 0; e < 8; ++e) { bp[q].v[e] = (bf16)0.f; bs[q].v[e] = (bf16)0.f; }

  auto issue = [&] __device__ (int s, int stage) __attribute__((always_inline)) {
    const int tb = top - s;
    const unsigned base = lds0 + (stage & 3) * SB;
#pragma unroll
    for (int t = 0; t < 3; ++t) {
      const char* src = reinterpret_cast<const char*>((t == 0 ? Kz : (t == 1 ? Qz : Gz)) + (long)(32 * tb) * D);
#pragma unroll
      for (int k = 0; k < 2; ++k) dma16(src + cp_off[k], base + t * TN::BYTES + (w + 4 * k) * 1024);
    }
    if (w == 0) {
      dma16(ldz + 32 * tb + 4 * (lane & 7), base + TILES);      // every 128-byte piece of the row: ldest of the block
      st_pre = st_src[32 * tb];
    }
    const char* bsrc = bt_src + ((long)(unsigned)(tb * (tb + 1)) << 10);
    dma16_nt(bsrc, base + TILES + 1024 + w * 2048);
    dma16_nt(bsrc + 1024, base + TILES + 1024 + w * 2048 + 1024);
  };
  auto stage_at = [&] __device__ (int s) __attribute__((always_inline)) -> char* { return lds + (s & 3) * SB; };
  auto pre_write = [&] __device__ (char* base) __attribute__((always_inline)) {
    if (w == 0) reinterpret_cast<float*>(base + TILES)[lane] = st_pre * st_mul;
  };
  auto ld_tr = [&] __device__ (const char* tile, int n, int q) __attribute__((always_inline)) -> Frag<T> {
    Frag<T> f;
    reinterpret_cast<v4s16*>(&f)[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s16_t)(tile + tr_a + n * 2048 + q * 256));
    reinterpret_cast<v4s16*>(&f)[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s16_t)(tile + tr_b + n * 2048 + q * 256));
    return f;
  };
  auto ld_nat = [&] __device__ (const char* tile, int q) __attribute__((always_inline)) -> Frag<T> {
    return *reinterpret_cast<const Frag<T>*>(tile + ((q & 1) ? nat_odd : nat_even) + 1024 * q);
  };
  // the first operands and the stats of a block, fetched ahead of its step
  auto preload = [&] __device__ (const char* base) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < PF; ++i) ring[i] = ld_nat(base, i);
    const float* stats = reinterpret_cast<const float*>(base + TILES);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const float4 x = *reinterpret_cast<const float4*>(stats + 8 * g + 4 * hi), y = *reinterpret_cast<const float4*>(stats + 32 + 8 * g + 4 * hi);
      S[4 * g] = x.x; S[4 * g + 1] = x.y; S[4 * g + 2] = x.z; S[4 * g + 3] = x.w;
      dP[4 * g] = y.x; dP[4 * g + 1] = y.y; dP[4 * g + 2] = y.z; dP[4 * g + 3] = y.w;
    }
  };
  // OUT: dV += P^T dO, dK += dS^T Q + dG^T K over the block's queries
  auto out_products = [&] __device__ (const char* base, const Frag<T> (&bg)[2]) __attribute__((always_inline)) {
#pragma unroll
    for (int q = 0; q < 2; ++q)
#pragma unroll
      for (int n = 0; n < NB; ++n) {
        mma(dVt[n], ld_tr(base + 2 * TN::BYTES, n, q), bp[q]);
        mma(dKt[n], ld_tr(base + TN::BYTES, n, q), bs[q]);
      }
#pragma unroll
    for (int q = 0; q < 2; ++q)
#pragma unroll
      for (int n = 0; n < NB; ++n) mma(dKt[n], ld_tr(base, n, q), bg[q]);
  };
  // One pipelined step on block s (stage `cur`) with the second half of block s - 1 (stage `prv`).  The matrix pipe runs
  // 48 + 2 instructions: K K^T of block s (slots 0-7), Q K^T - lse and dO V^T - delta (8-23), the three output products of
  // block s - 1 (24-47), the reverse running sum of the new dS.  The vector unit meanwhile turns last step's running sum
  // into dG (V2, slots 0-9), then works through the decay chain of block s (needs only K K^T) and its softmax chain.
  // A slot = one matrix instruction, the LDS reads of the operand PF slots ahead, and a share of the vector work;
  // scheduling fences keep the slots in this order (left alone the compiler issues the matrix instructions in runs,
  // each behind its own LDS read, and the single wave of the SIMD then waits where two waves would have covered for
  // one another).  The operands of the first slots and the stats of block s + 1 (stage `nxt`) are requested at the end.
  // GEN: the general form for the first and last steps of a wave (run-time `first` and `masked`); the first step of a
  // wave finds zero operands for the block before and parks the tile stores of V2.
  auto body = [&] __device__ (int s, const char* prv, const char* cur, const char* nxt, auto gen_c, const bool first, const bool masked)
                  __attribute__((always_inline)) {
    constexpr bool GEN = decltype(gen_c)::value;
    const int tb = top - s;
    const float* stats = reinterpret_cast<const float*>(cur + TILES);
    // A operand of the matrix instruction of slot i
    auto load_opnd = [&] __device__ (int i) __attribute__((always_inline)) -> Frag<T> {
      if (i < 8) return ld_nat(cur, i);
      if (i < 24) return ld_nat(cur + (1 + ((i - 8) & 1)) * TN::BYTES, (i - 8) >> 1);
      if (i < 40) return ld_tr(prv + ((i & 1) ? 1 : 2) * TN::BYTES, ((i - 24) >> 1) & 3, (i - 24) >> 3);
      return ld_tr(prv, (i - 40) & 3, (i - 40) >> 2);
    };
    f32x16 G, dG;
    Frag<T> bg[2], nbp[2], nbs[2];
    float lb[16];
    load_t16(stats + 64, hi, lb);
    typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
    // bias: the wave's two fp16 tiles (16 keys x 32 queries each); lane (g, c) of a tile owns 16 bytes: queries 4g..4g+3
    // of the block's first 16 queries, then of the second
    const f16x8 hb0 = *reinterpret_cast<const f16x8*>(cur + bias_lane), hb1 = *reinterpret_cast<const f16x8*>(cur + bias_lane + 512);
    const int tl0 = 32 * tb + 4 * hi - spos;        // query position minus key position for v = 0
    float afv[16];
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, 48>([&](auto ic) __attribute__((always_inline)) {
      constexpr int i = decltype(ic)::value;
      // ---- vector work of the slot
      // The vector work of a slot runs in three passes over its elements: tie the inputs to the slot, compute, tie the
      // results to the slot - so that the chains of the slot's elements can be interleaved with one another (a
      // transcendental needs an independent instruction behind it) but not moved out of the slot.
      //   slots 0-9:   V2 of the block before, dG = dl * F (16 elements over 10 slots)
      //   slots 10-34: decay chain; element v has its affinity in slot 10 + v + v / 2 (two slots out of three) and its
      //                dG / dl factor together with the next element's affinity
      //   slots 34-47: softmax chain; two elements in each of the first two slots, then one per slot
      // (the vector work has to be spread over all 48 slots: with the chains packed two elements per slot into slots
      // 10-33, fewer wait states but matrix instructions alone in the last 14 slots, the step is 2 % slower)
      auto vec = [&](auto pc) __attribute__((always_inline)) {
        constexpr int ph = decltype(pc)::value / 16, v = decltype(pc)::value % 16;
        constexpr bool u_v2 = i < 10 && (v * 10) / 16 == i;
        // element v: affinity in slot 10 + v + v / 2 (two slots out of three), its factor together with the next
        // element's affinity (two independent chains per slot cover the latency of the transcendentals)
        constexpr bool u_aff = i == 10 + v + v / 2;
        constexpr bool u_f = v < 15 ? i == 10 + (v + 1) + (v + 1) / 2 : i == 34;
        constexpr bool u_sm = i >= 34 && (i < 36 ? (v >> 1) == i - 34 : v == i - 32);
        if constexpr (u_v2) {
          if constexpr (ph == 0) { dG[v] = dB[v]; UA_PINV(dG, v) }
          if constexpr (ph == 1) {
            dG[v] *= F[v];
            dsrc_acc = __builtin_fmaf(dG[v], Gk[v], dsrc_acc);
            if constexpr (v & 1) { bg[v >> 3].v[(v & 7) - 1] = cvt<T>(dG[v - 1]); bg[v >> 3].v[v & 7] = cvt<T>(dG[v]); }
          }
          if constexpr (ph == 2 && (v & 1)) pin(dsrc_acc);
        }
        if constexpr (u_aff) {            // affinity
          if constexpr (ph == 0) UA_PINV(G, v)
          if constexpr (ph == 1) {
            const float gk = fmaxf(G[v], 0.f);
            Gk[v] = gk;
            afv[v] = affinity(__builtin_amdgcn_logf(gk), lb[v] + la);
          }
          if constexpr (ph == 2) pin(afv[v]);
        }
        if constexpr (u_f) {              // F = dG / dl = (2/3) A / ((clamp(A) - 1) G), zero where A exceeds the clamp
          if constexpr (ph == 0) pin(afv[v]);
          if constexpr (ph == 1) {
            const float af = afv[v];
            const float den15 = __builtin_fmaf(__builtin_amdgcn_fmed3f(af, kAMinBwd, kAMax), 1.5f, -1.5f);
            float f = (af <= kAMax) ? af * __builtin_amdgcn_rcpf(den15 * fmaxf(Gk[v], 1.0e-30f)) : 0.f;
            if (GEN) f = (masked && (tl0 + 8 * (v >> 2) + (v & 3)) <= 0) ? 0.f : f;
            F[v] = f;
          }
          if constexpr (ph == 2) UA_PINV(F, v)
        }
        if constexpr (u_sm) {             // softmax weight and score gradient
          constexpr int j = v >> 2, m = v & 3;
          if constexpr (ph == 0) { UA_PINV(S, v) UA_PINV(dP, v) }
          if constexpr (ph == 1) {
            const float bias = (float)((j & 1) ? hb1[4 * (j >> 1) + m] : hb0[4 * (j >> 1) + m]);
            float p = __builtin_amdgcn_exp2f(__builtin_fmaf(S[v], kLog2e, bias));
            if (GEN) p = ((masked && (tl0 + 8 * j + m) < 0) || tb > lane_reach) ? 0.f : p;
            S[v] = p;
            dP[v] *= p;
          }
          if constexpr (ph == 2) {
            UA_PINV(S, v) UA_PINV(dP, v)
            if constexpr (v & 1) {
              nbp[v >> 3].v[(v & 7) - 1] = cvt<T>(S[v - 1]); nbp[v >> 3].v[v & 7] = cvt<T>(S[v]);
              nbs[v >> 3].v[(v & 7) - 1] = cvt<T>(dP[v - 1]); nbs[v >> 3].v[v & 7] = cvt<T>(dP[v]);
            }
          }
        }
      };
      // the inputs are tied to the slot BEFORE its matrix instruction: an instruction that reads a value right behind the
      // (empty) assembly statement that ties it costs a wait state
      static_for<0, 16>(vec);
      // ---- matrix instruction of the slot, and the operand PF slots ahead
      // one wait for the operands of two slots (every wait is an instruction the lone wave has to issue): behind the
      // operands of slots i and i + 1 only those of slots i + 2 and i + 3 are in flight, one LDS read each for the input
      // products and two for the transposed operands of the output products
      if constexpr ((i & 1) == 0 && PF == 4) {
        constexpr int behind = (i + 2 < 24 ? 1 : (i + 2 < 48 ? 2 : 0)) + (i + 3 < 24 ? 1 : (i + 3 < 48 ? 2 : 0));
        __builtin_amdgcn_s_waitcnt(0xC07F | (behind << 8));          // lgkmcnt(behind), the other counters unconstrained
        if constexpr (i >= 24) __builtin_amdgcn_sched_barrier(0);     // or the matrix builtin is moved in front of the wait
      }
      if constexpr (i == 0) mma_v0(G, ring[i % PF], kp[i]);
      else if constexpr (i < 8) mma_v(G, ring[i % PF], kp[i]);
      else if constexpr (i < 24) { if constexpr ((i - 8) & 1) mma_v(dP, ring[i % PF], vf[(i - 8) >> 1]); else mma_v(S, ring[i % PF], kp[(i - 8) >> 1]); }
      else if constexpr (i < 40) { if constexpr (i & 1) mma(dKt[((i - 24) >> 1) & 3], ring[i % PF], bs[(i - 24) >> 3]); else mma(dVt[((i - 24) >> 1) & 3], ring[i % PF], bp[(i - 24) >> 3]); }
      else mma(dKt[(i - 40) & 3], ring[i % PF], bg[(i - 40) >> 2]);
      if constexpr (i + PF < 48) ring[i % PF] = load_opnd(i + PF);
      static_for<16, 48>(vec);
      if constexpr (i == 9) {
        char* p = dG_base + ((!GEN || !first) ? grp32(2 * (tb + 1), sb32) : st_head - 2048);
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          __builtin_nontemporal_store(reinterpret_cast<const u32x2*>(&bg[q])[0], reinterpret_cast<u32x2*>(p + 1024 * q + st_lane0));
          __builtin_nontemporal_store(reinterpret_cast<const u32x2*>(&bg[q])[1], reinterpret_cast<u32x2*>(p + 1024 * q + st_lane1));
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    });
#pragma unroll
    for (int q = 0; q < 2; ++q) { bp[q] = nbp[q]; bs[q] = nbs[q]; }
    {
      char* p = dS_base + grp32(2 * tb, sb32);
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        __builtin_nontemporal_store(reinterpret_cast<const u32x2*>(&bs[q])[0], reinterpret_cast<u32x2*>(p + 1024 * q + st_lane0));
        __builtin_nontemporal_store(reinterpret_cast<const u32x2*>(&bs[q])[1], reinterpret_cast<u32x2*>(p + 1024 * q + st_lane1));
      }
    }
    // ---- dB = (sum of dS over the blocks swept before) + reverse running sum of the block's dS
    // (matrix builtins: the compiler keeps `run` and the result in the accumulation half, inserts the waits their
    // operands need - they come straight from vector instructions - and V2 copies dB out next step)
    {
      f32x16 t = run;
      mma(t, __builtin_bit_cast(Frag<T>, tri[0]), bs[0]);
      mma(t, __builtin_bit_cast(Frag<T>, tri[1]), bs[1]);
      mma(run, __builtin_bit_cast(Frag<T>, ones), bs[0]);
      mma(run, __builtin_bit_cast(Frag<T>, ones), bs[1]);
      dB = t;
    }
    if (!GEN || !masked) preload(nxt);
  };
  // after a wave's last step: second half of its own block
  auto tail = [&] __device__ (int s, const char* cur) __attribute__((always_inline)) {
    Frag<T> bg[2];
    f32x16 dG;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      dG[v] = dB[v] * F[v];
      dsrc_acc = __builtin_fmaf(dG[v], Gk[v], dsrc_acc);
    }
#pragma unroll
    for (int q = 0; q < 2; ++q) bg[q] = as_operand<T>(dG, q);
    char* p = dG_base + grp32(2 * (top - s), sb32);
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      __builtin_nontemporal_store(reinterpret_cast<const u32x2*>(&bg[q])[0], reinterpret_cast<u32x2*>(p + 1024 * q + st_lane0));
      __builtin_nontemporal_store(reinterpret_cast<const u32x2*>(&bg[q])[1], reinterpret_cast<u32x2*>(p + 1024 * q + st_lane1));
    }
    out_products(cur, bg);
  };
  // one step in its general form (first and last steps of the waves)
  auto gen_step = [&] __device__ (int s) __attribute__((always_inline)) {
    __builtin_amdgcn_s_waitcnt(0x0F70);    // vmcnt(0): the tiles of block s + 1 (and every earlier request) have arrived
    if (s + 1 < total) pre_write(stage_at(s + 1));
    __syncthreads();
    if (s + 2 < total) issue(s + 2, s + 2);
    if (s >= s_lo && s <= s_hi) {
      if (s == s_lo) preload(stage_at(s));
      body(s, stage_at(s + 3), stage_at(s), stage_at(s + 1), TrueC(), s == s_lo, s == s_hi);
      if (s == s_hi) tail(s, stage_at(s));
    }
  };
  // fast steps: every wave issued eight tile stores after the loads of block s + 1; vmcnt(8) completes those loads (the
  // memory counter runs in issue order) and leaves the stores in flight
  {
    // the stage "before" step 0 only has to hold finite values (its products are taken with zero operands)
    issue(0, 3);
    issue(0, 0);
    __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0)
    pre_write(stage_at(0));
    if (total > 1) issue(1, 1);
    // steps in which every wave is past its first and before its last and every 16-key tile is within its reach:
    // (last tile to join) < s < total - 4
    int s_join = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) s_join = max(s_join, top - min(reach_z[i], top));
    const int fast0 = s_join + 1, fast1 = total - 4;
    int s = 0;
    for (; s < total && s < fast0; ++s) gen_step(s);
    for (; s < fast1; ++s) {
      __builtin_amdgcn_s_waitcnt(0x0F78);    // vmcnt(8)
      pre_write(stage_at(s + 1));
      __syncthreads();
      issue(s + 2, s + 2);
      body(s, stage_at(s + 3), stage_at(s), stage_at(s + 1), FalseC(), false, false);
    }
    for (; s < total; ++s) gen_step(s);
  }
  // epilogue
  const float tot = dsrc_acc + xor_lane(dsrc_acc, 32);
  const bool direct = a.direct;
  if (direct) {      // straight into the caller's tensor: dsrc = sum dA A / (3 src), sum dA A = 3/2 sum dG G
    if (hi == 0 && spos < L) a.dsrc_out[(long)zo * L + spos] = cvt<T>(1.5f * tot / (3.0f * (float)a.src_in[(long)zo * L + spos]));
  } else if (hi == 0) {
    a.dsrc_raw[(long)zo * Lp + spos] = 1.5f * tot;
  }
#pragma unroll
  for (int n = 0; n < NB; ++n) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int f0 = 32 * n + 8 * g + 4 * hi;
      const long o = ((long)zo * Lp + spos) * D + f0;
      *reinterpret_cast<float4*>(a.dKrow + o) = make_float4(dKt[n][4 * g], dKt[n][4 * g + 1], dKt[n][4 * g + 2], dKt[n][4 * g + 3]);
      if (!direct) {
        *reinterpret_cast<float4*>(a.dVrow + o) = make_float4(dVt[n][4 * g], dVt[n][4 * g + 1], dVt[n][4 * g + 2], dVt[n][4 * g + 3]);
      } else if (spos < L) {
        T* dst = a.dv_out + ((long)zo * L + spos) * a.d_out + f0;
#pragma unroll
        for (int v = 0; v < 4; ++v)
          if (f0 + v < a.d_out) dst[v] = cvt<T>(dVt[n][4 * g + v]);
      }
    }
  }
  }  // item
}

#undef UA_PINV

}  // namespace ua
