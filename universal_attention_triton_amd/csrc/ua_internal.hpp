// Host-side declarations shared by the translation units of libua_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace ua {

// type-erased argument block of k_bwd_keys (same field order as BwdArgs<T>)
struct BwdArgsV {
  const int *reach, *minkey, *masked_nz;
  const void *Kp, *Vp, *KT, *Qp, *QT, *dOp, *dOT;
  const float *lsrc, *ldest, *lse2, *delta, *C;
  float *dQacc, *dKdacc, *Dsuf, *dKrow, *dVrow, *dsrc_raw;
  void *dS_st, *dG_st;
  const void* Bt;
  int R, L, Lp, c, nch, chunked, skip_masked, split_r, key_parts;
  int direct, d_out;
  void *dk_out, *dv_out, *dsrc_out, *ddest_out;
  const void *src_in, *dest_in;
  int dO_rows;
  int keys_variant;     // UA_TUNE_BWD_KEYS
  int pair;             // UA_TUNE_CHUNKED_PAIR (chunked operator): see paired_items
};

// Every launcher returns hipGetLastError() after enqueuing.  dtype: 0 fp32, 1 bf16.  D in {64,128}.
// tiled: Kp is stored in tiles of 32 keys, k-group-major (fused mode) instead of row-major (chunked mode)
// knorm2 [Zk][Lp/32], qnorm2 [Zk*R][Lp/32] (optional): largest squared row norm of every block of 32 keys / queries,
// enables pruning; reach (optional): [Zk][Lp/16] out.  With reach given, minkey [Zk][Lp/32] is filled as well.
// Bt (optional, bf16 + tiled): fp16 bias tiles [Zk][Lp/32][Lp/16][1 KB] are written instead of the carries C
// variant (bias tiles only): UA_TUNE_CARRY
hipError_t launch_carry(int dtype, int D, const void* Kp, const float* lsrc, const float* ldest, float* C, int Lp, int Zk,
                        int tiled, const float* knorm2, const float* qnorm2, int R, int* reach, int* minkey, hipStream_t s,
                        void* Bt = nullptr, int variant = 0);
int fwd_fused_variants(int dtype, int D);
hipError_t launch_fwd_fused(int dtype, int D, int variant, const void* Qp, const void* Kp, const void* VT,
                            const float* lsrc, const float* ldest, const float* C, void* O, float* lse, float* lse2,
                            const int* reach, const int* minkey, int R, int L, int Lp, int d, int Zq, hipStream_t s,
                            const void* Bt = nullptr);   // Bt (bf16): bias tiles of launch_carry; variant is then UA_TUNE_FWD_TILES
hipError_t launch_fwd_chunked(int dtype, int D, const void* Qp, const void* Kp, const void* VT, const float* lsrc,
                              const float* ldest, void* out, void* denom, float* lse2, long o_sz, long o_st, long o_sd,
                              long o_si, int R, int L, int Lp, int d, int c, int nch, int Zk, hipStream_t s);
// chunk a multiple of 64: the chunked operator through the query-stationary kernel (tiled working tensors, carries
// C and reach / minkey from launch_carry); also fills the results of the queries that precede a chunk
hipError_t launch_fwd_chunked2(int dtype, int D, const void* Qp, const void* Kp, const void* Vp, const void* VT, const float* lsrc,
                               const float* ldest, const float* C, const int* reach, const int* minkey, void* out, void* denom,
                               float* lse2, long o_sz, long o_st, long o_sd, long o_si, int R, int L, int Lp, int d, int c, int nch,
                               int Zq, hipStream_t s, int pair = 0);
// Work items per workgroup of the kernels that can take two of complementary length (`pair` arguments, BwdArgsV::pair):
// 0 = two once the launch is large enough (the launcher's own rule), 1 = one, 2 = two.
inline int paired_items(int n_items, bool large_launch, int pair) {
  return (pair == 2 || (pair != 1 && large_launch)) ? (n_items + 1) / 2 : n_items;
}
// cols != 0: the kernel also produces dQ / dkcol through atomics (chunked mode, row-major working tensors);
// cols == 0: it records the suffix carries and launch_bwd_queries finishes the query side (tiled working tensors;
// with a.chunked set: the chunked operator for a chunk that is a multiple of 64).
// With a.key_parts > 1 (bf16 tiles, merged operator) the grid covers (kv head, part of its query groups) pairs.
hipError_t launch_bwd_keys(int dtype, int D, const BwdArgsV& a, int Zk, int cols, hipStream_t s);
// bf16 merged operator over bias tiles, one query group per kv head, D in {64,128}: 32 keys per wave (ua_keys4.hpp)
hipError_t launch_bwd_keys4(int D, const BwdArgsV& a, int Zk, hipStream_t s);
hipError_t launch_bwd_queries(int dtype, int D, const BwdArgsV& a, void* dq, int d, int Zk, hipStream_t s);
// bf16 only, a.dS_st / a.dG_st filled by launch_bwd_keys (cols == 0): the query side as pure matrix work over those tiles
// variant: UA_TUNE_BWD_QUERIES
hipError_t launch_bwd_queries_from_tiles(int D, const BwdArgsV& a, void* dq, int d, int Zq, hipStream_t s, int variant = 0);

// Stand-alone decay bias (affinity scores): aff [Z][L][L] in the dtype; working tensors tiled like the fused operator's.
hipError_t launch_aff_fwd(int dtype, int D, const void* Kp, const float* lsrc, const float* ldest, void* aff, int L, int Lp, int Z,
                          hipStream_t s, int pair = 0);
// DL [Z][L][L] float scratch; row, colp [Z][Lp][D] and gs_row, gs_col [Z][Lp] float scratch; src, dest: the caller's gates.
// Wst (bf16, L a multiple of 8, daff 16-byte aligned): [Z][tri_tiles(Lp/32)][1 KB] scratch that replaces DL and gs_col
hipError_t launch_aff_bwd(int dtype, int D, const void* Kp, const void* KT, const float* lsrc, const float* ldest, const void* daff,
                          float* DL, float* row, float* colp, float* gs_row, float* gs_col, const void* src, const void* dest,
                          void* dk, void* dsrc, void* ddest, int L, int Lp, int d, int Z, hipStream_t s, void* Wst = nullptr, int pair = 0);

}  // namespace ua
