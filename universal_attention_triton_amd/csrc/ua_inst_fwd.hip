// Instantiations and launchers of the forward kernels.
#include <algorithm>
#include <cstdint>
#include <cstdlib>
#include "ua_fused.hpp"
#include "ua_fwd.hpp"
#include "ua_internal.hpp"

namespace ua {

template <class K>
static void allow_lds(K kernel, size_t bytes) {
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

template <class T, int D>
static hipError_t carry_t(const void* Kp, const float* lsrc, const float* ldest, float* C, int Lp, int Zk, int tiled,
                          const float* knorm2, const float* qnorm2, int R, int* reach, int* minkey, hipStream_t s, void* Bt,
                          int variant) {
  constexpr int NST = 2;
  _Float16* none = nullptr;
  // bias tiles, variant 1: 4-wave workgroups (launches of under two 8-wave workgroups per CU are bound by the latency
  // of a workgroup's serial sweep and run faster as twice as many 4-wave workgroups)
  // variant 2: the same with two key groups per workgroup (half the workgroups; pays in small launches)
  if (tiled && Bt && sizeof(T) == 2 && (variant == 1 || variant == 2))
    hipLaunchKernelGGL((k_carry2<T, D, NST, true, true, 4>), dim3(variant == 2 ? (Lp / 64 + 1) / 2 : Lp / 64, Zk), dim3(256), 0, s, (const T*)Kp, lsrc, ldest, C, Lp, knorm2, qnorm2, R, reach, (_Float16*)Bt);
  else if (tiled && Bt && sizeof(T) == 2) hipLaunchKernelGGL((k_carry2<T, D, NST, true, true>), dim3(Lp / 128, Zk), dim3(512), 0, s, (const T*)Kp, lsrc, ldest, C, Lp, knorm2, qnorm2, R, reach, (_Float16*)Bt);
  else if constexpr (D == 256) return hipErrorInvalidValue;
  else if (tiled) hipLaunchKernelGGL((k_carry2<T, D, NST, true, false>), dim3(Lp / 128, Zk), dim3(512), 0, s, (const T*)Kp, lsrc, ldest, C, Lp, knorm2, qnorm2, R, reach, none);
  else hipLaunchKernelGGL((k_carry2<T, D, NST, false, false>), dim3(Lp / 128, Zk), dim3(512), 0, s, (const T*)Kp, lsrc, ldest, C, Lp, knorm2, qnorm2, R, reach, none);
  hipError_t e = hipGetLastError();
  if (e == hipSuccess && reach && minkey) {
    hipLaunchKernelGGL((k_minkey<>), dim3((Lp / 32 + 255) / 256, Zk), dim3(256), 0, s, (const int*)reach, minkey, Lp / 16);
    e = hipGetLastError();
  }
  return e;
}
hipError_t launch_carry(int dtype, int D, const void* Kp, const float* lsrc, const float* ldest, float* C, int Lp, int Zk,
                        int tiled, const float* knorm2, const float* qnorm2, int R, int* reach, int* minkey, hipStream_t s,
                        void* Bt, int variant) {
#define UA_ARGS Kp, lsrc, ldest, C, Lp, Zk, tiled, knorm2, qnorm2, R, reach, minkey, s, Bt, variant
  if (D == 256) return (dtype == 1 && tiled && Bt) ? carry_t<bf16, 256>(UA_ARGS) : hipErrorInvalidValue;   // bias tiles only
  if (dtype == 1) return D == 64 ? carry_t<bf16, 64>(UA_ARGS) : carry_t<bf16, 128>(UA_ARGS);
  return D == 64 ? carry_t<float, 64>(UA_ARGS) : carry_t<float, 128>(UA_ARGS);
#undef UA_ARGS
}

// explicit instantiations (the implicit ones are not emitted on the host side for these kernels)
#define UA_INST3(T, D, NST, NW, CH, BI, RB)                                                                             \
  template __global__ void k_fwd_fused2<T, D, NST, NW, CH, BI, RB>(const T*, const T*, const T*, const float*, const float*, \
                                                               const float*, T*, float*, float*, const int*, const int*, \
                                                               int, int, int, int, ChunkOut<T>, const _Float16*);
#define UA_INST2(T, D, NST, NW, CH, BI) UA_INST3(T, D, NST, NW, CH, BI, 1)
#define UA_INST(T, D, NST, NW, CH) UA_INST2(T, D, NST, NW, CH, false)
UA_INST3(bf16, 64, 1, 8, false, true, 2) UA_INST3(bf16, 128, 1, 8, false, true, 2) UA_INST3(bf16, 64, 1, 8, false, true, 4) UA_INST3(bf16, 128, 1, 8, false, true, 4)
UA_INST3(bf16, 256, 1, 8, false, true, 2) UA_INST3(bf16, 256, 1, 8, false, true, 4) UA_INST2(bf16, 256, 1, 8, false, true)
UA_INST2(bf16, 64, 1, 8, false, true) UA_INST2(bf16, 128, 1, 8, false, true) UA_INST2(bf16, 64, 1, 4, false, true) UA_INST2(bf16, 128, 1, 4, false, true)
template __global__ void k_fwd_fused3<64, 1>(const bf16*, const bf16*, const bf16*, bf16*, float*, float*, const int*, const int*, int, int, int, int, const _Float16*);
template __global__ void k_fwd_fused3<64, 2>(const bf16*, const bf16*, const bf16*, bf16*, float*, float*, const int*, const int*, int, int, int, int, const _Float16*);
template __global__ void k_fwd_fused3<64, 4>(const bf16*, const bf16*, const bf16*, bf16*, float*, float*, const int*, const int*, int, int, int, int, const _Float16*);
template __global__ void k_fwd_fused3<128, 1>(const bf16*, const bf16*, const bf16*, bf16*, float*, float*, const int*, const int*, int, int, int, int, const _Float16*);
template __global__ void k_fwd_fused3<128, 2>(const bf16*, const bf16*, const bf16*, bf16*, float*, float*, const int*, const int*, int, int, int, int, const _Float16*);
template __global__ void k_fwd_fused3<128, 4>(const bf16*, const bf16*, const bf16*, bf16*, float*, float*, const int*, const int*, int, int, int, int, const _Float16*);
UA_INST(bf16, 64, 1, 8, false) UA_INST(bf16, 64, 2, 8, false) UA_INST(bf16, 64, 2, 12, false) UA_INST(bf16, 64, 2, 16, false)
UA_INST(bf16, 128, 2, 4, false) UA_INST(bf16, 64, 2, 4, false) UA_INST(bf16, 128, 1, 8, false) UA_INST(bf16, 128, 2, 8, false) UA_INST(bf16, 128, 2, 12, false) UA_INST(bf16, 128, 2, 16, false)
UA_INST(float, 64, 1, 8, false) UA_INST(float, 128, 1, 8, false)
UA_INST(bf16, 64, 2, 8, true) UA_INST(bf16, 128, 2, 8, true) UA_INST(float, 64, 1, 8, true) UA_INST(float, 128, 1, 8, true)
#undef UA_INST
#undef UA_INST2
#undef UA_INST3

template <class T, int D, int NST, int NW>
static hipError_t fused_t(const void* Qp, const void* Kp, const void* VT, const float* lsrc, const float* ldest,
                          const float* C, void* O, float* lse, float* lse2, const int* reach, const int* minkey, int R, int L,
                          int Lp, int d, int Zq, hipStream_t s) {
  const _Float16* none = nullptr;
  hipLaunchKernelGGL((k_fwd_fused2<T, D, NST, NW, false>), dim3((Lp / 16 + NW - 1) / NW, Zq), dim3(64 * NW), 0, s, (const T*)Qp,
                     (const T*)Kp, (const T*)VT, lsrc, ldest, C, (T*)O, lse, lse2, reach, minkey, R, L, Lp, d, ChunkOut<T>{}, none);
  return hipGetLastError();
}
// bf16 with bias tiles from launch_carry; variant: UA_TUNE_FWD_TILES
//   0: k_fwd_fused3, one 32-query block per wave (256-query workgroups, two LDS stages)
//   1: k_fwd_fused2<BI>, 8-wave workgroups of 128 queries with a single LDS stage, two per CU, which cover each other's waits
//   2: the same in 64-query pieces (r = 1; small launches are bound by their longest workgroups)
// grouped queries: the groups of a kv head share the tiles of a 32-query block (see RB)
template <int D>
static hipError_t fused_bi(int variant, const void* Qp, const void* Kp, const void* VT, const float* lsrc, const float* ldest,
                           const float* C, void* O, float* lse, float* lse2, const int* reach, const int* minkey, int R, int L,
                           int Lp, int d, int Zq, hipStream_t s, const void* Bt) {
  using T = bf16;
  if constexpr (D == 256) variant = 1;       // 16 queries per wave: the accumulators of a 32-query block do not fit
  if constexpr (D != 256) if (variant == 0) {
    // two query blocks per workgroup once every CU gets at least two of the single ones
#define UA_F3(RB_)                                                                                                          \
  do {                                                                                                                      \
    const int n_blk_ = (Lp / 32 + 8 / RB_ - 1) / (8 / RB_);                                                                 \
    const int gx_ = (long)n_blk_ * (Zq / RB_) >= 2 * device_cus() ? (n_blk_ + 1) / 2 : n_blk_;                             \
    hipLaunchKernelGGL((k_fwd_fused3<D, RB_>), dim3(gx_, Zq / RB_), dim3(512), 0, s, (const T*)Qp,                          \
                       (const T*)Kp, (const T*)VT, (T*)O, lse, lse2, reach, minkey, R, L, Lp, d, (const _Float16*)Bt);      \
  } while (0)
    if (R % 4 == 0) UA_F3(4);
    else if (R % 2 == 0) UA_F3(2);
    else UA_F3(1);
#undef UA_F3
    return hipGetLastError();
  }
#define UA_SHARED(RB_)                                                                                                     \
  hipLaunchKernelGGL((k_fwd_fused2<T, D, 1, 8, false, true, RB_>), dim3(Lp / (128 / RB_), Zq / RB_), dim3(512), 0, s, (const T*)Qp, \
                     (const T*)Kp, (const T*)VT, lsrc, ldest, C, (T*)O, lse, lse2, reach, minkey, R, L, Lp, d, ChunkOut<T>{},      \
                     (const _Float16*)Bt)
  if (R % 4 == 0) UA_SHARED(4);
  else if (R % 2 == 0) UA_SHARED(2);
  else if (variant == 1 || D == 256)
    hipLaunchKernelGGL((k_fwd_fused2<T, D, 1, 8, false, true>), dim3(Lp / 128, Zq), dim3(512), 0, s, (const T*)Qp, (const T*)Kp,
                       (const T*)VT, lsrc, ldest, C, (T*)O, lse, lse2, reach, minkey, R, L, Lp, d, ChunkOut<T>{}, (const _Float16*)Bt);
  else if constexpr (D != 256)
    hipLaunchKernelGGL((k_fwd_fused2<T, D, 1, 4, false, true>), dim3(Lp / 64, Zq), dim3(256), 0, s, (const T*)Qp, (const T*)Kp,
                       (const T*)VT, lsrc, ldest, C, (T*)O, lse, lse2, reach, minkey, R, L, Lp, d, ChunkOut<T>{}, (const _Float16*)Bt);
#undef UA_SHARED
  return hipGetLastError();
}
// variants (bf16): 0 = 8 waves, double-buffered stages; 1 = 8 waves, single stage; 2 = 12 waves; 3 = 16 waves
// (both double-buffered).  fp32 always runs 8 waves with a single stage.
int fwd_fused_variants(int dtype, int D) { (void)D; return dtype == 1 ? 5 : 1; }
template <class T, int D>
static hipError_t fused_v(int variant, const void* Qp, const void* Kp, const void* VT, const float* lsrc, const float* ldest,
                          const float* C, void* O, float* lse, float* lse2, const int* reach, const int* minkey, int R, int L,
                          int Lp, int d, int Zq, hipStream_t s) {
#define UA_ARGS Qp, Kp, VT, lsrc, ldest, C, O, lse, lse2, reach, minkey, R, L, Lp, d, Zq, s
  switch (variant) {
    case 1: return fused_t<T, D, 1, 8>(UA_ARGS);
    case 2: return fused_t<T, D, 2, 12>(UA_ARGS);
    case 3: return fused_t<T, D, 2, 16>(UA_ARGS);
    case 4: return fused_t<T, D, 2, 4>(UA_ARGS);
    default: return fused_t<T, D, 2, 8>(UA_ARGS);
  }
#undef UA_ARGS
}
hipError_t launch_fwd_fused(int dtype, int D, int variant, const void* Qp, const void* Kp, const void* VT,
                            const float* lsrc, const float* ldest, const float* C, void* O, float* lse, float* lse2,
                            const int* reach, const int* minkey, int R, int L, int Lp, int d, int Zq, hipStream_t s,
                            const void* Bt) {
#define UA_ARGS Qp, Kp, VT, lsrc, ldest, C, O, lse, lse2, reach, minkey, R, L, Lp, d, Zq, s
  if (D == 256) return (dtype == 1 && Bt) ? fused_bi<256>(variant, UA_ARGS, Bt) : hipErrorInvalidValue;
  if (dtype == 1 && Bt) return D == 64 ? fused_bi<64>(variant, UA_ARGS, Bt) : fused_bi<128>(variant, UA_ARGS, Bt);
  if (dtype == 1) return D == 64 ? fused_v<bf16, 64>(variant, UA_ARGS) : fused_v<bf16, 128>(variant, UA_ARGS);
  return D == 64 ? fused_t<float, 64, 1, 8>(UA_ARGS) : fused_t<float, 128, 1, 8>(UA_ARGS);
#undef UA_ARGS
}

// chunked operator through the query-stationary kernel (chunk a multiple of 64; tiled working tensors)
template <class T, int D>
static hipError_t chunked2_t(const void* Qp, const void* Kp, const void* Vp, const void* VT, const float* lsrc, const float* ldest,
                             const float* C, const int* reach, const int* minkey, void* out, void* denom, float* lse2, long o_sz,
                             long o_st, long o_sd, long o_si, int R, int L, int Lp, int d, int c, int nch, int Zq, hipStream_t s, int pair) {
  constexpr int NST = sizeof(T) == 2 ? 2 : 1, NW = 8;
  constexpr long VV = 16 / (long)sizeof(T);
  const int ovec = out && o_sd == 1 && d % VV == 0 && (uintptr_t)out % 16 == 0 && o_sz % VV == 0 && o_st % VV == 0 && o_si % VV == 0;
  ChunkOut<T> co{(T*)out, (T*)denom, o_sz, o_st, o_sd, o_si, c, nch, ovec};
  // two query blocks per workgroup once every CU gets at least four of the single ones
  const int n_blk = (Lp / 16 + NW - 1) / NW, gx = paired_items(n_blk, (long)n_blk * Zq >= 4L * device_cus(), pair);
  hipLaunchKernelGGL((k_fwd_fused2<T, D, NST, NW, true>), dim3(gx, Zq), dim3(64 * NW), 0, s, (const T*)Qp,
                     (const T*)Kp, (const T*)VT, lsrc, ldest, C, (T*)nullptr, (float*)nullptr, lse2, reach, minkey, R, L, Lp, d, co, (const _Float16*)nullptr);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  if (out && nch > 1) {
    const int vec = ovec;
    const int slabs = (std::min((nch - 1) * c, L) + kMaskedSlab - 1) / kMaskedSlab;
    hipLaunchKernelGGL((k_chunk_masked_out<T, D>), dim3(slabs, nch, Zq), dim3(256), 0, s, (const T*)Vp, co, R, L, Lp, d, vec);
    if ((e = hipGetLastError()) != hipSuccess) return e;
  }
  if (nch > 1) {
    hipLaunchKernelGGL((k_chunk_masked_denom<T>), dim3((Lp + 255) / 256, Zq), dim3(256), 0, s, (T*)denom, lse2, L, Lp, c, nch);
    e = hipGetLastError();
  }
  return e;
}
hipError_t launch_fwd_chunked2(int dtype, int D, const void* Qp, const void* Kp, const void* Vp, const void* VT, const float* lsrc,
                               const float* ldest, const float* C, const int* reach, const int* minkey, void* out, void* denom,
                               float* lse2, long o_sz, long o_st, long o_sd, long o_si, int R, int L, int Lp, int d, int c, int nch,
                               int Zq, hipStream_t s, int pair) {
#define UA_ARGS Qp, Kp, Vp, VT, lsrc, ldest, C, reach, minkey, out, denom, lse2, o_sz, o_st, o_sd, o_si, R, L, Lp, d, c, nch, Zq, s, pair
  if (dtype == 1) return D == 64 ? chunked2_t<bf16, 64>(UA_ARGS) : chunked2_t<bf16, 128>(UA_ARGS);
  return D == 64 ? chunked2_t<float, 64>(UA_ARGS) : chunked2_t<float, 128>(UA_ARGS);
#undef UA_ARGS
}

template <class T, int D, int NW>
static hipError_t chunked_t(const void* Qp, const void* Kp, const void* VT, const float* lsrc, const float* ldest, void* out,
                            void* denom, float* lse2, long o_sz, long o_st, long o_sd, long o_si, int R, int L, int Lp,
                            int d, int c, int nch, int Zk, hipStream_t s) {
  const size_t lds = (64 * lds_stride<T>(D) + 32 * lds_stride<T>(32 * NW)) * sizeof(T) + (NW * 32 + D) * sizeof(float);
  allow_lds(k_fwd_chunked<T, D, NW>, lds);
  hipLaunchKernelGGL((k_fwd_chunked<T, D, NW>), dim3(nch, Zk), dim3(64 * NW), lds, s, (const T*)Qp, (const T*)Kp,
                     (const T*)VT, lsrc, ldest, (T*)out, (T*)denom, lse2, o_sz, o_st, o_sd, o_si, R, L, Lp,
                     d, c, nch);
  return hipGetLastError();
}
template <class T, int D>
static hipError_t chunked_nw(int NW, const void* Qp, const void* Kp, const void* VT, const float* lsrc, const float* ldest,
                             void* out, void* denom, float* lse2, long o_sz, long o_st, long o_sd, long o_si, int R, int L,
                             int Lp, int d, int c, int nch, int Zk, hipStream_t s) {
#define UA_ARGS Qp, Kp, VT, lsrc, ldest, out, denom, lse2, o_sz, o_st, o_sd, o_si, R, L, Lp, d, c, nch, Zk, s
  switch (NW) {
    case 1: return chunked_t<T, D, 1>(UA_ARGS);
    case 2: return chunked_t<T, D, 2>(UA_ARGS);
    case 4: return chunked_t<T, D, 4>(UA_ARGS);
    default: return chunked_t<T, D, 8>(UA_ARGS);
  }
#undef UA_ARGS
}
hipError_t launch_fwd_chunked(int dtype, int D, const void* Qp, const void* Kp, const void* VT, const float* lsrc,
                              const float* ldest, void* out, void* denom, float* lse2, long o_sz, long o_st, long o_sd,
                              long o_si, int R, int L, int Lp, int d, int c, int nch, int Zk, hipStream_t s) {
  int NW = c <= 32 ? 1 : c <= 64 ? 2 : c <= 128 ? 4 : 8;
#define UA_ARGS NW, Qp, Kp, VT, lsrc, ldest, out, denom, lse2, o_sz, o_st, o_sd, o_si, R, L, Lp, d, c, nch, Zk, s
  if (dtype == 1) return D == 64 ? chunked_nw<bf16, 64>(UA_ARGS) : chunked_nw<bf16, 128>(UA_ARGS);
  return D == 64 ? chunked_nw<float, 64>(UA_ARGS) : chunked_nw<float, 128>(UA_ARGS);
#undef UA_ARGS
}

}  // namespace ua
