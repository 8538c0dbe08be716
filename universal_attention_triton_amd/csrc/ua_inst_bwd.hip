// Instantiations and launcher of the key-stationary backward kernel.
#include "ua_bwd.hpp"
#include "ua_fused.hpp"
#include "ua_internal.hpp"
#include "ua_bwd_args.hpp"

namespace ua {

template <class T, int D, int NW, bool COLS>
static hipError_t bwd_t(const BwdArgsV& v, int Zk, hipStream_t s) {
  const BwdArgs<T> a = typed<T>(v);
  constexpr int CP = 32 * NW;
  const size_t lds = (3 * 32 * lds_stride<T>(D) + 3 * D * lds_stride<T>(32) + 32 * lds_stride<T>(CP)) * sizeof(T) + 64 * sizeof(float);
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(k_bwd_keys<T, D, NW, COLS>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  const int groups = v.chunked ? v.nch * ((v.c + CP - 1) / CP) : v.Lp / CP;
  hipLaunchKernelGGL((k_bwd_keys<T, D, NW, COLS>), dim3(groups, Zk), dim3(64 * NW), lds, s, a);
  return hipGetLastError();
}
// explicit instantiations (the implicit ones are not emitted on the host side for kernels holding lambdas)
#define UA_INST(T, D, NST)                                                          \
  template __global__ void k_bwd_keys2<T, D, NST, false, false, false>(BwdArgs<T>); \
  template __global__ void k_bwd_keys2<T, D, NST, true, false, false>(BwdArgs<T>);  \
  template __global__ void k_bwd_keys2<T, D, NST, false, true, false>(BwdArgs<T>);  \
  template __global__ void k_bwd_keys2<T, D, NST, true, true, false>(BwdArgs<T>);
UA_INST(bf16, 64, 2) UA_INST(bf16, 128, 2) UA_INST(float, 64, 1) UA_INST(float, 128, 1)
#undef UA_INST
template __global__ void k_bwd_keys2<bf16, 64, 2, false, false, true>(BwdArgs<bf16>);
template __global__ void k_bwd_keys2<bf16, 64, 2, true, false, true>(BwdArgs<bf16>);
template __global__ void k_bwd_keys2<bf16, 128, 2, false, false, true>(BwdArgs<bf16>);
template __global__ void k_bwd_keys2<bf16, 128, 2, true, false, true>(BwdArgs<bf16>);
template __global__ void k_bwd_keys2<bf16, 256, 2, false, false, true>(BwdArgs<bf16>);
template __global__ void k_bwd_keys2<bf16, 256, 2, true, false, true>(BwdArgs<bf16>);
template __global__ void k_bwd_keys2<bf16, 64, 2, false, true, true>(BwdArgs<bf16>);
template __global__ void k_bwd_keys2<bf16, 64, 2, true, true, true>(BwdArgs<bf16>);
template __global__ void k_bwd_keys2<bf16, 128, 2, false, true, true>(BwdArgs<bf16>);
template __global__ void k_bwd_keys2<bf16, 128, 2, true, true, true>(BwdArgs<bf16>);

template <class T, int D, int NST, bool MR, bool CH, bool TO>
static hipError_t bwd2_mr(const BwdArgs<T>& a, int Lp, int Zk, hipStream_t s, int pair = 0) {
  // two key groups per workgroup once every CU gets at least two of the single ones
  const int n_kg = Lp / 128, gx = paired_items(n_kg, (long)n_kg * Zk >= 2 * device_cus(), pair);
  hipLaunchKernelGGL((k_bwd_keys2<T, D, NST, MR, CH, TO>), dim3(gx, Zk), dim3(512), 0, s, a);
  return hipGetLastError();
}
template <class T, int D, int NST>
static hipError_t bwd2_t(const BwdArgsV& v, int Zk, hipStream_t s) {
  const BwdArgs<T> a = typed<T>(v);
  if constexpr (sizeof(T) == 2 && D == 128) {
    if (v.dS_st && !v.chunked && v.R == 1 && v.keys_variant == 1) return launch_bwd_keys4(D, v, Zk, s);
  }
  if constexpr (sizeof(T) == 2) {
    if (v.dS_st && !v.chunked)
      return v.R / a.key_parts > 1 ? bwd2_mr<T, D, NST, true, false, true>(a, v.Lp, Zk * a.key_parts, s)
                                   : bwd2_mr<T, D, NST, false, false, true>(a, v.Lp, Zk * a.key_parts, s);
    if (v.dS_st)
      return v.R > 1 ? bwd2_mr<T, D, NST, true, true, true>(a, v.Lp, Zk, s, v.pair) : bwd2_mr<T, D, NST, false, true, true>(a, v.Lp, Zk, s, v.pair);
  }
  if (v.chunked) return v.R > 1 ? bwd2_mr<T, D, NST, true, true, false>(a, v.Lp, Zk, s, v.pair) : bwd2_mr<T, D, NST, false, true, false>(a, v.Lp, Zk, s, v.pair);
  return v.R > 1 ? bwd2_mr<T, D, NST, true, false, false>(a, v.Lp, Zk, s) : bwd2_mr<T, D, NST, false, false, false>(a, v.Lp, Zk, s);
}
template <class T, int D>
static hipError_t bwd_nw(const BwdArgsV& v, int Zk, int cols, hipStream_t s) {
  if (!cols) return bwd2_t<T, D, (sizeof(T) == 2 ? 2 : 1)>(v, Zk, s);
  if (!v.chunked || v.c >= 128) return bwd_t<T, D, 4, true>(v, Zk, s);
  if (v.c > 32) return bwd_t<T, D, 2, true>(v, Zk, s);
  return bwd_t<T, D, 1, true>(v, Zk, s);
}
// head dims above 128: merged bf16 operator with tile exchange only
static hipError_t bwd_keys_256(const BwdArgsV& v, int Zk, hipStream_t s) {
  if (!v.dS_st || v.chunked) return hipErrorInvalidValue;
  const BwdArgs<bf16> a = typed<bf16>(v);
  return v.R / a.key_parts > 1 ? bwd2_mr<bf16, 256, 2, true, false, true>(a, v.Lp, Zk * a.key_parts, s)
                               : bwd2_mr<bf16, 256, 2, false, false, true>(a, v.Lp, Zk * a.key_parts, s);
}
hipError_t launch_bwd_keys(int dtype, int D, const BwdArgsV& a, int Zk, int cols, hipStream_t s) {
  if (D == 256) return (dtype == 1 && !cols) ? bwd_keys_256(a, Zk, s) : hipErrorInvalidValue;
  if (dtype == 1) return D == 64 ? bwd_nw<bf16, 64>(a, Zk, cols, s) : bwd_nw<bf16, 128>(a, Zk, cols, s);
  return D == 64 ? bwd_nw<float, 64>(a, Zk, cols, s) : bwd_nw<float, 128>(a, Zk, cols, s);
}

// explicit instantiations (the implicit ones are not emitted on the host side for this kernel)
#define UA_INST(T, D, NST)                                                      \
  template __global__ void k_bwd_queries2<T, D, NST, false>(BwdArgs<T>, T*, int); \
  template __global__ void k_bwd_queries2<T, D, NST, true>(BwdArgs<T>, T*, int);
UA_INST(bf16, 64, 2) UA_INST(bf16, 128, 2) UA_INST(float, 64, 1) UA_INST(float, 128, 1)
#undef UA_INST

template <class T, int D, int NST>
static hipError_t bwdq_t(const BwdArgsV& v, void* dq, int d, int Zk, hipStream_t s) {
  const BwdArgs<T> a = typed<T>(v);
  const dim3 grid(v.Lp / 128, v.split_r ? Zk * v.R : Zk);
  if (v.chunked) hipLaunchKernelGGL((k_bwd_queries2<T, D, NST, true>), grid, dim3(512), 0, s, a, (T*)dq, d);
  else hipLaunchKernelGGL((k_bwd_queries2<T, D, NST, false>), grid, dim3(512), 0, s, a, (T*)dq, d);
  return hipGetLastError();
}
hipError_t launch_bwd_queries(int dtype, int D, const BwdArgsV& a, void* dq, int d, int Zk, hipStream_t s) {
  if (D == 256) return hipErrorInvalidValue;   // the recomputing query side stops at 128
  if (dtype == 1) return D == 64 ? bwdq_t<bf16, 64, 2>(a, dq, d, Zk, s) : bwdq_t<bf16, 128, 2>(a, dq, d, Zk, s);
  return D == 64 ? bwdq_t<float, 64, 1>(a, dq, d, Zk, s) : bwdq_t<float, 128, 1>(a, dq, d, Zk, s);
}

template __global__ void k_bwd_queries3<bf16, 64, 2, 1>(BwdArgs<bf16>, bf16*, int);
template __global__ void k_bwd_queries3<bf16, 128, 2, 1>(BwdArgs<bf16>, bf16*, int);
template __global__ void k_bwd_queries3<bf16, 64, 2, 2>(BwdArgs<bf16>, bf16*, int);
template __global__ void k_bwd_queries3<bf16, 256, 2, 1>(BwdArgs<bf16>, bf16*, int);
template __global__ void k_bwd_queries3<bf16, 128, 2, 2>(BwdArgs<bf16>, bf16*, int);
hipError_t launch_bwd_queries_from_tiles(int D, const BwdArgsV& v, void* dq, int d, int Zq, hipStream_t s, int variant) {
  const BwdArgs<bf16> a = typed<bf16>(v);
  // steps of 32 keys (two workgroups per CU): four query blocks per workgroup once every CU gets at least eight of the
  // single ones, two once it gets four; steps of 64 keys: one block per workgroup
  const int n_blk = v.Lp / 128;
  const long n_wg = (long)n_blk * Zq;
  const bool half_steps = !(variant == 1 && D != 256);
  const int gx = !half_steps ? n_blk
                 : (n_blk % 4 == 0 && n_wg >= 8L * device_cus()) ? n_blk / 4
                 : n_wg >= 4L * device_cus() ? (n_blk + 1) / 2 : n_blk;
  const dim3 grid(gx, Zq);
#define UA_Q3(D_, HV_) hipLaunchKernelGGL((k_bwd_queries3<bf16, D_, 2, HV_>), grid, dim3(512), 0, s, a, (bf16*)dq, d)
  if (D == 256) UA_Q3(256, 1);              // steps of 32 keys only: a stage of 64 keys would not fit twice
  else if (variant == 1) { if (D == 64) UA_Q3(64, 2); else UA_Q3(128, 2); }
  else { if (D == 64) UA_Q3(64, 1); else UA_Q3(128, 1); }
#undef UA_Q3
  return hipGetLastError();
}

}  // namespace ua
