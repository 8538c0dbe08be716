// Instantiations and launcher of the key-stationary backward kernel.
#include "ua_bwd.hpp"
#include "ua_internal.hpp"

namespace ua {

template <class T, int D, int NW>
static hipError_t bwd_t(const BwdArgsV& v, int Zk, hipStream_t s) {
  BwdArgs<T> a;
  a.Kp = (const T*)v.Kp; a.Vp = (const T*)v.Vp; a.KT = (const T*)v.KT; a.Qp = (const T*)v.Qp; a.QT = (const T*)v.QT;
  a.dOp = (const T*)v.dOp; a.dOT = (const T*)v.dOT; a.lsrc = v.lsrc; a.ldest = v.ldest; a.lse2 = v.lse2; a.delta = v.delta;
  a.C = v.C;
  a.dQacc = v.dQacc; a.dKdacc = v.dKdacc; a.dKrow = v.dKrow; a.dVrow = v.dVrow; a.dsrc_raw = v.dsrc_raw;
  a.R = v.R; a.L = v.L; a.Lp = v.Lp; a.c = v.c; a.nch = v.nch; a.chunked = v.chunked; a.skip_masked = v.skip_masked;
  constexpr int CP = 32 * NW;
  const size_t lds = (3 * 32 * lds_stride<T>(D) + 3 * D * lds_stride<T>(32) + 32 * lds_stride<T>(CP)) * sizeof(T) + 64 * sizeof(float);
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(k_bwd_keys<T, D, NW>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  const int groups = v.chunked ? v.nch * ((v.c + CP - 1) / CP) : v.Lp / CP;
  hipLaunchKernelGGL((k_bwd_keys<T, D, NW>), dim3(groups, Zk), dim3(64 * NW), lds, s, a);
  return hipGetLastError();
}
template <class T, int D>
static hipError_t bwd_nw(const BwdArgsV& v, int Zk, hipStream_t s) {
  if (!v.chunked || v.c >= 128) return bwd_t<T, D, 4>(v, Zk, s);
  if (v.c > 32) return bwd_t<T, D, 2>(v, Zk, s);
  return bwd_t<T, D, 1>(v, Zk, s);
}
hipError_t launch_bwd_keys(int dtype, int D, const BwdArgsV& a, int Zk, hipStream_t s) {
  if (dtype == 1) return D == 64 ? bwd_nw<bf16, 64>(a, Zk, s) : bwd_nw<bf16, 128>(a, Zk, s);
  return D == 64 ? bwd_nw<float, 64>(a, Zk, s) : bwd_nw<float, 128>(a, Zk, s);
}

}  // namespace ua
