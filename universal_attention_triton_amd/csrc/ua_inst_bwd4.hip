// Instantiations and launcher of the key-stationary backward kernel on 32x32 tiles.
#include "ua_fused.hpp"
#include "ua_keys4.hpp"
#include "ua_bwd_args.hpp"

namespace ua {


template __global__ void k_bwd_keys4<128>(BwdArgs<bf16>);

hipError_t launch_bwd_keys4(int D, const BwdArgsV& v, int Zk, hipStream_t s) {
  if (!v.dS_st || !v.Bt || v.chunked || v.R != 1 || D != 128) return hipErrorInvalidValue;
  const BwdArgs<bf16> a = typed<bf16>(v);
  // two key groups per workgroup once every CU gets at least two of the single ones
  const int n_kg = v.Lp / 128, gx = paired_items(n_kg, (long)n_kg * Zk >= 2 * device_cus(), 0);
  hipLaunchKernelGGL((k_bwd_keys4<128>), dim3(gx, Zk), dim3(256), 0, s, a);
  return hipGetLastError();
}

}  // namespace ua
