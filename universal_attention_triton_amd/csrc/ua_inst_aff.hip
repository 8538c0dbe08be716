// Instantiations and launchers of the stand-alone decay-bias (affinity scores) kernels.
#include "ua_affinity.hpp"
#include "ua_internal.hpp"

namespace ua {

// explicit instantiations (the implicit ones are not emitted on the host side for kernels holding lambdas)
#define UA_INST(T, D)                                                                                                   \
  template __global__ void k_aff_fwd<T, D>(const T*, const float*, const float*, T*, int, int, int);                          \
  template __global__ void k_aff_bwd_side<T, D, false>(const T*, const T*, const float*, const float*, const float*, float*, \
                                                       float*, int, int);                                                \
  template __global__ void k_aff_bwd_side<T, D, true>(const T*, const T*, const float*, const float*, const float*, float*,  \
                                                      float*, int, int);
UA_INST(bf16, 64) UA_INST(bf16, 128) UA_INST(float, 64) UA_INST(float, 128)
#undef UA_INST
#define UA_INST(D)                                                                                                     \
  template __global__ void k_aff_bwd_keys<bf16, D>(const bf16*, const bf16*, const float*, const float*, const bf16*, bf16*, \
                                                   float*, float*, int, int);                                         \
  template __global__ void k_aff_bwd_cols<bf16, D>(const bf16*, const bf16*, float*, int, int);
UA_INST(64) UA_INST(128)
#undef UA_INST

// Launches of more workgroups than CUs give every workgroup two key groups of complementary length (the kernels see it
// from the grid): equal workgroups, half as many workgroup changes.  Launches that fit the CUs at once keep one group
// per workgroup.  (Measured on L = 4096 with 8 to 16 heads: several unequal workgroups per CU are the slowest form.)
static int paired_groups(int n_kg, int Z, int pair) { return paired_items(n_kg, (long)n_kg * Z > device_cus(), pair); }

template <class T, int D>
static hipError_t aff_fwd_t(const void* Kp, const float* lsrc, const float* ldest, void* aff, int L, int Lp, int Z, hipStream_t s, int pair) {
  const int vec = ((uintptr_t)aff % 16 == 0 && L % (16 / (int)sizeof(T)) == 0) ? 1 : 0;      // rows start 16-byte aligned
  hipLaunchKernelGGL((k_aff_fwd<T, D>), dim3(paired_groups(Lp / 128, Z, pair), Z), dim3(512), 0, s, (const T*)Kp, lsrc, ldest, (T*)aff, L, Lp, vec);
  return hipGetLastError();
}
hipError_t launch_aff_fwd(int dtype, int D, const void* Kp, const float* lsrc, const float* ldest, void* aff, int L, int Lp, int Z,
                          hipStream_t s, int pair) {
#define UA_ARGS Kp, lsrc, ldest, aff, L, Lp, Z, s, pair
  if (dtype == 1) return D == 64 ? aff_fwd_t<bf16, 64>(UA_ARGS) : aff_fwd_t<bf16, 128>(UA_ARGS);
  return D == 64 ? aff_fwd_t<float, 64>(UA_ARGS) : aff_fwd_t<float, 128>(UA_ARGS);
#undef UA_ARGS
}

template <class T, int D>
static hipError_t aff_bwd_t(const void* Kp, const void* KT, const float* lsrc, const float* ldest, const void* daff, float* DL,
                            float* row, float* colp, float* gs_row, float* gs_col, const void* src, const void* dest, void* dk,
                            void* dsrc, void* ddest, int L, int Lp, int d, int Z, hipStream_t s, void* Wst, int pair) {
  hipError_t e;
  if constexpr (sizeof(T) == 2) {
    if (Wst) {      // rows of daff 16-byte aligned: the gradient W travels as bf16 tiles instead of the float L x L tensor
      hipLaunchKernelGGL((k_aff_bwd_keys<T, D>), dim3(paired_groups(Lp / 128, Z, pair), Z), dim3(512), 0, s, (const T*)Kp, (const T*)KT, lsrc, ldest,
                         (const T*)daff, (T*)Wst, row, gs_row, L, Lp);
      if ((e = hipGetLastError()) != hipSuccess) return e;
      hipLaunchKernelGGL((k_aff_bwd_cols<T, D>), dim3(paired_groups(Lp / 128, Z, pair), Z), dim3(512), 0, s, (const T*)KT, (const T*)Wst, colp, L, Lp);
      if ((e = hipGetLastError()) != hipSuccess) return e;
      hipLaunchKernelGGL((k_aff_finish<T>), dim3((L + 3) / 4, Z), dim3(256), 0, s, (const float*)row, (const float*)colp,
                         (const float*)gs_row, (const float*)nullptr, (const T*)src, (const T*)dest, (T*)dk, (T*)dsrc, (T*)ddest, L,
                         Lp, D, d, (const T*)Kp);
      return hipGetLastError();
    }
  }
  hipLaunchKernelGGL((k_aff_revcumsum<T>), dim3((L + 255) / 256, Z), dim3(256), 0, s, (const T*)daff, DL, L);
  if ((e = hipGetLastError()) != hipSuccess) return e;
  hipLaunchKernelGGL((k_aff_bwd_side<T, D, false>), dim3(Lp / 128, Z), dim3(512), 0, s, (const T*)Kp, (const T*)KT, lsrc, ldest,
                     (const float*)DL, row, gs_row, L, Lp);
  if ((e = hipGetLastError()) != hipSuccess) return e;
  hipLaunchKernelGGL((k_aff_bwd_side<T, D, true>), dim3(Lp / 128, Z), dim3(512), 0, s, (const T*)Kp, (const T*)KT, lsrc, ldest,
                     (const float*)DL, colp, gs_col, L, Lp);
  if ((e = hipGetLastError()) != hipSuccess) return e;
  hipLaunchKernelGGL((k_aff_finish<T>), dim3((L + 3) / 4, Z), dim3(256), 0, s, (const float*)row, (const float*)colp,
                     (const float*)gs_row, (const float*)gs_col, (const T*)src, (const T*)dest, (T*)dk, (T*)dsrc, (T*)ddest, L, Lp,
                     D, d, (const T*)Kp);
  return hipGetLastError();
}
hipError_t launch_aff_bwd(int dtype, int D, const void* Kp, const void* KT, const float* lsrc, const float* ldest, const void* daff,
                          float* DL, float* row, float* colp, float* gs_row, float* gs_col, const void* src, const void* dest,
                          void* dk, void* dsrc, void* ddest, int L, int Lp, int d, int Z, hipStream_t s, void* Wst, int pair) {
#define UA_ARGS Kp, KT, lsrc, ldest, daff, DL, row, colp, gs_row, gs_col, src, dest, dk, dsrc, ddest, L, Lp, d, Z, s, Wst, pair
  if (dtype == 1) return D == 64 ? aff_bwd_t<bf16, 64>(UA_ARGS) : aff_bwd_t<bf16, 128>(UA_ARGS);
  return D == 64 ? aff_bwd_t<float, 64>(UA_ARGS) : aff_bwd_t<float, 128>(UA_ARGS);
#undef UA_ARGS
}

}  // namespace ua
