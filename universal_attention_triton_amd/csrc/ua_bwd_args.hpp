// Typed view of the type-erased argument block of the backward kernels.
#pragma once
#include "ua_bwd.hpp"
#include "ua_internal.hpp"

namespace ua {

template <class T>
static BwdArgs<T> typed(const BwdArgsV& v) {
  BwdArgs<T> a;
  a.reach = v.reach; a.minkey = v.minkey; a.masked_nz = v.masked_nz;
  a.Kp = (const T*)v.Kp; a.Vp = (const T*)v.Vp; a.KT = (const T*)v.KT; a.Qp = (const T*)v.Qp; a.QT = (const T*)v.QT;
  a.dOp = (const T*)v.dOp; a.dOT = (const T*)v.dOT; a.lsrc = v.lsrc; a.ldest = v.ldest; a.lse2 = v.lse2; a.delta = v.delta;
  a.C = v.C;
  a.dS_st = (T*)v.dS_st; a.dG_st = (T*)v.dG_st; a.Bt = (const _Float16*)v.Bt;
  a.dQacc = v.dQacc; a.dKdacc = v.dKdacc; a.Dsuf = v.Dsuf; a.dKrow = v.dKrow; a.dVrow = v.dVrow; a.dsrc_raw = v.dsrc_raw;
  a.R = v.R; a.L = v.L; a.Lp = v.Lp; a.c = v.c; a.nch = v.nch; a.chunked = v.chunked; a.skip_masked = v.skip_masked; a.split_r = v.split_r; a.key_parts = v.key_parts > 0 ? v.key_parts : 1;
  a.direct = v.direct; a.d_out = v.d_out; a.dk_out = (T*)v.dk_out; a.dv_out = (T*)v.dv_out; a.dsrc_out = (T*)v.dsrc_out;
  a.ddest_out = (T*)v.ddest_out; a.src_in = (const T*)v.src_in; a.dest_in = (const T*)v.dest_in;
  a.dO_rows = v.dO_rows;
  return a;
}


}  // namespace ua
