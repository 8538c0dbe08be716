"""HIP-backed operators with the interface of the reference's torch operators
(reference universal_attention_autograd.py): same class names, argument order, shapes and dtypes.

    UniversalAttention.apply(kc, vc, xq, static_src, static_dest) -> (out, denom)      ref :7-99
        kc, vc [b,h,n,c,d]; xq [b,h,r,l,d]; static_src [b,h,n,c]; static_dest [b,h,l]
        out [b,h,r,l,d,n], denom [b,h,r,l,n] in xq.dtype
    UniversalAttention2.apply(...)   same with xq [b,h,r,_n,_c,d], static_dest [b,h,_n,_c]  ref :102-276
    SMVecMatMul.apply(mat[...,d,n], vec[...,n]) -> [...,d]                              ref :278-297

`out` is returned with chunk-major storage (a permuted view): its values and shape are the
reference's, its strides are not.  All compute happens in libua_hip.so; tensors must live on the GPU.
"""
import torch
from torch.autograd import Function

from . import ops


class _ChunkedBase(Function):
    # gradients of (query, chunk) pairs whose query precedes the chunk are propagated exactly as the
    # reference does; set to True only when the upstream gradient is known to vanish there
    skip_masked = False
    # bf16, chunk a multiple of 64: True keeps the backward's workspace small (UA_FLAG_RECOMPUTE: its second kernel
    # recomputes the score and decay gradients instead of reading them from 2*L*L bytes per head)
    recompute = False

    @staticmethod
    def forward(ctx, kc, vc, xq, static_src, static_dest):
        need_grad = any(ctx.needs_input_grad)
        out, denom, ws = ops.chunked_forward(kc, vc, xq, static_src, static_dest, for_backward=need_grad,
                                             recompute=_ChunkedBase.recompute)
        ctx.save_for_backward(kc, vc, xq, static_src, static_dest, out)
        ctx.ws = ws if need_grad else None
        return out, denom

    @staticmethod
    def backward(ctx, g_out, g_denom):
        kc, vc, xq, static_src, static_dest, out = ctx.saved_tensors
        dk, dv, dq, dsrc, ddest = ops.chunked_backward(kc, vc, xq, static_src, static_dest, out, g_out, g_denom,
                                                       ws=ctx.ws, skip_masked=_ChunkedBase.skip_masked,
                                                       recompute=_ChunkedBase.recompute)
        ctx.ws = None
        return dk, dv, dq.view(xq.shape), dsrc.view(static_src.shape), ddest.view(static_dest.shape)


class UniversalAttention(_ChunkedBase):
    """1-D layout: xq [b,h,r,l,d], static_dest [b,h,l]."""

    @staticmethod
    def forward(ctx, kc, vc, xq, static_src, static_dest):
        b, h, r, l, d = xq.shape
        _, _, n, c, _ = kc.shape
        return _ChunkedBase.forward(ctx, kc, vc, xq, static_src, static_dest)


class UniversalAttention2(_ChunkedBase):
    """2-D layout: xq [b,h,r,_n,_c,d], static_dest [b,h,_n,_c]; the query tiling does not change the result."""

    @staticmethod
    def forward(ctx, kc, vc, xq, static_src, static_dest):
        b, h, r, _n, _c, d = xq.shape
        _, _, n_, c_, _ = kc.shape
        return _ChunkedBase.forward(ctx, kc, vc, xq, static_src, static_dest)


class SMVecMatMul(Function):
    @staticmethod
    def forward(ctx, mat, vec):
        ctx.save_for_backward(mat, vec)
        return ops.merge_forward(mat, vec)

    @staticmethod
    def backward(ctx, g):
        mat, vec = ctx.saved_tensors
        return ops.merge_backward(mat, vec, g)
