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
import threading

import torch
from torch.autograd import Function

from . import ops


# forward() has no ctx (new-style Function, like the reference's Triton-backed entry point,
# Universal_Attention/universal_attention.py:5-31); the forward state travels to setup_context through this slot
_handoff = threading.local()


def _put_state(out, state):
    _handoff.item = (out.data_ptr(), state)


def _take_state(out):
    item = getattr(_handoff, "item", None)
    _handoff.item = None
    return item[1] if item is not None and item[0] == out.data_ptr() else None


class _ChunkedBase(Function):
    # gradients of (query, chunk) pairs whose query precedes the chunk are propagated exactly as the
    # reference does; set to True only when the upstream gradient is known to vanish there
    skip_masked = False
    # bf16, chunk a multiple of 64: True keeps the backward's workspace small (UA_FLAG_RECOMPUTE: its second kernel
    # recomputes the score and decay gradients instead of reading them from 2*L*L bytes per head)
    recompute = False
    # What the backward gets from the forward besides the five inputs the reference keeps (universal_attention.py:27-31)
    # and `out`: True (default, like the fused operator): the whole forward state (ua_workspace_bytes(UA_OP_FWD) bytes:
    # packed inputs, decay carries of L * L / 4 bytes per kv head, float32 normalisers; 0.94 GB next to the 4.3 GB of
    # `out` at b=1 h=32 L=8192 d=128 chunk 128), so the backward neither repacks the inputs nor repeats the decay
    # pre-pass; "normalisers": only the
    # per-chunk normalisers in float32, 1/(d+1) of the size of `out`, which spare the backward a second run of the
    # forward kernel; False: nothing.
    keep_state = True
    # `out` is stored chunk-major ([b,h,r,n,L,d]) and returned as a permuted view with the reference's shape and values:
    # every kernel then moves 16 bytes per lane.  True allocates it contiguous like the reference does, for callers
    # that `.view()` it; the passes over it are then several times slower.
    contiguous_out = False

    @staticmethod
    def forward(kc, vc, xq, static_src, static_dest):
        keep = _ChunkedBase.keep_state if any(t.requires_grad for t in (kc, vc, xq, static_src, static_dest)) else False
        out, denom, state = ops.chunked_forward(kc, vc, xq, static_src, static_dest, keep_state=keep,
                                                recompute=_ChunkedBase.recompute,
                                                contiguous_out=_ChunkedBase.contiguous_out)
        _put_state(out, state)
        return out, denom

    @staticmethod
    def setup_context(ctx, inputs, output):
        kc, vc, xq, static_src, static_dest = inputs
        out, _ = output
        # `out` is the tensor the caller holds anyway (SMVecMatMul saves it too): saving it costs no memory
        ctx.save_for_backward(kc, vc, xq, static_src, static_dest, out)
        ctx.state = _take_state(out)

    @staticmethod
    def backward(ctx, g_out, g_denom):
        kc, vc, xq, static_src, static_dest, out = ctx.saved_tensors
        dk, dv, dq, dsrc, ddest = ops.chunked_backward(kc, vc, xq, static_src, static_dest, out, g_out, g_denom,
                                                       state=ctx.state, skip_masked=_ChunkedBase.skip_masked,
                                                       recompute=_ChunkedBase.recompute)
        ctx.state = None
        return dk, dv, dq.view(xq.shape), dsrc.view(static_src.shape), ddest.view(static_dest.shape)


class UniversalAttention(_ChunkedBase):
    """1-D layout: xq [b,h,r,l,d], static_dest [b,h,l]."""

    @staticmethod
    def forward(kc, vc, xq, static_src, static_dest):
        b, h, r, l, d = xq.shape
        _, _, n, c, _ = kc.shape
        return _ChunkedBase.forward(kc, vc, xq, static_src, static_dest)


class UniversalAttention2(_ChunkedBase):
    """2-D layout: xq [b,h,r,_n,_c,d], static_dest [b,h,_n,_c]; the query tiling does not change the result."""

    @staticmethod
    def forward(kc, vc, xq, static_src, static_dest):
        b, h, r, _n, _c, d = xq.shape
        _, _, n_, c_, _ = kc.shape
        return _ChunkedBase.forward(kc, vc, xq, static_src, static_dest)


class SMVecMatMul(Function):
    @staticmethod
    def forward(ctx, mat, vec):
        ctx.save_for_backward(mat, vec)
        return ops.merge_forward(mat, vec)

    @staticmethod
    def backward(ctx, g):
        mat, vec = ctx.saved_tensors
        return ops.merge_backward(mat, vec, g)
