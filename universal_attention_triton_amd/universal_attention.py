"""Entry points with the interface of the reference's Triton-backed module
(reference Universal_Attention/universal_attention.py:5-46), plus the fused operator.

    UniversalAttention.apply(kc, vc, xq, static_src, static_dest) -> (out, denom)
        kc, vc [b,h,n_,c_,d]; xq [b,h,r,_n,_c,d]; static_src [b,h,n_,c_]; static_dest [b,h,_n,_c]
        shape mismatches raise AssertionError, a wrong rank raises ValueError (tuple unpacking), as there.
    universal_attention(kc, vc, xq, static_src, static_dest) -> O [b,h,r,l,d]
        == SMVecMatMul(UniversalAttention(...)) without the per-chunk tensor (fused kernels).
    attention(q, k, v, causal, sm_scale, static_src, static_dest) -> o
        the (q,k,v) calling convention of the reference's second-generation kernel
        (Universal_Attention/triton/universal_attention_kernel_opt.py:433-583).
"""
import torch
from torch.autograd import Function

from . import ops
from .universal_attention_autograd import _ChunkedBase


class UniversalAttention(_ChunkedBase):
    @staticmethod
    def forward(ctx, kc, vc, xq, static_src, static_dest):
        b, h, r, _n, _c, d = xq.shape
        _, _, n_, c_, _ = kc.shape
        assert kc.shape == (b, h, n_, c_, d)
        assert vc.shape == (b, h, n_, c_, d)
        assert static_src.shape == (b, h, n_, c_)
        assert static_dest.shape == (b, h, _n, _c)
        return _ChunkedBase.forward(ctx, kc, vc, xq, static_src, static_dest)

    @staticmethod
    def backward(ctx, dout, ddenom):
        kc, vc, xq = ctx.saved_tensors[:3]
        b, h, r, _n, _c, d = xq.shape
        _, _, n_, c_, _ = kc.shape
        assert dout.shape == (b, h, r, n_ * c_, d, n_)
        assert ddenom.shape == (b, h, r, n_ * c_, n_)
        return _ChunkedBase.backward(ctx, dout, ddenom)


class _FusedUniversalAttention(Function):
    @staticmethod
    def forward(ctx, kc, vc, xq, static_src, static_dest, prune=False, recompute=False):
        need_grad = any(ctx.needs_input_grad)
        O, lse, ws = ops.fused_forward(kc, vc, xq, static_src, static_dest, for_backward=need_grad, prune=prune,
                                       recompute=recompute)
        ctx.prune, ctx.recompute = prune, recompute
        ctx.save_for_backward(kc, vc, xq, static_src, static_dest, O, lse)
        ctx.ws = ws if need_grad else None
        ctx.mark_non_differentiable(lse)
        return O.view(*xq.shape), lse

    @staticmethod
    def backward(ctx, dO, _dlse):
        kc, vc, xq, static_src, static_dest, O, lse = ctx.saved_tensors
        b, h, n, c, d = kc.shape
        dO = dO.reshape(b, h, xq.shape[2], n * c, d)
        dk, dv, dq, dsrc, ddest = ops.fused_backward(kc, vc, xq, static_src, static_dest, O, lse, dO, ws=ctx.ws, prune=ctx.prune,
                                                     recompute=ctx.recompute)
        ctx.ws = None
        return dk, dv, dq.view(xq.shape), dsrc.view(static_src.shape), ddest.view(static_dest.shape), None, None


def universal_attention(kc, vc, xq, static_src, static_dest, return_lse=False, prune=False, recompute=False):
    """Fused forward/backward.  Accepts the 1-D (xq [b,h,r,l,d]) and the 2-D (xq [b,h,r,_n,_c,d]) layouts;
    the result has xq's shape.  prune=True skips (key, query) pairs whose softmax weight is provably below 2^-48
    because of the accumulated decay: same results to float32 rounding, less work on long sequences.
    recompute=True (bf16): the backward keeps its workspace at O(L*L/16) bytes per head by recomputing the score and
    decay gradients in its second kernel instead of exchanging them through 2*L*L bytes per head (UA_FLAG_RECOMPUTE)."""
    O, lse = _FusedUniversalAttention.apply(kc, vc, xq, static_src, static_dest, prune, recompute)
    return (O, lse) if return_lse else O


def attention(q, k, v, causal=True, sm_scale=None, static_src=None, static_dest=None, warp_specialize=True, ac=False):
    """q [B,H_q,L,d], k,v [B,H_kv,L,d], static_src/static_dest [B,H_kv,L] -> o [B,H_q,L,d].

    Query head j uses kv head j % H_kv (reference universal_attention_kernel_opt.py:142).  As in the
    reference kernel, sm_scale is accepted and NOT applied (scores are k.q unscaled, :84-85, :152-153)."""
    assert causal, 'currently, only support causal-autoregressive style generation only.'
    B, Hq, L, d = q.shape
    Hkv = k.shape[1]
    assert Hq % Hkv == 0
    r = Hq // Hkv
    xq = q.view(B, r, Hkv, L, d).transpose(1, 2)                 # [B, H_kv, r, L, d]
    O = universal_attention(k.unsqueeze(2), v.unsqueeze(2), xq, static_src.unsqueeze(2), static_dest)
    return O.transpose(1, 2).reshape(B, Hq, L, d)
