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
from . import universal_attention_autograd as _chunked
from .universal_attention_autograd import _ChunkedBase


class _CheckedChunked2D(_ChunkedBase):
    @staticmethod
    def forward(kc, vc, xq, static_src, static_dest):
        b, h, r, _n, _c, d = xq.shape
        _, _, n_, c_, _ = kc.shape
        assert kc.shape == (b, h, n_, c_, d)
        assert vc.shape == (b, h, n_, c_, d)
        assert static_src.shape == (b, h, n_, c_)
        assert static_dest.shape == (b, h, _n, _c)
        return _ChunkedBase.forward(kc, vc, xq, static_src, static_dest)

    @staticmethod
    def backward(ctx, dout, ddenom, _dstate=None):
        kc, vc, xq = ctx.saved_tensors[:3]
        b, h, r, _n, _c, d = xq.shape
        _, _, n_, c_, _ = kc.shape
        assert dout.shape == (b, h, r, n_ * c_, d, n_)
        assert ddenom.shape == (b, h, r, n_ * c_, n_)
        return _ChunkedBase.backward(ctx, dout, ddenom)


class UniversalAttention(_chunked.UniversalAttention):
    """.apply(kc, vc, xq, static_src, static_dest) -> (out, denom), 2-D query layout, with the reference entry point's
    shape checks (Universal_Attention/universal_attention.py:8-13, :35-38)."""
    function = _CheckedChunked2D


_fused_bwd = _chunked.kernel_call(lambda *a: ops.fused_backward(*a[:8], state=a[8], prune=a[9], recompute=a[10]), "FusedBackward")


class _FusedUniversalAttention(Function):
    @staticmethod
    def forward(kc, vc, xq, static_src, static_dest, prune=False, recompute=False, keep_state=True):
        # the forward state (packed inputs + bias tiles) is kept for the backward unless the caller asks for the
        # reference's footprint (its five inputs, plus O and lse here)
        keep = keep_state and not recompute and any(t.requires_grad for t in (kc, vc, xq, static_src, static_dest))
        O, lse, state = ops.fused_forward(kc, vc, xq, static_src, static_dest, keep_state=keep, prune=prune, recompute=recompute)
        if state is None:
            state = torch.empty(0, dtype=torch.uint8, device=O.device)
        return O.view(*xq.shape), lse, state

    @staticmethod
    def setup_context(ctx, inputs, output):
        kc, vc, xq, static_src, static_dest, prune, recompute, _ = inputs
        O, lse, state = output
        ctx.prune, ctx.recompute = prune, recompute
        # the forward state travels as a third, non-differentiable output that universal_attention() drops
        ctx.save_for_backward(kc, vc, xq, static_src, static_dest, O, lse, state)
        ctx.mark_non_differentiable(lse, state)
        # no zero "gradients" are to be made up for lse and the state (a fill of the state's size per backward otherwise)
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, dO, _dlse, _dstate=None):
        kc, vc, xq, static_src, static_dest, O, lse, state = ctx.saved_tensors
        if dO is None:
            return (None,) * 8
        b, h, n, c, d = kc.shape
        r = xq.shape[2]
        dO = dO.reshape(b, h, r, n * c, d)
        dk, dv, dq, dsrc, ddest = _fused_bwd.apply(kc, vc, xq, static_src, static_dest, O.reshape(b, h, r, n * c, d), lse, dO,
                                                   state, ctx.prune, ctx.recompute)
        return dk, dv, dq.view(xq.shape), dsrc.view(static_src.shape), ddest.view(static_dest.shape), None, None, None


def universal_attention(kc, vc, xq, static_src, static_dest, return_lse=False, prune=False, recompute=False, keep_state=True):
    """Fused forward/backward.  Accepts the 1-D (xq [b,h,r,l,d]) and the 2-D (xq [b,h,r,_n,_c,d]) layouts;
    the result has xq's shape.  prune=True skips (key, query) pairs whose softmax weight is provably below 2^-48
    because of the accumulated decay: same results to float32 rounding, less work on long sequences.

    Memory between forward and backward: by default the forward state (packed inputs and, for bf16, the bias tiles: about
    Lp*Lp bytes per kv head, ops.retained_bytes) stays alive until the backward, whose scratch is allocated there.
    keep_state=False keeps nothing but the five inputs, O and lse, as the reference does
    (Universal_Attention/universal_attention.py:27-31); the backward then rebuilds the state first.
    recompute=True (bf16) implies that and also keeps the backward's workspace at O(L*L/16) bytes per head by
    recomputing the score and decay gradients in every kernel instead of exchanging tiles (UA_FLAG_RECOMPUTE)."""
    ops.autotune_on_first_call(kc, vc, xq, static_src, static_dest)          # only with UA_AUTOTUNE=1
    O, lse, _state = _FusedUniversalAttention.apply(kc, vc, xq, static_src, static_dest, prune, recompute, keep_state)
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
    # ac ("activation checkpointing" of the reference: do not keep the bias between forward and backward,
    # universal_attention_kernel_opt.py:494-497, :551-553) = keep no forward state here
    O = universal_attention(k.unsqueeze(2), v.unsqueeze(2), xq, static_src.unsqueeze(2), static_dest, keep_state=not ac)
    return O.transpose(1, 2).reshape(B, Hq, L, d)
