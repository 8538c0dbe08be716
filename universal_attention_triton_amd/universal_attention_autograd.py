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
import contextlib
import contextvars

import torch
from torch.autograd import Function

from . import ops


# Options of the chunked operators.  They are read when a Function is applied (in the caller's thread / context) and
# stay with that call: its backward uses the values its forward saw, whatever is set when the backward runs.
#   keep_state      what the backward gets from the forward besides the five inputs the reference keeps
#                   (universal_attention.py:27-31) and `out`: True (default, like the fused operator): the whole forward
#                   state (ua_workspace_bytes(UA_OP_FWD) bytes: packed inputs, decay carries of L * L / 4 bytes per kv
#                   head, float32 normalisers; 0.94 GB next to the 4.3 GB of `out` at b=1 h=32 L=8192 d=128 chunk 128), so
#                   the backward neither repacks the inputs nor repeats the decay pre-pass; "normalisers": only the
#                   per-chunk normalisers in float32, 1/(d+1) of the size of `out`, which spare the backward a second run
#                   of the forward kernel; False: nothing.
#   recompute       bf16, chunk a multiple of 64: True keeps the backward's workspace small (UA_FLAG_RECOMPUTE: its second
#                   kernel recomputes the score and decay gradients instead of reading them from 2*L*L bytes per head).
#   skip_masked     gradients of (query, chunk) pairs whose query precedes the chunk are propagated exactly as the
#                   reference does; True only when the upstream gradient is known to vanish there.
#   contiguous_out  `out` is stored chunk-major ([b,h,r,n,L,d]) and returned as a permuted view with the reference's shape
#                   and values: every kernel then moves 16 bytes per lane.  True allocates it contiguous like the
#                   reference does, for callers that `.view()` it; the passes over it are then several times slower.
_DEFAULTS = {"keep_state": True, "recompute": False, "skip_masked": False, "contiguous_out": False}
_options = contextvars.ContextVar("ua_chunked_options", default=_DEFAULTS)


@contextlib.contextmanager
def chunked_options(**kw):
    """with chunked_options(keep_state="normalisers", recompute=True): out, denom = UniversalAttention.apply(...)

    Applies to the Functions applied inside the block, in this thread (or asyncio task) only; blocks nest."""
    unknown = set(kw) - set(_DEFAULTS)
    if unknown:
        raise TypeError("unknown option(s) %s; known: %s" % (sorted(unknown), sorted(_DEFAULTS)))
    token = _options.set({**_options.get(), **kw})
    try:
        yield
    finally:
        _options.reset(token)


def kernel_call(fn, name):
    """fn(*args) -> tuple of tensors, as a Function without a backward of its own.  The hand-written backward passes are
    applied through one: under torch.func transforms a backward() receives wrapped tensors, and applying a Function is
    what hands the kernels the plain tensors underneath (outside of transforms it costs nothing: no graph is recorded
    while a backward runs)."""
    def forward(*args):
        return fn(*args)

    def setup_context(ctx, inputs, output):
        pass

    def backward(ctx, *grads):
        raise RuntimeError("%s: the hand-written backward passes of Universal Attention are not differentiable "
                           "(the reference's are not either)" % name)

    return type(name, (Function,), {"forward": staticmethod(forward), "setup_context": staticmethod(setup_context),
                                    "backward": staticmethod(backward)})


_chunked_bwd = kernel_call(lambda *a: ops.chunked_backward(*a[:8], state=a[8], skip_masked=a[9], recompute=a[10]), "ChunkedBackward")
_merge_bwd = kernel_call(lambda mat, vec, g: ops.merge_backward(mat, vec, g), "MergeBackward")


class _ChunkedBase(Function):
    """forward() has no ctx (new-style Function, like the reference's Triton-backed entry point,
    Universal_Attention/universal_attention.py:5-31), so torch.func transforms apply.  The forward state reaches the
    backward as a third, non-differentiable output; the public classes' apply() does not hand it to the caller."""

    @staticmethod
    def forward(kc, vc, xq, static_src, static_dest):
        opt = _options.get()
        keep = opt["keep_state"] if any(t.requires_grad for t in (kc, vc, xq, static_src, static_dest)) else False
        out, denom, state = ops.chunked_forward(kc, vc, xq, static_src, static_dest, keep_state=keep,
                                                recompute=opt["recompute"], contiguous_out=opt["contiguous_out"])
        if state is None:
            state = torch.empty(0, dtype=torch.uint8, device=out.device)
        return out, denom, state

    @staticmethod
    def setup_context(ctx, inputs, output):
        kc, vc, xq, static_src, static_dest = inputs
        out, _, state = output
        # `out` is the tensor the caller holds anyway (SMVecMatMul saves it too): saving it costs no memory
        ctx.save_for_backward(kc, vc, xq, static_src, static_dest, out, state)
        ctx.mark_non_differentiable(state)
        # no zero "gradient" is to be made up for the state output (it would be a fill of the state's size per backward)
        ctx.set_materialize_grads(False)
        ctx.opt = dict(_options.get())          # same call, same context as forward(): the values it used

    @staticmethod
    def backward(ctx, g_out, g_denom, _g_state=None):
        kc, vc, xq, static_src, static_dest, out, state = ctx.saved_tensors
        if g_out is None and g_denom is None:
            return None, None, None, None, None
        if g_out is None:
            g_out = torch.zeros_like(out)
        if g_denom is None:
            g_denom = torch.zeros(out.shape[:4] + out.shape[5:], dtype=out.dtype, device=out.device)
        dk, dv, dq, dsrc, ddest = _chunked_bwd.apply(kc, vc, xq, static_src, static_dest, out, g_out, g_denom, state,
                                                     ctx.opt["skip_masked"], ctx.opt["recompute"])
        return dk, dv, dq.view(xq.shape), dsrc.view(static_src.shape), ddest.view(static_dest.shape)


class _Chunked1D(_ChunkedBase):
    @staticmethod
    def forward(kc, vc, xq, static_src, static_dest):
        b, h, r, l, d = xq.shape
        _, _, n, c, _ = kc.shape
        return _ChunkedBase.forward(kc, vc, xq, static_src, static_dest)


class _Chunked2D(_ChunkedBase):
    @staticmethod
    def forward(kc, vc, xq, static_src, static_dest):
        b, h, r, _n, _c, d = xq.shape
        _, _, n_, c_, _ = kc.shape
        return _ChunkedBase.forward(kc, vc, xq, static_src, static_dest)


class UniversalAttention:
    """1-D layout: xq [b,h,r,l,d], static_dest [b,h,l].  Used through .apply() like the reference's Function; the
    autograd Function behind it is `function`."""
    function = _Chunked1D

    @classmethod
    def apply(cls, kc, vc, xq, static_src, static_dest):
        out, denom, _state = cls.function.apply(kc, vc, xq, static_src, static_dest)
        return out, denom


class UniversalAttention2(UniversalAttention):
    """2-D layout: xq [b,h,r,_n,_c,d], static_dest [b,h,_n,_c]; the query tiling does not change the result."""
    function = _Chunked2D


class SMVecMatMul(Function):
    @staticmethod
    def forward(mat, vec):
        return ops.merge_forward(mat, vec)

    @staticmethod
    def setup_context(ctx, inputs, output):
        ctx.save_for_backward(*inputs)

    @staticmethod
    def backward(ctx, g):
        mat, vec = ctx.saved_tensors
        return _merge_bwd.apply(mat, vec, g)
