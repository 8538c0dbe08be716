"""Stand-alone decay bias with the interface of the reference's AffinityScores
(Universal_Attention/triton/affinity_kernel_opt.py:425-450): for callers that hand the bias to a generic attention as an
additive mask (reference _debug.py:123-164).

    aff = AffinityScores.apply(k, src, dest)        k [b,h,l,d]; src, dest [b,h,l]  ->  aff [b,h,l,l] in k.dtype
    aff[b,h,t,s] = sum_{s<u<=t} log(1 - relu(k_s.k_u)^(2/3) (src_s dest_u)^(1/3))  for s < t, 0 for s == t, -1e12 for s > t
"""
from torch.autograd import Function

from . import ops


class AffinityScores(Function):
    @staticmethod
    def forward(k, src, dest):
        return ops.affinity_forward(k, src, dest)

    @staticmethod
    def setup_context(ctx, inputs, outputs):
        k, src, dest = inputs
        ctx.save_for_backward(k, src, dest)

    @staticmethod
    def backward(ctx, daff):
        k, src, dest = ctx.saved_tensors
        if daff is None:
            return None, None, None
        dk, dsrc, ddest = ops.affinity_backward(k, src, dest, daff)
        need = ctx.needs_input_grad
        return (dk if need[0] else None), (dsrc if need[1] else None), (ddest if need[2] else None)


_gen_affinity_scores = AffinityScores.apply
