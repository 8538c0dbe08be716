import os

import numpy as np
import torch

from oracle import ua_oracle as orc

NAMES = ("kc", "vc", "xq", "static_src", "static_dest")
# tolerances of the parity bar: relative error of the whole tensor (Frobenius norm)
TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2}


def rel_err(x, ref):
    x, ref = x.detach().double().cpu(), ref.detach().double().cpu()
    return float((x - ref).norm() / ref.norm().clamp_min(1e-30))


def dense_reference(inp, dtype64=torch.float64):
    """float64 dense oracle on the (already dtype-rounded) inputs: O, lse and the 5 gradients under dO."""
    b, h, n, c, d = inp["kc"].shape
    l = n * c
    leaves = [inp[k].detach().cpu().to(dtype64).requires_grad_() for k in NAMES]
    O, lse = orc.dense_forward(leaves[0].reshape(b, h, l, d), leaves[1].reshape(b, h, l, d), leaves[2].reshape(b, h, -1, l, d),
                               leaves[3].reshape(b, h, l), leaves[4].reshape(b, h, l), return_lse=True)
    grads = torch.autograd.grad(O, leaves, inp["dO"].detach().cpu().to(dtype64).reshape(O.shape))
    return O.detach(), lse.detach(), grads


def load_golden(name):
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    z = np.load(os.path.join(here, name + ".npz"))
    b, h, r, l, d, c, seed, is_bf16 = [int(x) for x in z["meta"]]
    dtype = torch.bfloat16 if is_bf16 else torch.float32
    t = {k: torch.from_numpy(z[k]) for k in z.files if k != "meta"}
    return t, dtype, (b, h, r, l, d, c, seed)


def key_gradient_bar(inp, dtype, exact_dkc):
    """Bar for the key gradient: the stated tolerance, or twice the error that the reference's own algorithm (the
    chunked restatement followed by the merge, run in `dtype`) makes against the float64 gradient on the same inputs,
    where that is larger.  d/dk of relu(k_s.k_u)^(2/3) is (2/3)(k_s.k_u)^(-1/3), singular at 0+: a pair with a tiny
    positive product amplifies the rounding of the product itself, so the error is a property of the inputs in
    `dtype`, not of a kernel.  Prints both terms so that a run shows which one set the bar."""
    args = [inp[k] for k in NAMES]
    out, denom = orc.chunked_forward(*args)
    d_out, d_denom = orc.merge_backward(out.float(), denom.float(), inp["dO"].float())
    own = rel_err(orc.chunked_backward(*args, d_out.to(dtype), d_denom)[0], exact_dkc)
    bar = max(TOL[dtype], 2 * own)
    print("key-gradient bar %.2e (stated %.0e, reference algorithm in %s misses float64 by %.2e)" % (bar, TOL[dtype], str(dtype)[6:], own), flush=True)
    return bar


def summation_order_sensitivity(inp, g_out, g_denom, dkc):
    """How far the float32 oracle's own dkc moves when the head dimension is summed in another order (features of k, v,
    q and of the upstream gradient permuted, result permuted back; largest move over the reversed order and four
    random ones): mathematically the same gradient, but the key-key products round differently and
    (2/3)(k_s.k_u)^(-1/3) amplifies that for tiny positive products (one pair with k_s.k_u = 5.6e-6 carries half of
    the whole tensor's error in the 512x64 case)."""
    d = inp["kc"].shape[-1]
    gen = torch.Generator().manual_seed(1)
    worst = 0.0
    for trial in range(5):
        perm = torch.arange(d).flip(0) if trial == 0 else torch.randperm(d, generator=gen)
        inv = torch.argsort(perm)
        args = [inp[k].float()[..., perm] for k in ("kc", "vc", "xq")] + [inp[k].float() for k in ("static_src", "static_dest")]
        g = orc.chunked_backward(*args, g_out.float()[..., perm, :], g_denom)
        worst = max(worst, rel_err(g[0][..., inv], dkc))
    return worst


def chunked_key_gradient_bar(inp, g_out, g_denom, dtype):
    """-> (float64 key gradient of the chunked backward, bar for a kernel's distance from it): the stated tolerance, or
    three times the larger of (a) the float32 restatement's own distance from float64 and (b) what the restatement moves
    under other summation orders of the head dimension.  The error is heavy-tailed (see key_gradient_bar), so a kernel's
    draw is allowed to exceed the restatement's by that factor, not more."""
    args = [inp[k].float() for k in NAMES]
    exact = orc.chunked_backward(*[inp[k].double() for k in NAMES], g_out.double(), g_denom.double())[0]
    own32 = orc.chunked_backward(*args, g_out.float(), g_denom.float())[0]
    own, moved = rel_err(own32, exact), summation_order_sensitivity(inp, g_out, g_denom.float(), own32)
    bar = max(TOL[dtype], 3 * max(own, moved))
    print("chunked key-gradient bar %.2e (stated %.0e; float32 restatement misses float64 by %.2e and moves by %.2e under "
          "other summation orders)" % (bar, TOL[dtype], own, moved), flush=True)
    return exact, bar
