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
