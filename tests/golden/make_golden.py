"""Writes the golden vectors under tests/golden/ by running the REFERENCE torch
operator (reference ``universal_attention_autograd.py``) on the CPU, once, in the
build container.  The reference is only imported here; the fixtures it writes
are data (inputs + expected outputs) and are what the tests read.

    python tests/golden/make_golden.py [/root/reference] [--only-2d]

What the vectors pin that nothing else does: the bit-level behaviour of the
torch path at its cast points (bf16 K.K^T / pow rounding, bf16 ``denom``), the
hand-written backward's epsilons, and the gradients of the fully masked
(query, chunk) pairs under an arbitrary upstream gradient.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))
from oracle.ua_oracle import make_inputs  # noqa: E402  (input recipe only)


def f32(x):
    return x.detach().float().cpu().numpy()


def run_case(ref, name, b, h, r, l, d, c, dtype, seed):
    inp = make_inputs(b, h, r, l, d, c, dtype=dtype, seed=seed)
    n = l // c
    g = torch.Generator().manual_seed(seed + 7)
    g_out = torch.randn(b, h, r, l, d, n, generator=g).to(dtype)
    g_denom = torch.randn(b, h, r, l, n, generator=g)            # always fp32 (autograd.py:48)
    leaves = [inp[k].clone().requires_grad_() for k in ("kc", "vc", "xq", "static_src", "static_dest")]

    # (i) arbitrary upstream on the chunked outputs
    out, denom = ref.UniversalAttention.apply(*leaves)
    grads = torch.autograd.grad([out, denom], leaves, [g_out, g_denom.to(denom.dtype)])
    # (ii) composite upstream: O = SMVecMatMul(out, denom), loss = <O, dO>
    out2, denom2 = ref.UniversalAttention.apply(*leaves)
    O = ref.SMVecMatMul.apply(out2, denom2)
    cgrads = torch.autograd.grad(O, leaves, inp["dO"])
    # 2-D tiling of the same operator (query chunks = key chunks)
    xq2 = inp["xq"].view(b, h, r, n, c, d)
    sd2 = inp["static_dest"].view(b, h, n, c)
    out2d, denom2d = ref.UniversalAttention2.apply(inp["kc"], inp["vc"], xq2, inp["static_src"], sd2)

    data = {k: f32(v) for k, v in inp.items()}
    data.update(g_out=f32(g_out), g_denom=f32(g_denom), out=f32(out), denom=f32(denom), O=f32(O),
                out2d=f32(out2d), denom2d=f32(denom2d))
    for nm, gr, cg in zip(("dkc", "dvc", "dxq", "dsrc", "ddest"), grads, cgrads):
        data[nm] = f32(gr)
        data["c_" + nm] = f32(cg)
    data["meta"] = np.array([b, h, r, l, d, c, seed, 1 if dtype == torch.bfloat16 else 0])
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **data)
    print("wrote", name, {k: v.shape for k, v in data.items() if k in ("out", "denom", "dkc")})


def run_case_2d(ref, name, b, h, r, l, d, c, qc, dtype, seed):
    """UniversalAttention2 (reference universal_attention_autograd.py:102-276) with query chunks of qc != c positions:
    forward and the five gradients of its own hand-written backward under an arbitrary upstream gradient."""
    inp = make_inputs(b, h, r, l, d, c, dtype=dtype, seed=seed)
    n = l // c
    g = torch.Generator().manual_seed(seed + 9)
    g_out = torch.randn(b, h, r, l, d, n, generator=g).to(dtype)
    g_denom = torch.randn(b, h, r, l, n, generator=g)
    xq2 = inp["xq"].view(b, h, r, l // qc, qc, d)
    sd2 = inp["static_dest"].view(b, h, l // qc, qc)
    leaves = [x.clone().requires_grad_() for x in (inp["kc"], inp["vc"], xq2, inp["static_src"], sd2)]
    out, denom = ref.UniversalAttention2.apply(*leaves)
    grads = torch.autograd.grad([out, denom], leaves, [g_out, g_denom.to(denom.dtype)])
    data = {k: f32(v) for k, v in inp.items()}
    data.update(g_out=f32(g_out), g_denom=f32(g_denom), out=f32(out), denom=f32(denom))
    for nm, gr in zip(("dkc", "dvc", "dxq", "dsrc", "ddest"), grads):
        data[nm] = f32(gr)
    data["meta"] = np.array([b, h, r, l, d, c, seed, 1 if dtype == torch.bfloat16 else 0])
    data["qc"] = np.array([qc])
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **data)
    print("wrote", name, {k: v.shape for k, v in data.items() if k in ("out", "denom", "dxq", "ddest")})


def run_cfg0(ref):
    """BASELINE config 0 at full size, forward only, fp32; inputs are regenerated
    from the seed by the test (a checksum guards the regeneration)."""
    b, h, r, l, d, c = 1, 4, 1, 512, 64, 64
    inp = make_inputs(b, h, r, l, d, c, dtype=torch.float32, seed=1000)
    out, denom = ref.UniversalAttention.apply(inp["kc"], inp["vc"], inp["xq"], inp["static_src"], inp["static_dest"])
    O = ref.SMVecMatMul.apply(out, denom)
    chk = np.array([float(inp[k].double().sum()) for k in ("kc", "vc", "xq", "static_src", "static_dest")])
    # the per-chunk `out` tensor is 4 MB: keep two chunks of it (first and last) plus everything merged
    np.savez_compressed(os.path.join(HERE, "cfg0_fwd_fp32.npz"), O=f32(O), denom=f32(denom),
                        out_first=f32(out[..., 0]), out_last=f32(out[..., -1]), input_checksum=chk,
                        meta=np.array([b, h, r, l, d, c, 1000, 0]))
    print("wrote cfg0_fwd_fp32")


def main():
    args = [a for a in sys.argv[1:] if not a.startswith("--")]
    ref_root = args[0] if args else "/root/reference"
    sys.path.insert(0, ref_root)
    import universal_attention_autograd as ref
    torch.manual_seed(0)
    if "--only-2d" in sys.argv:      # adds the 2-D fixtures without rewriting the others
        run_case_2d(ref, "tiny2d_fp32", 1, 2, 2, 64, 16, 16, 32, torch.float32, 13)
        run_case_2d(ref, "tiny2d_bf16", 1, 2, 2, 64, 16, 16, 32, torch.bfloat16, 13)
        return
    run_case_2d(ref, "tiny2d_fp32", 1, 2, 2, 64, 16, 16, 32, torch.float32, 13)
    run_case_2d(ref, "tiny2d_bf16", 1, 2, 2, 64, 16, 16, 32, torch.bfloat16, 13)
    run_case(ref, "tiny_fp32", 1, 2, 2, 64, 16, 16, torch.float32, 11)
    run_case(ref, "tiny_bf16", 1, 2, 2, 64, 16, 16, torch.bfloat16, 11)
    run_case(ref, "small_fp32", 1, 1, 1, 128, 32, 32, torch.float32, 12)
    run_case(ref, "small_bf16", 1, 1, 1, 128, 32, 32, torch.bfloat16, 12)
    run_cfg0(ref)


if __name__ == "__main__":
    main()
