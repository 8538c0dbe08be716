"""A bounded, seeded sweep over random shapes and flag combinations: the fused operator (L from 1 to 3000, head dims
from 8 to 256, up to 4 query groups, both dtypes, pruning / recomputation / shared key sweeps / no kept state) against
float64 autograd of the dense oracle, and the chunked operator (chunks 16 .. 256, arbitrary or merge-like upstream)
against the oracle's restatement of the reference operator.  Stops at the first failing case and prints it."""
import random

import pytest
import torch

from oracle import ua_oracle as orc
from tests.util import NAMES, TOL, dense_reference, rel_err

pytestmark = pytest.mark.gpu
LENGTHS = [1, 7, 16, 31, 33, 64, 100, 127, 128, 129, 200, 255, 257, 300, 384, 500, 513, 640, 777, 1024, 1500, 2049, 3000]


def _reference_bars(inp, dtype, exact, tol):
    """Per gradient: the larger of the tolerance and twice the error of the reference algorithm itself, evaluated in the
    same dtype on the same inputs (see test_hip_backward).  Two things make the reference itself miss the float64
    result by more than the tolerance on some random inputs: d/dG relu(G)^(2/3) is singular at 0+ (key gradient), and
    with a handful of positions a gate gradient is a sum of a few terms of both signs, so that operand rounding does
    not average out (L = 7, bf16: the reference is 1.7e-2 away in static_dest, 8 % in one of its elements).
    In float32 the key gradient's error hangs on how single key-key products round, which changes with the order the
    head dimension is summed in (0.9e-4 ... 5.6e-4 over six orders in one 777x48 case; in a 1024x32 case one pair with
    k_s.k_u = 1.03e-6, whose float32 value spreads by 1.4 % over the orders, carries 99.97 % of the kernel's error):
    its bar takes three times the worst of the given order, the reversed one and fourteen random ones (the spread is
    heavy-tailed: in a 640x96 case the kernel's own order gave 2.4 times that worst)."""
    def run(perm):
        args = [inp[k][..., perm] for k in NAMES[:3]] + [inp[k] for k in NAMES[3:]]
        out, denom = orc.chunked_forward(*args)
        d_out, d_denom = orc.merge_backward(out.float(), denom.float(), inp["dO"].float()[..., perm])
        g = orc.chunked_backward(*args, d_out.to(dtype), d_denom)
        inv = torch.argsort(perm)
        return [x[..., inv] for x in g[:3]] + list(g[3:])
    d = inp["kc"].shape[-1]
    g = run(torch.arange(d))
    bars = {"d" + k: max(tol, 2 * rel_err(x, y)) for k, x, y in zip(NAMES, g, exact)}
    if dtype == torch.float32:
        gen = torch.Generator().manual_seed(1)
        for trial in range(15):
            perm = torch.arange(d).flip(0) if trial == 0 else torch.randperm(d, generator=gen)
            bars["dkc"] = max(bars["dkc"], 3 * rel_err(run(perm)[0], exact[0]))
    return bars


def test_fused_operator_random_shapes_and_flags():
    from universal_attention_triton_amd import ops
    rng = random.Random(20260)
    relaxed = []          # cases judged by the reference algorithm's own error instead of the plain tolerance
    for it in range(40):
        b, h, r = rng.choice([1, 1, 2]), rng.choice([1, 2, 3]), rng.choice([1, 1, 2, 3, 4])
        L = rng.choice(LENGTHS)
        dtype = rng.choice([torch.float32, torch.bfloat16])
        d = rng.choice([8, 16, 24, 32, 48, 64, 72, 96, 128] + ([160, 256] if dtype == torch.bfloat16 else []))
        gm = rng.choice([0.0, 0.0, 2.0, -2.0])
        flags = dict(prune=rng.random() < 0.3, recompute=rng.random() < 0.3 and d <= 128, share_groups=rng.random() < 0.3)
        keep = rng.random() < 0.7
        seed = rng.randrange(10000)
        if L >= 1500:                # keep the float64 oracle of the long cases small
            b, h, r = 1, 1, min(r, 2)
        case = dict(it=it, shape=(b, h, r, L, d), dtype=str(dtype), gate_mean=gm, flags=flags, keep_state=keep, seed=seed)
        print("case", case, flush=True)
        inp = orc.make_inputs(b, h, r, L, d, L, dtype=dtype, seed=seed, gate_mean=gm)
        dev = {k: v.cuda() for k, v in inp.items()}
        a = [dev[k] for k in NAMES]
        O, lse, state = ops.fused_forward(*a, keep_state=keep, **flags)
        grads = ops.fused_backward(*a, O, lse, dev["dO"], state=state, **flags)
        torch.cuda.synchronize()
        O_ref, lse_ref, g_ref = dense_reference(inp)
        tol = TOL[dtype]
        errs = {"O": rel_err(O, O_ref), "lse": float((lse.cpu().double() - lse_ref).abs().max())}
        for k, g, gr in zip(NAMES, grads, g_ref):
            if float(gr.abs().max()) == 0.0:        # L = 1: every gradient is exactly zero; here rounding noise of dP - delta
                errs["d" + k] = float(g.float().abs().max().cpu()) * tol
            else:
                errs["d" + k] = rel_err(g.reshape(gr.shape), gr)
        bars = {k: tol for k in errs}
        if any(errs[k] > tol for k in errs if k.startswith("d")) and L > 1:
            # ill-conditioned inputs: hold the gradients to what the reference algorithm itself achieves in this dtype
            # (test_hip_paths holds dkc to 1e-4 on well-conditioned keys)
            missed = sorted(k for k in errs if k.startswith("d") and errs[k] > tol)
            ref_bars = _reference_bars(inp, dtype, g_ref, tol)
            for k in missed:          # only the tensors that missed take the reference's own error as their bar
                bars[k] = ref_bars[k]
            relaxed.append((it, case["shape"], case["dtype"], {k: "%.2e (bar %.2e)" % (errs[k], bars[k]) for k in missed}))
            print("   relaxed:", relaxed[-1], flush=True)
        bad = {k: (v, bars[k]) for k, v in errs.items() if not v <= bars[k]}
        assert not bad, (case, bad)
    print("cases judged by the reference algorithm's own error: %d of 40" % len(relaxed), relaxed, flush=True)
    assert len(relaxed) <= 8, relaxed


def test_chunked_operator_random_shapes_and_upstreams():
    from universal_attention_triton_amd import universal_attention_autograd as ua
    rng = random.Random(20261)
    done = 0
    relaxed = []
    while done < 16:
        b, h, r = rng.choice([1, 1, 2]), rng.choice([1, 2, 3]), rng.choice([1, 1, 2, 3])
        c = rng.choice([16, 32, 64, 64, 96, 128, 128, 192, 256])
        n = rng.choice([1, 2, 3, 5, 8])
        L = c * n
        if L > 1024:
            continue
        done += 1
        d = rng.choice([8, 16, 32, 48, 64, 72, 128])
        dtype = rng.choice([torch.float32, torch.bfloat16])
        gm = rng.choice([0.0, 0.0, 2.0, -2.0])
        composite = rng.random() < 0.4       # upstream that vanishes where a query precedes the chunk, as after a merge
        seed = rng.randrange(10000)
        case = dict(it=done, shape=(b, h, r, L, d, c), dtype=str(dtype), gate_mean=gm, merge_like=composite, seed=seed)
        print("case", case, flush=True)
        inp = orc.make_inputs(b, h, r, L, d, c, dtype=dtype, seed=seed, gate_mean=gm)
        g = torch.Generator().manual_seed(seed + 1)
        g_out = torch.randn(b, h, r, L, d, n, generator=g).to(dtype)
        g_denom = torch.randn(b, h, r, L, n, generator=g).to(dtype)
        if composite:
            t = torch.arange(L).view(L, 1, 1)
            live = t >= torch.arange(n).view(1, 1, n) * c
            g_out = g_out * live.to(dtype)
            g_denom = g_denom * live.view(L, n).to(dtype)
        args32 = [inp[k].float() for k in NAMES]
        out_ref, denom_ref = orc.chunked_forward(*args32)
        want = orc.chunked_backward(*args32, g_out.float(), g_denom.float())
        leaves = [inp[k].cuda().requires_grad_() for k in NAMES]
        out, denom = ua.UniversalAttention.apply(*leaves)
        grads = torch.autograd.grad([out, denom], leaves, [g_out.cuda(), g_denom.cuda()])
        torch.cuda.synchronize()
        tol = TOL[dtype]
        errs = {"out": rel_err(out, out_ref)}
        masked = denom_ref < -1e11
        got = denom.float().cpu()
        errs["denom"] = float(((got - denom_ref)[~masked].abs() / denom_ref[~masked].abs().clamp_min(1.0)).max()) if (~masked).any() else 0.0
        assert torch.equal(got[masked], denom_ref.to(dtype).float()[masked]), case
        for k, x, y in zip(NAMES, grads, want):
            errs["d" + k] = rel_err(x.reshape(y.shape), y)
        bars = {k: tol for k in errs}
        bars["denom"] = max(tol, 2 ** -8 if dtype == torch.bfloat16 else tol)      # denom is stored in the dtype
        if dtype == torch.float32 and errs["dkc"] > bars["dkc"]:
            # a key-key product very close to 0+ (d/dG relu(G)^(2/3) is singular there): judge both float32 results
            # by the float64 evaluation, the kernel being allowed twice the restatement's own error and three times
            # what the restatement moves under the reversed and fourteen random summation orders of the head dimension
            exact = orc.chunked_backward(*[inp[k].double() for k in NAMES], g_out.double(), g_denom.double())[0]
            errs["dkc"] = rel_err(grads[0].reshape(exact.shape), exact)
            bars["dkc"] = max(tol, 2 * rel_err(want[0], exact))
            gen = torch.Generator().manual_seed(1)
            for trial in range(15):
                perm = torch.arange(d).flip(0) if trial == 0 else torch.randperm(d, generator=gen)
                a2 = [x[..., perm] for x in args32[:3]] + args32[3:]
                g2 = orc.chunked_backward(*a2, g_out.float()[..., perm, :], g_denom.float())[0]
                bars["dkc"] = max(bars["dkc"], 3 * rel_err(g2[..., torch.argsort(perm)], exact))
            relaxed.append((done, "dkc %.2e under a computed bar of %.2e" % (errs["dkc"], bars["dkc"])))
        print("  " + "  ".join("%s %.1e/%.0e" % (k, v, bars[k]) for k, v in errs.items()), flush=True)
        bad = {k: (v, bars[k]) for k, v in errs.items() if not v <= bars[k]}
        assert not bad, (case, bad)
    print("cases with the key gradient judged by the restatement's own float32 error: %d of 16" % len(relaxed), relaxed, flush=True)
    assert len(relaxed) <= 4, relaxed
