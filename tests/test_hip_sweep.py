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


def _dkc_bar(inp, dtype, exact, tol):
    """d/dG relu(G)^(2/3) is singular at 0+: the bar for the key gradient is the larger of the tolerance and twice the
    error of the reference algorithm itself, evaluated in the same dtype on the same inputs (see test_hip_backward)."""
    args = [inp[k] for k in NAMES]
    out, denom = orc.chunked_forward(*args)
    d_out, d_denom = orc.merge_backward(out.float(), denom.float(), inp["dO"].float())
    g = orc.chunked_backward(*args, d_out.to(dtype), d_denom)
    return max(tol, 2 * rel_err(g[0], exact))


def test_fused_operator_random_shapes_and_flags():
    from universal_attention_triton_amd import ops
    rng = random.Random(20260)
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
        errs = {"O": rel_err(O, O_ref), "lse": float((lse.cpu().double() - lse_ref).abs().max()) / 10}
        for k, g, gr in zip(NAMES, grads, g_ref):
            if float(gr.abs().max()) == 0.0:        # L = 1: every gradient is exactly zero; here rounding noise of dP - delta
                errs["d" + k] = float(g.float().abs().max().cpu()) * tol
            else:
                errs["d" + k] = rel_err(g.reshape(gr.shape), gr)
        bars = {k: tol for k in errs}
        if dtype == torch.float32 and errs["dkc"] > tol:
            # random keys have products k_s.k_u arbitrarily close to 0+, where the float32 rounding of the product is
            # amplified (test_hip_paths holds dkc to 1e-4 on well-conditioned keys)
            bars["dkc"] = max(4e-4, _dkc_bar(inp, dtype, g_ref[0], tol))
        bad = {k: (v, bars[k]) for k, v in errs.items() if not v <= bars[k]}
        assert not bad, (case, bad)


def test_chunked_operator_random_shapes_and_upstreams():
    from universal_attention_triton_amd import universal_attention_autograd as ua
    rng = random.Random(20261)
    done = 0
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
        if dtype == torch.float32:
            bars["dkc"] = 5e-4      # the float32 restatement itself moves this far under a permutation of the head dim
        bad = {k: (v, bars[k]) for k, v in errs.items() if not v <= bars[k]}
        assert not bad, (case, bad)
