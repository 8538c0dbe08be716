"""Sizes at and beyond the limits of a single launch: chunks of 512 and more keys, more heads than grid rows."""
import pytest
import torch

from oracle import ua_oracle as orc
from tests.util import NAMES, TOL, chunked_key_gradient_bar, dense_reference, key_gradient_bar, rel_err

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(1, 2, 2, 1024, 64, 512), (1, 1, 1, 2048, 128, 1024), (2, 1, 1, 1536, 32, 768), (1, 1, 1, 1024, 64, 1024)])
def test_chunks_of_512_and_more_keys(shape, dtype):
    """Any multiple of 64 is a chunk size of the query-/key-stationary kernels (the reference takes any chunk that
    divides L, universal_attention_autograd.py:9-15): forward, backward under an arbitrary upstream gradient, and the
    reference's call sequence through the merge."""
    from universal_attention_triton_amd import ops, universal_attention_autograd as ua
    b, h, r, L, d, c = shape
    n = L // c
    print("case large chunk", shape, dtype, flush=True)
    inp = orc.make_inputs(b, h, r, L, d, c, dtype=dtype, seed=201)
    args32 = [inp[k].float() for k in NAMES]
    g = torch.Generator().manual_seed(8)
    g_out = torch.randn(b, h, r, L, d, n, generator=g).to(dtype)
    g_denom = torch.randn(b, h, r, L, n, generator=g).to(dtype)
    out_ref, denom_ref = orc.chunked_forward(*args32)
    want = orc.chunked_backward(*args32, g_out.float(), g_denom.float())
    leaves = [inp[k].cuda().requires_grad_() for k in NAMES]
    out, denom = ua.UniversalAttention.apply(*leaves)
    grads = torch.autograd.grad([out, denom], leaves, [g_out.cuda(), g_denom.cuda()])
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert rel_err(out, out_ref) <= tol, rel_err(out, out_ref)
    live = denom_ref > -1e11
    assert torch.equal(denom.float().cpu()[~live], denom_ref.to(dtype).float()[~live])
    assert rel_err(denom.float().cpu()[live], denom_ref[live]) <= tol
    exact, bar = chunked_key_gradient_bar(inp, g_out, g_denom, dtype) if dtype == torch.float32 else (want[0], tol)
    for name, x, y in zip(NAMES, grads, (exact,) + tuple(want[1:])):
        e = rel_err(x.reshape(y.shape), y)
        print("  d%-12s %.2e (bar %.2e)" % (name, e, bar if name == "kc" else tol), flush=True)
        assert e <= (bar if name == "kc" else tol), (name, e)
    # the call sequence with the merge equals the fused operator
    O_ref, _, g_ref = dense_reference(inp)
    leaves = [inp[k].cuda().requires_grad_() for k in NAMES]
    out, denom = ua.UniversalAttention.apply(*leaves)
    O = ua.SMVecMatMul.apply(out, denom)
    cg = torch.autograd.grad(O, leaves, inp["dO"].cuda())
    assert rel_err(O, O_ref) <= tol
    bar = key_gradient_bar(inp, dtype, g_ref[0])
    if dtype == torch.float32:
        d_out, d_denom = orc.merge_backward(out_ref, denom_ref, inp["dO"].float())
        bar = max(bar, chunked_key_gradient_bar(inp, d_out, d_denom, dtype)[1])
    for name, x, y in zip(NAMES, cg, g_ref):
        assert rel_err(x, y) <= (bar if name == "kc" else tol), (name, rel_err(x, y))


@pytest.mark.parametrize("shape", [(3, 16384, 2, 16, 16, 16), (1, 40000, 2, 32, 16, 16), (2, 9000, 1, 64, 16, 16)])
def test_more_heads_than_grid_rows_are_split_by_the_operators(shape):
    """b*h*r (times the chunks per row for the chunked operator) above 65535: the C entry points refuse, the Python
    operators run the call in pieces along b, then h.  Heads are independent, so every head must come out exactly as in a
    call on that head alone; a few heads are also held against the oracle."""
    from universal_attention_triton_amd import ops
    from universal_attention_triton_amd.universal_attention import universal_attention
    b, h, r, L, d, c = shape
    n = L // c
    print("case many heads", shape, flush=True)
    dtype = torch.float32
    inp = orc.make_inputs(b, h, r, L, d, c, dtype=dtype, seed=301)
    dev = {k: v.cuda() for k, v in inp.items()}
    a = [dev[k] for k in NAMES]
    fused_rows, chunked_rows = b * h * r, b * h * r * n
    assert chunked_rows > 65535
    picks = [(0, 0), (b - 1, h - 1), (b // 2, h // 3), (0, h // 2 + 1)]
    if fused_rows > 65535:
        leaves = [x.clone().requires_grad_() for x in a]
        O = universal_attention(*leaves)
        grads = torch.autograd.grad(O, leaves, dev["dO"])
        for bi, hi in picks:
            one = [x[bi:bi + 1, hi:hi + 1].clone().requires_grad_() for x in a]
            O1 = universal_attention(*one)
            g1 = torch.autograd.grad(O1, one, dev["dO"][bi:bi + 1, hi:hi + 1])
            assert torch.equal(O[bi:bi + 1, hi:hi + 1], O1)
            for x, y in zip(grads, g1):
                assert torch.equal(x[bi:bi + 1, hi:hi + 1], y)
        bi, hi = picks[2]
        sub = {k: v[bi:bi + 1, hi:hi + 1] for k, v in inp.items()}
        O_ref, _, g_ref = dense_reference(sub)
        assert rel_err(O[bi:bi + 1, hi:hi + 1], O_ref) <= TOL[dtype]
        for name, x, y in zip(NAMES, grads, g_ref):
            assert rel_err(x[bi:bi + 1, hi:hi + 1], y) <= (TOL[dtype] if name != "kc" else key_gradient_bar(sub, dtype, y)), name
    gen = torch.Generator().manual_seed(4)
    g_out = torch.randn(b, h, r, L, d, n, generator=gen).cuda()
    g_denom = torch.randn(b, h, r, L, n, generator=gen).cuda()
    out, denom, state = ops.chunked_forward(*a, keep_state=True)
    assert state is None and out.shape == (b, h, r, L, d, n)
    grads = ops.chunked_backward(*a, out, g_out, g_denom, state=None)
    for bi, hi in picks:
        one = [x[bi:bi + 1, hi:hi + 1] for x in a]
        out1, denom1, _ = ops.chunked_forward(*one)
        g1 = ops.chunked_backward(*one, out1, g_out[bi:bi + 1, hi:hi + 1], g_denom[bi:bi + 1, hi:hi + 1])
        assert torch.equal(out[bi:bi + 1, hi:hi + 1], out1) and torch.equal(denom[bi:bi + 1, hi:hi + 1], denom1)
        for x, y in zip(grads, g1):
            # chunks that are no multiple of 64 add up partial gradients with float atomics, in an order that varies
            assert rel_err(x[bi:bi + 1, hi:hi + 1].reshape(y.shape), y) <= 1e-5
    bi, hi = picks[1]
    ref = orc.chunked_forward(*[inp[k][bi:bi + 1, hi:hi + 1] for k in NAMES])
    assert rel_err(out[bi:bi + 1, hi:hi + 1], ref[0]) <= TOL[dtype]
