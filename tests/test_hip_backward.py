"""GPU parity of the backward kernels, called through the C ABI (ctypes -> libua_hip.so)."""
import pytest
import torch

from oracle import ua_oracle as orc
from tests.util import NAMES, TOL, dense_reference, key_gradient_bar, load_golden, rel_err, summation_order_sensitivity as _summation_order_sensitivity

pytestmark = pytest.mark.gpu

SHAPES = [  # b, h, r, L, d, c
    (1, 2, 2, 64, 16, 16),
    (1, 1, 1, 128, 32, 32),
    (2, 2, 1, 256, 64, 64),
    (1, 2, 1, 384, 128, 128),
    (1, 1, 2, 320, 80, 32),
]
GRADS = ("dkc", "dvc", "dxq", "dsrc", "ddest")


def _report(tag, got, want, tol, tol_dkc=None):
    errs = {n: rel_err(g.reshape(w.shape), w) for n, g, w in zip(GRADS, got, want)}
    print(tag, {k: "%.2e" % v for k, v in errs.items()}, flush=True)
    bad = {k: v for k, v in errs.items() if not v <= (tol_dkc if (k == "dkc" and tol_dkc) else tol)}
    assert not bad, bad


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
def test_fused_backward_matches_dense_autograd(shape, dtype):
    from universal_attention_triton_amd.universal_attention import universal_attention
    print("case fused_bwd", shape, dtype, flush=True)
    b, h, r, L, d, c = shape
    inp = orc.make_inputs(b, h, r, L, d, c, dtype=dtype, seed=31)
    O_ref, _, g_ref = dense_reference(inp)
    leaves = [inp[k].cuda().requires_grad_() for k in NAMES]
    O = universal_attention(*leaves)
    grads = torch.autograd.grad(O, leaves, inp["dO"].cuda())
    torch.cuda.synchronize()
    assert rel_err(O, O_ref) <= TOL[dtype]
    _report("fused", grads, g_ref, TOL[dtype], key_gradient_bar(inp, dtype, g_ref[0]))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
def test_chunked_backward_matches_oracle_arbitrary_upstream(shape, dtype):
    """Upstream gradients on the per-chunk tensors are arbitrary (not from a merge): the gradients of the
    fully masked (query, chunk) pairs must follow the reference's hand-written backward."""
    from universal_attention_triton_amd import universal_attention_autograd as ua
    print("case chunked_bwd", shape, dtype, flush=True)
    b, h, r, L, d, c = shape
    n = L // c
    inp = orc.make_inputs(b, h, r, L, d, c, dtype=dtype, seed=32)
    g = torch.Generator().manual_seed(5)
    g_out = torch.randn(b, h, r, L, d, n, generator=g).to(dtype)
    g_denom = torch.randn(b, h, r, L, n, generator=g)
    want = orc.chunked_backward(*[inp[k].float() for k in NAMES], g_out.float(), g_denom)
    leaves = [inp[k].cuda().requires_grad_() for k in NAMES]
    out, denom = ua.UniversalAttention.apply(*leaves)
    grads = torch.autograd.grad([out, denom], leaves, [g_out.cuda(), g_denom.to(dtype).cuda()])
    torch.cuda.synchronize()
    if dtype == torch.bfloat16:   # the oracle saw the unrounded g_denom; recompute with the rounded one
        want = orc.chunked_backward(*[inp[k].float() for k in NAMES], g_out.float(), g_denom.to(dtype).float())
    _report("chunked", grads, want, TOL[dtype])


@pytest.mark.parametrize("name", ["tiny_fp32", "tiny_bf16", "small_fp32", "small_bf16"])
def test_backward_matches_reference_golden(name):
    from universal_attention_triton_amd import universal_attention_autograd as ua
    print("case golden_bwd", name, flush=True)
    t, dtype, (b, h, r, l, d, c, seed) = load_golden(name)
    tol = TOL[dtype]
    leaves = [t[k].to(dtype).cuda().requires_grad_() for k in NAMES]
    out, denom = ua.UniversalAttention.apply(*leaves)
    grads = torch.autograd.grad([out, denom], leaves, [t["g_out"].to(dtype).cuda(), t["g_denom"].to(dtype).cuda()])
    torch.cuda.synchronize()
    _report("golden arbitrary", grads, [t[n] for n in GRADS], tol)
    # composite: O = SMVecMatMul(out, denom), upstream dO
    leaves = [t[k].to(dtype).cuda().requires_grad_() for k in NAMES]
    out, denom = ua.UniversalAttention.apply(*leaves)
    O = ua.SMVecMatMul.apply(out, denom)
    cgrads = torch.autograd.grad(O, leaves, t["dO"].to(dtype).cuda())
    torch.cuda.synchronize()
    assert rel_err(O, t["O"]) <= tol
    _report("golden composite", cgrads, [t["c_" + n] for n in GRADS], tol)


def test_merge_kernels_match_oracle():
    from universal_attention_triton_amd import universal_attention_autograd as ua
    torch.manual_seed(3)
    for dtype in (torch.float32, torch.bfloat16):
        mat = torch.randn(2, 3, 2, 40, 24, 6).to(dtype)
        vec = torch.randn(2, 3, 2, 40, 6).to(dtype)
        g = torch.randn(2, 3, 2, 40, 24).to(dtype)
        want = orc.merge(mat.float(), vec.float())
        wd = orc.merge_backward(mat.float(), vec.float(), g.float())
        m, v = mat.cuda().requires_grad_(), vec.cuda().requires_grad_()
        res = ua.SMVecMatMul.apply(m, v)
        dm, dv = torch.autograd.grad(res, [m, v], g.cuda())
        assert rel_err(res, want) <= TOL[dtype]
        assert rel_err(dm, wd[0]) <= TOL[dtype] and rel_err(dv, wd[1]) <= TOL[dtype]


FAST_CHUNK_SHAPES = [  # chunk a multiple of 64: key-/query-stationary kernels; b, h, r, L, d, c
    (1, 2, 2, 512, 64, 64),      # query groups, two chunks per 128-key workgroup
    (1, 1, 1, 768, 128, 192),    # chunk boundaries that are not multiples of 128
    (1, 1, 2, 512, 32, 256),     # one chunk spans two workgroups
    (2, 2, 3, 320, 16, 64),      # L a multiple of 64 but not of 128: a padded 64-key tile beyond the last chunk
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", FAST_CHUNK_SHAPES)
def test_chunked_backward_chunk_multiple_of_64(shape, dtype):
    """Arbitrary upstream gradients (the uniform-softmax region is live), with the forward's workspace and without
    it (recompute), then an upstream that is zero before each chunk (the region is skipped, with and without
    UA_FLAG_SKIP_MASKED)."""
    from universal_attention_triton_amd import ops
    print("case chunked_bwd_fast", shape, dtype, flush=True)
    b, h, r, L, d, c = shape
    n = L // c
    inp = orc.make_inputs(b, h, r, L, d, c, dtype=dtype, seed=33)
    g = torch.Generator().manual_seed(6)
    g_out = torch.randn(b, h, r, L, d, n, generator=g).to(dtype)
    g_denom = torch.randn(b, h, r, L, n, generator=g).to(dtype).float()
    ins = [inp[k].cuda() for k in NAMES]
    out, denom, ws = ops.chunked_forward(*ins, keep_state=True)
    want = orc.chunked_backward(*[inp[k].float() for k in NAMES], g_out.float(), g_denom)
    tol_dkc = max(TOL[dtype], 2 * _summation_order_sensitivity(inp, g_out, g_denom, want[0]))
    got = ops.chunked_backward(*ins, out, g_out.cuda(), g_denom.cuda(), state=ws)
    torch.cuda.synchronize()
    _report("with workspace", got, want, TOL[dtype], tol_dkc)
    got = ops.chunked_backward(*ins, out, g_out.cuda(), g_denom.cuda(), state=None)
    torch.cuda.synchronize()
    _report("recompute", got, want, TOL[dtype], tol_dkc)
    got = ops.chunked_backward(*ins, out, g_out.cuda(), g_denom.cuda(), state=None, recompute=True)
    torch.cuda.synchronize()
    _report("UA_FLAG_RECOMPUTE", got, want, TOL[dtype], tol_dkc)
    # upstream that vanishes wherever a query precedes the chunk
    t = torch.arange(L).view(L, 1, 1)
    live = (t >= torch.arange(n).view(1, 1, n) * c)
    g_out0 = g_out * live.to(dtype)
    g_denom0 = g_denom * live.view(L, n).float()
    want0 = orc.chunked_backward(*[inp[k].float() for k in NAMES], g_out0.float(), g_denom0)
    for skip in (False, True):
        got0 = ops.chunked_backward(*ins, out, g_out0.cuda(), g_denom0.cuda(), state=ws, skip_masked=skip)
        torch.cuda.synchronize()
        _report("zero before chunk, skip=%s" % skip, got0, want0, TOL[dtype], tol_dkc)
    got0 = ops.chunked_backward(*ins, out, g_out0.cuda(), g_denom0.cuda(), state=None, recompute=True)
    torch.cuda.synchronize()
    _report("zero before chunk, UA_FLAG_RECOMPUTE", got0, want0, TOL[dtype], tol_dkc)
