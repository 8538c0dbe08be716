"""Paths of the drop-in that share kernels with the main ones but have host code of their own: backward through the
2-D layout (reference UniversalAttention2.backward, universal_attention_autograd.py:172-276, and the Triton-side entry,
Universal_Attention/universal_attention.py:34-46) with query chunks that differ from the key chunks; all five gradients
through the (q, k, v) calling convention (universal_attention_kernel_opt.py:504-581); gates in another dtype than
q, k, v (universal_attention_kernel.py:825-829); well-conditioned float32 keys held to the plain 1e-4; what stays
allocated between forward and backward."""
import pytest
import torch

from oracle import ua_oracle as orc
from tests.util import NAMES, TOL, dense_reference, load_golden, rel_err

pytestmark = pytest.mark.gpu
GRADS = ("dkc", "dvc", "dxq", "dsrc", "ddest")


def _table(tag, got, want, tol):
    """tol: one bar for the five gradients, or {gradient: bar} (missing names take the "*" entry)"""
    errs = {n: rel_err(g.reshape(w.shape), w) for n, g, w in zip(GRADS, got, want)}
    bars = {n: (tol.get(n, tol.get("*")) if isinstance(tol, dict) else tol) for n in GRADS}
    print(tag, {k: "%.2e (bar %.1e)" % (v, bars[k]) for k, v in errs.items()}, flush=True)
    bad = {k: (v, bars[k]) for k, v in errs.items() if not v <= bars[k]}
    assert not bad, (tag, bad)


def _fp32_key_gradient_bar(oracle_dkc, exact_dkc):
    """float32 bar of the key gradient: d/dG relu(G)^(2/3) is singular at G -> 0+, and the reference's own float32
    operator misses float64 by more than 1e-4 on random keys; the kernel gets twice the error of the oracle's float32
    restatement on the same inputs, and never less than the plain 1e-4.  Every other gradient is held to 1e-4."""
    return max(1e-4, 2 * rel_err(oracle_dkc, exact_dkc))


@pytest.mark.parametrize("entry", ["autograd2", "triton_side"])
@pytest.mark.parametrize("name", ["tiny2d_fp32", "tiny2d_bf16"])
def test_backward_through_the_2d_layout_matches_reference_golden(name, entry):
    """Key chunks of 16, query chunks of 32, arbitrary (g_out, g_denom): the reference's UniversalAttention2 wrote these."""
    import numpy as np
    import os
    from universal_attention_triton_amd import universal_attention_autograd as ua
    from universal_attention_triton_amd.universal_attention import UniversalAttention as TritonSide
    t, dtype, (b, h, r, l, d, c, seed) = load_golden(name)
    qc = int(np.load(os.path.join(os.path.dirname(__file__), "golden", name + ".npz"))["qc"][0])
    tol = TOL[dtype]
    fn = ua.UniversalAttention2 if entry == "autograd2" else TritonSide
    xq2 = t["xq"].to(dtype).view(b, h, r, l // qc, qc, d)
    sd2 = t["static_dest"].to(dtype).view(b, h, l // qc, qc)
    leaves = [x.cuda().requires_grad_() for x in (t["kc"].to(dtype), t["vc"].to(dtype), xq2, t["static_src"].to(dtype), sd2)]
    out, denom = fn.apply(*leaves)
    assert out.shape == (b, h, r, l, d, l // c) and denom.shape == (b, h, r, l, l // c)
    grads = torch.autograd.grad([out, denom], leaves, [t["g_out"].to(dtype).cuda(), t["g_denom"].to(dtype).cuda()])
    torch.cuda.synchronize()
    assert grads[2].shape == xq2.shape and grads[4].shape == sd2.shape
    assert rel_err(out, t["out"]) <= tol
    _table("2-D layout %s %s" % (name, entry), grads, [t[n] for n in GRADS], tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_backward_through_the_2d_layout_matches_oracle_larger_case(dtype):
    """Chunk 64 keys x 32 queries, L = 256, arbitrary upstream: against the oracle's restatement of the 1-D backward."""
    from universal_attention_triton_amd import universal_attention_autograd as ua
    b, h, r, L, d, c, qc = 1, 2, 2, 256, 64, 64, 32
    inp = orc.make_inputs(b, h, r, L, d, c, dtype=dtype, seed=71)
    g = torch.Generator().manual_seed(9)
    g_out = torch.randn(b, h, r, L, d, L // c, generator=g).to(dtype)
    g_denom = torch.randn(b, h, r, L, L // c, generator=g).to(dtype)
    want = orc.chunked_backward(*[inp[k].float() for k in NAMES], g_out.float(), g_denom.float())
    tol = TOL[dtype]
    if dtype == torch.float32:
        # arbitrary upstream on the chunked operator: the -1e12 fill only swamps the score in float32, so float64 cannot
        # serve; the restatement's own float32 error in the key gradient is measured as its largest move under other
        # summation orders of the head dimension (same mathematics, other rounding of the key-key products)
        from tests.test_hip_backward import _summation_order_sensitivity
        tol = {"*": 1e-4, "dkc": max(1e-4, 2 * _summation_order_sensitivity(inp, g_out, g_denom.float(), want[0]))}
    xq2 = inp["xq"].view(b, h, r, L // qc, qc, d)
    sd2 = inp["static_dest"].view(b, h, L // qc, qc)
    leaves = [x.cuda().requires_grad_() for x in (inp["kc"], inp["vc"], xq2, inp["static_src"], sd2)]
    out, denom = ua.UniversalAttention2.apply(*leaves)
    grads = torch.autograd.grad([out, denom], leaves, [g_out.cuda(), g_denom.cuda()])
    torch.cuda.synchronize()
    _table("2-D layout oracle %s" % dtype, grads, want, tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_all_five_gradients_through_the_qkv_calling_convention(dtype):
    """attention(q, k, v, ...): r-major grouped queries (query head j uses kv head j % H_kv), head dim 80, ragged L;
    forward and backward against float64 autograd of the dense oracle; ac=True (keep no state) gives the same."""
    from universal_attention_triton_amd.universal_attention import attention
    B, Hkv, r, L, d = 1, 2, 3, 200, 80
    inp = orc.make_inputs(B, Hkv, r, L, d, 8, dtype=dtype, seed=43)
    O_ref, _, g_ref = dense_reference(inp)
    tol = TOL[dtype]
    if dtype == torch.float32:
        out32, denom32 = orc.chunked_forward(*[inp[k_] for k_ in NAMES])
        d_out, d_denom = orc.merge_backward(out32, denom32, inp["dO"])
        tol = {"*": 1e-4, "dkc": _fp32_key_gradient_bar(orc.chunked_backward(*[inp[k_] for k_ in NAMES], d_out, d_denom)[0], g_ref[0])}
    k = inp["kc"].reshape(B, Hkv, L, d).cuda().requires_grad_()
    v = inp["vc"].reshape(B, Hkv, L, d).cuda().requires_grad_()
    q = inp["xq"].transpose(1, 2).reshape(B, r * Hkv, L, d).cuda().requires_grad_()       # head j = rep * Hkv + kv
    src = inp["static_src"].reshape(B, Hkv, L).cuda().requires_grad_()
    dest = inp["static_dest"].cuda().requires_grad_()
    dO = inp["dO"].transpose(1, 2).reshape(B, r * Hkv, L, d).cuda()
    results = []
    for ac in (False, True):
        o = attention(q, k, v, True, 0.5, src, dest, ac=ac)
        gq, gk, gv, gs, gd = torch.autograd.grad(o, [q, k, v, src, dest], dO)
        torch.cuda.synchronize()
        assert rel_err(o.view(B, r, Hkv, L, d).transpose(1, 2), O_ref) <= TOL[dtype]
        got = [gk, gv, gq.view(B, r, Hkv, L, d).transpose(1, 2), gs, gd]
        _table("attention() %s ac=%s" % (dtype, ac), got, g_ref, tol)
        results.append(got)
    for a_, b_ in zip(*results):
        assert rel_err(a_, b_) <= (1e-5 if dtype == torch.float32 else 2e-3)


def test_fp32_key_gradient_meets_1e4_on_well_conditioned_keys():
    """d/dG relu(G)^(2/3) is singular at G -> 0+, which is why the other float32 tests give dkc a wider bar.  With keys in
    the positive orthant every product k_s.k_u is well above 1e-3 and every tensor, dkc included, meets the plain 1e-4,
    through the fused and the chunked operator."""
    from universal_attention_triton_amd import universal_attention_autograd as ua
    from universal_attention_triton_amd.universal_attention import universal_attention
    b, h, r, L, d, c = 1, 2, 2, 320, 64, 64
    inp = orc.make_inputs(b, h, r, L, d, c, dtype=torch.float32, seed=77)
    k = inp["kc"].abs() + 0.05
    inp["kc"] = k / k.norm(dim=-1, keepdim=True)
    flat = inp["kc"].reshape(b, h, L, d)
    assert float((flat @ flat.transpose(-1, -2)).min()) > 1e-3
    O_ref, _, g_ref = dense_reference(inp)
    leaves = [inp[k_].cuda().requires_grad_() for k_ in NAMES]
    O = universal_attention(*leaves)
    grads = torch.autograd.grad(O, leaves, inp["dO"].cuda())
    torch.cuda.synchronize()
    assert rel_err(O, O_ref) <= 1e-4
    _table("fused fp32 positive keys", grads, g_ref, 1e-4)
    leaves = [inp[k_].cuda().requires_grad_() for k_ in NAMES]
    out, denom = ua.UniversalAttention.apply(*leaves)
    O2 = ua.SMVecMatMul.apply(out, denom)
    grads2 = torch.autograd.grad(O2, leaves, inp["dO"].cuda())
    torch.cuda.synchronize()
    _table("chunked fp32 positive keys", grads2, g_ref, 1e-4)


@pytest.mark.parametrize("gates", ["fp32_both", "fp32_src_only"])
def test_float32_gates_next_to_bf16_tensors(gates):
    """The reference allocates dstatic_src in static_src.dtype and everything else in xq.dtype, i.e. float32 gates next to
    bf16 q, k, v are legal.  Checked against float64 autograd of the dense oracle on the same mixed-dtype inputs (the
    gates are NOT rounded to bf16), through the fused and the chunked operator; gradients come back in the gates' dtypes."""
    from universal_attention_triton_amd import universal_attention_autograd as ua
    from universal_attention_triton_amd.universal_attention import universal_attention
    b, h, r, L, d, c = 1, 2, 2, 256, 64, 64
    bf = torch.bfloat16
    inp = orc.make_inputs(b, h, r, L, d, c, dtype=torch.float32, seed=81)
    mixed = {k_: (inp[k_].to(bf) if k_ in ("kc", "vc", "xq") else inp[k_].clone()) for k_ in NAMES}
    if gates == "fp32_src_only":
        mixed["static_dest"] = mixed["static_dest"].to(bf)
    mixed["dO"] = inp["dO"].to(bf)
    # gates whose bf16 rounding would be visible: the result must follow the float32 values
    O_ref, _, g_ref = dense_reference(mixed)
    O_rounded, _, _ = dense_reference({k_: (v.to(bf) if k_ != "dO" else v) for k_, v in mixed.items()})
    leaves = [mixed[k_].cuda().requires_grad_() for k_ in NAMES]
    O = universal_attention(*leaves)
    grads = torch.autograd.grad(O, leaves, mixed["dO"].cuda())
    torch.cuda.synchronize()
    assert O.dtype == bf and grads[3].dtype == mixed["static_src"].dtype and grads[4].dtype == mixed["static_dest"].dtype
    assert rel_err(O, O_ref) <= TOL[bf]
    _table("fused mixed dtypes " + gates, grads, g_ref, TOL[bf])
    leaves = [mixed[k_].cuda().requires_grad_() for k_ in NAMES]
    out, denom = ua.UniversalAttention.apply(*leaves)
    O2 = ua.SMVecMatMul.apply(out, denom)
    grads2 = torch.autograd.grad(O2, leaves, mixed["dO"].cuda())
    torch.cuda.synchronize()
    assert grads2[3].dtype == mixed["static_src"].dtype
    _table("chunked mixed dtypes " + gates, grads2, g_ref, TOL[bf])
    if gates == "fp32_both":
        # the float32 gates are really used: the fused result is closer to the float32-gate oracle than the
        # oracle with rounded gates is
        assert rel_err(O, O_ref) < rel_err(O_rounded, O_ref) or rel_err(O_rounded, O_ref) < 2e-3


def test_memory_kept_between_forward_and_backward_at_the_headline_shape():
    """BASELINE config 2 (b=1 h=32 L=8192 d=128 bf16): between forward and backward the fused operator holds its inputs,
    O, lse and the forward state (packed inputs + bias tiles, <= 2.6 GB); the 4.8 GB of backward scratch only exist inside
    backward; keep_state=False holds nothing beyond inputs, O and lse."""
    from universal_attention_triton_amd import ops
    from universal_attention_triton_amd.universal_attention import universal_attention
    b, h, r, L, d = 1, 32, 1, 8192, 128
    inp = orc.make_inputs(b, h, r, L, d, 128, dtype=torch.bfloat16, seed=1002)
    leaves = [inp[k_].cuda().requires_grad_() for k_ in NAMES]
    dO = inp["dO"].cuda()
    torch.cuda.synchronize()
    base = torch.cuda.memory_allocated()
    out_bytes = b * h * r * L * d * 2 + b * h * r * L * 4
    for keep, budget in ((True, int(2.6e9)), (False, 0)):
        O = universal_attention(*leaves, keep_state=keep)
        torch.cuda.synchronize()
        held = torch.cuda.memory_allocated() - base
        assert held <= out_bytes + budget + (8 << 20), (keep, held)
        if keep:
            assert held >= out_bytes + ops.retained_bytes(*[x.detach() for x in leaves]) - (8 << 20)
        torch.cuda.reset_peak_memory_stats()
        grads = torch.autograd.grad(O, leaves, dO)
        torch.cuda.synchronize()
        peak = torch.cuda.max_memory_allocated() - base
        assert peak > held + int(4e9)            # the scratch lived inside backward only
        if keep:
            # ... and nothing of the state's size besides it: autograd must not make up a zero gradient for the hidden
            # state output (scratch 4.8 GB + the five gradients 0.27 GB + packed copies of O / dO)
            assert peak <= held + int(5.6e9), (peak, held)
        del O, grads
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() - base <= (8 << 20)


def test_memory_kept_between_forward_and_backward_by_the_chunked_functions():
    """bf16, b=1 h=8 L=4096 d=128 chunk 128: between forward and backward the chunked Function holds its inputs, `out`,
    `denom` (what the reference holds too) and, by default, the forward state (ops.retained_bytes(chunked=True): packed
    inputs, decay carries, normalisers); with "normalisers" only those (1/(d+1) of `out`), with False nothing more."""
    from universal_attention_triton_amd import ops
    from universal_attention_triton_amd import universal_attention_autograd as ua
    b, h, r, L, d, c = 1, 8, 1, 4096, 128, 128
    n = L // c
    inp = orc.make_inputs(b, h, r, L, d, c, dtype=torch.bfloat16, seed=1003)
    leaves = [inp[k_].cuda().requires_grad_() for k_ in NAMES]
    torch.cuda.synchronize()
    base = torch.cuda.memory_allocated()
    out_bytes = b * h * r * L * (d + 1) * n * 2
    state = ops.retained_bytes(*[x.detach() for x in leaves], chunked=True)
    assert state < out_bytes // 3
    slack = 8 << 20
    for keep, extra in ((True, state), ("normalisers", b * h * r * n * L * 4), (False, 0)):
        with ua.chunked_options(keep_state=keep):
            out, denom = ua.UniversalAttention.apply(*leaves)
        torch.cuda.synchronize()
        held = torch.cuda.memory_allocated() - base
        assert out_bytes + extra - slack <= held <= out_bytes + extra + slack, (keep, held, out_bytes, extra)
        grads = torch.autograd.grad([out, denom], leaves, [torch.ones_like(out), torch.zeros_like(denom)])
        del out, denom, grads
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() - base <= slack


@pytest.mark.parametrize("shape", [(1, 2, 1, 320, 160), (1, 1, 2, 200, 256), (2, 1, 4, 128, 136)])
def test_head_dims_above_128_bf16_fused_operator(shape):
    """The reference's second-generation kernel takes head dims up to 256 (zero-padded to a power of two,
    universal_attention_kernel_opt.py:441-456): forward and the five gradients at d = 160, 256 and 136 (r = 1, 2, 4)
    against float64 autograd of the dense oracle; float32 and the chunked operator refuse such head dims."""
    from universal_attention_triton_amd import _lib, ops
    from universal_attention_triton_amd.universal_attention import universal_attention
    b, h, r, L, d = shape
    bf = torch.bfloat16
    inp = orc.make_inputs(b, h, r, L, d, 8, dtype=bf, seed=91)
    O_ref, lse_ref, g_ref = dense_reference(inp)
    leaves = [inp[k_].cuda().requires_grad_() for k_ in NAMES]
    O, lse = universal_attention(*leaves, return_lse=True)
    grads = torch.autograd.grad(O, leaves, inp["dO"].cuda())
    torch.cuda.synchronize()
    assert rel_err(O, O_ref) <= TOL[bf], rel_err(O, O_ref)
    assert float((lse.cpu().double() - lse_ref).abs().max()) <= 2e-2
    _table("head dim %d" % d, grads, g_ref, TOL[bf])
    with pytest.raises(_lib.UaError):
        ops.fused_forward(*[x.detach().float() for x in leaves])
    with pytest.raises(_lib.UaError):
        ops.chunked_forward(*[x.detach() for x in leaves])


@pytest.mark.parametrize("recompute", [False, True])
def test_large_scores_and_deep_decay_bf16(recompute):
    """Unscaled scores of +-25 and gates near one: rows whose weight sits on keys with a decay bias of -20 to -40 (in
    log2 units).  The default bf16 path hands the bias from kernel to kernel as fp16 tiles (resolution 2^-6 between 16 and
    32, 2^-5 up to 64); the recomputing path keeps it in float32.  Both must meet the float64 dense oracle."""
    from universal_attention_triton_amd import ops
    bf = torch.bfloat16
    b, h, r, L, d = 1, 2, 1, 768, 64
    inp = orc.make_inputs(b, h, r, L, d, 64, dtype=bf, seed=95, gate_mean=2.0)
    inp["xq"] = (inp["xq"].float() * 8).to(bf)
    # make the decay deep: similar keys prune one another quickly
    k = inp["kc"].float().reshape(b, h, L, d)
    k = k * 0.5 + k.mean(dim=2, keepdim=True) * 4
    inp["kc"] = (k / k.norm(dim=-1, keepdim=True)).reshape(inp["kc"].shape).to(bf)
    O_ref, lse_ref, g_ref = dense_reference(inp)
    bias = orc.dense_bias(inp["kc"].double().reshape(b, h, L, d), inp["static_src"].double().reshape(b, h, L),
                          inp["static_dest"].double().reshape(b, h, L))
    scores = torch.einsum("bhsd,bhrtd->bhrst", inp["kc"].double().reshape(b, h, L, d), inp["xq"].double())
    causal = torch.ones(L, L, dtype=torch.bool).triu()                    # [s, t]: s <= t
    w = torch.softmax((scores + bias.unsqueeze(2)).masked_fill(~causal, float("-inf")), dim=-2)
    top = w.argmax(dim=-2)                                                # key carrying the most weight per query
    top_bias = bias.unsqueeze(2).expand_as(w).gather(-2, top.unsqueeze(-2)).squeeze(-2) / 0.6931471805599453
    print("scores up to %.1f, bias of the heaviest key: median %.1f, min %.1f (log2 units)"
          % (float(scores.abs().max()), float(top_bias.median()), float(top_bias.min())), flush=True)
    assert float(scores.abs().max()) > 15 and float(top_bias.min()) < -20
    dev = {k_: v.cuda() for k_, v in inp.items()}
    a = [dev[k_] for k_ in NAMES]
    O, lse, state = ops.fused_forward(*a, keep_state=True, recompute=recompute)
    grads = ops.fused_backward(*a, O, lse, dev["dO"], state=state, recompute=recompute)
    torch.cuda.synchronize()
    assert rel_err(O, O_ref) <= TOL[bf], rel_err(O, O_ref)
    _table("large scores recompute=%s" % recompute, grads, g_ref, TOL[bf])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_out_allocated_contiguous_like_the_reference(dtype):
    """`out` is normally a permuted view of chunk-major storage; with contiguous_out it is the reference's own layout
    (so `.view()` works on it), with the same values, and the backward reads it and a contiguous gradient alike."""
    from universal_attention_triton_amd import universal_attention_autograd as ua
    print("case contiguous out", dtype, flush=True)
    b, h, r, L, d, c = 1, 2, 2, 256, 32, 64
    n = L // c
    inp = orc.make_inputs(b, h, r, L, d, c, dtype=dtype, seed=77)
    g = torch.Generator().manual_seed(9)
    g_out = torch.randn(b, h, r, L, d, n, generator=g).to(dtype)
    g_denom = torch.randn(b, h, r, L, n, generator=g).to(dtype)
    results = []
    for contiguous in (False, True):
        leaves = [inp[k].cuda().requires_grad_() for k in NAMES]
        with ua.chunked_options(contiguous_out=contiguous):
            out, denom = ua.UniversalAttention.apply(*leaves)
        assert out.shape == (b, h, r, L, d, n)
        assert out.is_contiguous() == contiguous
        if contiguous:
            out.view(b * h * r, L, d * n)            # what fails on the permuted view
        grads = torch.autograd.grad([out, denom], leaves, [g_out.cuda(), g_denom.cuda()])
        torch.cuda.synchronize()
        results.append((out.detach().clone(), denom.detach().clone(), grads))
    (o0, d0, g0), (o1, d1, g1) = results
    assert torch.equal(o0, o1) and torch.equal(d0, d1)
    for name, x, y in zip(NAMES, g0, g1):
        assert rel_err(y, x) <= 1e-6, (name, rel_err(y, x))
    # the default layout is checked against the oracle in test_hip_backward.py; here the other four gradients once more
    # (float32 dkc has its own bar there: the singular derivative of relu(G)^(2/3))
    want = orc.chunked_backward(*[inp[k].float() for k in NAMES], g_out.float(), g_denom.float())
    for name, x, w in zip(NAMES, g1, want):
        if name != "kc":
            assert rel_err(x.reshape(w.shape), w) <= TOL[dtype], (name, rel_err(x.reshape(w.shape), w))


@pytest.mark.parametrize("dtype,c", [(torch.float32, 64), (torch.bfloat16, 128), (torch.bfloat16, 32)])
def test_what_the_chunked_function_keeps_for_its_backward_does_not_change_the_gradients(dtype, c):
    """The chunked Functions keep the whole forward state by default; with only the normalisers, or nothing, the
    backward rebuilds what it misses from the five inputs and must arrive at the same gradients, bit for bit where
    the kernels add in a fixed order (chunk a multiple of 64; the others add up dq with atomics)."""
    from universal_attention_triton_amd import universal_attention_autograd as ua
    print("case chunked keep modes", dtype, c, flush=True)
    b, h, r, L, d = 1, 2, 2, 384, 64
    n = L // c
    inp = orc.make_inputs(b, h, r, L, d, c, dtype=dtype, seed=31)
    g = torch.Generator().manual_seed(5)
    g_out = torch.randn(b, h, r, L, d, n, generator=g).to(dtype).cuda()
    g_denom = torch.randn(b, h, r, L, n, generator=g).to(dtype).cuda()
    results = []
    for keep in (True, "normalisers", False):
        leaves = [inp[k].cuda().requires_grad_() for k in NAMES]
        with ua.chunked_options(keep_state=keep):
            out, denom = ua.UniversalAttention.apply(*leaves)
        # the backward runs outside the block: it uses what its forward saw
        grads = torch.autograd.grad([out, denom], leaves, [g_out, g_denom])
        torch.cuda.synchronize()
        results.append((out.detach().clone(), grads))
    for o, grads in results[1:]:
        assert torch.equal(o, results[0][0])
        for name, x, y in zip(NAMES, grads, results[0][1]):
            assert torch.equal(x, y) if c % 64 == 0 else rel_err(x, y) <= 2.0 ** -7, (name, rel_err(x, y))
    want = orc.chunked_backward(*[inp[k].float() for k in NAMES], g_out.float().cpu(), g_denom.float().cpu())
    for name, x, w in zip(NAMES, results[0][1], want):
        if name != "kc" or dtype == torch.bfloat16:      # float32 dkc has its own bar in test_hip_backward.py
            assert rel_err(x.reshape(w.shape), w) <= TOL[dtype], (name, rel_err(x.reshape(w.shape), w))


@pytest.mark.parametrize("shape", [(1, 2, 2, 512, 64, 64), (1, 1, 1, 768, 128, 192), (2, 1, 1, 256, 128, 128)])
def test_upstream_gradient_read_in_place_equals_its_packed_copy(shape):
    """bf16, chunk a multiple of 64, nothing flowing to (query, later chunk) pairs: a chunk-major upstream gradient with
    rows of exactly the padded head dim is gathered by the key-side kernel from the caller's tensor; any other storage
    goes through a packed copy.  Same tiles either way; delta = sum_d out * g_out is summed in another order for the
    other storage (float32 rounding), which flips the last bf16 bit of a handful of gradient elements."""
    from universal_attention_triton_amd import ops
    print("case g_out in place", shape, flush=True)
    b, h, r, L, d, c = shape
    n = L // c
    dtype = torch.bfloat16
    inp = orc.make_inputs(b, h, r, L, d, c, dtype=dtype, seed=55)
    gen = torch.Generator().manual_seed(3)
    live = (torch.arange(L).view(L, 1, 1) >= torch.arange(n).view(1, 1, n) * c)
    g_ref_order = (torch.randn(b, h, r, L, d, n, generator=gen) * live).to(dtype).cuda()          # contiguous [.., L, d, n]
    g_denom = (torch.randn(b, h, r, L, n, generator=gen) * live.view(L, n)).to(dtype).float().cuda()
    ins = [inp[k].cuda() for k in NAMES]
    out, denom, state = ops.chunked_forward(*ins, keep_state=True)
    g_chunk_major = g_ref_order.permute(0, 1, 2, 5, 3, 4).contiguous().permute(0, 1, 2, 4, 5, 3)  # same values, [.., n, L, d] storage
    assert torch.equal(g_chunk_major, g_ref_order) and not g_chunk_major.is_contiguous()
    got_in_place = ops.chunked_backward(*ins, out, g_chunk_major, g_denom, state=state, skip_masked=True)
    got_packed = ops.chunked_backward(*ins, out, g_ref_order, g_denom, state=state, skip_masked=True)
    torch.cuda.synchronize()
    for name, x, y in zip(NAMES, got_in_place, got_packed):
        assert rel_err(x, y) <= 1e-4, (name, rel_err(x, y))
        assert int((x != y).sum()) <= x.numel() // 1000, (name, int((x != y).sum()))
    want = orc.chunked_backward(*[inp[k].float() for k in NAMES], g_ref_order.float().cpu(), g_denom.cpu())
    for name, x, w in zip(NAMES, got_in_place, want):
        assert rel_err(x.reshape(w.shape), w) <= TOL[dtype], (name, rel_err(x.reshape(w.shape), w))


@pytest.mark.parametrize("shape", [(1, 176, 1, 640, 64), (1, 88, 2, 896, 128)])
def test_launches_of_paired_work_items_with_an_odd_number_of_items(shape):
    """Launches with at least two workgroups per CU pair their work items (the key-stationary backward sweeps key groups
    g and last - g in one workgroup, the forward over bias tiles query blocks j and last - j): here the number of items is
    odd, so the middle one stays alone (5 or 7 key groups, 3 or 4 query blocks), and several heads spread over the
    launch are held to the float64 dense oracle."""
    from universal_attention_triton_amd import ops
    b, h, r, L, d = shape
    bf = torch.bfloat16
    inp = orc.make_inputs(b, h, r, L, d, L, dtype=bf, seed=4242, gate_mean=0.0)
    dev = {k: v.cuda() for k, v in inp.items()}
    a = [dev[k] for k in NAMES]
    O, lse, state = ops.fused_forward(*a, keep_state=True)
    grads = ops.fused_backward(*a, O, lse, dev["dO"], state=state)
    torch.cuda.synchronize()
    for hh in (0, 1, h // 2, h - 1):
        one = {k: v[:, hh:hh + 1] for k, v in inp.items()}
        O_ref, lse_ref, g_ref = dense_reference(one)
        assert rel_err(O[:, hh:hh + 1], O_ref) <= TOL[bf], hh
        assert float((lse[:, hh:hh + 1].cpu().double() - lse_ref).abs().max()) <= TOL[bf], hh
        _table("head %d of %s" % (hh, (shape,)), [x[:, hh:hh + 1] for x in grads], g_ref, TOL[bf])


def test_workspace_of_a_forward_that_also_wrote_the_normalisers_out_is_a_complete_state():
    """ua_fwd with lse2_out leaves a copy of the normalisers in the workspace, so that workspace alone (fwd_state
    without lse2_in) gives ua_bwd everything: same gradients, bit for bit, as after a forward without lse2_out."""
    import ctypes
    from universal_attention_triton_amd import _lib, ops
    b, h, r, L, d, c = 1, 2, 2, 384, 64, 128
    n = L // c
    dtype = torch.bfloat16
    inp = orc.make_inputs(b, h, r, L, d, c, dtype=dtype, seed=91)
    ins = [inp[k].cuda() for k in NAMES]
    gen = torch.Generator().manual_seed(4)
    g_out = torch.randn(b, h, r, L, d, n, generator=gen).to(dtype).cuda()
    g_denom = torch.randn(b, h, r, L, n, generator=gen).to(dtype).float().cuda()
    out_ref, denom_ref, state_ref = ops.chunked_forward(*ins, keep_state=True)
    want = ops.chunked_backward(*ins, out_ref, g_out, g_denom, state=state_ref)
    # the same forward through the C entry point with lse2_out, then the backward on its workspace
    lib = _lib.load()
    kc, vc, xq, src, dest, gflag = ops._prep(*ins)
    desc = ops._desc(kc, xq, True, gflag)
    ws = ops._workspace(desc, _lib.UA_OP_FWD, xq.device)
    ws.fill_(0x7f)                                                   # nothing may be left to chance
    out = torch.empty(b, h, r, n, L, d, dtype=dtype, device="cuda").permute(0, 1, 2, 4, 5, 3)
    denom = torch.empty(b, h, r, L, n, dtype=dtype, device="cuda")
    lse2 = torch.empty(b * h * r * n * (-(-L // 128) * 128), dtype=torch.float32, device="cuda")
    _, oc = ops._chunked(out)
    _lib.check(lib.ua_fwd(ctypes.byref(desc), ctypes.byref(ops._rows_k(kc)), ctypes.byref(ops._rows_k(vc)), ctypes.byref(ops._rows_q(xq)),
                          src.data_ptr(), dest.data_ptr(), ctypes.byref(oc), denom.data_ptr(), lse2.data_ptr(), ws.data_ptr(),
                          ws.numel(), ops._stream()), "ua_fwd")
    assert torch.equal(out, out_ref) and torch.equal(denom, denom_ref)
    got = ops.chunked_backward(*ins, out, g_out, g_denom, state=ws)
    torch.cuda.synchronize()
    for name, x, y in zip(NAMES, got, want):
        assert torch.equal(x, y), (name, rel_err(x, y))
