"""The autotune table on the GPU (reference: the @triton.autotune wrappers around every launch,
Universal_Attention/triton/universal_attention_kernel.py:10-25, universal_attention_kernel_opt.py:8-36): every variant of
every kernel slot on the default bf16 path meets the oracle; ua_autotune records a choice per slot; the entries shipped
for the benchmark shapes are as fast as what ua_autotune finds on this device (within 3 %)."""
import statistics

import pytest
import torch

from oracle import ua_oracle as orc
from universal_attention_triton_amd import ops
from .util import NAMES, TOL, dense_reference, rel_err

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def _step(a, dO):
    O, lse, ws = ops.fused_forward(*a, keep_state=True)
    g = ops.fused_backward(*a, O, lse, dO, state=ws)
    return O, lse, g


@pytest.mark.parametrize("shape", [(1, 2, 1, 1024 + 64, 128), (1, 2, 4, 512 + 32, 64), (2, 1, 2, 768, 128)])
def test_every_variant_of_every_slot_on_the_default_path_meets_the_oracle(shape):
    b, h, r, L, d = shape
    inp = orc.make_inputs(b, h, r, L, d, 32, dtype=BF, seed=61 + r)
    a = [inp[k].cuda() for k in NAMES]
    dO = inp["dO"].cuda()
    O_ref, lse_ref, g_ref = dense_reference(inp)
    for slot in ("carry", "fwd_tiles", "bwd_parts", "bwd_queries", "bwd_keys"):
        n = ops.tune_variants(a[0], a[2], slot)
        if slot == "bwd_keys":
            assert n == (2 if r == 1 and d > 64 else 1), (slot, n)
        else:
            assert n >= (1 if slot == "bwd_parts" and r == 1 else 2), (slot, n)
        for v in range(n):
            ops.tune_set(a[0], a[2], v, slot)
            try:
                O, lse, g = _step(a, dO)
                torch.cuda.synchronize()
            finally:
                ops.tune_set(a[0], a[2], -1, slot)
            assert rel_err(O, O_ref) <= TOL[BF], (slot, v, rel_err(O, O_ref))
            assert float((lse.cpu().double() - lse_ref).abs().max()) <= 2e-2, (slot, v)
            for name, x, ref in zip(NAMES, g, g_ref):
                assert rel_err(x.reshape(ref.shape), ref) <= TOL[BF], (slot, v, name, rel_err(x.reshape(ref.shape), ref))


def test_recomputing_forward_variants_agree_and_autotune_records_a_choice_per_slot():
    inp = orc.make_inputs(1, 2, 2, 1024 + 64, 128, 32, dtype=BF, seed=51)    # L not a multiple of 128/192/256
    a = [inp[k].cuda() for k in NAMES]
    O_ref, lse_ref, _ = dense_reference(inp)
    n = ops.tune_variants(a[0], a[2], "fwd_recompute")
    assert n >= 2
    results = []
    for v in range(n):
        ops.tune_set(a[0], a[2], v, "fwd_recompute")
        O, lse, _ = ops.fused_forward(*a, recompute=True)
        torch.cuda.synchronize()
        assert rel_err(O, O_ref) <= TOL[BF], (v, rel_err(O, O_ref))
        results.append(O.float().cpu())
    ops.tune_set(a[0], a[2], -1, "fwd_recompute")
    for v in range(1, n):
        assert rel_err(results[v], results[0]) <= 2e-3, v            # same arithmetic, different summation order
    chosen = ops.autotune(*a)
    assert set(chosen) == {"carry", "fwd_tiles", "bwd_parts", "bwd_queries"}, chosen      # r = 2: one key-side variant
    for slot, v in chosen.items():
        assert 0 <= v < ops.tune_variants(a[0], a[2], slot) and ops.tune_choice(a[0], a[2], slot) == v
    O, _, _ = ops.fused_forward(*a)
    assert rel_err(O, O_ref) <= TOL[BF]
    for slot in chosen:
        ops.tune_set(a[0], a[2], -1, slot)


def _median_ms(a, dO, reps=7):
    for _ in range(2):
        _step(a, dO)
    times = []
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        _step(a, dO)
        e1.record()
        e1.synchronize()
        times.append(e0.elapsed_time(e1))
    return statistics.median(times)


@pytest.mark.parametrize("cfg", [(1, 32, 1, 8192, 128, 1002), (1, 8, 4, 4096, 128, 1003)], ids=["config2", "config3"])
def test_shipped_table_is_within_3_percent_of_autotune_on_this_device(cfg):
    b, h, r, L, d, seed = cfg
    inp = orc.make_inputs(b, h, r, L, d, 128, dtype=BF, seed=seed)
    a = [inp[k].cuda() for k in NAMES]
    dO = inp["dO"].cuda()
    slots = [s for s in ("carry", "fwd_tiles", "bwd_parts", "bwd_queries", "bwd_keys") if ops.tune_variants(a[0], a[2], s) > 1]
    shipped = {s: ops.tune_choice(a[0], a[2], s) for s in slots}
    tuned = ops.autotune(*a, dO=dO)
    tuned = {s: tuned[s] for s in slots}
    try:
        if tuned != shipped:
            # alternate between the two tables so that clock and temperature drift hit both alike
            t = {"shipped": [], "tuned": []}
            for _ in range(5):
                for s in slots:
                    ops.tune_set(a[0], a[2], -1, s)
                t["shipped"].append(_median_ms(a, dO))
                for s in slots:
                    ops.tune_set(a[0], a[2], tuned[s], s)
                t["tuned"].append(_median_ms(a, dO))
            med = {k: statistics.median(v) for k, v in t.items()}
            # spread of a table's repeats without its fastest and slowest one (a first run after a switch is often an outlier)
            spread = max((sorted(v)[-2] - sorted(v)[1]) / statistics.median(v) for v in t.values())
            print("shipped", shipped, t["shipped"], "tuned", tuned, t["tuned"], "spread of the repeats %.1f %%" % (100 * spread), flush=True)
            if spread > 0.03:
                pytest.skip("repeats of one table differ by %.1f %% on this device: a 3 %% comparison is not resolved" % (100 * spread))
            assert med["shipped"] <= 1.03 * med["tuned"], (shipped, tuned, t)
    finally:
        for s in slots:
            ops.tune_set(a[0], a[2], -1, s)


def test_every_pairing_of_the_chunked_operator_and_of_the_bias_meets_the_oracle_and_their_tuners_record_a_choice():
    """Slots `chunked_pair` and `aff_pair`: one or two work items per workgroup (or by launch size) give the same results
    to rounding; autotune_chunked / autotune_affinity time the ops and leave a valid choice in the table."""
    from universal_attention_triton_amd.affinity import AffinityScores
    b, h, r, L, d, c = 1, 3, 2, 640, 64, 128                      # 5 key groups, 5 query blocks: odd, so pairs are ragged
    for dtype in (BF, torch.float32):
        inp = orc.make_inputs(b, h, r, L, d, c, dtype=dtype, seed=77)
        a = [inp[k].cuda() for k in NAMES]
        n = L // c
        g = torch.Generator().manual_seed(2)
        g_out = torch.randn(b, h, r, L, d, n, generator=g).to(dtype)
        g_denom = torch.randn(b, h, r, L, n, generator=g).to(dtype).float()
        args32 = [inp[k].float() for k in NAMES]
        out_ref, _ = orc.chunked_forward(*args32)
        want = orc.chunked_backward(*args32, g_out.float(), g_denom)
        assert ops.tune_variants(a[0], a[2], "chunked_pair") == 3
        res = []
        for v in range(3):
            ops.tune_set(a[0], a[2], v, "chunked_pair")
            try:
                out, denom, st = ops.chunked_forward(*a, keep_state=True)
                grads = ops.chunked_backward(*a, out, g_out.cuda(), g_denom.cuda(), state=st)
                torch.cuda.synchronize()
            finally:
                ops.tune_set(a[0], a[2], -1, "chunked_pair")
            assert rel_err(out, out_ref) <= TOL[dtype], (v, rel_err(out, out_ref))
            for name, x, y in zip(NAMES, grads, want):
                if name != "kc" or dtype == BF:                    # the float32 key gradient has its own bars in test_hip_backward
                    assert rel_err(x.reshape(y.shape), y) <= TOL[dtype], (v, name, rel_err(x.reshape(y.shape), y))
            res.append((out,) + tuple(grads))
        for v in (1, 2):
            for x, y in zip(res[v], res[0]):
                assert torch.equal(x, y), v                        # same work items, same order of additions inside each
        chosen = ops.autotune_chunked(*a, repeats=2)
        assert chosen.keys() == {"chunked_pair"} and 0 <= chosen["chunked_pair"] < 3
        assert ops.tune_get(a[0], a[2], "chunked_pair") == chosen["chunked_pair"]
        ops.tune_set(a[0], a[2], -1, "chunked_pair")
        # the stand-alone bias
        k = inp["kc"].reshape(b, h, L, d).cuda()
        src, dest = inp["static_src"].reshape(b, h, L).cuda(), inp["static_dest"].cuda()
        daff = torch.randn(b, h, L, L, generator=g).to(dtype).cuda()
        desc = ops._affinity_args(k, src, dest)[3]
        import ctypes
        from universal_attention_triton_amd import _lib
        lib = _lib.load()
        assert lib.ua_tune_variants(ctypes.byref(desc), _lib.UA_TUNE_AFF_PAIR) == 3
        res = []
        for v in range(3):
            _lib.check(lib.ua_tune_set(ctypes.byref(desc), _lib.UA_TUNE_AFF_PAIR, v), "ua_tune_set")
            try:
                aff = ops.affinity_forward(k, src, dest)
                res.append((aff,) + tuple(ops.affinity_backward(k, src, dest, daff)))
                torch.cuda.synchronize()
            finally:
                lib.ua_tune_set(ctypes.byref(desc), _lib.UA_TUNE_AFF_PAIR, -1)
        for v in (1, 2):
            for x, y in zip(res[v], res[0]):
                assert torch.equal(x, y), v
        leaves = [t.detach().requires_grad_() for t in (k, src, dest)]
        assert torch.equal(AffinityScores.apply(*leaves), res[0][0])          # checked against the oracle in test_hip_affinity
        chosen = ops.autotune_affinity(k, src, dest, repeats=2)
        assert 0 <= chosen["aff_pair"] < 3 and lib.ua_tune_get(ctypes.byref(desc), _lib.UA_TUNE_AFF_PAIR) == chosen["aff_pair"]
        lib.ua_tune_set(ctypes.byref(desc), _lib.UA_TUNE_AFF_PAIR, -1)


def test_first_call_autotune_is_opt_in_through_the_environment(monkeypatch):
    """UA_AUTOTUNE=1: the fused operator tunes itself the first time it meets a table key, once; without the variable it
    never does."""
    from universal_attention_triton_amd.universal_attention import universal_attention
    inp = orc.make_inputs(1, 2, 1, 384, 128, 128, dtype=BF, seed=5)
    a = [inp[k].cuda() for k in NAMES]
    slots = [s for s in ("carry", "fwd_tiles", "bwd_queries", "bwd_keys") if ops.tune_variants(a[0], a[2], s) > 1]
    O_ref, _, _ = dense_reference(inp)
    monkeypatch.delenv("UA_AUTOTUNE", raising=False)
    ops._first_call_tuned.clear()
    universal_attention(*a)
    assert all(ops.tune_get(a[0], a[2], s) == -1 for s in slots) and not ops._first_call_tuned
    monkeypatch.setenv("UA_AUTOTUNE", "1")
    calls = []
    real = ops.autotune
    monkeypatch.setattr(ops, "autotune", lambda *x, **kw: (calls.append(1), real(*x, **kw))[1])
    try:
        leaves = [t.clone().requires_grad_() for t in a]
        O = universal_attention(*leaves)
        O2 = universal_attention(*leaves)                 # same key: no second tuning run
        assert len(calls) == 1 and all(ops.tune_get(a[0], a[2], s) >= 0 for s in slots)
        assert rel_err(O, O_ref) <= TOL[BF] and torch.equal(O, O2)
        torch.autograd.grad(O, leaves, inp["dO"].cuda())
    finally:
        for s in slots:
            ops.tune_set(a[0], a[2], -1, s)
        ops._first_call_tuned.clear()


@pytest.mark.parametrize("prune", [False, True])
@pytest.mark.parametrize("shape", [(1, 2, 1, 1024 + 96, 100), (2, 1, 1, 2048, 128), (1, 3, 1, 130, 72), (1, 36, 1, 1920 - 40, 128)])
def test_key_side_variant_with_32_keys_per_wave_on_ragged_shapes_and_with_pruning(shape, prune):
    """Slot `bwd_keys`, variant 1 (one wave per SIMD, 32x32 tiles) against variant 0 and the oracle: L no multiple of 128,
    padded head dims, gates that make the decay fast (so that UA_FLAG_PRUNE shortens the sweeps of both variants); the
    last shape is a launch of at least two workgroups per CU, whose workgroups sweep two key groups each (15 groups: the
    middle one alone)."""
    b, h, r, L, d = shape
    inp = orc.make_inputs(b, h, r, L, d, 2, dtype=BF, seed=17, gate_mean=2.0)
    k = inp["kc"].float() + 2.0 * inp["kc"].float()[:, :, :1, :1, :]              # correlated keys: fast decay
    inp["kc"] = (k / k.norm(dim=-1, keepdim=True)).to(BF)
    a = [inp[k_].cuda() for k_ in NAMES]
    dO = inp["dO"].cuda()
    O_ref, _, g_ref = dense_reference(inp)
    assert ops.tune_variants(a[0], a[2], "bwd_keys") == 2
    res = []
    for v in (0, 1):
        ops.tune_set(a[0], a[2], v, "bwd_keys")
        try:
            O, lse, ws = ops.fused_forward(*a, keep_state=True, prune=prune)
            res.append(ops.fused_backward(*a, O, lse, dO, state=ws, prune=prune))
            torch.cuda.synchronize()
        finally:
            ops.tune_set(a[0], a[2], -1, "bwd_keys")
    for name, x0, x1, ref in zip(NAMES, res[0], res[1], g_ref):
        assert torch.isfinite(x1.float()).all(), name
        assert rel_err(x1, x0) <= 6e-3, (name, rel_err(x1, x0))
        assert rel_err(x1.reshape(ref.shape), ref) <= TOL[BF], (name, rel_err(x1.reshape(ref.shape), ref))
