"""CPU checks of the C ABI: the shared library loads, exports every symbol include/ua.h declares, and rejects
bad descriptors / workspaces with error codes (no kernel is launched here)."""
import ctypes
import os
import re

import pytest

from universal_attention_triton_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "ua.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ua_[a-z_0-9]+)\s*\(", text)))


def test_library_loads_and_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared_symbols()
    assert "ua_fused_fwd" in names and "ua_bwd" in names and len(names) >= 14
    for n in names:
        assert hasattr(lib, n), n
        assert n in _lib.SIGNATURES, "ctypes signature missing for " + n
    assert lib.ua_version() >= 1


def test_descriptor_validation_and_workspace_sizes():
    lib = _lib.load()
    ok = _lib.UaDesc(1, 32, 1, 8192, 128, 128, _lib.UA_BF16, 0)
    sizes = [lib.ua_workspace_bytes(ctypes.byref(ok), op) for op in range(4)]
    assert all(s > 0 for s in sizes) and sizes[1] >= sizes[0] and sizes[3] >= sizes[2]
    for bad, frag in [(_lib.UaDesc(1, 2, 1, 100, 64, 48, 1, 0), b"chunk"), (_lib.UaDesc(1, 2, 1, 128, 256, 32, 1, 0), b"head dim"),
                      (_lib.UaDesc(1, 2, 1, 128, 64, 32, 7, 0), b"dtype"), (_lib.UaDesc(0, 2, 1, 128, 64, 32, 1, 0), b"positive")]:
        assert lib.ua_workspace_bytes(ctypes.byref(bad), _lib.UA_OP_FWD) == 0
        assert frag in lib.ua_last_error()
    assert lib.ua_workspace_bytes(ctypes.byref(ok), 9) == 0
    # chunks: any multiple of 64; 16 and the other multiples of 32 up to 256
    for c, fine in ((512, True), (1024, True), (4096, True), (96, True), (16, True), (288, False), (48, False)):
        d = _lib.UaDesc(1, 2, 1, 8192 if c != 288 else 288 * 4, 64, c, _lib.UA_BF16, 0)
        d.L = c * 4 if c in (48, 96, 288) else 8192
        assert (lib.ua_workspace_bytes(ctypes.byref(d), _lib.UA_OP_FWD) > 0) == fine, c
    # more heads than grid rows: refused with the way out in the message (the Python operators split by themselves)
    many = _lib.UaDesc(3, 16384, 2, 16, 16, 16, _lib.UA_F32, 0)
    assert lib.ua_workspace_bytes(ctypes.byref(many), _lib.UA_OP_FUSED_FWD) == 0 and b"split the call along b or h" in lib.ua_last_error()
    # head dims the reference's self-test reaches (512, Universal_Attention/triton/universal_attention_kernel.py:1189) are refused
    wide = _lib.UaDesc(2, 4, 2, 2048, 512, 64, _lib.UA_BF16, 0)
    assert lib.ua_workspace_bytes(ctypes.byref(wide), _lib.UA_OP_FWD) == 0 and b"256" in lib.ua_last_error()


def test_workspace_follows_the_flags_and_the_group_layout():
    """Sizing rules of the bf16 fused operator (host logic only): recomputation needs less than the tile exchange; with
    grouped queries the key-side partial sums are kept per part of a kv head's groups, so the shared sweep
    (UA_FLAG_SHARE_GROUPS) never needs more, needs less where few kv heads call for several parts (config 3: two), and
    the same where the kv heads fill the device by themselves; fp32 ignores both flags."""
    lib = _lib.load()

    def size(b, h, r, L, d, dtype, flags, op=_lib.UA_OP_FUSED_BWD):
        desc = _lib.UaDesc(b, h, r, L, d, 128, dtype, flags)
        n = lib.ua_workspace_bytes(ctypes.byref(desc), op)
        assert n > 0, lib.ua_last_error()
        return n

    bf, f32 = _lib.UA_BF16, _lib.UA_F32
    assert size(1, 32, 1, 8192, 128, bf, _lib.UA_FLAG_RECOMPUTE) < size(1, 32, 1, 8192, 128, bf, 0) < 8 << 30
    few, many = (1, 8, 4, 4096, 128), (1, 64, 4, 4096, 128)
    assert size(*few, bf, _lib.UA_FLAG_SHARE_GROUPS) < size(*few, bf, 0)
    assert size(*many, bf, _lib.UA_FLAG_SHARE_GROUPS) == size(*many, bf, 0)
    # one more slice of the three key-side partial sums and of the decay-gradient tiles per extra part: config 3 has two parts
    Lp, D, tiles = 4096, 128, 16 * 32 * 33 + 8
    extra = 8 * (2 * Lp * D * 4 + Lp * 4 + tiles * 1024)
    assert abs(size(*few, bf, 0) - size(*few, bf, _lib.UA_FLAG_SHARE_GROUPS) - extra) <= 4 * 256
    for flags in (_lib.UA_FLAG_SHARE_GROUPS, _lib.UA_FLAG_RECOMPUTE):
        assert size(*few, f32, flags) == size(*few, f32, 0)
    assert size(*few, bf, 0, _lib.UA_OP_FUSED_FWD) == size(*few, bf, _lib.UA_FLAG_SHARE_GROUPS, _lib.UA_OP_FUSED_FWD)


def test_null_and_small_workspace_are_rejected_before_any_launch():
    lib = _lib.load()
    d = _lib.UaDesc(1, 1, 1, 128, 64, 32, _lib.UA_F32, 0)
    rows = _lib.UaRows(1, 0, 0, 0, 0, 64, 128)           # non-null dummy pointers: validation stops before use
    code = lib.ua_fused_fwd(ctypes.byref(d), ctypes.byref(rows), ctypes.byref(rows), ctypes.byref(rows), 1, 1, 1, 1, None, 0, None)
    assert code == -2 and b"workspace" in lib.ua_last_error()
    code = lib.ua_fused_fwd(ctypes.byref(d), ctypes.byref(rows), ctypes.byref(rows), ctypes.byref(rows), 1, 1, 1, 1, 256, 16, None)
    assert code == -2
    null_rows = _lib.UaRows(None, 0, 0, 0, 0, 64, 128)
    code = lib.ua_fused_fwd(ctypes.byref(d), ctypes.byref(null_rows), ctypes.byref(rows), ctypes.byref(rows), 1, 1, 1, 1, 256, 1 << 30, None)
    assert code == -1 and b"null" in lib.ua_last_error()
    with pytest.raises(_lib.UaError):
        _lib.check(code, "ua_fused_fwd")


def test_ops_refuse_cpu_tensors():
    import torch
    from universal_attention_triton_amd import ops
    k = torch.zeros(1, 1, 1, 32, 16)
    with pytest.raises(_lib.UaError):
        ops.fused_forward(k, k, torch.zeros(1, 1, 1, 32, 16), torch.ones(1, 1, 1, 32), torch.ones(1, 1, 32))


def test_tune_table_roundtrip_and_choice_order():
    """An entry wins over the built-in table and the heuristic; -1 removes it; out-of-range variants and unknown slots
    are refused; the slots report their variant counts (host logic only)."""
    lib = _lib.load()
    d = _lib.UaDesc(1, 2, 1, 1024, 128, 0, _lib.UA_BF16, 0)
    for slot, n_min in ((_lib.UA_TUNE_FWD_RECOMPUTE, 5), (_lib.UA_TUNE_CARRY, 2), (_lib.UA_TUNE_FWD_TILES, 3),
                        (_lib.UA_TUNE_BWD_PARTS, 1), (_lib.UA_TUNE_BWD_QUERIES, 2), (_lib.UA_TUNE_BWD_KEYS, 2),
                        (_lib.UA_TUNE_CHUNKED_PAIR, 3), (_lib.UA_TUNE_AFF_PAIR, 3)):
        n = lib.ua_tune_variants(ctypes.byref(d), slot)
        assert n >= n_min, (slot, n)
        base = lib.ua_tune_choice(ctypes.byref(d), slot)
        assert 0 <= base < n and lib.ua_tune_get(ctypes.byref(d), slot) == -1
        assert lib.ua_tune_set(ctypes.byref(d), slot, n - 1) == 0
        assert lib.ua_tune_get(ctypes.byref(d), slot) == n - 1 == lib.ua_tune_choice(ctypes.byref(d), slot)
        assert lib.ua_tune_set(ctypes.byref(d), slot, n) < 0
        assert lib.ua_tune_set(ctypes.byref(d), slot, -1) == 0
        assert lib.ua_tune_get(ctypes.byref(d), slot) == -1 and lib.ua_tune_choice(ctypes.byref(d), slot) == base
    assert lib.ua_tune_variants(ctypes.byref(d), 7) < 0
    # grouped queries: one variant per divisor of r; fp32 has a single variant everywhere but the recomputing forward
    g = _lib.UaDesc(1, 8, 4, 4096, 128, 0, _lib.UA_BF16, 0)
    assert lib.ua_tune_variants(ctypes.byref(g), _lib.UA_TUNE_BWD_PARTS) == 3
    assert lib.ua_tune_variants(ctypes.byref(g), _lib.UA_TUNE_FWD_TILES) == 2
    f = _lib.UaDesc(1, 8, 4, 4096, 128, 0, _lib.UA_F32, 0)
    assert [lib.ua_tune_variants(ctypes.byref(f), s) for s in (16, 17, 18, 19)] == [1, 1, 1, 1]


def test_number_of_key_side_parts_follows_the_table_and_sizes_the_workspace():
    lib = _lib.load()
    g = _lib.UaDesc(1, 8, 4, 4096, 128, 0, _lib.UA_BF16, 0)
    sizes = []
    for v in range(3):
        assert lib.ua_tune_set(ctypes.byref(g), _lib.UA_TUNE_BWD_PARTS, v) == 0
        sizes.append(lib.ua_workspace_bytes(ctypes.byref(g), _lib.UA_OP_FUSED_BWD))
    lib.ua_tune_set(ctypes.byref(g), _lib.UA_TUNE_BWD_PARTS, -1)
    assert sizes[0] < sizes[1] < sizes[2]
    shared = _lib.UaDesc(1, 8, 4, 4096, 128, 0, _lib.UA_BF16, _lib.UA_FLAG_SHARE_GROUPS)
    assert lib.ua_workspace_bytes(ctypes.byref(shared), _lib.UA_OP_FUSED_BWD) == sizes[0]


def test_tune_table_persists_through_json(tmp_path):
    from universal_attention_triton_amd import tune
    lib = _lib.load()
    tune.set_entry(2, 16, 1, 2048, 64, "bf16", "fwd_tiles", 2)
    tune.set_entry(1, 8, 4, 4096, 128, "bf16", "bwd_queries", 1)
    path = str(tmp_path / "ua_tune.json")
    tune.save(path)
    d1 = _lib.UaDesc(2, 16, 1, 2048, 64, 0, _lib.UA_BF16, 0)
    d2 = _lib.UaDesc(1, 8, 4, 4096, 128, 0, _lib.UA_BF16, 0)
    lib.ua_tune_set(ctypes.byref(d1), _lib.UA_TUNE_FWD_TILES, -1)
    lib.ua_tune_set(ctypes.byref(d2), _lib.UA_TUNE_BWD_QUERIES, -1)
    assert lib.ua_tune_get(ctypes.byref(d1), _lib.UA_TUNE_FWD_TILES) == -1
    assert tune.load(path) >= 2
    assert lib.ua_tune_get(ctypes.byref(d1), _lib.UA_TUNE_FWD_TILES) == 2
    assert lib.ua_tune_get(ctypes.byref(d2), _lib.UA_TUNE_BWD_QUERIES) == 1
    lib.ua_tune_set(ctypes.byref(d1), _lib.UA_TUNE_FWD_TILES, -1)
    lib.ua_tune_set(ctypes.byref(d2), _lib.UA_TUNE_BWD_QUERIES, -1)


def test_forward_state_plus_backward_scratch_is_the_whole_workspace():
    """Sizing rule of the split workspace: what a backward needs next to the forward state is the total minus the state."""
    lib = _lib.load()
    for d in (_lib.UaDesc(1, 32, 1, 8192, 128, 128, _lib.UA_BF16, 0), _lib.UaDesc(2, 3, 2, 300, 48, 0, _lib.UA_F32, 0),
              _lib.UaDesc(1, 8, 4, 4096, 128, 128, _lib.UA_BF16, _lib.UA_FLAG_RECOMPUTE)):
        for fwd, bwd, scratch in ((_lib.UA_OP_FUSED_FWD, _lib.UA_OP_FUSED_BWD, _lib.UA_OP_FUSED_BWD_SCRATCH),
                                  (_lib.UA_OP_FWD, _lib.UA_OP_BWD, _lib.UA_OP_BWD_SCRATCH)):
            if d.chunk == 0 and fwd == _lib.UA_OP_FWD:
                continue
            f, t, s = (lib.ua_workspace_bytes(ctypes.byref(d), op) for op in (fwd, bwd, scratch))
            assert f > 0 and s > 0 and f + s == t and f % 256 == 0
    big = _lib.UaDesc(1, 32, 1, 8192, 128, 128, _lib.UA_BF16, 0)
    assert lib.ua_workspace_bytes(ctypes.byref(big), _lib.UA_OP_FUSED_FWD) <= int(2.6e9)       # kept between forward and backward
    assert lib.ua_workspace_bytes(ctypes.byref(big), _lib.UA_OP_FUSED_BWD_SCRATCH) >= int(4e9)  # allocated inside backward


def test_mismatched_shapes_and_dtypes_are_refused_before_any_launch():
    """The kernels trust the descriptor, so the host checks the five tensors against one another (the reference fails in
    its own views / asserts on such inputs); runs on CPU tensors because the checks come before the device check."""
    import torch
    from universal_attention_triton_amd import ops
    b, h, n, c, d, r = 1, 2, 4, 16, 32, 2
    L = n * c
    kc, vc = torch.zeros(b, h, n, c, d), torch.zeros(b, h, n, c, d)
    xq, src, dest = torch.zeros(b, h, r, L, d), torch.ones(b, h, n, c), torch.ones(b, h, L)
    bad = [
        (kc, vc[:, :, :2], xq, src, dest),                         # vc shorter than kc
        (kc, vc, xq[:, :, :, : L // 2], src, dest),                # xq shorter than the keys
        (kc, vc, torch.zeros(b, h + 1, r, L, d), src, dest),       # other head count
        (kc, vc, torch.zeros(b, h, r, L, d + 8), src, dest),       # other head dim
        (kc, vc, xq, src[:, :, :2], dest),                         # gates of another length
        (kc, vc, xq, src, dest[:, :, : L - 1]),
        (kc, vc, torch.zeros(b, h, r, n, c // 2, d), src, dest),   # 2-D layout that does not cover L
        (kc[0], vc[0], xq[0], src[0], dest[0]),                    # wrong rank
    ]
    for args in bad:
        with pytest.raises(ValueError):
            ops.fused_forward(*args)
        with pytest.raises(ValueError):
            ops.chunked_forward(*args)
    with pytest.raises(TypeError):
        ops.fused_forward(kc, vc.bfloat16(), xq, src, dest)
    with pytest.raises(TypeError):
        ops.fused_forward(kc.half(), vc.half(), xq.half(), src, dest)
    with pytest.raises(_lib.UaError):                                  # well-formed, but not on the GPU
        ops.fused_forward(kc, vc, xq, src, dest)


def test_library_reports_the_hash_of_the_sources_it_was_built_from():
    from universal_attention_triton_amd import build
    assert _lib.load().ua_source_hash().decode() == build.source_hash()
