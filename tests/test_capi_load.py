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


def test_tune_table_roundtrip():
    lib = _lib.load()
    d = _lib.UaDesc(1, 2, 1, 1024, 128, 0, _lib.UA_BF16, 0)
    n = lib.ua_tune_variants(ctypes.byref(d), _lib.UA_OP_FUSED_FWD)
    assert n >= 1
    assert lib.ua_tune_set(ctypes.byref(d), _lib.UA_OP_FUSED_FWD, n - 1) == 0
    assert lib.ua_tune_get(ctypes.byref(d), _lib.UA_OP_FUSED_FWD) == n - 1
    assert lib.ua_tune_set(ctypes.byref(d), _lib.UA_OP_FUSED_FWD, n) < 0
    assert lib.ua_tune_set(ctypes.byref(d), _lib.UA_OP_FUSED_FWD, 0) == 0
