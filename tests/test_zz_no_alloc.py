"""The allocation-free forward (ua_fused_fwd_noalloc) against ua_fused_fwd through the C ABI: same kernels on the same
inputs, so the results must be bit-identical; two calls in a row, the second on a smaller problem (the built-in scratch
keeps the first call's contents); a problem beyond the built-in scratch is refused before any launch."""
import ctypes

import pytest
import torch

from oracle import ua_oracle as orc
from universal_attention_triton_amd import _lib, ops

pytestmark = pytest.mark.gpu


def _run_both(b, h, r, L, d, dtype, seed):
    inp = orc.make_inputs(b, h, r, L, d, 64, dtype=dtype, seed=seed)
    kc, vc, xq, src, dest = [inp[k].cuda() for k in ("kc", "vc", "xq", "static_src", "static_dest")]
    O_ref, lse_ref, _ = ops.fused_forward(kc, vc, xq, src, dest)
    O = torch.full((b, h, r, L, d), float("nan"), dtype=dtype, device="cuda")
    lse = torch.full((b, h, r, L), float("nan"), dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    ops.fused_forward_noalloc(kc, vc, xq, src.reshape(b, h, L), dest.reshape(b, h, L), O, lse)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.equal(O, O_ref) and torch.equal(lse, lse_ref)
    return O


def test_noalloc_forward_equals_workspace_forward_twice_second_smaller():
    _run_both(1, 4, 2, 1024, 128, torch.bfloat16, 11)
    _run_both(1, 2, 1, 320, 64, torch.bfloat16, 12)       # smaller: the scratch still holds the first call's state
    _run_both(2, 2, 1, 192, 48, torch.float32, 13)


def test_noalloc_forward_refuses_what_does_not_fit():
    lib = _lib.load()
    cap = lib.ua_noalloc_scratch_bytes()
    assert cap == 64 << 20
    big = _lib.UaDesc(1, 32, 1, 8192, 128, 0, _lib.UA_BF16, 0)
    assert lib.ua_workspace_bytes(ctypes.byref(big), _lib.UA_OP_FUSED_FWD) > cap
    rows = _lib.UaRows(1, 0, 0, 0, 0, 128, 8192)
    code = lib.ua_fused_fwd_noalloc(ctypes.byref(big), ctypes.byref(rows), ctypes.byref(rows), ctypes.byref(rows), 1, 1, 1, 1, None)
    assert code == -2
    assert b"built-in" in lib.ua_last_error()
