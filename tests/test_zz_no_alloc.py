"""The allocation-free forward (ua_fused_fwd_noalloc) against ua_fused_fwd through the C ABI: same kernels on the same
inputs, so the results must be bit-identical; two calls in a row, the second on a smaller problem (the built-in scratch
keeps the first call's contents); a problem beyond the built-in scratch is refused before any launch."""
import ctypes

import pytest
import torch

from oracle import ua_oracle as orc
from universal_attention_triton_amd import _lib, ops

pytestmark = pytest.mark.gpu


def _run_both(b, h, r, L, d, dtype, seed, warm=True):
    inp = orc.make_inputs(b, h, r, L, d, 64, dtype=dtype, seed=seed)
    kc, vc, xq, src, dest = [inp[k].cuda() for k in ("kc", "vc", "xq", "static_src", "static_dest")]
    O_ref, lse_ref, _ = ops.fused_forward(kc, vc, xq, src, dest)
    O = torch.full((b, h, r, L, d), float("nan"), dtype=dtype, device="cuda")
    lse = torch.full((b, h, r, L), float("nan"), dtype=torch.float32, device="cuda")
    src3, dest3 = src.reshape(b, h, L), dest.reshape(b, h, L)
    if warm:       # the first call on a device looks up the address of the built-in scratch and sets kernel attributes
        ops.fused_forward_noalloc(kc, vc, xq, src3, dest3, O, lse)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]          # the driver's view: would also show a hipMalloc inside the library
    ops.fused_forward_noalloc(kc, vc, xq, src3, dest3, O, lse)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.equal(O, O_ref) and torch.equal(lse, lse_ref)
    return kc, vc, xq, src3, dest3, O, lse, O_ref, lse_ref


def test_noalloc_forward_equals_workspace_forward_twice_second_smaller():
    _run_both(1, 4, 2, 1024, 128, torch.bfloat16, 11)
    _run_both(1, 2, 1, 320, 64, torch.bfloat16, 12)       # smaller: the scratch still holds the first call's state
    _run_both(2, 2, 1, 192, 48, torch.float32, 13)


def test_noalloc_forward_under_graph_capture_after_an_eager_first_call():
    """The first call per device must happen outside a capture (it looks up the scratch's address); later calls only
    enqueue kernels, so they can be captured: three replays on fresh inputs, each against the eager workspace forward."""
    b, h, r, L, d = 1, 2, 2, 320, 64
    kc, vc, xq, src3, dest3, O, lse, _, _ = _run_both(b, h, r, L, d, torch.bfloat16, 21)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops.fused_forward_noalloc(kc, vc, xq, src3, dest3, O, lse)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.fused_forward_noalloc(kc, vc, xq, src3, dest3, O, lse)
    for seed in (22, 23, 24):
        fresh = orc.make_inputs(b, h, r, L, d, 64, dtype=torch.bfloat16, seed=seed)
        for t, k in ((kc, "kc"), (vc, "vc"), (xq, "xq")):
            t.copy_(fresh[k])
        src3.copy_(fresh["static_src"].reshape(b, h, L))
        dest3.copy_(fresh["static_dest"].reshape(b, h, L))
        O.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        O_ref, lse_ref, _ = ops.fused_forward(kc, vc, xq, src3.view(b, h, L // 64, 64), dest3)
        torch.cuda.synchronize()
        assert torch.equal(O, O_ref) and torch.equal(lse, lse_ref), seed


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
