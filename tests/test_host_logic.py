"""Host-side logic that needs no GPU: the per-call options of the chunked operators and the splitting of calls with more
heads than grid rows."""
import threading

import pytest
import torch

from universal_attention_triton_amd import ops
from universal_attention_triton_amd import universal_attention_autograd as ua


def test_chunked_options_nest_restore_and_reject_unknown_names():
    base = dict(ua._options.get())
    assert base == {"keep_state": True, "recompute": False, "skip_masked": False, "contiguous_out": False}
    with ua.chunked_options(keep_state="normalisers"):
        assert ua._options.get()["keep_state"] == "normalisers" and ua._options.get()["recompute"] is False
        with ua.chunked_options(recompute=True, keep_state=False):
            assert ua._options.get()["keep_state"] is False and ua._options.get()["recompute"] is True
        assert ua._options.get()["keep_state"] == "normalisers" and ua._options.get()["recompute"] is False
    assert ua._options.get() == base
    with pytest.raises(TypeError):
        with ua.chunked_options(keep_stat=False):
            pass
    with pytest.raises(RuntimeError):
        with ua.chunked_options(skip_masked=True):
            raise RuntimeError("leaves the block")
    assert ua._options.get() == base                      # restored after an exception too


def test_chunked_options_do_not_leak_into_other_threads():
    seen = {}
    inside = threading.Event()
    done = threading.Event()

    def other():
        inside.wait(5)
        seen["other"] = dict(ua._options.get())
        done.set()

    t = threading.Thread(target=other)
    t.start()
    with ua.chunked_options(contiguous_out=True, keep_state=False):
        inside.set()
        done.wait(5)
        seen["mine"] = dict(ua._options.get())
    t.join()
    assert seen["mine"]["contiguous_out"] is True and seen["mine"]["keep_state"] is False
    assert seen["other"]["contiguous_out"] is False and seen["other"]["keep_state"] is True


@pytest.mark.parametrize("shape,chunked,pieces", [((3, 16384, 2, 1), False, 3), ((1, 40000, 2, 1), False, 2), ((2, 9000, 1, 4), True, 2),
                                                  ((1, 100, 2, 1), False, 1)])
def test_calls_with_more_heads_than_grid_rows_are_cut_along_b_then_h_and_joined(shape, chunked, pieces):
    """The wrapper around the operators: every piece stays within 65535 grid rows, the pieces cover every head exactly
    once, tensors are cut along b and h and results joined in order, the state of a split call is dropped."""
    b, h, r, n = shape
    calls = []

    def fake(kc, vc, xq, src, dest, keep_state=False, scale=1.0):
        pb, ph = kc.shape[:2]
        assert pb * ph * xq.shape[2] * (kc.shape[2] if chunked else 1) <= 65535
        assert vc.shape[:2] == xq.shape[:2] == src.shape[:2] == dest.shape[:2] == (pb, ph)
        calls.append((pb, ph, keep_state))
        return kc[..., 0, 0, :1] * scale + xq[:, :, 0, 0, :1], dest * 2, ("state" if keep_state else None)

    wrapped = ops._split_over_heads(5, chunked)(fake)
    kc = torch.arange(b * h, dtype=torch.float32).view(b, h, 1, 1, 1).expand(b, h, n, 2, 3)
    xq = torch.ones(b, h, r, 4, 3)
    src, dest = torch.zeros(b, h, n, 2), torch.arange(b * h, dtype=torch.float32).view(b, h, 1).expand(b, h, 4)
    out, dest2, state = wrapped(kc, kc, xq, src, dest, keep_state=True, scale=3.0)
    assert len(calls) == pieces
    assert sum(pb * ph for pb, ph, _ in calls) == b * h
    assert torch.equal(out, kc[..., 0, 0, :1] * 3.0 + 1.0) and torch.equal(dest2, dest * 2)
    if pieces == 1:
        assert state == "state" and calls[0][2] is True
    else:
        assert state is None and all(k is False for _, _, k in calls)


def test_a_single_kv_head_with_too_many_rows_is_refused():
    from universal_attention_triton_amd import _lib
    wrapped = ops._split_over_heads(5, True)(lambda *a, **k: None)
    kc = torch.zeros(1, 1, 70000, 1, 1)                      # 70000 chunks per row of one head
    with pytest.raises(_lib.UaError):
        wrapped(kc, kc, torch.zeros(1, 1, 1, 70000, 1), torch.zeros(1, 1, 70000, 1), torch.zeros(1, 1, 70000))
