"""Autograd wiring of the drop-in Functions on the GPU: nothing travels between calls through process-wide state.

Options are per call and per thread, the forward state is an output of the Function, and what the merge's backward
leaves for the chunked backward hangs on the gradient tensor itself, so that a gradient which is not exactly that
tensor (a second consumer of `out`, a hook that replaces it, an in-place change) takes the general path."""
import threading

import pytest
import torch

from oracle import ua_oracle as orc
from tests.util import NAMES, TOL, dense_reference, key_gradient_bar, rel_err

pytestmark = pytest.mark.gpu


def _leaves(inp):
    return [inp[k].cuda().requires_grad_() for k in NAMES]


def test_options_are_per_thread_and_per_call_on_separate_streams():
    """Two threads on two streams run the reference's call sequence at the same time, one with the defaults and one
    inside chunked_options(keep_state=False, contiguous_out=True): each sees its own options (the layout of `out`
    shows it), and each gets, bit for bit, the results of a run on its own with the same options."""
    from universal_attention_triton_amd import universal_attention_autograd as ua
    shapes = {"plain": (1, 2, 2, 512, 64, 64), "options": (1, 3, 1, 384, 32, 128)}
    inps = {k: orc.make_inputs(*s, dtype=torch.bfloat16, seed=11 + i) for i, (k, s) in enumerate(shapes.items())}
    want = {}
    for k, inp in inps.items():
        leaves = _leaves(inp)
        with ua.chunked_options(**({"keep_state": False, "contiguous_out": True} if k == "options" else {})):
            out, denom = ua.UniversalAttention.apply(*leaves)
        assert out.is_contiguous() == (k == "options")
        O = ua.SMVecMatMul.apply(out, denom)
        want[k] = (O.detach().clone(), torch.autograd.grad(O, leaves, inp["dO"].cuda()))
    torch.cuda.synchronize()
    got, errors = {}, []
    start = threading.Barrier(2)

    def work(name):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                leaves = _leaves(inps[name])
                dO = inps[name]["dO"].cuda()
                start.wait()
                for _ in range(3):
                    if name == "options":
                        with ua.chunked_options(keep_state=False, contiguous_out=True):
                            out, denom = ua.UniversalAttention.apply(*leaves)
                        assert out.is_contiguous()
                    else:
                        out, denom = ua.UniversalAttention.apply(*leaves)
                        assert not out.is_contiguous()            # the other thread's block does not reach this one
                    O = ua.SMVecMatMul.apply(out, denom)
                    grads = torch.autograd.grad(O, leaves, dO)
                stream.synchronize()
                got[name] = (O.detach(), grads)
        except BaseException as e:          # noqa: B902 - reported by the main thread
            errors.append((name, repr(e)))

    threads = [threading.Thread(target=work, args=(k,)) for k in shapes]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for k in shapes:
        assert torch.equal(got[k][0], want[k][0]), k
        for name, x, y in zip(NAMES, got[k][1], want[k][1]):
            assert torch.equal(x, y), (k, name, rel_err(x, y))
    with pytest.raises(TypeError):
        with ua.chunked_options(keep_stat=True):
            pass


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_torch_func_grad_and_vjp_through_the_new_style_functions(dtype):
    """torch.func.grad / vjp need Functions with setup_context (the reference's Triton-backed entry point is one,
    Universal_Attention/universal_attention.py:5-31): the chunked operator, the merge and the fused operator."""
    from universal_attention_triton_amd import universal_attention_autograd as ua
    from universal_attention_triton_amd.universal_attention import universal_attention
    inp = orc.make_inputs(1, 2, 2, 256, 32, 64, dtype=dtype, seed=21)
    O_ref, _, g_ref = dense_reference(inp)
    dev = [inp[k].cuda() for k in NAMES]
    dO = inp["dO"].cuda()

    def loss_chunked(kc, vc, xq, src, dest):
        out, denom = ua.UniversalAttention.apply(kc, vc, xq, src, dest)
        return (ua.SMVecMatMul.apply(out, denom).float() * dO.float()).sum()

    def loss_fused(kc, vc, xq, src, dest):
        return (universal_attention(kc, vc, xq, src, dest).float() * dO.float()).sum()

    bar = key_gradient_bar(inp, dtype, g_ref[0])
    for tag, loss in (("chunked", loss_chunked), ("fused", loss_fused)):
        grads = torch.func.grad(loss, argnums=(0, 1, 2, 3, 4))(*dev)
        for name, x, y in zip(NAMES, grads, g_ref):
            assert rel_err(x, y) <= (bar if name == "kc" else TOL[dtype]), (tag, name, rel_err(x, y))
    O, vjp = torch.func.vjp(lambda *a: universal_attention(*a), *dev)
    assert rel_err(O, O_ref) <= TOL[dtype]
    for name, x, y in zip(NAMES, vjp(dO), g_ref):
        assert rel_err(x, y) <= (bar if name == "kc" else TOL[dtype]), ("vjp", name, rel_err(x, y))


def _composite(ua, inp, extra=None, hook=None):
    leaves = _leaves(inp)
    out, denom = ua.UniversalAttention.apply(*leaves)
    if hook is not None:
        out.register_hook(hook)
    O = ua.SMVecMatMul.apply(out, denom)
    loss = (O.float() * inp["dO"].cuda().float()).sum()
    if extra is not None:
        loss = loss + extra(out, denom)
    return torch.autograd.grad(loss, leaves)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gradient_of_out_that_is_not_the_merge_s_own_tensor_takes_the_general_path(dtype, monkeypatch):
    """The chunked backward reuses the merge backward's delta only for the very gradient tensor that call returned.
    A second consumer of `out` (autograd adds the two gradients: a new tensor), a hook that returns another tensor and a
    hook that changes the gradient in place must all give the gradients of the reference's formulas; a hook that
    returns nothing leaves the shortcut in place.  Afterwards nothing of any call is left in the module."""
    from universal_attention_triton_amd import ops, universal_attention_autograd as ua
    b, h, r, L, d, c = 1, 2, 2, 256, 32, 64
    n = L // c
    inp = orc.make_inputs(b, h, r, L, d, c, dtype=dtype, seed=23)
    w_out = torch.randn(b, h, r, L, d, n, generator=torch.Generator().manual_seed(1)).to(dtype)
    used = []
    real = ops._delta_from_merge
    monkeypatch.setattr(ops, "_delta_from_merge", lambda *a: (used.append(real(*a) is not None), real(*a))[1])

    def oracle(scale_out=1.0, add_out=0.0):
        args = [inp[k].float() for k in NAMES]
        out, denom = orc.chunked_forward(*args)
        d_out, d_denom = orc.merge_backward(out, denom, inp["dO"].float())
        return orc.chunked_backward(*args, d_out * scale_out + add_out, d_denom)

    def check(tag, got, want, expect_shortcut):
        assert used and used[-1] == expect_shortcut, (tag, used)
        for name, x, y in zip(NAMES, got, want):
            bar = TOL[dtype] if name != "kc" or dtype == torch.bfloat16 else 1e-3      # float32 key gradient: bars in test_hip_backward
            assert rel_err(x.reshape(y.shape), y) <= bar, (tag, name, rel_err(x.reshape(y.shape), y))

    check("plain sequence", _composite(ua, inp), oracle(), True)
    check("second consumer of out", _composite(ua, inp, extra=lambda out, denom: (out.float() * w_out.cuda().float()).sum()),
          oracle(add_out=w_out.float()), False)
    check("hook returning another tensor", _composite(ua, inp, hook=lambda g: g * 2.0), oracle(scale_out=2.0), False)
    check("hook changing the gradient in place", _composite(ua, inp, hook=lambda g: g.mul_(2.0)), oracle(scale_out=2.0), False)
    seen = []
    check("hook that only looks", _composite(ua, inp, hook=lambda g: seen.append(g.shape)), oracle(), True)
    assert seen
    assert not any(isinstance(v, dict) and v for k, v in vars(ops).items() if k.startswith("_merge"))
