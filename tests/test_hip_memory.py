"""Memory held between forward and backward in a stack of layers, and what holding less costs in time."""
import time

import pytest
import torch

from tests.util import rel_err

pytestmark = pytest.mark.gpu


def test_four_layer_stack_keeps_one_forward_state_per_layer_unless_told_not_to():
    """Four attention layers with residual connections (projections and gates from one weight per layer, as the
    reference's driver builds them, main.py:19-31), bf16, b=1 h=8 r=2 L=4096 d=128.  With keep_state=True every layer
    holds its forward state (ops.retained_bytes) until its backward; with keep_state=False a layer holds what the
    reference holds (inputs, O) plus lse, and its backward rebuilds the state.  Same gradients either way."""
    from universal_attention_triton_amd import ops
    from universal_attention_triton_amd.universal_attention import universal_attention
    b, h, r, L, d, c, layers = 1, 8, 2, 4096, 128, 128, 4
    dtype = torch.bfloat16
    gen = torch.Generator(device="cuda").manual_seed(3)
    width = h * r * d
    x0 = (torch.randn(b, L, width, device="cuda", generator=gen) * 0.5).to(dtype).requires_grad_()
    scale = width ** -0.5
    W = [{k: (torch.randn(width, n, device="cuda", generator=gen) * scale).to(dtype).requires_grad_()
          for k, n in (("q", h * r * d), ("k", h * d), ("v", h * d), ("g", 2 * h))} for _ in range(layers)]

    def forward(keep):
        x = x0
        for w in W:
            q = (x @ w["q"]).view(b, L, h, r, d).permute(0, 2, 3, 1, 4)                   # [b,h,r,L,d]
            k = torch.nn.functional.normalize((x @ w["k"]).view(b, L, h, d).float(), dim=-1).to(dtype)
            k = k.permute(0, 2, 1, 3).reshape(b, h, L // c, c, d)
            v = (x @ w["v"]).view(b, L, h, d).permute(0, 2, 1, 3).reshape(b, h, L // c, c, d)
            g = torch.sigmoid((x @ w["g"]).float()).to(dtype).view(b, L, 2, h).permute(2, 0, 3, 1)   # [2,b,h,L]
            O = universal_attention(k, v, q, g[0].reshape(b, h, L // c, c), g[1], keep_state=keep)
            x = x + O.permute(0, 3, 1, 2, 4).reshape(b, L, width)
        return x

    kc_like = torch.empty(b, h, L // c, c, d, dtype=dtype, device="cuda")
    xq_like = torch.empty(b, h, r, L, d, dtype=dtype, device="cuda")
    src_like = torch.empty(b, h, L // c, c, dtype=dtype, device="cuda")
    dest_like = torch.empty(b, h, L, dtype=dtype, device="cuda")
    state = ops.retained_bytes(kc_like, kc_like, xq_like, src_like, dest_like)
    del kc_like, xq_like, src_like, dest_like
    params = [x0] + [w[k] for w in W for k in ("q", "k", "v", "g")]
    # one step first: the BLAS library takes its workspace from torch's allocator on first use and keeps it
    torch.autograd.grad(forward(True), params, torch.ones(b, L, width, dtype=dtype, device="cuda"))
    res = {}
    for keep in (True, False):
        for p in params:
            p.grad = None
        torch.cuda.synchronize()
        torch.cuda.empty_cache()
        base = torch.cuda.memory_allocated()
        torch.cuda.reset_peak_memory_stats()
        y = forward(keep)
        torch.cuda.synchronize()
        held = torch.cuda.memory_allocated() - base
        grads = torch.autograd.grad(y, params, torch.ones_like(y))
        torch.cuda.synchronize()
        peak = torch.cuda.max_memory_allocated() - base
        del y
        # time of a step
        for _ in range(2):
            torch.autograd.grad(forward(keep), params, torch.ones(b, L, width, dtype=dtype, device="cuda"))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(5):
            torch.autograd.grad(forward(keep), params, torch.ones(b, L, width, dtype=dtype, device="cuda"))
        torch.cuda.synchronize()
        res[keep] = dict(held=held, peak=peak, ms=(time.perf_counter() - t0) * 1e3 / 5, grads=[g.detach().clone() for g in grads])
        del grads
    per_layer = (res[True]["held"] - res[False]["held"]) / layers
    print("forward state per layer: %.1f MiB measured, %.1f MiB by ops.retained_bytes; held after the forward of %d layers: "
          "%.1f MiB (keep_state=True) / %.1f MiB (False); peak %.1f / %.1f MiB; step %.2f / %.2f ms"
          % (per_layer / 2**20, state / 2**20, layers, res[True]["held"] / 2**20, res[False]["held"] / 2**20,
             res[True]["peak"] / 2**20, res[False]["peak"] / 2**20, res[True]["ms"], res[False]["ms"]), flush=True)
    assert abs(per_layer - state) <= 0.02 * state + (4 << 20), (per_layer, state)
    assert res[False]["peak"] < res[True]["peak"]
    assert res[False]["ms"] < 1.6 * res[True]["ms"]          # rebuilding the state costs about the forward's pre-pass again
    for x, y in zip(res[True]["grads"], res[False]["grads"]):
        assert rel_err(x, y) <= 1e-6 or torch.equal(x, y), rel_err(x, y)
