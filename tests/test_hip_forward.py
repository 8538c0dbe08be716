"""GPU parity of the forward kernels, called through the C ABI (ctypes -> libua_hip.so)."""
import pytest
import torch

from oracle import ua_oracle as orc
from tests.util import NAMES, TOL, dense_reference, load_golden, rel_err

pytestmark = pytest.mark.gpu

SHAPES = [  # b, h, r, L, d, c
    (1, 2, 2, 64, 16, 16),
    (1, 1, 1, 128, 32, 32),
    (2, 2, 1, 256, 64, 64),
    (1, 2, 1, 384, 128, 128),
    (1, 1, 2, 320, 80, 32),      # L not a multiple of 128, d padded to 128
    (1, 2, 1, 512, 64, 256),
    (2, 2, 3, 320, 16, 64),      # chunk of 64, L = 5 chunks: the padding up to 384 holds a 64-key tile that belongs to no chunk
    (1, 1, 1, 192, 32, 192),     # likewise with a single chunk
]


def _inputs(shape, dtype, seed=0, gate_mean=0.0):
    b, h, r, L, d, c = shape
    return orc.make_inputs(b, h, r, L, d, c, dtype=dtype, seed=seed, gate_mean=gate_mean)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
def test_fused_forward_matches_dense_oracle(shape, dtype):
    from universal_attention_triton_amd import ops
    print("case fused_fwd", shape, dtype, flush=True)
    inp = _inputs(shape, dtype, seed=21)
    O_ref, lse_ref, _ = dense_reference(inp)
    dev = {k: v.cuda() for k, v in inp.items()}
    O, lse, _ = ops.fused_forward(*[dev[k] for k in NAMES])
    torch.cuda.synchronize()
    assert rel_err(O, O_ref) <= TOL[dtype], rel_err(O, O_ref)
    assert float((lse.cpu().double() - lse_ref).abs().max()) <= (1e-4 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
def test_chunked_forward_matches_oracle(shape, dtype):
    from universal_attention_triton_amd import ops
    print("case chunked_fwd", shape, dtype, flush=True)
    inp = _inputs(shape, dtype, seed=22)
    # oracle with the reference's cast points, evaluated in float32 on the dtype-rounded inputs
    out_ref, denom_ref = orc.chunked_forward(*[inp[k].float() for k in NAMES])
    dev = {k: v.cuda() for k, v in inp.items()}
    out, denom, _ = ops.chunked_forward(*[dev[k] for k in NAMES])
    torch.cuda.synchronize()
    assert out.shape == out_ref.shape and denom.shape == denom_ref.shape
    assert rel_err(out, out_ref) <= TOL[dtype], rel_err(out, out_ref)
    # denom holds float32(-1e12) for fully masked pairs: compare those exactly, the rest by value
    masked = denom_ref < -1e11
    got = denom.float().cpu()
    assert torch.equal(got[masked], denom_ref.to(dtype).float()[masked])
    dtol = 1e-4 if dtype == torch.float32 else 2e-2
    assert float(((got - denom_ref)[~masked].abs() / denom_ref[~masked].abs().clamp_min(1.0)).max()) <= dtol
    # merged result against the dense float64 oracle
    O_ref, _, _ = dense_reference(inp)
    O = orc.merge(out.float().cpu(), got)
    assert rel_err(O, O_ref) <= TOL[dtype], rel_err(O, O_ref)


@pytest.mark.parametrize("name", ["tiny_fp32", "tiny_bf16", "small_fp32", "small_bf16"])
def test_chunked_forward_matches_reference_golden(name):
    from universal_attention_triton_amd import universal_attention_autograd as ua
    print("case golden_fwd", name, flush=True)
    t, dtype, (b, h, r, l, d, c, seed) = load_golden(name)
    args = [t[k].to(dtype).cuda() for k in NAMES]
    out, denom = ua.UniversalAttention.apply(*args)
    torch.cuda.synchronize()
    assert rel_err(out, t["out"]) <= TOL[dtype], rel_err(out, t["out"])
    masked = t["denom"] < -1e11
    assert torch.equal(denom.float().cpu()[masked], t["denom"][masked])
    assert rel_err(denom.float().cpu()[~masked], t["denom"][~masked]) <= TOL[dtype]
    # 2-D layout entry point gives the same values
    from universal_attention_triton_amd.universal_attention import UniversalAttention as UA2D
    n = l // c
    out2, denom2 = UA2D.apply(args[0], args[1], args[2].view(b, h, r, n, c, d), args[3], args[4].view(b, h, n, c))
    assert torch.equal(out2, out) and torch.equal(denom2, denom)


def test_cfg0_forward_matches_reference_golden():
    """BASELINE config 0 (b1 h4 r1 L512 d64 c64 fp32) against the reference's own output."""
    import numpy as np, os
    from universal_attention_triton_amd import universal_attention_autograd as ua
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    z = np.load(os.path.join(here, "cfg0_fwd_fp32.npz"))
    b, h, r, l, d, c, seed, _ = [int(x) for x in z["meta"]]
    inp = orc.make_inputs(b, h, r, l, d, c, dtype=torch.float32, seed=seed)
    args = [inp[k].cuda() for k in NAMES]
    out, denom = ua.UniversalAttention.apply(*args)
    O = ua.SMVecMatMul.apply(out, denom)
    torch.cuda.synchronize()
    assert rel_err(O, torch.from_numpy(z["O"])) <= 1e-4
    assert rel_err(out[..., 0], torch.from_numpy(z["out_first"])) <= 1e-4
    assert rel_err(out[..., -1], torch.from_numpy(z["out_last"])) <= 1e-4
    dref = torch.from_numpy(z["denom"])
    masked = dref < -1e11
    assert torch.equal(denom.cpu()[masked], dref[masked])
    assert rel_err(denom.cpu()[~masked], dref[~masked]) <= 1e-4
    torch.testing.assert_close(O.cpu(), torch.from_numpy(z["O"]), rtol=1e-4, atol=1e-5)
