"""GPU parity of the stand-alone decay bias (reference AffinityScores, affinity_kernel_opt.py:425-462), called through
the C ABI."""
import pytest
import torch

from oracle import ua_oracle as orc
from tests.util import TOL, rel_err

pytestmark = pytest.mark.gpu

# b, h, L, d (ragged L, padded d).  bf16 with L a multiple of 8 runs the tile-exchanging backward, everything else the one
# with the float L x L running sum.  The last two launch more workgroups than the part has CUs, so that every workgroup
# takes two key groups of complementary length (5 and 3 groups: the middle one stays alone).
SHAPES = [(1, 2, 64, 16), (2, 2, 192, 64), (1, 1, 320, 80), (1, 2, 517, 128), (1, 2, 1032, 128), (1, 66, 520, 64),
          (2, 44, 384, 128)]


def _inputs(b, h, L, d, dtype, seed):
    inp = orc.make_inputs(b, h, 1, L, d, L, dtype=dtype, seed=seed)
    return inp["kc"].reshape(b, h, L, d), inp["static_src"].reshape(b, h, L), inp["static_dest"]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
def test_affinity_scores_forward_and_backward(shape, dtype):
    from universal_attention_triton_amd.affinity import AffinityScores
    b, h, L, d = shape
    print("case affinity", shape, dtype, flush=True)
    k, src, dest = _inputs(b, h, L, d, dtype, seed=71)
    # reference-grade values: float64 on the dtype-rounded inputs
    leaves64 = [x.double().requires_grad_() for x in (k, src, dest)]
    want = orc.affinity_scores(*leaves64)
    g = torch.Generator().manual_seed(7)
    daff = torch.randn(b, h, L, L, generator=g).to(dtype)
    visible = torch.ones(L, L, dtype=torch.bool).tril(0)                       # [t, s]: s <= t
    gw = torch.autograd.grad(want, leaves64, daff.double() * visible)          # the -1e12 fill carries no gradient
    leaves = [x.cuda().requires_grad_() for x in (k, src, dest)]
    aff = AffinityScores.apply(*leaves)
    grads = torch.autograd.grad(aff, leaves, daff.cuda())
    torch.cuda.synchronize()
    assert aff.dtype == dtype and aff.shape == (b, h, L, L)
    a = aff.float().cpu()
    assert bool((a[..., ~visible] == torch.tensor(-1e12, dtype=dtype).float()).all())
    assert bool((a.diagonal(dim1=-2, dim2=-1) == 0).all())
    # the bias grows to hundreds: a relative bar on the tensor, as everywhere else
    lower = visible[None, None].expand_as(a)
    assert rel_err(a[lower], want.detach()[lower]) <= (TOL[dtype] if dtype == torch.float32 else 4e-3)
    # dk: (2/3) G^(-1/3) amplifies the float32 rounding of tiny positive key-key products G, and here every pair carries
    # an upstream gradient of order sqrt(L); the bar follows how far a float32 evaluation of the oracle itself lands
    # from the float64 one (2e-4 at L = 517, 2e-3 at L = 1032)
    leaves32 = [x.float().requires_grad_() for x in (k, src, dest)]
    g32 = torch.autograd.grad(orc.affinity_scores(*leaves32), leaves32, daff.float() * visible)
    own = rel_err(g32[0], gw[0])
    tol_dk = max(TOL[dtype], 3 * own)
    print("  dk bar %.2e (stated %.0e, float32 evaluation of the oracle misses float64 by %.2e)" % (tol_dk, TOL[dtype], own), flush=True)
    for name, got, ref in zip(("dk", "dsrc", "ddest"), grads, gw):
        tol = TOL[dtype] if name != "dk" else tol_dk
        print("  %-6s %.2e (bar %.2e)" % (name, rel_err(got, ref), tol), flush=True)
        assert rel_err(got, ref) <= tol, (name, rel_err(got, ref), tol)


def test_affinity_scores_agree_with_the_bias_inside_the_fused_operator():
    """softmax(q k^T + aff) v with the stand-alone bias equals the fused operator."""
    from universal_attention_triton_amd.affinity import AffinityScores
    from universal_attention_triton_amd.universal_attention import universal_attention
    b, h, L, d, c = 1, 2, 256, 64, 64
    inp = orc.make_inputs(b, h, 1, L, d, c, dtype=torch.float32, seed=72)
    dev = {k: v.cuda() for k, v in inp.items()}
    k = dev["kc"].reshape(b, h, L, d)
    aff = AffinityScores.apply(k, dev["static_src"].reshape(b, h, L), dev["static_dest"])
    scores = torch.matmul(dev["xq"][:, :, 0], k.transpose(-1, -2)) + aff        # [b,h,t,s]
    O_sdpa = torch.matmul(torch.softmax(scores, dim=-1), dev["vc"].reshape(b, h, L, d))
    O = universal_attention(dev["kc"], dev["vc"], dev["xq"], dev["static_src"], dev["static_dest"])
    assert rel_err(O[:, :, 0], O_sdpa) <= 1e-4
