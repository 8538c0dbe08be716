"""Pins the CPU oracle: closed forms, brute force, textbook special cases,
float64 gradcheck, and the golden vectors written by the reference operator."""
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import ua_oracle as orc


def _rand(b, h, r, l, d, seed, dtype=torch.float64):
    inp = orc.make_inputs(b, h, r, l, d, l, dtype=torch.float32, seed=seed)
    k = inp["kc"].reshape(b, h, l, d).to(dtype)
    v = inp["vc"].reshape(b, h, l, d).to(dtype)
    return k, v, inp["xq"].to(dtype), inp["static_src"].reshape(b, h, l).to(dtype), inp["static_dest"].to(dtype)


def test_brute_force_closed_form_l2():
    k = [[0.6, 0.8], [1.0, 0.0]]
    v = [[1.0, 2.0], [3.0, -1.0]]
    q = [[[0.3, -0.2], [0.5, 0.7]]]
    src, dest = [0.4, 0.9], [0.7, 0.2]
    O = orc.brute_force(k, v, q, src, dest)
    # t=0 sees only s=0
    assert O[0][0] == pytest.approx(v[0])
    a01 = (0.6 ** (2 / 3)) * (0.4 ** (1 / 3)) * (0.2 ** (1 / 3))
    s0 = (0.6 * 0.5 + 0.8 * 0.7) + math.log(1 - a01)
    s1 = 1.0 * 0.5
    w0 = math.exp(s0) / (math.exp(s0) + math.exp(s1))
    assert O[0][1] == pytest.approx([w0 * 1 + (1 - w0) * 3, w0 * 2 - (1 - w0)], rel=1e-12)


def test_bias_uses_source_gate_of_key_and_dest_gate_of_query():
    # a transposed gate (src_u, dest_s) must give a different answer
    k, v, q, src, dest = _rand(1, 1, 1, 6, 4, seed=3)
    B = orc.dense_bias(k, src, dest)[0, 0]
    G = (k[0, 0] @ k[0, 0].T).clamp(min=0) ** (2 / 3)
    s, t = 1, 4
    want = sum(math.log1p(-float(G[s, u] * src[0, 0, s] ** (1 / 3) * dest[0, 0, u] ** (1 / 3))) for u in range(s + 1, t + 1))
    assert float(B[s, t]) == pytest.approx(want, rel=1e-12)
    assert float(B[t, t]) == 0.0 and float(B[t, s]) == 0.0


def test_dense_matches_brute_force():
    b, h, r, l, d = 1, 2, 2, 12, 4
    k, v, q, src, dest = _rand(b, h, r, l, d, seed=5)
    O = orc.dense_forward(k, v, q, src, dest)
    for hh in range(h):
        bf = torch.tensor(orc.brute_force(k[0, hh].tolist(), v[0, hh].tolist(), q[0, hh].tolist(),
                                          src[0, hh].tolist(), dest[0, hh].tolist()), dtype=torch.float64)
        torch.testing.assert_close(O[0, hh], bf, rtol=1e-11, atol=1e-12)


def test_vanishing_gates_reduce_to_causal_sdpa():
    b, h, r, l, d = 2, 2, 1, 32, 8
    k, v, q, src, dest = _rand(b, h, r, l, d, seed=6)
    src = torch.full_like(src, 1e-300)
    O = orc.dense_forward(k, v, q, src, dest)[:, :, 0]
    want = F.scaled_dot_product_attention(q[:, :, 0], k, v, is_causal=True, scale=1.0)
    torch.testing.assert_close(O, want, rtol=1e-10, atol=1e-12)
    # orthogonal-or-opposed keys: relu kills the affinity as well
    k2 = -k.abs()
    k2[..., 0, :] = k.abs()[..., 0, :] * 0  # first key zero
    O2 = orc.dense_forward(-k.abs() * 0 + k2, v, q, torch.ones_like(src), dest)[:, :, 0]
    G = k2 @ k2.transpose(-1, -2)
    if (G.triu(1) <= 0).all():
        want2 = F.scaled_dot_product_attention(q[:, :, 0], k2, v, is_causal=True, scale=1.0)
        torch.testing.assert_close(O2, want2, rtol=1e-10, atol=1e-12)


def test_dense_gradcheck_float64():
    b, h, r, l, d = 1, 1, 2, 6, 3
    k, v, q, src, dest = [x.clone().requires_grad_() for x in _rand(b, h, r, l, d, seed=7)]
    assert torch.autograd.gradcheck(orc.dense_forward, (k, v, q, src, dest), eps=1e-6, atol=1e-6, rtol=1e-5)


@pytest.mark.parametrize("c", [4, 8, 16, 32])
def test_merged_chunks_equal_dense_for_every_chunk_size(c):
    b, h, r, l, d = 1, 2, 2, 32, 8
    inp = orc.make_inputs(b, h, r, l, d, c, dtype=torch.float64, seed=8)
    out, denom = orc.chunked_forward(inp["kc"], inp["vc"], inp["xq"], inp["static_src"], inp["static_dest"])
    O = orc.merge(out, denom)
    want = orc.dense_forward(inp["kc"].reshape(b, h, l, d), inp["vc"].reshape(b, h, l, d), inp["xq"],
                             inp["static_src"].reshape(b, h, l), inp["static_dest"])
    # the chunked restatement keeps the reference's .float() cast of the affinity, so fp32 accuracy
    torch.testing.assert_close(O, want, rtol=5e-5, atol=1e-6)


def test_fully_masked_pairs_are_uniform():
    b, h, r, l, d, c = 1, 1, 1, 32, 8, 8
    inp = orc.make_inputs(b, h, r, l, d, c, dtype=torch.float32, seed=9)
    out, denom = orc.chunked_forward(inp["kc"], inp["vc"], inp["xq"], inp["static_src"], inp["static_dest"])
    i = 2  # chunk 2 holds keys 16..23; queries 0..15 see none of them
    torch.testing.assert_close(out[0, 0, 0, :16, :, i], inp["vc"][0, 0, i].mean(0).expand(16, d), rtol=1e-6, atol=1e-6)
    assert (denom[0, 0, 0, :16, i] == torch.tensor(-1e12, dtype=torch.float32)).all()
    # rows of the softmax sum to one: merged weights of masked chunks are exactly zero
    w = torch.softmax(denom, dim=-1)
    assert float(w[0, 0, 0, :16, i].abs().max()) == 0.0


def _load(golden_dir, name):
    z = np.load(os.path.join(golden_dir, name + ".npz"))
    b, h, r, l, d, c, seed, is_bf16 = [int(x) for x in z["meta"]]
    dtype = torch.bfloat16 if is_bf16 else torch.float32
    t = {k: torch.from_numpy(z[k]) for k in z.files if k != "meta"}
    return t, dtype, (b, h, r, l, d, c, seed)


@pytest.mark.parametrize("name", ["tiny_fp32", "tiny_bf16", "small_fp32", "small_bf16"])
def test_chunked_oracle_matches_reference_golden(golden_dir, name):
    t, dtype, (b, h, r, l, d, c, seed) = _load(golden_dir, name)
    regen = orc.make_inputs(b, h, r, l, d, c, dtype=dtype, seed=seed)
    args = [t[k].to(dtype) for k in ("kc", "vc", "xq", "static_src", "static_dest")]
    for k, a in zip(("kc", "vc", "xq", "static_src", "static_dest"), args):
        assert torch.equal(a, regen[k]), k
    out, denom = orc.chunked_forward(*args)
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(out.float(), t["out"], **tol)
    torch.testing.assert_close(denom.float(), t["denom"], **tol)
    torch.testing.assert_close(out.float(), t["out2d"], **tol)       # 2-D tiling gives the same values
    torch.testing.assert_close(orc.merge(out, denom).float(), t["O"], **tol)
    # arbitrary upstream
    g_out = t["g_out"].to(dtype)
    g_denom = t["g_denom"].to(dtype)
    grads = orc.chunked_backward(*args, g_out, g_denom)
    gtol = dict(rtol=1e-4, atol=1e-4) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)
    for nm, g in zip(("dkc", "dvc", "dxq", "dsrc", "ddest"), grads):
        torch.testing.assert_close(g.float(), t[nm], **gtol, msg=lambda m, nm=nm: nm + ": " + m)
    # composite upstream through the merge
    d_out, d_denom = orc.merge_backward(out, denom, t["dO"].to(dtype))
    cgrads = orc.chunked_backward(*args, d_out, d_denom)
    for nm, g in zip(("dkc", "dvc", "dxq", "dsrc", "ddest"), cgrads):
        torch.testing.assert_close(g.float(), t["c_" + nm], **gtol, msg=lambda m, nm=nm: "c_" + nm + ": " + m)


def test_cfg0_forward_matches_reference_golden(golden_dir):
    z = np.load(os.path.join(golden_dir, "cfg0_fwd_fp32.npz"))
    b, h, r, l, d, c, seed, _ = [int(x) for x in z["meta"]]
    inp = orc.make_inputs(b, h, r, l, d, c, dtype=torch.float32, seed=seed)
    chk = np.array([float(inp[k].double().sum()) for k in ("kc", "vc", "xq", "static_src", "static_dest")])
    np.testing.assert_allclose(chk, z["input_checksum"], rtol=1e-12)
    out, denom = orc.chunked_forward(inp["kc"], inp["vc"], inp["xq"], inp["static_src"], inp["static_dest"])
    torch.testing.assert_close(denom, torch.from_numpy(z["denom"]), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(out[..., 0], torch.from_numpy(z["out_first"]), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(out[..., -1], torch.from_numpy(z["out_last"]), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(orc.merge(out, denom), torch.from_numpy(z["O"]), rtol=1e-5, atol=1e-6)


def test_hand_written_backward_equals_autograd_of_dense():
    b, h, r, l, d, c = 1, 2, 2, 32, 8, 8
    inp = orc.make_inputs(b, h, r, l, d, c, dtype=torch.float64, seed=10)
    names = ("kc", "vc", "xq", "static_src", "static_dest")
    out, denom = orc.chunked_forward(*[inp[k] for k in names])
    d_out, d_denom = orc.merge_backward(out, denom, inp["dO"])
    hand = orc.chunked_backward(*[inp[k] for k in names], d_out, d_denom)
    leaves = [inp[k].clone().requires_grad_() for k in names]
    O = orc.dense_forward(leaves[0].reshape(b, h, l, d), leaves[1].reshape(b, h, l, d), leaves[2],
                          leaves[3].reshape(b, h, l), leaves[4])
    auto = torch.autograd.grad(O, leaves, inp["dO"])
    for nm, a, g in zip(names, auto, hand):
        torch.testing.assert_close(g, a, rtol=1e-5, atol=1e-7, msg=lambda m, nm=nm: nm + ": " + m)


def test_merge_backward_equals_autograd():
    torch.manual_seed(0)
    out = torch.randn(2, 3, 5, 4, 6, dtype=torch.float64, requires_grad=True)
    denom = torch.randn(2, 3, 5, 6, dtype=torch.float64, requires_grad=True)
    g = torch.randn(2, 3, 5, 4, dtype=torch.float64)
    O = (out * torch.softmax(denom, -1)[..., None, :]).sum(-1)
    want = torch.autograd.grad(O, [out, denom], g)
    got = orc.merge_backward(out.detach(), denom.detach(), g)
    torch.testing.assert_close(got[0], want[0])
    torch.testing.assert_close(got[1], want[1])
    torch.testing.assert_close(orc.merge(out.detach(), denom.detach()), O.detach())


def test_affinity_scores_restatement_matches_dense_bias_and_the_reference_mask():
    """orc.affinity_scores (reference affinity_kernel_opt.py:457-462): transposed dense_bias where the key does not
    come after the query, -1e12 elsewhere, in the input dtype; a brute-force loop on a tiny case pins the layout."""
    import math
    g = torch.Generator().manual_seed(11)
    b, h, L, d = 1, 2, 12, 8
    k = torch.randn(b, h, L, d, generator=g, dtype=torch.float64)
    k = k / k.norm(dim=-1, keepdim=True)
    src = torch.sigmoid(torch.randn(b, h, L, generator=g, dtype=torch.float64))
    dest = torch.sigmoid(torch.randn(b, h, L, generator=g, dtype=torch.float64))
    aff = orc.affinity_scores(k, src, dest)
    assert aff.shape == (b, h, L, L)
    for hh in range(h):
        for t in range(L):
            for s in range(L):
                if s > t:
                    assert aff[0, hh, t, s] == -1e12
                    continue
                tot = 0.0
                for u in range(s + 1, t + 1):
                    a = max(float(k[0, hh, s] @ k[0, hh, u]), 0.0) ** (2 / 3) * float(src[0, hh, s] * dest[0, hh, u]) ** (1 / 3)
                    tot += math.log1p(-min(a, 1 - 1e-6))
                assert abs(float(aff[0, hh, t, s]) - tot) <= 1e-12 * max(1.0, abs(tot))
    assert orc.affinity_scores(k.to(torch.bfloat16), src.to(torch.bfloat16), dest.to(torch.bfloat16)).dtype == torch.bfloat16
