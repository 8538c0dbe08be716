"""CPU oracle for Universal Attention -- TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this module: only the tests, the
smoke check and the benchmark's ``cpu_baseline`` leg use it, and only as the
checker.  The product path is the HIP library and fails loudly without it.

It restates, in plain PyTorch / Python, the algorithm of the reference's torch
operator (reference ``universal_attention_autograd.py``):

* ``chunked_forward``   follows ``UniversalAttention.forward``   (:9-38)
* ``chunked_backward``  follows ``UniversalAttention.backward``  (:47-99)
* ``merge`` / ``merge_backward`` follow ``SMVecMatMul``          (:278-297)
* ``dense_forward``     is the un-chunked closed form of the same operator
  (ordinary causal attention with the additive decay bias), differentiable by
  ``torch.autograd``; ``brute_force`` is the same thing as explicit Python
  loops in float64 for tiny inputs.

How each function is pinned (tests/test_oracle_*.py):

* ``brute_force``       hand-computed L=2 closed form; gates -> 0 reduces it to
                        textbook causal softmax attention (scale 1).
* ``dense_forward``     == ``brute_force`` on tiny inputs; == torch SDPA when the
                        bias vanishes; float64 ``gradcheck``.
* ``chunked_forward``   == golden vectors written by the reference operator
                        (tests/golden); merged result == ``dense_forward`` for
                        every chunk size; fully masked pairs give mean(V_chunk)
                        and float32(-1e12).
* ``chunked_backward``  == golden vectors; == autograd of ``dense_forward``
                        under a merged upstream gradient.
* ``merge``/``merge_backward``  == autograd of the plain softmax-weighted sum.
"""
from __future__ import annotations

import math

import torch

NEG_FILL = -1e12          # reference autograd.py:28
A_MAX = 1 - 1e-6          # reference autograd.py:26
A_MIN_BWD = 1e-6          # reference autograd.py:85


# --------------------------------------------------------------------------
# chunked operator with the reference's cast points
# --------------------------------------------------------------------------
def _decay_pieces(k_i, k_all_t, src3_i, dest3, first_col):
    """Return (G, E, A, bias) for one key chunk against the whole query axis.

    k_i [b,h,c,d], k_all_t [b,h,d,l], src3_i [b,h,c] (= src^(1/3)), dest3 [b,h,l].
    Cast points as in reference autograd.py:24-28: the K.K^T product, relu and
    pow(2/3) run in the input dtype, everything after is float32.
    """
    c = k_i.shape[-2]
    l = k_all_t.shape[-1]
    G = torch.matmul(k_i, k_all_t)                              # input dtype
    E = torch.pow(torch.relu(G), 2 / 3).float()
    A = E * src3_i[..., :, None] * dest3[..., None, :]
    logs = torch.log1p(-torch.clamp(A, min=0, max=A_MAX))
    logs = torch.triu(logs, diagonal=first_col + 1)             # keep s < t only
    bias = torch.cumsum(logs, dim=3)
    visible = torch.ones(c, l, dtype=torch.bool, device=k_i.device).triu(first_col)
    bias = torch.where(visible, bias, torch.full_like(bias, NEG_FILL))
    return G, E, A, bias


def chunked_forward(kc, vc, xq, static_src, static_dest):
    """kc,vc [b,h,n,c,d]; xq [b,h,r,l,d]; static_src [b,h,n,c]; static_dest [b,h,l].

    Returns out [b,h,r,l,d,n], denom [b,h,r,l,n] in xq.dtype.
    """
    b, h, r, l, d = xq.shape
    n, c = kc.shape[2], kc.shape[3]
    out = xq.new_empty(b, h, r, l, d, n)
    denom = xq.new_empty(b, h, r, l, n)
    src3 = static_src.pow(1 / 3)
    dest3 = static_dest.pow(1 / 3)
    k_all_t = kc.reshape(b, h, l, d).transpose(-1, -2)
    q_t = xq.transpose(-1, -2)                                   # b h r d l
    for i in range(n):
        k_i, v_i = kc[:, :, i], vc[:, :, i]
        _, _, _, bias = _decay_pieces(k_i, k_all_t, src3[:, :, i], dest3, i * c)
        score = torch.matmul(k_i[:, :, None], q_t) + bias[:, :, None]   # b h r c l (fp32)
        denom[..., i] = torch.logsumexp(score, dim=-2)
        prob = torch.softmax(score.transpose(-1, -2), dim=-1).to(xq.dtype)
        out[..., i] = torch.matmul(prob, v_i[:, :, None])
    return out, denom


def chunked_backward(kc, vc, xq, static_src, static_dest, g_out, g_denom):
    """Gradients of ``chunked_forward`` as the reference writes them by hand
    (autograd.py:47-99), including its epsilons and cast points."""
    b, h, r, l, d = xq.shape
    n, c = kc.shape[2], kc.shape[3]
    dkc = torch.zeros_like(kc)
    dvc = torch.zeros_like(vc)
    dxq = torch.zeros_like(xq)
    dsrc = torch.zeros_like(static_src)
    ddest = torch.zeros_like(static_dest)
    src3 = static_src.pow(1 / 3)
    dest3 = static_dest.pow(1 / 3)
    k_flat = kc.reshape(b, h, l, d)
    k_all_t = k_flat.transpose(-1, -2)
    q_t = xq.transpose(-1, -2)
    for i in range(n):
        k_i, v_i = kc[:, :, i], vc[:, :, i]
        src3_i = src3[:, :, i]
        go = g_out[..., i]                                       # b h r l d
        gd = g_denom[..., i]                                     # b h r l
        G, E, A, bias = _decay_pieces(k_i, k_all_t, src3_i, dest3, i * c)
        score = torch.matmul(k_i[:, :, None], q_t) + bias[:, :, None]   # b h r c l
        P = torch.softmax(score, dim=-2)

        dvc[:, :, i] += torch.matmul(P.to(dvc.dtype), go).sum(2)
        dP = torch.matmul(v_i[:, :, None], go.transpose(-1, -2))        # b h r c l
        dS = (dP - (dP * P).sum(-2, keepdim=True)) * P
        dS = dS + P * gd[..., None, :]
        dxq += torch.matmul(dS.to(dxq.dtype).transpose(-1, -2), k_i[:, :, None])
        dkc[:, :, i] += torch.matmul(
            dS.to(dkc.dtype).transpose(2, 3).flatten(3, 4), xq.flatten(2, 3))

        dB = dS.sum(2)                                           # b h c l
        dlog = dB.flip([3]).cumsum(3).flip([3]).triu(i * c + 1)  # suffix sums, s<t only
        dA = dlog / (A.clamp(min=A_MIN_BWD, max=A_MAX) - 1)
        dA = dA * A.ge(0) * A.le(A_MAX)
        dgate = (dA * E).to(static_src.dtype)
        dsrc[:, :, i] += (dgate * dest3[..., None, :]).sum(-1) / (3 * src3_i.pow(2))
        ddest += (dgate * src3_i[..., :, None]).sum(-2) / (3 * dest3.pow(2))

        dE = dA * (src3_i[..., :, None] * dest3[..., None, :])
        dG = dE.to(xq.dtype) * (G.abs().add(1e-9).pow(-1 / 3) * (2 / 3) * G.gt(0))
        dkc += torch.matmul(dG.transpose(-1, -2), k_i).view(b, h, n, c, d)
        dkc[:, :, i] += torch.matmul(dG, k_flat)
    return dkc, dvc, dxq, dsrc, ddest


def merge(out, denom):
    """SMVecMatMul.forward (autograd.py:280-283): softmax over the chunk axis of
    ``denom`` weights the per-chunk partial outputs."""
    w = torch.softmax(denom, dim=-1)
    return (out * w[..., None, :]).sum(-1)


def merge_backward(out, denom, g):
    """SMVecMatMul.backward (autograd.py:291-297)."""
    w = torch.softmax(denom, dim=-1)
    d_out = g[..., None] * w[..., None, :]
    d_w = (g[..., None] * out).sum(-2)
    d_denom = (d_w - (d_w * w).sum(-1, keepdim=True)) * w
    return d_out, d_denom


# --------------------------------------------------------------------------
# un-chunked closed form
# --------------------------------------------------------------------------
def dense_bias(k, static_src, static_dest):
    """B[s,t] = sum_{u=s+1..t} log(1 - clamp(relu(k_s.k_u)^(2/3) src_s^(1/3) dest_u^(1/3)))
    for s <= t (0 on the diagonal).  k [b,h,l,d], gates [b,h,l] -> [b,h,l(s),l(t)]."""
    G = torch.matmul(k, k.transpose(-1, -2))
    A = torch.relu(G).pow(2 / 3) * static_src.pow(1 / 3)[..., :, None] * static_dest.pow(1 / 3)[..., None, :]
    logs = torch.log1p(-A.clamp(min=0, max=A_MAX)).triu(1)
    return torch.cumsum(logs, dim=-1)


def affinity_scores(k, static_src, static_dest):
    """The bias as the L x L additive mask of the reference's stand-alone op (affinity_kernel_opt.py:457-462,
    _gen_affinity_scores_torch): [b,h,t,s], cumulative sum cast to k.dtype, -1e12 where the key comes after the query.
    Built on dense_bias, which the brute-force and closed-form tests pin."""
    B = dense_bias(k, static_src, static_dest).to(k.dtype)                      # [b,h,s,t]
    l = k.shape[-2]
    after = torch.ones(l, l, dtype=torch.bool, device=k.device).tril(-1)        # s > t
    return B.masked_fill(after, NEG_FILL).transpose(-1, -2).contiguous()


def dense_forward(k, v, q, static_src, static_dest, return_lse=False):
    """O[r,t] = sum_{s<=t} softmax_s(k_s.q_t + B[s,t]) v_s.

    k,v [b,h,l,d]; q [b,h,r,l,d]; gates [b,h,l].  Computed in the dtype given
    (use float64 for reference-grade values); differentiable.
    """
    l = k.shape[-2]
    B = dense_bias(k, static_src, static_dest)
    S = torch.matmul(k[:, :, None], q.transpose(-1, -2)) + B[:, :, None]   # b h r s t
    causal = torch.ones(l, l, dtype=torch.bool, device=k.device).triu(0)    # s <= t
    S = S.masked_fill(~causal, float("-inf"))
    lse = torch.logsumexp(S, dim=-2)                                         # b h r t
    P = torch.exp(S - lse[..., None, :])
    O = torch.matmul(P.transpose(-1, -2), v[:, :, None])
    return (O, lse) if return_lse else O


def brute_force(k, v, q, src, dest):
    """Float64 scalar loops for ONE (batch, head): k,v [l][d], q [r][l][d],
    src,dest [l] as nested lists / 1-D sequences.  Returns O[r][t][d] as lists.
    Written from the operator's definition, sharing no code with the above."""
    l, d, r = len(k), len(k[0]), len(q)
    dot = lambda x, y: sum(float(a) * float(b) for a, b in zip(x, y))
    logs = [[0.0] * l for _ in range(l)]
    for s in range(l):
        for u in range(s + 1, l):
            g = max(dot(k[s], k[u]), 0.0)
            a = (g ** (2.0 / 3.0)) * (float(src[s]) ** (1.0 / 3.0)) * (float(dest[u]) ** (1.0 / 3.0))
            a = min(max(a, 0.0), A_MAX)
            logs[s][u] = math.log1p(-a)
    O = [[[0.0] * d for _ in range(l)] for _ in range(r)]
    for g_ in range(r):
        for t in range(l):
            scores = []
            for s in range(t + 1):
                bias = sum(logs[s][u] for u in range(s + 1, t + 1))
                scores.append(dot(k[s], q[g_][t]) + bias)
            m = max(scores)
            w = [math.exp(x - m) for x in scores]
            z = sum(w)
            for s in range(t + 1):
                for e in range(d):
                    O[g_][t][e] += w[s] / z * float(v[s][e])
    return O


# --------------------------------------------------------------------------
# synthetic inputs shared by tests and the benchmark
# --------------------------------------------------------------------------
def make_inputs(b, h, r, l, d, c, dtype=torch.float32, seed=0, gate_mean=0.0, device="cpu"):
    """Seeded draws in float32 on the CPU, in a fixed order, then cast:
    kc ~ N(0,1) L2-normalised along d; vc, xq ~ N(0,1); gates = sigmoid(N(mu,1));
    dO ~ N(0,1).  Returns a dict in the 1-D layout of the reference operator."""
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(b, h, l, d, generator=g)
    k = k / k.norm(dim=-1, keepdim=True)
    v = torch.randn(b, h, l, d, generator=g)
    q = torch.randn(b, h, r, l, d, generator=g)
    src = torch.sigmoid(torch.randn(b, h, l, generator=g) + gate_mean)
    dest = torch.sigmoid(torch.randn(b, h, l, generator=g) + gate_mean)
    dO = torch.randn(b, h, r, l, d, generator=g)
    n = l // c
    cast = lambda x: x.to(dtype).to(device)
    return dict(
        kc=cast(k).view(b, h, n, c, d), vc=cast(v).view(b, h, n, c, d), xq=cast(q),
        static_src=cast(src).view(b, h, n, c), static_dest=cast(dest), dO=cast(dO))
