"""Model-side glue: call the fused operator on the tensors a decoder block holds, without copies.

The reference's driver (main.py:19-31) starts from projections laid out [batch, sequence, heads, head_dim] and one
tensor holding both gates, and reshapes them into the operator's chunked layout with transposes and views:

    xq = query_state.transpose(1, 2).view(b, n_kv, rep, s, d)
    kc = key_state.transpose(1, 2).view(b, n_kv, n_c, c, d)
    static = static.view(b, s, 2, n_kv).permute(2, 0, 3, 1);  static_src = static[0].view(b, n_kv, n_c, c);  static_dest = static[1]

Those views are not contiguous.  The HIP operator reads keys, values and queries through their strides (only the head
dimension must have stride 1), so nothing is copied on the way in except the two gate vectors (b*n_kv*s elements each).
"""
import torch

from .universal_attention import universal_attention


def split_gates(static, n_kv):
    """static [b, s, 2*n_kv] -> (static_src [b, n_kv, s], static_dest [b, n_kv, s]) as views (reference main.py:29-31)."""
    b, s, two_n = static.shape
    assert two_n == 2 * n_kv, "static must hold a source and a destination gate per kv head"
    st = static.view(b, s, 2, n_kv).permute(2, 0, 3, 1)
    return st[0], st[1]


def decoder_attention(query_state, key_state, value_state, static, chunk=128, prune=False, recompute=False):
    """query_state [b, s, n, d], key_state / value_state [b, s, n_kv, d], static [b, s, 2*n_kv] (gates in (0, 1))
    -> attention output [b, s, n, d] (a permuted view of the operator's [b, n_kv, rep, s, d] result).

    Query head j belongs to kv head j // rep (reference main.py:26: view(b, n_kv, rep, s, d)).  `chunk` only shapes the
    views the operator's interface asks for; the fused result does not depend on it.  Differentiable."""
    b, s, n, d = query_state.shape
    n_kv = key_state.shape[2]
    assert key_state.shape == (b, s, n_kv, d) and value_state.shape == (b, s, n_kv, d)
    assert n % n_kv == 0, "query heads must be a multiple of kv heads"
    rep = n // n_kv
    c = chunk if s % chunk == 0 else s
    xq = query_state.transpose(1, 2).unflatten(1, (n_kv, rep))          # [b, n_kv, rep, s, d], strided view
    kc = key_state.transpose(1, 2).unflatten(2, (s // c, c))            # [b, n_kv, n_c, c, d]
    vc = value_state.transpose(1, 2).unflatten(2, (s // c, c))
    src, dest = split_gates(static, n_kv)
    O = universal_attention(kc, vc, xq, src.unflatten(2, (s // c, c)), dest, prune=prune, recompute=recompute)
    return O.flatten(1, 2).transpose(1, 2)                              # [b, s, n, d]
