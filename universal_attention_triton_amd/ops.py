"""Host-side operators over the C ABI: tensor plumbing only (device memory, strides, streams)."""
import ctypes

import torch

from . import _lib
from ._lib import UaChunked, UaDesc, UaRows


def _dtype_code(t):
    if t.dtype == torch.bfloat16:
        return _lib.UA_BF16
    if t.dtype == torch.float32:
        return _lib.UA_F32
    raise TypeError("Universal Attention HIP kernels take float32 or bfloat16 tensors, got %s" % t.dtype)


def _require_gpu(*ts):
    for t in ts:
        if not t.is_cuda:
            raise _lib.UaError("Universal Attention HIP kernels need tensors on the GPU (got %s); there is no CPU path" % t.device)


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _last_contig(t):
    return t if t.stride(-1) == 1 else t.contiguous()


def _rows_k(t):
    """kc / vc: [b,h,n,c,d]"""
    return UaRows(t.data_ptr(), t.stride(0), t.stride(1), 0, t.stride(2), t.stride(3), t.shape[3])


def _rows_q(t):
    """xq: [b,h,r,l,d] or [b,h,r,_n,_c,d]"""
    if t.dim() == 5:
        return UaRows(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2), 0, t.stride(3), t.shape[3])
    return UaRows(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2), t.stride(3), t.stride(4), t.shape[4])


def _chunked(t):
    """[b,h,r,l,d,n] tensor -> (tensor kept alive, descriptor); the three leading dims must merge into one index,
    which `view` decides (it ignores the strides of size-1 dims); otherwise the tensor is copied."""
    L, d, n = t.shape[-3:]
    try:
        v = t.view(-1, L, d, n)
    except RuntimeError:
        t = t.contiguous()
        v = t.view(-1, L, d, n)
    return t, UaChunked(v.data_ptr(), v.stride(0), v.stride(1), v.stride(2), v.stride(3))


def _desc(kc, xq, chunked, flags=0):
    b, h, n, c, d = kc.shape
    r = xq.shape[2]
    return UaDesc(b, h, r, n * c, d, c if chunked else 0, _dtype_code(xq), flags)


def _workspace(desc, op, device):
    lib = _lib.load()
    nbytes = lib.ua_workspace_bytes(ctypes.byref(desc), op)
    if nbytes == 0:
        raise _lib.UaError("unsupported problem: " + lib.ua_last_error().decode())
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


def _prep(kc, vc, xq, static_src, static_dest):
    _require_gpu(kc, vc, xq, static_src, static_dest)
    if not (kc.dtype == vc.dtype == xq.dtype == static_src.dtype == static_dest.dtype):
        raise TypeError("all five inputs must share one dtype")
    b, h, n, c, d = kc.shape
    kc, vc, xq = _last_contig(kc), _last_contig(vc), _last_contig(xq)
    src = static_src.reshape(b, h, n * c).contiguous()
    dest = static_dest.reshape(b, h, n * c).contiguous()
    return kc, vc, xq, src, dest


def chunked_forward(kc, vc, xq, static_src, static_dest, for_backward=False, recompute=False):
    """-> out [b,h,r,l,d,n] (chunk-major storage, returned as a permuted view), denom [b,h,r,l,n], state
    recompute: size the state for a backward that runs with UA_FLAG_RECOMPUTE (pass the same value to chunked_backward)."""
    kc, vc, xq, src, dest = _prep(kc, vc, xq, static_src, static_dest)
    lib = _lib.load()
    b, h, n, c, d = kc.shape
    r = xq.shape[2]
    L = n * c
    desc = _desc(kc, xq, True, _lib.UA_FLAG_RECOMPUTE if recompute else 0)
    ws = _workspace(desc, _lib.UA_OP_BWD if for_backward else _lib.UA_OP_FWD, xq.device)
    store = torch.empty(b, h, r, n, L, d, dtype=xq.dtype, device=xq.device)
    out = store.permute(0, 1, 2, 4, 5, 3)
    denom = torch.empty(b, h, r, L, n, dtype=xq.dtype, device=xq.device)
    _, oc = _chunked(out)
    _lib.check(lib.ua_fwd(ctypes.byref(desc), ctypes.byref(_rows_k(kc)), ctypes.byref(_rows_k(vc)), ctypes.byref(_rows_q(xq)),
                          src.data_ptr(), dest.data_ptr(), ctypes.byref(oc), denom.data_ptr(), ws.data_ptr(), ws.numel(), _stream()),
               "ua_fwd")
    return out, denom, ws


def chunked_backward(kc, vc, xq, static_src, static_dest, out, g_out, g_denom, ws=None, skip_masked=False, recompute=False):
    kc, vc, xq, src, dest = _prep(kc, vc, xq, static_src, static_dest)
    lib = _lib.load()
    b, h, n, c, d = kc.shape
    r = xq.shape[2]
    L = n * c
    desc = _desc(kc, xq, True, (_lib.UA_FLAG_SKIP_MASKED if skip_masked else 0) | (_lib.UA_FLAG_RECOMPUTE if recompute else 0))
    has_fwd = ws is not None
    need = lib.ua_workspace_bytes(ctypes.byref(desc), _lib.UA_OP_BWD)
    if ws is None or ws.numel() < need:
        ws, has_fwd = _workspace(desc, _lib.UA_OP_BWD, xq.device), False
    out_t, oc = _chunked(out)
    g_out_t, gc = _chunked(g_out.to(xq.dtype))
    gd = g_denom.float().contiguous()
    dk = torch.empty(b, h, n, c, d, dtype=kc.dtype, device=kc.device)
    dv = torch.empty_like(dk)
    dq = torch.empty(b, h, r, L, d, dtype=xq.dtype, device=xq.device)
    dsrc = torch.empty(b, h, L, dtype=src.dtype, device=src.device)
    ddest = torch.empty_like(dsrc)
    _lib.check(lib.ua_bwd(ctypes.byref(desc), ctypes.byref(_rows_k(kc)), ctypes.byref(_rows_k(vc)), ctypes.byref(_rows_q(xq)),
                          src.data_ptr(), dest.data_ptr(), ctypes.byref(oc), ctypes.byref(gc), gd.data_ptr(), dk.data_ptr(),
                          dv.data_ptr(), dq.data_ptr(), dsrc.data_ptr(), ddest.data_ptr(), ws.data_ptr(), ws.numel(),
                          1 if has_fwd else 0, _stream()), "ua_bwd")
    del out_t, g_out_t
    return dk, dv, dq, dsrc, ddest


def _fused_flags(prune, recompute, share_groups=False):
    return ((_lib.UA_FLAG_PRUNE if prune else 0) | (_lib.UA_FLAG_RECOMPUTE if recompute else 0)
            | (_lib.UA_FLAG_SHARE_GROUPS if share_groups else 0))


def fused_forward(kc, vc, xq, static_src, static_dest, for_backward=False, prune=False, recompute=False, share_groups=False):
    """-> O [b,h,r,l,d], lse [b,h,r,l] (float32), state

    prune: skip (key, query) pairs whose softmax weight is provably below 2^-48 because of the accumulated decay
    (UA_FLAG_PRUNE); the backward that receives the returned state follows the same selection.
    recompute: size the state for a backward that runs with UA_FLAG_RECOMPUTE (pass the same value to fused_backward).
    share_groups: likewise for UA_FLAG_SHARE_GROUPS (grouped queries: one key-side sweep per kv head whatever the shape)."""
    kc, vc, xq, src, dest = _prep(kc, vc, xq, static_src, static_dest)
    lib = _lib.load()
    b, h, n, c, d = kc.shape
    r = xq.shape[2]
    L = n * c
    desc = _desc(kc, xq, False, _fused_flags(prune, recompute, share_groups))
    ws = _workspace(desc, _lib.UA_OP_FUSED_BWD if for_backward else _lib.UA_OP_FUSED_FWD, xq.device)
    O = torch.empty(b, h, r, L, d, dtype=xq.dtype, device=xq.device)
    lse = torch.empty(b, h, r, L, dtype=torch.float32, device=xq.device)
    _lib.check(lib.ua_fused_fwd(ctypes.byref(desc), ctypes.byref(_rows_k(kc)), ctypes.byref(_rows_k(vc)), ctypes.byref(_rows_q(xq)),
                                src.data_ptr(), dest.data_ptr(), O.data_ptr(), lse.data_ptr(), ws.data_ptr(), ws.numel(), _stream()),
               "ua_fused_fwd")
    return O, lse, ws


def fused_backward(kc, vc, xq, static_src, static_dest, O, lse, dO, ws=None, prune=False, recompute=False, share_groups=False,
                   _ws_override=None):
    """ws: the state fused_forward returned for the same inputs (skips the recompute and keeps its pruning);
    prune only matters when ws is None.  recompute: UA_FLAG_RECOMPUTE (small workspace, slower; bf16 only)."""
    kc, vc, xq, src, dest = _prep(kc, vc, xq, static_src, static_dest)
    lib = _lib.load()
    b, h, n, c, d = kc.shape
    r = xq.shape[2]
    L = n * c
    desc = _desc(kc, xq, False, _fused_flags(prune, recompute, share_groups))
    has_fwd = ws is not None
    need = lib.ua_workspace_bytes(ctypes.byref(desc), _lib.UA_OP_FUSED_BWD)
    if _ws_override is not None:
        ws, has_fwd = _ws_override, False
    elif ws is None or ws.numel() < need:
        ws, has_fwd = _workspace(desc, _lib.UA_OP_FUSED_BWD, xq.device), False
    O = O.contiguous()
    dO = dO.to(xq.dtype).contiguous()
    lse = lse.float().contiguous()
    dk = torch.empty(b, h, n, c, d, dtype=kc.dtype, device=kc.device)
    dv = torch.empty_like(dk)
    dq = torch.empty(b, h, r, L, d, dtype=xq.dtype, device=xq.device)
    dsrc = torch.empty(b, h, L, dtype=src.dtype, device=src.device)
    ddest = torch.empty_like(dsrc)
    _lib.check(lib.ua_fused_bwd(ctypes.byref(desc), ctypes.byref(_rows_k(kc)), ctypes.byref(_rows_k(vc)), ctypes.byref(_rows_q(xq)),
                                src.data_ptr(), dest.data_ptr(), O.data_ptr(), lse.data_ptr(), dO.data_ptr(), dk.data_ptr(),
                                dv.data_ptr(), dq.data_ptr(), dsrc.data_ptr(), ddest.data_ptr(), ws.data_ptr(), ws.numel(),
                                1 if has_fwd else 0, _stream()), "ua_fused_bwd")
    return dk, dv, dq, dsrc, ddest


def _merge_views(mat):
    """mat [..., L, d, n] -> 4-D view [Z, L, d, n] whose Z stride is uniform"""
    L, d, n = mat.shape[-3:]
    if mat.dim() == 4:
        m4 = mat
    else:
        try:
            m4 = mat.view(-1, L, d, n)
        except RuntimeError:
            m4 = mat.reshape(-1, L, d, n)
    return m4, UaChunked(m4.data_ptr(), m4.stride(0), m4.stride(1), m4.stride(2), m4.stride(3))


def merge_forward(mat, vec):
    """SMVecMatMul forward: mat [..., L, d, n], vec [..., L, n] -> [..., L, d]"""
    _require_gpu(mat, vec)
    lib = _lib.load()
    L, d, n = mat.shape[-3:]
    m4, mc = _merge_views(mat)
    vec_c = vec.to(mat.dtype).contiguous()
    rows = m4.shape[0] * L
    res = torch.empty(*mat.shape[:-2], d, dtype=mat.dtype, device=mat.device)
    _lib.check(lib.ua_merge_fwd(_dtype_code(mat), rows, L, d, n, ctypes.byref(mc), vec_c.data_ptr(), res.data_ptr(), _stream()),
               "ua_merge_fwd")
    return res


def merge_backward(mat, vec, g):
    _require_gpu(mat, vec, g)
    lib = _lib.load()
    L, d, n = mat.shape[-3:]
    m4, mc = _merge_views(mat)
    vec_c = vec.to(mat.dtype).contiguous()
    g_c = g.to(mat.dtype).contiguous()
    rows = m4.shape[0] * L
    # chunk-major storage: the gradient is consumed chunk by chunk by the chunked backward
    store = torch.empty(m4.shape[0], n, L, d, dtype=mat.dtype, device=mat.device)
    d4 = store.permute(0, 2, 3, 1)
    dc = UaChunked(d4.data_ptr(), d4.stride(0), d4.stride(1), d4.stride(2), d4.stride(3))
    d_vec = torch.empty(*vec.shape, dtype=mat.dtype, device=mat.device)
    _lib.check(lib.ua_merge_bwd(_dtype_code(mat), rows, L, d, n, ctypes.byref(mc), vec_c.data_ptr(), g_c.data_ptr(), ctypes.byref(dc),
                                d_vec.data_ptr(), _stream()), "ua_merge_bwd")
    d_mat = d4.unflatten(0, tuple(mat.shape[:-3])) if mat.dim() != 4 else d4
    return d_mat, d_vec.to(vec.dtype)


def autotune(kc, vc, xq, static_src, static_dest, dO=None, backward=True):
    """What the reference's @triton.autotune does on first call: runs the fused operator once on these inputs, then
    times every variant of every kernel on its path on the device (ua_autotune) and records the fastest of each in the
    library's table.  Returns {slot name: variant} for the slots that have more than one variant here."""
    lib = _lib.load()
    O, lse, ws = fused_forward(kc, vc, xq, static_src, static_dest, for_backward=True)
    kc_, vc_, xq_, _, _ = _prep(kc, vc, xq, static_src, static_dest)
    desc = _desc(kc_, xq_, False)
    _lib.check(lib.ua_autotune(ctypes.byref(desc), _lib.UA_OP_FUSED_FWD, ws.data_ptr(), ws.numel(), _stream()), "ua_autotune")
    if backward and xq.dtype == torch.bfloat16:
        # the number of key-side parts changes the workspace: tune it on a workspace large enough for every choice
        if dO is None:
            dO = torch.ones_like(O)
        need = max(_with_parts(desc, v, lambda: lib.ua_workspace_bytes(ctypes.byref(desc), _lib.UA_OP_FUSED_BWD))
                   for v in range(lib.ua_tune_variants(ctypes.byref(desc), _lib.UA_TUNE_BWD_PARTS)))
        big = torch.empty(need, dtype=torch.uint8, device=xq.device)
        fused_backward(kc, vc, xq, static_src, static_dest, O, lse, dO, ws=None, _ws_override=big)
        _lib.check(lib.ua_autotune(ctypes.byref(desc), _lib.UA_OP_FUSED_BWD, big.data_ptr(), big.numel(), _stream()), "ua_autotune")
    out = {name: lib.ua_tune_get(ctypes.byref(desc), slot) for name, slot in _lib.TUNE_SLOTS.items()
           if lib.ua_tune_variants(ctypes.byref(desc), slot) > 1 and lib.ua_tune_get(ctypes.byref(desc), slot) >= 0}
    from . import tune
    for name, v in out.items():
        tune.record(desc, name, v)
    return out


def _with_parts(desc, variant, fn):
    lib = _lib.load()
    old = lib.ua_tune_get(ctypes.byref(desc), _lib.UA_TUNE_BWD_PARTS)
    lib.ua_tune_set(ctypes.byref(desc), _lib.UA_TUNE_BWD_PARTS, variant)
    try:
        return fn()
    finally:
        lib.ua_tune_set(ctypes.byref(desc), _lib.UA_TUNE_BWD_PARTS, old)


def _slot(slot):
    return _lib.TUNE_SLOTS[slot] if isinstance(slot, str) else slot


def tune_variants(kc, xq, slot="fwd_tiles"):
    return _lib.load().ua_tune_variants(ctypes.byref(_desc(kc, xq, False)), _slot(slot))


def tune_set(kc, xq, variant, slot="fwd_tiles"):
    _lib.check(_lib.load().ua_tune_set(ctypes.byref(_desc(kc, xq, False)), _slot(slot), variant), "ua_tune_set")


def tune_get(kc, xq, slot="fwd_tiles"):
    return _lib.load().ua_tune_get(ctypes.byref(_desc(kc, xq, False)), _slot(slot))


def tune_choice(kc, xq, slot="fwd_tiles"):
    return _lib.load().ua_tune_choice(ctypes.byref(_desc(kc, xq, False)), _slot(slot))


def _affinity_args(k, src, dest):
    _require_gpu(k, src, dest)
    if not (k.dtype == src.dtype == dest.dtype):
        raise TypeError("k, src and dest must share one dtype")
    b, h, L, d = k.shape
    assert src.shape == (b, h, L) and dest.shape == (b, h, L)
    k = _last_contig(k)
    desc = UaDesc(b, h, 1, L, d, 0, _dtype_code(k), 0)
    rows = UaRows(k.data_ptr(), k.stride(0), k.stride(1), 0, 0, k.stride(2), L)
    return k, src.contiguous(), dest.contiguous(), desc, rows


def affinity_forward(k, src, dest):
    """k [b,h,L,d], src, dest [b,h,L] -> aff [b,h,L,L] (k.dtype): bias of key s towards query t at aff[b,h,t,s]"""
    k, src, dest, desc, rows = _affinity_args(k, src, dest)
    lib = _lib.load()
    b, h, L, _ = k.shape
    ws = torch.empty(lib.ua_affinity_workspace_bytes(ctypes.byref(desc), 0), dtype=torch.uint8, device=k.device)
    aff = torch.empty(b, h, L, L, dtype=k.dtype, device=k.device)
    _lib.check(lib.ua_affinity_fwd(ctypes.byref(desc), ctypes.byref(rows), src.data_ptr(), dest.data_ptr(), aff.data_ptr(),
                                   ws.data_ptr(), ws.numel(), _stream()), "ua_affinity_fwd")
    return aff


def affinity_backward(k, src, dest, daff):
    """-> dk [b,h,L,d], dsrc, ddest [b,h,L]"""
    k, src, dest, desc, rows = _affinity_args(k, src, dest)
    lib = _lib.load()
    b, h, L, d = k.shape
    daff = daff.to(k.dtype).contiguous()
    if daff.data_ptr() % 16:        # a contiguous view at an odd offset of its storage
        daff = daff.clone()
    ws = torch.empty(lib.ua_affinity_workspace_bytes(ctypes.byref(desc), 1), dtype=torch.uint8, device=k.device)
    dk = torch.empty(b, h, L, d, dtype=k.dtype, device=k.device)
    dsrc = torch.empty(b, h, L, dtype=k.dtype, device=k.device)
    ddest = torch.empty_like(dsrc)
    _lib.check(lib.ua_affinity_bwd(ctypes.byref(desc), ctypes.byref(rows), src.data_ptr(), dest.data_ptr(), daff.data_ptr(),
                                   dk.data_ptr(), dsrc.data_ptr(), ddest.data_ptr(), ws.data_ptr(), ws.numel(), _stream()),
               "ua_affinity_bwd")
    return dk, dsrc, ddest


def fused_forward_noalloc(kc, vc, xq, static_src, static_dest, O, lse):
    """ua_fused_fwd_noalloc: the fused forward into caller-provided O [b,h,r,l,d] (xq.dtype) and lse [b,h,r,l]
    (float32), with the library's built-in scratch instead of a workspace.  Nothing is allocated, so nothing is copied
    either: every tensor must already be laid out as the C ABI wants it (unit feature stride, contiguous gates and
    outputs); problems beyond ua_noalloc_scratch_bytes() raise UaError."""
    _require_gpu(kc, vc, xq, static_src, static_dest, O, lse)
    if not (kc.dtype == vc.dtype == xq.dtype == static_src.dtype == static_dest.dtype == O.dtype) or lse.dtype != torch.float32:
        raise TypeError("inputs and O share one dtype, lse is float32")
    for t in (kc, vc, xq):
        if t.stride(-1) != 1:
            raise ValueError("unit feature stride required (no copies are made)")
    for t in (static_src, static_dest, O, lse):
        if not t.is_contiguous():
            raise ValueError("gates and outputs must be contiguous (no copies are made)")
    lib = _lib.load()
    desc = _desc(kc, xq, False, 0)
    _lib.check(lib.ua_fused_fwd_noalloc(ctypes.byref(desc), ctypes.byref(_rows_k(kc)), ctypes.byref(_rows_k(vc)),
                                        ctypes.byref(_rows_q(xq)), static_src.data_ptr(), static_dest.data_ptr(), O.data_ptr(),
                                        lse.data_ptr(), _stream()), "ua_fused_fwd_noalloc")
    return O, lse
