"""Host-side operators over the C ABI: tensor plumbing only (device memory, strides, streams)."""
import ctypes
import functools
import weakref

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
    """Checks the shapes against one another (the kernels trust the descriptor), makes the feature stride 1 and the
    gates contiguous [b,h,L].  -> kc, vc, xq, src, dest, gate flag.

    dtypes: kc, vc and xq share one dtype (float32 or bfloat16).  The gates may have it too; any other combination
    (float32 gates next to bfloat16 tensors, as the reference allows: its dstatic_src follows static_src.dtype,
    Universal_Attention/triton/universal_attention_kernel.py:825-829) runs with float32 gates."""
    if kc.dim() != 5 or vc.dim() != 5 or xq.dim() not in (5, 6):
        raise ValueError("kc, vc [b,h,n,c,d] and xq [b,h,r,l,d] or [b,h,r,_n,_c,d] expected, got %s %s %s"
                         % (tuple(kc.shape), tuple(vc.shape), tuple(xq.shape)))
    if not (kc.dtype == vc.dtype == xq.dtype):
        raise TypeError("kc, vc and xq must share one dtype, got %s %s %s" % (kc.dtype, vc.dtype, xq.dtype))
    b, h, n, c, d = kc.shape
    L = n * c
    seq = xq.shape[3] if xq.dim() == 5 else xq.shape[3] * xq.shape[4]
    if vc.shape != kc.shape:
        raise ValueError("vc %s does not match kc %s" % (tuple(vc.shape), tuple(kc.shape)))
    if xq.shape[0] != b or xq.shape[1] != h or xq.shape[-1] != d or seq != L:
        raise ValueError("xq %s does not match kc %s: need [b=%d, h=%d, r, %d positions, d=%d]" % (tuple(xq.shape), tuple(kc.shape), b, h, L, d))
    if static_src.numel() != b * h * L or static_dest.numel() != b * h * L or static_src.shape[:2] != (b, h) or static_dest.shape[:2] != (b, h):
        raise ValueError("gates %s / %s do not match [b=%d, h=%d, %d positions]" % (tuple(static_src.shape), tuple(static_dest.shape), b, h, L))
    _dtype_code(xq)
    _require_gpu(kc, vc, xq, static_src, static_dest)
    kc, vc, xq = _last_contig(kc), _last_contig(vc), _last_contig(xq)
    same = static_src.dtype == xq.dtype and static_dest.dtype == xq.dtype
    gdt = xq.dtype if same else torch.float32
    src = static_src.reshape(b, h, L).to(gdt).contiguous()
    dest = static_dest.reshape(b, h, L).to(gdt).contiguous()
    gflag = _lib.UA_FLAG_GATES_F32 if (gdt == torch.float32 and xq.dtype != torch.float32) else 0
    return kc, vc, xq, src, dest, gflag


# One grid row per head: the entry points refuse more than 65535 of them (b * h * r, times the chunks per row for the
# chunked operator).  Heads are independent, so the operators below split such a call along b, then h, run the pieces one
# after the other and join the results; the pieces keep no forward state (the backward rebuilds it per piece).
_GRID_ROWS = 65535


def _split_over_heads(n_tensors, chunked):
    def wrap(fn):
        @functools.wraps(fn)
        def run(*args, **kw):
            kc, xq = args[0], args[2]
            b, h = kc.shape[:2]
            per_head = xq.shape[2] * (kc.shape[2] if chunked else 1)
            if b * h * per_head <= _GRID_ROWS:
                return fn(*args, **kw)
            if per_head > _GRID_ROWS:
                raise _lib.UaError("%d grid rows per kv head exceed the limit of %d" % (per_head, _GRID_ROWS))
            step_h = min(h, _GRID_ROWS // per_head)
            step_b = max(1, _GRID_ROWS // (h * per_head)) if step_h == h else 1
            kw = {**kw, "state": None} if "state" in kw else dict(kw, **({"keep_state": False} if "keep_state" in kw else {}))
            rows = []
            for b0 in range(0, b, step_b):
                row = []
                for h0 in range(0, h, step_h):
                    # tensors beyond the per-head ones (a forward state passed by position) belong to the whole call: dropped
                    piece = [a[b0:b0 + step_b, h0:h0 + step_h] if i < n_tensors else (None if torch.is_tensor(a) else a)
                             for i, a in enumerate(args)]
                    row.append(fn(*piece, **kw))
                rows.append([None if row[0][i] is None else (row[0][i] if len(row) == 1 else torch.cat([p[i] for p in row], 1))
                             for i in range(len(row[0]))])
            return tuple(None if rows[0][i] is None else (rows[0][i] if len(rows) == 1 else torch.cat([r_[i] for r_ in rows], 0))
                         for i in range(len(rows[0])))
        return run
    return wrap


@_split_over_heads(5, True)
def chunked_forward(kc, vc, xq, static_src, static_dest, keep_state=False, recompute=False, contiguous_out=False):
    """-> out [b,h,r,l,d,n] (chunk-major storage, returned as a permuted view), denom [b,h,r,l,n], state
    contiguous_out: allocate `out` contiguous in the reference's index order instead (what `.view()` on it needs; the
    kernels then write 2-byte elements n * 2 bytes apart and every pass over `out` is several times slower).
    keep_state: what chunked_backward gets from the forward.  False: nothing (it rebuilds everything, including a
    second run of the forward kernel).  "normalisers": the per-chunk normalisers in float32 (1/(d+1) of the size of
    `out`; the backward then only repacks the inputs and rebuilds the decay carries).  True: the whole forward state (the
    workspace, ua_workspace_bytes(UA_OP_FWD) bytes).
    recompute: the flags of the state must match the backward's (pass the same value to chunked_backward)."""
    kc, vc, xq, src, dest, gflag = _prep(kc, vc, xq, static_src, static_dest)
    lib = _lib.load()
    b, h, n, c, d = kc.shape
    r = xq.shape[2]
    L = n * c
    desc = _desc(kc, xq, True, (_lib.UA_FLAG_RECOMPUTE if recompute else 0) | gflag)
    ws = _workspace(desc, _lib.UA_OP_FWD, xq.device)
    if contiguous_out:
        out = torch.empty(b, h, r, L, d, n, dtype=xq.dtype, device=xq.device)
    else:
        out = torch.empty(b, h, r, n, L, d, dtype=xq.dtype, device=xq.device).permute(0, 1, 2, 4, 5, 3)
    denom = torch.empty(b, h, r, L, n, dtype=xq.dtype, device=xq.device)
    _, oc = _chunked(out)
    lse2 = None
    if keep_state == "normalisers":
        lse2 = torch.empty(b * h * r * n * (-(-L // 128) * 128), dtype=torch.float32, device=xq.device)
    _lib.check(lib.ua_fwd(ctypes.byref(desc), ctypes.byref(_rows_k(kc)), ctypes.byref(_rows_k(vc)), ctypes.byref(_rows_q(xq)),
                          src.data_ptr(), dest.data_ptr(), ctypes.byref(oc), denom.data_ptr(),
                          lse2.data_ptr() if lse2 is not None else None, ws.data_ptr(), ws.numel(), _stream()), "ua_fwd")
    return out, denom, (lse2 if lse2 is not None else (ws if keep_state else None))


def _gate_grads(b, h, L, src, static_src, static_dest):
    dsrc = torch.empty(b, h, L, dtype=src.dtype, device=src.device)
    return dsrc, torch.empty_like(dsrc)


# merge_backward attaches to the gradient tensor it returns for `mat` what a chunked_backward that receives exactly that
# tensor can reuse: the per-(row, chunk) term delta = sum_d out g_out - g_denom, with the identities of the tensors it
# belongs to.  The note lives on the tensor object and dies with it; a gradient that was accumulated with another one,
# replaced by a hook or modified in place is another object or version and simply has no (valid) note.
_NOTE = "_ua_merge_note"


def _delta_from_merge(out, g_out, g_denom, L, n):
    note = getattr(g_out, _NOTE, None)
    if note is None:
        return None
    w_vec, out_id, v_mat, v_vec, delta = note
    # `out`: alive since the forward, so the tensor merged at that address with this shape and these strides was this one
    if w_vec() is g_denom and out_id == (out.data_ptr(), tuple(out.shape), tuple(out.stride()), out._version) \
            and g_out._version == v_mat and g_denom._version == v_vec and delta.shape[1] == n and delta.shape[2] >= L:
        return delta
    return None


@_split_over_heads(8, True)
def chunked_backward(kc, vc, xq, static_src, static_dest, out, g_out, g_denom, state=None, skip_masked=False, recompute=False):
    """state: what chunked_forward(keep_state=True) returned for the same inputs and flags, or None.
    When (g_out, g_denom) are the very tensors merge_backward produced from `out` (the reference's call sequence), the
    backward takes delta = sum_d out g_out - g_denom from that call instead of reading both 4-GB-class tensors again,
    and knows that the gradients vanish where a query precedes a chunk."""
    src_dtype, dest_dtype = static_src.dtype, static_dest.dtype
    if state is not None and state.numel() == 0:
        state = None
    delta = None
    if kc.shape[3] % 64 == 0:
        delta = _delta_from_merge(out, g_out, g_denom, kc.shape[2] * kc.shape[3], kc.shape[2])
        if delta is not None:
            skip_masked = True
    kc, vc, xq, src, dest, gflag = _prep(kc, vc, xq, static_src, static_dest)
    lib = _lib.load()
    b, h, n, c, d = kc.shape
    r = xq.shape[2]
    L = n * c
    desc = _desc(kc, xq, True, (_lib.UA_FLAG_SKIP_MASKED if skip_masked else 0) | (_lib.UA_FLAG_RECOMPUTE if recompute else 0) | gflag)
    lse2 = None
    if state is not None and state.dtype == torch.float32:        # the normalisers alone
        lse2, state = state, None
        if lse2.numel() != b * h * r * n * (-(-L // 128) * 128):
            lse2 = None
    if state is not None and state.numel() < lib.ua_workspace_bytes(ctypes.byref(desc), _lib.UA_OP_FWD):
        state = None
    ws = _workspace(desc, _lib.UA_OP_BWD_SCRATCH if state is not None else _lib.UA_OP_BWD, xq.device)
    out_t, oc = _chunked(out)
    g_out_t, gc = _chunked(g_out.to(xq.dtype))
    gd = g_denom.float().contiguous()
    dk = torch.empty(b, h, n, c, d, dtype=kc.dtype, device=kc.device)
    dv = torch.empty_like(dk)
    dq = torch.empty(b, h, r, L, d, dtype=xq.dtype, device=xq.device)
    dsrc, ddest = _gate_grads(b, h, L, src, static_src, static_dest)
    _lib.check(lib.ua_bwd(ctypes.byref(desc), ctypes.byref(_rows_k(kc)), ctypes.byref(_rows_k(vc)), ctypes.byref(_rows_q(xq)),
                          src.data_ptr(), dest.data_ptr(), ctypes.byref(oc), ctypes.byref(gc), gd.data_ptr(), dk.data_ptr(),
                          dv.data_ptr(), dq.data_ptr(), dsrc.data_ptr(), ddest.data_ptr(),
                          delta.data_ptr() if delta is not None else None, lse2.data_ptr() if lse2 is not None else None,
                          state.data_ptr() if state is not None else None, ws.data_ptr(), ws.numel(), _stream()), "ua_bwd")
    del out_t, g_out_t
    return dk, dv, dq, dsrc.to(src_dtype), ddest.to(dest_dtype)


def _fused_flags(prune, recompute, share_groups=False):
    return ((_lib.UA_FLAG_PRUNE if prune else 0) | (_lib.UA_FLAG_RECOMPUTE if recompute else 0)
            | (_lib.UA_FLAG_SHARE_GROUPS if share_groups else 0))


@_split_over_heads(5, False)
def fused_forward(kc, vc, xq, static_src, static_dest, keep_state=False, prune=False, recompute=False, share_groups=False,
                  _ws=None):
    """-> O [b,h,r,l,d], lse [b,h,r,l] (float32), state

    keep_state: return the forward state (the workspace: packed inputs and, for bf16, the bias tiles;
    ua_workspace_bytes(UA_OP_FUSED_FWD) bytes) so that fused_backward need not rebuild it; otherwise state is None.
    prune: skip (key, query) pairs whose softmax weight is provably below 2^-48 because of the accumulated decay
    (UA_FLAG_PRUNE); a backward that receives the returned state follows the same selection.
    recompute, share_groups: flags of the state; pass the same values to fused_backward."""
    kc, vc, xq, src, dest, gflag = _prep(kc, vc, xq, static_src, static_dest)
    lib = _lib.load()
    b, h, n, c, d = kc.shape
    r = xq.shape[2]
    L = n * c
    desc = _desc(kc, xq, False, _fused_flags(prune, recompute, share_groups) | gflag)
    ws = _ws if _ws is not None else _workspace(desc, _lib.UA_OP_FUSED_FWD, xq.device)
    O = torch.empty(b, h, r, L, d, dtype=xq.dtype, device=xq.device)
    lse = torch.empty(b, h, r, L, dtype=torch.float32, device=xq.device)
    _lib.check(lib.ua_fused_fwd(ctypes.byref(desc), ctypes.byref(_rows_k(kc)), ctypes.byref(_rows_k(vc)), ctypes.byref(_rows_q(xq)),
                                src.data_ptr(), dest.data_ptr(), O.data_ptr(), lse.data_ptr(), ws.data_ptr(), ws.numel(), _stream()),
               "ua_fused_fwd")
    return O, lse, (ws if keep_state else None)


@_split_over_heads(8, False)
def fused_backward(kc, vc, xq, static_src, static_dest, O, lse, dO, state=None, prune=False, recompute=False, share_groups=False,
                   _ws=None):
    """state: what fused_forward(keep_state=True) returned for the same inputs and flags (skips the recompute and keeps
    its pruning), or None; prune only matters without it.  recompute: UA_FLAG_RECOMPUTE (small workspace, slower; bf16)."""
    src_dtype, dest_dtype = static_src.dtype, static_dest.dtype
    kc, vc, xq, src, dest, gflag = _prep(kc, vc, xq, static_src, static_dest)
    lib = _lib.load()
    b, h, n, c, d = kc.shape
    r = xq.shape[2]
    L = n * c
    desc = _desc(kc, xq, False, _fused_flags(prune, recompute, share_groups) | gflag)
    if state is not None and state.numel() == 0:
        state = None
    if state is not None and state.numel() < lib.ua_workspace_bytes(ctypes.byref(desc), _lib.UA_OP_FUSED_FWD):
        state = None
    ws = _ws if _ws is not None else _workspace(desc, _lib.UA_OP_FUSED_BWD_SCRATCH if state is not None else _lib.UA_OP_FUSED_BWD, xq.device)
    O = O.contiguous()
    dO = dO.to(xq.dtype).contiguous()
    lse = lse.float().contiguous()
    dk = torch.empty(b, h, n, c, d, dtype=kc.dtype, device=kc.device)
    dv = torch.empty_like(dk)
    dq = torch.empty(b, h, r, L, d, dtype=xq.dtype, device=xq.device)
    dsrc, ddest = _gate_grads(b, h, L, src, static_src, static_dest)
    _lib.check(lib.ua_fused_bwd(ctypes.byref(desc), ctypes.byref(_rows_k(kc)), ctypes.byref(_rows_k(vc)), ctypes.byref(_rows_q(xq)),
                                src.data_ptr(), dest.data_ptr(), O.data_ptr(), lse.data_ptr(), dO.data_ptr(), dk.data_ptr(),
                                dv.data_ptr(), dq.data_ptr(), dsrc.data_ptr(), ddest.data_ptr(),
                                state.data_ptr() if state is not None else None, ws.data_ptr(), ws.numel(), _stream()), "ua_fused_bwd")
    return dk, dv, dq, dsrc.to(src_dtype), ddest.to(dest_dtype)


def retained_bytes(kc, vc, xq, static_src, static_dest, recompute=False, chunked=False):
    """Bytes of forward state the fused operator (chunked=True: the chunked operator with keep_state=True) keeps alive
    between forward and backward (fused operator with recompute: 0)."""
    kc, vc, xq, src, dest, gflag = _prep(kc, vc, xq, static_src, static_dest)
    if recompute and not chunked:
        return 0
    desc = _desc(kc, xq, chunked, gflag | (_lib.UA_FLAG_RECOMPUTE if recompute else 0))
    return _lib.load().ua_workspace_bytes(ctypes.byref(desc), _lib.UA_OP_FWD if chunked else _lib.UA_OP_FUSED_FWD)


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
    Lp = -(-L // 128) * 128
    # the per-(row, chunk) term is only worth keeping where a chunked backward can take it: chunks that are a multiple of 64
    delta = None
    if L % n == 0 and (L // n) % 64 == 0:
        delta = torch.zeros(m4.shape[0], n, Lp, dtype=torch.float32, device=mat.device)
    _lib.check(lib.ua_merge_bwd(_dtype_code(mat), rows, L, d, n, ctypes.byref(mc), vec_c.data_ptr(), g_c.data_ptr(), ctypes.byref(dc),
                                d_vec.data_ptr(), delta.data_ptr() if delta is not None else None, _stream()), "ua_merge_bwd")
    d_mat = d4.unflatten(0, tuple(mat.shape[:-3])) if mat.dim() != 4 else d4
    d_vec = d_vec.to(vec.dtype)
    if delta is None:
        return d_mat, d_vec
    try:
        setattr(d_mat, _NOTE, (weakref.ref(d_vec), (mat.data_ptr(), tuple(mat.shape), tuple(mat.stride()), mat._version),
                               d_mat._version, d_vec._version, delta))
    except (AttributeError, TypeError):          # a tensor subclass without instance attributes: no note, no shortcut
        pass
    return d_mat, d_vec


def autotune(kc, vc, xq, static_src, static_dest, dO=None, backward=True):
    """What the reference's @triton.autotune does on first call: runs the fused operator once on these inputs, then
    times every variant of every kernel on its path on the device (ua_autotune) and records the fastest of each in the
    library's table.  Returns {slot name: variant} for the slots that have more than one variant here."""
    lib = _lib.load()
    kc_, vc_, xq_, _, _, gflag = _prep(kc, vc, xq, static_src, static_dest)
    desc = _desc(kc_, xq_, False, gflag)
    bwd = backward and xq.dtype == torch.bfloat16
    # state and scratch in one buffer; the number of key-side parts changes its size: large enough for every choice
    n_parts = lib.ua_tune_variants(ctypes.byref(desc), _lib.UA_TUNE_BWD_PARTS) if bwd else 1
    need = max(_with_parts(desc, v if n_parts > 1 else -1, lambda: lib.ua_workspace_bytes(ctypes.byref(desc), _lib.UA_OP_FUSED_BWD))
               for v in range(n_parts))
    fwd_bytes = lib.ua_workspace_bytes(ctypes.byref(desc), _lib.UA_OP_FUSED_FWD)
    if need == 0 or fwd_bytes == 0:
        raise _lib.UaError("unsupported problem: " + lib.ua_last_error().decode())
    big = torch.empty(need, dtype=torch.uint8, device=xq.device)
    O, lse, _ = fused_forward(kc, vc, xq, static_src, static_dest, _ws=big)
    _lib.check(lib.ua_autotune(ctypes.byref(desc), _lib.UA_OP_FUSED_FWD, big.data_ptr(), big.numel(), _stream()), "ua_autotune")
    if bwd:
        if dO is None:
            dO = torch.ones_like(O)
        fused_backward(kc, vc, xq, static_src, static_dest, O, lse, dO, state=big, _ws=big[fwd_bytes:])
        _lib.check(lib.ua_autotune(ctypes.byref(desc), _lib.UA_OP_FUSED_BWD, big.data_ptr(), big.numel(), _stream()), "ua_autotune")
    out = {name: lib.ua_tune_get(ctypes.byref(desc), slot) for name, slot in _lib.TUNE_SLOTS.items()
           if lib.ua_tune_variants(ctypes.byref(desc), slot) > 1 and lib.ua_tune_get(ctypes.byref(desc), slot) >= 0}
    from . import tune
    for name, v in out.items():
        tune.record(desc, name, v)
    return out



def _time_variants(desc, slot, run, repeats=5):
    """Times run() under every variant of `slot` for desc (median of `repeats` after one warm-up each, hipEvents on the
    current stream), records the fastest in the library's table and returns it."""
    lib = _lib.load()
    n = lib.ua_tune_variants(ctypes.byref(desc), slot)
    best, best_ms = 0, None
    for v in range(n):
        _lib.check(lib.ua_tune_set(ctypes.byref(desc), slot, v), "ua_tune_set")
        run()
        ms = []
        for _ in range(repeats):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            run()
            e1.record()
            e1.synchronize()
            ms.append(e0.elapsed_time(e1))
        med = sorted(ms)[len(ms) // 2]
        if best_ms is None or med < best_ms:
            best, best_ms = v, med
    _lib.check(lib.ua_tune_set(ctypes.byref(desc), slot, best), "ua_tune_set")
    from . import tune
    name = next(k for k, s_ in _lib.TUNE_SLOTS.items() if s_ == slot)
    tune.record(desc, name, best)
    return best


def autotune_chunked(kc, vc, xq, static_src, static_dest, repeats=5):
    """Chunked operator with a chunk that is a multiple of 64: times its forward + backward under each variant of the
    slot `chunked_pair` (work items per workgroup) on these inputs and records the fastest.  -> {"chunked_pair": variant}"""
    if kc.shape[3] % 64:
        return {}
    kc_, _, xq_, _, _, gflag = _prep(kc, vc, xq, static_src, static_dest)
    desc = _desc(kc_, xq_, False, gflag)
    g = {}

    def run():
        out, denom, state = chunked_forward(kc, vc, xq, static_src, static_dest, keep_state=True)
        if "out" not in g:
            g["out"], g["denom"] = torch.ones_like(out), torch.zeros(denom.shape, dtype=torch.float32, device=denom.device)
        chunked_backward(kc, vc, xq, static_src, static_dest, out, g["out"], g["denom"], state=state)

    with torch.no_grad():
        return {"chunked_pair": _time_variants(desc, _lib.UA_TUNE_CHUNKED_PAIR, run, repeats)}


def autotune_affinity(k, src, dest, repeats=5):
    """Stand-alone bias: times its forward + backward under each variant of the slot `aff_pair` and records the fastest."""
    k_, src_, dest_, desc, _ = _affinity_args(k, src, dest)
    daff = torch.ones(*k.shape[:3], k.shape[2], dtype=k.dtype, device=k.device)

    def run():
        affinity_forward(k, src, dest)
        affinity_backward(k, src, dest, daff)

    with torch.no_grad():
        return {"aff_pair": _time_variants(desc, _lib.UA_TUNE_AFF_PAIR, run, repeats)}


_first_call_tuned = set()


def autotune_on_first_call(kc, vc, xq, static_src, static_dest):
    """UA_AUTOTUNE=1 in the environment: the fused operator tunes itself the first time it meets a table key (dtype,
    padded head dim, r, size buckets of L and b*h), as the reference's @triton.autotune does per key
    (universal_attention_kernel_opt.py:24-44).  Synchronises the device, so not for code under graph capture."""
    import os
    if os.environ.get("UA_AUTOTUNE") != "1" or torch.cuda.is_current_stream_capturing():
        return None
    b, h, n, c, d = kc.shape
    L = n * c
    key = (xq.dtype, 64 if d <= 64 else (128 if d <= 128 else 256), xq.shape[2], max(0, (L - 1).bit_length() - 7), (b * h - 1).bit_length())
    if key in _first_call_tuned:
        return None
    _first_call_tuned.add(key)
    with torch.no_grad():
        return autotune(*[t.detach() for t in (kc, vc, xq, static_src, static_dest)])

def _with_parts(desc, variant, fn):
    lib = _lib.load()
    if variant < 0:
        return fn()
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
    b, h, n, c, d = kc.shape
    if vc.shape != kc.shape or xq.shape[:2] != (b, h) or xq.shape[-1] != d or xq.numel() != b * h * xq.shape[2] * n * c * d \
            or static_src.numel() != b * h * n * c or static_dest.numel() != b * h * n * c \
            or O.numel() != xq.numel() or lse.numel() * d != xq.numel():
        raise ValueError("shapes of the tensors do not match one another")
    _lib.check(lib.ua_fused_fwd_noalloc(ctypes.byref(desc), ctypes.byref(_rows_k(kc)), ctypes.byref(_rows_k(vc)),
                                        ctypes.byref(_rows_q(xq)), static_src.data_ptr(), static_dest.data_ptr(), O.data_ptr(),
                                        lse.data_ptr(), _stream()), "ua_fused_fwd_noalloc")
    return O, lse
