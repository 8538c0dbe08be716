"""ctypes binding of libua_hip.so (the C ABI declared in include/ua.h).

The library is the product path: there is no CPU or PyTorch fallback.  Loading fails
loudly when the shared object is missing, and every op raises if the C call reports an error.
"""
import ctypes
import os
import threading

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libua_hip.so")

UA_F32, UA_BF16 = 0, 1
UA_OP_FWD, UA_OP_BWD, UA_OP_FUSED_FWD, UA_OP_FUSED_BWD, UA_OP_BWD_SCRATCH, UA_OP_FUSED_BWD_SCRATCH = 0, 1, 2, 3, 4, 5
UA_TUNE_FWD_RECOMPUTE, UA_TUNE_CARRY, UA_TUNE_FWD_TILES, UA_TUNE_BWD_PARTS, UA_TUNE_BWD_QUERIES, UA_TUNE_BWD_KEYS = 2, 16, 17, 18, 19, 20
UA_TUNE_CHUNKED_PAIR, UA_TUNE_AFF_PAIR = 21, 22
TUNE_SLOTS = {"fwd_recompute": 2, "carry": 16, "fwd_tiles": 17, "bwd_parts": 18, "bwd_queries": 19, "bwd_keys": 20,
              "chunked_pair": 21, "aff_pair": 22}
UA_FLAG_SKIP_MASKED = 1
UA_FLAG_RECOMPUTE = 4
UA_FLAG_PRUNE = 2
UA_FLAG_SHARE_GROUPS = 8
UA_FLAG_GATES_F32 = 16

c_void_p, c_int, c_size_t, c_int64, c_int32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_int64, ctypes.c_int32


class UaDesc(ctypes.Structure):
    _fields_ = [(n, c_int32) for n in ("b", "h", "r", "L", "d", "chunk", "dtype", "flags")]


class UaRows(ctypes.Structure):
    _fields_ = [("ptr", c_void_p)] + [(n, c_int64) for n in ("stride_b", "stride_h", "stride_r", "stride_outer", "stride_inner")] + [("inner_len", c_int32)]


class UaChunked(ctypes.Structure):
    _fields_ = [("ptr", c_void_p)] + [(n, c_int64) for n in ("stride_z", "stride_t", "stride_d", "stride_i")]


P = ctypes.POINTER
# name -> (restype, argtypes); every symbol include/ua.h declares
SIGNATURES = {
    "ua_version": (c_int, []),
    "ua_last_error": (ctypes.c_char_p, []),
    "ua_source_hash": (ctypes.c_char_p, []),
    "ua_workspace_bytes": (c_size_t, [P(UaDesc), c_int]),
    "ua_fwd": (c_int, [P(UaDesc), P(UaRows), P(UaRows), P(UaRows), c_void_p, c_void_p, P(UaChunked), c_void_p, c_void_p, c_void_p, c_size_t,
                       c_void_p]),
    "ua_bwd": (c_int, [P(UaDesc), P(UaRows), P(UaRows), P(UaRows), c_void_p, c_void_p, P(UaChunked), P(UaChunked), c_void_p,
                       c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "ua_fused_fwd": (c_int, [P(UaDesc), P(UaRows), P(UaRows), P(UaRows), c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "ua_noalloc_scratch_bytes": (c_size_t, []),
    "ua_fused_fwd_noalloc": (c_int, [P(UaDesc), P(UaRows), P(UaRows), P(UaRows), c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ua_fused_bwd": (c_int, [P(UaDesc), P(UaRows), P(UaRows), P(UaRows), c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                             c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "ua_merge_fwd": (c_int, [c_int, c_int64, c_int32, c_int32, c_int32, P(UaChunked), c_void_p, c_void_p, c_void_p]),
    "ua_merge_bwd": (c_int, [c_int, c_int64, c_int32, c_int32, c_int32, P(UaChunked), c_void_p, c_void_p, P(UaChunked), c_void_p, c_void_p,
                             c_void_p]),
    "ua_affinity_workspace_bytes": (c_size_t, [P(UaDesc), c_int]),
    "ua_affinity_fwd": (c_int, [P(UaDesc), P(UaRows), c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "ua_affinity_bwd": (c_int, [P(UaDesc), P(UaRows), c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                                c_void_p]),
    "ua_autotune": (c_int, [P(UaDesc), c_int, c_void_p, c_size_t, c_void_p]),
    "ua_tune_get": (c_int, [P(UaDesc), c_int]),
    "ua_tune_set": (c_int, [P(UaDesc), c_int, c_int]),
    "ua_tune_variants": (c_int, [P(UaDesc), c_int]),
    "ua_tune_choice": (c_int, [P(UaDesc), c_int]),
    "ua_prof_enable": (None, [c_int]),
    "ua_prof_collect": (c_int, [ctypes.c_char_p, c_size_t]),
}

_lib = None
_lock = threading.Lock()


class UaError(RuntimeError):
    pass


def load():
    """Returns the loaded library; raises if it has not been built (python -m universal_attention_triton_amd.build)."""
    global _lib
    env_file = None
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise UaError("%s is missing: build it with `python -m universal_attention_triton_amd.build` "
                              "(there is no fallback path)" % LIB_PATH)
            lib = ctypes.CDLL(LIB_PATH)
            for name, (res, args) in SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype, fn.argtypes = res, args
            # a library older than the sources beside it would silently test and benchmark other code
            csrc = os.path.join(HERE, "csrc")
            if os.path.isdir(csrc) and os.environ.get("UA_ALLOW_STALE_LIB") != "1":
                from .build import source_hash
                built, now = lib.ua_source_hash().decode(), source_hash()
                if built != now:
                    raise UaError("%s was built from other sources (hash %s, sources now %s): rebuild it with "
                                  "`python -m universal_attention_triton_amd.build`" % (LIB_PATH, built, now))
            _lib = lib
            env_file = os.environ.get("UA_TUNE_FILE")
    if env_file and os.path.exists(env_file) and not getattr(load, "_env_done", False):
        load._env_done = True
        from . import tune
        tune.load(env_file)
    return _lib


def check(code, what):
    if code < 0:
        raise UaError("%s failed (%d): %s" % (what, code, load().ua_last_error().decode()))
    return code


def prof_enable(on=True):
    load().ua_prof_enable(1 if on else 0)


def prof_collect():
    """-> {kernel group: (launches, total_ms)} since the last call; synchronises the device."""
    buf = ctypes.create_string_buffer(8192)
    load().ua_prof_collect(buf, len(buf))
    out = {}
    for item in buf.value.decode().split(";"):
        if item:
            name, cnt, ms = item.rsplit(":", 2)
            out[name] = (int(cnt), float(ms))
    return out
