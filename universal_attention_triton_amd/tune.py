"""Persistence of the library's autotune table (what the reference's Triton autotuner keeps in its cache).

    save(path)            entries set by ops.autotune / ua_tune_set in this process -> JSON
    load(path)            JSON -> the library's table
    UA_TUNE_FILE=<path>   loaded once when the package is imported (if the file exists)

An entry is {"slot": name, "b": ..., "h": ..., "r": ..., "L": ..., "d": ..., "dtype": "bf16"|"fp32", "variant": v}: one
representative problem of the table key (kernel slot, dtype, padded head dim, r, log2 buckets of L and of b*h).
"""
import ctypes
import json
import os

from . import _lib

_recorded = {}


def record(desc, slot_name, variant):
    key = (slot_name, desc.b, desc.h, desc.r, desc.L, desc.d, desc.dtype)
    _recorded[key] = variant


def set_entry(b, h, r, L, d, dtype, slot_name, variant):
    lib = _lib.load()
    desc = _lib.UaDesc(b, h, r, L, d, 0, _lib.UA_BF16 if dtype in ("bf16", _lib.UA_BF16) else _lib.UA_F32, 0)
    _lib.check(lib.ua_tune_set(ctypes.byref(desc), _lib.TUNE_SLOTS[slot_name], variant), "ua_tune_set")
    record(desc, slot_name, variant)


def entries():
    return [{"slot": k[0], "b": k[1], "h": k[2], "r": k[3], "L": k[4], "d": k[5], "dtype": "bf16" if k[6] == _lib.UA_BF16 else "fp32",
             "variant": v} for k, v in sorted(_recorded.items())]


def save(path):
    with open(path, "w") as f:
        json.dump({"version": 1, "entries": entries()}, f, indent=1)


def load(path):
    with open(path) as f:
        data = json.load(f)
    n = 0
    for e in data.get("entries", []):
        set_entry(e["b"], e["h"], e["r"], e["L"], e["d"], e["dtype"], e["slot"], e["variant"])
        n += 1
    return n


def load_env():
    path = os.environ.get("UA_TUNE_FILE")
    if path and os.path.exists(path):
        return load(path)
    return 0
