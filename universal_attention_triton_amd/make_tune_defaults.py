"""Regenerates csrc/ua_tune_defaults.inc: runs ua_autotune on this GPU for the shapes of the reference's benchmark
recipes (and the repository's BASELINE configurations) and writes one built-in table entry per (kernel slot, shape).
Rebuild the library afterwards.  `python -m universal_attention_triton_amd.make_tune_defaults [repeats]`"""
import collections
import os
import sys

import torch

from . import _lib, ops

# b, h(kv), r, L, d  (bf16): BASELINE configs 1-4; the reference's "important config to test on" (_debug.py:599) and
# the sizes of its gen-2 shape list (_debug.py:542-577)
SHAPES = [(2, 16, 1, 2048, 64), (1, 32, 1, 8192, 128), (1, 8, 4, 4096, 128), (1, 8, 1, 32768, 128),
          (8, 4, 1, 4096, 80), (4, 8, 2, 2048, 128), (2, 8, 4, 1024, 64), (1, 16, 1, 4096, 128), (1, 32, 1, 4096, 128)]


def _inputs(b, h, r, L, d, c=128):
    g = torch.Generator(device="cuda").manual_seed(7)
    k = torch.randn(b, h, L // c, c, d, device="cuda", generator=g)
    k = (k / k.norm(dim=-1, keepdim=True)).bfloat16()
    v = torch.randn(b, h, L // c, c, d, device="cuda", generator=g).bfloat16()
    q = torch.randn(b, h, r, L, d, device="cuda", generator=g).bfloat16()
    src = torch.sigmoid(torch.randn(b, h, L // c, c, device="cuda", generator=g)).bfloat16()
    dest = torch.sigmoid(torch.randn(b, h, L, device="cuda", generator=g)).bfloat16()
    return k, v, q, src, dest


def main(repeats=3):
    lib = _lib.load()
    lines = []
    for (b, h, r, L, d) in SHAPES:
        a = _inputs(b, h, r, L, d)
        votes = collections.defaultdict(collections.Counter)
        for _ in range(repeats):
            for slot, v in ops.autotune(*a).items():
                votes[slot][v] += 1
            for slot in votes:
                ops.tune_set(a[0], a[2], -1, slot)
        D = 64 if d <= 64 else 128
        lb = next(i for i in range(32) if (128 << i) >= L)
        zb = next(i for i in range(32) if (1 << i) >= b * h)
        for slot, cnt in sorted(votes.items()):
            v = cnt.most_common(1)[0][0]
            lines.append("  {%d, %d, %d, %d, %d, %d},   // %s  b=%d h=%d r=%d L=%d d=%d  votes %s"
                         % (_lib.TUNE_SLOTS[slot], D, r, lb, zb, v, slot, b, h, r, L, d, dict(cnt)))
            print(lines[-1], flush=True)
        del a
        torch.cuda.empty_cache()
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "ua_tune_defaults.inc")
    if os.environ.get("UA_TUNE_DEFAULTS_OUT"):
        out = os.environ["UA_TUNE_DEFAULTS_OUT"]
    with open(out, "w") as f:
        f.write("// {slot, padded head dim, r, L bucket (128 << b >= L), b*h bucket (1 << b >= b*h), variant}; bf16\n")
        f.write("// written by make_tune_defaults.py from ua_autotune runs on one MI355X\n")
        f.write("\n".join(lines) + "\n")
    print("wrote", out)


if __name__ == "__main__":
    main(int(sys.argv[1]) if len(sys.argv) > 1 else 3)
