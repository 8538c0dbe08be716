"""Builds libua_hip.so (gfx950) from csrc/ with hipcc.  `python -m universal_attention_triton_amd.build`."""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libua_hip.so")
UNITS = ["ua_capi", "ua_inst_fwd", "ua_inst_bwd", "ua_inst_bwd4", "ua_inst_aff"]
# packed-fp32 instructions are disabled for every device compile of this library
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-honor-nans", "-Wall", "-Wno-unused-function", "-Wno-unused-variable", "-Wno-unused-but-set-variable", "-Wno-unused-local-typedef", "-Wno-unused-value", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def source_hash():
    """Hash of everything the library is compiled from; the library reports the hash it was built with
    (ua_source_hash) and _lib.load refuses a library whose sources have changed since."""
    import hashlib
    h = hashlib.sha256()
    files = sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hip", ".hpp", ".inc")))
    files.append(os.path.join(HERE, "..", "include", "ua.h"))
    for f in files:
        h.update(os.path.basename(f).encode())
        with open(f, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def _compile(unit, objdir, extra):
    src, obj = os.path.join(CSRC, unit + ".hip"), os.path.join(objdir, unit + ".o")
    cmd = ["hipcc", *FLAGS, *extra, "-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    log = "\n".join(l for l in res.stderr.splitlines() if "not a recognized feature" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (unit, log))
    return obj, log


def build(verbose=False, extra=()):
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    tag = ['-DUA_SOURCE_HASH="%s"' % source_hash()]
    with concurrent.futures.ThreadPoolExecutor(max_workers=len(UNITS)) as ex:
        results = list(ex.map(lambda u: _compile(u, objdir, list(extra) + (tag if u == "ua_capi" else [])), UNITS))
    objs = [o for o, _ in results]
    res = subprocess.run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs], capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stderr)
    for _, log in results:      # compiler warnings are always shown: an uninitialised pointer on the host side faults the GPU
        if log.strip() and (verbose or "warning:" in log):
            print(log)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
