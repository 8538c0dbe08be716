"""Headline benchmark: fused Universal Attention forward + backward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2] [--no-cpu] [--calibrate-copy]

A step is one forward + backward of the fused operator over one synthetic batch (inputs resident in HBM,
upstream gradient dO shaped like the output).  Prints ONE JSON line:
  value     algorithmic TFLOP/s of the whole step ((1+2r) + (3+5r)) * d * L^2 * b * h flops, causal pairs only
  roofline  the dominant kernel (k_bwd_keys: the six causal products it evaluates, G, S, dP, dV, dK(score side),
            dK(decay side) = (2+4r) d L^2 b h flops per launch) against the bf16 dense MFMA peak, its duration
            measured with hipEvents on the launch stream during the timed steps
  config.pruned_mode  the same step with the optional pruning of provably negligible pairs (never part of `value`)
  config.recompute_mode  the same step with UA_FLAG_RECOMPUTE: no per-pair tensor passes through HBM (never `value`)
  cpu_baseline  the oracle (a port of the reference's torch operator) timed on the host cores on a bounded sample:
            whole kv heads of the same workload, one after the other, until about 10 s have passed
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

CONFIGS = {  # BASELINE.json configs: b, h, r, L, d, chunk, dtype, gate_mean, passes
    0: dict(b=1, h=4, r=1, L=512, d=64, c=64, dtype="fp32", mu=0.0, bwd=False),
    1: dict(b=2, h=16, r=1, L=2048, d=64, c=128, dtype="bf16", mu=0.0, bwd=False),
    2: dict(b=1, h=32, r=1, L=8192, d=128, c=128, dtype="bf16", mu=0.0, bwd=True),
    3: dict(b=1, h=8, r=4, L=4096, d=128, c=128, dtype="bf16", mu=0.0, bwd=True),
    4: dict(b=1, h=8, r=1, L=32768, d=128, c=128, dtype="bf16", mu=2.0, bwd=True),
}
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}   # MI355X dense MFMA peaks


def flops(cfg):
    base = cfg["d"] * cfg["L"] ** 2 * cfg["b"] * cfg["h"]
    r = cfg["r"]
    return (1 + 2 * r) * base, (3 + 5 * r) * base


def kernel_flops(cfg, name):
    """Causal-pair flops of the products one launch of a fused-path kernel evaluates (2 d per pair and product)."""
    base = cfg["d"] * cfg["L"] ** 2 * cfg["b"] * cfg["h"]
    r = cfg["r"]
    return {"k_carry": 1, "k_fwd_fused": 2 * r, "k_bwd_keys": 2 + 4 * r, "k_bwd_queries": 5 * r}[name] * base


def hbm_kernels(cfg, kern):
    """Achieved GB/s of the kernels of the fused bf16 step whose algorithmic work is moving bytes: bytes they must read and
    write once (tile tensors of 1 KB tiles over the causal triangle, fp32 partial gradients, packed inputs) over their
    measured time, against the 8 TB/s of HBM3E."""
    if cfg["dtype"] != "bf16":
        return None
    Zk = cfg["b"] * cfg["h"]
    Zq = Zk * cfg["r"]
    L, d = cfg["L"], cfg["d"]
    Lp, D = -(-L // 128) * 128, 64 if d <= 64 else 128
    n32 = Lp // 32
    tri = (n32 * (n32 + 1) + 8) * 1024                     # bytes of one tile tensor per head
    split = cfg["r"] > 1 and Zk * (Lp // 128) <= 384       # separate key sweeps per query group
    Zs = Zq if split else Zk
    rows = lambda Z, width, esz: Z * Lp * width * esz
    bytes_of = {
        "k_carry": Zk * tri + rows(Zk, D, 2),
        "pack_inputs": (2 * Zk + Zq) * (L * d * 2 + 2 * Lp * D * 2),
    }
    if cfg["bwd"]:
        bytes_of.update({
            "k_bwd_queries": (Zq + Zs) * tri + rows(Zk, D, 2) + Zq * L * d * 2 + rows(Zq, D, 4),
            "k_bwd_finish": rows(2 * Zs + Zq, D, 4) + rows(Zk, D, 2) + 2 * Zk * L * d * 2,
            "pack_dO+delta": Zq * (2 * L * d * 2 + 2 * Lp * D * 2),
        })
    out = {}
    for k, nbytes in bytes_of.items():
        if k in kern and kern[k] > 0:
            gbs = nbytes / (kern[k] * 1e-3) / 1e9
            out[k] = {"GB": round(nbytes / 1e9, 3), "GB/s": round(gbs, 1), "frac_of_8TB/s": round(gbs / 8000.0, 3)}
    return out


def cpu_baseline(cfg, index, budget_s=10.0):
    """Oracle forward + backward (merge included) on whole kv heads of the workload, one at a time."""
    from oracle import ua_oracle as orc
    torch.set_num_threads(min(16, os.cpu_count() or 1))   # the GPU box grants 16 host cores per GPU
    dt = torch.bfloat16 if cfg["dtype"] == "bf16" else torch.float32
    names = ("kc", "vc", "xq", "static_src", "static_dest")
    heads, spent = 0, 0.0
    while heads < cfg["b"] * cfg["h"] and spent < budget_s:
        inp = orc.make_inputs(1, 1, cfg["r"], cfg["L"], cfg["d"], cfg["c"], dtype=dt, seed=1000 + index + heads,
                              gate_mean=cfg["mu"])
        t0 = time.time()
        out, denom = orc.chunked_forward(*[inp[k] for k in names])
        O = orc.merge(out, denom)
        if cfg["bwd"]:
            d_out, d_denom = orc.merge_backward(out, denom, inp["dO"])
            orc.chunked_backward(*[inp[k] for k in names], d_out, d_denom.float())
            del d_out, d_denom
        spent += time.time() - t0
        heads += 1
        del O, out, denom
    f, bw = flops(dict(cfg, b=1, h=1))
    if not cfg["bwd"]:
        bw = 0
    return {"value": round(heads * (f + bw) / spent / 1e12, 4), "unit": "TFLOP/s", "cores": torch.get_num_threads(),
            "kind": "port", "seconds": round(spent, 2), "ms_per_step_extrapolated": round(spent / heads * cfg["b"] * cfg["h"] * 1e3, 1),
            "sample": "%d of %d kv heads of the workload (each b=1,h=1,r=%d,L=%d,d=%d,chunk=%d): chunked forward + merge%s "
                      "of the oracle, heads run one after the other"
                      % (heads, cfg["b"] * cfg["h"], cfg["r"], cfg["L"], cfg["d"], cfg["c"], " + backward" if cfg["bwd"] else "")}


def parity_one_head(cfg, inp, O, grads, head=(0, 0)):
    """Largest relative error (Frobenius norm per tensor) of O and the five gradients of one (batch, kv head) against the
    oracle, the reference's chunked torch operator restated, evaluated in float32 on the same dtype-rounded inputs."""
    from oracle import ua_oracle as orc
    names = ("kc", "vc", "xq", "static_src", "static_dest")
    bi, hi = head
    one = [inp[k][bi:bi + 1, hi:hi + 1].float() for k in names]
    out, denom = orc.chunked_forward(*one)
    errs = {"O": float(((O[bi:bi + 1, hi:hi + 1].float().cpu() - orc.merge(out, denom)).norm() / orc.merge(out, denom).norm()))}
    if grads is not None:
        d_out, d_denom = orc.merge_backward(out, denom, inp["dO"][bi:bi + 1, hi:hi + 1].float())
        ref = orc.chunked_backward(*one, d_out, d_denom.float())
        for k, g, r in zip(names, grads, ref):
            g1 = g[bi:bi + 1, hi:hi + 1].float().cpu().reshape(r.shape)
            errs["d" + k] = float((g1 - r).norm() / r.norm())
    worst = max(errs, key=errs.get)
    return {"max_rel_err": round(errs[worst], 6), "tensor": worst, "head": list(head), "tolerance": 2e-2 if cfg["dtype"] == "bf16" else 1e-4,
            "against": "oracle (reference torch operator restated, float32) on the same inputs, one (batch, kv head)"}


# HBM bytes per launch of the roofline kernel, from the TCC counters FETCH_SIZE and WRITE_SIZE of two `rocprofv3 --pmc`
# runs of this script, each scaled by what the same counter reads for the plain 1 GiB copy of --calibrate-copy
# (profiles/counters_cfg2_keys_variants_cfg4_chunked.md, taken 2026-11-25; key: config, api, roofline kernel group).
# Config 2: 2.60 GB read (the fp16 bias tiles plus operand tiles) + 4.52 GB written (the dS / dG tiles k_bwd_queries3
# consumes) by k_bwd_keys2; config 4: 9.76 + 17.51 GB by k_bwd_keys4; the chunked call sequence at the config 2 shape:
# 2.88 + 4.89 GB by k_bwd_keys2.  The counters cannot be collected by a plain run of this script, so the figures are dated
# measurements; configurations without one report null.
MEASURED_TRAFFIC = {(2, "fused", "k_bwd_keys"): 7.11e9, (4, "fused", "k_bwd_keys"): 27.27e9, (2, "chunked", "k_bwd_keys"): 7.76e9}


def bench_sdpa(args, cfg):
    """Calibration, not the product: PyTorch's own scaled_dot_product_attention (plain causal attention, no decay bias)
    at the config's shape, forward and forward + backward, with each backend that runs here."""
    import torch.nn.functional as F
    b, h, L, d = cfg["b"], cfg["h"] * cfg["r"], cfg["L"], cfg["d"]
    dt = torch.bfloat16 if cfg["dtype"] == "bf16" else torch.float32
    q = torch.randn(b, h, L, d, device="cuda", dtype=dt, requires_grad=True)
    k = torch.randn_like(q, requires_grad=True)
    v = torch.randn_like(q, requires_grad=True)
    do = torch.randn_like(q)

    def timed(bwd, n=20):
        def run():
            o = F.scaled_dot_product_attention(q, k, v, is_causal=True)
            if bwd:
                torch.autograd.grad(o, [q, k, v], do)
        for _ in range(3):
            run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            run()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / n

    res = {"default backend": {"fwd_ms": round(timed(False), 4), "fwd_bwd_ms": round(timed(True), 4)}}
    try:
        from torch.nn.attention import SDPBackend, sdpa_kernel
        for name, be in (("flash", SDPBackend.FLASH_ATTENTION), ("memory-efficient", SDPBackend.EFFICIENT_ATTENTION)):
            try:
                with sdpa_kernel(be):
                    res[name] = {"fwd_ms": round(timed(False), 4), "fwd_bwd_ms": round(timed(True), 4)}
            except Exception as e:      # a backend that does not take this shape
                res[name] = {"error": str(e)[:80]}
    except ImportError:
        pass
    best = min(x["fwd_bwd_ms"] for x in res.values() if "fwd_bwd_ms" in x)
    print(json.dumps({"metric": "torch scaled_dot_product_attention, causal, no decay bias: fwd+bwd", "value": best, "unit": "ms",
                      "n_gpus": 1, "steps": 20, "warmup": 3, "ms_per_step": best, "higher_is_better": False, "scaling": "weak",
                      "vs_baseline": None, "dtype": cfg["dtype"], "data": "synthetic",
                      "config": {"workload": "plain causal attention at the shape of BASELINE config %d: b=%d heads=%d L=%d d=%d"
                                 % (args.config, b, h, L, d), "backends": res}}))


def bench_affinity(args, cfg, inp):
    """The stand-alone decay bias (AffinityScores: k, src, dest -> aff [b,h,L,L]) forward and backward at the config's
    key shape; both directions are bound by the L x L tensor they write or read."""
    from universal_attention_triton_amd import ops
    b, h, L, d = cfg["b"], cfg["h"], cfg["L"], cfg["d"]
    k = inp["kc"].reshape(b, h, L, d).cuda()
    src = inp["static_src"].reshape(b, h, L).cuda()
    dest = inp["static_dest"].reshape(b, h, L).cuda()
    esz = k.element_size()
    daff = torch.empty(b, h, L, L, dtype=k.dtype, device="cuda").normal_()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
    t_f = t_b = 0.0
    for i in range(args.warmup + args.steps):
        ev[0].record()
        aff = ops.affinity_forward(k, src, dest)
        ev[1].record()
        grads = ops.affinity_backward(k, src, dest, daff)
        ev[2].record()
        torch.cuda.synchronize()
        if i >= args.warmup:
            t_f += ev[0].elapsed_time(ev[1])
            t_b += ev[1].elapsed_time(ev[2])
        del aff, grads
    t_f /= args.steps
    t_b /= args.steps
    nbytes = b * h * L * L * esz
    gbs_f, gbs_b = nbytes / (t_f * 1e-3) / 1e9, nbytes / (t_b * 1e-3) / 1e9
    print(json.dumps({
        "metric": "stand-alone decay bias forward+backward", "value": round(t_f + t_b, 4), "unit": "ms", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(t_f + t_b, 4), "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": cfg["dtype"], "data": "synthetic",
        "config": {"workload": "AffinityScores forward+backward, keys of BASELINE config %d: b=%d h=%d L=%d d=%d"
                               % (args.config, b, h, L, d), "forward_ms": round(t_f, 4), "backward_ms": round(t_b, 4),
                   "backward_GB/s_of_daff": round(gbs_b, 1)},
        "roofline": {"bound": "hbm", "kernel": "k_aff_fwd", "achieved": round(gbs_f, 1), "peak": 8000.0, "unit": "GB/s",
                     "frac": round(gbs_f / 8000.0, 4), "traffic": None}}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default: enough for a timed region of about 1 s)")
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", type=int, default=2)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-parity", action="store_true", help="skip the one-head oracle check of the outputs and gradients")
    ap.add_argument("--chunk", type=int, default=None, help="--api chunked: keys per chunk (default: the config's, 128)")
    ap.add_argument("--api", choices=["fused", "chunked", "affinity", "sdpa"], default="fused",
                    help="fused (default): universal_attention(); chunked: the reference's call sequence "
                         "UniversalAttention.apply + SMVecMatMul.apply, which materialises out[b,h,r,L,d,n]")
    ap.add_argument("--no-pruned", action="store_true",
                    help="skip the extra timings of the optional modes (pruned, recomputing, less state kept for the "
                         "backward): keeps a profiler's per-kernel statistics to the launches `value` is made of")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 1 GiB device-to-device copy, the known-size kernel that HBM counters of a "
                         "profiler run are scaled against")
    ap.add_argument("--tune", action="append", default=[], metavar="SLOT=VARIANT",
                    help="run with this kernel variant instead of the table's choice (e.g. bwd_keys=1); never the default line")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (every (batch, kv head) is independent; nothing here uses a "
                 "second device). Re-run with --gpus 1.")
    from oracle import ua_oracle as orc
    from universal_attention_triton_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):            # only a tree without a built library builds it first
        from universal_attention_triton_amd import build as _build
        _build.build()
    from universal_attention_triton_amd.universal_attention import universal_attention

    cfg = dict(CONFIGS[args.config])
    if args.chunk:
        cfg["c"] = args.chunk
    if args.steps is None:      # about one second of timed steps
        args.steps = {0: 2000, 1: 2000, 2: 200, 3: 600, 4: 50}[args.config] if args.api == "fused" else 40
    dt = torch.bfloat16 if cfg["dtype"] == "bf16" else torch.float32
    inp = orc.make_inputs(cfg["b"], cfg["h"], cfg["r"], cfg["L"], cfg["d"], cfg["c"], dtype=dt, seed=1000 + args.config,
                          gate_mean=cfg["mu"])
    names = ("kc", "vc", "xq", "static_src", "static_dest")
    leaves = [inp[k].cuda().requires_grad_() for k in names]
    dO = inp["dO"].cuda()
    if args.tune:
        from universal_attention_triton_amd import ops as _ops
        for item in args.tune:
            slot, variant = item.split("=")
            _ops.tune_set(leaves[0].detach(), leaves[2].detach(), int(variant), slot)

    if args.api == "affinity":
        return bench_affinity(args, cfg, inp)
    if args.api == "sdpa":
        return bench_sdpa(args, cfg)
    if args.api == "chunked":
        import universal_attention_autograd as ref_api

        def step(prune=False):
            out_c, denom_c = ref_api.UniversalAttention.apply(*leaves)
            O = ref_api.SMVecMatMul.apply(out_c, denom_c)
            return torch.autograd.grad(O, leaves, dO) if cfg["bwd"] else O
    elif cfg["bwd"]:
        def step(prune=False, recompute=False):
            O = universal_attention(*leaves, prune=prune, recompute=recompute)
            return torch.autograd.grad(O, leaves, dO)
    else:
        def step(prune=False, recompute=False):
            with torch.no_grad():
                return universal_attention(*leaves, prune=prune, recompute=recompute)

    if args.calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").fill_(1.0)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    _lib.prof_collect()
    _lib.prof_enable(True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    _lib.prof_enable(False)
    prof = _lib.prof_collect()
    ms = elapsed * 1e3 / args.steps
    f_fwd, f_bwd = flops(cfg)
    if not cfg["bwd"]:
        f_bwd = 0
    dom = "k_bwd_keys" if cfg["bwd"] else "k_fwd_fused"
    if args.api == "chunked":
        dom = "k_fwd_chunked"
    kern = {k: round(v[1] / v[0], 4) for k, v in prof.items()}
    dom_ms = prof[dom][1] / prof[dom][0]
    peak = PEAK_TFLOPS[cfg["dtype"]]
    if args.api == "chunked":
        # the chunked forward is bound by writing out[b,h,r,L,d,n] and denom[b,h,r,L,n]
        n_chunks = cfg["L"] // cfg["c"]
        esz = 2 if cfg["dtype"] == "bf16" else 4
        out_bytes = cfg["b"] * cfg["h"] * cfg["r"] * cfg["L"] * n_chunks * (cfg["d"] + 1) * esz
        gbs = out_bytes / (dom_ms * 1e-3) / 1e9
        roof = {"bound": "hbm", "kernel": dom, "achieved": round(gbs, 1), "peak": 8000.0, "unit": "GB/s",
                "frac": round(gbs / 8000.0, 4), "traffic": None}
    achieved = kernel_flops(cfg, dom if args.api == "fused" else "k_fwd_fused") / (dom_ms * 1e-3) / 1e12
    out = {
        "metric": "fwd+bwd ms and TFLOP/s (bf16, L=8192, d=128) on 1 MI355X; % MFMA peak", "value": round((f_fwd + f_bwd) / (ms * 1e-3) / 1e12, 2),
        "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": cfg["dtype"], "data": "synthetic",
        "config": {"workload": "BASELINE config %d: fused %s b=%d h=%d r=%d L=%d d=%d%s"
                               % (args.config, "fwd+bwd" if cfg["bwd"] else "fwd only", cfg["b"], cfg["h"], cfg["r"], cfg["L"], cfg["d"],
                                  ", upstream dO like the output" if cfg["bwd"] else ""),
                   "pct_of_mfma_peak": round(100 * (f_fwd + f_bwd) / (ms * 1e-3) / 1e12 / peak, 2),
                   "kernel_ms": kern, **({"tune_override": args.tune} if args.tune else {})},
        "roofline": {"bound": "mfma", "kernel": dom, "achieved": round(achieved, 2), "peak": peak, "unit": "TFLOP/s",
                     "frac": round(achieved / peak, 4), "traffic": MEASURED_TRAFFIC.get((args.config, args.api, dom)) if not args.tune and not args.chunk else None},
    }
    if args.api == "fused":
        hk = hbm_kernels(cfg, kern)
        if hk:
            out["config"]["hbm_kernels"] = hk
        if cfg["bwd"]:
            from universal_attention_triton_amd import ops
            out["config"]["bytes_retained_fwd_to_bwd"] = {
                "forward_state": ops.retained_bytes(*[x.detach() for x in leaves]),
                "O_and_lse": leaves[2].numel() * leaves[2].element_size() + leaves[2].numel() // cfg["d"] * 4,
                "note": "the backward's scratch is allocated inside backward; keep_state=False retains O and lse only"}
            if not args.no_pruned:
                # the same step holding nothing between forward and backward (the backward rebuilds the state first)
                n_lean = max(3, args.steps // 4)
                for _ in range(2):
                    torch.autograd.grad(universal_attention(*leaves, keep_state=False), leaves, dO)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(n_lean):
                    torch.autograd.grad(universal_attention(*leaves, keep_state=False), leaves, dO)
                torch.cuda.synchronize()
                out["config"]["bytes_retained_fwd_to_bwd"]["keep_state_false_ms_per_step"] = round((time.perf_counter() - t0) * 1e3 / n_lean, 4)
    if not args.no_parity and args.api in ("fused", "chunked"):
        res = step()
        torch.cuda.synchronize()
        if cfg["bwd"]:
            with torch.no_grad():
                O_chk = universal_attention(*leaves)
            out["parity"] = parity_one_head(cfg, inp, O_chk, res)
        else:
            out["parity"] = parity_one_head(cfg, inp, res, None)
        del res
    if args.api == "chunked":
        out["roofline"] = roof
        out["config"]["workload"] += "; chunked API (reference call sequence, chunk %d)" % cfg["c"]
        out["config"].pop("pct_of_mfma_peak", None)
        # the same sequence with only the float32 normalisers kept for the backward instead of the whole forward state
        # (1/(d+1) of the size of `out`; the backward then repacks the inputs and repeats the decay pre-pass)
        from universal_attention_triton_amd import ops, universal_attention_autograd as own_api
        if not args.no_pruned:
            with own_api.chunked_options(keep_state="normalisers"):
                n_full = max(3, args.steps // 4)
                for _ in range(2):
                    step()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(n_full):
                    step()
                torch.cuda.synchronize()
                out["config"]["keep_state_normalisers"] = {"ms_per_step": round((time.perf_counter() - t0) * 1e3 / n_full, 4),
                                                           "note": "optional: only the normalisers retained for the backward; not `value`"}
        out["config"]["bytes_retained_fwd_to_bwd"] = {
            "forward_state": int(ops.retained_bytes(*[x.detach() for x in leaves], chunked=True)),
            "out_and_denom": int(cfg["b"] * cfg["h"] * cfg["r"] * cfg["L"] * (cfg["d"] + 1) * (cfg["L"] // cfg["c"])
                                 * (2 if cfg["dtype"] == "bf16" else 4))}
        if not args.no_cpu:
            out["cpu_baseline"] = cpu_baseline(cfg, args.config)
        print(json.dumps(out))
        return
    # the same step with UA_FLAG_PRUNE (pairs whose softmax weight is provably below 2^-48 are skipped): reported
    # beside the headline, never as `value`, because it executes fewer pairs than the flop count assumes
    if not args.no_pruned:
        for _ in range(2):
            step(prune=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step(prune=True)
        torch.cuda.synchronize()
        ms_p = (time.perf_counter() - t0) * 1e3 / args.steps
        out["config"]["pruned_mode"] = {"ms_per_step": round(ms_p, 4), "speedup": round(ms / ms_p, 2),
                                        "note": "optional exact pruning of negligible pairs; not counted in value"}
    # the same step with UA_FLAG_RECOMPUTE (bf16): every kernel evaluates the affinity chain and the score / decay
    # gradients itself, so that neither the bias nor the gradients of a (key, query) pair ever travel through HBM (only
    # one carry per key and 16 queries does); more vector work, a quarter of the workspace
    if not args.no_pruned and cfg["dtype"] == "bf16" and cfg["d"] <= 128:
        n_rc = max(3, args.steps // 4)
        for _ in range(2):
            step(recompute=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n_rc):
            step(recompute=True)
        torch.cuda.synchronize()
        ms_r = (time.perf_counter() - t0) * 1e3 / n_rc
        out["config"]["recompute_mode"] = {"ms_per_step": round(ms_r, 4), "tflops": round((f_fwd + f_bwd) / (ms_r * 1e-3) / 1e12, 2),
                                           "note": "optional: no per-pair tensor passes through HBM; not `value`"}
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(cfg, args.config)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
