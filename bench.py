"""Headline benchmark: fused Universal Attention forward + backward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2] [--no-cpu] [--calibrate-copy]

A step is one forward + backward of the fused operator over one synthetic batch (inputs resident in HBM,
upstream gradient dO shaped like the output).  Prints ONE JSON line:
  value     algorithmic TFLOP/s of the whole step ((1+2r) + (3+5r)) * d * L^2 * b * h flops, causal pairs only
  roofline  the dominant kernel (k_bwd_keys: the six causal products it evaluates, G, S, dP, dV, dK(score side),
            dK(decay side) = (2+4r) d L^2 b h flops per launch) against the bf16 dense MFMA peak, its duration
            measured with hipEvents on the launch stream during the timed steps
  config.pruned_mode  the same step with the optional pruning of provably negligible pairs (never part of `value`)
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


# HBM bytes per launch of the roofline kernel, from the TCC counters FETCH_SIZE and WRITE_SIZE of two `rocprofv3 --pmc`
# runs of this script, each scaled by what the same counter reads for the plain 1 GiB copy of --calibrate-copy
# (profiles/bench_cfg2_fused_fwd_bwd.md: 3.74 GB read + 4.58 GB written by k_bwd_keys2).  A measured constant, not
# collected by a default run; configurations without such a measurement report null.
MEASURED_TRAFFIC = {(2, "k_bwd_keys"): 8.32e9}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", type=int, default=2)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--api", choices=["fused", "chunked"], default="fused",
                    help="fused (default): universal_attention(); chunked: the reference's call sequence "
                         "UniversalAttention.apply + SMVecMatMul.apply, which materialises out[b,h,r,L,d,n]")
    ap.add_argument("--no-pruned", action="store_true",
                    help="skip the extra timing of the optional pruned mode (keeps a profiler's per-kernel statistics "
                         "to the launches `value` is made of)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 1 GiB device-to-device copy, the known-size kernel that HBM counters of a "
                         "profiler run are scaled against")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (every (batch, kv head) is independent; nothing here uses a "
                 "second device). Re-run with --gpus 1.")
    from oracle import ua_oracle as orc
    from universal_attention_triton_amd import _lib
    from universal_attention_triton_amd.universal_attention import universal_attention

    cfg = CONFIGS[args.config]
    dt = torch.bfloat16 if cfg["dtype"] == "bf16" else torch.float32
    inp = orc.make_inputs(cfg["b"], cfg["h"], cfg["r"], cfg["L"], cfg["d"], cfg["c"], dtype=dt, seed=1000 + args.config,
                          gate_mean=cfg["mu"])
    names = ("kc", "vc", "xq", "static_src", "static_dest")
    leaves = [inp[k].cuda().requires_grad_() for k in names]
    dO = inp["dO"].cuda()

    if args.api == "chunked":
        import universal_attention_autograd as ref_api

        def step(prune=False):
            out_c, denom_c = ref_api.UniversalAttention.apply(*leaves)
            O = ref_api.SMVecMatMul.apply(out_c, denom_c)
            return torch.autograd.grad(O, leaves, dO) if cfg["bwd"] else O
    elif cfg["bwd"]:
        def step(prune=False):
            O = universal_attention(*leaves, prune=prune)
            return torch.autograd.grad(O, leaves, dO)
    else:
        def step(prune=False):
            with torch.no_grad():
                return universal_attention(*leaves, prune=prune)

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
                   "kernel_ms": kern},
        "roofline": {"bound": "mfma", "kernel": dom, "achieved": round(achieved, 2), "peak": peak, "unit": "TFLOP/s",
                     "frac": round(achieved / peak, 4), "traffic": MEASURED_TRAFFIC.get((args.config, dom))},
    }
    if args.api == "chunked":
        out["roofline"] = roof
        out["config"]["workload"] += "; chunked API (reference call sequence, chunk %d)" % cfg["c"]
        out["config"].pop("pct_of_mfma_peak", None)
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
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(cfg, args.config)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
