"""Benchmark of the single-GPU MoE MLP hot path on one MI355X.

A step is one forward + backward of ``FMoETransformerMLP`` over one batch of
synthetic tokens that is already resident in HBM.  The default workload is the
Mixtral-like layer the target is quoted on (32768 tokens, d_model 4096,
d_hidden 14336, 8 experts, top-2, bf16, GELU, fused pipeline with 4 chunks).

Prints ONE JSON line with the whole-job tokens/s, a ``roofline`` object for the
dominant kernel (timed with HIP events on the stream it is launched on, inside
this script) and a ``cpu_baseline`` object (the brute-force CPU oracle timed on a
bounded sample of the same workload on the host cores).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

CONFIGS = {
    # name: tokens, d_model, d_hidden, experts, top_k, dtype, fused, description
    "config1": dict(n=4096, d=512, h=1024, e=8, k=2, dtype="f32", fuse=False,
                    text="config1: 4096 tokens, d512/h1024, 8 experts top-2, fp32 GELU"),
    "config2": dict(n=16384, d=1024, h=4096, e=16, k=2, dtype="bf16", fuse=False, cap=2458,
                    text="config2: GShard top-2, 16384 tokens, d1024/h4096, 16 experts, capacity 2458/expert"),
    "config3": dict(n=16384, d=2048, h=8192, e=64, k=1, dtype="bf16", fuse=False, zipf=1.2,
                    text="config3: Switch top-1, 16384 tokens, d2048/h8192, 64 experts, Zipf(1.2) routing"),
    "config4": dict(n=32768, d=4096, h=14336, e=8, k=2, dtype="bf16", fuse=True,
                    text="config4: Mixtral-like, 32768 tokens, d4096/h14336, 8 experts top-2, bf16 GELU, "
                         "fused pipeline 4 chunks"),
    "config5": dict(n=8192, d=2048, h=1024, e=256, k=8, dtype="bf16", fuse=False, ebias=0.5,
                    text="config5: 8192 tokens, d2048/h1024, 256 experts top-8, biased logits"),
}

PEAK = {"bf16": 2500.0, "f32": 157.3}  # dense MFMA TFLOP/s, MI355X
# HBM-side bytes per launch of the grouped GEMM at config 4 (rocprofv3 FETCH_SIZE + WRITE_SIZE, each scaled by
# what the same counter reads for a copy kernel of known size: 1.984 and 1.000); measured offline, not in this
# script -- the counters need their own profiler runs.  Per class the mean over its launches of a step: forward
# (2.96 + 0.93 and 2.95 + 0.13 GB), data-grad (3.41 + 0.47 and 2.95 + 0.13 GB), weight-grad (17.65 + 0.94 GB, all rows).
TRAFFIC_BYTES = {"config4": {"gemm_fwd": 3.49e9, "gemm_dgrad": 3.48e9, "gemm_wgrad": 18.6e9}}
TRAFFIC_SOURCE = "profiles/grouped_gemm_bf16_config4_hbm_traffic.md (rocprofv3 --pmc runs, not this run)"
HBM_PEAK_GBS = 8000.0


def build_layer(cfg, device, gate_linear=False):
    import torch
    import fastermoe_amd as fmoe
    from fastermoe_amd.gates.base_gate import BaseGate
    from fastermoe_amd.functions import gate_topk
    from fastermoe_amd.gates.utils import limit_by_capacity

    dtype = torch.bfloat16 if cfg["dtype"] == "bf16" else torch.float32
    n, e, k = cfg["n"], cfg["e"], cfg["k"]
    gen = torch.Generator().manual_seed(42 + int(cfg["text"][6]))
    logits = torch.randn(n, e, generator=gen)
    if "ebias" in cfg:
        logits = logits + cfg["ebias"] * torch.randn(e, generator=gen)
    if "zipf" in cfg:
        p = torch.arange(1, e + 1, dtype=torch.float64) ** -cfg["zipf"]
        perm = torch.randperm(e, generator=gen)
        pick = perm[torch.multinomial(p / p.sum(), n, replacement=True, generator=gen)]
        logits = torch.full((n, e), -10.0).scatter_(1, pick.view(n, 1), 10.0)
    logits = logits.to(device)

    class SyntheticGate(BaseGate):
        """Top-k over fixed seeded logits, scores = softmax over the selected logits
        (unit score for top-1); optional per-expert capacity through the capacity kernels."""

        def __init__(self, d_model, num_expert, world_size, top_k=2):
            super().__init__(num_expert, world_size)
            self.top_k = top_k

        def forward(self, inp):
            idx, score = gate_topk(logits, self.top_k, score_mode=1)
            score = score.to(inp.dtype)
            if "cap" in cfg:
                _, _, idx = limit_by_capacity(idx, self.num_expert, 1, cfg["cap"])
            return idx, score

    class LinearSoftmaxGate(fmoe.gates.NaiveGate):
        """The real thing: ``nn.Linear(d_model, experts)`` inside the step, top-k of its logits and the
        softmax over the selected ones as scores (NaiveGate with normalised scores)."""

        def forward(self, inp):
            idx, score = gate_topk(self.gate(inp), self.top_k, score_mode=1)
            return idx, score

    layer = fmoe.FMoETransformerMLP(num_expert=e, d_model=cfg["d"], d_hidden=cfg["h"], top_k=k,
                                    gate=LinearSoftmaxGate if gate_linear else SyntheticGate,
                                    activation=torch.nn.GELU())
    layer.enable_fuse = cfg["fuse"]
    layer = layer.to(dtype).to(device)
    gen2 = torch.Generator().manual_seed(7)
    x = torch.randn(n, cfg["d"], generator=gen2).to(dtype).to(device).requires_grad_(True)
    grad = torch.randn(n, cfg["d"], generator=gen2).to(dtype).to(device)
    return layer, x, grad


def step(layer, x, grad):
    layer.zero_grad(set_to_none=True)
    x.grad = None
    out = layer(x)
    out.backward(grad)


def gemm_algorithmic_bytes(cfg, rows, experts_used):
    """Bytes the six grouped products of a step must move at least: every operand read once, every
    result written once.  Per linear (in, out): forward reads rows*in + E'*in*out and writes rows*out,
    data-grad reads rows*out + E'*in*out and writes rows*in, weight-grad reads rows*(in + out) and
    writes E*in*out (E' = experts that have rows)."""
    e_bytes = 2 if cfg["dtype"] == "bf16" else 4
    d, h = cfg["d"], cfg["h"]
    per_linear = 3 * rows * (d + h) + (2 * experts_used + cfg["e"]) * d * h
    return 2 * per_linear * e_bytes


def time_steps(layer, x, grad, steps, warmup):
    """`warmup` untimed steps, then exactly `steps` timed ones between two device synchronisations
    (host clock), every step also bracketed by HIP events on the current stream (the fused pipeline
    forks from and joins to it).  Returns (mean ms per step by the host clock, median and mean ms per
    step by the events)."""
    import torch
    for _ in range(warmup):
        step(layer, x, grad)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for a, b in ev:
        a.record()
        step(layer, x, grad)
        b.record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    per = sorted(a.elapsed_time(b) for a, b in ev)
    return elapsed / steps * 1e3, per[len(per) // 2], sum(per) / len(per)


def measure(cfg, name, device, steps, warmup, profile_steps, permutes_alone):
    """Times `steps` forward + backward steps of the layer of `cfg` (after `warmup`), then `profile_steps`
    more with the library's per-launch HIP-event brackets switched on."""
    import torch
    from fastermoe_amd import _lib, fmoe_native
    layer, x, grad = build_layer(cfg, device)
    ms_per_step, ms_median, ms_event_mean = time_steps(layer, x, grad, steps, warmup)
    tokens_per_s = cfg["n"] / (ms_per_step * 1e-3)

    # per-kernel timing: HIP events recorded by the library on the stream each kernel runs on
    _lib.profile_enable(True)
    _lib.profile_collect()
    for _ in range(profile_steps):
        step(layer, x, grad)
    prof = _lib.profile_collect()
    _lib.profile_enable(False)

    # rows that were routed (the layer itself never reads this number on the host)
    n, k, d = cfg["n"], cfg["k"], cfg["d"]
    with torch.no_grad():
        idx, _ = layer.gate(x)
        cnt, pos_buf, s2r = fmoe_native.route(idx.contiguous(), cfg["e"])
        cnt_cpu = cnt.cpu()
        rows, used = int(cnt_cpu.sum()), int((cnt_cpu > 0).sum())
    # flop per step of every GEMM class: two products of 2 * rows * d * h each (forward: both linears; data
    # gradient: both; weight gradient: both) -- 12 * rows * d * h per step in all
    class_flop = 4.0 * rows * cfg["d"] * cfg["h"]

    kernels = {}
    for kname, (launches, ms, work) in prof.items():
        if launches == 0:
            continue
        is_gemm = kname.startswith("gemm")
        if is_gemm:
            work = class_flop * profile_steps
        rate = work / (ms * 1e-3) / (1e12 if is_gemm else 1e9)
        kernels[kname] = {"launches_per_step": launches / profile_steps,
                          "avg_ms": round(ms / launches, 4), "ms_per_step": round(ms / profile_steps, 4),
                          "work_per_launch": work / launches,
                          "achieved": round(rate, 2), "unit": "TFLOP/s" if is_gemm else "GB/s"}
    gemm_names = [k for k in kernels if k.startswith("gemm")]
    peak = PEAK[cfg["dtype"]]
    gemm_ms = sum(kernels[k]["ms_per_step"] for k in gemm_names)
    gemm_flop = sum(kernels[k]["work_per_launch"] * kernels[k]["launches_per_step"] for k in gemm_names)

    gemm_bytes = gemm_algorithmic_bytes(cfg, rows, used)
    mfma_frac = gemm_flop / (gemm_ms * 1e-3) / 1e12 / peak
    hbm_frac = gemm_bytes / (gemm_ms * 1e-3) / 1e9 / HBM_PEAK_GBS
    gemm_all = {"tflops": round(gemm_flop / (gemm_ms * 1e-3) / 1e12, 2), "frac_of_mfma_peak": round(mfma_frac, 4),
                "algorithmic_gbytes_per_step": round(gemm_bytes / 1e9, 3),
                "frac_of_hbm_peak": round(hbm_frac, 4), "bound": "mfma" if mfma_frac >= hbm_frac else "hbm",
                "ms_per_step": round(gemm_ms, 3)}

    # the roof of the GEMM class with the most time per step: the nearer of the two
    dominant = max(gemm_names, key=lambda kk: kernels[kk]["ms_per_step"])
    dk = kernels[dominant]
    dom_frac_mfma = dk["achieved"] / peak
    # bytes per launch of the dominant class: its share of the step's algorithmic bytes by product
    e_bytes = 2 if cfg["dtype"] == "bf16" else 4
    per = {"gemm_fwd": 2 * (rows * (cfg["d"] + cfg["h"]) + used * cfg["d"] * cfg["h"]),
           "gemm_dgrad": 2 * (rows * (cfg["d"] + cfg["h"]) + used * cfg["d"] * cfg["h"]),
           "gemm_wgrad": 2 * (rows * (cfg["d"] + cfg["h"]) + cfg["e"] * cfg["d"] * cfg["h"])}
    dom_bytes_per_launch = per[dominant] * e_bytes / dk["launches_per_step"]
    dom_frac_hbm = dom_bytes_per_launch / (dk["avg_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS
    if dom_frac_mfma >= dom_frac_hbm:
        roofline = {"kernel": "grouped_gemm_kernel (" + dominant + ")", "bound": "mfma",
                    "achieved": round(dk["achieved"], 2), "peak": peak, "unit": "TFLOP/s",
                    "frac": round(dom_frac_mfma, 4), "flop_per_launch": dk["work_per_launch"],
                    "avg_launch_ms": dk["avg_ms"], "frac_of_hbm_peak": round(dom_frac_hbm, 4)}
    else:
        roofline = {"kernel": "grouped_gemm_kernel (" + dominant + ")", "bound": "hbm",
                    "achieved": round(dom_bytes_per_launch / (dk["avg_ms"] * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS,
                    "unit": "GB/s", "frac": round(dom_frac_hbm, 4), "bytes_per_launch": dom_bytes_per_launch,
                    "avg_launch_ms": dk["avg_ms"], "frac_of_mfma_peak": round(dom_frac_mfma, 4)}
    roofline["traffic"] = TRAFFIC_BYTES.get(name, {}).get(dominant) if cfg["fuse"] else None
    if roofline["traffic"] is not None:
        roofline["traffic_source"] = TRAFFIC_SOURCE

    permute_alone = None
    if permutes_alone:
        # the row permutes alone (inside the fused pipeline they share the chip with the GEMMs)
        with torch.no_grad():
            pos = pos_buf[:rows]
            tok = pos // k
            _lib.profile_enable(True)
            _lib.profile_collect()
            for _ in range(10):
                buf = fmoe_native.gather_rows(x.detach(), tok)            # local scatter
                fmoe_native.gather_rows(buf, s2r, n * k)                   # local gather (copy)
            gather_alone = _lib.profile_collect()["gather_rows"]
            for _ in range(10):
                fmoe_native.reduce_slots(buf, s2r, n, k)                   # backward of the scatter
            reduce_alone = _lib.profile_collect()["reduce_slots"]
            _lib.profile_enable(False)
        permute_alone = {
            "gather_rows": {"GB/s": round(gather_alone[2] / gather_alone[1] / 1e6, 1),
                            "frac_of_hbm_peak": round(gather_alone[2] / gather_alone[1] / 1e6 / HBM_PEAK_GBS, 4)},
            "reduce_slots": {"GB/s": round(reduce_alone[2] / reduce_alone[1] / 1e6, 1),
                             "frac_of_hbm_peak": round(reduce_alone[2] / reduce_alone[1] / 1e6 / HBM_PEAK_GBS, 4)},
        }
        del buf
    del layer, x, grad
    torch.cuda.empty_cache()
    return {"ms_per_step": round(ms_per_step, 3), "ms_per_step_median": round(ms_median, 3),
            "ms_per_step_event_mean": round(ms_event_mean, 3), "routed_rows": rows,
            "tokens_per_s": round(tokens_per_s, 1), "kernels": kernels,
            "gemm_all": gemm_all, "roofline": roofline, "permute_alone": permute_alone}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="config4", choices=sorted(CONFIGS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", dest="other_configs", action="store_false",
                    help="skip the short runs of configurations 1, 2, 3 and 5 that follow the headline workload")
    ap.add_argument("--profile-steps", type=lambda v: max(1, int(v)), default=3,
                    help="steps run with the library's per-launch HIP-event brackets after the timed ones (at least 1)")
    ap.add_argument("--no-gate-linear", dest="gate_linear", action="store_false",
                    help="skip the second figure with the gate's linear layer inside the step")
    ap.add_argument("--fuse", choices=["auto", "on", "off"], default="auto",
                    help="override the configuration's choice of the fused pipeline")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run only a plain row-copy kernel of known size (1 GiB read + 1 GiB written per launch); "
                         "used to scale rocprofv3's FETCH_SIZE / WRITE_SIZE counters")
    ap.add_argument("--reference-gemm", action="store_true",
                    help="time one expert's forward GEMM of the workload (rows/experts x d_model x d_hidden) with the "
                         "grouped kernel and with the vendor library (torch.nn.functional.linear), on N(0,1) and on "
                         "all-zero operands; shows how much of the datasheet peak the power envelope leaves")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures the single-GPU MoE path only; run with --gpus 1 "
                 "(multi-GPU expert parallelism is not part of it)")

    import torch
    from fastermoe_amd import _lib

    if args.config == "config4":
        os.environ.setdefault("FMOE_FUSE_GRAN", "4")  # the headline configuration is quoted on 4 chunks
    cfg = dict(CONFIGS[args.config])
    if args.fuse != "auto":
        cfg["fuse"] = args.fuse == "on"
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    device = torch.device("cuda:0")
    _lib.load()
    if args.copy_calibration:
        from fastermoe_amd import fmoe_native
        rows, width = 131072, 4096  # bf16: 1 GiB in, 1 GiB out
        src = torch.randn(rows, width, device=device).to(torch.bfloat16)
        ident = torch.arange(rows, dtype=torch.int64, device=device)
        for _ in range(5):
            fmoe_native.gather_rows(src, ident)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "gather_rows_vec_kernel", "bytes_read": rows * width * 2,
                          "bytes_written": rows * width * 2, "launches": 5}))
        return
    if args.reference_gemm:
        from fastermoe_amd import fmoe_native
        dtype = torch.bfloat16 if cfg["dtype"] == "bf16" else torch.float32
        rows = cfg["n"] * cfg["k"] // cfg["e"]
        cnt = torch.tensor([rows], dtype=torch.int64)

        def timed(fn, iters=10):
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(iters):
                fn()
            b.record()
            torch.cuda.synchronize()
            return a.elapsed_time(b) / iters

        out = {"shape": [rows, cfg["d"], cfg["h"]], "dtype": cfg["dtype"], "unit": "TFLOP/s"}
        flop = 2.0 * rows * cfg["d"] * cfg["h"]
        for name in ("normal", "zeros"):
            xx = torch.randn(rows, cfg["d"], device=device).to(dtype)
            ww = torch.randn(1, cfg["h"], cfg["d"], device=device).to(dtype)
            if name == "zeros":
                xx.zero_()
                ww.zero_()
            out["grouped_kernel_" + name] = round(flop / timed(lambda: fmoe_native.linear_forward(xx, cnt, ww, None)) / 1e9, 1)
            out["vendor_library_" + name] = round(flop / timed(lambda: torch.nn.functional.linear(xx, ww[0])) / 1e9, 1)
        print(json.dumps(out))
        return
    m = measure(cfg, args.config, device, args.steps, args.warmup, args.profile_steps, permutes_alone=True)

    result = {
        "metric": "moe_mlp_fwd_bwd_tokens_per_s", "value": m["tokens_per_s"], "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": m["ms_per_step"],
        "ms_per_step_median_hip_events": m["ms_per_step_median"], "ms_per_step_mean_hip_events": m["ms_per_step_event_mean"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": cfg["dtype"],
        "data": "synthetic",
        "config": {"workload": cfg["text"], "tokens": cfg["n"], "d_model": cfg["d"], "d_hidden": cfg["h"],
                   "experts": cfg["e"], "top_k": cfg["k"], "fused": cfg["fuse"],
                   "chunks": (int(os.environ["FMOE_FUSE_GRAN"]) if "FMOE_FUSE_GRAN" in os.environ else "chosen by the library")
                   if cfg["fuse"] else 1,
                   "routed_rows": m["routed_rows"],
                   "gate": "top-k over fixed seeded logits; the gate's own linear layer is not part of the step "
                           "(with_gate_linear: the same layer with nn.Linear(d_model, experts) inside the step)"},
        "roofline": m["roofline"],
        "gemm_all": m["gemm_all"],
        "kernels": m["kernels"],
        "permute_alone": m["permute_alone"],
        "hbm_peak_gbs": HBM_PEAK_GBS,
    }

    if args.gate_linear:
        # the same workload with the gate's own linear layer inside the step
        layer, x, grad = build_layer(cfg, device, gate_linear=True)
        ms, med, _ = time_steps(layer, x, grad, max(5, args.steps // 2), 3)
        result["with_gate_linear"] = {"ms_per_step": round(ms, 3), "ms_per_step_median_hip_events": round(med, 3),
                                      "tokens_per_s": round(cfg["n"] / (ms * 1e-3), 1),
                                      "gate": "nn.Linear(d_model, experts) + top-k + softmax over the selected logits"}
        del layer, x, grad
        torch.cuda.empty_cache()

    if args.other_configs and args.config == "config4":
        # the other workloads (parity-test configurations), 5 warm-up + 20 timed steps each
        others = {}
        for name in ("config1", "config2", "config3", "config5"):
            o = measure(dict(CONFIGS[name]), name, device, 20, 5, 3, permutes_alone=False)
            others[name] = {"workload": CONFIGS[name]["text"], "dtype": CONFIGS[name]["dtype"],
                            "ms_per_step": o["ms_per_step"], "ms_per_step_median_hip_events": o["ms_per_step_median"],
                            "routed_rows": o["routed_rows"], "tokens_per_s": o["tokens_per_s"],
                            "gemm_ms_per_step": o["gemm_all"]["ms_per_step"],
                            "gemm_frac_of_mfma_peak": o["gemm_all"]["frac_of_mfma_peak"],
                            "gemm_frac_of_hbm_peak": o["gemm_all"]["frac_of_hbm_peak"],
                            "bound": o["gemm_all"]["bound"],
                            "kernels_ms_per_step": {k: v["ms_per_step"] for k, v in o["kernels"].items()}}
        result["other_configs"] = others

    if not args.no_cpu_baseline:
        from oracle import moe as omoe
        sample = {"config1": cfg["n"], "config4": 4096}.get(args.config, 4096)
        sample = min(sample, cfg["n"])
        tps, cores, best, median = omoe.time_cpu_baseline(sample, cfg["d"], cfg["h"], cfg["e"], cfg["k"], "gelu",
                                                          seed=1, repeats=3, threads=min(os.cpu_count() or 1, 16),
                                                          warmup=1, return_median=True)
        result["cpu_baseline"] = {"value": round(tps, 1), "unit": "tokens/s", "cores": cores, "kind": "port",
                                  "median_value": round(sample / median, 1),
                                  "sample": f"{sample} of {cfg['n']} tokens, same d_model/d_hidden/experts/top_k, "
                                            f"fp32, fwd+bwd, 1 warm-up + 3 timed iterations, best {best:.1f} s, "
                                            f"median {median:.1f} s (value = best)"}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
