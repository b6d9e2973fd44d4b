"""Benchmark of the MoE layer hot path on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W [--workload c2]

A step is one moe_forward over one batch of synthetic input already resident in
HBM.  Prints ONE JSON line: MoE-layer tokens/s, the roofline of the dominant
kernel (gate_up grouped GEMM, priced against the dense bf16 MFMA peak) from HIP
events recorded inside the timed steps, and the CPU baseline (the oracle's
restatement of the reference's CPU/OpenMP path) timed on this host on a bounded
prefix of the same batch.  At the default workload the line also carries
"decode_mxfp4", a side figure for the decode-regime configuration (64 tokens,
MXFP4 expert weights) priced against the HBM peak; `--workload c5` makes that
configuration the one measured.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0
# What the box itself reaches with no algorithm in the way (second denominators,
# reported next to the published peaks): v_mfma_f32_32x32x16_bf16 from registers
# on all 256 CUs (profiles/mfma_register_rate.md) and a plain read stream over
# 2 GB (profiles/l2_ingest_ceiling.md).
SETTLE_STEPS = 200  # untimed calls in front of the warm-up steps, see run_leg
MEASURED_MFMA_TFLOPS = 1880.0
MEASURED_HBM_STREAM_GBS = 6150.0

# HBM bytes per gate_up launch at the c2 workload from rocprofv3 --pmc
# (FETCH_SIZE + WRITE_SIZE, scaled by the same counters on a copy kernel);
# None until measured for the workload being run.
MEASURED_TRAFFIC_BYTES = {"c2": 1.70e9, "c5": 0.290e9}  # profiles/bench_c2_counters.md, bench_c5_mxfp4_decode.md


def cpu_baseline(shape, L, budget_s=15.0):
    """Times the reference's CPU path (per-token GEMV, OpenMP over output rows,
    float products accumulated in double; run.cpp:356-369, :662-745) on a prefix
    of the batch sized for about budget_s seconds: the reference's own forward()
    compiled from its sources (oracle/_ref, kind "reference") where that library
    is there and loads, otherwise the oracle's restatement of it (kind "port")."""
    from oracle import binding as ob
    w = [L[k] for k in ("w_router", "b_router", "w_mlp1", "b_mlp1", "w_mlp2", "b_mlp2")]
    x = L["x"]

    def port(rows):
        ob.moe_layer(np.ascontiguousarray(x[:rows]), None, *w, shape.topk, shape.limit, mode=0)

    def reference(rows):
        # forward() normalises its input row itself (unit norm weight): feed rows
        # of the same scale; the work does not depend on the values
        ob.ref_moe_forward(np.ascontiguousarray(x[:rows]), *w, shape.topk, shape.limit)

    kind, run = "port", port
    if ob.ref_available():
        try:
            reference(1)
            kind, run = "reference", reference
        except Exception:  # the library does not load on this host: time the restatement
            pass
    n0 = min(8, x.shape[0])
    t0 = time.perf_counter()
    run(n0)
    per_tok = (time.perf_counter() - t0) / n0
    n = int(max(16, min(x.shape[0], 2048, budget_s / max(per_tok, 1e-6))))
    t0 = time.perf_counter()
    run(n)
    dt = time.perf_counter() - t0
    return {"value": n / dt, "unit": "tokens/s", "cores": ob.num_threads(), "kind": kind,
            "sample": f"first {n} of {x.shape[0]} tokens, fp32 host weights, {dt:.1f} s"}


def run_leg(shape, steps, warmup, device_timed=False):
    """Uploads the workload's layer, runs `warmup` + `steps` forwards and returns
    (seconds per step, stage times in ms from HIP events in the timed steps,
    calls measured, host-side layer or None).  Seconds per step are wall-clock
    time around the steps between two synchronisations; device_timed takes them
    from two HIP events around the steps enqueued by one library call instead (a
    step of 150 us is otherwise timed by the interpreter's call overhead)."""
    from gpt_oss_amd import abi, synth
    T, H, IM, E = shape.tokens, shape.hidden, shape.inter, shape.experts
    moe = abi.Moe(H, IM, E, max_tokens=T, swiglu_limit=shape.limit)
    if shape.name == "c5":  # MXFP4 expert weights, read as MXFP4 by the GEMMs
        L = None
        wr, br = synth.make_router(shape)
        b1k, s1, b1, b2k, s2, b2 = synth.make_experts_mxfp4(shape)
        moe.upload_layer_mxfp4(0, wr, br, b1k, s1, b1, b2k, s2, b2)
        x = synth.make_activations(shape)
    else:
        L = synth.make_layer(shape, seed=0)
        moe.upload_layer(0, *[L[k] for k in ("w_router", "b_router", "w_mlp1", "b_mlp1", "w_mlp2", "b_mlp2")])
        x = L["x"]
    dx = abi.DevBuf.from_numpy(synth.to_bf16_bits(x))
    dout = abi.DevBuf(T * H * 4)
    # The clocks of an idle GPU take a few hundred calls to settle: a fixed run-in
    # in front of the warm-up steps (reported as "settle_steps"), so that a short
    # run times the same state as a long one.
    for _ in range(SETTLE_STEPS + warmup):
        moe.forward(0, dx, None, T, dout)
    abi.sync()
    # HIP events at the stage boundaries of the last few timed steps: an event
    # between two kernels costs a few microseconds, so most steps run without.
    n_prof = min(16, max(1, steps // 4))
    moe.profile_enable(0)  # creates the events outside the timed region
    abi.sync()
    t0 = time.perf_counter()
    for i in range(steps):
        if i == steps - n_prof:
            moe.profile_enable(n_prof)
        moe.forward(0, dx, None, T, dout)
    abi.sync()
    elapsed = time.perf_counter() - t0
    stages, n_meas = moe.profile_read()
    if device_timed:
        elapsed = moe.time_forward(0, dx, None, T, dout, warmup, steps) * 1e-3
    moe.close()
    return elapsed / steps, stages, n_meas, L


def mxfp4_weight_bytes(shape):
    # nibbles + one scale byte per 32 weights
    return shape.experts * 3 * shape.hidden * shape.inter * (0.5 + 1.0 / 32)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="c2", help="c2 (headline), c3a, c3b, c4, c5 (MXFP4 decode)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-decode", action="store_true",
                    help="c2 only: skip the decode-regime side figure (workload c5)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)",
              file=sys.stderr)
        sys.exit(2)

    from gpt_oss_amd import abi, synth
    if abi.device_count() < 1:
        print("no GPU visible: the HIP path is required, there is no CPU fallback", file=sys.stderr)
        sys.exit(3)

    shape = synth.CONFIGS[args.workload]
    T, H, IM, E, K = shape.tokens, shape.hidden, shape.inter, shape.experts, shape.topk
    mxfp4 = shape.name == "c5"
    s_per_step, stages, n_meas, L = run_leg(shape, args.steps, args.warmup)

    A = T * K
    flops_gate_up = 2.0 * A * H * 2 * IM
    flops_down = 2.0 * A * IM * H
    both = (flops_gate_up + flops_down) / ((stages["gate_up"] + stages["down"]) * 1e-3) / 1e12
    router_bytes = T * H * 2 + E * H * 2 + E * 2 + T * K * 8
    combine_bytes = A * H * 2 + T * H * 4
    if mxfp4:
        # a stream of weights: gate_up reads two thirds of them
        achieved = mxfp4_weight_bytes(shape) * 2 / 3 / (stages["gate_up"] * 1e-3) / 1e9
        roofline = {"bound": "hbm", "kernel": "grouped_gemm_kernel<gate_up, MXFP4>",
                    "achieved": achieved, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "frac": achieved / PEAK_HBM_GBS, "traffic": MEASURED_TRAFFIC_BYTES.get(shape.name),
                    "measured_peak": MEASURED_HBM_STREAM_GBS,
                    "frac_of_measured_peak": achieved / MEASURED_HBM_STREAM_GBS}
    else:
        achieved = flops_gate_up / (stages["gate_up"] * 1e-3) / 1e12
        roofline = {"bound": "mfma", "kernel": "grouped_gemm_kernel<gate_up>",
                    "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                    "frac": achieved / PEAK_BF16_TFLOPS, "traffic": MEASURED_TRAFFIC_BYTES.get(shape.name),
                    "measured_peak": MEASURED_MFMA_TFLOPS,
                    "frac_of_measured_peak": achieved / MEASURED_MFMA_TFLOPS}
    weights = "MXFP4 expert weights" if mxfp4 else "bf16 weights"
    result = {
        "metric": "MoE-layer tokens/sec",
        "value": T / s_per_step,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_steps": SETTLE_STEPS,
        "ms_per_step": s_per_step * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"{shape.name}: {T} tokens, hidden {H}, intermediate {IM}, "
                               f"{E} experts, top-{K}, {weights}, fp32 accumulate, seed 0"},
        "roofline": roofline,
        "expert_gemms": {"tflops": both, "frac_bf16_peak": both / PEAK_BF16_TFLOPS},
        "stage_us": {k: v * 1e3 for k, v in stages.items()},
        "router_gbs": router_bytes / (stages["router"] * 1e-3) / 1e9,
        "combine_gbs": combine_bytes / (stages["combine"] * 1e-3) / 1e9,
        "events_calls": n_meas,
    }
    if shape.name == "c2" and not args.no_decode:
        # Side figure, not the headline value: the decode-regime configuration,
        # priced against the HBM peak on the weight bytes its GEMMs stream.
        c5 = synth.CONFIGS["c5"]
        s5, st5, _, _ = run_leg(c5, 200, 20, device_timed=True)
        wb = mxfp4_weight_bytes(c5)
        gemm_s = (st5["gate_up"] + st5["down"]) * 1e-3
        result["decode_mxfp4"] = {
            "workload": f"c5: {c5.tokens} tokens, {c5.experts} experts, MXFP4 expert weights",
            "tokens_per_s": c5.tokens / s5, "us_per_step": s5 * 1e6,
            "stage_us": {k: v * 1e3 for k, v in st5.items()},
            "weight_bytes": wb, "gemm_gbs": wb / gemm_s / 1e9,
            "gemm_frac_hbm_peak": wb / gemm_s / 1e9 / PEAK_HBM_GBS,
            "layer_gbs": wb / s5 / 1e9}
    if not args.no_cpu_baseline and L is not None:
        result["cpu_baseline"] = cpu_baseline(shape, L)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
