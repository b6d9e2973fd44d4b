"""Benchmark of the MoE layer hot path on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W [--workload c2]

A step is one moe_forward over one batch of synthetic input already resident in
HBM.  Prints ONE JSON line: MoE-layer tokens/s, the roofline of the dominant
kernel (gate_up grouped GEMM, priced against the dense bf16 MFMA peak) from HIP
events recorded inside the timed steps, and the CPU baseline (the oracle's
restatement of the reference's CPU/OpenMP path) timed on this host on a bounded
prefix of the same batch.
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

# HBM bytes per gate_up launch at the c2 workload from rocprofv3 --pmc
# (FETCH_SIZE + WRITE_SIZE, scaled by the same counters on a copy kernel);
# None until measured for the workload being run.
MEASURED_TRAFFIC_BYTES = {"c2": 1.552e9}  # profiles/bench_c2_counters.md


def cpu_baseline(shape, L, budget_s=15.0):
    """Times the reference's CPU algorithm (per-token GEMV, OpenMP over output
    rows, float products accumulated in double; run.cpp:356-369, :662-745) on a
    prefix of the batch sized for about budget_s seconds."""
    from oracle import binding as ob
    w = [L[k] for k in ("w_router", "b_router", "w_mlp1", "b_mlp1", "w_mlp2", "b_mlp2")]
    x = L["x"]
    n0 = min(8, x.shape[0])
    t0 = time.perf_counter()
    ob.moe_layer(np.ascontiguousarray(x[:n0]), None, *w, shape.topk, shape.limit, mode=0)
    per_tok = (time.perf_counter() - t0) / n0
    n = int(max(16, min(x.shape[0], 2048, budget_s / max(per_tok, 1e-6))))
    t0 = time.perf_counter()
    ob.moe_layer(np.ascontiguousarray(x[:n]), None, *w, shape.topk, shape.limit, mode=0)
    dt = time.perf_counter() - t0
    return {"value": n / dt, "unit": "tokens/s", "cores": ob.num_threads(), "kind": "port",
            "sample": f"first {n} of {x.shape[0]} tokens, fp32 host weights, {dt:.1f} s"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c2", help="c2 (headline), c3a, c3b, c4")
    ap.add_argument("--no-cpu-baseline", action="store_true")
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
    L = synth.make_layer(shape, seed=0)
    moe = abi.Moe(H, IM, E, max_tokens=T, swiglu_limit=shape.limit)
    moe.upload_layer(0, *[L[k] for k in ("w_router", "b_router", "w_mlp1", "b_mlp1", "w_mlp2", "b_mlp2")])
    dx = abi.DevBuf.from_numpy(synth.to_bf16_bits(L["x"]))
    dout = abi.DevBuf(T * H * 4)

    for _ in range(args.warmup):
        moe.forward(0, dx, None, T, dout)
    abi.sync()
    n_prof = min(args.steps, 256)
    moe.profile_enable(n_prof)  # HIP events at the stage boundaries of the timed steps
    abi.sync()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        moe.forward(0, dx, None, T, dout)
    abi.sync()
    elapsed = time.perf_counter() - t0
    stages, n_meas = moe.profile_read()

    ms_per_step = elapsed / args.steps * 1e3
    tokens_per_s = T / (elapsed / args.steps)
    A = T * K
    flops_gate_up = 2.0 * A * H * 2 * IM
    flops_down = 2.0 * A * IM * H
    achieved = flops_gate_up / (stages["gate_up"] * 1e-3) / 1e12
    both = (flops_gate_up + flops_down) / ((stages["gate_up"] + stages["down"]) * 1e-3) / 1e12
    router_bytes = T * H * 2 + E * H * 2 + E * 2 + T * K * 8
    combine_bytes = A * H * 2 + T * H * 4
    result = {
        "metric": "MoE-layer tokens/sec",
        "value": tokens_per_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"{shape.name}: {T} tokens, hidden {H}, intermediate {IM}, "
                               f"{E} experts, top-{K}, bf16 weights, fp32 accumulate, seed 0"},
        "roofline": {"bound": "mfma", "kernel": "grouped_gemm_kernel<gate_up>",
                     "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_BF16_TFLOPS,
                     "traffic": MEASURED_TRAFFIC_BYTES.get(shape.name)},
        "expert_gemms": {"tflops": both, "frac_bf16_peak": both / PEAK_BF16_TFLOPS},
        "stage_us": {k: v * 1e3 for k, v in stages.items()},
        "router_gbs": router_bytes / (stages["router"] * 1e-3) / 1e9,
        "combine_gbs": combine_bytes / (stages["combine"] * 1e-3) / 1e9,
        "events_calls": n_meas,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(shape, L)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
