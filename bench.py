"""Benchmark of the MoE layer hot path on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W [--workload c2]

A step is one moe_forward over one batch of synthetic input already resident in
HBM.  Prints ONE JSON line: MoE-layer tokens/s, the roofline of the dominant
kernel (the gate_up grouped GEMM) priced against whichever of the dense bf16
MFMA peak and the HBM peak binds the workload, from HIP events recorded inside
the timed steps, and the CPU baseline (the reference's CPU/OpenMP path) timed on
this host on a bounded prefix of the same batch.  At the default workload the
line also carries "decode_mxfp4", a side figure for the decode-regime
configuration (64 tokens, MXFP4 expert weights; `--workload c5` makes that
configuration the one measured), "prefill_mxfp4", the headline batch with
MXFP4 expert weights, and "other_workloads", short legs of the remaining
benchmark configurations (c3a, c3b, c4), and "zero_weights_yardstick", the
headline workload once more with all-zero expert matrices (the same kernels at
the clock the GPU holds when their operands do not toggle).  None of them is
part of `value`.
"""
from __future__ import annotations

import argparse
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0
SETTLE_STEPS = 200  # untimed calls in front of the warm-up steps, see run_leg
# which roofline binds the gate_up GEMM of a workload: rows per expert
# (4 T / E) against the machine balance of 312 flop per byte
BOUND = {"c2": "mfma", "c3a": "hbm", "c3b": "mfma", "c4": "hbm", "c5": "hbm", "d4": "mfma"}


def cpu_model() -> str:
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def measured_traffic(workload: str):
    """HBM bytes per gate_up launch from the rocprofv3 --pmc summary of this
    workload under profiles/ (FETCH_SIZE + WRITE_SIZE, scaled by the same
    counters on a copy of known size), or None where no such summary exists.
    Read at run time so that the figure is the profile's, never a constant here."""
    path = os.path.join(ROOT, "profiles", f"bench_{workload}_counters.md")
    try:
        m = re.search(r"gate_up traffic bytes per launch:\s*([0-9.eE+]+)", open(path).read())
        return float(m.group(1)) if m else None
    except OSError:
        return None


def cpu_baseline(shape, L, budget_s=12.0):
    """Times the reference's CPU path (per-token GEMV, OpenMP over output rows,
    float products accumulated in double; run.cpp:356-369, :662-745) on a prefix
    of the batch sized for about budget_s seconds.  kind "reference": the
    reference's own forward() compiled from its sources (oracle/_ref: -O3
    -fopenmp, built where the sources are, hence without -march=native).  The
    restatement of the same path, compiled on this host with the reference's
    flags (-O3 -fopenmp -march=native), is timed next to it ("port_value").
    Where oracle/_ref is missing the restatement is the baseline (kind "port")."""
    from oracle import binding as ob
    w = [L[k] for k in ("w_router", "b_router", "w_mlp1", "b_mlp1", "w_mlp2", "b_mlp2")]
    x = L["x"]
    flags_port = "-O3 -fopenmp -march=native, built on this host"
    try:
        native = ob.lib_native()
    except Exception as e:  # no compiler or make on this host: the portable build that came along
        print(f"oracle: native build failed ({e}); timing the portable build", file=sys.stderr)
        native = None
        flags_port = "-O2 -fopenmp (portable build; the native build failed on this host)"

    def port(rows):
        ob.moe_layer(np.ascontiguousarray(x[:rows]), None, *w, shape.topk, shape.limit, mode=0, use_lib=native)

    def reference(rows):
        # forward() normalises its input row itself (unit norm weight): feed rows
        # of the same scale; the work does not depend on the values
        ob.ref_moe_forward(np.ascontiguousarray(x[:rows]), *w, shape.topk, shape.limit)

    def timed(run, share):
        n0 = min(8, x.shape[0])
        t0 = time.perf_counter()
        run(n0)
        per_tok = (time.perf_counter() - t0) / n0
        n = int(max(16, min(x.shape[0], 2048, share / max(per_tok, 1e-6))))
        t0 = time.perf_counter()
        run(n)
        dt = time.perf_counter() - t0
        return n / dt, n, dt

    have_ref = False
    if ob.ref_available():
        try:
            reference(1)
            have_ref = True
        except Exception as e:  # the library does not load on this host
            print(f"oracle/_ref does not load here ({e}); timing the restatement", file=sys.stderr)
    pv, pn, pdt = timed(port, budget_s * (0.4 if have_ref else 1.0))
    out = {"unit": "tokens/s", "cores": ob.num_threads(), "cpu": cpu_model()}
    if have_ref:
        rv, rn, rdt = timed(reference, budget_s * 0.6)
        out.update({"value": rv, "kind": "reference",
                    "sample": f"first {rn} of {x.shape[0]} tokens, fp32 host weights, {rdt:.1f} s",
                    "flags": "-O3 -fopenmp (reference sources; built off this host, so without -march=native)",
                    "port_value": pv,
                    "port_sample": f"first {pn} tokens, {pdt:.1f} s; {flags_port}"})
    else:
        out.update({"value": pv, "kind": "port",
                    "sample": f"first {pn} of {x.shape[0]} tokens, fp32 host weights, {pdt:.1f} s",
                    "flags": flags_port})
    return out


def run_leg(shape, steps, warmup, device_timed=False, mxfp4=None, zero_expert_weights=False, layer=None):
    """Uploads the workload's layer, runs `warmup` + `steps` forwards and returns
    (seconds per step, stage times in ms from HIP events in the timed steps,
    calls measured, median seconds per step, host-side layer or None).  Seconds
    per step are wall-clock time around the steps between two synchronisations;
    device_timed takes them from two HIP events around the steps enqueued by one
    library call instead (a step of 150 us is otherwise timed by the
    interpreter's call overhead).  The median is over per-step HIP-event
    intervals of a further run of max(steps, 50) steps.  zero_expert_weights: a
    yardstick, not a workload -- the expert matrices and biases are uploaded as
    zeros (router, routing, tile plan, instructions and memory traffic are those
    of the workload; what changes is how many bits toggle in the matrix cores).
    layer: a host-side layer of this shape to use instead of generating one (it
    is zeroed in place when zero_expert_weights is set)."""
    from gpt_oss_amd import abi, synth
    T, H, IM, E = shape.tokens, shape.hidden, shape.inter, shape.experts
    moe = abi.Moe(H, IM, E, max_tokens=T, swiglu_limit=shape.limit)
    if mxfp4 is None:
        mxfp4 = shape.name == "c5"
    if mxfp4:  # MXFP4 expert weights, read as MXFP4 by the GEMMs
        L = None
        wr, br = synth.make_router(shape)
        b1k, s1, b1, b2k, s2, b2 = synth.make_experts_mxfp4(shape)
        moe.upload_layer_mxfp4(0, wr, br, b1k, s1, b1, b2k, s2, b2)
        x = synth.make_activations(shape)
    else:
        L = layer if layer is not None else synth.make_layer(shape, seed=0)
        if zero_expert_weights:
            for k in ("w_mlp1", "b_mlp1", "w_mlp2", "b_mlp2"):
                L[k][...] = 0
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
    each = moe.time_forward_each(0, dx, None, T, dout, max(steps, 50))
    moe.close()
    return elapsed / steps, stages, n_meas, float(np.median(each)) * 1e-3, L


def side_leg(name, steps=60, warmup=10):
    """One of the other benchmark configurations as a side figure of the default
    line: tokens/s, stage times and the gate_up GEMM against the roofline that
    binds it (published peaks), measured like the headline workload."""
    shape = synth_configs()[name]
    T, H, IM, E, K = shape.tokens, shape.hidden, shape.inter, shape.experts, shape.topk
    s_step, st, _, med, _ = run_leg(shape, steps, warmup)
    A = T * K
    t_gu, t_dn = st["gate_up"] * 1e-3, st["down"] * 1e-3
    fl_gu, fl_dn = 2.0 * A * H * 2 * IM, 2.0 * A * IM * H
    by_gu = E * 2 * IM * H * 2.0 + A * H * 2 + A * IM * 2
    by_dn = E * H * IM * 2.0 + A * IM * 2 + A * H * 4
    bound = BOUND[name]
    ach = fl_gu / t_gu / 1e12 if bound == "mfma" else by_gu / t_gu / 1e9
    return {"workload": f"{name}: {T} tokens, {E} experts, bf16 weights" + (", Zipf(1.2) routing" if shape.zipf else ""),
            "tokens_per_s": T / s_step, "us_per_step": s_step * 1e6, "median_us_per_step": med * 1e6,
            "stage_us": {k: v * 1e3 for k, v in st.items()},
            "gate_up_roofline": {"bound": bound, "achieved": ach, "unit": "TFLOP/s" if bound == "mfma" else "GB/s",
                                 "frac": ach / (PEAK_BF16_TFLOPS if bound == "mfma" else PEAK_HBM_GBS)},
            "expert_gemms": {"tflops": (fl_gu + fl_dn) / (t_gu + t_dn) / 1e12,
                             "frac_bf16_peak": (fl_gu + fl_dn) / (t_gu + t_dn) / 1e12 / PEAK_BF16_TFLOPS,
                             "gbs": (by_gu + by_dn) / (t_gu + t_dn) / 1e9,
                             "frac_hbm_peak": (by_gu + by_dn) / (t_gu + t_dn) / 1e9 / PEAK_HBM_GBS}}


def synth_configs():
    from gpt_oss_amd import synth
    return synth.CONFIGS


def mxfp4_weight_bytes(shape):
    # nibbles + one scale byte per 32 weights
    return shape.experts * 3 * shape.hidden * shape.inter * (0.5 + 1.0 / 32)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="c2",
                    help="c2 (headline), c3a, c3b, c4, c5 (MXFP4 decode); d4: yardstick, four dense GEMMs of 4096 rows")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--zero-expert-weights", action="store_true",
                    help="yardstick, bf16 workloads only: the expert matrices are uploaded as zeros (same routing, "
                         "tiles, instructions and traffic; the line is marked and is not a benchmark result)")
    ap.add_argument("--no-decode", action="store_true",
                    help="c2 only: skip the side figures (MXFP4 weights: workload c5 and c2's batch; "
                         "the other configurations c3a, c3b, c4)")
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
    if args.zero_expert_weights:
        if mxfp4:
            print("--zero-expert-weights is for the bf16 workloads", file=sys.stderr)
            sys.exit(2)
        args.no_decode = args.no_cpu_baseline = True  # a yardstick line carries neither
    s_per_step, stages, n_meas, median_s, L = run_leg(shape, args.steps, args.warmup,
                                                      zero_expert_weights=args.zero_expert_weights)

    A = T * K
    flops_gate_up = 2.0 * A * H * 2 * IM
    flops_down = 2.0 * A * IM * H
    t_gate_up = stages["gate_up"] * 1e-3
    t_gemms = (stages["gate_up"] + stages["down"]) * 1e-3
    both = (flops_gate_up + flops_down) / t_gemms / 1e12
    w_elem = (0.5 + 1.0 / 32) if mxfp4 else 2.0  # bytes per expert weight in HBM
    # algorithmic bytes: every expert matrix once, routed rows in, activations / fp32 rows out
    bytes_gate_up = E * 2 * IM * H * w_elem + A * H * 2 + A * IM * 2
    bytes_down = E * H * IM * w_elem + A * IM * 2 + A * H * 4
    router_bytes = T * H * 2 + E * H * 2 + E * 2 + T * K * 8
    dispatch_bytes = T * K * 4 + A * 4 + (E + 1) * 4
    combine_bytes = A * H * 2 + T * H * 4
    mfma_tflops = flops_gate_up / t_gate_up / 1e12
    hbm_gbs = bytes_gate_up / t_gate_up / 1e9
    kernel = "grouped_gemm_kernel<gate_up%s>" % (", MXFP4" if mxfp4 else "")
    if BOUND[shape.name] == "mfma":
        roofline = {"bound": "mfma", "kernel": kernel, "achieved": mfma_tflops, "peak": PEAK_BF16_TFLOPS,
                    "unit": "TFLOP/s", "frac": mfma_tflops / PEAK_BF16_TFLOPS}
    else:
        roofline = {"bound": "hbm", "kernel": kernel, "achieved": hbm_gbs, "peak": PEAK_HBM_GBS,
                    "unit": "GB/s", "frac": hbm_gbs / PEAK_HBM_GBS}
    # `peak` is the published figure.  Next to it, what this GPU sustains on the
    # same instruction from registers alone (all 256 CUs, operands of unit scale)
    # and on plain streams through HBM, measured now by the library's yardsticks.
    roofline["peak_kind"] = "published"
    try:
        tf, ghz = abi.yardstick_mfma(256, 20000, data=2)   # activations against weights, as in the layer
        tf1, ghz1 = abi.yardstick_mfma(256, 20000, data=1)  # both operands of unit scale
        tf0, ghz0 = abi.yardstick_mfma(256, 20000, data=0)
        copy_gbs, read_gbs = abi.yardstick_hbm(1 << 30, 10)
        roofline["measured_peak_tflops"] = tf
        roofline["measured_peak_gbs"] = max(copy_gbs, read_gbs)
        roofline["measured_peak"] = {
            "mfma_tflops": tf, "mfma_shader_ghz": ghz,
            "mfma_tflops_unit_scale_operands": tf1, "mfma_shader_ghz_unit_scale_operands": ghz1,
            "mfma_tflops_zero_operands": tf0, "mfma_shader_ghz_zero_operands": ghz0,
            "hbm_copy_gbs": copy_gbs, "hbm_read_gbs": read_gbs,
            "how": "moe_yardstick_mfma: v_mfma_f32_32x32x16_bf16 from registers, 256 workgroups x 4 waves, "
                   "16 accumulators each, pseudo-random operands (unit scale against scale 0.02, as "
                   "activations meet weights); moe_yardstick_hbm: copy (read + write bytes) and read-only "
                   "kernels over 1 GiB"}
        roofline["frac_of_measured_peak"] = (mfma_tflops / tf if roofline["bound"] == "mfma"
                                             else hbm_gbs / max(copy_gbs, read_gbs))
    except abi.MoeError as e:
        roofline["measured_peak"] = {"error": str(e)}
    roofline["traffic"] = measured_traffic(shape.name)
    roofline["traffic_source"] = (f"profiles/bench_{shape.name}_counters.md (rocprofv3 --pmc run of this workload, "
                                  "not this run)" if roofline["traffic"] is not None else None)
    # the other roofline of the same kernel, for the workloads near the machine balance
    roofline["frac_mfma_peak"] = mfma_tflops / PEAK_BF16_TFLOPS
    roofline["frac_hbm_peak"] = hbm_gbs / PEAK_HBM_GBS
    weights = "MXFP4 expert weights" if mxfp4 else "bf16 weights"
    if args.zero_expert_weights:
        weights = "bf16 weights ALL ZERO (yardstick: not a benchmark result)"
    result = {
        "metric": "MoE-layer tokens/sec",
        "value": T / s_per_step,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_steps": SETTLE_STEPS,
        "ms_per_step": s_per_step * 1e3,
        "median_ms_per_step": median_s * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"{shape.name}: {T} tokens, hidden {H}, intermediate {IM}, "
                               f"{E} experts, top-{K}, {weights}, fp32 accumulate, seed 0"},
        "roofline": roofline,
        "expert_gemms": {"tflops": both, "frac_bf16_peak": both / PEAK_BF16_TFLOPS,
                         "gbs": (bytes_gate_up + bytes_down) / t_gemms / 1e9,
                         "frac_hbm_peak": (bytes_gate_up + bytes_down) / t_gemms / 1e9 / PEAK_HBM_GBS},
        "stage_us": {k: v * 1e3 for k, v in stages.items()},
        "router_gbs": router_bytes / (stages["router"] * 1e-3) / 1e9,
        # up to 64 tokens no dispatch kernel runs (the other kernels find their rows themselves):
        # the stage's interval is then only the distance between two events
        "dispatch_gbs": dispatch_bytes / (stages["dispatch"] * 1e-3) / 1e9 if T > 64 else None,
        "combine_gbs": combine_bytes / (stages["combine"] * 1e-3) / 1e9,
        "events_calls": n_meas,
    }
    if shape.name == "c2" and not args.no_decode:
        # Side figure, not the headline value: the decode-regime configuration,
        # priced against the HBM peak on the weight bytes its GEMMs stream.
        c5 = synth.CONFIGS["c5"]
        s5, st5, _, med5, _ = run_leg(c5, 200, 20, device_timed=True)
        wb = mxfp4_weight_bytes(c5)
        gemm_s = (st5["gate_up"] + st5["down"]) * 1e-3
        result["decode_mxfp4"] = {
            "workload": f"c5: {c5.tokens} tokens, {c5.experts} experts, MXFP4 expert weights",
            "tokens_per_s": c5.tokens / s5, "us_per_step": s5 * 1e6, "median_us_per_step": med5 * 1e6,
            "stage_us": {k: v * 1e3 for k, v in st5.items()},
            "weight_bytes": wb, "gemm_gbs": wb / gemm_s / 1e9,
            "gemm_frac_hbm_peak": wb / gemm_s / 1e9 / PEAK_HBM_GBS,
            "layer_gbs": wb / s5 / 1e9}
        # Second side figure: the headline batch with the expert weights in the
        # checkpoint's own MXFP4 form (config 5's value distribution) instead of
        # config 2's bf16 matrices.  The arithmetic is the same bf16 MFMA with
        # fp32 accumulation; the weights arrive as 0.53 bytes each.
        s4, st4, _, med4, _ = run_leg(shape, 100, 20, mxfp4=True)
        tg, td = st4["gate_up"] * 1e-3, st4["down"] * 1e-3
        result["prefill_mxfp4"] = {
            "workload": f"{T} tokens, {E} experts, MXFP4 expert weights (c2's batch, c5's weights)",
            "tokens_per_s": T / s4, "us_per_step": s4 * 1e6, "median_us_per_step": med4 * 1e6,
            "stage_us": {k: v * 1e3 for k, v in st4.items()},
            "gate_up_tflops": flops_gate_up / tg / 1e12,
            "gate_up_frac_bf16_peak": flops_gate_up / tg / 1e12 / PEAK_BF16_TFLOPS,
            "expert_gemms_tflops": (flops_gate_up + flops_down) / (tg + td) / 1e12,
            "expert_gemms_frac_bf16_peak": (flops_gate_up + flops_down) / (tg + td) / 1e12 / PEAK_BF16_TFLOPS}
        # The other benchmark configurations (skewed routing at 512 and 7168
        # tokens, the 128-expert shape), each a short leg of its own.
        result["other_workloads"] = {n: side_leg(n) for n in ("c3a", "c3b", "c4")}
    if not args.no_cpu_baseline and L is not None:
        result["cpu_baseline"] = cpu_baseline(shape, L)
    if shape.name == "c2" and not args.no_decode and L is not None:
        # Yardstick, not a result: the headline workload once more with the expert
        # matrices uploaded as zeros -- same routing, tiles, instructions and memory
        # traffic; the matrix cores' operands stop toggling and the GPU holds a
        # higher clock.  Says how much of the distance to the published peak is
        # the clock under load and how much the kernels' idle cycles.
        _, stz, _, _, _ = run_leg(shape, 60, 10, zero_expert_weights=True, layer=L)
        tg, td = stz["gate_up"] * 1e-3, stz["down"] * 1e-3
        result["zero_weights_yardstick"] = {
            "workload": "c2 with all-zero expert weights (not a benchmark result)",
            "stage_us": {k: v * 1e3 for k, v in stz.items()},
            "gate_up_tflops": flops_gate_up / tg / 1e12,
            "gate_up_frac_bf16_peak": flops_gate_up / tg / 1e12 / PEAK_BF16_TFLOPS,
            "expert_gemms_frac_bf16_peak": (flops_gate_up + flops_down) / (tg + td) / 1e12 / PEAK_BF16_TFLOPS}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
