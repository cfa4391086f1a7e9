#!/usr/bin/env python3
"""Benchmark of the plan-scoring hot path on one MI355X.

A step = one pass over the whole batch, inputs already resident in HBM: the scoring kernel
(iteration time, peak memory, feasibility flag per plan) followed by the device-wide top-k.
Workload: the GPT-3 13B op graph (523 ops), 1,048,576 seeded synthetic plans at D = 32.
Prints one JSON line (metric, roofline of the scoring kernel, CPU baseline).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# Counter readings of the scoring kernel on the default workload, which a run of this script cannot take itself
# (rocprofv3 --pmc passes): copied from the committed summary named in "source".  "library" is
# superscaler_amd.build.source_hash() of the library sources they were taken on: when the sources no longer hash to
# it the readings are left out of the line (with a note) instead of being reported for another kernel.
# HBM bytes per plan and launch = FETCH_SIZE + WRITE_SIZE, each scaled by the reading of a plain 256 MiB copy in
# the same pass; vector instructions per op and wavefront = SQ_INSTS_VALU / SQ_WAVES / ops; 14 of them are the
# reference's own fp64 arithmetic (nine adds / multiply-adds, five maxima).
PROFILE_COUNTERS = {
    ("gpt3_13b", 523): {"source": "profiles/score_kernel_gpt3_13b.md", "library": "b570eaebab746de3", "traffic_bytes_per_plan": 1715.0,
                        "valu_per_op_per_wavefront": 35.1, "valu_busy": 0.78},
}
# the other configured workloads, timed after the headline measurement (kernel only, HIP events on the launch stream)
OTHER_WORKLOADS = ("gpt3_1_3b", "t5_770m", "wresnet_1b", "gpt3_175b")
OTHER_PLANS = 262144
ESSENTIAL_VALU_PER_OP = 14


def cpu_baseline(tables, batch, threads):
    """The oracle on the host's cores: its C restatement (one plan after the other per thread, the
    reference's own order of operations) over the whole batch with `threads` threads, and on one
    thread over a slice; the loop-faithful Python oracle on one core for scale."""
    from tests.helpers import c_oracle_for, oracle_config, oracle_for, plan_arrays
    co = c_oracle_for(tables)
    arrays = plan_arrays(batch, tables)
    P = batch.n_plans
    co.score_arrays(*[a[:4096] for a in arrays], threads=threads)          # warm-up
    t0 = time.perf_counter()
    co.score_arrays(*arrays, threads=threads)
    dt_all = time.perf_counter() - t0
    n1 = min(P, 131072)
    t0 = time.perf_counter()
    co.score_arrays(*[a[:n1] for a in arrays], threads=1)
    dt_one = time.perf_counter() - t0
    orc = oracle_for(tables)
    npy = min(P, 8192)           # about 14 s of the Python oracle at 523 ops
    cfgs = [oracle_config(batch, p, tables) for p in range(npy)]
    t0 = time.perf_counter()
    for c in cfgs:
        orc.score(c)
    dt_py = time.perf_counter() - t0
    cpu_model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            cpu_model = next((ln.split(":", 1)[1].strip() for ln in f if ln.startswith("model name")), cpu_model)
    except OSError:
        pass
    # the stated baseline is the reference's way of running: pure Python, one process, one core
    return {"value": npy / dt_py, "unit": "plans/s", "cores": 1, "kind": "port", "cpu_model": cpu_model,
            "sample": f"first {npy} plans of the same batch in {dt_py:.2f} s, loop-faithful Python oracle "
                      "(oracle/aceso_oracle.py), 1 process",
            "c_port_value": P / dt_all, "c_port_cores": threads,
            "c_port_sample": f"all {P} plans in {dt_all:.2f} s, C oracle (oracle/aceso_oracle.c), {threads} OpenMP threads",
            "c_port_single_core_value": n1 / dt_one,
            "c_port_single_core_sample": f"first {n1} plans, {dt_one:.2f} s, 1 thread"}


def kernel_name(tables):
    """The instantiation plain scoring of a large batch runs (the library's choice, ensure_stage_ws in ace_eval.hip)."""
    deferred = tables.graph.num_ops < 65536 and (tables.n_windows == 1 or tables.rows.shape[0] <= 256)
    return "ace_score_kernel<BD=false,RANGED=false,WIN=%s,DEFER=%s>" % ("true" if tables.n_windows > 1 else "false",
                                                                          "true" if deferred else "false")


def other_workloads(steps):
    """Scoring kernel alone on the other configured workloads: {name: kernel, ms, bytes per plan, roofline fraction}."""
    from superscaler_amd import synth
    from superscaler_amd.evaluator import PlanEvaluator
    out = {}
    for name in OTHER_WORKLOADS:
        w = synth.WORKLOADS[name]
        tables = synth.make_tables(w)
        batch = synth.make_plans(w, tables, n_plans=OTHER_PLANS, workers=min(16, os.cpu_count() or 1))
        ev = PlanEvaluator(tables, device="cuda:0")
        d = ev.upload(batch)
        # (the plans of each workload are drawn on the host for seconds while the GPU idles: as many untimed launches
        # as timed ones first, like the headline measurement's warm-up)
        ev.time_score_kernel(d, reps=max(steps, 20))
        ms = ev.time_score_kernel(d, reps=max(steps, 20))
        bpp = 3 * d.num_ops + 19
        gbps = bpp * d.n_plans / (ms * 1e-3) / 1e9
        out[name] = {"kernel": kernel_name(tables), "ops": d.num_ops, "plans": d.n_plans, "kernel_ms": ms,
                     "plans_per_s_kernel": d.n_plans / (ms * 1e-3), "algorithmic_bytes_per_plan": bpp,
                     "achieved_GBps": gbps, "frac": gbps / HBM_PEAK_GBPS}
        ev.close()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="gpt3_13b")
    ap.add_argument("--plans", type=int, default=None)
    ap.add_argument("--topk", type=int, default=64)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--pp", type=int, nargs="+", default=None,
                    help="restrict the pipeline depths the plans are drawn from (profiling aid)")
    ap.add_argument("--no-pcie-rate", action="store_true", help="skip the host-memory-in measurement")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="skip the kernel timings of the other configured workloads (config.other_workloads)")
    ap.add_argument("--regrouped-too", action="store_true",
                    help="also time the step on a copy of the batch regrouped on the device beforehand (by pipeline "
                         "depth and first stage boundaries; ace_group_keys / ace_gather_plans), as a secondary figure")
    ap.add_argument("--calibration-copy-mib", type=int, default=0,
                    help="also run one plain device-to-device copy of this many MiB (a kernel of known "
                         "traffic, to scale FETCH_SIZE / WRITE_SIZE counter readings)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this evaluator runs on ONE GPU (plans are independent; device counts of the plans "
              "are cost-model inputs only). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    from superscaler_amd import synth
    from superscaler_amd.evaluator import PlanEvaluator
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)

    w = synth.WORKLOADS[args.workload]
    if args.pp:
        import dataclasses
        w = dataclasses.replace(w, pp_choices=list(args.pp))
    n_plans = args.plans or w.n_plans
    tables = synth.make_tables(w)
    t0 = time.perf_counter()
    batch = synth.make_plans(w, tables, n_plans=n_plans, workers=min(16, os.cpu_count() or 1))
    gen_s = time.perf_counter() - t0
    ev = PlanEvaluator(tables, device="cuda:0")
    d = ev.upload(batch)                      # the plans as the generator emitted them
    P, N = d.n_plans, d.num_ops
    it = torch.empty(P, dtype=torch.float64, device="cuda:0")
    pk = torch.empty(P, dtype=torch.float64, device="cuda:0")
    fe = torch.empty(P, dtype=torch.uint8, device="cuda:0")
    st = torch.empty(P, dtype=torch.uint8, device="cuda:0")

    def step(db):
        ev.score(db, out=(it, pk, fe, st))
        return ev.topk(it, fe, args.topk)

    def timed(db):
        for _ in range(args.warmup):
            step(db)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            out = step(db)
        torch.cuda.synchronize()
        return time.perf_counter() - t0, out

    elapsed, (idx, val, cnt) = timed(d)
    ms_per_step = elapsed / args.steps * 1e3
    plans_per_s = P * args.steps / elapsed
    # dominant kernel: the scoring kernel, timed with HIP events on its launch stream
    kern_ms = ev.time_score_kernel(d, reps=max(args.steps, 5))
    secondary = {}
    if args.regrouped_too:
        ev.group(d)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        dg = ev.group(d)
        torch.cuda.synchronize()
        secondary["regrouping_ms"] = (time.perf_counter() - t0) * 1e3
        elapsed_g, (idx2, val2, cnt2) = timed(dg)
        assert torch.equal(idx, idx2) and torch.equal(val, val2), "grouped storage changed the ranking"
        secondary["value_plans_regrouped_beforehand"] = P * args.steps / elapsed_g
        secondary["kernel_ms_plans_regrouped_beforehand"] = ev.time_score_kernel(dg, reps=max(args.steps, 5))
        elapsed, (idx, val, cnt) = timed(d)        # (leaves the generator-order results in the output tensors)
    # what a caller holding its plans in host memory sees: page-locked buffers in, global top-k out, the upload of one
    # batch overlapped with the scoring of the one before (never the headline value)
    if not args.no_pcie_rate:
        n_host = 4
        hb = ev.pinned_plan_batch(P)
        hb.codes[...] = batch.codes
        hb.hdr[...] = batch.hdr
        ev.score_stream([hb], args.topk)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        hidx, hval, hseen = ev.score_stream([hb] * n_host, args.topk)
        torch.cuda.synchronize()
        dt_host = time.perf_counter() - t0
        assert hseen == n_host * P and hval[0] == val[0].item()
        secondary["pcie_inclusive_plans_per_s"] = hseen / dt_host
        secondary["pcie_inclusive_note"] = (f"{n_host} x {P} plans from page-locked host memory through score_stream "
                                            f"({N} B of plan bytes each, {hseen * (N + 16) / dt_host / 1e9:.1f} GB/s over the bus)")
    algo_bytes = (3 * N + 19) * P            # canonical encoding: 3 bytes per op + 2 + 17 bytes of results
    moved_bytes = d.bytes_moved_per_plan * P + 17 * P
    achieved = algo_bytes / (kern_ms * 1e-3) / 1e9
    n_feasible = int(fe.sum().item())
    best = val[0].item() if n_feasible else None
    counters = PROFILE_COUNTERS.get((w.name, N)) if P == w.n_plans and not args.pp else None
    counters_note = None
    from superscaler_amd import build as lib_build
    if counters and counters["library"] != lib_build.source_hash():
        counters_note = (f'the counter readings of {counters["source"]} were taken on library sources {counters["library"]}; '
                         f"these sources hash to {lib_build.source_hash()}: readings left out")
        counters = None

    out = {
        "metric": "plans scored/sec at GPT-3 13B op graph (1M plans); % HBM roofline",
        "value": plans_per_s, "unit": "plans/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f64", "data": "synthetic",
        "config": dict({"workload": f"{w.name}: {N}-op graph, {P} seeded plans, D={w.num_gpus}, "
                                    f"PP in {w.pp_choices}, mbs in {w.mbs_list}, recompute p={w.recompute_p}, "
                                    f"memory cap {w.memory_limit:.0f} MB, global batch {w.global_batch}, top-{args.topk}",
                        "step": "score kernel + device-wide top-k, inputs resident in HBM",
                        "layout": "plans in the generator's order (each workgroup of the kernel deals its 1,024 plans to "
                                  "its lanes by pipeline depth; nothing is reordered beforehand)",
                        "feasible_plans": n_feasible, "best_iter_ms": best, "plan_generation_s": round(gen_s, 1)},
                       **secondary),
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS,
                     "traffic": counters["traffic_bytes_per_plan"] * P if counters else None,
                     "traffic_source": f'{counters["source"]} (library sources {counters["library"]})' if counters else counters_note,
                     "algorithmic_bytes": algo_bytes,
                     "kernel": kernel_name(tables), "kernel_ms": kern_ms,
                     "algorithmic_bytes_per_plan": 3 * N + 19,
                     "bytes_moved_per_plan": d.bytes_moved_per_plan + 17,
                     "achieved_on_bytes_moved": moved_bytes / (kern_ms * 1e-3) / 1e9,
                     "note": "HBM is the nominal roofline of this path (plan bytes streamed once, tables in LDS); inside the CU "
                             "the kernel is held by vector-instruction issue and LDS reads, see roofline_valu_issue"},
    }
    if counters:
        # the bound that holds: one vector instruction per SIMD and quad-cycle; the time of the kernel is the number
        # of vector instructions its wavefronts issue
        v = counters["valu_per_op_per_wavefront"]
        out["roofline_valu_issue"] = {"bound": "valu_issue", "unit": "vector instructions per op per wavefront",
                                      "essential": ESSENTIAL_VALU_PER_OP, "achieved": v,
                                      "frac": ESSENTIAL_VALU_PER_OP / v, "simd_valu_busy": counters["valu_busy"],
                                      "source": counters["source"]}
    if args.calibration_copy_mib > 0:
        src = torch.zeros(args.calibration_copy_mib << 20, dtype=torch.uint8, device="cuda:0")
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        out["config"]["calibration_copy_bytes"] = int(src.numel())
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(tables, batch, threads=min(16, os.cpu_count() or 1))
    ev.close()
    if not args.no_other_workloads and args.workload == "gpt3_13b" and not args.pp:
        out["config"]["other_workloads"] = other_workloads(args.steps)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
