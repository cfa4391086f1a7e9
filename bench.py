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
# HBM bytes per plan of one scoring-kernel launch on the default workload, from two rocprofv3 --pmc
# runs (FETCH_SIZE, then WRITE_SIZE) scaled by the readings of a plain 256 MiB copy in the same
# runs (factors 2.000 and 1.000), keyed by (workload, ops, plans grouped at upload):
# 1,049 B read + 681 B written with the grouped layout, 1,334 + 618 in the generator's order.
MEASURED_TRAFFIC_BYTES_PER_PLAN = {("gpt3_13b", 523, True): 1731.0, ("gpt3_13b", 523, False): 1952.0}


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
    npy = min(P, 1024)
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
    return {"value": P / dt_all, "unit": "plans/s", "cores": threads, "kind": "port", "cpu_model": cpu_model,
            "sample": f"all {P} plans of the same batch in {dt_all:.2f} s, C oracle (oracle/aceso_oracle.c), "
                      f"{threads} OpenMP threads",
            "single_core_value": n1 / dt_one, "single_core_sample": f"first {n1} plans, {dt_one:.2f} s, 1 thread",
            "python_oracle_value": npy / dt_py,
            "python_oracle_sample": f"first {npy} plans, {dt_py:.2f} s, pure-Python oracle, 1 process"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="gpt3_13b")
    ap.add_argument("--plans", type=int, default=None)
    ap.add_argument("--topk", type=int, default=64)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--pp", type=int, nargs="+", default=None,
                    help="restrict the pipeline depths the plans are drawn from (profiling aid)")
    ap.add_argument("--caller-order", action="store_true",
                    help="keep the plans in the generator's order in HBM instead of grouping them by pipeline "
                         "depth and first stage boundaries at upload (results are in the generator's order either way)")
    ap.add_argument("--no-layout-comparison", action="store_true",
                    help="do not also time the kernel on the plans in the generator's order (keeps a profiler's "
                         "per-kernel average to the benchmark's own layout)")
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
    d_plain = ev.upload(batch)
    d, group_ms = d_plain, None
    if not args.caller_order:
        # grouped storage, made on the device from the plain upload; timed, but not part of the step
        ev.group(d_plain)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        d = ev.group(d_plain)
        torch.cuda.synchronize()
        group_ms = (time.perf_counter() - t0) * 1e3
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
    plain_plans_per_s = plans_per_s
    if not args.caller_order and not args.no_layout_comparison:
        elapsed_plain, (idx2, val2, cnt2) = timed(d_plain)
        plain_plans_per_s = P * args.steps / elapsed_plain
        assert torch.equal(idx, idx2) and torch.equal(val, val2), "grouped storage changed the ranking"

    # dominant kernel: the scoring kernel, timed with HIP events on its launch stream
    kern_ms = ev.time_score_kernel(d, reps=max(args.steps, 5))
    kern_ms_caller_order = kern_ms
    if not args.caller_order and not args.no_layout_comparison:
        kern_ms_caller_order = ev.time_score_kernel(d_plain, reps=max(args.steps, 5))
    algo_bytes = (3 * N + 19) * P            # canonical encoding: 3 bytes per op + 2 + 17 bytes of results
    moved_bytes = d.bytes_moved_per_plan * P + 17 * P
    achieved = algo_bytes / (kern_ms * 1e-3) / 1e9
    n_feasible = int(fe.sum().item())
    best = val[0].item() if n_feasible else None

    out = {
        "metric": "plans scored/sec at GPT-3 13B op graph (1M plans); % HBM roofline",
        "value": plans_per_s, "unit": "plans/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f64", "data": "synthetic",
        "config": {"workload": f"{w.name}: {N}-op graph, {P} seeded plans, D={w.num_gpus}, "
                               f"PP in {w.pp_choices}, mbs in {w.mbs_list}, recompute p={w.recompute_p}, "
                               f"memory cap {w.memory_limit:.0f} MB, global batch {w.global_batch}, top-{args.topk}",
                   "step": "score kernel + device-wide top-k, inputs resident in HBM",
                   "layout": ("plans in the generator's order" if args.caller_order else
                              "resident plans regrouped once on the device (by pipeline depth and first two stage "
                              "boundaries, wavefronts dealt to the workgroups) before the timed steps; results and "
                              "top-k indices in the generator's order"),
                   "regrouping_ms": group_ms,
                   "value_plans_in_generator_order": plain_plans_per_s,
                   "feasible_plans": n_feasible, "best_iter_ms": best, "plan_generation_s": round(gen_s, 1)},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS,
                     "traffic": (MEASURED_TRAFFIC_BYTES_PER_PLAN[(w.name, N, not args.caller_order)] * P
                                 if (w.name, N, not args.caller_order) in MEASURED_TRAFFIC_BYTES_PER_PLAN else None),
                     "algorithmic_bytes": algo_bytes,
                     "kernel": "ace_score_kernel<BD=false,RANGED=false,WIN=false,DEFER=true>", "kernel_ms": kern_ms,
                     "kernel_ms_plans_in_generator_order": kern_ms_caller_order,
                     "algorithmic_bytes_per_plan": 3 * N + 19,
                     "bytes_moved_per_plan": d.bytes_moved_per_plan + 17,
                     "achieved_on_bytes_moved": moved_bytes / (kern_ms * 1e-3) / 1e9},
    }
    if args.calibration_copy_mib > 0:
        src = torch.zeros(args.calibration_copy_mib << 20, dtype=torch.uint8, device="cuda:0")
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        out["config"]["calibration_copy_bytes"] = int(src.numel())
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(tables, batch, threads=min(16, os.cpu_count() or 1))
    ev.close()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
