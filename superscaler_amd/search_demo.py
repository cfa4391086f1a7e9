"""Streamed scoring plus a host search loop on one MI355X, end to end.

    python -m superscaler_amd.search_demo --workload gpt3_175b --stream-plans 4194304 --batch 262144 \
        --steps 200 --neighbours 16384

Part 1 streams seeded synthetic plans through `PlanEvaluator.score_stream` in batches (upload of
batch k+1 overlapped with the kernels of batch k) and keeps the global top-k.  Part 2 runs the
batched local search of `neighbours.hill_climb` from the best streamed plan: every step builds the
neighbours as byte edits on the host, drops the ones already visited, optionally re-chooses their
recompute bits with check_recompute, and scores them in one launch.  Prints one JSON line with the
timings.  The search policy of the reference (aceso_policy.py) is not reproduced here.
"""
import argparse
import json
import time

import numpy as np


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="gpt3_175b")
    ap.add_argument("--stream-plans", type=int, default=4194304)
    ap.add_argument("--batch", type=int, default=262144)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--neighbours", type=int, default=16384)
    ap.add_argument("--topk", type=int, default=64)
    ap.add_argument("--greedy-recompute", action="store_true")
    ap.add_argument("--device-moves", action="store_true",
                    help="expand the move descriptors on the device (visited set over 128-bit plan keys)")
    ap.add_argument("--workers", type=int, default=16)
    ap.add_argument("--distinct-batches", type=int, default=0,
                    help="generate only this many different batches and cycle through them (0 = all different); "
                         "takes the host's plan generator out of the streamed part's wall time")
    args = ap.parse_args(argv)

    from . import synth
    from .aceso_cost_model import CostModel
    from .neighbours import VisitedKeys, VisitedPlans, hill_climb

    w = synth.WORKLOADS[args.workload]
    graph = synth.make_graph(w)
    cm = CostModel(synth.make_settings(w), synth.make_db(w, graph), graph)
    ev = cm.evaluator
    n_batches = (args.stream_plans + args.batch - 1) // args.batch
    gen_s = [0.0]
    kept = {}

    def make(j):
        jj = j % args.distinct_batches if args.distinct_batches else j
        return synth.make_plans(w, cm.tables, n_plans=min(args.batch, args.stream_plans - j * args.batch),
                                seed_offset=1000 + jj, workers=args.workers)

    pre = [make(j) for j in range(min(args.distinct_batches, n_batches))]

    def batches():
        for j in range(n_batches):
            t0 = time.perf_counter()
            b = pre[j % len(pre)].slice(0, min(args.batch, args.stream_plans - j * args.batch)) if pre else make(j)
            gen_s[0] += time.perf_counter() - t0
            kept.clear()
            kept[j] = b                       # the last batch stays around in case it holds the winner
            yield b

    t0 = time.perf_counter()
    idx, val, seen = ev.score_stream(batches(), args.topk)
    stream_s = time.perf_counter() - t0
    out = {"workload": w.name, "ops": graph.num_ops, "streamed_plans": seen, "batches": n_batches,
           "stream_wall_s": round(stream_s, 3), "of_which_plan_generation_s": round(gen_s[0], 3),
           "stream_plans_per_s": seen / stream_s, "distinct_batches": args.distinct_batches or n_batches,
           "stream_feasible_in_topk": int(len(idx)), "stream_best_ms": float(val[0]) if len(val) else None}

    if args.steps > 0:
        if len(idx):
            j, r = divmod(int(idx[0]), args.batch)
            src = kept[j] if j in kept else make(j)
            start = src.slice(r, r + 1)
        else:
            start = synth.make_plans(w, cm.tables, n_plans=1, seed_offset=1)
        visited = VisitedKeys() if args.device_moves else VisitedPlans()
        trace = []
        t0 = time.perf_counter()
        plan, t, m = hill_climb(cm, start, steps=args.steps, n_neighbours=args.neighbours, seed=7,
                                on_step=lambda s, t_, m_: trace.append(t_), visited=visited,
                                greedy_recompute=args.greedy_recompute, device_moves=args.device_moves)
        search_s = time.perf_counter() - t0
        out.update({"search_steps": args.steps, "neighbours_per_step": args.neighbours,
                    "search_wall_s": round(search_s, 3), "search_steps_per_s": args.steps / search_s,
                    "neighbours_generated_per_s": args.steps * args.neighbours / search_s,
                    "distinct_plans_scored": len(visited) if visited is not None else None,
                    "greedy_recompute": bool(args.greedy_recompute), "device_moves": bool(args.device_moves),
                    "search_start_ms": float(val[0]) if len(val) else None, "search_best_ms": t, "search_best_mb": m,
                    "improving_steps": int(np.sum(np.diff([trace[0]] + trace) < 0)) if trace else 0})
    cm.close()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
