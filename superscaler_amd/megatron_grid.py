"""Uniform (Megatron-style) plan grid: enumerate -> score on the GPU in one batch -> keep the
feasible plans -> rank.  The batched form of the reference's search/gen_megatron_plan.py:
enumeration rules :24-99, feasibility `max memory < limit` (strict, :111), one plan per distinct
iteration time keeping the lower-memory one (:113-119), ascending order (:131-135)."""
from typing import List, Optional, Tuple

import numpy as np

from .aceso_cost_model import CostModel
from .plan import AcesoConfig, get_config


def _balance_configs(cm: CostModel, pp: int, tp: int, dp: int, mbs: int, recomp: bool, num_layers) -> List[AcesoConfig]:
    """gen_megatron_plan.py:24-70."""
    ops = cm.graph.ops
    n = len(ops)
    model = cm.settings.model_name
    rc = [1 if recomp else 0] * n
    if model in ("gpt", "t5", "scale-layer"):
        rc[0] = 0
        rc[-1] = 0
    tps, dps, algo = [tp] * n, [dp] * n, [0] * n
    gbs = cm.settings.global_batch_size
    if model in ("gpt", "scale-layer"):
        if num_layers % pp:
            return []
        nops = [(num_layers // pp) * 13 for _ in range(pp)]
        nops[0] += 1
        nops[-1] += 2
        return [get_config(nops, tps, dps, rc, mbs, gbs, ops, algo)]
    if model == "t5":
        if pp == 1:
            return [get_config([num_layers * (13 + 21) + 5], tps, dps, rc, mbs, gbs, ops, algo)]
        out = []
        for k in range(1, pp):
            if num_layers % k == 0 and num_layers % (pp - k) == 0:
                nops = [(num_layers // k) * 13 for _ in range(k)]
                nops[0] += 1
                nops[-1] += 1
                nops += [(num_layers // (pp - k)) * 21 for _ in range(pp - k)]
                nops[k] += 1
                nops[-1] += 2
                out.append(get_config(nops, tps, dps, rc, mbs, gbs, ops, algo))
        return out
    if model == "resnet":
        layers = (n - 6) // 8
        nops = [(layers // pp) * 8 for _ in range(pp)]
        nops[0] += 4
        nops[-1] += 2
        nops[-1] += (layers - (layers // pp) * pp) * 8
        return [get_config(nops, tps, dps, rc, mbs, gbs, ops, algo)]
    raise RuntimeError(f"model {model} not supported yet.")


def enumerate_grid(cm: CostModel, num_gpus: int, num_layers: Optional[int], start_num_stages: int = 1,
                   end_num_stages: Optional[int] = None) -> List[AcesoConfig]:
    """gen_megatron_plan.py:85-99: every (pp, tp, dp, micro-batch, recompute) that divides evenly."""
    end = min(num_gpus, 16) if end_num_stages is None else end_num_stages
    mbs_list = cm.db.mbs_list
    out = []
    for pp in range(start_num_stages, end + 1):
        for tp in cm.db.tp_list:
            if num_gpus % (pp * tp):
                continue
            dp = num_gpus // (pp * tp)
            for mbs in mbs_list:
                if mbs // dp not in mbs_list:
                    continue
                for recomp in (True, False):
                    out += [c for c in _balance_configs(cm, pp, tp, dp, mbs, recomp, num_layers)
                            if all(len(st.ops) > 0 for st in c.stages)]
    return out


def best_uniform_plans(cm: CostModel, num_gpus: int, num_layers: Optional[int], num_saved: int = 1,
                       start_num_stages: int = 1, end_num_stages: Optional[int] = None
                       ) -> List[Tuple[float, float, AcesoConfig]]:
    """The `num_saved` fastest feasible uniform plans as (iteration ms, peak MB, config)."""
    configs = enumerate_grid(cm, num_gpus, num_layers, start_num_stages, end_num_stages)
    if not configs:
        return []
    it, pk, fe = cm.score_batch(configs, strict=True)          # one launch for the whole grid
    best = {}
    for i in np.flatnonzero(fe):
        t, m = float(it[i]), float(pk[i])
        if t not in best or m < best[t][0]:
            best[t] = (m, i)
    return [(t, best[t][0], configs[best[t][1]]) for t in sorted(best)[:num_saved]]


def main(argv=None) -> int:
    """Command line with the arguments gen_megatron_plan.py reads (aceso_utils.py:359-531, the subset
    this script uses): scores the whole uniform grid in one launch and writes the fastest feasible
    plans as JSON files the runtime accepts, named like the reference's (:135)."""
    import argparse
    import time
    from .plan import dump_config_to_json
    from .profile_db import CostModelSettings
    ap = argparse.ArgumentParser(description=main.__doc__)
    ap.add_argument("--model-name", required=True, choices=["gpt", "t5", "resnet", "scale-layer"])
    ap.add_argument("--model-size", required=True)
    ap.add_argument("--num-layers", type=int, default=None)
    ap.add_argument("--global-batch-size", type=int, default=1024)
    ap.add_argument("--micro-batch-size", type=int, nargs="+", default=[1, 2, 4, 8])
    ap.add_argument("--num-nodes", type=int, default=1)
    ap.add_argument("--num-gpus-per-node", type=int, default=8)
    ap.add_argument("--memory-limit", type=float, default=28000)
    ap.add_argument("--max-tp", type=int, default=None)
    ap.add_argument("--start-num-stages", type=int, default=1)
    ap.add_argument("--end-num-stages", type=int, default=None)
    ap.add_argument("--num-of-saved-configs", type=int, default=1)
    ap.add_argument("--profiled-time-path", required=True, help="directory of the profiled CSV files, with the trailing /")
    ap.add_argument("--config-save-path", default="./")
    args = ap.parse_args(argv)
    num_gpus = args.num_nodes * args.num_gpus_per_node
    settings = CostModelSettings(model_name=args.model_name, micro_batch_size=list(args.micro_batch_size),
                                 num_gpus_per_node=args.num_gpus_per_node, global_batch_size=args.global_batch_size,
                                 memory_limit=args.memory_limit, max_tp=args.max_tp or args.num_gpus_per_node)
    t0 = time.time()
    cm = CostModel.from_directory(settings, args.model_name, args.model_size, args.profiled_time_path,
                                  num_layers=args.num_layers)
    try:
        best = best_uniform_plans(cm, num_gpus, args.num_layers, args.num_of_saved_configs, args.start_num_stages,
                                  args.end_num_stages)
    finally:
        cm.close()
    if not best:
        print("no feasible config")
    for k, (t, m, cfg) in enumerate(best):
        name = f"{args.config_save_path}{args.model_name}_{args.model_size}_{args.num_layers}layers_megatron_est_{int(t)}.json"
        dump_config_to_json(cfg, name, args.model_name, args.model_size, args.num_layers)
        print(f"best_{k}: {t:.2f} ms, {m:.2f} MB, {cfg.num_stages} stages, micro-batch {cfg.micro_bs} -> {name}")
    print(f"[TOTAL TIME] {time.time() - t0} s.")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
