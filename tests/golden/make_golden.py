#!/usr/bin/env python3
"""Writes the golden vectors under tests/golden/ by running the REFERENCE cost model.

Run in the build container only (it needs /root/reference):

    python tests/golden/make_golden.py

For each model family it (1) copies the few profile-database CSV files the case needs from
the reference tree into tests/golden/db_<case>/ (data files, not source), (2) starts one
child interpreter whose sys.argv carries the flags the reference's import-time argparse
needs, imports the reference's aceso_cost_model there, (3) builds seeded random multi-stage
plans and records what the reference returns for them into tests/golden/<case>.json.

The functions covered are the ones no reference-held output pins: multi-stage / mixed-tp /
resharding-active predict_time_breakdown (all lists it writes), predict_stage_time and its
delta variants, predict_stage_memory (breakdown), get_reserved_memory_list, check_recompute,
predict_value_after_move, wrap_predict_delta_time.  Floats are stored via repr and
round-trip exactly through JSON.
"""
import json
import os
import random
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
REF = "/root/reference"

CASES = {
    # name: (model, size, db dir, mbs list, nodes, gpus/node, global_bs, memory_limit, num_layers)
    "gpt_1_3B": ("gpt", "1_3B", "profiler/profiled-time-eurosys", [1, 2, 4, 8], 2, 4, 512, 12000, 24),
    "resnet_500M": ("resnet", "500M", "profiler/profiled-time-miniset", [32, 64], 1, 4, 768, 12000, None),
    "t5_770M": ("t5", "770M", "profiler/profiled-time-miniset", [1, 2, 4, 8], 1, 4, 512, 9000, 24),
}


def copy_db(case):
    model, size, db, mbs_list, nodes, gpn, gbs, limit, _ = CASES[case]
    dst = os.path.join(HERE, f"db_{case}")
    os.makedirs(dst, exist_ok=True)
    src = os.path.join(REF, db)
    max_tp = min(gpn, 8)
    names = []
    tp = 1
    while tp <= max_tp:
        for m in mbs_list:
            for a in ([0] if model == "t5" else [0, 1]):
                names.append(f"{model}_{size}_mbs{m}_tp{tp}_algo{a}.csv")
        if tp > 1 and model != "t5":
            prims = ["all_gather", "all_reduce", "reduce_scatter", "all_to_all"] if model == "gpt" \
                else ["all_gather", "all_to_all"]
            for p in prims:
                names.append(f"prim_{model}_{size}_{p}_{tp}gpus.csv")
        tp *= 2
    names += ["p2p_intra_node.csv", "p2p_inter_node.csv"]
    for n in names:
        if os.path.exists(os.path.join(src, n)):
            shutil.copyfile(os.path.join(src, n), os.path.join(dst, n))
    return dst


# ------------------------------------------------------------------------------------------
# child: runs inside an interpreter whose argv the reference parses at import
# ------------------------------------------------------------------------------------------
def rand_plan(rng, full_ops, tunable, num_gpus, mbs_list, max_stages, max_tp, uniform_stage=False):
    n = len(full_ops)
    while True:
        S = rng.choice([s for s in (1, 2, 3, 4) if s <= max_stages])
        # stage device counts: powers of two summing to num_gpus
        gl = [1] * S
        while sum(gl) < num_gpus:
            cand = [i for i in range(S) if gl[i] <= num_gpus - sum(gl) and gl[i] < 8]
            if not cand:
                break
            gl[rng.choice(cand)] *= 2
        if sum(gl) != num_gpus:
            continue
        cuts = sorted(rng.sample(range(1, n), S - 1))
        bounds = [0] + cuts + [n]
        nops = [bounds[i + 1] - bounds[i] for i in range(S)]
        tp, dp, rc, algo = [], [], [], []
        for s in range(S):
            g = gl[s]
            cur = rng.choice([t for t in (1, 2, 4, 8) if t <= g and t <= max_tp])
            for k in range(nops[s]):
                if not uniform_stage and rng.random() < 0.04:
                    cur = rng.choice([t for t in (1, 2, 4, 8) if t <= g and t <= max_tp])
                tp.append(cur)
                dp.append(g // cur)
                rc.append(1 if rng.random() < 0.4 else 0)
                name = full_ops[bounds[s] + k]
                algo.append(1 if (name in tunable and rng.random() < 0.15) else 0)
        ok_mbs = [b for b in mbs_list if all((b // d) in mbs_list for d in set(dp))]
        if not ok_mbs:
            continue
        return nops, tp, dp, rc, algo, rng.choice(ok_mbs)


def child(case):
    model, size, db, mbs_list, nodes, gpn, gbs, limit, num_layers = CASES[case]
    dbdir = os.path.join(HERE, f"db_{case}") + "/"
    sys.argv = ["golden", "--model-name", model, "--model-size", size,
                "--num-nodes", str(nodes), "--num-gpus-per-node", str(gpn),
                "--global-batch-size", str(gbs), "--memory-limit", str(limit),
                "--profiled-time-path", dbdir, "--micro-batch-size"] + [str(m) for m in mbs_list]
    sys.path.insert(0, os.path.join(REF, "search"))
    import aceso_cost_model as cm          # noqa: the reference, imported to record its outputs
    from aceso_utils import get_config
    from model_ops_info import get_full_op_list, get_tunable_op_list
    args = cm.args
    cm.read_profiled_time(model, size, dbdir)
    full_ops = get_full_op_list(args)
    tunable = [] if model == "t5" else get_tunable_op_list(args)
    rng = random.Random(0xACE50 + sum(map(ord, case)))
    num_gpus = nodes * gpn
    out = {"case": case, "model_name": model, "model_size": size, "micro_batch_size": mbs_list,
           "num_nodes": nodes, "num_gpus_per_node": gpn, "global_batch_size": gbs,
           "memory_limit": limit, "num_layers": num_layers, "num_ops": len(full_ops), "plans": []}
    n_plans = 16 if model == "gpt" else 8
    for p in range(n_plans):
        nops, tp, dp, rc, algo, mbs = rand_plan(rng, full_ops, tunable, num_gpus, mbs_list, 4, min(gpn, 8),
                                                uniform_stage=(p % 4 == 3))
        config = get_config(nops, tp, dp, rc, mbs, gbs, full_ops, algo)
        cm.predict_time_breakdown(config)
        rec = {"num_ops_in_each_stage": nops, "tp": tp, "dp": dp, "recompute_ops": rc, "algo": algo,
               "micro_batch_size": mbs,
               "time_list": config.time_list, "memory_list": config.memory_list,
               "compute_time_list": config.compute_time_list, "total_gpu_time": config.total_gpu_time,
               "breakdown_ideal_time_per_gpu": config.breakdown_ideal_time_per_gpu,
               "breakdown_eff_loss_time_per_gpu": config.breakdown_eff_loss_time_per_gpu,
               "breakdown_recomp_time_per_gpu": config.breakdown_recomp_time_per_gpu,
               "efficient_time_list": config.efficient_time_list,
               "reserved_memory_list": cm.get_reserved_memory_list(config),
               "stage_time": [], "stage_time_delta": [], "stage_memory": [], "stage_memory_breakdown": [],
               "check_recompute": [], "value_after_move": [], "delta_time": []}
        for st in config.stages:
            rec["stage_time"].append(cm.predict_stage_time(st.ops, st.recompute_ops, st.tp_size, st.dp_size, mbs, st.algo))
            rec["stage_time_delta"].append([
                cm.predict_stage_time(st.ops, st.recompute_ops, st.tp_size, st.dp_size, mbs, st.algo,
                                      delta=True, on_the_right=r, decrease=d)
                for r in (False, True) for d in (False, True)])
            rec["stage_memory"].append(cm.predict_stage_memory(st.ops, st.recompute_ops, st.tp_size, st.dp_size, mbs, st.num_stages_behind, st.algo))
            rec["stage_memory_breakdown"].append(list(cm.predict_stage_memory(st.ops, st.recompute_ops, st.tp_size, st.dp_size, mbs, st.num_stages_behind, st.algo, breakdown=True)))
            rec["check_recompute"].append(cm.check_recompute(st.ops, mbs, st.tp_size, st.dp_size, st.num_stages_behind, st.algo))
        S = config.num_stages
        for b in range(S):
            for partner in (b - 1, b + 1):
                if 0 <= partner < S and len(config.stages[b].ops) > 3:
                    k = rng.randint(1, min(3, len(config.stages[b].ops) - 1))
                    for metric in ("time", "memory"):
                        v, r = cm.predict_value_after_move(config, b, partner, k, metric)
                        rec["value_after_move"].append([b, partner, k, metric, v, list(r)])
                    for dec in (True, False):
                        rec["delta_time"].append([b, partner, k, dec,
                                                  cm.wrap_predict_delta_time(config, b, partner, k, decrease=dec)])
        out["plans"].append(rec)
    with open(os.path.join(HERE, f"{case}.json"), "w") as f:
        json.dump(out, f)
    print(f"[golden] {case}: {len(out['plans'])} plans written")


def main():
    if len(sys.argv) > 2 and sys.argv[1] == "--child":
        return child(sys.argv[2])
    for case in CASES:
        copy_db(case)
        subprocess.run([sys.executable, os.path.abspath(__file__), "--child", case], check=True,
                       stdout=subprocess.DEVNULL if os.environ.get("GOLDEN_QUIET") else None)
    # the single-GPU known-answer plans and the database files they index (data files)
    kat = os.path.join(HERE, "kat")
    os.makedirs(kat, exist_ok=True)
    eur = os.path.join(REF, "profiler/profiled-time-eurosys")
    for n in ["gpt_350M_mbs1_tp1_algo0.csv", "gpt_350M_mbs8_tp1_algo0.csv",
              "resnet_500M_mbs16_tp1_algo0.csv", "resnet_500M_mbs64_tp1_algo0.csv",
              "t5_770M_mbs1_tp1_algo0.csv", "t5_770M_mbs2_tp1_algo0.csv",
              "p2p_intra_node.csv", "p2p_inter_node.csv"] + \
             [f"prim_gpt_13B_{p}_{n}gpus.csv" for p in ("all_gather", "all_reduce", "reduce_scatter", "all_to_all") for n in (2, 4, 8)] + \
             [f"gpt_13B_mbs{m}_tp{t}_algo{a}.csv" for m in (1, 2, 4, 8) for t in (1, 2, 4, 8) for a in (0, 1)]:
        shutil.copyfile(os.path.join(eur, n), os.path.join(kat, n))
    for n in ["gpt_350M_mbs8_recomp.json", "resnet_500M_mbs64_recomp.json", "t5_770M_mbs2_recomp.json"]:
        shutil.copyfile(os.path.join(REF, "search/single_gpu_configs", n), os.path.join(kat, n))


if __name__ == "__main__":
    main()
