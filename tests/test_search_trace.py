"""The calls the reference's own search makes into its cost model, replayed on this one.

tests/golden/search_trace_<case>.json (tests/golden/make_golden.py, child_search_trace): search/aceso_search.py's
run_search for 2, 3 and 4 pipeline stages, a few trials each, with every call that aceso_search.py, aceso_prims.py and
aceso_policy.py made into aceso_cost_model recorded -- function, arguments, what came back, and for the two functions
that write into the plan (predict_time_breakdown, update_recompute) what they left there.  The plans and stages are the
ones real moves produce (one-op stages, stages after GPU moves, recompute lists of check_recompute's own making), the
argument forms the ones the callers use (positional and keyword).  Every recorded call must return the same here, to
the last bit, on the CPU build of the kernels and on the GPU.

The reference's two memo tables (stage memory, stage time) are keyed by a stage's first op NAME, its length and its
per-op lists, so in a model whose layers differ (T5: encoder and decoder) two different stages can share an entry, and
what check_recompute starts from then depends on what was asked before.  The fixture holds the entries each recorded
call hit (`memo`); the replay puts exactly those in place before the call."""
import json
import os

import pytest

from superscaler_amd.plan import get_config
from tests.test_cost_model_api import make_model
from tests.test_initial_plans import pack_runs

CASES = ["gpt_1_3B", "resnet_500M", "t5_770M"]
BREAKDOWN = ("time_list", "memory_list", "compute_time_list", "total_gpu_time", "efficient_time_list",
             "breakdown_ideal_time_per_gpu", "breakdown_eff_loss_time_per_gpu", "breakdown_recomp_time_per_gpu")


def decode(x, fx, m):
    """make_golden's `plain` undone: plans, op-name slices and run-length integer lists back to what the callers passed."""
    if isinstance(x, dict):
        if "config" in x:
            d = x["config"]
            flat = lambda runs: [v for v, n in runs for _ in range(n)]
            return get_config(d["num_ops_in_each_stage"], flat(d["tp"]), flat(d["dp"]), flat(d["recompute_ops"]),
                              d["micro_batch_size"], fx["global_batch_size"], m.graph.ops, flat(d["algo"]))
        if "ops" in x:
            return m.graph.ops[x["ops"][0]:x["ops"][0] + x["ops"][1]]
        if "runs" in x:
            return [v for v, n in x["runs"] for _ in range(n)]
        raise AssertionError(x)
    if isinstance(x, list):
        return [decode(v, fx, m) for v in x]
    return x


def plain_result(r):
    if isinstance(r, tuple):
        return [plain_result(v) for v in r]
    if isinstance(r, list):
        return [plain_result(v) for v in r]
    return r


def replay(golden_dir, case, backend, extras=False):
    with open(os.path.join(golden_dir, f"search_trace_{case}{'__extras' if extras else ''}.json")) as f:
        fx = json.load(f)
    g, m = make_model(golden_dir, case, backend)
    counts = {}
    bad = []
    try:
        for name, calls in fx["calls"].items():
            counts[name] = len(calls)
            for k, call in enumerate(calls):
                # the cost model's two memo tables as the reference had them for this call: the entries it hit
                m.stage_memory_set.clear()
                m.stage_time_set.clear()
                for e in call.get("memo", []):
                    lists = {key: [v for v, n in e[key] for _ in range(n)] for key in ("tp", "dp", "rc", "algo")}
                    key = f"ops{e['first']}{e['n']}tp{lists['tp']}dp{lists['dp']}rc{lists['rc']}algo{lists['algo']}bs{e['bs']}"
                    if e["kind"] == "memory":
                        m.stage_memory_set[key + f"stage{e['nsb']}"] = e["value"]
                    else:
                        m.stage_time_set[key] = e["value"]
                args = decode(call["args"], fx, m)
                kwargs = {key: decode(v, fx, m) for key, v in call["kwargs"].items()}
                got = plain_result(getattr(m, name)(*args, **kwargs))
                want = decode(call["returns"], fx, m) if not isinstance(call["returns"], dict) or "config" not in call["returns"] \
                    else call["returns"]
                ok = got == want
                if name == "predict_time_breakdown":
                    ok = ok and all(getattr(args[0], key) == call["after"][key] for key in BREAKDOWN)
                if name == "update_recompute":
                    ok = ok and pack_runs(args[0]) == call["after"]
                if not ok:
                    bad.append((name, k))
    finally:
        if backend == "gpu":
            m.close()
    return counts, bad


def check(counts, bad, case):
    assert not bad, bad[:10]
    assert counts["predict_time_breakdown"] >= 30 and counts["update_recompute"] >= 30
    assert counts["predict_value_after_move"] >= 50 and counts["predict_stage_time_helper"] >= 60
    assert counts["check_recompute"] >= 30 and counts["predict_stage_time"] >= 30 and counts["predict_stage_memory"] >= 30


@pytest.mark.parametrize("extras", [False, True], ids=["default", "extras"])
@pytest.mark.parametrize("case", CASES)
def test_the_searchs_calls_return_what_the_reference_returned_emu(golden_dir, case, extras):
    counts, bad = replay(golden_dir, case, "emu", extras)
    check(counts, bad, case)
    if extras:           # (the optional actions and --predict-delta-time: see make_golden.TRACE_EXTRAS)
        assert counts["wrap_predict_delta_time"] >= 60


@pytest.mark.gpu
@pytest.mark.parametrize("extras", [False, True], ids=["default", "extras"])
@pytest.mark.parametrize("case", CASES)
def test_the_searchs_calls_return_what_the_reference_returned_gpu(golden_dir, case, extras):
    counts, bad = replay(golden_dir, case, "gpu", extras)
    check(counts, bad, case)


# ---- the searches over the binding: what they found, re-scored by today's code -------------------------------------
# tests/golden/make_golden.py (child_binding_search) ran the reference's unchanged aceso_search.py twice, once with its
# cost model module replaced by superscaler_amd/binding/aceso_cost_model.py (scoring through the CPU build of the kernel
# source) and once on its own cost model, and kept per stage count what each run returned (best time, its peak
# memory, explored plans) and the plan file each wrote (aceso_utils.py:137-211; per-op lists as runs).  Those runs need
# the reference's files and happen where the fixtures are written.  The tests below run today's code on the records:
# every kept plan is scored again -- CPU build of the kernels here, the library on the GPU -- and must give, to the
# last bit, the time and memory the REFERENCE's cost model gave for that plan file (child_score_plans:
# "plan_scores_by_the_reference"), for the plan the binding's search wrote and for the one the reference's own wrote.
# (The number a search returns is the best time it saw; with the fine-tuning actions on, the plan it writes can be
# another one, so the returned numbers are compared between the two runs and the plans are compared by their scores.)

SWEEP_SETTINGS = {
    "extras": {}, "stages1568": {}, "imbgpu": {}, "imbop": {},
    "min": dict(memory_pred_type="MIN"), "noflex": dict(flex_recompute=False), "peakbwd": dict(peak_mem_in_backward=700),
    "noreserved": dict(consider_reserved_space=False), "noshared": dict(consider_shared_space=False),
    "collmem": dict(consider_collective_memory=True),
}
# (model, size, database directory under tests/golden, micro-batch sizes, gpus per node, global batch, memory limit, layers)
BINDING_CASES = {
    "gpt_1_3B": ("gpt", "1_3B", "db_gpt_1_3B", [1, 2, 4, 8], 4, 512, 12000, 24),
    "resnet_500M": ("resnet", "500M", "db_resnet_500M", [32, 64], 4, 768, 12000, None),
    "t5_770M": ("t5", "770M", "db_t5_770M", [1, 2, 4, 8], 4, 512, 9000, 24),
    "gpt_13B": ("gpt", "13B", "kat", [1, 2, 4, 8], 8, 1024, 28000, 40),
}


def binding_model(golden_dir, case, backend, **settings):
    from superscaler_amd import aceso_cost_model as acm
    from superscaler_amd.profile_db import CostModelSettings
    from tests.helpers import EmuEvaluator
    model, size, db, mbs, gpn, gbs, limit, layers = BINDING_CASES[case]
    st = CostModelSettings(model_name=model, micro_batch_size=mbs, num_gpus_per_node=gpn, global_batch_size=gbs,
                           memory_limit=limit, **settings)
    m = acm.CostModel.from_directory(st, model, size, os.path.join(golden_dir, db) + "/", num_layers=layers)
    if backend == "emu":
        m._evaluator = EmuEvaluator(m.tables)
    return m


def rescore(m, fx):
    """Scores every plan the record keeps; returns how many, after checking each against the recorded numbers."""
    from superscaler_amd.plan import config_from_json
    n = 0
    for side, numbers in (("best_plan_with_the_binding", "with_the_binding"),
                          ("best_plan_with_the_reference_cost_model", "with_the_reference_cost_model")):
        for stages, plan in fx[side].items():
            want = fx["plan_scores_by_the_reference"][side][stages]
            assert (plan is None) == (want is None) == (fx[numbers][stages] is None), (side, stages)
            if plan is None:
                continue
            assert plan["per_op_lists_as_runs"] and plan["num_stages"] == int(stages)
            d = dict(plan)
            for key in ("model_parallel_size_of_each_op", "data_parallel_size_of_each_op", "recompute_ops", "algo_of_each_op"):
                d[key] = [[v for v, k in runs for _ in range(k)] for runs in plan[key]]
            c = config_from_json(d, m.graph.ops)
            m.predict_time_breakdown(c)
            assert [max(c.time_list), max(c.memory_list)] == want, (side, stages)
            n += 1
    return n


def check_record(golden_dir, name, backend, case=None, **settings):
    with open(os.path.join(golden_dir, f"search_binding_{name}.json")) as f:
        fx = json.load(f)
    m = binding_model(golden_dir, case or fx["case"], backend, **settings)
    try:
        n = rescore(m, fx)
    finally:
        if backend == "gpu":
            m.close()
    # the two searches returned the same numbers after the same number of explored plans, and wrote the same plan files
    assert fx["with_the_binding"] == fx["with_the_reference_cost_model"], name
    assert fx["best_plan_with_the_binding"] == fx["best_plan_with_the_reference_cost_model"], name
    assert fx["explored_with_the_binding"] == fx["explored_with_the_reference_cost_model"], name
    return fx, n


def _found_the_same_plans(golden_dir, case, backend):
    fx, n = check_record(golden_dir, case, backend)
    assert set(fx["with_the_binding"]) == {"2", "3", "4"} and n == 6
    assert all(v is not None and v[0] > 0 for v in fx["with_the_binding"].values())
    assert all(k >= 4 for k in fx["explored_with_the_binding"].values())
    if case == "gpt_1_3B":
        # search/gen_megatron_plan.py, run as the script it is over the binding, wrote the plan files it writes with
        # the reference's own cost model (child_binding_grid)
        assert fx["grid_files_identical"] is True and len(fx["grid_files_with_the_binding"]) == 4
        assert fx["grid_files_with_the_binding"] == fx["grid_files_with_the_reference_cost_model"]


@pytest.mark.parametrize("case", CASES)
def test_the_references_search_over_the_binding_found_the_same_plans(golden_dir, case):
    _found_the_same_plans(golden_dir, case, "emu")
    # aceso_search.py:4, aceso_prims.py:7, gen_megatron_plan.py:8 import these names from aceso_cost_model
    wanted = {"read_profiled_time", "predict_time_breakdown", "update_recompute", "get_reserved_memory_list",
              "wrap_predict_delta_time", "predict_stage_time_helper", "predict_value_after_move", "check_recompute",
              "predict_stage_time", "predict_stage_memory"}
    import ast
    import superscaler_amd
    path = os.path.join(os.path.dirname(superscaler_amd.__file__), "binding", "aceso_cost_model.py")
    with open(path) as f:
        tree = ast.parse(f.read())
    exported = {a.asname or a.name for node in ast.walk(tree) if isinstance(node, ast.ImportFrom) for a in node.names}
    assert wanted <= exported
    import superscaler_amd.aceso_cost_model as api
    assert all(callable(getattr(api, name)) for name in exported - {"parse_args"})


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES)
def test_the_references_search_over_the_binding_found_the_same_plans_gpu(golden_dir, case):
    _found_the_same_plans(golden_dir, case, "gpu")


def _long_search(golden_dir, case, backend):
    """The same comparison at ten times the length: 40 trials of up to 7 hops (the hop count of the reference's own
    search scripts), both runs made by the fixture generator at that length (GOLDEN_TRIALS=40 GOLDEN_HOPS=7)."""
    fx, n = check_record(golden_dir, f"{case}__long", backend)
    assert fx["flags"][fx["flags"].index("--max-num-trials") + 1] == "40" and fx["flags"][fx["flags"].index("--max-num-hops") + 1] == "7"
    assert set(fx["with_the_binding"]) == {"2", "3", "4"} and n == 6
    assert all(k >= 20 for k in fx["explored_with_the_binding"].values())


@pytest.mark.parametrize("case", CASES)
def test_the_long_search_over_the_binding_found_the_same_plans(golden_dir, case):
    _long_search(golden_dir, case, "emu")


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES)
def test_the_long_search_over_the_binding_found_the_same_plans_gpu(golden_dir, case):
    _long_search(golden_dir, case, "gpu")


def _further_settings(golden_dir, backend):
    """The same comparison (short searches) under the reference's other settings: the optional actions with the
    delta-time prediction, MIN memory prediction, no flex recompute, a backward peak, no reserved / no shared space,
    collective memory, 1 / 5 / 6 / 8 stages, the other starting points (make_golden.BINDING_SWEEPS): 27 records, each
    with the same best plans and the same number of explored plans on both sides; every plan re-scored under the
    record's settings."""
    import glob
    files = sorted(glob.glob(os.path.join(golden_dir, "search_binding_*__sweep_*.json")))
    assert len(files) == 27
    names, plans = set(), 0
    for path in files:
        name = os.path.basename(path)[len("search_binding_"):-5]
        sweep = name.split("__sweep_")[1]
        names.add(sweep)
        fx, n = check_record(golden_dir, name, backend, **SWEEP_SETTINGS[sweep])
        assert n >= 2, path
        plans += n
    assert names == set(SWEEP_SETTINGS) and plans >= 140


def test_the_search_over_the_binding_under_further_settings(golden_dir):
    _further_settings(golden_dir, "emu")


@pytest.mark.gpu
def test_the_search_over_the_binding_under_further_settings_gpu(golden_dir):
    _further_settings(golden_dir, "gpu")


def _on_32_gpus(golden_dir, backend):
    """GPT-13B (523 ops) on 4 nodes of 8 GPUs -- tensor parallelism up to 8, stages across node boundaries -- with 4, 5, 6, 8
    and 16 pipeline stages, 8 trials of up to 5 hops: same best plans and same number of explored plans (437 to 17,270)
    over the binding as with the reference's own cost model; the ten plans re-scored."""
    fx, n = check_record(golden_dir, "gpt_13B__big", backend)
    assert set(fx["with_the_binding"]) == {"4", "5", "6", "8", "16"} and n == 10
    assert all(v is not None and v[1] <= 28000 for v in fx["with_the_binding"].values())
    assert max(fx["explored_with_the_binding"].values()) > 10000


def test_the_search_over_the_binding_on_32_gpus(golden_dir):
    _on_32_gpus(golden_dir, "emu")


@pytest.mark.gpu
def test_the_search_over_the_binding_on_32_gpus_gpu(golden_dir):
    _on_32_gpus(golden_dir, "gpu")
