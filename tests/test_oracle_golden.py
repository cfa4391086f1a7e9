"""The oracle against vectors the reference itself produced (tests/golden/make_golden.py):
multi-stage, mixed tp/dp/algo/recompute plans on the reference's own profile databases.
Every float must be bit-identical (the oracle restates the same operations in the same order)."""
import json
import os

import pytest

from oracle.aceso_oracle import Oracle, Settings, get_config, get_full_op_list

CASES = ["gpt_1_3B", "resnet_500M", "t5_770M"]


def load_case(golden_dir, case):
    with open(os.path.join(golden_dir, f"{case}.json")) as f:
        g = json.load(f)
    st = Settings(model_name=g["model_name"], micro_batch_size=g["micro_batch_size"],
                  num_gpus_per_node=g["num_gpus_per_node"], memory_limit=g["memory_limit"])
    orc = Oracle(st)
    orc.read_profiled_time(g["model_name"], g["model_size"], os.path.join(golden_dir, f"db_{case}") + "/")
    full = get_full_op_list(g["model_name"], orc.op_list, g["num_layers"])
    assert len(full) == g["num_ops"]
    return g, orc, full


def make_config(g, p, full):
    return get_config(p["num_ops_in_each_stage"], p["tp"], p["dp"], p["recompute_ops"],
                      p["micro_batch_size"], g["global_batch_size"], full, p["algo"])


@pytest.mark.parametrize("case", CASES)
def test_predict_time_breakdown_bit_exact(golden_dir, case):
    g, orc, full = load_case(golden_dir, case)
    for p in g["plans"]:
        c = make_config(g, p, full)
        orc.predict_time_breakdown(c)
        for k in ["time_list", "memory_list", "compute_time_list", "total_gpu_time",
                  "breakdown_ideal_time_per_gpu", "breakdown_eff_loss_time_per_gpu",
                  "breakdown_recomp_time_per_gpu", "efficient_time_list"]:
            assert getattr(c, k) == p[k], k
        assert orc.get_reserved_memory_list(c) == p["reserved_memory_list"]


@pytest.mark.parametrize("case", CASES)
def test_stage_queries_bit_exact(golden_dir, case):
    g, orc, full = load_case(golden_dir, case)
    for p in g["plans"]:
        c = make_config(g, p, full)
        mbs = p["micro_batch_size"]
        for s, st in enumerate(c.stages):
            a = (st.ops, st.recompute_ops, st.tp_size, st.dp_size, mbs)
            assert orc.predict_stage_time(*a, st.algo) == p["stage_time"][s]
            got = [orc.predict_stage_time(*a, st.algo, delta=True, on_the_right=r, decrease=d)
                   for r in (False, True) for d in (False, True)]
            assert got == p["stage_time_delta"][s]
            assert orc.predict_stage_memory(*a, st.num_stages_behind, st.algo) == p["stage_memory"][s]
            assert list(orc.predict_stage_memory(*a, st.num_stages_behind, st.algo, breakdown=True)) == \
                p["stage_memory_breakdown"][s]


@pytest.mark.parametrize("case", CASES)
def test_recompute_and_moves_bit_exact(golden_dir, case):
    g, orc, full = load_case(golden_dir, case)
    n_nontrivial = 0
    for p in g["plans"]:
        c = make_config(g, p, full)
        mbs = p["micro_batch_size"]
        for s, st in enumerate(c.stages):
            rc = orc.check_recompute(st.ops, mbs, st.tp_size, st.dp_size, st.num_stages_behind, st.algo)
            assert rc == p["check_recompute"][s]
            n_nontrivial += int(sum(rc) > 0)
        for b, partner, k, metric, v, r in p["value_after_move"]:
            gv, gr = orc.predict_value_after_move(c, b, partner, k, metric)
            assert gv == v and list(gr) == r
        for b, partner, k, dec, v in p["delta_time"]:
            assert orc.wrap_predict_delta_time(c, b, partner, k, decrease=dec) == v
    assert n_nontrivial > 0, "golden set must exercise the greedy recompute loop"


def test_golden_exercises_resharding(golden_dir):
    """At least some GPT golden plans must have a non-zero resharding term, otherwise the
    fixtures would not pin get_op_spec / get_reshard_primitives / get_reshard_time."""
    g, orc, full = load_case(golden_dir, "gpt_1_3B")
    hits = 0
    for p in g["plans"]:
        c = make_config(g, p, full)
        for st in c.stages:
            mbs_list = [c.micro_bs // d for d in st.dp_size]
            orc.args.resharding = True
            with_r = orc.get_time_v3(st.ops, mbs_list, st.tp_size, st.algo, st.dp_size, False, False)
            orc.args.resharding = False
            without = orc.get_time_v3(st.ops, mbs_list, st.tp_size, st.algo, st.dp_size, False, False)
            orc.args.resharding = True
            hits += int(with_r[2] != without[2] or with_r[3] != without[3])
    assert hits >= 8


# ---- the reference's non-default switches (tests/golden/variants, written by the reference) ------
VARIANT_SETTINGS = {
    "min": dict(memory_pred_type="MIN"),
    "collmem": dict(consider_collective_memory=True),
    "min_collmem": dict(memory_pred_type="MIN", consider_collective_memory=True),
    "noshared": dict(consider_shared_space=False),
    "noreserved": dict(consider_reserved_space=False),
    "noflex": dict(flex_recompute=False),
    "peakbwd": dict(peak_mem_in_backward=700),
}


def variant_files(golden_dir):
    d = os.path.join(golden_dir, "variants")
    return sorted(f[:-5] for f in os.listdir(d) if f.endswith(".json"))


def load_variant(golden_dir, name):
    case, variant = name.split("__")
    with open(os.path.join(golden_dir, "variants", f"{name}.json")) as f:
        g = json.load(f)
    st = Settings(model_name=g["model_name"], micro_batch_size=g["micro_batch_size"],
                  num_gpus_per_node=g["num_gpus_per_node"], memory_limit=g["memory_limit"], **VARIANT_SETTINGS[variant])
    orc = Oracle(st)
    orc.read_profiled_time(g["model_name"], g["model_size"], os.path.join(golden_dir, f"db_{case}") + "/")
    full = get_full_op_list(g["model_name"], orc.op_list, g["num_layers"])
    return g, orc, full


ALL_VARIANTS = variant_files(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))


def test_every_switch_has_vectors():
    assert len(ALL_VARIANTS) == 19
    for case in CASES:
        for v in VARIANT_SETTINGS:
            assert f"{case}__{v}" in ALL_VARIANTS or (case == "t5_770M" and "collmem" in v)


@pytest.mark.parametrize("name", ALL_VARIANTS)
def test_non_default_switches_bit_exact(golden_dir, name):
    g, orc, full = load_variant(golden_dir, name)
    _, plain, _ = load_case(golden_dir, name.split("__")[0])       # default switches: pinned by the base vectors
    differs = 0
    for p in g["plans"]:
        c = make_config(g, p, full)
        orc.predict_time_breakdown(c)
        for k in ["time_list", "memory_list", "efficient_time_list"]:
            assert getattr(c, k) == p[k], k
        assert orc.get_reserved_memory_list(c) == p["reserved_memory_list"]
        mbs = p["micro_batch_size"]
        for s, st in enumerate(c.stages):
            assert list(orc.predict_stage_memory(st.ops, st.recompute_ops, st.tp_size, st.dp_size, mbs,
                                                 st.num_stages_behind, st.algo, breakdown=True)) == p["stage_memory_breakdown"][s]
            assert orc.check_recompute(st.ops, mbs, st.tp_size, st.dp_size, st.num_stages_behind, st.algo) == p["check_recompute"][s]
        for b, partner, k, metric, v, r in p["value_after_move"]:
            gv, gr = orc.predict_value_after_move(c, b, partner, k, metric)
            assert gv == v and list(gr) == r
        c0 = make_config(g, p, full)
        plain.predict_time_breakdown(c0)
        rc0 = [plain.check_recompute(st.ops, mbs, st.tp_size, st.dp_size, st.num_stages_behind, st.algo) for st in c0.stages]
        differs += int(c0.memory_list != p["memory_list"] or rc0 != p["check_recompute"])
    # the switch must matter on these plans, or the vectors would pin nothing
    assert differs > 0, name


@pytest.mark.parametrize("case", CASES)
def test_value_after_gpu_move_bit_exact(golden_dir, case):
    """predict_value_after_move with inc_gpus / dec_gpus for dim tp and dp (aceso_cost_model.py:715-728)."""
    g, orc, full = load_case(golden_dir, case)
    n = 0
    for p in g["plans"]:
        c = make_config(g, p, full)
        for b, dim, inc, metric, v, r in p["value_after_gpu_move"]:
            gv, gr = orc.predict_value_after_move(c, b, None, 0, metric, inc_gpus=inc, dec_gpus=not inc, dim=dim)
            assert gv == v and list(gr) == r
            n += 1
    assert n > 20
