"""The drop-in module (superscaler_amd/aceso_cost_model.py) against the vectors the reference
wrote for the same calls (tests/golden/*.json): every list predict_time_breakdown fills, the
single-stage queries and their delta variants, the greedy recompute pass, what-if moves.

Two backends run the same assertions: "gpu" goes through libace_eval.so on a real device;
"emu" (CPU suite) swaps the evaluator for the bounds-checked CPU build of the same kernel
source, so that the host-side logic of the module is covered without a GPU."""
import json
import os

import numpy as np
import pytest

from superscaler_amd import aceso_cost_model as acm
from superscaler_amd.plan import get_config
from superscaler_amd.profile_db import CostModelSettings
from tests.helpers import EmuEvaluator, emu_score

CASES = ["gpt_1_3B", "resnet_500M", "t5_770M"]


def make_model(golden_dir, case, backend, variant=None):
    from tests.test_oracle_golden import VARIANT_SETTINGS
    name = f"{case}.json" if variant is None else os.path.join("variants", f"{case}__{variant}.json")
    with open(os.path.join(golden_dir, name)) as f:
        g = json.load(f)
    st = CostModelSettings(model_name=g["model_name"], micro_batch_size=g["micro_batch_size"],
                           num_gpus_per_node=g["num_gpus_per_node"], global_batch_size=g["global_batch_size"],
                           memory_limit=g["memory_limit"], **(VARIANT_SETTINGS[variant] if variant else {}))
    m = acm.CostModel.from_directory(st, g["model_name"], g["model_size"],
                                     os.path.join(golden_dir, f"db_{case}") + "/", num_layers=g["num_layers"])
    if backend == "emu":
        m._evaluator = EmuEvaluator(m.tables)
    else:
        import torch
        assert torch.cuda.is_available()
    return g, m


def cfg_of(g, m, p):
    return get_config(p["num_ops_in_each_stage"], p["tp"], p["dp"], p["recompute_ops"], p["micro_batch_size"],
                      g["global_batch_size"], m.graph.ops, p["algo"])


def _run_all(g, m):
    cfgs = [cfg_of(g, m, p) for p in g["plans"]]
    # batched entry point: one launch for all plans
    m.predict_time_breakdown_batch(cfgs)
    for c, p in zip(cfgs, g["plans"]):
        for k in ["time_list", "memory_list", "compute_time_list", "total_gpu_time", "breakdown_ideal_time_per_gpu",
                  "breakdown_eff_loss_time_per_gpu", "breakdown_recomp_time_per_gpu", "efficient_time_list"]:
            assert getattr(c, k) == p[k], k
    # single-plan entry point gives the same
    c0 = cfg_of(g, m, g["plans"][0])
    m.predict_time_breakdown(c0)
    assert c0.time_list == g["plans"][0]["time_list"] and c0.efficient_time_list == g["plans"][0]["efficient_time_list"]
    for c, p in list(zip(cfgs, g["plans"]))[:6]:
        mbs = p["micro_batch_size"]
        assert m.get_reserved_memory_list(c) == p["reserved_memory_list"]
        for s, st in enumerate(c.stages):
            a = (st.ops, st.recompute_ops, st.tp_size, st.dp_size, mbs)
            assert m.predict_stage_time(*a, st.algo) == p["stage_time"][s]
            got = [m.predict_stage_time(*a, st.algo, delta=True, on_the_right=r, decrease=d)
                   for r in (False, True) for d in (False, True)]
            assert got == p["stage_time_delta"][s]
            assert m.predict_stage_memory(*a, st.num_stages_behind, st.algo) == p["stage_memory"][s]
            assert list(m.predict_stage_memory(*a, st.num_stages_behind, st.algo, breakdown=True)) == p["stage_memory_breakdown"][s]
            assert m.check_recompute(st.ops, mbs, st.tp_size, st.dp_size, st.num_stages_behind, st.algo) == p["check_recompute"][s]
        for b, partner, k, metric, v, r in p["value_after_move"]:
            gv, gr = m.predict_value_after_move(c, b, partner, k, metric)
            assert gv == v and list(gr) == r
        for b, partner, k, dec, v in p["delta_time"]:
            assert m.wrap_predict_delta_time(c, b, partner, k, decrease=dec) == v
    # the lockstep batched greedy pass gives the same lists as the one-by-one calls
    qs, want = [], []
    for c, p in list(zip(cfgs, g["plans"]))[:8]:
        for s, st in enumerate(c.stages):
            qs.append((st.ops, p["micro_batch_size"], st.tp_size, st.dp_size, st.num_stages_behind, st.algo))
            want.append(p["check_recompute"][s])
    assert m.check_recompute_batch(qs) == want
    cs = [cfg_of(g, m, p) for p in g["plans"][:4]]
    m.update_recompute_batch(cs)
    assert [[st.recompute_ops for st in c.stages] for c in cs] == [p["check_recompute"] for p in g["plans"][:4]]
    # update_recompute rewrites the stages' recompute lists with check_recompute's answer
    c = cfg_of(g, m, g["plans"][1])
    m.update_recompute(c)
    assert [st.recompute_ops for st in c.stages] == g["plans"][1]["check_recompute"]


def _check_arrays_recompute(g, m):
    """update_recompute on encoded plans reproduces the reference's check_recompute for every stage."""
    cfgs = [cfg_of(g, m, p) for p in g["plans"]]
    batch = m.encode(cfgs)
    out = m.update_recompute_arrays(batch)
    assert np.array_equal(out.hdr, batch.hdr) and np.array_equal(out.codes & 0xF7, batch.codes & 0xF7)
    for k, p in enumerate(g["plans"]):
        got = out.to_config(k, m.tables)
        assert [st.recompute_ops for st in got.stages] == p["check_recompute"]


@pytest.mark.parametrize("case", CASES)
def test_recompute_arrays_match_reference_emu(golden_dir, case):
    g, m = make_model(golden_dir, case, "emu")
    _check_arrays_recompute(g, m)


@pytest.mark.parametrize("name,limit", [("gpt3_1_3b", 9000.0), ("t5_770m", 6000.0), ("wresnet_1b", 1500.0)])
def test_recompute_arrays_match_the_staged_loop(name, limit):
    """On synthetic plans far above the memory limit (many greedy rounds, partial groups) the
    array form equals check_recompute_batch, which the reference's own vectors pin."""
    import dataclasses
    from superscaler_amd import synth
    w = synth.WORKLOADS[name]
    graph = synth.make_graph(w)
    st = dataclasses.replace(synth.make_settings(w), memory_limit=limit)
    m = acm.CostModel(st, synth.make_db(w, graph), graph)
    m._evaluator = EmuEvaluator(m.tables)
    batch = synth.make_plans(w, m.tables, n_plans=24, seed_offset=5)
    out = m.update_recompute_arrays(batch)
    rounds = 0
    for k in range(batch.n_plans):
        c = batch.to_config(k, m.tables)
        qs = [(s.ops, c.micro_bs, s.tp_size, s.dp_size, s.num_stages_behind, s.algo) for s in c.stages]
        want = m.check_recompute_batch(qs)
        got = [s.recompute_ops for s in out.to_config(k, m.tables).stages]
        assert got == want
        rounds += sum(1 for r in want if 0 < sum(r) < len(r))
    assert rounds > 10, "the limit should force partial recomputation in many stages"


@pytest.mark.parametrize("name,limits", [("gpt3_1_3b", (20000.0, 9000.0, 3000.0)), ("wresnet_1b", (4000.0, 1500.0, 600.0)),
                                         ("gpt3_13b", (60000.0, 30000.0))])
def test_check_recompute_equals_the_oracles_loop(name, limits):
    """check_recompute evaluates several greedy rounds ahead in one launch and replays the reference's
    bookkeeping over the records; the oracle runs the reference's loop round by round.  Limits from
    mild (few whole groups) to harsh (every group, prefixes, stages that cannot be brought under it)."""
    import dataclasses
    from superscaler_amd import synth
    from tests.helpers import oracle_for
    w = synth.WORKLOADS[name]
    graph = synth.make_graph(w)
    launches = 0
    for limit in limits:
        st = dataclasses.replace(synth.make_settings(w), memory_limit=limit)
        m = acm.CostModel(st, synth.make_db(w, graph), graph)
        ev = EmuEvaluator(m.tables)
        calls = []
        score = ev.score_host
        ev.score_host = lambda *a, **k: (calls.append(1), score(*a, **k))[1]
        m._evaluator = ev
        orc = oracle_for(m.tables)
        batch = synth.make_plans(w, m.tables, n_plans=6, seed_offset=31)
        kinds = set()
        for k in range(batch.n_plans):
            c = batch.to_config(k, m.tables)
            qs = [(s.ops, c.micro_bs, s.tp_size, s.dp_size, s.num_stages_behind, s.algo) for s in c.stages]
            want = [orc.check_recompute(*q) for q in qs]
            assert m.check_recompute_batch(qs) == want
            assert [m.check_recompute(*q) for q in qs[:2]] == want[:2]
            kinds |= {"none" if not any(r) else "all" if all(r) else "some" for r in want}
        launches += len(calls)
        assert "some" in kinds or "all" in kinds
    assert launches > 0


@pytest.mark.parametrize("case", CASES)
def test_api_matches_reference_emu(golden_dir, case):
    g, m = make_model(golden_dir, case, "emu")
    _run_all(g, m)


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES)
def test_api_matches_reference_gpu(golden_dir, case):
    g, m = make_model(golden_dir, case, "gpu")
    try:
        _run_all(g, m)
        _check_arrays_recompute(g, m)
    finally:
        m.close()


def test_errors_match_reference_behaviour(golden_dir):
    g, m = make_model(golden_dir, "gpt_1_3B", "emu")
    p = g["plans"][0]
    c = cfg_of(g, m, p)
    c.micro_bs = 3                       # not a profiled micro-batch size -> KeyError (aceso_cost_model.py:25)
    with pytest.raises(KeyError):
        m.predict_time_breakdown(c)
    st = cfg_of(g, m, p).stages[0]
    with pytest.raises(KeyError):
        m.predict_stage_time(st.ops, st.recompute_ops, st.tp_size, st.dp_size, 3, st.algo)
    with pytest.raises(RuntimeError):
        m.predict_value_after_move(cfg_of(g, m, p), 0, 0, 0, "throughput")
    with pytest.raises(ValueError):
        m.predict_stage_time(["enc-MLP-gelu", "encoder-embedding"], [0, 0], [1, 1], [1, 1], 1, [0, 0])


@pytest.mark.gpu
def test_module_level_calls_as_the_reference_makes_them(golden_dir):
    """The way aceso_search.py / aceso_prims.py use the module (aceso_search.py:4, aceso_prims.py:7): an argparse
    namespace, read_profiled_time(), then the functions by name -- against the reference's own vectors."""
    import argparse
    with open(os.path.join(golden_dir, "gpt_1_3B.json")) as f:
        g = json.load(f)
    ns = argparse.Namespace(model_name=g["model_name"], model_size=g["model_size"], micro_batch_size=g["micro_batch_size"],
                            num_gpus_per_node=g["num_gpus_per_node"], num_nodes=g["num_nodes"],
                            global_batch_size=g["global_batch_size"], memory_limit=g["memory_limit"], max_tp=None,
                            num_layers=g["num_layers"], consider_shared_space=True, consider_reserved_space=True,
                            flex_recompute=True, peak_mem_in_backward=0, memory_pred_type="MAX", resharding=None,
                            consider_collective_memory=False, support_comm_predict=False)
    acm.configure(ns)
    try:
        n_types = acm.read_profiled_time(g["model_name"], g["model_size"], os.path.join(golden_dir, "db_gpt_1_3B") + "/")
        assert isinstance(n_types, int) and n_types == len(acm._m().db.op_names) > 0
        for p in g["plans"][:6]:
            c = cfg_of(g, acm._m(), p)
            assert acm.predict_time_breakdown(c) is None
            assert c.time_list == p["time_list"] and c.memory_list == p["memory_list"]
            assert acm.get_reserved_memory_list(c) == p["reserved_memory_list"]
            mbs = p["micro_batch_size"]
            for s, st in enumerate(c.stages):
                assert acm.predict_stage_time(st.ops, st.recompute_ops, st.tp_size, st.dp_size, mbs, st.algo) == p["stage_time"][s]
                assert acm.predict_stage_memory(st.ops, st.recompute_ops, st.tp_size, st.dp_size, mbs, st.num_stages_behind,
                                                st.algo) == p["stage_memory"][s]
                assert acm.check_recompute(st.ops, mbs, st.tp_size, st.dp_size, st.num_stages_behind, st.algo) == p["check_recompute"][s]
            for b, partner, k, metric, v, r in p["value_after_move"]:
                gv, gr = acm.predict_value_after_move(c, b, partner, k, metric)
                assert gv == v and list(gr) == r
            for b, partner, k, dec, v in p["delta_time"]:
                assert acm.wrap_predict_delta_time(c, b, partner, k, decrease=dec) == v
            acm.update_recompute(c)
            assert [st.recompute_ops for st in c.stages] == p["check_recompute"]
    finally:
        if acm._model is not None:
            acm._model.close()
        acm._model = None
        acm.args = None


def test_module_level_api_requires_configuration():
    acm._model = None
    with pytest.raises(RuntimeError):
        acm.predict_time_breakdown(None)


# ---- uniform plan grid (the batched form of search/gen_megatron_plan.py) -----------------------
def _grid_check(golden_dir, backend):
    from superscaler_amd.megatron_grid import best_uniform_plans, enumerate_grid
    from tests.helpers import oracle_for
    g, m = make_model(golden_dir, "gpt_1_3B", backend)
    try:
        num_gpus = g["num_nodes"] * g["num_gpus_per_node"]
        configs = enumerate_grid(m, num_gpus, g["num_layers"])
        assert len(configs) > 20
        got = best_uniform_plans(m, num_gpus, g["num_layers"], num_saved=5)
        # the reference's selection (gen_megatron_plan.py:101-135) on the oracle's numbers
        orc = oracle_for(m.tables)
        from oracle.aceso_oracle import get_config as oget
        feasible = {}
        for c in configs:
            flat = lambda key: [x for st in c.stages for x in getattr(st, key)]
            oc = oget([len(st.ops) for st in c.stages], flat("tp_size"), flat("dp_size"), flat("recompute_ops"),
                      c.micro_bs, c.global_bs, m.graph.ops, flat("algo"))
            orc.predict_time_breakdown(oc)
            t, mem = max(oc.time_list), max(oc.memory_list)
            if mem < g["memory_limit"]:
                if t not in feasible or mem < feasible[t]:
                    feasible[t] = mem
        want = [(t, feasible[t]) for t in sorted(feasible)[:5]]
        assert [(t, mem) for t, mem, _ in got] == want and len(want) > 0
    finally:
        m.close()


def test_uniform_grid_emu(golden_dir):
    _grid_check(golden_dir, "emu")


@pytest.mark.gpu
def test_uniform_grid_gpu(golden_dir):
    _grid_check(golden_dir, "gpu")


ATTRS = ["time_list", "memory_list", "compute_time_list", "total_gpu_time", "breakdown_ideal_time_per_gpu",
         "breakdown_eff_loss_time_per_gpu", "breakdown_recomp_time_per_gpu", "efficient_time_list"]


def _candidate_list_check(golden_dir, case, backend):
    """The search's candidate loop (aceso_search.py:121-145: every new config scored, the fastest one whose memory fits
    kept) with the candidates handed over in ONE call: predict_time_breakdown_batch fills every attribute
    predict_time_breakdown fills, with the same values, and the selection made from them is the same."""
    g, m = make_model(golden_dir, case, backend)
    try:
        one_by_one = [cfg_of(g, m, p) for p in g["plans"]]
        for c in one_by_one:
            m.predict_time_breakdown(c)
        batched = [cfg_of(g, m, p) for p in g["plans"]]
        m.predict_time_breakdown_batch(batched)
        for a, b in zip(one_by_one, batched):
            for k in ATTRS:
                assert getattr(a, k) == getattr(b, k), k

        def pick(configs, initial_time):
            best, best_t = None, initial_time
            for k, c in enumerate(configs):
                if max(c.time_list) < best_t and max(c.memory_list) <= g["memory_limit"]:
                    best, best_t = k, max(c.time_list)
            return best
        fits = [max(c.time_list) for c in one_by_one if max(c.memory_list) <= g["memory_limit"]]
        for t0 in [float("inf")] + sorted(fits)[1:3]:
            assert pick(one_by_one, t0) == pick(batched, t0)
        assert (pick(batched, float("inf")) is not None) == bool(fits)
    finally:
        m.close()


@pytest.mark.parametrize("case", CASES)
def test_candidate_list_in_one_call_emu(golden_dir, case):
    _candidate_list_check(golden_dir, case, "emu")


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES)
def test_candidate_list_in_one_call_gpu(golden_dir, case):
    _candidate_list_check(golden_dir, case, "gpu")


def _grid_files_check(golden_dir, backend, tmp_path):
    """The plan files the reference's own search/gen_megatron_plan.py wrote for the GPT-1.3B database
    (tests/golden/megatron_grid_gpt_1_3B.json, made by tests/golden/make_golden.py: run_grid): same file names (the
    truncated predicted time is part of them), same order, same JSON content."""
    from superscaler_amd import megatron_grid
    from superscaler_amd.plan import dump_config_to_json
    with open(os.path.join(golden_dir, "megatron_grid_gpt_1_3B.json")) as f:
        fx = json.load(f)
    g, m = make_model(golden_dir, "gpt_1_3B", backend)
    try:
        best = megatron_grid.best_uniform_plans(m, g["num_nodes"] * g["num_gpus_per_node"], fx["num_layers"], fx["num_of_saved_configs"])
        names = [f"{g['model_name']}_{g['model_size']}_{fx['num_layers']}layers_megatron_est_{int(t)}.json" for t, _, _ in best]
        assert names == sorted(fx["files"], key=lambda n: int(n.rsplit("_", 1)[1][:-5])) and len(names) == fx["num_of_saved_configs"]
        for name, (t, mem, cfg) in zip(names, best):
            path = str(tmp_path / name)
            dump_config_to_json(cfg, path, g["model_name"], g["model_size"], fx["num_layers"])
            with open(path) as f:
                assert json.load(f) == fx["files"][name], name
    finally:
        m.close()


def test_uniform_grid_writes_the_reference_files_emu(golden_dir, tmp_path):
    _grid_files_check(golden_dir, "emu", tmp_path)


@pytest.mark.gpu
def test_uniform_grid_writes_the_reference_files_gpu(golden_dir, tmp_path):
    _grid_files_check(golden_dir, "gpu", tmp_path)


@pytest.mark.gpu
def test_recompute_arrays_gpu_equals_cpu_build():
    """2,048 GPT-3 13B plans under a 40 GB cap: the array-form greedy loop gives the same bits whether
    its stage records come from the GPU or from the CPU build of the kernel source."""
    import dataclasses
    from superscaler_amd import synth
    w = synth.WORKLOADS["gpt3_13b"]
    graph = synth.make_graph(w)
    st = dataclasses.replace(synth.make_settings(w), memory_limit=40000.0)
    m = acm.CostModel(st, synth.make_db(w, graph), graph)
    try:
        batch = synth.make_plans(w, m.tables, n_plans=2048, seed_offset=9)
        on_gpu = m.update_recompute_arrays(batch, on_device=False)
        assert np.array_equal(on_gpu.codes, m.update_recompute_arrays(batch).codes)      # selection on the device
        real, m._evaluator = m._evaluator, EmuEvaluator(m.tables)
        on_cpu = m.update_recompute_arrays(batch)
        m._evaluator = real
        assert np.array_equal(on_gpu.codes, on_cpu.codes)
        frac = (on_gpu.codes & 8).astype(bool).mean()
        assert 0.1 < frac < 0.9
    finally:
        m.close()


@pytest.mark.gpu
def test_uniform_grid_command_line(golden_dir, tmp_path, capsys):
    """`python -m superscaler_amd.megatron_grid` on the reference's GPT-1.3B database: writes plan JSON
    files the loader reads back, best first, and the best one is what best_uniform_plans returns."""
    from superscaler_amd import megatron_grid
    from superscaler_amd.plan import config_from_json
    with open(os.path.join(golden_dir, "gpt_1_3B.json")) as f:
        g = json.load(f)
    argv = ["--model-name", g["model_name"], "--model-size", g["model_size"], "--num-layers", str(g["num_layers"]),
            "--global-batch-size", str(g["global_batch_size"]), "--micro-batch-size"] + [str(x) for x in g["micro_batch_size"]] + \
           ["--num-nodes", "2", "--num-gpus-per-node", str(g["num_gpus_per_node"]), "--memory-limit", str(g["memory_limit"]),
            "--profiled-time-path", os.path.join(golden_dir, "db_gpt_1_3B") + "/", "--config-save-path", str(tmp_path) + "/",
            "--num-of-saved-configs", "3"]
    assert megatron_grid.main(argv) == 0
    out = capsys.readouterr().out
    files = sorted(tmp_path.glob("*.json"))
    assert 1 <= len(files) <= 3 and "best_0" in out
    _, m = make_model(golden_dir, "gpt_1_3B", "gpu")
    try:
        want = megatron_grid.best_uniform_plans(m, 2 * g["num_gpus_per_node"], g["num_layers"], 3)
        assert len(want) == len(files)
        names = {f.name for f in files}
        for t, mem, cfg in want:
            assert f"gpt_{g['model_size']}_{g['num_layers']}layers_megatron_est_{int(t)}.json" in names
        best = config_from_json(str(tmp_path / f"gpt_{g['model_size']}_{g['num_layers']}layers_megatron_est_{int(want[0][0])}.json"), m.graph.ops)
        m.predict_time_breakdown(best)
        assert max(best.time_list) == want[0][0] and max(best.memory_list) == want[0][1]
    finally:
        m.close()


@pytest.mark.gpu
@pytest.mark.parametrize("name,limit", [("gpt3_1_3b", 9000.0), ("gpt3_13b", 40000.0), ("t5_770m", 6000.0), ("wresnet_1b", 1500.0)])
def test_recompute_on_the_device_equals_the_array_form(name, limit):
    """The greedy loop with its selection on the device (ace_recompute_groups / ace_recompute_select)
    sets exactly the bits the numpy form sets."""
    import dataclasses
    from superscaler_amd import synth
    w = synth.WORKLOADS[name]
    graph = synth.make_graph(w)
    st = dataclasses.replace(synth.make_settings(w), memory_limit=limit)
    m = acm.CostModel(st, synth.make_db(w, graph), graph)
    try:
        batch = synth.make_plans(w, m.tables, n_plans=1500, seed_offset=17)
        want = m.update_recompute_arrays(batch, on_device=False)
        d = m.update_recompute_device(m.evaluator.upload(batch))
        N, G = batch.num_ops, (batch.num_ops + 15) // 16
        got = d.codes.permute(1, 0, 2).reshape(batch.n_plans, G * 16).cpu().numpy()
        assert np.array_equal(got[:, :N], want.codes) and not got[:, N:].any()
        frac = (want.codes & 8).astype(bool).mean()
        assert 0.02 < frac < 0.98
    finally:
        m.close()


# ---- check_recompute on stages the greedy pass cannot help -------------------------------------
def _no_group_stages(m):
    """Stages with nothing to recompute (one op, ops the pass never picks) and ordinary ones, each under
    limits from "below the weights alone" to "fits anyway"."""
    ops = m.graph.ops
    N = len(ops)
    flags = m.graph.flags
    norc = [i for i in range(N) if int(flags[m._type_index[ops[i]]]) & acm.og.F_NO_RECOMPUTE]
    slices = [(0, 1), (0, 2), (N - 1, N), (N - 2, N), (1, 2), (1, 14), (0, 30)]
    for i in norc[:3]:
        slices.append((i, i + 1))
    # maximal runs of never-picked ops
    run_lo = None
    for i in range(N + 1):
        is_norc = i < N and i in set(norc)
        if is_norc and run_lo is None:
            run_lo = i
        if not is_norc and run_lo is not None:
            slices.append((run_lo, i))
            run_lo = None
    return sorted(set(slices))


def _check_no_group(name, backend):
    import dataclasses
    from superscaler_amd import synth
    from tests.helpers import oracle_for
    w = synth.WORKLOADS[name]
    graph = synth.make_graph(w)
    mbs = w.mbs_list[-1]
    for limit in (1.0, 200.0, 1e9):
        st = dataclasses.replace(synth.make_settings(w), memory_limit=limit)
        m = acm.CostModel(st, synth.make_db(w, graph), graph)
        if backend == "emu":
            m._evaluator = EmuEvaluator(m.tables)
        try:
            orc = oracle_for(m.tables)
            qs = []
            for lo, hi in _no_group_stages(m):
                n = hi - lo
                for nsb in (0, 3):
                    qs.append((graph.ops[lo:hi], mbs, [1] * n, [1] * n, nsb, [0] * n))
            want = [orc.check_recompute(*q) for q in qs]
            assert any(not any(r) for r in want)
            assert m.check_recompute_batch(qs) == want
            assert [m.check_recompute(*q) for q in qs[:6]] == want[:6]
            # the callers of the same path
            cfg = get_config([1, len(graph.ops) - 1], [1] * len(graph.ops), [1] * len(graph.ops), [0] * len(graph.ops),
                             mbs, w.global_batch, graph.ops, [0] * len(graph.ops))
            m.update_recompute(cfg, 0)
            assert cfg.stages[0].recompute_ops == orc.check_recompute(graph.ops[:1], mbs, [1], [1], 1, [0])
        finally:
            m.close()


@pytest.mark.parametrize("name", ["gpt3_1_3b", "wresnet_1b", "t5_770m"])
def test_check_recompute_without_a_recomputable_group_emu(name):
    """aceso_cost_model.py:822-872 returns the zero list for a stage above the limit in which no op group can be
    recomputed (a one-op stage, embedding / post-process ops only); so must every form of the call here."""
    _check_no_group(name, "emu")


@pytest.mark.gpu
def test_check_recompute_without_a_recomputable_group_gpu():
    _check_no_group("gpt3_1_3b", "gpu")


# ---- the reference's vectors for its non-default switches and for inc_gpus / dec_gpus moves ---------
from tests.test_oracle_golden import ALL_VARIANTS


def _run_variant(g, m):
    cfgs = [cfg_of(g, m, p) for p in g["plans"]]
    m.predict_time_breakdown_batch(cfgs)
    for c, p in zip(cfgs, g["plans"]):
        for k in ["time_list", "memory_list", "efficient_time_list"]:
            assert getattr(c, k) == p[k], k
        assert m.get_reserved_memory_list(c) == p["reserved_memory_list"]
        mbs = p["micro_batch_size"]
        for s, st in enumerate(c.stages):
            assert list(m.predict_stage_memory(st.ops, st.recompute_ops, st.tp_size, st.dp_size, mbs, st.num_stages_behind,
                                               st.algo, breakdown=True)) == p["stage_memory_breakdown"][s]
        for b, partner, k, metric, v, r in p["value_after_move"]:
            gv, gr = m.predict_value_after_move(c, b, partner, k, metric)
            assert gv == v and list(gr) == r
    qs = [(st.ops, p["micro_batch_size"], st.tp_size, st.dp_size, st.num_stages_behind, st.algo)
          for c, p in zip(cfgs, g["plans"]) for st in c.stages]
    assert m.check_recompute_batch(qs) == [r for p in g["plans"] for r in p["check_recompute"]]
    # the batch scorer (scores, flags) and the array form of update_recompute under the same switches
    it, pk, fe = m.score_batch(cfgs)
    assert list(it) == [max(p["time_list"]) for p in g["plans"]] and list(pk) == [max(p["memory_list"]) for p in g["plans"]]
    assert list(fe) == [int(max(p["memory_list"]) <= g["memory_limit"]) for p in g["plans"]]
    out = m.update_recompute_arrays(m.encode(cfgs))
    for k, p in enumerate(g["plans"]):
        assert [st.recompute_ops for st in out.to_config(k, m.tables).stages] == p["check_recompute"]


@pytest.mark.parametrize("name", ALL_VARIANTS)
def test_non_default_switches_match_reference_emu(golden_dir, name):
    g, m = make_model(golden_dir, *name.split("__")[:1], "emu", variant=name.split("__")[1])
    _run_variant(g, m)


@pytest.mark.gpu
@pytest.mark.parametrize("name", ALL_VARIANTS)
def test_non_default_switches_match_reference_gpu(golden_dir, name):
    g, m = make_model(golden_dir, *name.split("__")[:1], "gpu", variant=name.split("__")[1])
    try:
        _run_variant(g, m)
    finally:
        m.close()


def _run_gpu_moves(g, m):
    n = 0
    for p in g["plans"]:
        c = cfg_of(g, m, p)
        for b, dim, inc, metric, v, r in p["value_after_gpu_move"]:
            gv, gr = m.predict_value_after_move(c, b, None, 0, metric, inc_gpus=inc, dec_gpus=not inc, dim=dim)
            assert gv == v and list(gr) == r
            n += 1
    assert n > 20


@pytest.mark.parametrize("case", CASES)
def test_value_after_gpu_move_matches_reference_emu(golden_dir, case):
    g, m = make_model(golden_dir, case, "emu")
    _run_gpu_moves(g, m)


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES)
def test_value_after_gpu_move_matches_reference_gpu(golden_dir, case):
    g, m = make_model(golden_dir, case, "gpu")
    try:
        _run_gpu_moves(g, m)
    finally:
        m.close()


def test_record_cache_survives_its_own_eviction(golden_dir):
    """Single-stage records are kept by their queries' lists and the table is emptied when it has grown too large: a call
    some of whose queries are in the table and some not must get all its records also when the table is emptied on that
    call (the emptying once happened between the look-up and the read: KeyError in a long search)."""
    g, m = make_model(golden_dir, "resnet_500M", "emu")
    ops = m.graph.ops
    q = lambda lo, n, bit: (ops[lo:lo + n], [bit] * n, [1] * n, [1] * n, 32, 0, [0] * n)
    first = m._stage_records([q(3, 5, 0)])
    m._record_cache_max = 1
    both = m._stage_records([q(3, 5, 0), q(20, 7, 1)])             # one known, one new, table at its limit
    assert np.array_equal(both[0], first[0], equal_nan=True)
    more = m._stage_records([q(20, 7, 1), q(3, 5, 0), q(40, 4, 0), q(41, 4, 1)])
    assert np.array_equal(more[0], both[1], equal_nan=True) and np.array_equal(more[1], first[0], equal_nan=True)
    fresh = make_model(golden_dir, "resnet_500M", "emu")[1]
    assert np.array_equal(fresh._stage_records([q(40, 4, 0), q(41, 4, 1)]), more[2:], equal_nan=True)


def _scan_twice(m, cfg, stage, partner, metric, step=1):
    """The op migration's call pattern (aceso_prims.py:168-185): every op count from 0 up, then again from 0."""
    out = []
    for _ in range(2):
        for k in range(0, len(cfg.stages[stage].ops), step):
            value, rc = m.predict_value_after_move(cfg, stage, partner, k, metric)
            out.append((k, value, list(rc)))
    return out


def _scans_check(golden_dir, case, backend):
    """predict_value_after_move answers a scan over op counts from results evaluated ahead: values, recompute lists, the
    memo table and its counters must be those of the one-by-one path (look_ahead = 0), also where the table holds
    another stage's memory under a scanned stage's key (the reference's key collisions, forced here)."""
    g, plain = make_model(golden_dir, case, backend)
    _, ahead = make_model(golden_dir, case, backend)
    try:
        plain.look_ahead = 0
        assert ahead.look_ahead > 0
        for m in (plain, ahead):
            m.settings.memory_limit = g["memory_limit"] * 0.6                # most stages must recompute
        plans = [p for p in g["plans"] if len(p["num_ops_in_each_stage"]) > 1][:3]
        recomputing = 0
        for pi, p in enumerate(plans):
            cfg_a, cfg_b = cfg_of(g, plain, p), cfg_of(g, ahead, p)
            for stage, partner in ((0, 1), (1, 0)):
                for metric, step in (("time_with_efficiency", 1), ("memory", 1), ("time", 3)):
                    if pi == 1 and metric == "memory":
                        # a collision on the way: some scanned key already holds another start
                        st = cfg_a.stages[stage]
                        k = max(1, len(st.ops) // 2)
                        sl = slice(None, -k) if stage < partner else slice(k, None)
                        key = (f"ops{st.ops[sl][0]}{len(st.ops[sl])}tp{st.tp_size[sl]}dp{st.dp_size[sl]}rc{[0] * len(st.ops[sl])}"
                               f"algo{st.algo[sl]}bs{cfg_a.micro_bs}stage{st.num_stages_behind}")
                        for m in (plain, ahead):
                            m.stage_memory_set[key] = g["memory_limit"] * 0.9
                    want = _scan_twice(plain, cfg_a, stage, partner, metric, step)
                    got = _scan_twice(ahead, cfg_b, stage, partner, metric, step)
                    assert got == want, (case, pi, stage, partner, metric)
                    recomputing += sum(sum(rc) for _, _, rc in want)
                # the same scan with --predict-delta-time (aceso_prims.py:174-177): wrap_predict_delta_time per op count
                for decrease in (True, False):
                    for step in (1, 2):
                        counts = list(range(0, len(cfg_a.stages[stage].ops), step)) * 2
                        want_d = [plain.wrap_predict_delta_time(cfg_a, stage, partner, k, decrease) for k in counts]
                        got_d = [ahead.wrap_predict_delta_time(cfg_b, stage, partner, k, decrease) for k in counts]
                        assert got_d == want_d, (case, pi, stage, partner, decrease, step)
                    assert ahead.stage_memory_set == plain.stage_memory_set
                    assert (ahead.stage_memory_visit, ahead.stage_memory_hit) == (plain.stage_memory_visit, plain.stage_memory_hit)
        assert ahead.scan_ahead_used > 0 and plain.scan_ahead_used == 0
        assert ahead.scan_ahead_dropped > 0                    # the forced collision was met
        assert recomputing > 0                                 # and the limit did make stages recompute
    finally:
        plain.close()
        ahead.close()


@pytest.mark.parametrize("case", CASES)
def test_scans_over_op_counts_emu(golden_dir, case):
    _scans_check(golden_dir, case, "emu")


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES)
def test_scans_over_op_counts_gpu(golden_dir, case):
    _scans_check(golden_dir, case, "gpu")


def test_a_failing_evaluation_ahead_leaves_the_call_to_the_ordinary_path(golden_dir, monkeypatch):
    """Whatever evaluating later op counts raises must not surface in the call that only asked for an earlier one."""
    g, plain = make_model(golden_dir, "gpt_1_3B", "emu")
    _, ahead = make_model(golden_dir, "gpt_1_3B", "emu")
    plain.look_ahead = 0

    def boom(*a, **k):
        raise KeyError("a later op count's stage")
    monkeypatch.setattr(ahead, "_scan_ahead", boom)
    p = [p for p in g["plans"] if len(p["num_ops_in_each_stage"]) > 1][0]
    want = _scan_twice(plain, cfg_of(g, plain, p), 0, 1, "time")
    got = _scan_twice(ahead, cfg_of(g, ahead, p), 0, 1, "time")
    assert got == want and ahead.scan_ahead_used == 0
    assert ahead.stage_memory_set == plain.stage_memory_set


def test_t5_memo_collision_host_api_and_batched_forms(golden_dir):
    """The reference's memo table of stage memory is keyed by a stage's first op NAME, its length and its per-op lists
    (aceso_cost_model.py:743-767): in T5 an all-encoder stage and a stage of the same length that runs on into the
    decoder share a key.  check_recompute on the second one then starts from the first one's memory if that was asked
    about before -- in the reference and, with `reference_memo` (the default), here.  Without the table (and in the
    batched forms, which have none) every stage starts from its own memory.  This pins which answer each path gives."""
    g, m = make_model(golden_dir, "t5_770M", "emu")
    ops = m.graph.ops
    n, mbs = 120, 4
    A, B = ops[1:1 + n], ops[274:274 + n]
    assert A[0] == B[0] == "enc-1st-layernorm" and A != B and any(o.startswith("dec") for o in B)
    lists = ([1] * n, [1] * n, 1, [0] * n)              # tp, dp, stages behind, algo
    m.clear_memo()
    alone = m.check_recompute(B, mbs, *lists)
    m.clear_memo()
    first = m.check_recompute(A, mbs, *lists)
    after_a = m.check_recompute(B, mbs, *lists)          # same key as A: starts from A's memory
    assert sum(alone) == 46 and sum(after_a) == 118 and sum(first) == 116
    # the table switched off: history does not matter
    m.clear_memo()
    m.reference_memo = False
    assert m.check_recompute(A, mbs, *lists) == first and m.check_recompute(B, mbs, *lists) == alone
    m.reference_memo = True
    # the batched form without the table gives every stage its own answer whatever was asked before ...
    m.clear_memo()
    m.check_recompute(A, mbs, *lists)
    q = lambda o: (o, mbs) + lists
    assert m.check_recompute_batch([q(A), q(B)], memo=False) == [first, alone]
    # ... and with the table it is the one-by-one sequence
    m.clear_memo()
    assert m.check_recompute_batch([q(A), q(B)], memo=True) == [first, after_a]
    assert len(m.stage_memory_set) > 0
    m.clear_memo()
    assert len(m.stage_memory_set) == 0 and m.stage_memory_visit == 0
