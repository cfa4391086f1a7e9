"""The search's starting plans and the cost model's command line against what the reference produced.

tests/golden/initial_<case>.json: what generate_initial_config (search/aceso_utils.py:537-721) returned for its four
built-in starting points, 1 to 8 stages, both --init-dim values and both settings of flex recompute -- a plan, None, or
the exception it ended with.  tests/golden/main_<case>.json: standard output and --save-to-csv file of
search/aceso_cost_model.py run as a script (:926-932) on plan files (the ones gen_megatron_plan.py wrote, the
reference's single-GPU plans, and seeded multi-stage plans with resharding).  Both written by
tests/golden/make_golden.py."""
import json
import os
import types

import pytest

from superscaler_amd import initial_plans
from tests.test_cost_model_api import make_model

CASES = ["gpt_1_3B", "resnet_500M", "t5_770M"]


def pack_runs(config):
    """The form the fixture holds (make_golden.pack_plan_runs): per-op values as [value, count] runs over all stages, as
    the stage objects hold them (the reference's imbalance_op start keeps per-op lists longer than a short model's op
    list; that is compared as it is)."""
    def runs(key):
        out = []
        for st in config.stages:
            for x in getattr(st, key):
                if out and out[-1][0] == int(x):
                    out[-1][1] += 1
                else:
                    out.append([int(x), 1])
        return out
    return {"num_ops_in_each_stage": [len(st.ops) for st in config.stages], "tp": runs("tp_size"), "dp": runs("dp_size"),
            "recompute_ops": runs("recompute_ops"), "algo": runs("algo"), "micro_batch_size": config.micro_bs,
            "num_gpus": [st.num_gpus for st in config.stages]}


@pytest.mark.parametrize("case", CASES)
def test_initial_plans_are_the_references(golden_dir, case):
    with open(os.path.join(golden_dir, f"initial_{case}.json")) as f:
        fx = json.load(f)
    g, m = make_model(golden_dir, case, "emu")
    ops = m.graph.ops
    seen = {"plan": 0, "none": 0, "error": 0}
    for point, init_dim, flex, num_stages, want in fx["plans"]:
        args = types.SimpleNamespace(num_gpus=fx["num_nodes"] * fx["num_gpus_per_node"], global_batch_size=fx["global_batch_size"],
                                     micro_batch_size=fx["micro_batch_size"], max_tp=fx["max_tp"], flex_recompute=flex,
                                     init_dim=init_dim, model_name=fx["model_name"], num_layers=fx["num_layers"],
                                     initial_point=point)
        label = (point, init_dim, flex, num_stages)
        if want is not None and "error" in want:
            with pytest.raises(Exception) as e:
                initial_plans.generate_initial_config(num_stages, args, ops)
            assert type(e.value).__name__ == want["error"], label
            seen["error"] += 1
            continue
        got = m.generate_initial_config(num_stages, args)
        if want is None:
            assert got is None, label
            seen["none"] += 1
            continue
        seen["plan"] += 1
        assert pack_runs(got) == want, label
    assert seen["plan"] >= 28 and seen["none"] >= 6
    if case != "gpt_1_3B":
        assert seen["error"] >= 4


def test_sort_configs_orders_like_the_reference(golden_dir):
    from superscaler_amd.plan import sort_configs
    with open(os.path.join(golden_dir, "initial_gpt_1_3B.json")) as f:
        fx = json.load(f)
    assert len(fx["sort"]) == 4
    for rec in fx["sort"]:
        objs = [types.SimpleNamespace(time_list=t, total_gpu_time=g, k=k)
                for k, (t, g) in enumerate(zip(rec["time_list"], rec["total_gpu_time"]))]
        assert [o.k for o in sort_configs(objs, "max_stage_time")] == rec["max_stage_time"]
        assert [o.k for o in sort_configs(objs, "total_gpu_time")] == rec["by_total_gpu_time"]
    with pytest.raises(RuntimeError):
        sort_configs([], "other")


def run_command_line(golden_dir, case, backend, tmp_path, capsys, monkeypatch):
    from superscaler_amd import aceso_cost_model as api
    with open(os.path.join(golden_dir, f"main_{case}.json")) as f:
        fx = json.load(f)
    g, _ = make_model(golden_dir, case, "emu")
    if backend == "emu":
        # the command line builds its own model: give it the CPU emulation of the kernels instead of the GPU library
        from tests.helpers import EmuEvaluator

        def emu_of(self):
            if "_emu" not in self.__dict__:
                self.__dict__["_emu"] = EmuEvaluator(self.tables)
            return self.__dict__["_emu"]
        monkeypatch.setattr(api.CostModel, "evaluator", property(emu_of))
    for run in fx["runs"]:
        plan_file = tmp_path / run["plan_file"]
        plan_file.write_text(json.dumps(run["plan"]))
        csv_file = tmp_path / "out.csv"
        single = run["single_gpu"]
        argv = ["--num-nodes", "1" if single else str(g["num_nodes"]), "--num-gpus-per-node", "1" if single else str(g["num_gpus_per_node"]),
                "--global-batch-size", str(g["global_batch_size"]), "--memory-limit", str(g["memory_limit"]),
                "--profiled-time-path", os.path.join(golden_dir, f"db_{case}") + "/", "--micro-batch-size"] + \
               [str(x) for x in g["micro_batch_size"]] + ["--initial-point", str(plan_file), "--save-to-csv", str(csv_file)]
        if isinstance(run["plan"].get("num_layers"), int):
            argv += ["--num-layers", str(run["plan"]["num_layers"])]
        capsys.readouterr()
        assert api.main(argv) == 0
        out = capsys.readouterr().out
        assert out == run["stdout"], run["plan_file"]
        assert csv_file.read_text() == run["csv"], run["plan_file"]


@pytest.mark.parametrize("case", CASES)
def test_command_line_prints_and_saves_what_the_reference_does_emu(golden_dir, case, tmp_path, capsys, monkeypatch):
    run_command_line(golden_dir, case, "emu", tmp_path, capsys, monkeypatch)


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES)
def test_command_line_prints_and_saves_what_the_reference_does_gpu(golden_dir, case, tmp_path, capsys, monkeypatch):
    run_command_line(golden_dir, case, "gpu", tmp_path, capsys, monkeypatch)
