"""`python -m superscaler_amd.run_reference <script> <flags>`: a search script that imports `aceso_cost_model` gets this
library's binding, with the script's own directory supplying `aceso_utils.parse_args` as the reference's does
(aceso_cost_model.py:5,10).  The script here is a stand-in written for the test (a few lines that load a database, score
recorded plans and print the results the way a caller would); the reference's real scripts run through the same launcher
where the fixtures are written (tests/golden/make_golden.py, child_binding_search / child_binding_grid)."""
import contextlib
import io
import json
import os
import sys
import textwrap

import pytest

from superscaler_amd import aceso_cost_model as acm
from superscaler_amd import run_reference
from tests.helpers import EmuEvaluator

UTILS = textwrap.dedent('''
    import argparse, sys
    def parse_args():
        ap = argparse.ArgumentParser()
        ap.add_argument("--model-name"); ap.add_argument("--model-size"); ap.add_argument("--num-layers", type=int)
        ap.add_argument("--micro-batch-size", type=int, nargs="+"); ap.add_argument("--global-batch-size", type=int)
        ap.add_argument("--num-nodes", type=int); ap.add_argument("--num-gpus-per-node", type=int)
        ap.add_argument("--memory-limit", type=float); ap.add_argument("--profiled-time-path"); ap.add_argument("--plans")
        a = ap.parse_args()
        a.max_tp = None; a.consider_shared_space = True; a.consider_reserved_space = True; a.flex_recompute = True
        a.peak_mem_in_backward = 0; a.memory_pred_type = "MAX"; a.resharding = None; a.consider_collective_memory = False
        return a
''')

SCRIPT = textwrap.dedent('''
    import json
    from aceso_utils import parse_args
    from aceso_cost_model import read_profiled_time, predict_time_breakdown, update_recompute, get_reserved_memory_list
    import aceso_cost_model
    from superscaler_amd.plan import get_config
    args = parse_args()
    read_profiled_time(args.model_name, args.model_size, args.profiled_time_path)
    ops = aceso_cost_model._gpu._m().graph.ops
    out = []
    for p in json.load(open(args.plans))["plans"][:5]:
        c = get_config(p["num_ops_in_each_stage"], p["tp"], p["dp"], p["recompute_ops"], p["micro_batch_size"],
                       args.global_batch_size, ops, p["algo"])
        predict_time_breakdown(c)
        reserved = get_reserved_memory_list(c)
        update_recompute(c)
        out.append([c.time_list, c.memory_list, reserved, [st.recompute_ops for st in c.stages]])
    if __name__ == "__main__":
        print(json.dumps(out))
''')


def _run(golden_dir, tmp_path, monkeypatch, emu):
    case = "gpt_1_3B"
    with open(os.path.join(golden_dir, f"{case}.json")) as f:
        g = json.load(f)
    (tmp_path / "aceso_utils.py").write_text(UTILS)
    (tmp_path / "my_search.py").write_text(SCRIPT)
    if emu:
        def emu_of(self):
            if "_emu" not in self.__dict__:
                self.__dict__["_emu"] = EmuEvaluator(self.tables)
            return self.__dict__["_emu"]
        monkeypatch.setattr(acm.CostModel, "evaluator", property(emu_of))
    monkeypatch.setattr(sys, "argv", list(sys.argv))
    monkeypatch.setattr(sys, "path", list(sys.path))
    saved = {k: sys.modules.get(k) for k in ("aceso_cost_model", "aceso_utils")}
    argv = [str(tmp_path / "my_search.py"), "--model-name", g["model_name"], "--model-size", g["model_size"], "--num-layers",
            str(g["num_layers"]), "--micro-batch-size", *map(str, g["micro_batch_size"]), "--global-batch-size",
            str(g["global_batch_size"]), "--num-nodes", str(g["num_nodes"]), "--num-gpus-per-node", str(g["num_gpus_per_node"]),
            "--memory-limit", str(g["memory_limit"]), "--profiled-time-path", os.path.join(golden_dir, f"db_{case}") + "/",
            "--plans", os.path.join(golden_dir, f"{case}.json")]
    buf = io.StringIO()
    try:
        with contextlib.redirect_stdout(buf):
            assert run_reference.main(argv) == 0
    finally:
        if acm._model is not None:
            if not emu:
                acm._model.close()
            acm._model = None
        acm.args = None
        for k, v in saved.items():
            if v is None:
                sys.modules.pop(k, None)
            else:
                sys.modules[k] = v
    got = json.loads(buf.getvalue().strip().splitlines()[-1])
    assert len(got) == 5
    for (times, mems, reserved, rcs), p in zip(got, g["plans"]):
        assert times == p["time_list"] and mems == p["memory_list"] and reserved == p["reserved_memory_list"]
        assert rcs == p["check_recompute"]


def test_a_script_run_through_the_launcher_gets_the_binding_emu(golden_dir, tmp_path, monkeypatch):
    _run(golden_dir, tmp_path, monkeypatch, emu=True)


@pytest.mark.gpu
def test_a_script_run_through_the_launcher_gets_the_binding_gpu(golden_dir, tmp_path, monkeypatch):
    _run(golden_dir, tmp_path, monkeypatch, emu=False)


def test_the_launcher_without_a_script(capsys):
    assert run_reference.main([]) == 2
    assert "run_reference" in capsys.readouterr().out
    assert run_reference.main(["/nonexistent/aceso_search.py"]) == 2
