"""One case of tests/test_kernel_loop_cpu.py, run as a child process (`python -m tests.emu.guarded_case
WORKLOAD MODE N_PLANS`): the scoring kernel's own loop on the CPU behind guard pages.  Prints "ok"
when every output equals the state-machine emulation's (NaNs included); an out-of-range index in the
loop ends this process with SIGSEGV instead.

MODE: plain | breakdown | ranged | junk (random bytes for codes, headers and padding: results are not
compared, the loop only has to stay inside its arrays) | golden_resnet (the reference's ResNet plans)."""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from superscaler_amd import synth  # noqa: E402
from superscaler_amd.plan import PlanBatch  # noqa: E402
from tests.helpers import emu_kernel_score, emu_score, kernel_layout  # noqa: E402


def same(a, b):
    return all(np.array_equal(x, y, equal_nan=True) for x, y in zip(a, b) if x is not None)


def stage_ranges(batch):
    """(plan index, [lo, hi)) of every stage of every plan."""
    P, N = batch.codes.shape
    plan, lo = np.nonzero(batch.codes & 16)
    hi = np.append(lo[1:], N)
    hi[np.append(plan[1:] != plan[:-1], True)] = N
    return plan, np.stack([lo, hi], axis=1).astype(np.uint32)


def main(workload, mode, n):
    if mode == "golden_resnet":
        from superscaler_amd.opgraph import OpGraph
        from superscaler_amd.plan import get_config
        from superscaler_amd.profile_db import CostModelSettings, ProfileDB
        from superscaler_amd.tables import compile_tables
        gdir = os.path.join(ROOT, "tests", "golden")
        with open(os.path.join(gdir, "resnet_500M.json")) as f:
            g = json.load(f)
        st = CostModelSettings(model_name=g["model_name"], micro_batch_size=g["micro_batch_size"],
                               num_gpus_per_node=g["num_gpus_per_node"], global_batch_size=g["global_batch_size"],
                               memory_limit=g["memory_limit"])
        db = ProfileDB.from_directory(g["model_name"], g["model_size"], os.path.join(gdir, "db_resnet_500M") + "/", st)
        graph = OpGraph.build(g["model_name"], db.op_names, g["num_layers"])
        tables = compile_tables(graph, db, st)
        cfgs = [get_config(p["num_ops_in_each_stage"], p["tp"], p["dp"], p["recompute_ops"], p["micro_batch_size"],
                           g["global_batch_size"], graph.ops, p["algo"]) for p in g["plans"]]
        batch = PlanBatch.from_configs(cfgs, tables)
        assert same(emu_kernel_score(tables, batch, breakdown=True), emu_score(tables, batch, breakdown=True))
        assert same(emu_kernel_score(tables, batch), emu_score(tables, batch))
        print("ok")
        return
    w = synth.WORKLOADS[workload]
    tables = synth.make_tables(w)
    batch = synth.make_plans(w, tables, n_plans=n, seed_offset=5)
    if mode == "plain":
        assert same(emu_kernel_score(tables, batch), emu_score(tables, batch))
        assert same(emu_kernel_score(tables, batch, strict=True, memory_limit=1.0), emu_score(tables, batch, strict=True, memory_limit=1.0))
    elif mode == "breakdown":
        assert same(emu_kernel_score(tables, batch, breakdown=True), emu_score(tables, batch, breakdown=True))
    elif mode == "ranged":
        plan, rg = stage_ranges(batch)
        q = PlanBatch(np.ascontiguousarray(batch.codes[plan]), np.ascontiguousarray(batch.hdr[plan]))
        q.hdr[:, 0] = (q.hdr[:, 0] & 0xff00) | 1          # single-stage queries
        assert same(emu_kernel_score(tables, q, ranges=rg), emu_score(tables, q, ranges=rg))
        # ranges that do not fit the plan are flagged, not followed
        bad = rg.copy()
        bad[::3, 1] = tables.graph.num_ops + 7
        bad[1::3, 0] = bad[1::3, 1]
        assert same(emu_kernel_score(tables, q, ranges=bad), emu_score(tables, q, ranges=bad))
    elif mode == "junk":
        rng = np.random.default_rng(3)
        P, N = batch.codes.shape
        G = (N + 15) // 16
        for trial in range(3):
            raw = rng.integers(0, 256, size=(G, P, 16), dtype=np.uint8)
            if trial == 1:                       # valid plans, junk only in the padding bytes
                raw = kernel_layout(batch.codes)
                pad = rng.integers(0, 256, size=(P, G * 16 - N), dtype=np.uint8)
                raw.transpose(1, 0, 2).reshape(P, G * 16)[:, N:] = pad
            hdr = rng.integers(0, 2 ** 32, size=(P, 4), dtype=np.uint64).astype(np.uint32) if trial != 1 else batch.hdr
            junk = PlanBatch(batch.codes, np.ascontiguousarray(hdr))
            out = emu_kernel_score(tables, junk, raw_codes=raw)
            emu_kernel_score(tables, junk, raw_codes=raw, breakdown=True)
            rg = rng.integers(0, 2 ** 32, size=(P, 2), dtype=np.uint64).astype(np.uint32)
            emu_kernel_score(tables, junk, raw_codes=raw, ranges=rg)
            if trial == 1:
                assert same(out, emu_score(tables, batch))
    else:
        raise SystemExit(f"unknown mode {mode}")
    print("ok")


if __name__ == "__main__":
    main(sys.argv[1], sys.argv[2], int(sys.argv[3]))
