"""One case of tests/test_kernel_loop_cpu.py, run as a child process (`python -m tests.emu.guarded_case
WORKLOAD MODE N_PLANS`): the scoring kernel's own loop on the CPU behind guard pages.  Prints "ok"
when every output equals the state-machine emulation's (NaNs included); an out-of-range index in the
loop ends this process with SIGSEGV instead.

MODE: plain | collective (plain with consider_collective_memory) | breakdown | ranged | junk (random bytes for codes, headers and padding: results are not
compared, the loop only has to stay inside its arrays) | golden_resnet (the reference's ResNet plans) |
moves (csrc/ace_edit_kernels.h: move descriptors -> plans and keys, against the numpy forms; then random
descriptors) | recompute (check_recompute's loop for device-resident batches, run on CPU tensors with
the host build of the selection kernels, against the array form; then random stage tables)."""
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
    if mode == "collective":
        # consider_collective_memory: longer rows (memory tables after the cost tables), hence more row windows
        import dataclasses
        from superscaler_amd.tables import compile_tables
        graph = synth.make_graph(w)
        tables = compile_tables(graph, synth.make_db(w, graph),
                                dataclasses.replace(synth.make_settings(w), consider_collective_memory=True))
        assert tables.flags & 8
        mode = "plain"
    if mode == "plain":
        assert same(emu_kernel_score(tables, batch), emu_score(tables, batch))
        assert same(emu_kernel_score(tables, batch, strict=True, memory_limit=1.0), emu_score(tables, batch, strict=True, memory_limit=1.0))
        # plans stored in another order, results in the caller's order (ace_batch_t.d_order)
        from superscaler_amd.evaluator import depth_order
        perm = depth_order(batch)
        assert sorted(perm.tolist()) == list(range(batch.n_plans)) and not np.array_equal(perm, np.arange(batch.n_plans))
        stored = PlanBatch(np.ascontiguousarray(batch.codes[perm]), np.ascontiguousarray(batch.hdr[perm]))
        assert same(emu_kernel_score(tables, stored, order=perm), emu_score(tables, batch))
        assert same(emu_kernel_score(tables, stored, order=perm, breakdown=True), emu_score(tables, batch, breakdown=True))
        # the device's sort keys (ace_group_keys) give the same order
        import ctypes
        from superscaler_amd.evaluator import deal_slots
        from tests.helpers import emu_lib
        keys = np.zeros(batch.n_plans, dtype=np.uint64)
        raw = kernel_layout(batch.codes)
        hdr32 = np.ascontiguousarray(batch.hdr)
        assert emu_lib().ace_emu_group_keys(ctypes.c_void_p(raw.ctypes.data), ctypes.c_void_p(hdr32.ctypes.data),
                                            ctypes.c_longlong(batch.n_plans), ctypes.c_int(batch.num_ops),
                                            ctypes.c_void_p(keys.ctypes.data)) == 0
        assert np.array_equal(np.argsort(keys, kind="stable")[deal_slots(batch.n_plans)], perm)
        # ... and the gather puts the plans into that order (entries that are no index: the plan stays)
        co, ho = np.zeros_like(raw), np.zeros_like(hdr32)
        p32 = perm.astype(np.uint32)
        vp = ctypes.c_void_p
        assert emu_lib().ace_emu_gather_plans(vp(raw.ctypes.data), vp(hdr32.ctypes.data), vp(p32.ctypes.data),
                                              ctypes.c_longlong(batch.n_plans), ctypes.c_int(batch.num_ops),
                                              vp(co.ctypes.data), vp(ho.ctypes.data)) == 0
        assert np.array_equal(co, kernel_layout(stored.codes)) and np.array_equal(ho, stored.hdr)
        p32[::7] = 0xfffffff0
        assert emu_lib().ace_emu_gather_plans(vp(raw.ctypes.data), vp(hdr32.ctypes.data), vp(p32.ctypes.data),
                                              ctypes.c_longlong(batch.n_plans), ctypes.c_int(batch.num_ops),
                                              vp(co.ctypes.data), vp(ho.ctypes.data)) == 0
        assert np.array_equal(ho[::7], hdr32[::7])
        # entries that are no index of the batch: nothing is written for those slots
        wild = perm.astype(np.uint32).copy()
        wild[::5] = np.random.default_rng(1).integers(batch.n_plans, 2 ** 32, size=len(wild[::5]), dtype=np.uint64).astype(np.uint32)
        got, ref = emu_kernel_score(tables, stored, order=wild, breakdown=True), emu_score(tables, batch, breakdown=True)
        keep = np.ones(batch.n_plans, dtype=bool)
        keep[perm[::5]] = False
        assert all(np.array_equal(g[keep], r[keep], equal_nan=True) for g, r in zip(got, ref))
        assert all(not np.any(g[~keep]) for g in got)
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
    elif mode == "moves":
        import ctypes
        from superscaler_amd.neighbours import apply_moves_host, plan_keys_host, sample_moves
        from tests.helpers import emu_lib
        lib = emu_lib()
        vp = ctypes.c_void_p
        lib.ace_emu_apply_moves.restype = ctypes.c_int
        lib.ace_emu_apply_moves.argtypes = [vp, vp, ctypes.c_int, vp, ctypes.c_longlong, ctypes.c_int, ctypes.c_int, vp, vp, vp]
        rng = np.random.default_rng(9)
        N = tables.graph.num_ops
        G = (N + 15) // 16

        def expand(templates, moves, keys):
            T, m = templates.n_plans, len(moves)
            tc = np.zeros((T, G * 16), dtype=np.uint8)
            tc[:, :N] = templates.codes
            th = np.ascontiguousarray(templates.hdr)
            mv = np.ascontiguousarray(moves, dtype=np.uint32)
            co = np.zeros((G, m, 16), dtype=np.uint8)
            ho = np.zeros((m, 4), dtype=np.uint32)
            ko = np.zeros((m, 2), dtype=np.uint64) if keys else None
            assert lib.ace_emu_apply_moves(tc.ctypes.data, th.ctypes.data, T, mv.ctypes.data, m, N, tables.db.n_algo,
                                           co.ctypes.data, ho.ctypes.data, ko.ctypes.data if keys else None) == 0
            return co, ho, ko

        for p in range(min(n, 4)):
            templates, moves = sample_moves(batch.slice(p, p + 1), tables, 700, rng)
            want = apply_moves_host(templates, moves, tables.db.n_algo)
            co, ho, ko = expand(templates, moves, True)
            assert np.array_equal(co, kernel_layout(want.codes)) and np.array_equal(ho, want.hdr)
            assert np.array_equal(ko, plan_keys_host(want))
            junk = rng.integers(0, 2 ** 32, size=(512, 4), dtype=np.uint64).astype(np.uint32)
            junk[::2, 0] &= 0x0007ffff                 # half of them with a known op and a small template index
            expand(templates, junk, True)
            expand(templates, junk, False)
    elif mode == "recompute":
        import dataclasses
        from superscaler_amd import aceso_cost_model as acm
        from tests.helpers import EmuDeviceEvaluator
        limit = {"gpt3_1_3b": 9000.0, "gpt3_13b": 40000.0, "t5_770m": 6000.0, "wresnet_1b": 1500.0, "gpt3_175b": 60000.0}[workload]
        graph = synth.make_graph(w)
        st = dataclasses.replace(synth.make_settings(w), memory_limit=limit)
        cm = acm.CostModel(st, synth.make_db(w, graph), graph)
        cm._evaluator = EmuDeviceEvaluator(cm.tables)
        want = cm.update_recompute_arrays(batch)
        d = cm.update_recompute_device(cm.evaluator.upload(batch))
        N = batch.num_ops
        got = d.codes.permute(1, 0, 2).reshape(batch.n_plans, -1).numpy()
        assert np.array_equal(got[:, :N], want.codes) and not got[:, N:].any()
        assert (want.codes & 8).any() and not (want.codes & 8).all()      # the greedy loop had work to do
        # random stage tables: the kernels flag or ignore what lies outside the batch
        import ctypes
        import torch
        from superscaler_amd.evaluator import AceRcTablesStruct
        rng = np.random.default_rng(4)
        ev = cm.evaluator
        nq, nt = 300, len(cm.tables.db.op_names)
        act = np.ascontiguousarray(cm.tables.db.tables["activations"], dtype=np.float64)
        types = np.ascontiguousarray(cm.tables.graph.type_of_pos, dtype=np.int32)
        norec = np.zeros(nt, dtype=np.uint8)
        codes = d.codes.clone()
        t = AceRcTablesStruct(codes.data_ptr(), batch.n_plans, types.ctypes.data, act.ctypes.data, norec.ctypes.data, N, nt,
                              act.shape[1], act.shape[2], act.shape[3])
        q = [np.ascontiguousarray(rng.integers(-5, m, size=nq), dtype=np.int32) for m in (batch.n_plans + 5, N + 5, N + 5, 20)]
        mrow = rng.integers(0, 2 ** 32, size=nq, dtype=np.uint64).astype(np.uint32)
        sums, first, bad = np.zeros((nq, nt)), np.full((nq, nt), N, dtype=np.int32), np.zeros(nq, dtype=np.int32)
        assert ev.lib.ace_recompute_groups(ctypes.byref(t), nq, *[a.ctypes.data for a in q], mrow.ctypes.data, sums.ctypes.data,
                                           first.ctypes.data, bad.ctypes.data, None) == 0
        first = rng.integers(-3, N + 3, size=(nq, nt)).astype(np.int32)     # even with garbage group tables
        done, alive = np.zeros((nq, nt), dtype=np.uint8), np.ones(nq, dtype=np.uint8)
        mem = rng.uniform(0, 2 * limit, size=nq)
        assert ev.lib.ace_recompute_select(ctypes.byref(t), codes.data_ptr(), nq, *[a.ctypes.data for a in q], mrow.ctypes.data,
                                           sums.ctypes.data, first.ctypes.data, done.ctypes.data, mem.ctypes.data, float(limit),
                                           alive.ctypes.data, None) == 0
    else:
        raise SystemExit(f"unknown mode {mode}")
    print("ok")


if __name__ == "__main__":
    main(sys.argv[1], sys.argv[2], int(sys.argv[3]))
