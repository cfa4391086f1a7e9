"""GPU parity: the HIP kernels, called through the C ABI, against the oracle on the same seeded
inputs.  Bar: iteration time and peak memory bit-identical (tolerance 0, well inside the 1e-9
relative the task allows), feasibility flags and top-k indices identical."""
import json
import os

import numpy as np
import pytest

from superscaler_amd import synth
from superscaler_amd.opgraph import OpGraph
from superscaler_amd.plan import PlanBatch, get_config
from superscaler_amd.profile_db import CostModelSettings, ProfileDB
from superscaler_amd.tables import compile_tables
from tests.helpers import c_oracle_scores, emu_score, oracle_for, oracle_scores

pytestmark = pytest.mark.gpu

CASES = [("gpt3_1_3b", 4096, 4096), ("t5_770m", 4096, 256), ("wresnet_1b", 8192, 1024),
         ("gpt3_13b", 8192, 512), ("gpt3_175b", 2048, 64)]


@pytest.fixture(scope="module")
def torch_mod():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch


@pytest.fixture(scope="module", params=CASES, ids=[c[0] for c in CASES])
def case(request, torch_mod):
    from superscaler_amd.evaluator import PlanEvaluator
    name, n, n_oracle = request.param
    w = synth.WORKLOADS[name]
    tables = synth.make_tables(w)
    batch = synth.make_plans(w, tables, n_plans=n)
    ev = PlanEvaluator(tables)
    yield w, tables, batch, ev, n_oracle
    ev.close()


def test_scores_match_oracle(case):
    w, tables, batch, ev, n_oracle = case
    print(f"[case] {w.name} plans={batch.n_plans} oracle_plans={n_oracle}", flush=True)
    it, pk, fe, st = ev.score_host(batch)
    assert (st == 0).all()
    orc = oracle_for(tables)
    oit, opk, ofe, _ = oracle_scores(orc, batch, tables, idx=range(n_oracle))
    assert np.array_equal(it[:n_oracle], oit)
    assert np.array_equal(pk[:n_oracle], opk)
    assert np.array_equal(fe[:n_oracle], ofe)
    # a limit in the middle of the batch: flags must follow the oracle's memory exactly, for <= and <
    mid = float(np.median(opk))
    for strict in (False, True):
        _, _, fe_mid, _ = ev.score_host(batch.slice(0, n_oracle), memory_limit=mid, strict=strict)
        want = (opk < mid) if strict else (opk <= mid)
        assert np.array_equal(fe_mid, want.astype(np.uint8)) and 0 < fe_mid.sum() < n_oracle
    # the CPU build of the same state machine covers the whole batch
    eit, epk, efe, est, _ = emu_score(tables, batch)
    assert np.array_equal(it, eit) and np.array_equal(pk, epk) and np.array_equal(fe, efe)


def test_stage_records_match(case):
    w, tables, batch, ev, n_oracle = case
    sub = batch.slice(0, 512)
    it, pk, fe, st, rec = ev.score_host(sub, breakdown=True)
    eit, epk, efe, est, erec = emu_score(tables, sub, breakdown=True)
    assert np.array_equal(it, eit) and np.array_equal(pk, epk)
    assert np.array_equal(rec, erec)


def test_topk_matches_oracle_order(case, torch_mod):
    w, tables, batch, ev, n_oracle = case
    d = ev.upload(batch)
    it, pk, fe, st = ev.score(d)
    for k in (1, 10, 64):
        idx, val, cnt = ev.topk(it, fe, k)
        torch_mod.cuda.synchronize()
        hit, hfe = it.cpu().numpy(), fe.cpu().numpy()
        order = np.lexsort((np.arange(len(hit)), np.where(hfe > 0, hit, np.inf)))
        nfeas = int(hfe.sum())
        want = order[:min(k, nfeas)]
        got = idx.cpu().numpy()
        assert int(cnt.item()) == min(k, nfeas)
        assert np.array_equal(got[:len(want)], want)
        assert np.array_equal(val.cpu().numpy()[:len(want)], hit[want])
        assert (got[len(want):] == -1).all()


def test_topk_ties_pick_lowest_index(torch_mod):
    from superscaler_amd.evaluator import PlanEvaluator
    w = synth.WORKLOADS["gpt3_1_3b"]
    tables = synth.make_tables(w)
    ev = PlanEvaluator(tables)
    t = torch_mod.tensor([5.0, 3.0, 3.0, 9.0, 1.0, 3.0, 3.0, 3.0] * 500, dtype=torch_mod.float64, device="cuda")
    f = torch_mod.ones(t.numel(), dtype=torch_mod.uint8, device="cuda")
    f[4::8] = 0
    for k in (3, 7, 100, 2500):
        idx, val, cnt = ev.topk(t, f, k)
        ht, hf = t.cpu().numpy(), f.cpu().numpy()
        order = np.lexsort((np.arange(len(ht)), np.where(hf > 0, ht, np.inf)))
        assert np.array_equal(idx.cpu().numpy(), order[:k])
    # fewer feasible plans than k
    f[:] = 0
    f[10] = 1
    idx, val, cnt = ev.topk(t, f, 4)
    assert idx.cpu().tolist() == [10, -1, -1, -1] and int(cnt.item()) == 1
    ev.close()


def test_topk_short_form_edges(torch_mod):
    """The three-launch form of the top-k (small k): inputs on which the sample's bound lets nearly everything through (all
    times equal, a million of them), heavy duplication, negative zero and
    infinities, all infeasible, a single entry -- against a stable sort; and the same results as the multi-launch form."""
    from superscaler_amd.evaluator import PlanEvaluator
    torch = torch_mod
    w = synth.WORKLOADS["gpt3_1_3b"]
    ev = PlanEvaluator(synth.make_tables(w))
    rng = np.random.default_rng(5)

    def check(ht, hf, ks):
        t = torch.from_numpy(ht).cuda()
        f = torch.from_numpy(hf).cuda()
        key = np.where((hf > 0) & ~np.isnan(ht), ht, np.inf)
        order = np.lexsort((np.arange(len(ht)), key))
        n_ok = int(np.isfinite(key).sum()) if not np.isinf(ht[hf > 0]).any() else None
        for k in ks:
            idx, val, cnt = ev.topk(t, f, k)
            idx, val = idx.cpu().numpy(), val.cpu().numpy()
            n = int(cnt.item())
            if n_ok is not None:
                assert n == min(k, n_ok)
            assert np.array_equal(idx[:n], order[:n]) and np.array_equal(val[:n], ht[order[:n]]), (len(ht), k)
            assert (idx[n:] == -1).all()

    n = 1 << 20
    check(np.full(n, 7.25), np.ones(n, dtype=np.uint8), [1, 64, 256])                      # one value: every entry passes the filter
    check(rng.integers(0, 50, n).astype(np.float64), (rng.random(n) < 0.9).astype(np.uint8), [64, 200])   # 50 distinct values
    t = rng.lognormal(3.0, 1.0, 300000)
    t[::1000] = 0.0
    t[1::1000] = -0.0
    check(t, (rng.random(300000) < 0.5).astype(np.uint8), [8, 64, 256, 257, 300])           # (257, 300: the multi-launch form)
    check(rng.random(5000), np.zeros(5000, dtype=np.uint8), [64])                           # nothing feasible
    check(rng.random(70), np.ones(70, dtype=np.uint8), [64, 100])                           # fewer entries than the sample, than k
    check(np.array([3.5]), np.ones(1, dtype=np.uint8), [1, 5])
    # equal keys at the k-th place: a few entries below a mass of equal ones (the equal ones are only counted per stretch
    # of the input and read back in index order), the mass starting late in the input, infeasible entries inside it,
    # just enough equal ones to be listed one by one, and equal ones one per stretch of 8,192
    t = np.full(n, 9.5)
    t[rng.choice(n, 40, replace=False)] = rng.random(40)
    check(t, np.ones(n, dtype=np.uint8), [1, 39, 40, 41, 64, 256])
    t = rng.random(n) + 20.0
    t[700000:] = 3.0
    f = np.ones(n, dtype=np.uint8)
    f[700000:700100] = 0
    f[700105::2] = 0
    t[5] = 1.0
    check(t, f, [1, 2, 64, 256])
    t = rng.random(n) + 20.0
    t[rng.choice(n, 2000, replace=False)] = 4.0
    check(t, np.ones(n, dtype=np.uint8), [64, 256])
    t = rng.random(n) + 20.0
    t[4096::8192] = 4.0
    t[4097::8192 * 3] = 4.0
    check(t, np.ones(n, dtype=np.uint8), [8, 64, 200])
    check(np.arange(n, 0, -1, dtype=np.float64), np.ones(n, dtype=np.uint8), [1, 64, 256])   # falling times: the best are neighbours
    check(np.arange(n, dtype=np.float64), np.ones(n, dtype=np.uint8), [64])
    t = np.full(1 << 24, 2.0)                                                              # n * k at the short form's limit
    t[123457] = 1.0
    check(t, np.ones(1 << 24, dtype=np.uint8), [1, 4])
    t = rng.random(100000)
    f = np.zeros(100000, dtype=np.uint8)
    f[rng.choice(100000, 40, replace=False)] = 1
    check(t, f, [64])                                                                       # fewer feasible entries than k, none in the sample
    # enough candidates below the threshold (the selection that keeps them in registers): a thousand distinct values, so
    # that the k-th place lies inside about a thousand equal keys and is decided by the index digits; inputs a little
    # larger than the sample; a k-th place deep inside the candidates
    check(rng.integers(0, 1000, n).astype(np.float64), (rng.random(n) < 0.9).astype(np.uint8), [1, 64, 256])
    check(rng.random(20000), np.ones(20000, dtype=np.uint8), [1, 64, 256])
    check(rng.lognormal(0.0, 2.0, 70000), (rng.random(70000) < 0.3).astype(np.uint8), [1, 5, 64, 255, 256])
    check(-rng.lognormal(0.0, 2.0, 70000), np.ones(70000, dtype=np.uint8), [64, 256])        # negative times: the keys' other branch
    ev.close()


GOLDEN = ["gpt_1_3B", "resnet_500M", "t5_770M"]


@pytest.mark.parametrize("name", GOLDEN)
def test_reference_golden_vectors(name, golden_dir, torch_mod):
    """Plans scored by the reference itself on its own profile databases."""
    from superscaler_amd.evaluator import PlanEvaluator
    with open(os.path.join(golden_dir, f"{name}.json")) as f:
        g = json.load(f)
    st = CostModelSettings(model_name=g["model_name"], micro_batch_size=g["micro_batch_size"],
                           num_gpus_per_node=g["num_gpus_per_node"], global_batch_size=g["global_batch_size"],
                           memory_limit=g["memory_limit"])
    db = ProfileDB.from_directory(g["model_name"], g["model_size"], os.path.join(golden_dir, f"db_{name}") + "/", st)
    graph = OpGraph.build(g["model_name"], db.op_names, g["num_layers"])
    tables = compile_tables(graph, db, st)
    cfgs = [get_config(p["num_ops_in_each_stage"], p["tp"], p["dp"], p["recompute_ops"], p["micro_batch_size"],
                       g["global_batch_size"], graph.ops, p["algo"]) for p in g["plans"]]
    batch = PlanBatch.from_configs(cfgs, tables)
    ev = PlanEvaluator(tables)
    it, pk, fe, stt, rec = ev.score_host(batch, breakdown=True)
    for k, p in enumerate(g["plans"]):
        assert it[k] == max(p["time_list"])
        assert pk[k] == max(p["memory_list"])
        assert fe[k] == int(max(p["memory_list"]) <= g["memory_limit"])
        for s in range(len(p["time_list"])):
            assert rec[k, s, 16] == p["memory_list"][s]
    ev.close()


def test_grouped_storage_returns_results_in_the_callers_order(torch_mod):
    """ace_batch_t.d_order: plans stored sorted by depth and first cut score exactly as in their own order,
    stage records included."""
    from superscaler_amd.evaluator import PlanEvaluator, depth_order
    for name, n in (("gpt3_13b", 20000), ("wresnet_1b", 5000), ("t5_770m", 3000)):
        w = synth.WORKLOADS[name]
        tables = synth.make_tables(w)
        batch = synth.make_plans(w, tables, n_plans=n, seed_offset=21)
        ev = PlanEvaluator(tables)
        plain = ev.score_host(batch)
        grouped = ev.score_host(batch, group_by_depth=True)
        assert all(np.array_equal(a, b, equal_nan=True) for a, b in zip(plain, grouped))
        small = batch.slice(0, 512)
        plain = ev.score_host(small, breakdown=True)
        grouped = ev.score_host(small, breakdown=True, group_by_depth=True)
        S = small.hdr[:, 0] & 0xff
        used = np.arange(16)[None, :] < S[:, None]
        assert all(np.array_equal(a, b, equal_nan=True) for a, b in zip(plain[:4], grouped[:4]))
        assert np.array_equal(plain[4][used], grouped[4][used], equal_nan=True)
        d = ev.upload(batch, group_by_depth=True)
        perm = depth_order(batch)
        assert np.array_equal(d.order.cpu().numpy(), perm) and not np.array_equal(perm, np.arange(n))
        # the same grouping made on the device from a plain upload
        g = ev.group(ev.upload(batch))
        assert np.array_equal(g.order.cpu().numpy(), perm)
        assert torch_mod.equal(g.codes, d.codes) and torch_mod.equal(g.hdr, d.hdr)
        it, pk, fe, st = ev.score(g)
        assert all(np.array_equal(a, b.cpu().numpy(), equal_nan=True) for a, b in zip(ev.score_host(batch), (it, pk, fe, st)))
        ev.close()


@pytest.mark.parametrize("name", ["gpt3_13b", "wresnet_1b"])
def test_every_settings_combination_matches_the_c_oracle(name, torch_mod):
    """MAX / MIN memory prediction, shared-buffer rule, reserved space, resharding on and off: the kernels
    against the C oracle (which the CPU suite pins to the Python oracle for the same combinations)."""
    import dataclasses
    import itertools
    from superscaler_amd.evaluator import PlanEvaluator
    w = synth.WORKLOADS[name]
    graph = synth.make_graph(w)
    db = synth.make_db(w, graph)
    batch = synth.make_plans(w, synth.make_tables(w), n_plans=3000, seed_offset=78)
    answers = set()
    combos = [c + (False,) for c in itertools.product(("MAX", "MIN"), (True, False), (True, False), (True, False))]
    combos += [(pred, shared, True, True, True) for pred in ("MAX", "MIN") for shared in (True, False)]   # collective memory
    for pred, shared, reserved, resh, coll in combos:
        st = dataclasses.replace(synth.make_settings(w), memory_pred_type=pred, consider_shared_space=shared,
                                 consider_reserved_space=reserved, resharding=resh, consider_collective_memory=coll)
        tables = compile_tables(graph, db, st)
        ev = PlanEvaluator(tables)
        it, pk, fe, status = ev.score_host(batch, group_by_depth=shared)
        _, _, _, _, rec = ev.score_host(batch.slice(0, 256), breakdown=True)
        ev.close()
        cit, cpk, cfe, cer, tl, ml = c_oracle_scores(tables, batch, threads=8, lists=True)
        assert not cer.any() and (status == 0).all()
        assert np.array_equal(it, cit) and np.array_equal(pk, cpk) and np.array_equal(fe, cfe), (pred, shared, reserved, resh, coll)
        S = batch.hdr[:256, 0] & 0xff
        used = np.arange(16)[None, :] < S[:, None]
        assert np.array_equal(rec[:, :, 16][used], ml[:256][used])
        answers.add((float(pk.sum()), float(it.sum())))
    assert len(answers) >= 10


@pytest.mark.parametrize("name", ["gpt3_1_3b", "wresnet_1b"])
def test_large_batches_of_every_loop_variant_match_the_c_oracle(name, torch_mod):
    """The assembly op loop has one text per (resharding on / off, reserved-memory rule, rows resident / windowed), and
    only batches of 128 workgroups or more run it over windowed rows: each of the six settings at 131,072 + 77 plans
    against the C oracle, every plan."""
    import dataclasses
    from superscaler_amd.evaluator import PlanEvaluator
    w = synth.WORKLOADS[name]
    graph = synth.make_graph(w)
    db = synth.make_db(w, graph)
    batch = synth.make_plans(w, synth.make_tables(w), n_plans=131072 + 77, seed_offset=81, workers=8)
    answers = set()
    for resh in (True, False):
        for pred, reserved in (("MAX", True), ("MIN", True), ("MAX", False)):
            st = dataclasses.replace(synth.make_settings(w), memory_pred_type=pred, consider_reserved_space=reserved, resharding=resh)
            tables = compile_tables(graph, db, st)
            ev = PlanEvaluator(tables)
            it, pk, fe, status = ev.score_host(batch)
            ev.close()
            cit, cpk, cfe, cer = c_oracle_scores(tables, batch, threads=16)
            assert not cer.any() and (status == 0).all()
            assert np.array_equal(it, cit) and np.array_equal(pk, cpk) and np.array_equal(fe, cfe), (pred, reserved, resh)
            answers.add((float(pk.sum()), float(it.sum())))
    assert len(answers) == 6


@pytest.mark.parametrize("name", ["gpt3_1_3b", "wresnet_1b"])
def test_collective_memory_switch_matches_the_oracle(name, torch_mod):
    """consider_collective_memory (aceso_cost_model.py:462-483): the buffers of the resharding collectives enter the
    reserved memory; the rows grow by the memory tables, so these runs also use the windowed kernel."""
    import dataclasses
    from superscaler_amd.evaluator import PlanEvaluator
    w = synth.WORKLOADS[name]
    graph = synth.make_graph(w)
    db = synth.make_db(w, graph)
    batch = synth.make_plans(w, synth.make_tables(w), n_plans=192, seed_offset=79)
    changed = 0
    for pred in ("MAX", "MIN"):
        st = dataclasses.replace(synth.make_settings(w), memory_pred_type=pred, consider_collective_memory=True)
        tables = compile_tables(graph, db, st)
        ev = PlanEvaluator(tables)
        it, pk, fe, status, rec = ev.score_host(batch, breakdown=True)
        it2, pk2, fe2, status2 = ev.score_host(batch)
        ev.close()
        oit, opk, ofe, cfgs = oracle_scores(oracle_for(tables), batch, tables)
        assert (status == 0).all() and np.array_equal(it, oit) and np.array_equal(pk, opk) and np.array_equal(fe, ofe)
        assert np.array_equal(it2, oit) and np.array_equal(pk2, opk) and np.array_equal(fe2, ofe)
        for p, c in enumerate(cfgs):
            assert [rec[p, s, 16] for s in range(c.num_stages)] == list(c.memory_list)
        off = compile_tables(graph, db, dataclasses.replace(st, consider_collective_memory=False))
        changed += int((oracle_scores(oracle_for(off), batch, off)[1] != opk).sum())
    assert changed > 0


def test_full_size_properties(torch_mod):
    """GPT-3 13B at the benchmark's full size (1,048,576 plans), which the oracle cannot cover:
    size-independent properties, an oracle spot check and the top-k against a stable sort."""
    from superscaler_amd.evaluator import PlanEvaluator
    w = synth.WORKLOADS["gpt3_13b"]
    tables = synth.make_tables(w)
    ev = PlanEvaluator(tables)
    n = w.n_plans
    assert n == 1048576
    batch = synth.make_plans(w, tables, n_plans=n, seed_offset=7, workers=8)
    # 48 plans spread over the batch against the oracle, bit for bit
    sample = np.random.Generator(np.random.PCG64(3)).choice(n, size=48, replace=False)
    d = ev.upload(batch)
    t_it, t_pk, t_fe, t_st = ev.score(d)
    oit, opk, ofe, _ = oracle_scores(oracle_for(tables), batch, tables, idx=sample)
    assert np.array_equal(t_it.cpu().numpy()[sample], oit) and np.array_equal(t_pk.cpu().numpy()[sample], opk)
    assert np.array_equal(t_fe.cpu().numpy()[sample], ofe)
    # every one of the 1,048,576 plans against the C oracle, bit for bit
    cit, cpk, cfe, cer = c_oracle_scores(tables, batch, threads=16)
    assert not cer.any() and (t_st.cpu().numpy() == 0).all()
    assert np.array_equal(t_it.cpu().numpy(), cit) and np.array_equal(t_pk.cpu().numpy(), cpk)
    assert np.array_equal(t_fe.cpu().numpy(), cfe)
    # top-64 = the first 64 of a stable ascending sort of the feasible plans
    idx, val, cnt = ev.topk(t_it, t_fe, 64)
    h_it, h_fe = t_it.cpu().numpy(), t_fe.cpu().numpy()
    feas = np.flatnonzero(h_fe)
    order = feas[np.argsort(h_it[feas], kind="stable")][:64]
    assert int(cnt.item()) == 64 and np.array_equal(idx.cpu().numpy(), order) and np.array_equal(val.cpu().numpy(), h_it[order])
    # duplicated plans score identically; a permuted batch gives permuted results
    perm = np.random.Generator(np.random.PCG64(1)).permutation(n)
    it, pk, fe, st = ev.score_host(batch)
    it2, pk2, fe2, st2 = ev.score_host(PlanBatch(batch.codes[perm], batch.hdr[perm]))
    assert np.array_equal(it[perm], it2) and np.array_equal(pk[perm], pk2) and np.array_equal(fe[perm], fe2)
    assert (st == 0).all() and np.isfinite(it).all()
    # clearing every recompute bit can only remove recompute time (memory may move either way:
    # the peak segment can outweigh what recomputation saves)
    nb = PlanBatch(batch.codes & np.uint8(0xF7), batch.hdr)
    it3, pk3, fe3, _ = ev.score_host(nb)
    assert (it3 <= it).all() and (it3 < it).any()
    # a single-stage plan's iteration time is (number of micro-batches) x (stage time)
    one = np.flatnonzero((batch.hdr[:, 0] & 0xff) == 1)[:2048]
    _, _, _, _, rec = ev.score_host(PlanBatch(batch.codes[one], batch.hdr[one]), breakdown=True)
    nbm1 = tables.nb_minus_1[(batch.hdr[one, 0] >> 8) & 0xff]
    assert np.array_equal(it[one], rec[:, 0, 15] * nbm1 + rec[:, 0, 15])
    # feasibility is monotone in the limit
    _, _, fe_lo, _ = ev.score_host(batch, memory_limit=40000.0)
    _, _, fe_hi, _ = ev.score_host(batch, memory_limit=160000.0)
    assert (fe_lo <= fe).all() and (fe <= fe_hi).all()
    ev.close()


@pytest.mark.parametrize("name,n", [("gpt3_1_3b", 4096), ("t5_770m", 65536), ("wresnet_1b", 262144), ("gpt3_175b", 262144)])
def test_configured_sizes_match_c_oracle(name, n, torch_mod):
    """The other configurations at their full batch sizes (gpt3_175b: one of its 262,144-plan batches;
    wresnet_1b runs the windowed kernel): every plan bit-identical to the C oracle, the top-64 equal
    to a stable sort."""
    from superscaler_amd.evaluator import PlanEvaluator
    w = synth.WORKLOADS[name]
    tables = synth.make_tables(w)
    batch = synth.make_plans(w, tables, n_plans=n, seed_offset=13, workers=8)
    ev = PlanEvaluator(tables)
    it, pk, fe, st = ev.score_host(batch)
    cit, cpk, cfe, cer = c_oracle_scores(tables, batch, threads=16)
    assert not cer.any() and (st == 0).all()
    assert np.array_equal(it, cit) and np.array_equal(pk, cpk) and np.array_equal(fe, cfe)
    d = ev.upload(batch)
    t_it, t_pk, t_fe, _ = ev.score(d)
    idx, val, cnt = ev.topk(t_it, t_fe, 64)
    feas = np.flatnonzero(cfe)
    order = feas[np.argsort(cit[feas], kind="stable")][:64]
    assert int(cnt.item()) == len(order) and np.array_equal(idx.cpu().numpy()[:len(order)], order)
    ev.close()


def test_windowed_rows_ragged_batch_and_small_batch_agree(torch_mod):
    """wresnet_1b (rows windowed) at a size that is not a whole number of workgroups and large enough for the kernel
    whose op loop fetches its own windows: every plan bit-identical to the C oracle, also after a second call on the
    same handle, and identical to what the small-batch kernel (C++ loop, the tables' own windows) gives for a slice."""
    from superscaler_amd.evaluator import PlanEvaluator
    w = synth.WORKLOADS["wresnet_1b"]
    tables = synth.make_tables(w)
    n = 131072 + 517
    batch = synth.make_plans(w, tables, n_plans=n, seed_offset=29, workers=8)
    ev = PlanEvaluator(tables)
    cit, cpk, cfe, cer = c_oracle_scores(tables, batch, threads=16)
    for _ in range(2):
        it, pk, fe, st = ev.score_host(batch)
        assert (st == 0).all()
        assert np.array_equal(it, cit) and np.array_equal(pk, cpk) and np.array_equal(fe, cfe)
    lo, hi = n - 3000, n
    sit, spk, sfe, sst = ev.score_host(batch.slice(lo, hi))
    assert np.array_equal(sit, cit[lo:hi]) and np.array_equal(spk, cpk[lo:hi]) and np.array_equal(sfe, cfe[lo:hi])
    ev.close()


@pytest.mark.parametrize("name", list(synth.WORKLOADS))
def test_stage_records_match_c_oracle_lists(name, torch_mod):
    """The per-stage records (breakdown kernel; windowed for wresnet_1b) against the C oracle's
    time_list / memory_list for a few thousand plans: memory per stage directly, time through
    time_list[s] = t_s * (nb - 1) + sum(t)."""
    from superscaler_amd.evaluator import PlanEvaluator
    from superscaler_amd.tables import R_STAGE_MB, R_STAGE_MS
    w = synth.WORKLOADS[name]
    tables = synth.make_tables(w)
    batch = synth.make_plans(w, tables, n_plans=4000, seed_offset=31, workers=4)
    ev = PlanEvaluator(tables)
    it, pk, fe, st, rec = ev.score_host(batch, breakdown=True)
    ev.close()
    cit, cpk, cfe, cer, tl, ml = c_oracle_scores(tables, batch, threads=8, lists=True)
    assert not cer.any() and np.array_equal(it, cit) and np.array_equal(pk, cpk) and np.array_equal(fe, cfe)
    S = (batch.hdr[:, 0] & 0xff).astype(int)
    nbm1 = tables.nb_minus_1[(batch.hdr[:, 0] >> 8) & 0xff]
    tsum = np.zeros(batch.n_plans)
    for s in range(16):
        tsum = np.where(S > s, tsum + rec[:, s, R_STAGE_MS], tsum)
    for s in range(16):
        m = S > s
        assert np.array_equal(rec[m, s, R_STAGE_MB], ml[m, s])
        assert np.array_equal((rec[:, s, R_STAGE_MS] * nbm1 + tsum)[m], tl[m, s])


def test_odd_table_geometries(torch_mod):
    """Corners of the table geometry (helpers.odd_workloads: one tp, one micro-batch size, exactly 16 ops, six
    micro-batch sizes, stages wider than a node, short ResNets) with 3,000 plans each: scores, flags and the
    per-stage memory against the C oracle, in plain and in grouped storage, and the top 32."""
    from superscaler_amd.evaluator import PlanEvaluator
    from superscaler_amd.tables import R_STAGE_MB
    from tests.helpers import odd_workloads
    for w in odd_workloads():
        tables = synth.make_tables(w)
        batch = synth.make_plans(w, tables, n_plans=3000, seed_offset=5, workers=2)
        print(f"[case] {w.name} ops={tables.graph.num_ops} windows={tables.n_windows}", flush=True)
        cit, cpk, cfe, cer, tl, ml = c_oracle_scores(tables, batch, threads=8, lists=True)
        assert not cer.any()
        ev = PlanEvaluator(tables)
        for grouped in (False, True):
            it, pk, fe, st = ev.score_host(batch, group_by_depth=grouped)
            assert (st == 0).all() and np.array_equal(it, cit) and np.array_equal(pk, cpk) and np.array_equal(fe, cfe), (w.name, grouped)
        _, _, _, _, rec = ev.score_host(batch, breakdown=True)
        S = (batch.hdr[:, 0] & 0xff).astype(int)
        for s in range(16):
            assert np.array_equal(rec[S > s, s, R_STAGE_MB], ml[S > s, s]), w.name
        d = ev.upload(batch)
        dit, _, dfe, _ = ev.score(d)[:4]
        idx, val, cnt = ev.topk(dit, dfe, 32)
        feas = np.flatnonzero(cfe)
        order = feas[np.argsort(cit[feas], kind="stable")][:32]
        assert int(cnt.item()) == len(order) and np.array_equal(idx.cpu().numpy()[:len(order)], order), w.name
        ev.close()


def test_small_calls_take_the_same_answers_through_the_pinned_buffers(torch_mod):
    """score_host sends small batches through one pinned buffer each way (layout done on the host); the
    results must be the bytes of the general path (upload + score), for whole plans, stage records and
    single-stage queries, with the last 16-op group full (16 ops) and partly filled (523, 134 ops)."""
    from superscaler_amd.evaluator import PlanEvaluator
    from tests.helpers import odd_workloads
    for w in [synth.WORKLOADS["gpt3_13b"], synth.WORKLOADS["wresnet_1b"], odd_workloads()[1]]:
        tables = synth.make_tables(w)
        N = tables.graph.num_ops
        ev = PlanEvaluator(tables)
        for n in (1, 7, 300):
            batch = synth.make_plans(w, tables, n_plans=n, seed_offset=n)
            for breakdown in (False, True):
                small = ev._score_small(batch, float(w.memory_limit), False, breakdown, None)
                assert small is not None
                big = ev.score(ev.upload(batch), breakdown=breakdown)
                for a, b in zip(small, big):
                    assert np.array_equal(a, b.cpu().numpy()), (w.name, n, breakdown)
            # every plan's first stage as a single-stage query
            cut = np.where((batch.codes[:, 1:] & 16) != 0, np.arange(1, N)[None, :], N).min(axis=1)
            ranges = np.stack([np.zeros(n, dtype=np.uint32), cut.astype(np.uint32)], axis=1)
            small = ev._score_small(batch, float(w.memory_limit), False, True, ranges)
            big = ev.score(ev.upload(batch, ranges=ranges), breakdown=True)
            assert np.array_equal(small[3], big[3].cpu().numpy())
            assert np.array_equal(small[4][:, 0], big[4][:, 0].cpu().numpy()), (w.name, n)
        ev.close()


def test_handles_coexist_and_release_their_memory(torch_mod):
    """Two handles with different tables alive at once (interleaved launches, one of them with windowed rows)
    keep to their own tables and workspaces; creating and destroying handles leaves no device memory behind."""
    from superscaler_amd.evaluator import PlanEvaluator
    torch = torch_mod
    ta, tb = synth.make_tables(synth.WORKLOADS["gpt3_1_3b"]), synth.make_tables(synth.WORKLOADS["wresnet_1b"])
    ba = synth.make_plans(synth.WORKLOADS["gpt3_1_3b"], ta, n_plans=5000, seed_offset=3)
    bb = synth.make_plans(synth.WORKLOADS["wresnet_1b"], tb, n_plans=5000, seed_offset=3)
    want_a, want_b = c_oracle_scores(ta, ba, threads=8), c_oracle_scores(tb, bb, threads=8)
    ea, eb = PlanEvaluator(ta), PlanEvaluator(tb)
    da, db = ea.upload(ba), eb.upload(bb)
    for _ in range(3):
        oa, ob = ea.score(da), eb.score(db)
        oa2 = ea.score(da, breakdown=True)
        for got, want in ((oa, want_a), (ob, want_b), (oa2, want_a)):
            assert all(np.array_equal(g.cpu().numpy(), w) for g, w in zip(got[:3], want[:3]))
    ea.close()
    eb.close()
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    free0 = torch.cuda.mem_get_info()[0]
    for k in range(40):
        ev = PlanEvaluator(ta if k % 2 else tb)
        ev.score_host(ba.slice(0, 2000) if k % 2 else bb.slice(0, 2000))        # allocates the handle's workspace too
        ev.close()
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    assert free0 - torch.cuda.mem_get_info()[0] < (8 << 20)


def test_captured_step_replays_to_the_eager_results(torch_mod):
    """score + top-k recorded in a HIP graph: four replays, with eager launches and synchronisations between
    them and the outputs cleared before each, give the eager step's bytes; after an edit of the resident
    plans in place the replay gives the edited batch's results."""
    from superscaler_amd.evaluator import PlanEvaluator
    torch = torch_mod
    w = synth.WORKLOADS["gpt3_13b"]
    tables = synth.make_tables(w)
    batch = synth.make_plans(w, tables, n_plans=200000, seed_offset=12, workers=4)
    ev = PlanEvaluator(tables)
    d = ev.upload(batch)
    eager = ev.score(d)
    etop = ev.topk(eager[0], eager[2], 64)
    torch.cuda.synchronize()
    want = [t.clone() for t in eager] + [t.clone() for t in etop]
    g = ev.capture_step(d, 64)
    for r in range(4):
        for t in g.scores:
            t.zero_()
        (scores, top) = g.replay()
        torch.cuda.synchronize()
        assert all(torch.equal(a, b) for a, b in zip(list(scores) + list(top), want)), r
        other = ev.score(ev.upload(batch.slice(0, 5000)))          # eager work between the replays
        ev.topk(other[0], other[2], 8)
        torch.cuda.synchronize()
    # edit in place: clear every recompute bit of the resident plans, replay, compare with a fresh eager step
    d.codes &= 0xF7
    (scores, top) = g.replay()
    torch.cuda.synchronize()
    fresh = ev.score(d)
    ftop = ev.topk(fresh[0], fresh[2], 64)
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip(list(scores) + list(top), list(fresh) + list(ftop)))
    assert not torch.equal(scores[1], want[1])
    # a larger batch would make the library reallocate the workspace whose address the graph holds
    from superscaler_amd.evaluator import AceError
    bigger = ev.upload(synth.make_plans(w, tables, n_plans=201000, seed_offset=13, workers=4))
    with pytest.raises(AceError):
        ev.score(bigger)
    # ... whichever call gets there: the library itself refuses (ace_reserve fixed the workspace)
    with pytest.raises(AceError):
        ev.time_score_kernel(bigger, 1)
    # a larger top-k takes a workspace of its own; the recorded one stays alive with the graph
    ev.topk(fresh[0], fresh[2], 4096)
    junk = [torch.full((1 << 20,), 7, dtype=torch.uint8, device="cuda") for _ in range(8)]     # what the allocator might hand out again
    (scores, top) = g.replay()
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip(list(scores) + list(top), list(fresh) + list(ftop)))
    del junk
    g.release()
    ev.score(bigger)
    with pytest.raises(AceError):
        g.replay()
    torch.cuda.synchronize()
    ev.close()


def test_known_answers_single_gpu_plans(golden_dir, torch_mod):
    """The reference tree's own single-GPU plans and published predictions
    (results/ref/perf_model_{time,mem}_large_{gpt,resnet}.csv), through the GPU path."""
    from superscaler_amd import aceso_cost_model as acm
    from superscaler_amd.plan import config_from_json
    kat = os.path.join(golden_dir, "kat") + "/"
    st = CostModelSettings(model_name="gpt", micro_batch_size=[1, 2, 4, 8], num_gpus_per_node=1, global_batch_size=1024)
    m = acm.CostModel.from_directory(st, "gpt", "350M", kat, num_layers=24)
    cfg = config_from_json(kat + "gpt_350M_mbs8_recomp.json", m.graph.ops)
    m.predict_time_breakdown(cfg)
    assert f"{max(cfg.time_list) / 1000:.2f}" == "200.71"
    assert abs(max(cfg.time_list) - 200712.935038) < 1e-5
    reserved = m.get_reserved_memory_list(cfg)
    assert reserved == [5120.0] and abs(cfg.memory_list[0] - 19712.64) < 1e-6
    m.close()
    st = CostModelSettings(model_name="resnet", micro_batch_size=[16, 32, 48, 64], num_gpus_per_node=1, global_batch_size=1536)
    m = acm.CostModel.from_directory(st, "resnet", "500M", kat)
    cfg = config_from_json(kat + "resnet_500M_mbs64_recomp.json", m.graph.ops)
    m.predict_time_breakdown(cfg)
    reserved = m.get_reserved_memory_list(cfg)
    assert reserved == [3432.0] and int(cfg.memory_list[0] - reserved[0]) == 16519
    assert abs(max(cfg.time_list) / 1000 - 67.13) / 67.13 < 0.005
    m.close()


def _tiny_gpt(num_layers, pp_choices, num_gpus=16):
    import dataclasses
    w = dataclasses.replace(synth.WORKLOADS["gpt3_13b"], name=f"tiny{num_layers}", num_layers=num_layers,
                            num_gpus=num_gpus, pp_choices=pp_choices, memory_limit=30000.0)
    tables = synth.make_tables(w)
    return w, tables


@pytest.mark.parametrize("layers,pp,n_plans", [(1, [16], 1), (1, [16], 1025), (1, [1, 2], 64), (5, [1, 4, 16], 3000)])
def test_edge_shapes(layers, pp, n_plans, torch_mod):
    """Op count a multiple of 16 (one layer = 16 ops), every op its own stage (16 stages on 16 ops),
    a single plan, a plan count that is not a multiple of the workgroup size."""
    from superscaler_amd.evaluator import PlanEvaluator
    w, tables = _tiny_gpt(layers, pp)
    assert tables.graph.num_ops == 13 * layers + 3
    batch = synth.make_plans(w, tables, n_plans=n_plans)
    ev = PlanEvaluator(tables)
    it, pk, fe, st = ev.score_host(batch)
    it2, pk2, fe2, st2, rec = ev.score_host(batch, breakdown=True)
    orc = oracle_for(tables)
    n = min(n_plans, 200)
    oit, opk, ofe, _ = oracle_scores(orc, batch, tables, idx=range(n))
    assert (st == 0).all()
    assert np.array_equal(it[:n], oit) and np.array_equal(pk[:n], opk) and np.array_equal(fe[:n], ofe)
    assert np.array_equal(it, it2) and np.array_equal(pk, pk2) and np.array_equal(fe, fe2)
    eit, epk, efe, _, _ = emu_score(tables, batch)
    assert np.array_equal(it, eit) and np.array_equal(pk, epk)
    d = ev.upload(batch)
    dit, dpk, dfe, dst = ev.score(d)
    idx, val, cnt = ev.topk(dit, dfe, 5)
    order = np.lexsort((np.arange(n_plans), np.where(fe > 0, it, np.inf)))[:min(5, int(fe.sum()))]
    assert np.array_equal(idx.cpu().numpy()[:len(order)], order)
    ev.close()


def test_bytes_past_the_last_op_are_ignored(torch_mod):
    """The 16-byte words of the last op group are padded; whatever sits in the padding must not matter."""
    from superscaler_amd.evaluator import PlanEvaluator
    w = synth.WORKLOADS["gpt3_13b"]                      # 523 ops: 11 real bytes + 5 of padding in the last word
    tables = synth.make_tables(w)
    batch = synth.make_plans(w, tables, n_plans=3000, seed_offset=4)
    ev = PlanEvaluator(tables)
    d = ev.upload(batch)
    clean = [t.cpu().numpy() for t in ev.score(d)]
    assert batch.num_ops % 16 != 0
    d.codes[-1, :, batch.num_ops % 16:] = 0xFF
    dirty = [t.cpu().numpy() for t in ev.score(d)]
    _, _, _, _, rec_dirty = [t.cpu().numpy() for t in ev.score(d, breakdown=True)]
    for a, b in zip(clean, dirty):
        assert np.array_equal(a, b)
    eit, epk, _, _, erec = emu_score(tables, batch.slice(0, 64), breakdown=True)
    assert np.array_equal(rec_dirty[:64], erec) and (clean[3] == 0).all()
    ev.close()


def test_unscorable_and_malformed_plans_are_flagged(torch_mod):
    """A micro-batch / stage-size pair outside the profiled grid gives NaN + status 1 (the reference
    raises KeyError); inconsistent stage bits give status 3; neighbours in the batch are unaffected."""
    from superscaler_amd.evaluator import PlanEvaluator
    w, tables = _tiny_gpt(5, [1, 2, 4])
    batch = synth.make_plans(w, tables, n_plans=64)
    ev = PlanEvaluator(tables)
    it0, pk0, fe0, st0 = ev.score_host(batch)
    bad = PlanBatch(batch.codes.copy(), batch.hdr.copy())
    bad.hdr[3, 0] = (bad.hdr[3, 0] & 0xff) | (0 << 8)      # micro-batch 1 ...
    bad.hdr[3, 1] = 0x4444                                  # ... on 16-device stages: 1 // dp is not profiled
    bad.hdr[3, 0] = 4                                       # (and claim four stages)
    bad.codes[3] &= 0xEF
    bad.codes[3, [0, 10, 20, 30]] |= 16
    bad.codes[7, 5] |= 16                                   # one stage bit more than num_stages says
    d = ev.upload(bad, validate=False)
    it, pk, fe, st = [t.cpu().numpy() for t in ev.score(d)]
    assert st[3] == 1 and np.isnan(it[3]) and np.isnan(pk[3]) and fe[3] == 0
    assert st[7] == 3 and fe[7] == 0
    keep = np.ones(64, dtype=bool)
    keep[[3, 7]] = False
    assert (st[keep] == 0).all() and np.array_equal(it[keep], it0[keep]) and np.array_equal(fe[keep], fe0[keep])
    ev.close()


@pytest.mark.parametrize("name", ["gpt3_13b", "wresnet_1b"])
def test_plans_around_the_sixteen_stage_limit_agree_with_the_breakdown_kernel(name, torch_mod):
    """The assembly op loop counts a plan's stages by the offset of its next workspace record and stops storing records
    at the sixteenth: plans cut into 15, 16, 17, 18 and 40 stages, with headers that claim that count or 16, must come
    out of plain scoring (assembly loop) exactly as out of the per-stage breakdown (C++ loop) -- a seventeenth stage is a
    malformed plan whatever the header says, and must not touch another plan's records."""
    from superscaler_amd.evaluator import PlanEvaluator
    w = synth.WORKLOADS[name]
    tables = synth.make_tables(w)
    n = 4096
    good = synth.make_plans(w, tables, n_plans=n, seed_offset=88, workers=8)
    bad = PlanBatch(good.codes.copy(), good.hdr.copy())
    N = bad.codes.shape[1]
    rng = np.random.default_rng(5)
    counts = [15, 16, 17, 18, 40]
    counts = [c for c in counts if c <= N]
    touched = np.zeros(n, dtype=bool)
    for r in range(0, n, 3):
        c = counts[(r // 3) % len(counts)]
        cuts = np.sort(rng.choice(np.arange(1, N), size=c - 1, replace=False))
        bad.codes[r] &= np.uint8(0xef)
        bad.codes[r, 0] |= 16
        bad.codes[r, cuts] |= 16
        claim = c if (r // 3) % 2 == 0 else 16
        bad.hdr[r, 0] = (bad.hdr[r, 0] & ~np.uint32(0xff)) | np.uint32(claim)
        touched[r] = True
    ev = PlanEvaluator(tables)
    d = ev.upload(bad, validate=False)
    it, pk, fe, st = [t.cpu().numpy() for t in ev.score(d)]
    bit, bpk, bfe, bst, _ = [t.cpu().numpy() for t in ev.score(d, breakdown=True)]
    assert np.array_equal(st, bst) and np.array_equal(fe, bfe)
    assert np.array_equal(it, bit, equal_nan=True) and np.array_equal(pk, bpk, equal_nan=True)
    # more than sixteen stages: never a valid plan
    over = np.array([touched[r] and counts[(r // 3) % len(counts)] > 16 for r in range(n)])
    assert (st[over] != 0).all() and not fe[over].any()
    # their neighbours in the batch (and in the workgroup's workspace) are untouched
    git, gpk, gfe, gst = ev.score_host(good)
    assert np.array_equal(it[~touched], git[~touched]) and np.array_equal(pk[~touched], gpk[~touched])
    ev.close()


@pytest.mark.parametrize("name,n", [("gpt3_13b", 20000), ("gpt3_13b", 140000), ("wresnet_1b", 20000), ("t5_770m", 20000)])
def test_corrupted_batches_plain_scoring_equals_the_breakdown_kernel(name, n, torch_mod):
    """Plain scoring runs the assembly op loop (over windowed rows for wresnet_1b), the per-stage breakdown the C++ loop
    (which the CPU suite runs on random bytes against the state machine): on batches with flipped stage and recompute
    bits, stage counts that do not match, micro-batch indices and stage sizes outside the tables, both must give the same
    times, memories, flags and status bytes, plan by plan -- and leave the untouched plans of the batch as they were."""
    from superscaler_amd.evaluator import PlanEvaluator
    w = synth.WORKLOADS[name]
    tables = synth.make_tables(w)
    good = synth.make_plans(w, tables, n_plans=n, seed_offset=61, workers=8)
    rng = np.random.default_rng(17)
    bad = PlanBatch(good.codes.copy(), good.hdr.copy())
    N = bad.codes.shape[1]
    hit = rng.random(n) < 0.3
    rows = np.flatnonzero(hit)
    kind = rng.integers(0, 6, len(rows))
    for r, kd in zip(rows, kind):
        if kd == 0:
            bad.codes[r, rng.integers(1, N, 3)] ^= 16                      # stage bits set or cleared
        elif kd == 1:
            bad.codes[r, rng.integers(0, N, 5)] ^= 8                       # recompute bits
        elif kd == 2:
            bad.hdr[r, 0] = (bad.hdr[r, 0] & ~np.uint32(0xff)) | np.uint32(rng.integers(0, 40))    # stage count
        elif kd == 3:
            bad.hdr[r, 0] = (bad.hdr[r, 0] & np.uint32(0xff)) | np.uint32(int(rng.integers(0, 16)) << 8)   # micro-batch index
        elif kd == 4:
            bad.hdr[r, 1] = np.uint32(rng.integers(0, 1 << 32))            # stage sizes
        else:
            bad.codes[r] = rng.integers(0, 32, N, dtype=np.uint8)          # every byte random (five bits used)
            bad.codes[r, 0] |= 16
    ev = PlanEvaluator(tables)
    d = ev.upload(bad, validate=False)
    it, pk, fe, st = [t.cpu().numpy() for t in ev.score(d)]
    bit, bpk, bfe, bst, _ = [t.cpu().numpy() for t in ev.score(d, breakdown=True)]
    assert np.array_equal(st, bst) and np.array_equal(fe, bfe)
    assert np.array_equal(it, bit, equal_nan=True) and np.array_equal(pk, bpk, equal_nan=True)
    git, gpk, gfe, gst = ev.score_host(good)
    assert (gst == 0).all() and len(set(st[hit].tolist())) >= 3
    assert np.array_equal(it[~hit], git[~hit]) and np.array_equal(pk[~hit], gpk[~hit]) and np.array_equal(fe[~hit], gfe[~hit])
    ev.close()


def test_streamed_batches_match_one_shot(torch_mod):
    """GPT-3 175B-shaped graph (1,251 ops), plans streamed in batches with overlapped upload: the
    merged top-k equals the top-k of the same plans scored in one piece."""
    from superscaler_amd.evaluator import PlanEvaluator
    w = synth.WORKLOADS["gpt3_175b"]
    tables = synth.make_tables(w)
    ev = PlanEvaluator(tables)
    parts = [synth.make_plans(w, tables, n_plans=8192, seed_offset=100 + j) for j in range(4)]
    limit = 400000.0        # a cap that leaves some of these 64-GPU-per-stage plans feasible
    idx, val, seen = ev.score_stream(iter(parts), k=32, memory_limit=limit)
    assert seen == 4 * 8192
    whole = PlanBatch.concat(parts)
    it, pk, fe, st = ev.score_host(whole, memory_limit=limit)
    order = np.lexsort((np.arange(len(it)), np.where(fe > 0, it, np.inf)))[:min(32, int(fe.sum()))]
    assert int(fe.sum()) > 0
    assert np.array_equal(idx, order) and np.array_equal(val, it[order])
    ev.close()
