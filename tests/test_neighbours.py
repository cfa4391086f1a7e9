"""Array-form neighbour moves stay on the profiled grid and score exactly like the oracle; the
batched local search only ever accepts plans the oracle agrees are feasible and faster."""
import numpy as np
import pytest

from superscaler_amd import synth
from superscaler_amd.neighbours import (VisitedKeys, VisitedPlans, apply_moves_host, hill_climb, make_neighbours,
                                        plan_keys_host, sample_moves)
from superscaler_amd.plan import PlanBatch, config_details, is_visited, mark_visited, num_visited, validate_batch
from tests.helpers import emu_score, oracle_for, oracle_scores


@pytest.mark.parametrize("name", ["gpt3_1_3b", "gpt3_13b", "t5_770m"])
def test_neighbours_are_valid_and_score_like_the_oracle(name):
    w = synth.WORKLOADS[name]
    tables = synth.make_tables(w)
    base = synth.make_plans(w, tables, n_plans=8, seed_offset=3)
    rng = np.random.default_rng(5)
    orc = oracle_for(tables)
    changed = 0
    for p in range(4):
        nb = make_neighbours(base.slice(p, p + 1), tables, 96, rng)
        assert validate_batch(nb, tables) is None
        it, pk, fe, st, _ = emu_score(tables, nb)
        assert (st == 0).all(), "a move left the profiled grid"
        oit, opk, ofe, _ = oracle_scores(orc, nb, tables, idx=range(0, 96, 3))
        assert np.array_equal(it[::3], oit) and np.array_equal(pk[::3], opk) and np.array_equal(fe[::3], ofe)
        changed += int((nb.codes != base.codes[p]).any(axis=1).sum() + (nb.hdr != base.hdr[p]).any(axis=1).sum())
        # device counts are preserved by every move
        g = lambda h: sum(1 << ((int(h[1]) | (int(h[2]) << 32)) >> (4 * s) & 15) for s in range(int(h[0]) & 0xff))
        assert all(g(h) == w.num_gpus for h in nb.hdr)
    assert changed > 100


def test_visited_set_matches_the_reference_string_key():
    """Two plans share a key iff their config_details strings (the reference's visited key) are equal."""
    w = synth.WORKLOADS["gpt3_1_3b"]
    tables = synth.make_tables(w)
    base = synth.make_plans(w, tables, n_plans=2, seed_offset=7)
    nb = make_neighbours(base.slice(0, 1), tables, 300, np.random.default_rng(2))
    batch = PlanBatch.concat([base, nb])
    strings = [config_details(batch.to_config(p, tables), get_string=True) for p in range(batch.n_plans)]
    keys = [k.tobytes() for k in VisitedPlans.keys(batch)]
    for a in range(0, batch.n_plans, 7):
        for b in range(batch.n_plans):
            assert (strings[a] == strings[b]) == (keys[a] == keys[b])
    assert len(set(strings)) < batch.n_plans      # the sample does contain repeats
    vs = VisitedPlans()
    first = vs.unseen(batch)
    assert first.sum() == len(set(strings)) and first[0]
    seen = set()
    for p in range(batch.n_plans):                # exactly the first occurrence of every string is kept
        assert first[p] == (strings[p] not in seen)
        seen.add(strings[p])
    vs.mark(batch, rows=np.flatnonzero(first)[:10])
    again = vs.unseen(batch)
    assert again.sum() == first.sum() - 10 and len(vs) == 10
    # the reference's dict-of-lists helpers
    d = {}
    assert not is_visited(d, "k", 1) and num_visited(d, "k") == 0
    mark_visited(d, "k", 1)
    mark_visited(d, "k", 2)
    assert is_visited(d, "k", 2) and not is_visited(d, "k", 3) and num_visited(d, "k") == 2
    assert config_details(None) == ""


def test_plan_keys_separate_distinct_plans_and_key_set_behaves():
    w = synth.WORKLOADS["gpt3_13b"]
    tables = synth.make_tables(w)
    base = synth.make_plans(w, tables, n_plans=3, seed_offset=8)
    nb = PlanBatch.concat([make_neighbours(base.slice(p, p + 1), tables, 4000, np.random.default_rng(p)) for p in range(3)])
    keys = plan_keys_host(nb)
    assert keys.shape == (nb.n_plans, 2) and keys.dtype == np.uint64
    first = VisitedPlans().unseen(nb)
    as_tuples = [tuple(k) for k in keys.tolist()]
    assert len(set(as_tuples)) == int(first.sum())             # no collision, no split
    # (either half alone separates these plans too: the two mixing functions are independent)
    assert len(np.unique(keys[:, 0])) == int(first.sum()) and len(np.unique(keys[:, 1])) == int(first.sum())
    vk = VisitedKeys()
    assert np.array_equal(vk.unseen(keys), first)
    vk.mark(keys[:5000])
    seen = set(as_tuples[:5000])
    want = first & ~np.array([k in seen for k in as_tuples])
    assert np.array_equal(vk.unseen(keys), want)
    assert len(vk) == len(seen)
    # the same after the small array has been folded into the large one, and with keys marked twice
    vk.SMALL_LIMIT = 100
    vk.mark(keys[4000:5000])
    assert len(vk._small) == 0 and len(vk) == len(seen) and np.array_equal(vk.unseen(keys), want)
    vk.mark(keys[4500:5500])
    seen |= set(as_tuples[5000:5500])
    want = first & ~np.array([k in seen for k in as_tuples])
    assert len(vk) == len(seen) and np.array_equal(vk.unseen(keys), want)
    # a header-only change (another micro-batch size) changes both halves of the key
    h = nb.hdr.copy()
    h[:, 0] ^= 1 << 8
    assert not np.any(plan_keys_host(PlanBatch(nb.codes, h)) == keys)


def test_plans_that_collide_in_one_half_of_the_key_stay_distinct():
    """Two plans whose first 64-bit key words are equal (a collision of one mixing function: crafted here by
    overwriting that word, which is what a 64-bit visited set would have seen) are still two plans to VisitedKeys, in
    the batch, in the small array and in the large one; the reference's string sets never confuse plans
    (aceso_utils.py:831-850)."""
    w = synth.WORKLOADS["gpt3_1_3b"]
    tables = synth.make_tables(w)
    nb = make_neighbours(synth.make_plans(w, tables, n_plans=1, seed_offset=3), tables, 64, np.random.default_rng(0))
    keys = plan_keys_host(nb)
    distinct = np.flatnonzero(VisitedPlans().unseen(nb))[:6]
    k = keys[distinct].copy()
    k[:, 0] = k[0, 0]                                 # all six collide in the first half
    assert len({tuple(x) for x in k.tolist()}) == 6
    vk = VisitedKeys()
    assert vk.unseen(k).all()                         # within one batch
    vk.mark(k[:2])
    assert vk.unseen(k).tolist() == [False, False, True, True, True, True]     # against the small array
    vk.SMALL_LIMIT = 1
    vk.mark(k[2:4])
    assert len(vk._small) == 0 and len(vk) == 4
    assert vk.unseen(k).tolist() == [False, False, False, False, True, True]   # against the large array
    # and the same plan twice is one plan
    assert vk.unseen(np.concatenate([k[4:5], k[4:5]])).tolist() == [True, False]


@pytest.mark.gpu
def test_hill_climb_improves_and_agrees_with_the_oracle():
    from superscaler_amd.aceso_cost_model import CostModel
    w = synth.WORKLOADS["gpt3_1_3b"]
    graph = synth.make_graph(w)
    cm = CostModel(synth.make_settings(w), synth.make_db(w, graph), graph)
    start = synth.make_plans(w, cm.tables, n_plans=1, seed_offset=11)
    trace = []
    visited = VisitedPlans()
    plan, t, m = hill_climb(cm, start, steps=20, n_neighbours=2048, seed=1, on_step=lambda s, t, m: trace.append(t),
                            visited=visited)
    assert len(visited) > 20
    orc = oracle_for(cm.tables)
    (t0,), _, (f0,), _ = oracle_scores(orc, start, cm.tables)
    (t1,), (m1,), (f1,), _ = oracle_scores(orc, plan, cm.tables)
    assert f1 == 1 and t1 == t and m1 == m
    assert t1 < t0 or not f0
    assert all(a >= b for a, b in zip(trace, trace[1:]))
    # with check_recompute applied to every neighbour the accepted plan carries exactly those bits
    plan2, t2, m2 = hill_climb(cm, start, steps=6, n_neighbours=512, seed=2, greedy_recompute=True)
    assert np.array_equal(cm.update_recompute_arrays(plan2).codes, plan2.codes) or t2 == (t0 if f0 else float("inf"))
    (t3,), (m3,), (f3,), _ = oracle_scores(orc, plan2, cm.tables)
    assert (f3 == 1 and t3 == t2 and m3 == m2) or t2 == float("inf")
    # neighbours expanded on the device from move descriptors: the plan handed back scores as reported
    vkeys = VisitedKeys()
    plan4, t4, m4 = hill_climb(cm, start, steps=10, n_neighbours=2048, seed=3, device_moves=True, visited=vkeys)
    assert len(vkeys) > 100
    (t5,), (m5,), (f5,), _ = oracle_scores(orc, plan4, cm.tables)
    assert (f5 == 1 and t5 == t4 and m5 == m4 and t4 < t0) or not f0
    # the same with check_recompute's choice made on the device for every neighbour
    plan6, t6, m6 = hill_climb(cm, start, steps=6, n_neighbours=1024, seed=4, device_moves=True, visited=VisitedKeys(),
                               greedy_recompute=True)
    assert np.array_equal(cm.update_recompute_arrays(plan6).codes, plan6.codes) or t6 == (t0 if f0 else float("inf"))
    (t7,), (m7,), (f7,), _ = oracle_scores(orc, plan6, cm.tables)
    assert (f7 == 1 and t7 == t6 and m7 == m6) or t6 == float("inf")
    cm.close()


@pytest.mark.gpu
def test_stream_and_search_demo_runs(capsys):
    """The end-to-end demo (streamed batches -> global top-k -> batched local search) at a small size."""
    import json
    from superscaler_amd import search_demo
    search_demo.main(["--workload", "gpt3_1_3b", "--stream-plans", "10000", "--batch", "4096", "--steps", "4",
                      "--neighbours", "512", "--greedy-recompute", "--workers", "2"])
    out = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert out["streamed_plans"] == 10000 and out["batches"] == 3
    assert out["search_best_ms"] <= out["search_start_ms"]


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["gpt3_1_3b", "gpt3_13b", "t5_770m", "wresnet_1b"])
def test_moves_expand_on_the_device_like_on_the_host(name):
    """ace_apply_moves writes byte for byte what apply_moves_host builds, in the kernel's layout,
    and the batch scores the same either way."""
    import torch
    from superscaler_amd.evaluator import PlanEvaluator
    w = synth.WORKLOADS[name]
    tables = synth.make_tables(w)
    ev = PlanEvaluator(tables)
    rng = np.random.default_rng(11)
    for p in range(3):
        base = synth.make_plans(w, tables, n_plans=4, seed_offset=40 + p).slice(p, p + 1)
        templates, moves = sample_moves(base, tables, 5000, rng)
        host = apply_moves_host(templates, moves, tables.db.n_algo)
        assert len(np.unique(moves[:, 0] >> 16)) >= 2
        d = ev.apply_moves(templates, moves)
        N, G = host.num_ops, (host.num_ops + 15) // 16
        got = d.codes.permute(1, 0, 2).reshape(host.n_plans, G * 16).cpu().numpy()
        assert np.array_equal(got[:, :N], host.codes) and not got[:, N:].any()
        assert np.array_equal(d.hdr.cpu().numpy().view(np.uint32), host.hdr)
        # the plan keys of the kernel = the host's, and they separate exactly the distinct plans of the batch
        d2, keys = ev.apply_moves(templates, moves, with_keys=True)
        keys = keys.cpu().numpy().view(np.uint64)
        assert np.array_equal(keys, plan_keys_host(host))
        assert len({tuple(k) for k in keys.tolist()}) == int(VisitedPlans().unseen(host).sum())
        vk = VisitedKeys()
        first = vk.unseen(keys)
        assert np.array_equal(first, VisitedPlans().unseen(host))
        vk.mark(keys[first][:7])
        assert vk.unseen(keys).sum() == first.sum() - 7
        a = [t.cpu().numpy() for t in ev.score(d)]
        b = ev.score_host(host)
        for x, y in zip(a, b):
            assert np.array_equal(x, y, equal_nan=True)
    ev.close()
