"""Array-form neighbour moves stay on the profiled grid and score exactly like the oracle; the
batched local search only ever accepts plans the oracle agrees are feasible and faster."""
import numpy as np
import pytest

from superscaler_amd import synth
from superscaler_amd.neighbours import hill_climb, make_neighbours
from superscaler_amd.plan import validate_batch
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


@pytest.mark.gpu
def test_hill_climb_improves_and_agrees_with_the_oracle():
    from superscaler_amd.aceso_cost_model import CostModel
    w = synth.WORKLOADS["gpt3_1_3b"]
    graph = synth.make_graph(w)
    cm = CostModel(synth.make_settings(w), synth.make_db(w, graph), graph)
    start = synth.make_plans(w, cm.tables, n_plans=1, seed_offset=11)
    trace = []
    plan, t, m = hill_climb(cm, start, steps=20, n_neighbours=2048, seed=1, on_step=lambda s, t, m: trace.append(t))
    orc = oracle_for(cm.tables)
    (t0,), _, (f0,), _ = oracle_scores(orc, start, cm.tables)
    (t1,), (m1,), (f1,), _ = oracle_scores(orc, plan, cm.tables)
    assert f1 == 1 and t1 == t and m1 == m
    assert t1 < t0 or not f0
    assert all(a >= b for a, b in zip(trace, trace[1:]))
    cm.close()
