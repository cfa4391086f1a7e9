"""The kernel's per-plan state machine (compiled for the CPU with bounds checks) and the table
compiler, against the oracle: every value bit-identical."""
import numpy as np
import pytest

from superscaler_amd import synth
from superscaler_amd.tables import (R_ACT, R_BWD, R_FWD, R_IDEAL_BWD, R_IDEAL_FWD, R_IDEAL_IN, R_IDEAL_OUT,
                                    R_IN_COMM, R_INPUTS, R_OUT_COMM, R_PEAK, R_RECOMP, R_RESERVED, R_SAVED,
                                    R_STAGE_MB, R_STAGE_MS, R_WEIGHTS)
from tests.helpers import emu_score, oracle_for, oracle_scores

CASES = [("gpt3_1_3b", 96), ("t5_770m", 48), ("wresnet_1b", 128), ("gpt3_13b", 96), ("gpt3_175b", 16)]


@pytest.fixture(scope="module", params=CASES, ids=[c[0] for c in CASES])
def case(request):
    name, n = request.param
    w = synth.WORKLOADS[name]
    tables = synth.make_tables(w)
    batch = synth.make_plans(w, tables, n_plans=n)
    return w, tables, batch, oracle_for(tables)


def test_scores_bit_exact(case):
    w, tables, batch, orc = case
    oit, opk, ofe, _ = oracle_scores(orc, batch, tables)
    for defer in (False, True):     # stage tails evaluated in place / stashed and replayed after the op loop
        it, pk, fe, st, _ = emu_score(tables, batch, defer=defer)
        assert (st == 0).all()
        assert np.array_equal(it, oit)
        assert np.array_equal(pk, opk)
        assert np.array_equal(fe, ofe)
    # strict comparison flips only plans that sit exactly on the limit
    it2, pk2, fe2, _, _ = emu_score(tables, batch, memory_limit=float(np.median(opk)), strict=True)
    assert np.array_equal(fe2, (opk < float(np.median(opk))).astype(np.uint8))


def test_stage_records_bit_exact(case):
    w, tables, batch, orc = case
    it, pk, fe, st, rec = emu_score(tables, batch, breakdown=True)
    it0, pk0, _, _, _ = emu_score(tables, batch)
    assert np.array_equal(it, it0) and np.array_equal(pk, pk0)
    for p in range(min(batch.n_plans, 24)):
        cfg = batch.to_config(p, tables)
        from tests.helpers import oracle_config
        oc = oracle_config(batch, p, tables)
        gpn = tables.settings.num_gpus_per_node
        till = 0
        for s, stg in enumerate(oc.stages):
            mbs = [oc.micro_bs // d for d in stg.dp_size]
            in_cross = (till % gpn == 0) and till > 0
            till += stg.num_gpus
            out_cross = till % gpn == 0
            f, b, ic, ocm, _ = orc.get_time_v3(stg.ops, mbs, stg.tp_size, stg.algo, stg.dp_size, in_cross, out_cross)
            r = rec[p, s]
            assert (r[R_FWD], r[R_BWD], r[R_IN_COMM], r[R_OUT_COMM]) == (f, b, ic, ocm)
            assert r[R_RECOMP] == orc.get_recompute_time_v3(stg.ops, stg.recompute_ops, mbs, stg.tp_size, stg.algo)
            wts, inputs, acts = orc.get_memory_v3(stg.ops, mbs, stg.tp_size, stg.algo)
            assert (r[R_WEIGHTS], r[R_INPUTS], r[R_ACT]) == (wts, inputs, acts)
            assert r[R_SAVED] == orc.get_activations_v3(stg.ops, stg.recompute_ops, mbs, stg.tp_size, stg.algo)
            assert r[R_PEAK] == orc.get_peak_activations(stg.ops, stg.recompute_ops, mbs, stg.tp_size, stg.algo)
            assert r[R_RESERVED] == orc.get_reserved_memory(stg.ops, mbs, stg.tp_size, stg.dp_size, stg.algo, wts)
            n = len(stg.ops)
            f1, b1, i1, o1, _ = orc.get_time_v3(stg.ops, [oc.micro_bs] * n, [1] * n, stg.algo, [1] * n, in_cross, out_cross)
            assert (r[R_IDEAL_FWD], r[R_IDEAL_BWD], r[R_IDEAL_IN], r[R_IDEAL_OUT]) == (f1, b1, i1, o1)
            assert r[R_STAGE_MB] == orc.predict_stage_memory(stg.ops, stg.recompute_ops, stg.tp_size, stg.dp_size,
                                                             oc.micro_bs, stg.num_stages_behind, stg.algo)
            assert r[R_STAGE_MS] == (f + b + ic + ocm + r[R_RECOMP]) / 1000


@pytest.mark.parametrize("name", list(synth.WORKLOADS))
def test_row_windows_never_restage_in_the_padding(name):
    """The kernel walks 16 * ceil(N / 16) positions (the last group is padded) and restages rows where a
    position equals the next window start: that may happen n_windows - 1 times, never in the padding
    (for N = 134 a final entry of 136 would be met at padded position 136 and index past the window arrays)."""
    t = synth.make_tables(synth.WORKLOADS[name])
    N = t.graph.num_ops
    walked = 16 * ((N + 15) // 16)
    wp = [int(x) for x in t.win_pos]
    assert wp[0] == 0 and len(wp) == t.n_windows + 1 and len(t.win_row_begin) == t.n_windows + 1
    assert all(a < b and a % 4 == 0 and a < N for a, b in zip(wp[:-1], wp[1:]))
    assert wp[-1] >= walked
    w, next_win, restaged = 1, wp[1], 0
    for i in range(walked):
        if i % 4 == 0 and i == next_win:
            assert w < t.n_windows
            restaged += 1
            w += 1
            next_win = wp[w]
    assert restaged == t.n_windows - 1


def settings_matrix():
    """Every combination of the switches that change what the model returns (aceso_utils.py:359-531)."""
    import itertools
    for pred, shared, reserved, resh, pmb in itertools.product(("MAX", "MIN"), (True, False), (True, False), (True, False), (0, 1500)):
        yield dict(memory_pred_type=pred, consider_shared_space=shared, consider_reserved_space=reserved,
                   resharding=resh, peak_mem_in_backward=pmb)
        if resh and reserved and pmb == 0:      # where the collectives' buffers can enter the reserved memory (:462-483)
            yield dict(memory_pred_type=pred, consider_shared_space=shared, consider_reserved_space=reserved,
                       resharding=resh, peak_mem_in_backward=pmb, consider_collective_memory=True)


@pytest.mark.parametrize("name", ["gpt3_1_3b", "wresnet_1b"])
def test_every_settings_combination_matches_the_oracle(name):
    """MAX / MIN memory prediction, shared-buffer rule, reserved space, resharding on and off (peak_mem_in_backward
    only enters check_recompute): kernel source on the CPU (stage tails in place and deferred, stage records) and
    the C restatement against the Python oracle, bit for bit."""
    import dataclasses
    from superscaler_amd.tables import compile_tables
    from tests.helpers import c_oracle_scores
    w = synth.WORKLOADS[name]
    graph = synth.make_graph(w)
    db = synth.make_db(w, graph)
    base = synth.make_tables(w)
    batch = synth.make_plans(w, base, n_plans=24, seed_offset=77)
    seen = set()
    for kw in settings_matrix():
        st = dataclasses.replace(synth.make_settings(w), **kw)
        tables = compile_tables(graph, db, st)
        orc = oracle_for(tables)
        oit, opk, ofe, cfgs = oracle_scores(orc, batch, tables)
        for defer in (False, True):
            it, pk, fe, status, _ = emu_score(tables, batch, defer=defer)
            assert (status == 0).all() and np.array_equal(it, oit) and np.array_equal(pk, opk) and np.array_equal(fe, ofe), kw
        cit, cpk, cfe, cer = c_oracle_scores(tables, batch)
        assert not cer.any() and np.array_equal(cit, oit) and np.array_equal(cpk, opk) and np.array_equal(cfe, ofe), kw
        _, _, _, _, rec = emu_score(tables, batch, breakdown=True)
        for p, c in enumerate(cfgs):
            assert [rec[p, s, R_STAGE_MB] for s in range(c.num_stages)] == list(c.memory_list), kw
        seen.add((tuple(opk.tolist()), tuple(oit.tolist())))
    assert len(seen) >= 10         # the switches do change the answers


def test_odd_table_geometries():
    """Corners of the table geometry (see helpers.odd_workloads): state machine, the kernel's own loop and the C
    restatement against the Python oracle, bit for bit."""
    from tests.helpers import c_oracle_scores, emu_kernel_score, odd_workloads
    shapes = set()
    for w in odd_workloads():
        tables = synth.make_tables(w)
        batch = synth.make_plans(w, tables, n_plans=w.n_plans)
        orc = oracle_for(tables)
        oit, opk, ofe, _ = oracle_scores(orc, batch, tables)
        for defer in (False, True):
            it, pk, fe, st, _ = emu_score(tables, batch, defer=defer)
            assert (st == 0).all() and np.array_equal(it, oit) and np.array_equal(pk, opk) and np.array_equal(fe, ofe), w.name
        out = emu_kernel_score(tables, batch)
        assert np.array_equal(out[0], oit) and np.array_equal(out[1], opk) and np.array_equal(out[2], ofe), w.name
        cit, cpk, cfe, cer = c_oracle_scores(tables, batch)
        assert not cer.any() and np.array_equal(cit, oit) and np.array_equal(cpk, opk) and np.array_equal(cfe, ofe), w.name
        shapes.add((tables.graph.num_ops, len(tables.db.tp_list), len(tables.db.mbs_list), tables.n_windows))
    assert len(shapes) == 10
