"""The C oracle (oracle/aceso_oracle.c) bit for bit against the Python oracle and against the
vectors the reference itself wrote."""
import numpy as np
import pytest

from oracle.c_oracle import COracle
from superscaler_amd import synth
from superscaler_amd.plan import PlanBatch
from tests.helpers import c_oracle_scores, oracle_config, oracle_for, oracle_scores
from tests.test_oracle_golden import CASES, load_case, make_config


@pytest.mark.parametrize("name", list(synth.WORKLOADS))
def test_c_oracle_equals_python_oracle(name):
    w = synth.WORKLOADS[name]
    tables = synth.make_tables(w)
    n = 160 if w.name != "gpt3_175b" else 48
    batch = synth.make_plans(w, tables, n_plans=n, seed_offset=21)
    orc = oracle_for(tables)
    oit, opk, ofe, cfgs = oracle_scores(orc, batch, tables)
    it, pk, fe, er, tl, ml = c_oracle_scores(tables, batch, lists=True)
    assert (er == 0).all()
    assert np.array_equal(it, oit) and np.array_equal(pk, opk) and np.array_equal(fe, ofe)
    for p, c in enumerate(cfgs):
        assert list(tl[p, :c.num_stages]) == c.time_list and list(ml[p, :c.num_stages]) == c.memory_list
    # strict comparison and another limit
    lim = float(np.median(opk))
    _, _, fe2, _ = c_oracle_scores(tables, batch, strict=True, memory_limit=lim)
    assert np.array_equal(fe2, (opk < lim).astype(np.uint8))
    # several threads give the same answers
    it4, pk4, fe4, _ = c_oracle_scores(tables, batch, threads=4, memory_limit=w.memory_limit)
    assert np.array_equal(it4, oit) and np.array_equal(pk4, opk) and np.array_equal(fe4, ofe)


def test_c_oracle_flags_what_the_reference_raises():
    w = synth.WORKLOADS["gpt3_13b"]
    tables = synth.make_tables(w)
    batch = synth.make_plans(w, tables, n_plans=64, seed_offset=2)
    orc = oracle_for(tables)
    hdr = batch.hdr.copy()
    hdr[:, 0] = (hdr[:, 0] & 0xff) | (0 << 8)            # micro-batch 1 everywhere: micro_bs // dp leaves the grid
    bad = PlanBatch(batch.codes, hdr)
    _, _, fe, er = c_oracle_scores(tables, bad)
    raised = []
    for p in range(bad.n_plans):
        try:
            orc.score(oracle_config(bad, p, tables))
            raised.append(0)
        except KeyError:
            raised.append(1)
    assert list(er) == raised and sum(raised) > 10 and (fe[np.array(raised) == 1] == 0).all()


@pytest.mark.parametrize("case", CASES)
def test_c_oracle_reference_vectors(golden_dir, case):
    g, orc, full = load_case(golden_dir, case)
    co = COracle(orc, full, g["global_batch_size"])
    cfgs = [make_config(g, p, full) for p in g["plans"]]
    it, pk, fe, er, tl, ml = co.score_configs(cfgs, lists=True)
    assert (er == 0).all()
    for k, p in enumerate(g["plans"]):
        S = len(p["time_list"])
        assert list(tl[k, :S]) == p["time_list"] and list(ml[k, :S]) == p["memory_list"]
        assert it[k] == max(p["time_list"]) and pk[k] == max(p["memory_list"])
        assert fe[k] == (max(p["memory_list"]) <= g["memory_limit"])


from tests.test_oracle_golden import ALL_VARIANTS, load_variant


@pytest.mark.parametrize("name", ALL_VARIANTS)
def test_c_oracle_reference_vectors_non_default_switches(golden_dir, name):
    """The reference's own numbers under MIN / collective memory / no shared space / no reserved space
    (the switches that change scoring; flex_recompute and peak_mem_in_backward only steer check_recompute)."""
    g, orc, full = load_variant(golden_dir, name)
    co = COracle(orc, full, g["global_batch_size"])
    cfgs = [make_config(g, p, full) for p in g["plans"]]
    it, pk, fe, er, tl, ml = co.score_configs(cfgs, lists=True)
    assert (er == 0).all()
    for k, p in enumerate(g["plans"]):
        S = len(p["time_list"])
        assert list(tl[k, :S]) == p["time_list"] and list(ml[k, :S]) == p["memory_list"]
        assert it[k] == max(p["time_list"]) and pk[k] == max(p["memory_list"])
