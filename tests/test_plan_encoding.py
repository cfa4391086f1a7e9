"""Host-side plan plumbing: object form <-> array form, JSON form, legality, error behaviour."""
import json
import os

import numpy as np
import pytest

from superscaler_amd import synth
from superscaler_amd.plan import (PlanBatch, check_legality, config_from_json, config_to_json_dict,
                                  cross_node_bits, validate_batch)


@pytest.fixture(scope="module")
def small():
    w = synth.WORKLOADS["gpt3_1_3b"]
    tables = synth.make_tables(w)
    return w, tables, synth.make_plans(w, tables, n_plans=64)


def test_roundtrip_object_and_array_form(small):
    w, tables, batch = small
    assert validate_batch(batch, tables) is None
    cfgs = [batch.to_config(p, tables) for p in range(batch.n_plans)]
    again = PlanBatch.from_configs(cfgs, tables)
    assert np.array_equal(again.codes, batch.codes) and np.array_equal(again.hdr, batch.hdr)
    c = cfgs[3]
    assert sum(len(s.ops) for s in c.stages) == tables.graph.num_ops
    assert all(t * d == s.num_gpus for s in c.stages for t, d in zip(s.tp_size, s.dp_size))
    assert [s.num_stages_behind for s in c.stages] == list(range(c.num_stages - 1, -1, -1))
    assert sum(s.num_gpus for s in c.stages) == w.num_gpus


def test_device_layout_is_plan_minor(small):
    w, tables, batch = small
    dev = batch.device_codes_host()
    P, N = batch.codes.shape
    assert dev.shape == ((N + 15) // 16, P, 16)
    assert dev[2, 5, 7] == batch.codes[5, 2 * 16 + 7]
    assert (dev[-1, :, N % 16:] == 0).all()


def test_cross_node_bits_follow_the_reference_rule():
    # aceso_cost_model.py:572-574 with 4 GPUs per node and stages of 2, 2, 4 devices
    bits = cross_node_bits([2, 2, 4], 4)
    assert bits & 0xffff == 0b100                    # only stage 2 starts on a node boundary (> 0)
    assert bits >> 16 == 0b110                       # stages 1 and 2 end on one
    assert cross_node_bits([1], 1) >> 16 == 1


def test_encoder_errors(small):
    w, tables, batch = small
    c = batch.to_config(0, tables)
    c.micro_bs = 3
    with pytest.raises(KeyError):                    # aceso_cost_model.py:25
        PlanBatch.from_configs([c], tables)
    c = batch.to_config(0, tables)
    c.stages[0].tp_size[0] *= 2                      # tp*dp no longer constant inside the stage
    with pytest.raises(ValueError):
        PlanBatch.from_configs([c], tables)
    c = batch.to_config(0, tables)
    c.stages[-1].ops.pop()
    with pytest.raises(ValueError):
        PlanBatch.from_configs([c], tables)
    bad = PlanBatch(batch.codes.copy(), batch.hdr.copy())
    bad.codes[0, 0] &= 0xEF
    assert "op 0" in validate_batch(bad, tables) or "stage-start" in validate_batch(bad, tables)


def test_json_form_and_legality(golden_dir, small):
    w, tables, batch = small
    c = batch.to_config(1, tables)
    d = config_to_json_dict(c, "gpt", "1_3B")
    assert d["num_stages"] == c.num_stages and d["hidden_size"] == 2048 and d["num_layers"] == 24
    c2 = config_from_json(json.loads(json.dumps(d)), tables.graph.ops)
    assert [s.tp_size for s in c2.stages] == [s.tp_size for s in c.stages]
    assert [s.recompute_ops for s in c2.stages] == [s.recompute_ops for s in c.stages]
    # the reference's own single-GPU plan file parses and writes back identically where fields overlap
    with open(os.path.join(golden_dir, "kat", "gpt_350M_mbs8_recomp.json")) as f:
        ref = json.load(f)
    from superscaler_amd.opgraph import GPT_TYPES, OpGraph
    g = OpGraph.build("gpt", GPT_TYPES, 24)
    cfg = config_from_json(ref, g.ops)
    out = config_to_json_dict(cfg, "gpt", "350M")
    assert out == ref
    assert check_legality(cfg, 1, 1, 1)
    assert check_legality(c, w.num_gpus, w.gpus_per_node, 1) == all(s.num_gpus in (1, 2, 4, 8) for s in c.stages)
    assert not check_legality(c, w.num_gpus + 1, w.gpus_per_node, 1)


def test_small_call_packing_is_the_kernel_layout():
    """evaluator.pack_small_inputs (one pinned buffer for codes, headers and ranges of a small host call) against
    the plan-minor layout built the plain way, with the last 16-op group full, partly filled and the only one."""
    import numpy as np
    from superscaler_amd.evaluator import pack_small_inputs
    from superscaler_amd.plan import PlanBatch
    from tests.helpers import kernel_layout
    rng = np.random.default_rng(5)
    for P, N in ((1, 523), (7, 16), (33, 134), (5, 9), (64, 1251), (3, 32)):
        codes = rng.integers(0, 32, size=(P, N), dtype=np.uint8)
        hdr = rng.integers(0, 2 ** 32, size=(P, 4), dtype=np.uint64).astype(np.uint32)
        ranges = rng.integers(0, N, size=(P, 2), dtype=np.uint64).astype(np.uint32)
        G = (N + 15) // 16
        for rg in (None, ranges):
            buf = np.full(G * P * 16 + P * 16 + P * 8 + 64, 0xAB, dtype=np.uint8)
            n = pack_small_inputs(buf, PlanBatch(codes, hdr), rg)
            assert n == G * P * 16 + P * 16 + (P * 8 if rg is not None else 0)
            assert np.array_equal(buf[:G * P * 16].reshape(G, P, 16), kernel_layout(codes))
            assert np.array_equal(buf[G * P * 16:G * P * 16 + P * 16].view(np.uint32).reshape(P, 4), hdr)
            if rg is not None:
                assert np.array_equal(buf[G * P * 16 + P * 16:n].view(np.uint32).reshape(P, 2), rg)
            assert (buf[n:] == 0xAB).all()
