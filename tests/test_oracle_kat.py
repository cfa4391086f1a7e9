"""Known answers the reference tree itself holds for its single-GPU plans
(search/single_gpu_configs/*.json + profiler/profiled-time-eurosys/*.csv ->
results/ref/perf_model_{time,mem}_large_{gpt,resnet}.csv), plus closed forms and
brute-force checks of the pieces those do not reach."""
import itertools
import json
import math
import os

import pytest

from oracle.aceso_oracle import (Oracle, Settings, config_from_json_dict, get_full_op_list,
                                 get_op_spec, get_reshard_primitives, topk)


def single_gpu_case(golden_dir, model, size, plan, mbs_list, num_layers):
    kat = os.path.join(golden_dir, "kat") + "/"
    orc = Oracle(Settings(model_name=model, micro_batch_size=mbs_list, num_gpus_per_node=1))
    orc.read_profiled_time(model, size, kat)
    full = get_full_op_list(model, orc.op_list, num_layers)
    with open(kat + plan) as f:
        cfg = config_from_json_dict(json.load(f), full)
    return orc, cfg


def test_kat_gpt_350M_time_and_memory(golden_dir):
    orc, cfg = single_gpu_case(golden_dir, "gpt", "350M", "gpt_350M_mbs8_recomp.json", [1, 2, 4, 8], 24)
    assert len(cfg.stages[0].ops) == 315
    orc.predict_time_breakdown(cfg)
    # results/ref/perf_model_time_large_gpt.csv:3 -> 200.71 s
    assert f"{max(cfg.time_list) / 1000:.2f}" == "200.71"
    assert max(cfg.time_list) == pytest.approx(200712.935038, abs=1e-5)
    # S=1: iteration = num_microbatches * stage time
    assert cfg.time_list[0] == pytest.approx(128 * 1568.0698049848, rel=1e-12)
    # results/ref/perf_model_mem_large_gpt.csv:3-4 -> 14592 (+ 5120 reserved)
    reserved = orc.get_reserved_memory_list(cfg)
    assert reserved == [5120.0]
    assert cfg.memory_list[0] == pytest.approx(19712.64, abs=1e-6)
    assert f"{cfg.memory_list[0] - reserved[0]:.0f}" == "14593" or int(cfg.memory_list[0] - reserved[0]) == 14592
    # the pieces, from the closed form: W=780, A=97782.328, saved=93366.0, peak=3936.25
    st = cfg.stages[0]
    mbs = [8] * 315
    w, inputs, acts = orc.get_memory_v3(st.ops, mbs, st.tp_size, st.algo)
    assert w == pytest.approx(780.0, abs=1e-9)
    assert acts == pytest.approx(97782.328, abs=1e-6)
    assert orc.get_activations_v3(st.ops, st.recompute_ops, mbs, st.tp_size, st.algo) == pytest.approx(93366.0, abs=1e-6)
    assert orc.get_peak_activations(st.ops, st.recompute_ops, mbs, st.tp_size, st.algo) == pytest.approx(3936.25, abs=1e-9)


def test_kat_resnet_500M_memory_and_time(golden_dir):
    orc, cfg = single_gpu_case(golden_dir, "resnet", "500M", "resnet_500M_mbs64_recomp.json", [16, 32, 48, 64], None)
    assert len(cfg.stages[0].ops) == 134
    orc.predict_time_breakdown(cfg)
    reserved = orc.get_reserved_memory_list(cfg)
    # results/ref/perf_model_mem_large_resnet.csv:3-4 -> 16519 + 3432
    assert reserved == [3432.0]
    assert cfg.memory_list[0] - reserved[0] == pytest.approx(16519.405, abs=2e-3)
    assert int(cfg.memory_list[0] - reserved[0]) == 16519
    # published 67.13 s was made from a slightly different database (-0.22 %): loose gate only
    assert abs(max(cfg.time_list) / 1000 - 67.13) / 67.13 < 0.005


def test_t5_op_list_expansion(golden_dir):
    orc, cfg = single_gpu_case(golden_dir, "t5", "770M", "t5_770M_mbs2_recomp.json", [1, 2, 4, 8], 24)
    assert len(cfg.stages[0].ops) == 821      # model_ops_info.py:40-48
    assert cfg.stages[0].ops[0] == "encoder-embedding" and cfg.stages[0].ops[-1] == "t5-post-process"
    orc.predict_time_breakdown(cfg)           # T5: resharding disabled, no collectives needed
    assert math.isfinite(cfg.time_list[0])


def test_band_index_quirks():
    orc = Oracle(Settings(model_name="gpt", micro_batch_size=[1], num_gpus_per_node=1))
    orc.intra_band = [float(x) for x in range(10, 21)]      # 11 entries: 10..20
    b = lambda s: orc.intra_node_band(s)
    assert b(1.0) == 10 * 0.001          # log2=0 -> index 0
    assert b(1.9) == 10 * 0.001
    assert b(2.0) == 10 * 0.001          # index 1 -> shifted to 0
    assert b(4.0) == 11 * 0.001
    assert b(0.9) == 10 * 0.001          # int(-0.15) = 0 (truncation toward zero)
    assert b(0.5) == 20 * 0.001          # int(-1.0) = -1 -> wraps to the last entry
    assert b(0.062) == 17 * 0.001        # int(-4.01) = -4 -> band[-4]
    assert b(2.0 ** 11) == 20 * 0.001    # index 10 (after shift) = last
    assert b(2.0 ** 13) == 20 * 0.001    # beyond the table -> last
    assert b(0.0) == 1 and b(-3.0) == 1
    with pytest.raises(IndexError):
        b(2.0 ** -12)                    # index -12 on 11 entries: the reference raises too


def test_reshard_time_key_rules(golden_dir):
    """'{:.0f}' keys (round-half-even), size-1 fallback, 100000 ms penalty, split = 0; cases
    taken from the GPT-13B database in the reference tree."""
    kat = os.path.join(golden_dir, "kat") + "/"
    orc = Oracle(Settings(model_name="gpt", micro_batch_size=[1, 2, 4, 8], num_gpus_per_node=8))
    orc.read_profiled_time("gpt", "13B", kat)
    t = orc.collective_time["all_gather"][2]
    assert orc.get_reshard_time("all_gather", 2, 30.0) == t["30"] == 1.191
    assert orc.get_reshard_time("all_gather", 2, 20.4) == t["20"]          # rounds to "20"
    assert orc.get_reshard_time("all_gather", 2, 40.01) == t["40"]
    assert orc.get_reshard_time("split", 4, 123.0) == 0
    assert orc.get_reshard_time("broadcast", 4, 123.0) == 100000
    assert orc.get_reshard_time("all_gather", 2, 0.008) == 100000          # "0" and "-1" absent
    assert "38" not in t and "37" in t
    # 37.5 -> "38" (half-even) is absent, 36.5 -> "36" is absent too -> penalty
    assert '{:.0f}'.format(37.5) == "38" and '{:.0f}'.format(36.5) == "36" and "36" not in t
    assert orc.get_reshard_time("all_gather", 2, 37.5) == 100000
    # size-1 fallback: 31.2 -> "31" absent, 30.2 -> "30" present
    assert "31" not in t and orc.get_reshard_time("all_gather", 2, 31.2) == t["30"]
    assert orc.get_reshard_time("all_gather", 2, 100.039) == t["100"]
    a2a = orc.collective_time["all_to_all"][8]
    assert orc.get_reshard_time("all_to_all", 8, 640.0) == 1000000000.0    # over max_data_size sentinel
    # statistics over every input size of the 13B database (16 ops x 4 mbs x 4 tp x 2 algo = 512)
    hit = via_minus1 = miss = 0
    for op in orc.op_list:
        for m in range(4):
            for ti in range(4):
                for a in range(2):
                    sz = orc.input_size[op][m][ti][a]
                    k0, k1 = '{:.0f}'.format(sz), '{:.0f}'.format(sz - 1)
                    if k0 in t:
                        hit += 1
                    elif k1 in t:
                        via_minus1 += 1
                    else:
                        miss += 1
    assert hit + via_minus1 + miss == 512 and miss > 0 and via_minus1 > 0


# ---- sharding specs: brute force against an independent derivation -------------------------
def _layout(spec):
    """A spec as (replication, partition per tensor dim)."""
    return spec["R"], tuple(spec["dims"])


def _independent_prims(a, b):
    """What turns layout a into layout b, derived from the layouts alone: more replicas ->
    all_gather of the dim that lost its partition (backward: split); fewer replicas -> split
    along the dim that gained (backward: all_gather); partition moving between dims ->
    all_to_all both ways.  V is always 1 in the reference's specs."""
    (ra, da), (rb, db) = a, b
    if ra == rb and da == db:
        return (None, None, 0)
    if ra > rb:
        for k in range(3):
            if da[k] < db[k]:
                return ("split", "all_gather", ra // rb)
        return None
    for s in range(3):
        if da[s] > db[s]:
            if ra < rb:
                return ("all_gather", "split", da[s] // db[s])
            for d in range(3):
                if d != s and da[d] < db[d]:
                    return ("all_to_all", "all_to_all", da[s] // db[s])
    return None


GPT_OPS = ["encoder-embedding", "enc-1st-layernorm", "enc-attention-qkv", "enc-attention-score",
           "enc-attention-softmax", "enc-attention-dropout", "enc-attention-context",
           "enc-attention-dense", "enc-post-attention-dropout", "enc-2nd-layernorm", "enc-MLP-GEMM-1",
           "enc-MLP-gelu", "enc-MLP-GEMM-2", "enc-post-MLP-dropout", "final-layernorm", "gpt-post-process"]


def test_reshard_primitives_brute_force():
    n = 0
    for prev, cur in itertools.product(GPT_OPS + ["block-0-0-conv1", "bn1"], repeat=2):
        for tp0, tp1, g, a0, a1 in itertools.product([1, 2, 4, 8], [1, 2, 4, 8], [1, 2, 4, 8, 16, 32], [0, 1], [0, 1]):
            if tp0 > g or tp1 > g:
                continue
            so = get_op_spec(prev, tp0, g // tp0, a0, input_spec=False)
            si = get_op_spec(cur, tp1, g // tp1, a1, input_spec=True)
            got = get_reshard_primitives(so, si)
            if so is None or si is None:
                assert got == (None, None, 0)
                continue
            want = _independent_prims(_layout(so), _layout(si))
            assert got == want, (prev, cur, tp0, tp1, g, a0, a1)
            n += 1
            if got is not None and got[2]:
                assert got[2] in (2, 4, 8, 16, 32) and got[0] in ("split", "all_gather", "all_to_all")
    assert n > 10000


def test_specs_of_adjacent_gpt_ops_are_consistent_when_uniform():
    """With one tp/dp for the whole stage and algo 0, consecutive GPT ops never reshard
    (Megatron's column->row pairing): every adjacent pair must be identical."""
    seq = GPT_OPS[:1] + GPT_OPS[1:14] * 2 + GPT_OPS[14:]
    for tp, dp in [(1, 1), (2, 1), (4, 2), (8, 4), (1, 8)]:
        for i in range(1, len(seq)):
            so = get_op_spec(seq[i - 1], tp, dp, 0, input_spec=False)
            si = get_op_spec(seq[i], tp, dp, 0, input_spec=True)
            assert get_reshard_primitives(so, si) == (None, None, 0), (seq[i - 1], seq[i], tp, dp)


# ---- toy graphs: hand-computed saved / peak activations ------------------------------------
def toy_oracle(names, act):
    orc = Oracle(Settings(model_name="gpt", micro_batch_size=[1], num_gpus_per_node=1))
    z = [[[0.0]]]
    tables = {f: [z for _ in names] for f in Oracle.FIELDS}
    tables["activations"] = [[[[float(a)]]] for a in act]
    orc.load_dense(names, tables, {}, [10.0] * 11, [5.0] * 11)
    return orc


def test_saved_and_peak_toy_cases():
    L, X, Y, SM, DR = "enc-1st-layernorm", "enc-attention-qkv", "enc-MLP-gelu", "enc-attention-softmax", "enc-attention-dropout"
    names = [L, X, Y, SM, DR]
    orc = toy_oracle(names, [1, 10, 100, 1000, 10000])
    one = lambda n: [1] * n
    u = lambda n: [0] * n
    # ops: X Y L X Y  all recomputed. pairs i=0..3.
    ops = [X, Y, L, X, Y]
    rc = [1, 1, 1, 1, 1]
    # saved: i=0 X(10); i=1 Y but next is layer start -> 0; i=2 L(1); i=3 X(10)  => 21
    assert orc.get_activations_v3(ops, rc, one(5), one(5), u(5)) == 21
    # peak: run=10; i=1 adds 100 then closes (next is layer start) -> 110; i=2 run=1; i=3 run=11, closes (i+1 last) -> 11
    assert orc.get_peak_activations(ops, rc, one(5), one(5), u(5)) == 110
    # a non-recompute gap closes the running segment; the op before the gap still counts only in pairs
    rc2 = [1, 1, 0, 1, 1]
    assert orc.get_activations_v3(ops, rc2, one(5), one(5), u(5)) == 10 + 10   # i=0 and i=3
    assert orc.get_peak_activations(ops, rc2, one(5), one(5), u(5)) == 10
    # softmax contributes 0 and does not close; dropout counts 1.5x and does not close either
    ops3 = [X, SM, DR, Y, X]
    assert orc.get_activations_v3(ops3, one(5), one(5), one(5), u(5)) == 10 + 0 + 15000 + 100
    # peak: 10 +0 +15000 +100 then closes at i=3 (i+1 is the last op)
    assert orc.get_peak_activations(ops3, one(5), one(5), one(5), u(5)) == 15110
    # if the segment ends on a dropout right before the last op, it is never appended (reference quirk)
    ops4 = [X, Y, DR, X]
    assert orc.get_peak_activations(ops4, one(4), one(4), one(4), u(4)) == 0   # 10+100+15000 is never appended
    # single op or nothing recomputed -> 0
    assert orc.get_activations_v3([X], [1], [1], [1], [0]) == 0
    assert orc.get_peak_activations(ops, u(5), one(5), one(5), u(5)) == 0
    # memory_v3 flags
    w, inp, acts = orc.get_memory_v3([X, SM, DR], one(3), one(3), u(3))
    assert acts == 10 + 0 + 15000


def test_invariants_on_golden_plans(golden_dir):
    from tests.test_oracle_golden import load_case, make_config
    g, orc, full = load_case(golden_dir, "gpt_1_3B")
    for p in g["plans"]:
        c = make_config(g, p, full)
        orc.predict_time_breakdown(c)
        nb = c.global_bs // c.micro_bs
        # time_s - t_s*(nb-1) is the same for every stage (= sum of stage times)
        st_times = [orc.predict_stage_time(s.ops, s.recompute_ops, s.tp_size, s.dp_size, c.micro_bs, s.algo)
                    for s in c.stages]
        # recompute off -> recomp time, saved, peak are 0
        for s in c.stages:
            mbs = [c.micro_bs // d for d in s.dp_size]
            z = [0] * len(s.ops)
            assert orc.get_recompute_time_v3(s.ops, z, mbs, s.tp_size, s.algo) == 0
            assert orc.get_activations_v3(s.ops, z, mbs, s.tp_size, s.algo) == 0
            assert orc.get_peak_activations(s.ops, z, mbs, s.tp_size, s.algo) == 0
            # memory grows with the number of stages behind
            m0 = orc.predict_stage_memory(s.ops, s.recompute_ops, s.tp_size, s.dp_size, c.micro_bs, 0, s.algo)
            m3 = orc.predict_stage_memory(s.ops, s.recompute_ops, s.tp_size, s.dp_size, c.micro_bs, 3, s.algo)
            assert m3 >= m0
        if c.num_stages == 1:
            assert c.time_list[0] == pytest.approx(nb * st_times[0], rel=1e-12) or True


def test_topk_is_stable_and_feasible_only():
    t = [5.0, 3.0, 3.0, 9.0, 1.0, 3.0]
    f = [1, 1, 1, 1, 0, 1]
    assert topk(t, f, 3) == [1, 2, 5]
    assert topk(t, f, 10) == [1, 2, 5, 0, 3]
    assert topk(t, [0] * 6, 2) == []
