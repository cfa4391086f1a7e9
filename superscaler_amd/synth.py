"""Seeded synthetic workloads: op graphs, profile databases and plan batches shaped like the
benchmark configurations (GPT-3 1.3B / T5 770M / Wide-ResNet 1B / GPT-3 13B / GPT-3 175B).

Databases follow the reference's table semantics (search/aceso_cost_model.py:27-183): eight
fields indexed [op type][micro-batch][tp][algo], times in microseconds, sizes in MB,
collective times in ms keyed by the size string, p2p bandwidth per power-of-two size bucket.
Plans follow what the reference's search produces (search/aceso_utils.py:96-115, :760-774):
pipeline stages are contiguous op ranges, a stage owns a power-of-two number of devices, each
op has its own tp (dp = stage devices / tp), partition algorithm and recompute bit, and the
micro-batch size is such that micro_bs // dp is a profiled size for every op.

Everything is drawn from numpy's PCG64 with a fixed seed, so CPU and GPU boxes see the same
bytes.
"""
import math
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import numpy as np

from . import opgraph as og
from .plan import PlanBatch
from .profile_db import CostModelSettings, ProfileDB
from .tables import CompiledTables, compile_tables

# saturating bandwidth curves, GB/s per size bucket 1 MB .. 1 GB (11 buckets, the shape of the
# reference's p2p_intra_node.csv / p2p_inter_node.csv)
INTRA_BAND = [round(43.0 * (1 - math.exp(-(k + 1.6) / 2.4)), 2) for k in range(11)]
INTER_BAND = [round(5.5 * (1 - math.exp(-(k + 3.0) / 2.2)), 2) for k in range(11)]


@dataclass
class Workload:
    name: str
    model_name: str
    num_layers: Optional[int]
    hidden: int
    seq: int
    dec_seq: int
    mbs_list: List[int]
    num_gpus: int
    gpus_per_node: int
    global_batch: int
    memory_limit: float
    pp_choices: List[int]
    n_plans: int
    recompute_p: float
    conv: bool = False
    resnet_blocks: Tuple[int, ...] = (3, 4, 6, 3)
    seed: int = 0xACE50


WORKLOADS: Dict[str, Workload] = {
    # GPT-3 1.3B: 24 layers x 13 ops + 3 = 315 ops, D = 4
    "gpt3_1_3b": Workload("gpt3_1_3b", "gpt", 24, 2048, 2048, 0, [1, 2, 4, 8, 16], 4, 4, 512, 28000.0,
                          [1, 2, 4], 4096, 0.3, seed=0xACE51),
    # T5 770M: 24 + 24 layers, 821 ops, D = 8
    "t5_770m": Workload("t5_770m", "t5", 24, 1024, 512, 128, [1, 2, 4, 8, 16], 8, 8, 512, 28000.0,
                        [1, 2, 4, 8], 65536, 0.3, seed=0xACE52),
    # Wide-ResNet 1B: 134 ops, one table row per op, D = 16
    "wresnet_1b": Workload("wresnet_1b", "resnet", None, 320, 224, 0, [1, 2, 4, 8, 16], 16, 8, 768, 28000.0,
                           [1, 2, 4, 8], 262144, 0.3, conv=True, seed=0xACE53),
    # GPT-3 13B: 40 layers -> 523 ops, D = 32, 80 GB devices
    "gpt3_13b": Workload("gpt3_13b", "gpt", 40, 5120, 2048, 0, [1, 2, 4, 8], 32, 8, 1024, 81920.0,
                         [1, 2, 4, 8, 16], 1048576, 0.5, seed=0xACE54),
    # GPT-3 175B-shaped: 96 layers -> 1251 ops, D = 1024 (a cost-model input only)
    "gpt3_175b": Workload("gpt3_175b", "gpt", 96, 12288, 2048, 0, [1, 2, 4, 8], 1024, 8, 1024, 81920.0,
                          [16], 4194304, 0.5, seed=0xACE55),
}


def _type_names(w: Workload) -> List[str]:
    if w.model_name == "gpt":
        return list(og.GPT_TYPES)
    if w.model_name == "t5":
        return list(og.T5_TYPES)
    return og.resnet_types(w.resnet_blocks)


def make_graph(w: Workload) -> og.OpGraph:
    return og.OpGraph.build(w.model_name, _type_names(w), w.num_layers)


def _shape_mb(w: Workload, name: str, b: int, tp: int) -> Tuple[float, float, float, float]:
    """(input, output, weights, activations) MB of one op in fp16 for micro-batch b at tp."""
    mb = 1.0 / (1 << 20)
    if w.model_name in ("gpt", "t5"):
        h = w.hidden
        s = w.dec_seq if name.startswith("dec") or name.startswith("t5-post") else w.seq
        u = b * s * h * 2 * mb                       # one [b, s, h] fp16 tensor
        heads = max(h // 128, 1)
        sc = b * heads * s * s * 2 * mb / tp         # attention scores
        if "embedding" in name:
            return b * s * 4 * mb, u, 51200 * h * 2 * mb / tp, 1.5 * u
        if "layernorm" in name:
            return u, 2 * u, 0.0, u + 0.016
        if "qkv" in name:
            return 2 * u, 4 * u / tp + u, 3 * h * h * 2 * mb / tp, 3 * u / tp
        if "score" in name:
            return 4 * u / tp + u, sc + 2 * u / tp + u, 0.0, sc
        if "softmax" in name:
            return sc + 2 * u / tp + u, sc + 2 * u / tp + u, 0.0, sc
        if "attention-dropout" in name:
            return sc + 2 * u / tp + u, sc + 2 * u / tp + u, 0.0, 1.5 * sc
        if "context" in name:
            return sc + 2 * u / tp + u, u / tp + u, 0.0, u / tp
        if "dense" in name:
            return u / tp + u, 2 * u + 0.01, h * h * 2 * mb / tp, u
        if "post-attention-dropout" in name or "post-MLP-dropout" in name:
            return 2 * u + 0.01, u, 0.0, 1.5 * u
        if "GEMM-1" in name:
            return 2 * u, 4 * u / tp + u + 0.039, 4 * h * h * 2 * mb / tp, 4 * u / tp
        if "gelu" in name:
            return 4 * u / tp + u + 0.039, 4 * u / tp + u, 0.0, 4 * u / tp
        if "GEMM-2" in name:
            return 4 * u / tp + u, 2 * u + 0.01, 4 * h * h * 2 * mb / tp, u
        if "post-process" in name:
            return u, 0.0, 51200 * h * 2 * mb / tp, b * s * 51200 * 2 * mb / tp + 0.025
        return u, u, 0.0, u
    # resnet: bottleneck blocks, channels 64..2048 x width factor 2, image 224
    stage = 0
    res = 56
    ch = w.hidden
    if name.startswith("block-"):
        stage = int(name.split("-")[1])
        res = 56 >> stage
        ch = w.hidden * (1 << stage)
    elif name in ("conv1", "bn1", "relu1"):
        res, ch = 112, 64
    elif name == "maxpool":
        res, ch = 56, 64
    elif name in ("avgpool", "fc"):
        res, ch = 1, w.hidden * 8 * 4
    t = b * ch * res * res * 2 * mb
    if "conv" in name or "downsample" in name:
        wgt = ch * ch * 9 * 2 * mb / tp
        return t, t / tp if tp > 1 else t, wgt, t / tp if tp > 1 else t
    if name == "fc":
        return t, b * 1000 * 2 * mb, ch * 1000 * 2 * mb / tp, b * 1000 * 2 * mb
    return t, t, 0.002 if "bn" in name else 0.0, t


def make_db(w: Workload, graph: og.OpGraph, drop_collective_keys: int = 3) -> ProfileDB:
    rng = np.random.Generator(np.random.PCG64(w.seed))
    names = graph.type_names
    tp_list = [t for t in (1, 2, 4, 8) if t <= min(w.gpus_per_node, 8)]
    n_algo = 1 if w.model_name == "t5" else 2
    db = ProfileDB.empty(w.model_name, names, w.mbs_list, tp_list, n_algo)
    M, T = len(w.mbs_list), len(tp_list)
    mu, sigma = (-1.5, 1.2) if w.conv else (-2.0, 1.0)
    base_ms = rng.lognormal(mu, sigma, size=len(names))
    for ty, name in enumerate(names):
        tunable = bool(graph.flags[ty] & og.F_TUNABLE)
        for mi, b in enumerate(w.mbs_list):
            for ti, tp in enumerate(tp_list):
                fwd_ms = base_ms[ty] * b / (tp ** 0.85 if tunable else 1.0) * rng.uniform(0.9, 1.1)
                bwd_ms = 2.0 * fwd_ms * rng.uniform(0.9, 1.1)
                insz, outsz, wgt, act = _shape_mb(w, name, b, tp)
                for a in range(n_algo):
                    f = rng.uniform(0.9, 1.1) if (a == 1 and tunable) else 1.0
                    db.tables["fwd"][ty, mi, ti, a] = round(fwd_ms * f * 1000.0, 3)
                    db.tables["bwd"][ty, mi, ti, a] = round(bwd_ms * f * 1000.0, 3)
                    db.tables["input_size"][ty, mi, ti, a] = round(insz, 3)
                    db.tables["output_size"][ty, mi, ti, a] = round(outsz, 3)
                    db.tables["weights"][ty, mi, ti, a] = round(wgt, 3)
                    db.tables["activations"][ty, mi, ti, a] = round(act, 3)
                    db.tables["reserved_fwd"][ty, mi, ti, a] = round(act, 3) if (ty % 3 == 0) else 0.0
                    db.tables["reserved_bwd"][ty, mi, ti, a] = round(2.0 * act, 3) if (ty % 4 != 1) else 0.0
    # collectives: one entry per rounded input size that occurs, minus a few to keep the
    # "unprofiled size" paths (size-1 key, 100000 ms penalty) alive
    if w.model_name != "t5":
        prims = ["all_gather", "all_reduce", "reduce_scatter", "all_to_all"] if w.model_name == "gpt" \
            else ["all_gather", "all_to_all"]
        keys = sorted({"{:.0f}".format(float(x)) for x in db.tables["input_size"].ravel()}, key=float)
        dropped = set(keys[5::max(len(keys) // max(drop_collective_keys, 1), 1)][:drop_collective_keys])
        for prim in prims:
            db.collectives[prim] = {}
            for n in tp_list[1:]:
                scale = {"all_gather": 1.0, "all_reduce": 2.0, "reduce_scatter": 1.0, "all_to_all": 0.7}[prim]
                db.collectives[prim][n] = {k: round(0.05 + scale * float(k) * (n - 1) / n / 100.0, 3)
                                           for k in keys if k not in dropped}
    db.intra_band = list(INTRA_BAND)
    db.inter_band = list(INTER_BAND)
    return db


def make_settings(w: Workload) -> CostModelSettings:
    return CostModelSettings(model_name=w.model_name, micro_batch_size=list(w.mbs_list),
                             num_gpus_per_node=w.gpus_per_node, global_batch_size=w.global_batch,
                             memory_limit=w.memory_limit, max_tp=min(w.gpus_per_node, 8))


def make_tables(w: Workload) -> CompiledTables:
    graph = make_graph(w)
    return compile_tables(graph, make_db(w, graph), make_settings(w))


# ------------------------------------------------------------------------------------------
# plans
# ------------------------------------------------------------------------------------------
def _random_compositions(rng, n: int, S: int, total: int, cap_log: int) -> np.ndarray:
    """n random ways to write `total` (a power of two) as S powers of two, each <= 2**cap_log, as
    log2 values [n, S]: start from all ones and keep doubling a random stage that still fits."""
    g = np.ones((n, S), dtype=np.int64)
    while True:
        left = total - g.sum(axis=1)
        todo = left > 0
        if not todo.any():
            return np.log2(g).astype(np.int64)
        ok = (g <= left[:, None]) & (g < (1 << cap_log)) & todo[:, None]
        if not ok.any(axis=1)[todo].all():
            raise ValueError("device count cannot be split into the requested number of stages")
        pick = np.argmax(rng.random((n, S)) * ok, axis=1)
        rows = np.flatnonzero(todo)
        g[rows, pick[rows]] *= 2


def make_plans(w: Workload, tables: CompiledTables, n_plans: Optional[int] = None, seed_offset: int = 0,
               run_p: float = 0.04, algo_p: float = 0.1, chunk: int = 16384, workers: int = 8) -> PlanBatch:
    """Seeded random plans in array form.  Per plan: PP from w.pp_choices; distinct sorted random
    stage cuts; micro-batch from the profiled set; stage device counts = a random composition of
    w.num_gpus into powers of two such that every stage still has a tp for which micro_bs // dp is
    profiled; per-op tp in contiguous runs (a new run starts with probability run_p), drawn from
    the tps the stage allows; recompute ~ Bernoulli(w.recompute_p); algo ~ Bernoulli(algo_p) on
    tunable ops."""
    P = int(n_plans if n_plans is not None else w.n_plans)
    graph, db = tables.graph, tables.db
    N, A, T, M = graph.num_ops, db.n_algo, len(db.tp_list), len(db.mbs_list)
    tunable = (graph.flags[graph.type_of_pos] & og.F_TUNABLE) != 0
    # allowed tp logs per (micro-batch index, glog)
    allowed = [[tables.allowed_tp_logs(b, gl) for gl in range(16)] for b in range(M)]
    # per micro-batch index: the largest stage that still has a scorable tp (all smaller ones do too)
    cap_log = [max([gl for gl in range(16) if allowed[b][gl]] or [-1]) for b in range(M)]
    full_log = w.num_gpus.bit_length() - 1
    valid_by_S: Dict[int, List[int]] = {}
    for S in w.pp_choices:
        for b in range(M):
            if S <= N and S <= w.num_gpus and cap_log[b] >= 0 and (S << min(cap_log[b], full_log)) >= w.num_gpus:
                valid_by_S.setdefault(S, []).append(b)
    if not valid_by_S:
        raise ValueError("no (pipeline depth, micro-batch) combination is scorable for this workload")
    S_choices = sorted(valid_by_S)

    # allowed tp logs as flat tables indexed by (micro-batch index * 16 + glog)
    cnt = np.zeros(M * 16, dtype=np.float32)
    tab = np.zeros((M * 16, T), dtype=np.uint8)
    for b in range(M):
        for gl in range(16):
            al = allowed[b][gl]
            cnt[b * 16 + gl] = len(al)
            tab[b * 16 + gl, :len(al)] = al
    tab_flat = tab.ravel()
    pos16 = np.arange(N, dtype=np.int16)[None, :]

    def one_chunk(ci: int) -> Tuple[np.ndarray, np.ndarray]:
        lo = ci * chunk
        n = min(chunk, P - lo)
        rng = np.random.Generator(np.random.PCG64([w.seed, 0x9E3779B9, seed_offset, ci]))
        S_arr = rng.choice(S_choices, size=n)
        b_arr = np.zeros(n, dtype=np.int64)
        glog = np.zeros((n, 16), dtype=np.uint8)
        for S in S_choices:
            sel = np.flatnonzero(S_arr == S)
            if not len(sel):
                continue
            bs = rng.choice(valid_by_S[S], size=len(sel))
            b_arr[sel] = bs
            for b in valid_by_S[S]:
                sub = sel[bs == b]
                if len(sub):
                    glog[sub[:, None], np.arange(S)[None, :]] = _random_compositions(
                        rng, len(sub), S, w.num_gpus, min(cap_log[b], full_log))
        # cuts: S-1 distinct sorted positions in 1..N-1 (sorted draws from N-1-(S-1)+1 values, plus rank)
        ns = np.zeros((n, N), dtype=np.uint8)
        ns[:, 0] = 1
        for r_S in np.unique(S_arr):
            if r_S <= 1:
                continue
            sel = np.flatnonzero(S_arr == r_S)
            k = int(r_S) - 1
            uu = np.sort(rng.random((len(sel), k)), axis=1)
            cuts = 1 + np.floor(uu * ((N - 1) - k + 1)).astype(np.int64) + np.arange(k)[None, :]
            ns[sel[:, None], cuts] = 1
        stage_id = np.cumsum(ns, axis=1, dtype=np.uint8) - np.uint8(1)               # [n, N]
        # per-op tp: contiguous runs, drawn from what the op's stage allows
        run_start = (rng.random((n, N), dtype=np.float32) < np.float32(run_p)) | (ns == 1)
        last_start = np.maximum.accumulate(np.where(run_start, pos16, np.int16(0)), axis=1)
        key = np.take_along_axis(glog, stage_id, axis=1) + (b_arr * 16).astype(np.uint8)[:, None]
        pick = (rng.random((n, N), dtype=np.float32) * cnt[key]).astype(np.uint8)
        t_draw = tab_flat[key.astype(np.int32) * T + pick]
        t_op = np.take_along_axis(t_draw, last_start.astype(np.int64), axis=1)
        rc = (rng.random((n, N), dtype=np.float32) < np.float32(w.recompute_p)).astype(np.uint8)
        codes = (t_op * np.uint8(A)) | (rc << 3) | (ns << 4)
        if A == 2:
            codes |= ((rng.random((n, N), dtype=np.float32) < np.float32(algo_p)) & tunable[None, :]).astype(np.uint8)
        hdr = np.zeros((n, 4), dtype=np.uint32)
        hdr[:, 0] = S_arr | (b_arr << 8)
        gword = np.zeros(n, dtype=np.uint64)
        cross = np.zeros(n, dtype=np.uint32)
        till = np.zeros(n, dtype=np.int64)
        for s in range(int(S_arr.max())):
            live = S_arr > s
            gs = glog[:, s].astype(np.int64)
            gword |= np.where(live, gs, 0).astype(np.uint64) << np.uint64(4 * s)
            incross = live & (till % w.gpus_per_node == 0) & (till > 0)
            till = till + np.where(live, 1 << gs, 0)
            outcross = live & (till % w.gpus_per_node == 0)
            cross |= (incross.astype(np.uint32) << np.uint32(s)) | (outcross.astype(np.uint32) << np.uint32(16 + s))
        hdr[:, 1] = (gword & np.uint64(0xFFFFFFFF)).astype(np.uint32)
        hdr[:, 2] = (gword >> np.uint64(32)).astype(np.uint32)
        hdr[:, 3] = cross
        return codes, hdr

    n_chunks = (P + chunk - 1) // chunk
    if n_chunks > 1 and workers > 1:
        from concurrent.futures import ThreadPoolExecutor
        with ThreadPoolExecutor(max_workers=workers) as ex:
            parts = list(ex.map(one_chunk, range(n_chunks)))
    else:
        parts = [one_chunk(ci) for ci in range(n_chunks)]
    return PlanBatch(np.concatenate([c for c, _ in parts]), np.concatenate([h for _, h in parts]))
