"""Plans: the reference's object form and the structure-of-arrays form the GPU scores.

Object form mirrors search/aceso_utils.py:58-115 (AcesoStageInfo / AcesoConfig / get_config)
and its JSON layout (:137-242) so the reference's search code can hand its own objects in:
only attributes are read, any object with the same fields works.

Array form (`PlanBatch`): one byte per (plan, op) --
    bits 0-2  tp_log2 * n_algo + algo        bit 3  recompute        bit 4  first op of a stage
plus four 32-bit words per plan --
    [0] num_stages | micro-batch index << 8
    [1..2] log2(stage gpus), 4 bits per stage
    [3] in-cross-node bit per stage | out-cross-node bits << 16   (aceso_cost_model.py:572-574)
"""
import itertools
import json
from dataclasses import dataclass, field
from typing import List, Optional, Sequence

import numpy as np

from .tables import MAX_STAGES, CompiledTables


@dataclass
class AcesoStageInfo:
    index: int
    num_stages_behind: int
    num_gpus: int
    ops: List[str]
    recompute_ops: List[int]
    tp_size: List[int]
    dp_size: List[int]
    algo: List[int]


@dataclass
class AcesoConfig:
    global_bs: int
    micro_bs: int
    stages: List[AcesoStageInfo]
    num_stages: int
    history: str = ""
    time_list: List[float] = field(default_factory=list)
    memory_list: List[float] = field(default_factory=list)
    compute_time_list: List[float] = field(default_factory=list)
    total_gpu_time: float = 0
    breakdown_ideal_time_per_gpu: List[float] = field(default_factory=list)
    breakdown_eff_loss_time_per_gpu: List[float] = field(default_factory=list)
    breakdown_recomp_time_per_gpu: List[float] = field(default_factory=list)
    efficient_time_list: List[float] = field(default_factory=list)
    adaptive_times: int = 0


def get_config(num_ops_list, tp_size_list, dp_size_list, recompute_ops, aggregate_mbs, global_batch_size,
               full_op_list, algo_list) -> AcesoConfig:
    """Flat per-op lists + ops per stage -> AcesoConfig (aceso_utils.py:96-115): a stage's
    device count is tp*dp of its first op."""
    stages, start = [], 0
    num_stages = len(num_ops_list)
    for i, n in enumerate(num_ops_list):
        end = start + n
        stages.append(AcesoStageInfo(
            index=i, num_stages_behind=num_stages - 1 - i,
            num_gpus=tp_size_list[start] * dp_size_list[start],
            ops=list(full_op_list[start:end]), recompute_ops=list(recompute_ops[start:end]),
            tp_size=list(tp_size_list[start:end]), dp_size=list(dp_size_list[start:end]),
            algo=list(algo_list[start:end])))
        start = end
    return AcesoConfig(global_bs=global_batch_size, micro_bs=aggregate_mbs, stages=stages, num_stages=num_stages)


def config_from_json(path_or_dict, full_op_list) -> AcesoConfig:
    """Plan JSON as the reference writes it (aceso_utils.py:137-211) -> AcesoConfig (:213-242)."""
    d = path_or_dict
    if not isinstance(d, dict):
        with open(d) as f:
            d = json.load(f)
    flat = lambda ll: [x for l in ll for x in l]
    return get_config(d["num_ops_in_each_stage"], flat(d["model_parallel_size_of_each_op"]),
                      flat(d["data_parallel_size_of_each_op"]), flat(d["recompute_ops"]),
                      d["micro_batch_size"], d["global_batch_size"], full_op_list, flat(d["algo_of_each_op"]))


def config_details(config, get_string=False):
    """Per-stage op counts, tp, dp, recompute, micro-batch and algo of a plan, as the reference's
    visited sets key on (aceso_utils.py:117-135; same string when get_string is set)."""
    if config is None:
        return ""
    num_ops_stage = [len(st.ops) for st in config.stages[:config.num_stages]]
    tp_size_list = [st.tp_size for st in config.stages[:config.num_stages]]
    dp_size_list = [st.dp_size for st in config.stages[:config.num_stages]]
    recompute_ops = [st.recompute_ops for st in config.stages[:config.num_stages]]
    algo_list = [st.algo for st in config.stages[:config.num_stages]]
    if get_string:
        return f"{num_ops_stage}, {tp_size_list}, {dp_size_list}, {recompute_ops}, {config.micro_bs}, {algo_list}"
    return num_ops_stage, tp_size_list, dp_size_list, recompute_ops, config.micro_bs, algo_list


def is_visited(visited_set, hash_str, target=""):
    """aceso_utils.py:831-838"""
    return hash_str in visited_set and target in visited_set[hash_str]


def mark_visited(visited_set, hash_str, target=""):
    """aceso_utils.py:840-844"""
    visited_set.setdefault(hash_str, []).append(target)


def num_visited(visited_set, hash_str):
    """aceso_utils.py:846-850"""
    return len(visited_set.get(hash_str, ()))


def cross_node_bits(stage_gpus: Sequence[int], gpus_per_node: int) -> int:
    """in/out cross-node flags of every stage (aceso_cost_model.py:572-574)."""
    bits, till_now = 0, 0
    for s, g in enumerate(stage_gpus):
        if till_now % gpus_per_node == 0 and till_now > 0:
            bits |= 1 << s
        till_now += g
        if till_now % gpus_per_node == 0:
            bits |= 1 << (16 + s)
    return bits


def _flat_ints(stages, key: str, count: int) -> np.ndarray:
    """The per-op list `key` of all stages as one int64 array of `count` entries (ValueError if the lengths do not add
    up).  Small non-negative values, the usual case, go through bytes(): three times faster than numpy's own conversion
    of a Python list."""
    flat = []
    for st in stages:
        flat += getattr(st, key)
    try:
        a = np.frombuffer(bytes(flat), dtype=np.uint8).astype(np.int64)
    except (ValueError, TypeError):          # a value outside 0..255, or not a plain int
        a = np.fromiter(flat, dtype=np.int64, count=len(flat))
    if len(a) != count:
        raise ValueError(f"{key}: {len(a)} entries for {count} ops")
    return a


@dataclass
class PlanBatch:
    codes: np.ndarray        # uint8 [P, N]
    hdr: np.ndarray          # uint32 [P, 4]

    @property
    def n_plans(self):
        return self.codes.shape[0]

    @property
    def num_ops(self):
        return self.codes.shape[1]

    def slice(self, lo, hi):
        return PlanBatch(self.codes[lo:hi], self.hdr[lo:hi])

    @staticmethod
    def concat(batches):
        return PlanBatch(np.concatenate([b.codes for b in batches]), np.concatenate([b.hdr for b in batches]))

    # ---- object form -> array form -----------------------------------------------------------
    @classmethod
    def from_configs(cls, configs: Sequence, tables: CompiledTables, single_stage_intra_node: bool = False):
        """Encode AcesoConfig-like objects.  Raises KeyError for a micro-batch size that is not
        profiled (as aceso_cost_model.py:22-25 does) and ValueError for plans the encoding cannot
        hold.  `single_stage_intra_node` forces both cross-node flags off, which is what the
        single-stage queries do (aceso_cost_model.py:494-495)."""
        db = tables.db
        N = tables.graph.num_ops
        A = db.n_algo
        mbs_index = {m: k for k, m in enumerate(db.mbs_list)}
        # tp size -> index in the profile database (0xff: not profiled), as a lookup table
        tp_lut = np.full(max(db.tp_list) + 2, 0xff, dtype=np.uint8)
        tp_lut[np.asarray(db.tp_list)] = np.arange(len(db.tp_list), dtype=np.uint8)
        P = len(configs)
        codes = np.zeros((P, N), dtype=np.uint8)
        hdr = np.zeros((P, 4), dtype=np.uint32)
        gpn = tables.settings.num_gpus_per_node
        chain = itertools.chain.from_iterable
        for p, cfg in enumerate(configs):
            S = cfg.num_stages
            if S < 1 or S > MAX_STAGES:
                raise ValueError(f"plan {p}: {S} stages (1..{MAX_STAGES} supported)")
            bidx = mbs_index[cfg.micro_bs]
            stages = cfg.stages
            lens = [len(st.ops) for st in stages]
            glogs = 0
            gl = []
            for s, st in enumerate(stages):
                if lens[s] == 0:
                    raise ValueError(f"plan {p}: stage {s} is empty")
                g = st.tp_size[0] * st.dp_size[0]
                if g & (g - 1) or g.bit_length() - 1 > 15:
                    raise ValueError(f"plan {p}: stage {s} has {g} devices (power of two expected)")
                gl.append(g)
                glogs |= (g.bit_length() - 1) << (4 * s)
                for d in set(st.dp_size):
                    if cfg.micro_bs // d not in mbs_index:
                        raise KeyError(cfg.micro_bs // d)
            total = sum(lens)
            if total != N:
                raise ValueError(f"plan {p} has {total} ops, the op graph {N}")
            # the per-op lists of all stages, flattened once each
            tp, dp, al, rc = (_flat_ints(stages, key, N) for key in ("tp_size", "dp_size", "algo", "recompute_ops"))
            g_of_op = np.repeat(np.asarray(gl, dtype=np.int64), lens)
            bad = np.flatnonzero(tp * dp != g_of_op)
            if len(bad):
                s = int(np.searchsorted(np.cumsum(lens), bad[0], side="right"))
                raise ValueError(f"plan {p}: stage {s} mixes tp*dp products")
            t = tp_lut[np.clip(tp, 0, len(tp_lut) - 1)]
            if (t == 0xff).any():
                raise ValueError(f"plan {p}: tp size {int(tp[np.flatnonzero(t == 0xff)[0]])} is not in the profile database")
            if ((al < 0) | (al >= A)).any():
                raise ValueError(f"plan {p}: algo index outside the profile database")
            row = (t * A + al.astype(np.uint8)) | ((rc == 1).astype(np.uint8) << 3)
            starts = np.cumsum([0] + lens[:-1])
            row[starts] |= 1 << 4
            codes[p] = row
            hdr[p, 0] = S | (bidx << 8)
            hdr[p, 1] = glogs & 0xFFFFFFFF
            hdr[p, 2] = glogs >> 32
            hdr[p, 3] = 0 if single_stage_intra_node else cross_node_bits(gl, gpn)
        return cls(codes, hdr)

    # ---- array form -> object form -------------------------------------------------------------
    def to_config(self, p: int, tables: CompiledTables, cls_config=AcesoConfig, cls_stage=AcesoStageInfo):
        db = tables.db
        A = db.n_algo
        row = self.codes[p]
        S = int(self.hdr[p, 0] & 0xff)
        micro_bs = db.mbs_list[int(self.hdr[p, 0] >> 8) & 0xff]
        glogs = int(self.hdr[p, 1]) | (int(self.hdr[p, 2]) << 32)
        starts = np.flatnonzero(row & 16).tolist() + [len(row)]
        assert len(starts) - 1 == S and starts[0] == 0
        ops = tables.graph.ops
        stages = []
        for s in range(S):
            lo, hi = starts[s], starts[s + 1]
            g = 1 << ((glogs >> (4 * s)) & 15)
            c = row[lo:hi] & 7
            tp = [db.tp_list[int(x) // A] for x in c]
            stages.append(cls_stage(index=s, num_stages_behind=S - 1 - s, num_gpus=g, ops=list(ops[lo:hi]),
                                    recompute_ops=[int(x) for x in (row[lo:hi] >> 3) & 1], tp_size=tp,
                                    dp_size=[g // t for t in tp], algo=[int(x) % A for x in c]))
        return cls_config(global_bs=tables.settings.global_batch_size, micro_bs=micro_bs, stages=stages, num_stages=S)

    # ---- device layout -------------------------------------------------------------------------
    def device_codes_host(self) -> np.ndarray:
        """[ceil(N/16)][P][16] uint8, the layout ace_batch_t.d_codes expects (built on the host)."""
        P, N = self.codes.shape
        G = (N + 15) // 16
        padded = np.zeros((P, G * 16), dtype=np.uint8)
        padded[:, :N] = self.codes
        return np.ascontiguousarray(padded.reshape(P, G, 16).transpose(1, 0, 2))


def validate_batch(batch: PlanBatch, tables: CompiledTables) -> Optional[str]:
    """Cheap structural check of an array-form batch; returns a message or None."""
    P, N = batch.codes.shape
    if N != tables.graph.num_ops:
        return f"batch has {N} ops per plan, op graph {tables.graph.num_ops}"
    if P == 0:
        return "empty batch"
    S = batch.hdr[:, 0] & 0xff
    if np.any(S < 1) or np.any(S > MAX_STAGES):
        return "num_stages outside 1..16"
    if np.any(((batch.codes >> 4) & 1).sum(axis=1) != S):
        return "stage-start bits disagree with num_stages"
    if np.any((batch.codes[:, 0] & 16) == 0):
        return "op 0 must start a stage"
    if np.any((batch.hdr[:, 0] >> 8) & 0xff >= len(tables.db.mbs_list)):
        return "micro-batch index outside the profile database"
    if np.any((batch.codes & 7) >= tables.C):
        return "tp/algo code outside the profile database"
    return None


# model_size -> (num_layers, seq_len, hidden, ffn_hidden, heads, kv_channels, vocab)  (aceso_utils.py:27-34)
GPT_CONFIGS = {
    "350M": (24, 2048, 1024, 4096, 16, 64, 51200), "1_3B": (24, 2048, 2048, 8192, 32, 64, 51200),
    "2_6B": (32, 2048, 2560, 10240, 32, 80, 51200), "6_7B": (32, 2048, 4096, 16384, 32, 128, 51200),
    "13B": (40, 2048, 5120, 20480, 40, 128, 51200), "scale-layer": (1, 2048, 512, 2048, 8, 64, 51200),
}
# model_size -> (num_layers, enc_seq, dec_seq, hidden, ffn_hidden, heads, kv_channels, vocab)  (aceso_utils.py:38-45)
T5_CONFIGS = {
    "770M": (24, 2048, 512, 1024, 4096, 16, 64, 30592), "3B": (24, 2048, 512, 1024, 16384, 32, 128, 30592),
    "6B": (24, 2048, 512, 1024, 32768, 64, 128, 30592), "11B": (24, 2048, 512, 1024, 65536, 128, 128, 30592),
    "22B": (48, 2048, 512, 1024, 65536, 128, 128, 30592),
}
# model_size -> (blocks per stage, in_channels, width_factor)  (aceso_utils.py:16-24)
RESNET_CONFIGS = {
    "250M": ([3, 4, 6, 3], 160, 2), "500M": ([3, 4, 6, 3], 224, 2), "1B": ([3, 4, 6, 3], 320, 2),
    "2B": ([3, 4, 6, 3], 448, 2), "4B": ([3, 4, 6, 3], 640, 2), "6_8B": ([3, 4, 6, 3], 320, 16),
    "13B": ([3, 4, 23, 3], 320, 16),
}


def config_to_json_dict(config, model_name: str, model_size: str, num_layers=None) -> dict:
    """The plan JSON the training runtime consumes (aceso_utils.py:137-211), as a dict."""
    if model_name == "scale-layer":
        model_name, model_size = "gpt", "scale-layer"
    d = {"model_name": model_name, "model_size": model_size}
    if model_name == "resnet":
        layers, in_channels, width = RESNET_CONFIGS[model_size]
        d.update(num_layers=layers, in_channels=in_channels, width_factor=width)
    elif model_name == "gpt":
        n, seq, hidden, _, heads, _, _ = GPT_CONFIGS[model_size]
        d.update(num_layers=num_layers if num_layers is not None else n, seq_length=seq,
                 max_position_embeddings=seq, num_attention_heads=heads, hidden_size=hidden)
    elif model_name == "t5":
        n, enc, dec, hidden, ffn, heads, kv, _ = T5_CONFIGS[model_size]
        d.update(num_layers=num_layers if num_layers is not None else n, encoder_seq_length=enc,
                 decoder_seq_length=dec, max_position_embeddings=enc, num_attention_heads=heads, kv_channels=kv,
                 hidden_size=hidden, ffn_hidden_size=ffn)
    else:
        raise RuntimeError(f"{model_name} not supportted.")
    d["global_batch_size"] = config.global_bs
    d["micro_batch_size"] = config.micro_bs
    d["num_stages"] = config.num_stages
    d["num_gpus"] = [st.num_gpus for st in config.stages]
    d["checkpoint_activations"] = [max(st.recompute_ops) > 0 for st in config.stages]
    d["resharding_stages"] = [max(st.tp_size) != min(st.tp_size) or max(st.dp_size) != min(st.dp_size) or
                              max(st.algo) != min(st.algo) for st in config.stages]
    d["num_ops_in_each_stage"] = [len(st.ops) for st in config.stages]
    d["model_parallel_size_of_each_op"] = [list(st.tp_size) for st in config.stages]
    d["data_parallel_size_of_each_op"] = [list(st.dp_size) for st in config.stages]
    d["recompute_ops"] = [list(st.recompute_ops) for st in config.stages]
    d["algo_of_each_op"] = [list(st.algo) for st in config.stages]
    return d


def dump_config_to_json(config, file_name: str, model_name: str, model_size: str, num_layers=None) -> None:
    with open(file_name, "w") as f:
        json.dump(config_to_json_dict(config, model_name, model_size, num_layers), f, indent=4)


def sort_configs(config_list, sort_metric):
    """aceso_utils.py:723-758: scored plans in ascending order of their slowest stage ("max_stage_time") or of
    `total_gpu_time`; plans that compare equal keep their order (the reference inserts a plan in front of the first
    one that is strictly larger).  For encoded batches the same order comes from CostModel.top_k."""
    if sort_metric == "max_stage_time":
        return sorted(config_list, key=lambda c: max(c.time_list))
    if sort_metric == "total_gpu_time":
        return sorted(config_list, key=lambda c: c.total_gpu_time)
    raise RuntimeError(f"sort_metric {sort_metric} not supported.")


def save_config_info_to_csv(config, reserved_mem_list, file_name: str) -> None:
    """aceso_utils.py:244-252: one line per stage of a scored plan (time, total / normal / reserved memory)."""
    import csv
    rows = [["stage-index", "time", "memory(total)", "memory(normal)", "memory(reserved)"]]
    for i in range(config.num_stages):
        rows.append([f"stage-{i}", f"{config.time_list[i]:.2f}", f"{config.memory_list[i]:.2f}",
                     f"{(config.memory_list[i] - reserved_mem_list[i]):.2f}", f"{reserved_mem_list[i]:.2f}"])
    with open(file_name, mode="w", newline="") as f:
        csv.writer(f).writerows(rows)


def check_legality(config, num_gpus: int, num_gpus_per_node: int, num_nodes: int) -> bool:
    """aceso_utils.py:760-774: stage sizes in {1,2,4,8}, all devices used, node boundaries fall on
    stage boundaries."""
    total, from_start = 0, []
    for st in config.stages:
        if st.num_gpus not in (1, 2, 4, 8):
            return False
        total += st.num_gpus
        from_start.append(total)
    if total != num_gpus:
        return False
    return all(num_gpus_per_node * i in from_start for i in range(1, num_nodes + 1))
