"""Op graphs and per-op rules of the three model families the Aceso cost model scores.

Mirrors the reference's search/model_ops_info.py (op lists :10-53, tunable ops :55-74,
never-recomputed ops :76-90, sharding specs :92-150) and the name predicates buried in
search/aceso_cost_model.py (:386-388, :408-412, :433-439, :798), but as data: every rule is
turned into a per-op-type flag or a small integer "layout kind" once, so that nothing on the
scoring path ever looks at an op name again.
"""
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import numpy as np

# ---- layout kinds (reference: model_ops_info.py:92-150) -------------------------------------
# A sharding spec there is {"R": replicas, "V": 1, "dims": [d0, d1, d2]} built from the op's
# tp and dp.  Only four shapes (plus "no spec") ever occur:
K_NONE = 0   # None: compares identical to anything (aceso_cost_model.py:187-188)
K_REP_D1 = 1  # R=tp, dims [1, dp, 1]
K_REP_D0 = 2  # R=tp, dims [dp, 1, 1]
K_D1_D2 = 3  # R=1,  dims [1, dp, tp]
K_D0_D1 = 4  # R=1,  dims [dp, tp, 1]


def kind_layout(kind: int, tp: int, dp: int) -> Optional[Tuple[int, Tuple[int, int, int]]]:
    """(replicas, per-dim partitions) of a layout kind at a given tp/dp."""
    if kind == K_NONE:
        return None
    if kind == K_REP_D1:
        return tp, (1, dp, 1)
    if kind == K_REP_D0:
        return tp, (dp, 1, 1)
    if kind == K_D1_D2:
        return 1, (1, dp, tp)
    if kind == K_D0_D1:
        return 1, (dp, tp, 1)
    raise ValueError(kind)


# (input kind, output kind) per algo for the GPT-style ops; model_ops_info.py:93-147
_COL = (K_REP_D1, K_D1_D2)   # column-parallel GEMM: replicated in, hidden-dim-split out
_ROW = (K_D1_D2, K_REP_D1)   # row-parallel GEMM
_GPT_KINDS = {
    "encoder-embedding": ((K_NONE, K_REP_D1),) * 2,
    "enc-1st-layernorm": ((K_REP_D1, K_REP_D1),) * 2,
    "enc-2nd-layernorm": ((K_REP_D1, K_REP_D1),) * 2,
    "final-layernorm": ((K_REP_D1, K_REP_D0),) * 2,
    "enc-attention-qkv": (_COL, _ROW),
    "enc-MLP-GEMM-1": (_COL, _ROW),
    "enc-attention-score": ((K_D1_D2, K_D0_D1),) * 2,
    "enc-attention-softmax": ((K_D0_D1, K_D0_D1),) * 2,
    "enc-attention-dropout": ((K_D0_D1, K_D0_D1),) * 2,
    "enc-attention-context": ((K_D0_D1, K_D1_D2),) * 2,
    "enc-attention-dense": (_ROW, _COL),
    "enc-MLP-GEMM-2": (_ROW, _COL),
    "enc-post-attention-dropout": ((K_REP_D1, K_REP_D1),) * 2,
    "enc-post-MLP-dropout": ((K_REP_D1, K_REP_D1),) * 2,
    "enc-MLP-gelu": ((K_D1_D2, K_D1_D2),) * 2,
    "gpt-post-process": ((K_REP_D0, K_NONE),) * 2,
}
_RESNET_MARKS = ("conv", "downsample", "bn", "relu", "pool", "fc")  # model_ops_info.py:149


def spec_kinds(op_name: str) -> Tuple[Tuple[int, int], Tuple[int, int]]:
    """((in kind, out kind) for algo 0, same for algo 1).  Names the reference's if-chain
    does not know fall through to None there, i.e. K_NONE."""
    if op_name in _GPT_KINDS:
        return _GPT_KINDS[op_name]
    if any(m in op_name for m in _RESNET_MARKS):
        return ((K_REP_D0, K_REP_D0),) * 2
    return ((K_NONE, K_NONE),) * 2


# prim ids used in the device tables
P_NONE, P_SPLIT, P_ALL_GATHER, P_ALL_TO_ALL, P_ALL_REDUCE, P_REDUCE_SCATTER = range(6)
PRIM_NAMES = {P_SPLIT: "split", P_ALL_GATHER: "all_gather", P_ALL_TO_ALL: "all_to_all",
              P_ALL_REDUCE: "all_reduce", P_REDUCE_SCATTER: "reduce_scatter"}


class InconsistentSpecs(Exception):
    """No resharding rule applies (the reference then fails to unpack a None,
    aceso_cost_model.py:344)."""


def reshard_prims(src, dst) -> Tuple[int, int, int]:
    """(forward prim, backward prim, group size) that turns layout `src` (what the previous op
    produced) into layout `dst` (what the next op needs); aceso_cost_model.py:200-245 with
    V == 1 throughout (so its all_reduce / reduce_scatter branches cannot fire)."""
    if src is None or dst is None or src == dst:
        return P_NONE, P_NONE, 0
    (rs, ds), (rd, dd) = src, dst
    if rs > rd:
        if any(ds[k] < dd[k] for k in range(3)):
            return P_SPLIT, P_ALL_GATHER, rs // rd
        raise InconsistentSpecs((src, dst))
    for s in range(3):
        if ds[s] > dd[s]:
            if rs < rd:
                return P_ALL_GATHER, P_SPLIT, ds[s] // dd[s]
            for d in range(3):
                if d != s and ds[d] < dd[d]:
                    return P_ALL_TO_ALL, P_ALL_TO_ALL, ds[s] // dd[s]
    raise InconsistentSpecs((src, dst))


# ---- per-type flags -----------------------------------------------------------------------
F_ACT_X1_5 = 1      # activation counted 1.5x (aceso_cost_model.py:386)
F_ACT_ZERO = 2      # activation shares its producer's buffer, counted 0 (:388)
F_LAYER_START = 4   # recompute segments end in front of this op (:412, :439)
F_TUNABLE = 8       # supports tensor parallelism (model_ops_info.py:55-74)
F_NO_RECOMPUTE = 16  # never chosen by the greedy recompute pass (model_ops_info.py:76-90, cost_model:798)


def type_flags(model_name: str, op_name: str) -> int:
    f = 0
    if op_name == "enc-attention-dropout":
        f |= F_ACT_X1_5
    if (op_name in ("enc-attention-softmax", "bn1") or "-bn3" in op_name or
            ("-downsample" in op_name and "0-0" not in op_name)):
        f |= F_ACT_ZERO
    if op_name == "enc-1st-layernorm" or "-conv1" in op_name:
        f |= F_LAYER_START
    if model_name in ("gpt", "scale-layer"):
        tunable = op_name in ("encoder-embedding", "enc-attention-qkv", "enc-attention-dense",
                              "enc-MLP-GEMM-1", "enc-MLP-GEMM-2")
        norc = op_name in ("encoder-embedding", "gpt-post-process")
    elif model_name == "t5":
        tunable = op_name in ("encoder-embedding", "enc-attention-qkv", "enc-attention-dense",
                              "enc-MLP-GEMM-1", "enc-MLP-GEMM-2", "dec-attention-qkv-1",
                              "dec-attention-dense-1", "dec-attention-qkv-2", "dec-attention-dense-2",
                              "dec-MLP-GEMM-1", "dec-MLP-GEMM-2")
        norc = op_name in ("encoder-embedding", "decoder-embedding", "t5-post-process")
    elif model_name == "resnet":
        tunable = "conv" in op_name or "downsample" in op_name
        norc = op_name == "conv1"
    else:
        raise RuntimeError(f"model {model_name} not supported yet.")
    # the greedy pass also never starts a group at a layer start or a relu (cost_model:798)
    if f & F_LAYER_START or "-relu" in op_name:
        norc = True
    return f | (F_TUNABLE if tunable else 0) | (F_NO_RECOMPUTE if norc else 0)


# ---- op-name lists ------------------------------------------------------------------------
GPT_TYPES = ["encoder-embedding", "enc-1st-layernorm", "enc-attention-qkv", "enc-attention-score",
             "enc-attention-softmax", "enc-attention-dropout", "enc-attention-context",
             "enc-attention-dense", "enc-post-attention-dropout", "enc-2nd-layernorm",
             "enc-MLP-GEMM-1", "enc-MLP-gelu", "enc-MLP-GEMM-2", "enc-post-MLP-dropout",
             "final-layernorm", "gpt-post-process"]

T5_TYPES = GPT_TYPES[:14] + ["enc-final-layernorm", "decoder-embedding", "dec-1st-layernorm"] + \
    [f"dec-attention-{x}-1" for x in ("qkv", "score", "softmax", "dropout", "context", "dense")] + \
    ["dec-post-attention-dropout-1", "dec-2nd-layernorm"] + \
    [f"dec-attention-{x}-2" for x in ("qkv", "score", "softmax", "dropout", "context", "dense")] + \
    ["dec-post-attention-dropout-2", "dec-3rd-layernorm", "dec-MLP-GEMM-1", "dec-MLP-gelu",
     "dec-MLP-GEMM-2", "dec-post-MLP-dropout", "dec-final-layernorm", "t5-post-process"]


def resnet_types(blocks: Sequence[int] = (3, 4, 6, 3)) -> List[str]:
    names = ["conv1", "bn1", "relu1", "maxpool"]
    for b, n in enumerate(blocks):
        for k in range(n):
            names += [f"block-{b}-{k}-{x}" for x in
                      ("conv1", "bn1", "conv2", "bn2", "conv3", "bn3", "downsample", "relu")]
    return names + ["avgpool", "fc"]


def full_op_list(model_name: str, op_list: Sequence[str], num_layers: Optional[int]) -> List[str]:
    """The op sequence of the whole model from the database's op list
    (model_ops_info.py:30-53): GPT = head + 13-op layer x L + 2 tail ops; T5 = encoder
    (1 + 13 L + 1) then decoder (1 + 21 L + 2); ResNet = the list itself."""
    op_list = list(op_list)
    if model_name in ("gpt", "scale-layer"):
        return [op_list[0]] + op_list[1:14] * num_layers + op_list[14:]
    if model_name == "t5":
        return ([op_list[0]] + op_list[1:14] * num_layers + [op_list[14]] +
                [op_list[15]] + op_list[16:37] * num_layers + op_list[37:])
    if model_name == "resnet":
        return op_list
    raise RuntimeError(f"model {model_name} not supported yet.")


@dataclass
class OpGraph:
    """One model's op sequence in index form."""
    model_name: str
    type_names: List[str]          # distinct op names = rows of the profile database
    ops: List[str]                 # op name per position
    type_of_pos: np.ndarray        # int32 [N]
    flags: np.ndarray              # int32 [n_types]

    @property
    def num_ops(self) -> int:
        return len(self.ops)

    @classmethod
    def build(cls, model_name: str, type_names: Sequence[str], num_layers: Optional[int] = None):
        type_names = list(type_names)
        ops = full_op_list(model_name, type_names, num_layers)
        index = {n: k for k, n in enumerate(type_names)}
        return cls(model_name=model_name, type_names=type_names, ops=ops,
                   type_of_pos=np.array([index[o] for o in ops], dtype=np.int32),
                   flags=np.array([type_flags(model_name, n) for n in type_names], dtype=np.int32))
