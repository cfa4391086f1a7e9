"""The profiled-op database the cost model scores plans against, as dense arrays.

File formats are the reference profiler's (profiler/op_profiler.py:461-482 op tables,
profiler/comm_profiler.py:160-169 collectives, profiler/p2p_band_profiler.py:22-63
bandwidth) and the loading rules are those of search/aceso_cost_model.py:27-183:
missing op files leave the 1,000,000 default in place, collectives are keyed by the
size string as written in the file, the inter-node bandwidth table falls back to the
intra-node one.
"""
import csv
import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import numpy as np

FIELDS = ("fwd", "bwd", "input_size", "output_size", "weights", "activations",
          "reserved_fwd", "reserved_bwd")
MISSING = 1000000.0   # aceso_cost_model.py:97-106

# aceso_utils.py:48-52 (bytes of fp32 master params / optimizer state per weight byte)
MEMORY_RATIO = {"resnet": (0, 2), "gpt": (2, 4), "t5": (2, 4), "scale-layer": (2, 4)}


@dataclass
class CostModelSettings:
    """The flags of the reference's argparse singleton that change what the model returns
    (aceso_utils.py:359-531)."""
    model_name: str
    micro_batch_size: List[int]
    num_gpus_per_node: int
    global_batch_size: int = 1024
    memory_limit: float = 28000.0
    max_tp: Optional[int] = None
    consider_shared_space: bool = True
    consider_reserved_space: bool = True
    flex_recompute: bool = True
    peak_mem_in_backward: int = 0
    memory_pred_type: str = "MAX"
    resharding: Optional[bool] = None
    consider_collective_memory: bool = False     # aceso_utils.py:448, aceso_cost_model.py:462-478

    def __post_init__(self):
        if self.max_tp is None:
            self.max_tp = self.num_gpus_per_node
        if self.resharding is None:
            self.resharding = self.model_name != "t5"
        if self.model_name not in MEMORY_RATIO:
            raise RuntimeError(f"model {self.model_name} is not supported yet.")
        if self.memory_pred_type not in ("MAX", "MIN"):
            raise RuntimeError(f"unknown args.memory_pred_type {self.memory_pred_type}")

    @property
    def memory_main_params(self):
        return MEMORY_RATIO[self.model_name][0]

    @property
    def memory_optimizer(self):
        return MEMORY_RATIO[self.model_name][1]


@dataclass
class ProfileDB:
    model_name: str
    op_names: List[str]
    mbs_list: List[int]
    tp_list: List[int]                      # 1, 2, 4, ... (powers of two)
    n_algo: int
    tables: Dict[str, np.ndarray]           # field -> float64 [n_types, n_mbs, n_tp, n_algo]
    collectives: Dict[str, Dict[int, Dict[str, float]]] = field(default_factory=dict)
    intra_band: List[float] = field(default_factory=list)
    inter_band: List[float] = field(default_factory=list)

    @classmethod
    def empty(cls, model_name, op_names, mbs_list, tp_list, n_algo):
        shape = (len(op_names), len(mbs_list), len(tp_list), n_algo)
        return cls(model_name, list(op_names), list(mbs_list), list(tp_list), n_algo,
                   {f: np.full(shape, MISSING, dtype=np.float64) for f in FIELDS})

    # ---- reference file format ------------------------------------------------------------
    @staticmethod
    def tp_sizes(model_name, model_size, max_tp):
        """aceso_cost_model.py:35-45."""
        small = (model_name == "gpt" and model_size == "350M") or (model_name == "t5" and model_size == "220M")
        cap = min(max_tp, 4 if small else 8)
        out, tp = [], 1
        while tp <= cap:
            out.append(tp)
            tp *= 2
        return out

    @classmethod
    def from_directory(cls, model_name, model_size, time_path, settings: CostModelSettings, verbose=False):
        """Load `<model>_<size>_mbs{m}_tp{t}_algo{a}.csv`, `prim_*_{n}gpus.csv` and
        `p2p_{intra,inter}_node.csv` from `time_path` (must end with the path separator, the
        reference concatenates strings)."""
        mbs_list = list(settings.micro_batch_size)
        tp_list = cls.tp_sizes(model_name, model_size, settings.max_tp)
        n_algo = 1 if model_name == "t5" else 2
        stem = "gpt_scale-layer" if model_name == "scale-layer" else \
            f"{model_name}_{'11B' if (model_name == 't5' and model_size == '22B') else model_size}"
        # the op list is whatever the first micro-batch size's tp1/algo0 file lists (model_ops_info.py:10-28)
        op_names = []
        with open(f"{time_path}{stem}_mbs{mbs_list[0]}_tp1_algo0.csv") as f:
            for k, row in enumerate(csv.reader(f)):
                if k > 0:
                    op_names.append(row[0])
        db = cls.empty(model_name, op_names, mbs_list, tp_list, n_algo)
        index = {n: k for k, n in enumerate(op_names)}
        cols = ["fwd", "bwd", "input_size", "output_size", "weights", "activations"]
        if settings.consider_reserved_space:
            cols += ["reserved_fwd", "reserved_bwd"]
        for mi, mbs in enumerate(mbs_list):
            for ti, tp in enumerate(tp_list):
                for ai in range(n_algo):
                    path = f"{time_path}{stem}_mbs{mbs}_tp{tp}_algo{ai}.csv"
                    try:
                        with open(path) as f:
                            for k, row in enumerate(csv.reader(f)):
                                if k > 0:
                                    t = index[row[0]]
                                    for c, name in enumerate(cols):
                                        db.tables[name][t, mi, ti, ai] = float(row[1 + c])
                    except (OSError, KeyError, ValueError, IndexError):
                        if verbose:
                            print(f"file ({path}) not exist, or the file is not formatted as expected.")
        prims = {"gpt": ["all_gather", "all_reduce", "reduce_scatter", "all_to_all"],
                 "scale-layer": ["all_gather", "all_reduce", "reduce_scatter", "all_to_all"],
                 "t5": [], "resnet": ["all_gather", "all_to_all"]}[model_name]
        cstem = "gpt_scale-layer" if model_name == "scale-layer" else f"{model_name}_{model_size}"
        for prim in prims:
            db.collectives[prim] = {}
            for n in tp_list[1:]:
                d = {}
                with open(f"{time_path}prim_{cstem}_{prim}_{n}gpus.csv") as f:   # missing file raises, as in the reference
                    for k, row in enumerate(csv.reader(f)):
                        if k > 0:
                            d[row[0]] = float(row[1])
                db.collectives[prim][n] = d

        def band(path):
            with open(path) as f:
                rows = list(csv.reader(f))
            return [float(x) for x in rows[1]]
        db.intra_band = band(time_path + "p2p_intra_node.csv")
        try:
            db.inter_band = band(time_path + "p2p_inter_node.csv")
        except OSError:
            if verbose:
                print("inter-node bandwidth file is not found, using intra-node bandwidth instead.")
            db.inter_band = list(db.intra_band)
        return db

    # ---- lookups with the reference's quirks ----------------------------------------------
    def reshard_time(self, prim: str, num_devices: int, data_size: float) -> float:
        """Milliseconds of one collective (aceso_cost_model.py:247-260): exact string key of
        the size rounded half-to-even, else the key of size-1, else 100000; split is free.
        KeyError if the primitive / group size was never profiled."""
        if prim == "split":
            return 0.0
        if prim not in ("all_reduce", "all_gather", "reduce_scatter", "all_to_all"):
            return 100000.0
        table = self.collectives[prim][num_devices]
        key = "{:.0f}".format(float(data_size))
        if key in table:
            return table[key]
        key = "{:.0f}".format(float(data_size) - 1)
        if key in table:
            return table[key]
        return 100000.0

    @staticmethod
    def p2p_time(data_size: float, band: List[float]) -> float:
        """size / bandwidth(size) of aceso_cost_model.py:275-299, 328-336: bucket
        int(log2(size)) (truncated toward zero), shifted down by one when >= 1, clamped to
        the last bucket above, wrapping Python-style below zero; GB/s * 0.001; sizes <= 0
        divide by 1.  NaN where the reference would raise IndexError."""
        if data_size > 0:
            idx = int(math.log(data_size, 2))
            if idx >= 1:
                idx -= 1
            if idx >= len(band):
                bw = band[-1] * 0.001
            elif idx < -len(band):
                return math.nan
            else:
                bw = band[idx] * 0.001
        else:
            bw = 1
        return data_size / bw
