"""CPU oracle for the Aceso plan cost model -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
file; the product package (superscaler_amd/) never does.

It is a loop-faithful restatement of the reference's pure-Python cost model
(/root/reference/search/aceso_cost_model.py, model_ops_info.py, aceso_utils.py): the same
evaluation order, the same operations in the same association, so that every float it
returns is bit-identical to what the reference computes from the same tables.  State that
the reference keeps in module globals / the argparse singleton is explicit here
(`Settings`, `Oracle`).

Pinning status (what independently checks each function; see tests/test_oracle_*.py):
  read_profiled_time / get_time_v3 / bands / recompute time / 1F1B composition:
      KAT-1  gpt_350M single-GPU plan -> 200.71 s published, closed form 200712.935038 ms
  get_memory_v3 / get_activations_v3 / get_peak_activations / get_reserved_memory /
  predict_stage_memory:
      KAT-2  gpt_350M -> 14592 + 5120 MB published;  KAT-3 resnet_500M -> 16519 + 3432 MB
  get_op_spec / get_reshard_primitives: brute force over all spec-kind pairs against an
      independent "what collective turns layout X into layout Y" derivation
  get_reshard_time: key rounding / size-1 fallback / penalty cases from the GPT-13B DB
  multi-stage predict_time_breakdown, efficient_time_list, check_recompute,
  wrap_predict_delta_time, predict_value_after_move: golden vectors written by the
      reference itself (tests/golden/make_golden.py -> tests/golden/*.json)
"""
import csv
import math
from dataclasses import dataclass, field
from typing import List, Optional

# aceso_utils.py:48-52
MEMORY_RATIO = {
    "resnet": {"main_params": 0, "optimizer": 2},
    "gpt": {"main_params": 2, "optimizer": 4},
    "t5": {"main_params": 2, "optimizer": 4},
    "scale-layer": {"main_params": 2, "optimizer": 4},  # aceso_utils.py:516-518
}

MISSING = 1000000  # aceso_cost_model.py:98-106 default for absent table entries


@dataclass
class Settings:
    """The subset of the reference's argparse singleton the cost model reads
    (aceso_utils.py:359-531)."""
    model_name: str
    micro_batch_size: List[int]
    num_gpus_per_node: int
    memory_limit: float = 28000            # aceso_utils.py:377
    max_tp: Optional[int] = None           # aceso_utils.py:503-504 -> num_gpus_per_node
    consider_shared_space: bool = True     # aceso_utils.py:423
    consider_reserved_space: bool = True   # aceso_utils.py:424
    flex_recompute: bool = True            # aceso_utils.py:426
    peak_mem_in_backward: int = 0          # aceso_utils.py:430
    support_comm_predict: bool = False     # aceso_utils.py:435
    consider_collective_memory: bool = False  # aceso_utils.py:448
    memory_pred_type: str = "MAX"          # aceso_utils.py:405
    memory_main_params: float = field(init=False)
    memory_optimizer: float = field(init=False)
    resharding: bool = field(init=False)

    def __post_init__(self):
        if self.max_tp is None:
            self.max_tp = self.num_gpus_per_node
        self.memory_main_params = MEMORY_RATIO[self.model_name]["main_params"]
        self.memory_optimizer = MEMORY_RATIO[self.model_name]["optimizer"]
        self.resharding = self.model_name != "t5"  # aceso_utils.py:523-526


# ----------------------------------------------------------------------------------------
# plan containers (aceso_utils.py:58-115)
# ----------------------------------------------------------------------------------------
@dataclass
class StageInfo:
    index: int
    num_stages_behind: int
    num_gpus: int
    ops: List[str]
    recompute_ops: List[int]
    tp_size: List[int]
    dp_size: List[int]
    algo: List[int]


@dataclass
class Config:
    global_bs: int
    micro_bs: int
    stages: List[StageInfo]
    num_stages: int
    time_list: List[float] = field(default_factory=list)
    memory_list: List[float] = field(default_factory=list)
    compute_time_list: List[float] = field(default_factory=list)
    total_gpu_time: float = 0
    breakdown_ideal_time_per_gpu: List[float] = field(default_factory=list)
    breakdown_eff_loss_time_per_gpu: List[float] = field(default_factory=list)
    breakdown_recomp_time_per_gpu: List[float] = field(default_factory=list)
    efficient_time_list: List[float] = field(default_factory=list)


def get_config(num_ops_list, tp_size_list, dp_size_list, recompute_ops, aggregate_mbs,
               global_batch_size, full_op_list, algo_list):
    """aceso_utils.py:96-115."""
    op_start_index = 0
    num_stages = len(num_ops_list)
    stages = []
    for i in range(num_stages):
        n = num_ops_list[i]
        stages.append(StageInfo(
            index=i,
            num_stages_behind=(num_stages - 1 - i),
            num_gpus=tp_size_list[op_start_index] * dp_size_list[op_start_index],
            ops=list(full_op_list[op_start_index: op_start_index + n]),
            recompute_ops=list(recompute_ops[op_start_index: op_start_index + n]),
            tp_size=list(tp_size_list[op_start_index: op_start_index + n]),
            dp_size=list(dp_size_list[op_start_index: op_start_index + n]),
            algo=list(algo_list[op_start_index: op_start_index + n])))
        op_start_index += n
    return Config(global_bs=global_batch_size, micro_bs=aggregate_mbs, stages=stages,
                  num_stages=num_stages)


def config_from_json_dict(d, full_op_list):
    """aceso_utils.py:213-242 (read_config_from_json), given the parsed JSON dict."""
    flat = lambda ll: [x for l in ll for x in l]
    return get_config(d["num_ops_in_each_stage"],
                      flat(d["model_parallel_size_of_each_op"]),
                      flat(d["data_parallel_size_of_each_op"]),
                      flat(d["recompute_ops"]),
                      d["micro_batch_size"], d["global_batch_size"],
                      full_op_list, flat(d["algo_of_each_op"]))


def get_full_op_list(model_name, op_list, num_layers):
    """model_ops_info.py:30-53."""
    if model_name in ["gpt", "scale-layer"]:
        return [op_list[0]] + op_list[1:14] * num_layers + op_list[14:]
    elif model_name == "t5":
        return ([op_list[0]] + op_list[1:14] * num_layers + [op_list[14]] +
                [op_list[15]] + op_list[16:37] * num_layers + op_list[37:])
    elif model_name == "resnet":
        return list(op_list)
    raise RuntimeError(f"model {model_name} not supported yet.")


def get_no_recompute_op_list(model_name):
    """model_ops_info.py:76-90."""
    if model_name in ["gpt", "scale-layer"]:
        return ["encoder-embedding", "gpt-post-process"]
    elif model_name == "t5":
        return ["encoder-embedding", "decoder-embedding", "t5-post-process"]
    elif model_name == "resnet":
        return ["conv1"]
    raise RuntimeError(f"model {model_name} not supported yet.")


# ----------------------------------------------------------------------------------------
# sharding specs (model_ops_info.py:92-150) and resharding primitives
# ----------------------------------------------------------------------------------------
def get_op_spec(op_name, tp_size, dp_size, algo_index, input_spec):
    """model_ops_info.py:92-150."""
    if op_name in ["encoder-embedding"]:
        if input_spec:
            return None
        return {"R": tp_size, "V": 1, "dims": [1, dp_size, 1]}
    elif op_name in ["enc-1st-layernorm", "enc-2nd-layernorm"]:
        return {"R": tp_size, "V": 1, "dims": [1, dp_size, 1]}
    elif op_name in ["final-layernorm"]:
        if input_spec:
            return {"R": tp_size, "V": 1, "dims": [1, dp_size, 1]}
        return {"R": tp_size, "V": 1, "dims": [dp_size, 1, 1]}
    elif op_name in ["enc-attention-qkv", "enc-MLP-GEMM-1"]:
        if algo_index == 0:
            if input_spec:
                return {"R": tp_size, "V": 1, "dims": [1, dp_size, 1]}
            return {"R": 1, "V": 1, "dims": [1, dp_size, tp_size]}
        elif algo_index == 1:
            if input_spec:
                return {"R": 1, "V": 1, "dims": [1, dp_size, tp_size]}
            return {"R": tp_size, "V": 1, "dims": [1, dp_size, 1]}
    elif op_name in ["enc-attention-score"]:
        if input_spec:
            return {"R": 1, "V": 1, "dims": [1, dp_size, tp_size]}
        return {"R": 1, "V": 1, "dims": [dp_size, tp_size, 1]}
    elif op_name in ["enc-attention-softmax", "enc-attention-dropout"]:
        return {"R": 1, "V": 1, "dims": [dp_size, tp_size, 1]}
    elif op_name in ["enc-attention-context"]:
        if input_spec:
            return {"R": 1, "V": 1, "dims": [dp_size, tp_size, 1]}
        return {"R": 1, "V": 1, "dims": [1, dp_size, tp_size]}
    elif op_name in ["enc-attention-dense", "enc-MLP-GEMM-2"]:
        if algo_index == 0:
            if input_spec:
                return {"R": 1, "V": 1, "dims": [1, dp_size, tp_size]}
            return {"R": tp_size, "V": 1, "dims": [1, dp_size, 1]}
        elif algo_index == 1:
            if input_spec:
                return {"R": tp_size, "V": 1, "dims": [1, dp_size, 1]}
            return {"R": 1, "V": 1, "dims": [1, dp_size, tp_size]}
    elif op_name in ["enc-post-attention-dropout", "enc-post-MLP-dropout"]:
        return {"R": tp_size, "V": 1, "dims": [1, dp_size, 1]}
    elif op_name in ["enc-MLP-gelu"]:
        return {"R": 1, "V": 1, "dims": [1, dp_size, tp_size]}
    elif op_name in ["gpt-post-process"]:
        if input_spec:
            return {"R": tp_size, "V": 1, "dims": [dp_size, 1, 1]}
        return None
    elif ("conv" in op_name or "downsample" in op_name or "bn" in op_name or
          "relu" in op_name or "pool" in op_name or "fc" in op_name):
        return {"R": tp_size, "V": 1, "dims": [dp_size, 1, 1]}
    return None


def identical_spec(input_spec, required_spec):
    """aceso_cost_model.py:185-198."""
    if input_spec is None or required_spec is None:
        return True
    identical = True
    if input_spec["R"] != required_spec["R"]:
        identical = False
    if input_spec["V"] != required_spec["V"]:
        identical = False
    for k in range(len(input_spec["dims"])):
        if input_spec["dims"][k] != required_spec["dims"][k]:
            identical = False
    return identical


def get_reshard_primitives(input_spec, required_spec):
    """aceso_cost_model.py:200-245.  Falls off the end (returns None) when no rule
    matches, exactly like the reference (the caller then fails to unpack)."""
    if identical_spec(input_spec, required_spec):
        return None, None, 0
    if input_spec["R"] > required_spec["R"]:
        for k in range(len(input_spec["dims"])):
            if input_spec["dims"][k] < required_spec["dims"][k]:
                assert input_spec["R"] % required_spec["R"] == 0
                return "split", "all_gather", input_spec["R"] // required_spec["R"]
    elif input_spec["V"] > required_spec["V"]:
        if input_spec["R"] < required_spec["R"]:
            assert input_spec["V"] % required_spec["V"] == 0
            return "all_reduce", None, input_spec["V"] // required_spec["V"]
        for k in range(len(input_spec["dims"])):
            if input_spec["dims"][k] < required_spec["dims"][k]:
                assert input_spec["V"] % required_spec["V"] == 0
                return "reduce_scatter", "all_gather", input_spec["V"] // required_spec["V"]
    else:
        for s in range(len(input_spec["dims"])):
            if input_spec["dims"][s] > required_spec["dims"][s]:
                if input_spec["R"] < required_spec["R"]:
                    assert input_spec["dims"][s] % required_spec["dims"][s] == 0
                    return "all_gather", "split", input_spec["dims"][s] // required_spec["dims"][s]
                for d in range(len(input_spec["dims"])):
                    if d != s and input_spec["dims"][d] < required_spec["dims"][d]:
                        assert input_spec["dims"][s] % required_spec["dims"][s] == 0
                        return "all_to_all", "all_to_all", input_spec["dims"][s] // required_spec["dims"][s]
    return None


def get_reshard_memory(prim, num_devices, data_size):
    """aceso_cost_model.py:262-273."""
    assert num_devices > 1
    if prim in ("all_reduce", "reduce_scatter", "split"):
        return data_size
    elif prim in ("all_gather", "all_to_all"):
        return data_size * num_devices


class Oracle:
    """The reference's module state (tables + args) and its functions, as one object."""

    FIELDS = ("compute_fwd_time", "compute_bwd_time", "input_size", "output_size",
              "weights", "activations", "reserved_fwd", "reserved_bwd")

    def __init__(self, settings: Settings):
        self.args = settings
        self.global_mbs_index = None
        self.op_list = None
        self.ops_not_recomputed = get_no_recompute_op_list(settings.model_name)
        self.collective_time = {}
        self.intra_band = None
        self.inter_band = None
        self.stage_memory_set = {}
        for f in self.FIELDS:
            setattr(self, f, {})

    # --- table loading -------------------------------------------------------------
    def _tp_size_list(self, model_name, model_size):
        """aceso_cost_model.py:35-45."""
        if (model_name == "gpt" and model_size == "350M") or (model_name == "t5" and model_size == "220M"):
            max_tp_size = min(self.args.max_tp, 4)
        else:
            max_tp_size = min(self.args.max_tp, 8)
        out, tp = [], 1
        while tp <= max_tp_size:
            out.append(tp)
            tp *= 2
        return out

    def _alloc(self, op_list, n_mbs, n_tp, n_algo):
        """aceso_cost_model.py:64-106."""
        for f in self.FIELDS:
            setattr(self, f, {op: [[[MISSING for _ in range(n_algo)] for _ in range(n_tp)]
                                   for _ in range(n_mbs)] for op in op_list})

    def read_op_list(self, model_name, model_size, time_path):
        """model_ops_info.py:10-28."""
        if model_name == "scale-layer":
            src = time_path + f"gpt_scale-layer_mbs{self.args.micro_batch_size[0]}_tp1_algo0.csv"
        else:
            if model_name == "t5" and model_size == "22B":
                model_size = "11B"
            src = time_path + model_name + f"_{model_size}_mbs{self.args.micro_batch_size[0]}_tp1_algo0.csv"
        op_list = []
        with open(src) as f:
            for k, row in enumerate(csv.reader(f)):
                if k > 0:
                    op_list.append(row[0])
        return op_list

    def read_profiled_time(self, model_name, model_size, time_path):
        """aceso_cost_model.py:27-183."""
        args = self.args
        mbs_list = args.micro_batch_size
        self.global_mbs_index = {mbs_list[i]: i for i in range(len(mbs_list))}
        tp_size_list = self._tp_size_list(model_name, model_size)
        comm_num_gpus_list = tp_size_list[1:]
        algo_list = [0] if model_name == "t5" else [0, 1]
        if self.op_list is None:
            self.op_list = self.read_op_list(model_name, model_size, time_path)
        if model_name == "t5" and model_size == "22B":
            model_size = "11B"
        self._alloc(self.op_list, len(mbs_list), len(tp_size_list), len(algo_list))
        for mbs in mbs_list:
            for tp in tp_size_list:
                mi = self.global_mbs_index[mbs]
                ti = int(math.log(tp, 2))
                for ai in algo_list:
                    if model_name == "scale-layer":
                        src = time_path + f"gpt_scale-layer_mbs{mbs}_tp{tp}_algo{ai}.csv"
                    else:
                        src = time_path + model_name + f"_{model_size}_mbs{mbs}_tp{tp}_algo{ai}.csv"
                    try:
                        with open(src) as f:
                            for k, row in enumerate(csv.reader(f)):
                                if k > 0:
                                    op = row[0]
                                    self.compute_fwd_time[op][mi][ti][ai] = float(row[1])
                                    self.compute_bwd_time[op][mi][ti][ai] = float(row[2])
                                    self.input_size[op][mi][ti][ai] = float(row[3])
                                    self.output_size[op][mi][ti][ai] = float(row[4])
                                    self.weights[op][mi][ti][ai] = float(row[5])
                                    self.activations[op][mi][ti][ai] = float(row[6])
                                    if args.consider_reserved_space:
                                        self.reserved_fwd[op][mi][ti][ai] = float(row[7])
                                        self.reserved_bwd[op][mi][ti][ai] = float(row[8])
                    except Exception:
                        pass  # the reference prints a warning and keeps the 1e6 defaults
        self.collective_time = {}
        if model_name in ["gpt", "scale-layer"]:
            prim_list = ["all_gather", "all_reduce", "reduce_scatter", "all_to_all"]
        elif model_name == "t5":
            prim_list = []
        else:
            prim_list = ["all_gather", "all_to_all"]
        for prim in prim_list:
            self.collective_time[prim] = {}
            for n in comm_num_gpus_list:
                self.collective_time[prim][n] = {}
                if model_name == "scale-layer":
                    src = time_path + f"prim_gpt_scale-layer_{prim}_{n}gpus.csv"
                else:
                    src = time_path + f"prim_{model_name}_{model_size}_{prim}_{n}gpus.csv"
                with open(src) as f:
                    for k, row in enumerate(csv.reader(f)):
                        if k > 0:
                            self.collective_time[prim][n][row[0]] = float(row[1])
        self.intra_band = None
        try:
            with open(time_path + "p2p_intra_node.csv") as f:
                for idx, row in enumerate(csv.reader(f)):
                    if idx == 1:
                        self.intra_band = [float(x) for x in row]
        except Exception:
            pass
        try:
            with open(time_path + "p2p_inter_node.csv") as f:
                for idx, row in enumerate(csv.reader(f)):
                    if idx == 1:
                        self.inter_band = [float(x) for x in row]
        except Exception:
            self.inter_band = self.intra_band
        return len(self.op_list)

    def load_dense(self, op_names, tables, collectives, intra_band, inter_band):
        """Same state as read_profiled_time, from in-memory data (synthetic databases).
        `tables[field]` is a nested list / array [op][mbs][tp][algo]; `collectives` is
        {prim: {num_gpus: {str_key: ms}}} with the reference's string keys."""
        mbs_list = self.args.micro_batch_size
        self.global_mbs_index = {mbs_list[i]: i for i in range(len(mbs_list))}
        self.op_list = list(op_names)
        for f in self.FIELDS:
            arr = tables[f]
            setattr(self, f, {op: [[[float(x) for x in row_t] for row_t in row_m]
                                   for row_m in arr[k]] for k, op in enumerate(op_names)})
        self.collective_time = {p: {int(n): dict(d) for n, d in v.items()}
                                for p, v in collectives.items()}
        self.intra_band = [float(x) for x in intra_band]
        self.inter_band = [float(x) for x in inter_band]

    # --- lookups ----------------------------------------------------------------------
    def get_mbs_index(self, mbs):
        """aceso_cost_model.py:22-25 (KeyError for an unprofiled micro-batch size)."""
        return self.global_mbs_index[mbs]

    def get_reshard_time(self, prim, num_devices, data_size):
        """aceso_cost_model.py:247-260."""
        assert num_devices > 1
        if prim in ["all_reduce", "all_gather", "reduce_scatter", "all_to_all"]:
            key = '{:.0f}'.format(float(data_size))
            table = self.collective_time[prim][num_devices]
            if key in table:
                return table[key]
            elif '{:.0f}'.format(float(data_size) - 1) in table:
                return table['{:.0f}'.format(float(data_size) - 1)]
            else:
                return 100000
        elif prim in ["split"]:
            return 0
        else:
            return 100000

    @staticmethod
    def _band(band, data_size):
        """aceso_cost_model.py:275-299 (shared body of intra/inter_node_band)."""
        if data_size > 0:
            index = int(math.log(data_size, 2))
            if index >= 1:
                index -= 1
            if index >= len(band):
                return band[-1] * 0.001
            else:
                return band[index] * 0.001  # negative index wraps, as in the reference
        else:
            return 1

    def intra_node_band(self, data_size):
        return self._band(self.intra_band, data_size)

    def inter_node_band(self, data_size):
        return self._band(self.inter_band, data_size)

    # --- stage time -------------------------------------------------------------------
    def get_time_v3(self, ops, mbs, tp, algo, dp, in_cross_node, out_cross_node):
        """aceso_cost_model.py:301-356."""
        if len(ops) == 0:
            return 0, 0, 0, 0, 0
        args = self.args
        fwd_comp, bwd_comp, in_comm, out_comm, tp_comm = 0, 0, 0, 0, 0
        for i in range(len(ops)):
            op_name = ops[i]
            mi = self.get_mbs_index(mbs[i])
            ti = int(math.log(tp[i], 2))
            ai = algo[i]
            fwd_comp += self.compute_fwd_time[op_name][mi][ti][ai]
            bwd_comp += self.compute_bwd_time[op_name][mi][ti][ai]
            if args.support_comm_predict:
                for suffix in ["qkv", "dense", "GEMM", "conv", "downsample"]:
                    if suffix in op_name:
                        tp_comm += self.get_reshard_time("all_reduce", tp[i], self.output_size[op_name][mi][ti][ai]) * 1000
        in_mi = self.get_mbs_index(mbs[0])
        in_ti = int(math.log(tp[0], 2))
        out_mi = self.get_mbs_index(mbs[-1])
        out_ti = int(math.log(tp[0], 2))  # sic: tp[0], not tp[-1] (aceso_cost_model.py:322)
        input_comm_size = self.input_size[ops[0]][in_mi][in_ti][algo[0]]
        output_comm_size = self.output_size[ops[-1]][out_mi][out_ti][algo[-1]]
        if in_cross_node:
            in_comm = input_comm_size / self.inter_node_band(input_comm_size)
        else:
            in_comm = input_comm_size / self.intra_node_band(input_comm_size)
        if out_cross_node:
            out_comm = output_comm_size / self.inter_node_band(output_comm_size)
        else:
            out_comm = output_comm_size / self.intra_node_band(output_comm_size)
        fwd_reshard = 0
        bwd_reshard = 0
        if args.resharding:
            for i in range(1, len(ops)):
                prev_spec = get_op_spec(ops[i - 1], tp[i - 1], dp[i - 1], algo[i - 1], input_spec=False)
                current_spec = get_op_spec(ops[i], tp[i], dp[i], algo[i], input_spec=True)
                fwd_prim, bwd_prim, num_devices = get_reshard_primitives(prev_spec, current_spec)
                mi = self.get_mbs_index(mbs[i])
                ti = int(math.log(tp[i], 2))
                if fwd_prim is not None:
                    fwd_reshard += self.get_reshard_time(fwd_prim, num_devices, self.input_size[ops[i]][mi][ti][algo[i]])
                if bwd_prim is not None:
                    bwd_reshard += self.get_reshard_time(bwd_prim, num_devices, self.input_size[ops[i]][mi][ti][algo[i]])
        in_comm += fwd_reshard * 1000
        out_comm += bwd_reshard * 1000
        tp_comm += fwd_reshard * 1000 + bwd_reshard * 1000
        return fwd_comp, bwd_comp, in_comm, out_comm, tp_comm

    def get_recompute_time_v3(self, ops, recompute_ops, mbs, tp, algo):
        """aceso_cost_model.py:358-373."""
        if len(ops) == 0 or sum(recompute_ops) == 0:
            return 0
        fwd_comp = 0
        for i in range(len(ops)):
            if recompute_ops[i] == 1:
                mi = self.get_mbs_index(mbs[i])
                ti = int(math.log(tp[i], 2))
                fwd_comp += self.compute_fwd_time[ops[i]][mi][ti][algo[i]]
        return fwd_comp

    # --- stage memory -----------------------------------------------------------------
    @staticmethod
    def _zero_act(name):
        """The 'shares its buffer' predicate of aceso_cost_model.py:388/410/433."""
        return (name in ["enc-attention-softmax", "bn1"] or "-bn3" in name or
                ("-downsample" in name and "0-0" not in name))

    @staticmethod
    def _layer_start(name):
        """aceso_cost_model.py:412/439."""
        return name in ["enc-1st-layernorm"] or "-conv1" in name

    def get_memory_v3(self, ops, mbs, tp, algo):
        """aceso_cost_model.py:375-394."""
        shared = self.args.consider_shared_space
        in_mi = self.get_mbs_index(mbs[0])
        in_ti = int(math.log(tp[0], 2))
        inputs = self.input_size[ops[0]][in_mi][in_ti][algo[0]]
        _activations = 0
        _weights = 0
        for i in range(len(ops)):
            mi = self.get_mbs_index(mbs[i])
            ti = int(math.log(tp[i], 2))
            ai = algo[i]
            if shared and ops[i] == "enc-attention-dropout":
                _activations += self.activations[ops[i]][mi][ti][ai] * 1.5
            elif shared and self._zero_act(ops[i]):
                _activations += 0
            else:
                _activations += self.activations[ops[i]][mi][ti][ai]
            _weights += self.weights[ops[i]][mi][ti][ai]
        return _weights, inputs, _activations

    def get_activations_v3(self, ops, recompute_ops, mbs, tp, algo):
        """aceso_cost_model.py:396-417."""
        if len(ops) <= 1 or sum(recompute_ops) == 0:
            return 0
        shared = self.args.consider_shared_space
        saved = 0
        for i in range(len(ops) - 1):
            if recompute_ops[i] == 1 and recompute_ops[i + 1] == 1:
                mi = self.get_mbs_index(mbs[i])
                ti = int(math.log(tp[i], 2))
                ai = algo[i]
                if shared and ops[i] == "enc-attention-dropout":
                    saved += self.activations[ops[i]][mi][ti][ai] * 1.5
                elif shared and self._zero_act(ops[i]):
                    saved += 0
                elif self._layer_start(ops[i + 1]):
                    saved += 0
                else:
                    saved += self.activations[ops[i]][mi][ti][ai]
        return saved

    def get_peak_activations(self, ops, recompute_ops, mbs, tp, algo):
        """aceso_cost_model.py:419-447."""
        if len(ops) <= 1 or sum(recompute_ops) == 0:
            return 0
        shared = self.args.consider_shared_space
        saved = 0
        saved_list = [0]
        for i in range(len(ops) - 1):
            if recompute_ops[i] == 1 and recompute_ops[i + 1] == 1:
                mi = self.get_mbs_index(mbs[i])
                ti = int(math.log(tp[i], 2))
                ai = algo[i]
                if shared and self._zero_act(ops[i]):
                    saved += 0
                elif shared and ops[i] == "enc-attention-dropout":
                    saved += self.activations[ops[i]][mi][ti][ai] * 1.5
                else:
                    saved += self.activations[ops[i]][mi][ti][ai]
                    if self._layer_start(ops[i + 1]) or i + 1 == len(ops) - 1:
                        saved_list.append(saved)
                        saved = 0
            else:
                if saved > 0:
                    saved_list.append(saved)
                    saved = 0
        return max(saved_list)

    def get_reserved_memory(self, ops, mbs, tp, dp, algo, memory_weights):
        """aceso_cost_model.py:449-485."""
        args = self.args
        cur_f = 0
        cur_b = 0
        for i in range(len(ops) - 1):
            mi = self.get_mbs_index(mbs[i])
            ti = int(math.log(tp[i], 2))
            ai = algo[i]
            if self.reserved_fwd[ops[i]][mi][ti][ai] > cur_f:
                cur_f = self.reserved_fwd[ops[i]][mi][ti][ai]
            if self.reserved_bwd[ops[i]][mi][ti][ai] > cur_b:
                cur_b = self.reserved_bwd[ops[i]][mi][ti][ai]
        max_collective = 0
        if args.consider_collective_memory:
            if args.resharding:
                for i in range(1, len(ops)):
                    prev_spec = get_op_spec(ops[i - 1], tp[i - 1], dp[i - 1], algo[i - 1], input_spec=False)
                    current_spec = get_op_spec(ops[i], tp[i], dp[i], algo[i], input_spec=True)
                    fwd_prim, bwd_prim, num_devices = get_reshard_primitives(prev_spec, current_spec)
                    mi = self.get_mbs_index(mbs[i])
                    ti = int(math.log(tp[i], 2))
                    sz = self.input_size[ops[i]][mi][ti][algo[i]]
                    if fwd_prim is not None:
                        c = get_reshard_memory(fwd_prim, num_devices, sz)
                        if c > max_collective:
                            max_collective = c
                    if bwd_prim is not None:
                        c = get_reshard_memory(bwd_prim, num_devices, sz)
                        if c > max_collective:
                            max_collective = c
        if args.memory_pred_type == "MAX":
            return max(cur_f + cur_b, memory_weights) + max_collective
        elif args.memory_pred_type == "MIN":
            return max(cur_f, cur_b, memory_weights, max_collective)
        else:
            raise RuntimeError(f"unknown args.memory_pred_type {args.memory_pred_type}")

    def get_activation_size(self, op_name, mbs, tp, algo_index=0):
        """aceso_cost_model.py:487-491."""
        return self.activations[op_name][self.get_mbs_index(mbs)][int(math.log(tp, 2))][algo_index]

    # --- single-stage API (aceso_cost_model.py:493-539) ----------------------------------
    def predict_stage_time(self, ops, recompute_ops, tp_size, dp_size, base_batch_size, algo_list,
                           delta=False, on_the_right=False, decrease=True):
        """aceso_cost_model.py:493-512."""
        mbs_list = [base_batch_size // dp_size[j] for j in range(len(ops))]
        fwd_comp, bwd_comp, in_comm, out_comm, _ = self.get_time_v3(ops, mbs_list, tp_size, algo_list, dp_size, False, False)
        recomp_time = self.get_recompute_time_v3(ops, recompute_ops, mbs_list, tp_size, algo_list)
        if not delta:
            sum_time = fwd_comp + bwd_comp + in_comm + out_comm + recomp_time
        else:
            if on_the_right and decrease:
                sum_time = fwd_comp + bwd_comp - in_comm + out_comm + recomp_time
            elif not on_the_right and decrease:
                sum_time = fwd_comp + bwd_comp + in_comm - out_comm + recomp_time
            elif on_the_right and not decrease:
                sum_time = fwd_comp + bwd_comp + in_comm - out_comm + recomp_time
            else:
                sum_time = fwd_comp + bwd_comp - in_comm + out_comm + recomp_time
        return sum_time / 1000

    def predict_stage_memory(self, ops, recompute_ops, tp_size, dp_size, base_batch_size,
                             num_stages_behind, algo_list, breakdown=False):
        """aceso_cost_model.py:514-539."""
        args = self.args
        mbs_list = [base_batch_size // dp_size[j] for j in range(len(ops))]
        memory_weights, inputs, activations = self.get_memory_v3(ops, mbs_list, tp_size, algo_list)
        memory_gradients = memory_weights
        memory_main_params = memory_weights * args.memory_main_params
        memory_optimizer = memory_weights * args.memory_optimizer
        saved_activations = self.get_activations_v3(ops, recompute_ops, mbs_list, tp_size, algo_list)
        peak_activations = self.get_peak_activations(ops, recompute_ops, mbs_list, tp_size, algo_list)
        if args.consider_reserved_space:
            memory_reserved = self.get_reserved_memory(ops, mbs_list, tp_size, dp_size, algo_list, memory_weights)
        else:
            memory_reserved = 0
        memory_activations = (inputs + activations - saved_activations) * (num_stages_behind)
        memory_peak = inputs + activations - saved_activations + peak_activations
        memory_weights += memory_main_params
        memory_sum = memory_weights + memory_gradients + memory_optimizer + memory_activations + memory_peak + memory_reserved
        if breakdown:
            return memory_weights, memory_gradients, memory_optimizer, memory_activations, memory_peak, memory_reserved
        return memory_sum

    # --- whole plan (aceso_cost_model.py:541-672) ---------------------------------------
    def predict_time_breakdown(self, config):
        """aceso_cost_model.py:541-672 (printing paths dropped); mutates `config`."""
        args = self.args
        base_batch_size = config.micro_bs
        num_batches = config.global_bs // base_batch_size
        _time_list, memory_list, compute_time_list = [], [], []
        efficiency_list, gpu_time_list = [], []
        ideal_per_gpu, eff_loss_list, recomp_list = [], [], []
        num_gpus_till_now = 0
        for i in range(config.num_stages):
            stage = config.stages[i]
            ops, num_gpus = stage.ops, stage.num_gpus
            tp_size, dp_size, algo_list = stage.tp_size, stage.dp_size, stage.algo
            recompute_ops = stage.recompute_ops
            mbs_list = [base_batch_size // dp_size[j] for j in range(len(ops))]
            in_cross_node = (num_gpus_till_now % args.num_gpus_per_node) == 0 and num_gpus_till_now > 0
            num_gpus_till_now += num_gpus
            out_cross_node = (num_gpus_till_now % args.num_gpus_per_node) == 0
            fwd_comp, bwd_comp, in_comm, out_comm, tp_comm = self.get_time_v3(
                ops, mbs_list, tp_size, algo_list, dp_size, in_cross_node, out_cross_node)
            recomp_time = self.get_recompute_time_v3(ops, recompute_ops, mbs_list, tp_size, algo_list)
            sum_time = (fwd_comp + bwd_comp + in_comm + out_comm + recomp_time) / 1000
            _time_list.append(sum_time)
            compute_time_list.append((fwd_comp + bwd_comp + recomp_time) / 1000)
            gpu_time_list.append(sum_time * num_gpus)
            _mbs_list = [base_batch_size for _ in range(len(ops))]
            _tp_size = [1 for _ in range(len(ops))]
            _dp_size = [1 for _ in range(len(ops))]
            _fwd, _bwd, _in, _out, _ = self.get_time_v3(ops, _mbs_list, _tp_size, algo_list, _dp_size,
                                                        in_cross_node, out_cross_node)
            ideal_time = (_fwd + _bwd + _in + _out) / 1000
            eff_loss_time = (fwd_comp + bwd_comp) - (_fwd + _bwd) / num_gpus
            ideal_per_gpu.append(((_fwd + _bwd) / num_gpus) / 1000)
            eff_loss_list.append(eff_loss_time / 1000)
            recomp_list.append(recomp_time / 1000)
            mw, mg, mo, ma, mp, mr = self.predict_stage_memory(
                ops, recompute_ops, tp_size, dp_size, base_batch_size, stage.num_stages_behind,
                algo_list, breakdown=True)
            memory_list.append(mw + mg + mo + ma + mp + mr)
            efficiency_list.append(ideal_time / (sum_time * num_gpus))
        sum_stage_time = sum(_time_list)
        time_list = [(_time_list[i] * (num_batches - 1) + sum_stage_time) for i in range(config.num_stages)]
        config.time_list = time_list
        config.memory_list = memory_list
        config.compute_time_list = compute_time_list
        config.total_gpu_time = sum(gpu_time_list) * (num_batches - 1)
        config.breakdown_ideal_time_per_gpu = ideal_per_gpu
        config.breakdown_eff_loss_time_per_gpu = eff_loss_list
        config.breakdown_recomp_time_per_gpu = recomp_list
        max_time = max(time_list)
        max_mem = args.memory_limit
        efficient_time_list = []
        for i in range(config.num_stages):
            used_time = time_list[i]
            used_memory = memory_list[i]
            if sum(config.stages[i].recompute_ops) > 0:
                idle_time = (max_time - used_time) / 2
            else:
                idle_under_time = max_time - used_time
                idle_under_memory = ((max_mem - used_memory) / used_memory) * used_time
                if idle_under_memory > idle_under_time:
                    idle_time = idle_under_time
                else:
                    idle_time = idle_under_memory + (idle_under_time - idle_under_memory) / 2
            efficient_time_list.append(idle_time * config.stages[i].num_gpus * efficiency_list[i])
        config.efficient_time_list = efficient_time_list

    def get_reserved_memory_list(self, config):
        """aceso_cost_model.py:674-691."""
        out = []
        if config is not None:
            for stage in config.stages:
                out.append(self.predict_stage_memory(
                    stage.ops, stage.recompute_ops, stage.tp_size, stage.dp_size, config.micro_bs,
                    stage.num_stages_behind, stage.algo, breakdown=True)[5])
        return out

    def predict_value_after_move(self, config, bottleneck, partner, num_ops_moved, metric,
                                 inc_gpus=False, dec_gpus=False, dim=None):
        """aceso_cost_model.py:693-739."""
        st = config.stages[bottleneck]
        ops, tp_size, dp_size = list(st.ops), list(st.tp_size), list(st.dp_size)
        algo_list, recompute_ops = list(st.algo), list(st.recompute_ops)
        if num_ops_moved > 0:
            if bottleneck < partner:
                ops, tp_size = ops[:-num_ops_moved], tp_size[:-num_ops_moved]
                dp_size, algo_list = dp_size[:-num_ops_moved], algo_list[:-num_ops_moved]
            else:
                ops, tp_size = ops[num_ops_moved:], tp_size[num_ops_moved:]
                dp_size, algo_list = dp_size[num_ops_moved:], algo_list[num_ops_moved:]
        if inc_gpus:
            if dim == "tp":
                tp_size = [t * 2 for t in tp_size]
            elif dim == "dp":
                dp_size = [d * 2 for d in dp_size]
        if dec_gpus:
            if dim == "tp":
                tp_size = [t // 2 for t in tp_size]
            elif dim == "dp":
                dp_size = [d // 2 for d in dp_size]
        if num_ops_moved > 0 or inc_gpus or dec_gpus:
            recompute_ops = self.check_recompute(ops, config.micro_bs, tp_size, dp_size,
                                                 st.num_stages_behind, algo_list)
        if metric in ["time", "time_with_efficiency"]:
            value = self.predict_stage_time(ops, recompute_ops, tp_size, dp_size, config.micro_bs, algo_list)
        elif metric == "memory":
            value = self.predict_stage_memory(ops, recompute_ops, tp_size, dp_size, config.micro_bs,
                                              st.num_stages_behind, algo_list)
        else:
            raise RuntimeError(f"metric {metric} not implemented.")
        return value, recompute_ops

    # --- recomputation (aceso_cost_model.py:743-883) ----------------------------------------
    def predict_stage_memory_helper(self, ops, recompute_ops, tp_size, dp_size, base_batch_size,
                                    num_stages_behind, algo_list):
        """aceso_cost_model.py:747-767 (memo keyed on the same string)."""
        key = f"ops{ops[0]}{len(ops)}tp{tp_size}dp{dp_size}rc{recompute_ops}algo{algo_list}bs{base_batch_size}stage{num_stages_behind}"
        if self.stage_memory_set.get(key) is not None:
            return self.stage_memory_set[key]
        v = self.predict_stage_memory(ops, recompute_ops, tp_size, dp_size, base_batch_size,
                                      num_stages_behind, algo_list)
        self.stage_memory_set[key] = v
        return v

    def get_next_recompute_op_group(self, ops, op_groups, exceed_memory):
        """aceso_cost_model.py:794-820."""
        max_saved_size = 0
        max_saved_op_name = None
        for op_name in op_groups:
            g = op_groups[op_name]
            if (not g["recomputed"] and g["sum_size"] > max_saved_size and
                    op_name not in ["enc-1st-layernorm"] and "-conv1" not in op_name and
                    "-relu" not in op_name and op_name not in self.ops_not_recomputed):
                max_saved_size = g["sum_size"]
                max_saved_op_name = op_name
        if max_saved_size == 0:
            return None, None
        g = op_groups[max_saved_op_name]
        g["recomputed"] = True
        next_op_index = g["index"][0] + 1
        if next_op_index >= len(ops):
            return None, None
        op_groups[ops[next_op_index]]["recomputed"] = True
        if max_saved_size < exceed_memory:
            return g["index"], g["activation_size"]
        saved_size = 0
        index = 0
        while saved_size <= exceed_memory and index < len(g["activation_size"]):
            saved_size += g["activation_size"][index]
            index += 1
        return list(g["index"][:index]), list(g["activation_size"][:index])

    def check_recompute(self, ops, base_batch_size, tp_size, dp_size, num_stages_behind, algo_list):
        """aceso_cost_model.py:822-872."""
        args = self.args
        num_ops = len(ops)
        if not args.flex_recompute:
            return [1 for _ in range(num_ops)]
        recompute_ops = [0 for _ in range(num_ops)]
        stage_memory = self.predict_stage_memory_helper(ops, recompute_ops, tp_size, dp_size,
                                                        base_batch_size, num_stages_behind, algo_list)
        stage_memory += args.peak_mem_in_backward
        if stage_memory - args.memory_limit <= 0:
            return recompute_ops
        op_groups = {}
        for index in range(len(ops)):
            if ops[index] not in op_groups:
                op_groups[ops[index]] = {"index": [], "activation_size": [], "recomputed": False, "sum_size": 0}
            g = op_groups[ops[index]]
            g["index"].append(index)
            sz = self.get_activation_size(ops[index], base_batch_size // dp_size[index], tp_size[index],
                                          algo_list[index]) * (num_stages_behind + 1)
            g["activation_size"].append(sz)
            g["sum_size"] += sz
        mbs_list = [base_batch_size // dp_size[i] for i in range(len(dp_size))]
        initial_saved = 0
        current_peak = self.get_peak_activations(ops, recompute_ops, mbs_list, tp_size, algo_list)
        while stage_memory - args.memory_limit > 0:
            idx_group, _sizes = self.get_next_recompute_op_group(ops, op_groups, stage_memory - args.memory_limit)
            if idx_group is not None:
                for k in range(len(idx_group)):
                    si = idx_group[k]
                    if si >= 0:
                        recompute_ops[si] = 1
                        if si < len(ops) - 1:
                            recompute_ops[si + 1] = 1
                    else:
                        break
            else:
                break
            new_saved = self.get_activations_v3(ops, recompute_ops, mbs_list, tp_size, algo_list)
            stage_memory -= (new_saved - initial_saved) * (num_stages_behind + 1)
            initial_saved = new_saved
            new_peak = self.get_peak_activations(ops, recompute_ops, mbs_list, tp_size, algo_list)
            stage_memory += (new_peak - current_peak)
            current_peak = new_peak
        return recompute_ops

    def update_recompute(self, config, stage_idx=None):
        """aceso_cost_model.py:874-883."""
        stages = [stage_idx] if stage_idx is not None else list(range(config.num_stages))
        for k in stages:
            st = config.stages[k]
            st.recompute_ops = self.check_recompute(st.ops, config.micro_bs, st.tp_size, st.dp_size,
                                                    st.num_stages_behind, st.algo)

    def wrap_predict_delta_time(self, config, longest_stage, shortest_stage, num_ops_moved, decrease=True):
        """aceso_cost_model.py:885-922."""
        st = config.stages[longest_stage]
        ops, recompute_ops = st.ops, st.recompute_ops
        tp_size, dp_size, algo_list = st.tp_size, st.dp_size, st.algo
        num_ops = len(ops)
        if longest_stage < shortest_stage and decrease:
            ops = ops[num_ops - num_ops_moved:]
            recompute_ops = list(recompute_ops[num_ops - num_ops_moved:])
            tp_size = tp_size[num_ops - num_ops_moved:]
            dp_size = dp_size[num_ops - num_ops_moved:]
            algo_list = algo_list[num_ops - num_ops_moved:]
        elif longest_stage > shortest_stage and decrease:
            ops = ops[0:num_ops_moved]
            recompute_ops = list(recompute_ops[0:num_ops_moved])
            tp_size = tp_size[0:num_ops_moved]
            dp_size = dp_size[0:num_ops_moved]
            algo_list = algo_list[0:num_ops_moved]
        elif longest_stage < shortest_stage and not decrease:
            ops = ops[num_ops - num_ops_moved:]
            recompute_ops = [0 for _ in range(num_ops_moved)]
            tp_size = [config.stages[longest_stage + 1].tp_size[0] for _ in range(num_ops_moved)]
            dp_size = [config.stages[longest_stage + 1].dp_size[0] for _ in range(num_ops_moved)]
            algo_list = algo_list[num_ops - num_ops_moved:]
        elif longest_stage > shortest_stage and not decrease:
            ops = ops[0:num_ops_moved]
            recompute_ops = [0 for _ in range(num_ops_moved)]
            tp_size = [config.stages[longest_stage - 1].tp_size[-1] for _ in range(num_ops_moved)]
            dp_size = [config.stages[longest_stage - 1].dp_size[-1] for _ in range(num_ops_moved)]
            algo_list = algo_list[0:num_ops_moved]
        else:
            raise RuntimeError("")
        return self.predict_stage_time(ops, recompute_ops, tp_size, dp_size, config.micro_bs, algo_list,
                                       delta=True, on_the_right=longest_stage < shortest_stage,
                                       decrease=decrease)

    # --- batch semantics used by callers (aceso_search.py:66, gen_megatron_plan.py:106-135) ---
    def score(self, config, strict=False):
        """(iteration ms, peak MB, feasible) as the callers derive them:
        max(time_list), max(memory_list), and `<=` (search) or `<` (strict) memory_limit."""
        self.predict_time_breakdown(config)
        t, m = max(config.time_list), max(config.memory_list)
        return t, m, (m < self.args.memory_limit) if strict else (m <= self.args.memory_limit)


def topk(iter_ms, feasible, k):
    """Ascending by time, stable (ties keep the lower plan index), feasible plans only:
    the order sort_configs (aceso_utils.py:723-740) and gen_megatron_plan.py:131-135 produce."""
    idx = [i for i in range(len(iter_ms)) if feasible[i]]
    idx.sort(key=lambda i: iter_ms[i])  # list.sort is stable
    return idx[:k]
