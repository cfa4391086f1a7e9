"""The search's starting plans: `generate_initial_config` of the reference (search/aceso_utils.py:537-721) with its
four built-in starting points, and the plan-file fall-through.

Host-side plan construction only (no scoring): the search scores what this returns through the cost model.  The
arguments are read from an argparse-like namespace with the reference's attribute names (`num_gpus`,
`global_batch_size`, `micro_batch_size`, `max_tp`, `flex_recompute`, `init_dim`, `model_name`, `num_layers`,
`initial_point`); the op list is passed in, since here it belongs to the loaded cost model (`CostModel.graph.ops`)
and not to a module-level singleton.

Behaviour kept as it is in the reference, including what looks accidental: a GPU count the doubling loop cannot
reach returns None (balance, imbalance_op) or raises TypeError (test: its fall-back call has the wrong number of
arguments, :594); imbalance_op sets every recompute bit when flex_recompute is ON and none when it is off (:698-701),
the opposite of balance (:567-570); imbalance_op knows only ResNet-50-shaped and GPT-shaped graphs and ends in
UnboundLocalError for any other model (:680-694); the imbalance_gpu loop walks the micro-batch sizes with an assert
(:643-645).  tests/test_initial_plans.py compares all of it with what the reference returned."""
from typing import List, Optional, Sequence

from .plan import AcesoConfig, config_from_json, get_config

INITIAL_POINTS = ("balance", "imbalance_gpu", "imbalance_op", "test")


def _double_in_turn(num_stages: int, num_gpus: int, max_tp: int) -> Optional[List[int]]:
    """One GPU per stage, then rounds over the stages from the first on, doubling a stage while it is below max_tp and
    the GPUs left cover the doubling (:543-551, :668-676).  None when the total is not reached."""
    gpus = [1] * num_stages
    progress = True
    while sum(gpus) < num_gpus and progress:
        progress = False
        for i in range(num_stages):
            left = num_gpus - sum(gpus)
            if left > 0 and gpus[i] < max_tp and gpus[i] <= left:
                gpus[i] *= 2
                progress = True
    return gpus if sum(gpus) == num_gpus else None


def _even_split(num_ops: int, num_stages: int) -> List[int]:
    """Equal op counts, the remainder to the last stage (:553-555)."""
    per = [num_ops // num_stages] * num_stages
    per[-1] += num_ops - num_stages * (num_ops // num_stages)
    return per


def _per_op(values: Sequence[int], counts: Sequence[int]) -> List[int]:
    return [v for v, n in zip(values, counts) for _ in range(n)]


def generate_balance_config(full_op_list, num_stages, args) -> Optional[AcesoConfig]:
    """aceso_utils.py:537-576."""
    gpus = _double_in_turn(num_stages, args.num_gpus, args.max_tp)
    if gpus is None:
        return None
    num_ops = len(full_op_list)
    per = _even_split(num_ops, num_stages)
    tp: List[int] = []
    dp: List[int] = []
    if args.init_dim == "tp":
        tp, dp = _per_op(gpus, per), _per_op([1] * num_stages, per)
    elif args.init_dim == "dp":
        tp, dp = _per_op([2] * num_stages, per), _per_op([g // 2 for g in gpus], per)
    recompute = [0 if args.flex_recompute else 1] * num_ops
    return get_config(per, tp, dp, recompute, args.micro_batch_size[0], args.global_batch_size, full_op_list, [0] * num_ops)


def generate_test_config(full_op_list, num_stages, args) -> AcesoConfig:
    """aceso_utils.py:578-617: GPUs handed out from the last stage backwards, op counts in proportion to them."""
    num_gpus = args.num_gpus
    gpus = [1] * num_stages
    left = num_gpus - num_stages
    while left > 0:
        before = left
        for i in reversed(range(num_stages)):
            if gpus[i] <= left and gpus[i] == min(gpus) and gpus[i] <= 4:
                left -= gpus[i]
                gpus[i] *= 2
                break
        if left == before:
            break
    if sum(gpus) != num_gpus:
        # (:594 calls generate_initial_config with three arguments; it takes two)
        raise TypeError("generate_initial_config() takes 2 positional arguments but 3 were given")
    num_ops = len(full_op_list)
    per = [int(num_ops * (g / num_gpus)) for g in gpus]
    per[-1] += num_ops - sum(per)
    return get_config(per, _per_op(gpus, per), _per_op([1] * num_stages, per), [0] * num_ops, args.micro_batch_size[0],
                      args.global_batch_size, full_op_list, [0] * num_ops)


def generate_imbalance_gpu_config(full_op_list, num_stages, args) -> AcesoConfig:
    """aceso_utils.py:619-660: even op counts; GPUs doubled from the last stage backwards as long as the micro-batch
    size per replica stays a profiled one, moving to the next micro-batch size when no stage can take more."""
    micro_sizes = list(args.micro_batch_size)
    micro_bs = micro_sizes[0]
    num_ops = len(full_op_list)
    per = _even_split(num_ops, num_stages)
    gpus = [1] * num_stages
    left = args.num_gpus - num_stages
    which = 0
    while left > 0:
        found = False
        for i in reversed(range(num_stages)):
            replicas = gpus[i] * 2 // args.max_tp
            if gpus[i] <= left and (replicas == 0 or micro_bs // replicas in micro_sizes):
                left -= gpus[i]
                gpus[i] *= 2
                found = True
                break
        if not found:
            which += 1
            assert which < len(micro_sizes)
            micro_bs = micro_sizes[which]
    tp = [g if g <= args.max_tp else args.max_tp for g in gpus]
    dp = [1 if g <= args.max_tp else g // args.max_tp for g in gpus]
    return get_config(per, _per_op(tp, per), _per_op(dp, per), [0] * num_ops, micro_bs, args.global_batch_size,
                      full_op_list, [0] * num_ops)


def generate_imbalance_op_config(full_op_list, num_stages, args) -> Optional[AcesoConfig]:
    """aceso_utils.py:662-708: one layer per stage and all the others in one stage (the first for ResNet, the last
    for GPT)."""
    gpus = _double_in_turn(num_stages, args.num_gpus, args.max_tp)
    if gpus is None:
        return None
    num_ops = len(full_op_list)
    layers = [1] * num_stages
    if args.model_name == "resnet":
        layers[0] += 33 - num_stages
        per = [n * 8 for n in layers]
        per[0] += 4
        per[-1] += 2
    elif args.model_name in ("gpt", "scale-layer"):
        layers[-1] += args.num_layers - num_stages
        per = [n * 13 for n in layers]
        per[0] += 1
        per[-1] += 2
    else:
        raise UnboundLocalError("local variable 'num_ops_per_stage' referenced before assignment")
    recompute = [1 if args.flex_recompute else 0] * num_ops
    return get_config(per, _per_op(gpus, per), _per_op([1] * num_stages, per), recompute, args.micro_batch_size[0],
                      args.global_batch_size, full_op_list, [0] * num_ops)


def generate_initial_config(num_stages, args, full_op_list) -> Optional[AcesoConfig]:
    """aceso_utils.py:710-721; `args.initial_point` that names none of the built-in starting points is the path of a
    plan file (read_config_from_json, :213-242)."""
    point = args.initial_point
    if point == "balance":
        return generate_balance_config(full_op_list, num_stages, args)
    if point == "imbalance_gpu":
        return generate_imbalance_gpu_config(full_op_list, num_stages, args)
    if point == "imbalance_op":
        return generate_imbalance_op_config(full_op_list, num_stages, args)
    if point == "test":
        return generate_test_config(full_op_list, num_stages, args)
    return config_from_json(point, full_op_list)
