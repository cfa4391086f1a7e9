"""What the reference's search reports about the plans it found: the one-line plan summary it logs and keeps as a
plan's history, the per-stage-count result block with its CSV files, and the final ranking of the stage counts with the
copies of the best plan files (search/aceso_utils.py:776-829, :254-260, :852-927).

Host-side formatting and file output only; the figures come from the cost model (`time_list`, `memory_list` of a scored
plan, `CostModel.get_reserved_memory_list`).  The ranking across stage counts is the reference's stable insertion on
strict "<" (:866-877): of two stage counts with the same iteration time the one met first stays ahead.  The arguments
are read from an argparse-like namespace with the reference's attribute names.  tests/test_search_report.py compares
printed text and written files with what the reference printed and wrote."""
import csv
import os
import shutil
from typing import Dict, List, Optional, Sequence

from .plan import config_details, save_config_info_to_csv

MAX_VALUE = 2 ** 30          # aceso_utils.py:16


def format_size_list(size_list: Sequence[Sequence[int]]) -> str:
    """aceso_utils.py:776-786: one entry per stage, "v" where the stage's ops agree and "min~max" where not; every entry
    is followed by ", ", the last one too."""
    parts = []
    for sizes in size_list:
        lo, hi = min(sizes), max(sizes)
        parts.append(f"{hi}, " if lo == hi else f"{lo}~{hi}, ")
    return "[" + "".join(parts) + "]"


def plan_summary(config, info: str = "") -> str:
    """The line of aceso_utils.py:802-803 for a scored plan."""
    num_ops, tp, dp, recompute, micro_bs, algo = config_details(config)
    stages = config.stages[:config.num_stages]
    return ("{}|{:.2f}|{:.2f}| op = {}| tp = {} | dp = {} | algo = {} | rc = {} | gpus = {} | micro_bs = {} | time = {} "
            "| memory = {}").format(info, max(config.time_list), max(config.memory_list), num_ops, format_size_list(tp),
                                    format_size_list(dp), format_size_list(algo), [sum(r) for r in recompute],
                                    [st.num_gpus for st in stages], micro_bs, [int(t) for t in config.time_list],
                                    [int(m) for m in config.memory_list])


def print_simple_config_info(config, info="", add_history=False, print_recompute_ops=False, print_debug_info=False):
    """aceso_utils.py:788-829."""
    if config is None:
        return
    line = plan_summary(config, info)
    if print_debug_info:
        print(line)
    if add_history:
        config.history += line + "\n"
    if not print_recompute_ops:
        return
    stages = config.stages[:config.num_stages]
    for i, st in enumerate(stages):
        chosen = [j for j, bit in enumerate(st.recompute_ops) if bit == 1]
        print(f"[stage {i} recompute_ops] " + "".join(f"{j}," for j in chosen))
        print(f"stage {i}: " + "".join(st.ops[j] + ", " for j in chosen))
    for i, st in enumerate(stages):
        print(f"[stage {i} algo1] " + "".join(f"[{j}] {st.ops[j]} " for j, a in enumerate(st.algo) if a == 1))


def _write_rows(file_name: str, rows) -> None:
    with open(file_name, "w", newline="") as f:
        csv.writer(f).writerows(rows)


def save_distribution_to_csv(num_targets_list: List[int], num_hops_list: List[int], file_name: str) -> None:
    """aceso_utils.py:254-260."""
    _write_rows(file_name, [["num_targets"] + list(num_targets_list), ["num_hops"] + list(num_hops_list)])


def save_search_trend_in_csv(search_time_list: List[float], exec_time_list: List[float], file_name: str) -> None:
    """aceso_utils.py:852-861."""
    assert len(search_time_list) == len(exec_time_list)
    _write_rows(file_name, [["search_time (s)", "config time (ms)"]] + [list(p) for p in zip(search_time_list, exec_time_list)])


def accumulated_search_seconds(search_time_list: Sequence[float]) -> List[int]:
    """The time axis of the trend file (aceso_utils.py:913-921): 0 for the first trial, then the running sum of each
    later trial's time rounded up to whole seconds as int(t + 1); the first trial's own time is not counted."""
    out, total = [], 0
    for i, t in enumerate(search_time_list):
        if i:
            total += int(t + 1)
        out.append(total)
    return out


def print_search_details(config, args, num_stages, num_targets_list, num_hops_list, search_time_list, config_time_list,
                         reserved_mem_list, num_explored_cases) -> None:
    """aceso_utils.py:900-925: the result block of one stage count, the plan's per-stage CSV, the distribution of targets
    and hops, and the trend of the best time over the trials."""
    print(f"\n========== Best Result (num_stages = {num_stages}) ==========")
    if config is not None:
        print_simple_config_info(config, print_recompute_ops=args.print_recompute_ops, print_debug_info=True)
        print(config.history)
        print(f"num_targets: {num_targets_list}")
        print(f"num_hops: {num_hops_list}")
        stem = f"{args.model_name}_{args.model_size}_{config.num_stages}stages_{args.config_suffix}.csv"
        save_config_info_to_csv(config, reserved_mem_list, f"{args.config_save_path}csv/info_{stem}")
        save_distribution_to_csv(num_targets_list, num_hops_list, f"{args.log_path}trends/distribution_{stem}")
    else:
        print("No feasible solution.")
    accum = accumulated_search_seconds(search_time_list)
    print(f"search time = {sum(search_time_list):.2f} s.  {accum} \nnum_explored_cases = {num_explored_cases}")
    print(f"time trend: {list(map(int, config_time_list))}\n")
    save_search_trend_in_csv(accum, config_time_list,
                             f"{args.log_path}trends/{args.model_name}_{args.model_size}_{num_stages}stages_init_"
                             f"{args.initial_point}_{args.max_num_hops}hops_{args.config_suffix}.csv")


def rank_stage_counts(result_dict: Dict[int, Optional[tuple]], start_num_stages: int, end_num_stages: int) -> List[int]:
    """The stage counts with a result, best iteration time first (aceso_utils.py:865-879): counts are met in ascending
    order and put before the first kept one that is strictly slower, so equal times keep the order they were met in;
    a result whose time is not positive, or not below MAX_VALUE, is left out."""
    times: List[float] = []
    counts: List[int] = []
    for i in range(start_num_stages, end_num_stages + 1):
        r = result_dict.get(i)
        if r is None:
            continue
        t = r[0]
        if not t > 0:
            continue
        for j, kept in enumerate(times + [MAX_VALUE]):
            if t < kept:
                times.insert(j, t)
                counts.insert(j, i)
                break
    return counts


def save_and_print_top_configs(result_dict, args) -> None:
    """aceso_utils.py:863-898: copy the plan files of the best stage counts into top_configs/ and print the table.
    result_dict: {num_stages: (time ms, memory MB, explored cases, search time, case distribution) or None}."""
    ranked = rank_stage_counts(result_dict, args.start_num_stages, args.end_num_stages)
    keep = min(args.end_num_stages - args.start_num_stages + 1, args.num_of_saved_configs, len(ranked))
    rows = []
    for stage_num in ranked[:keep]:
        name = f"{args.model_name}_{args.model_size}_{stage_num}stages_{args.config_suffix}.json"
        src = f"{args.config_save_path}{name}"
        if os.path.exists(src):
            shutil.copy(src, f"{args.config_save_path}top_configs/{name}")
        t, mem, explored = result_dict[stage_num][:3]
        rows.append([stage_num, f"{t / 1000:.2f}", f"{args.global_batch_size / (t / 1000):.2f}", f"{mem:.0f}", f"{explored}"])
    header = ["# of stages", "est_iteration_time(s)", "est_thpt(samples/s)", "est_mem(MB)", "# of explored cases"]
    widths = [len(h) for h in header]
    print("\t".join(f"{h:<{w}}" for h, w in zip(header, widths)))
    for row in rows:
        print("\t".join(f"{v:<{w}}" for v, w in zip(row, widths)))
