"""GPU-backed stand-in for the reference's search/aceso_cost_model.py.

Same function names, argument meaning and error behaviour as the module that
search/aceso_search.py:4, search/aceso_prims.py:7 and search/gen_megatron_plan.py:8 import,
so the search loop, the policy and the move primitives keep running unchanged on the host
while every number comes from the HIP kernels (libace_eval.so through `PlanEvaluator`).
There is no CPU scoring path in this module: without the library or a GPU it raises.

What stays on the host, on purpose:
  * control flow of the greedy recompute pass (check_recompute, aceso_cost_model.py:794-872),
    which asks the GPU for the stage's memory / saved / peak activations at every step;
  * the float compositions the reference performs on per-stage values (time breakdown lists,
    delta-time sign variants, memory breakdown tuple): they are evaluated here with Python
    floats from the per-stage records the kernel writes, i.e. the same IEEE operations in
    the same order as the reference.

New, batched entry points (no reference counterpart): predict_time_breakdown_batch(),
score_batch(), top_k().

Module-level use mirrors the reference: `configure(args)` once (the reference evaluates its
argparse singleton at import, aceso_cost_model.py:10), `read_profiled_time(...)`, then the
functions below.
"""
import math
from typing import List, Optional, Sequence

import numpy as np

from . import opgraph as og
from .plan import AcesoConfig, AcesoStageInfo, PlanBatch, get_config  # noqa: F401 (re-exported)
from .profile_db import CostModelSettings, ProfileDB
from .tables import (MAX_STAGES, R_ACT, R_BWD, R_FWD, R_IDEAL_BWD, R_IDEAL_FWD, R_IDEAL_IN, R_IDEAL_OUT, R_IN_COMM,
                     R_INPUTS, R_OUT_COMM, R_PEAK, R_RECOMP, R_RESERVED, R_SAVED, R_RESHARD, R_STAGE_MB, R_STAGE_MS,
                     R_WEIGHTS, STAGE_REC, CompiledTables, compile_tables)


def settings_from_args(args) -> CostModelSettings:
    """The reference's argparse namespace (aceso_utils.py:455-531) -> CostModelSettings."""
    gpn = args.num_gpus_per_node
    return CostModelSettings(
        model_name=args.model_name, micro_batch_size=list(args.micro_batch_size), num_gpus_per_node=gpn,
        global_batch_size=args.global_batch_size if getattr(args, "global_batch_size", None) else 1024,
        memory_limit=float(getattr(args, "memory_limit", 28000)), max_tp=getattr(args, "max_tp", None) or gpn,
        consider_shared_space=getattr(args, "consider_shared_space", True),
        consider_reserved_space=getattr(args, "consider_reserved_space", True),
        flex_recompute=getattr(args, "flex_recompute", True),
        peak_mem_in_backward=getattr(args, "peak_mem_in_backward", 0),
        memory_pred_type=getattr(args, "memory_pred_type", "MAX"),
        resharding=getattr(args, "resharding", None),
        consider_collective_memory=bool(getattr(args, "consider_collective_memory", False)))


class CostModel:
    """One profile database + op graph + settings, scored on one GPU."""

    def __init__(self, settings: CostModelSettings, db: ProfileDB, graph: og.OpGraph, device="cuda:0"):
        self.settings = settings
        self.db = db
        self.graph = graph
        self.tables: CompiledTables = compile_tables(graph, db, settings)
        self.device = device
        self._evaluator = None        # created on first use: HIP must be initialised after any fork()
        # check_recompute starts from the reference's memo table (see check_recompute_batch); False: always from the
        # stage's own memory
        self.reference_memo = True
        self._record_cache = {}       # single-stage records by (first op, micro-batch index, stage size, code bytes)
        self._record_cache_max = 8192 # emptied when it has grown beyond this many records
        # predict_value_after_move: how many op counts a scan over them may be evaluated ahead (0: never); the scans seen
        # lately with their evaluated-ahead results
        self.look_ahead = 32
        self._scans = {}
        self.scan_ahead_used, self.scan_ahead_evaluated, self.scan_ahead_dropped = 0, 0, 0
        self._tp_lut = np.zeros(max(db.tp_list) + 1, dtype=np.uint8)      # tp size -> its index in the database
        self._tp_lut[np.asarray(db.tp_list)] = np.arange(len(db.tp_list), dtype=np.uint8)
        self._mbs_index = {m: k for k, m in enumerate(db.mbs_list)}
        self._type_index = {n: k for k, n in enumerate(db.op_names)}
        self._first_pos = {}
        for i, name in enumerate(graph.ops):
            self._first_pos.setdefault(name, []).append(i)
        self._slice_cache = {}
        self._op_types = np.asarray([self._type_index[name] for name in graph.ops], dtype=np.int64)
        # memo caches with the reference's keys and hit counters (aceso_cost_model.py:743-791)
        self.stage_memory_set, self.stage_memory_visit, self.stage_memory_hit = {}, 0, 0
        self.stage_time_set, self.stage_time_visit, self.stage_time_hit = {}, 0, 0

    @classmethod
    def from_directory(cls, args_or_settings, model_name, model_size, time_path, num_layers=None, device="cuda:0"):
        st = args_or_settings if isinstance(args_or_settings, CostModelSettings) else settings_from_args(args_or_settings)
        db = ProfileDB.from_directory(model_name, model_size, time_path, st, verbose=True)
        if num_layers is None:
            num_layers = getattr(args_or_settings, "num_layers", None)
        graph = og.OpGraph.build("gpt" if model_name == "scale-layer" else model_name, db.op_names, num_layers)
        return cls(st, db, graph, device)

    @property
    def evaluator(self):
        if self._evaluator is None:
            from .evaluator import PlanEvaluator
            self._evaluator = PlanEvaluator(self.tables, self.device)
        return self._evaluator

    def close(self):
        if self._evaluator is not None:
            self._evaluator.close()
            self._evaluator = None

    # ---- batched scoring ------------------------------------------------------------------------
    def encode(self, configs: Sequence) -> PlanBatch:
        return PlanBatch.from_configs(configs, self.tables)

    def score_batch(self, plans, memory_limit: Optional[float] = None, strict: bool = False):
        """(iter_ms, peak_mb, feasible) numpy arrays for a PlanBatch or a list of configs."""
        batch = plans if isinstance(plans, PlanBatch) else self.encode(plans)
        it, pk, fe, st = self.evaluator.score_host(batch, memory_limit, strict)
        self._raise_for_status(st)
        return it, pk, fe

    def top_k(self, plans, k: int, memory_limit: Optional[float] = None, strict: bool = False):
        """Indices and times of the k fastest feasible plans (ascending, ties -> lower index)."""
        batch = plans if isinstance(plans, PlanBatch) else self.encode(plans)
        ev = self.evaluator
        d = ev.upload(batch)
        it, pk, fe, st = ev.score(d, memory_limit, strict)
        idx, val, cnt = ev.topk(it, fe, k)
        n = int(cnt.item())
        return idx[:n].cpu().numpy(), val[:n].cpu().numpy()

    @staticmethod
    def _raise_for_status(status):
        bad = np.flatnonzero(status)
        if len(bad):
            p = int(bad[0])
            if int(status[p]) == 1:
                raise KeyError(f"plan {p}: a micro-batch size, collective or spec pairing is outside the profile "
                               "database (the reference raises KeyError / TypeError here)")
            raise ValueError(f"plan {p}: malformed encoding")

    def predict_time_breakdown_batch(self, configs: Sequence) -> None:
        """predict_time_breakdown for many plans with one kernel launch; fills the same attributes."""
        if not configs:
            return
        batch = self.encode(configs)
        it, pk, fe, st, rec = self.evaluator.score_host(batch, breakdown=True)
        self._raise_for_status(st)
        for p, cfg in enumerate(configs):
            self._fill_breakdown(cfg, rec[p])

    def _fill_breakdown(self, config, rec, print_time=False, print_memory=False):
        """aceso_cost_model.py:541-672 from the kernel's per-stage records."""
        args = self.settings
        num_batches = config.global_bs // config.micro_bs
        _time_list, memory_list, compute_time_list, efficiency_list, gpu_time_list = [], [], [], [], []
        ideal_per_gpu, eff_loss_list, recomp_list = [], [], []
        time_strings, memory_strings = [], []
        for i in range(config.num_stages):
            r = rec[i].tolist()
            num_gpus = config.stages[i].num_gpus
            fwd, bwd, in_comm, out_comm, recomp = r[R_FWD], r[R_BWD], r[R_IN_COMM], r[R_OUT_COMM], r[R_RECOMP]
            sum_time = (fwd + bwd + in_comm + out_comm + recomp) / 1000
            _time_list.append(sum_time)
            compute_time_list.append((fwd + bwd + recomp) / 1000)
            gpu_time_list.append(sum_time * num_gpus)
            _fwd, _bwd, _in, _out = r[R_IDEAL_FWD], r[R_IDEAL_BWD], r[R_IDEAL_IN], r[R_IDEAL_OUT]
            ideal_time = (_fwd + _bwd + _in + _out) / 1000
            eff_loss_time = (fwd + bwd) - (_fwd + _bwd) / num_gpus
            ideal_per_gpu.append(((_fwd + _bwd) / num_gpus) / 1000)
            eff_loss_list.append(eff_loss_time / 1000)
            recomp_list.append(recomp / 1000)
            mw, mg, mo, ma, mp, mr = self._memory_breakdown(r, config.stages[i].num_stages_behind)
            memory_sum = mw + mg + mo + ma + mp + mr
            memory_list.append(memory_sum)
            efficiency_list.append(ideal_time / (sum_time * num_gpus))
            if print_time:
                time_strings.append("[stage {}], {:.2f}, {:.2f}, {:.2f}, {:.2f}, {:.2f}, {:.2f}, ".format(
                    i, fwd / 1000 * num_batches, (bwd + recomp) / 1000 * num_batches, recomp / 1000 * num_batches,
                    in_comm / 1000 * num_batches, out_comm / 1000 * num_batches, r[R_RESHARD] / 1000 * num_batches))
            if print_memory:
                memory_strings.append(f"[stage {i}] memory = {memory_sum:.2f} MB. weights = {mw:.0f}, gradients = {mg:.0f}, "
                                      f"optimizer = {mo:.0f}, activations = {ma:.0f}, peak += {mp:.0f}, "
                                      f"memory_reserved = {mr:.0f}")
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
            used_time, used_memory = time_list[i], memory_list[i]
            if sum(config.stages[i].recompute_ops) > 0:
                idle_time = (max_time - used_time) / 2
            else:
                under_time = max_time - used_time
                under_memory = ((max_mem - used_memory) / used_memory) * used_time
                idle_time = under_time if under_memory > under_time else under_memory + (under_time - under_memory) / 2
            efficient_time_list.append(idle_time * config.stages[i].num_gpus * efficiency_list[i])
        config.efficient_time_list = efficient_time_list
        if print_time:
            b = max(range(config.num_stages), key=lambda k: (time_list[k], -k))
            print("overall time = {:.2f} ms".format(max_time))
            print("stage, fwd_comp, bwd_comp+recomp, recomp, in_comm(+reshard), out_comm(+reshard), reshard, sum(us)")
            for i in range(config.num_stages):
                print((" * " if i == b else "") + time_strings[i] + f"{time_list[i]:.2f}")
        if print_memory:
            b = max(range(config.num_stages), key=lambda k: (memory_list[k], -k))
            print("\nmax allocated memory = {:.2f} MB".format(max(memory_list)))
            for i in range(config.num_stages):
                print((" * " if i == b else "") + memory_strings[i])
            print(" ")

    def _memory_breakdown(self, r, num_stages_behind):
        """The 6-tuple of predict_stage_memory(breakdown=True) (aceso_cost_model.py:517-537)."""
        args = self.settings
        memory_weights = r[R_WEIGHTS]
        memory_gradients = memory_weights
        memory_main_params = memory_weights * args.memory_main_params
        memory_optimizer = memory_weights * args.memory_optimizer
        inputs, activations, saved, peak = r[R_INPUTS], r[R_ACT], r[R_SAVED], r[R_PEAK]
        memory_reserved = r[R_RESERVED] if args.consider_reserved_space else 0
        memory_activations = (inputs + activations - saved) * (num_stages_behind)
        memory_peak = inputs + activations - saved + peak
        memory_weights += memory_main_params
        return memory_weights, memory_gradients, memory_optimizer, memory_activations, memory_peak, memory_reserved

    # ---- the reference's function set --------------------------------------------------------------
    def predict_time_breakdown(self, config, print_time=False, print_memory=False):
        """aceso_cost_model.py:541: writes time_list, memory_list, ... onto `config`."""
        batch = self.encode([config])
        it, pk, fe, st, rec = self.evaluator.score_host(batch, breakdown=True)
        self._raise_for_status(st)
        self._fill_breakdown(config, rec[0], print_time, print_memory)

    def _locate(self, ops: Sequence[str]) -> int:
        """First position at which `ops` occurs as a contiguous slice of the model's op sequence."""
        n = len(ops)
        key = (ops[0], n, ops[-1])
        lo = self._slice_cache.get(key)
        full = self.graph.ops
        if lo is not None and full[lo:lo + n] == list(ops):
            return lo
        for lo in self._first_pos.get(ops[0], ()):
            if lo + n <= len(full) and full[lo:lo + n] == list(ops):
                self._slice_cache[key] = lo
                return lo
        raise ValueError("the op list is not a contiguous slice of the model's op sequence")

    def _stage_records(self, queries) -> np.ndarray:
        """One GPU launch for single-stage queries [(ops, recompute_ops, tp, dp, micro_bs, num_stages_behind, algo)];
        returns the stage records [len(queries), STAGE_REC].  Cross-node flags are off, as in
        predict_stage_time (aceso_cost_model.py:494-495).

        Records already computed for the same stage (same op range, per-op lists and micro-batch size) are reused: the
        search asks about the stage it has just run check_recompute on, and about the same stages again and again.  The
        table is keyed by the query's lists as bytes, so a query that is in it costs no encoding either.  The number of
        stages behind is not part of the key: it enters only the record's total-memory field, which nothing on the host
        reads (cleared below where it would be another stage count's)."""
        P = len(queries)
        cache = self._record_cache
        if len(cache) > self._record_cache_max:
            cache.clear()            # (before the look-ups below: what this call hits must still be there when it is read)
        keys, los, todo, first = [], [], [], {}
        for p, (ops, rc, tp, dp, micro_bs, nsb, algo) in enumerate(queries):
            n = len(ops)
            if n == 0:
                raise ValueError("empty stage")
            if not 0 <= nsb < MAX_STAGES:
                raise ValueError("num_stages_behind outside 0..15")
            lo = self._locate(ops)
            try:
                key = (lo, n, micro_bs, bytes(tp), bytes(dp), bytes(algo), bytes(rc))
            except (ValueError, TypeError):          # an entry that is no small integer: evaluated, not kept
                key = ("unkeyed", p)
            keys.append(key)
            los.append(lo)
            if key not in cache and key not in first:        # (equal queries inside one call are evaluated once)
                first[key] = p
                todo.append(p)
        if todo:
            codes, hdr, ranges = self._encode_stage_queries([queries[p] for p in todo], [los[p] for p in todo])
            it, pk, fe, st, rec = self.evaluator.score_host(PlanBatch(codes, hdr), breakdown=True, ranges=ranges)
            self._raise_for_status(st)
            for j, p in enumerate(todo):
                cache[keys[p]] = (rec[j, 0, :].copy(), queries[p][5] + 1)
        out = np.empty((P, STAGE_REC), dtype=np.float64)
        for p in range(P):
            r, stages = cache[keys[p]]
            out[p] = r
            if stages != queries[p][5] + 1:
                out[p, R_STAGE_MB] = math.nan
        for key in first:
            if key[0] == "unkeyed":
                del cache[key]
        return out

    def _encode_stage_queries(self, queries, los):
        """Codes, headers and op ranges of single-stage queries as the ranged kernel reads them; `los`: where each
        query's op list starts in the model's op sequence."""
        N, A = self.graph.num_ops, self.db.n_algo
        tp_index = {t: k for k, t in enumerate(self.db.tp_list)}
        P = len(queries)
        codes = np.zeros((P, N), dtype=np.uint8)
        hdr = np.zeros((P, 4), dtype=np.uint32)
        ranges = np.zeros((P, 2), dtype=np.uint32)
        # (the queries of one call are mostly one stage under different recompute lists: its tp / dp / algo lists are
        # checked and encoded once)
        shared = {}
        for p, (ops, rc, tp, dp, micro_bs, nsb, algo) in enumerate(queries):
            n, lo = len(ops), los[p]
            who = (id(ops), id(tp), id(dp), id(algo), micro_bs)
            if who not in shared:
                dp_a = np.asarray(dp, dtype=np.int64)
                tp_a = np.asarray(tp, dtype=np.int64)
                for d in set(dp_a.tolist()):
                    self._mbs_index[micro_bs // d]          # KeyError like aceso_cost_model.py:22-25
                g = int(tp_a[0] * dp_a[0])
                if g & (g - 1) or (tp_a * dp_a != g).any():
                    raise ValueError("a stage's tp*dp must be one power of two")
                for x in set(tp_a.tolist()):
                    tp_index[x]                              # KeyError for a tp size that was not profiled
                t = self._tp_lut[tp_a]
                shared[who] = (g, t * A + np.asarray(algo, dtype=np.uint8))
            g, base = shared[who]
            bidx = self._mbs_index[micro_bs]
            if isinstance(rc, (bytes, bytearray)):           # (check_recompute_batch's own trial states)
                r = (np.frombuffer(rc, dtype=np.uint8) == 1).astype(np.uint8)
            else:
                r = (np.asarray(rc) == 1).astype(np.uint8)
            codes[p, lo:lo + n] = base | (r << 3)
            codes[p, lo] |= 1 << 4
            hdr[p, 0] = (nsb + 1) | (bidx << 8)
            hdr[p, 1] = g.bit_length() - 1
            ranges[p] = (lo, lo + n)
        return codes, hdr, ranges

    def predict_stage_time(self, ops, recompute_ops, tp_size, dp_size, base_batch_size, algo_list,
                           delta=False, on_the_right=False, decrease=True):
        """aceso_cost_model.py:493-512 (ms; cross-node bandwidth never used here)."""
        if len(ops) == 0:
            return 0 / 1000
        r = self._stage_records([(ops, recompute_ops, tp_size, dp_size, base_batch_size, 0, algo_list)])[0].tolist()
        return self._stage_time_of(r, delta, on_the_right, decrease)

    @staticmethod
    def _stage_time_of(r, delta=False, on_the_right=False, decrease=True):
        """The sum of aceso_cost_model.py:505-512 over one stage record."""
        fwd_comp, bwd_comp, in_comm, out_comm, recomp_time = r[R_FWD], r[R_BWD], r[R_IN_COMM], r[R_OUT_COMM], r[R_RECOMP]
        if not delta:
            sum_time = fwd_comp + bwd_comp + in_comm + out_comm + recomp_time
        elif on_the_right == decrease:
            sum_time = fwd_comp + bwd_comp - in_comm + out_comm + recomp_time
        else:
            sum_time = fwd_comp + bwd_comp + in_comm - out_comm + recomp_time
        return sum_time / 1000

    def predict_stage_memory(self, ops, recompute_ops, tp_size, dp_size, base_batch_size, num_stages_behind,
                             algo_list, breakdown=False):
        """aceso_cost_model.py:514-539 (MB)."""
        r = self._stage_records([(ops, recompute_ops, tp_size, dp_size, base_batch_size, num_stages_behind, algo_list)])[0].tolist()
        mw, mg, mo, ma, mp, mr = self._memory_breakdown(r, num_stages_behind)
        if breakdown:
            return mw, mg, mo, ma, mp, mr
        return mw + mg + mo + ma + mp + mr

    def get_reserved_memory_list(self, config):
        """aceso_cost_model.py:674-691."""
        if config is None:
            return []
        qs = [(st.ops, st.recompute_ops, st.tp_size, st.dp_size, config.micro_bs, st.num_stages_behind, st.algo)
              for st in config.stages]
        rec = self._stage_records(qs)
        return [float(rec[i, R_RESERVED]) if self.settings.consider_reserved_space else 0 for i in range(len(qs))]

    def get_activation_size(self, op_name, mbs, tp, algo_index=0):
        """aceso_cost_model.py:487-491: one raw table entry."""
        return float(self.db.tables["activations"][self._type_index[op_name], self._mbs_index[mbs],
                                                    int(math.log(tp, 2)), algo_index])

    def _activation_sizes(self, ops, micro_bs, tp_size, dp_size, algo_list, factor):
        """[get_activation_size(ops[i], micro_bs // dp_size[i], tp_size[i], algo_list[i]) * factor for every i], as Python
        floats (the same table entries and the same product, taken with one indexing operation)."""
        n = len(ops)
        try:
            lo = self._locate(ops)
            types = self._op_types[lo:lo + n]
        except ValueError:                      # not a slice of the model's op sequence: by name
            types = np.fromiter((self._type_index[name] for name in ops), dtype=np.int64, count=n)
        def mapped(values, fn):
            # fn over a list with few distinct values
            a = np.asarray(values, dtype=np.int64)
            distinct = np.unique(a)
            return np.asarray([fn(int(v)) for v in distinct], dtype=np.int64)[np.searchsorted(distinct, a)]

        mbs = mapped(dp_size, lambda d: self._mbs_index[micro_bs // d])
        tps = mapped(tp_size, lambda t: int(math.log(t, 2)))
        algos = np.asarray(algo_list, dtype=np.int64)
        return (self.db.tables["activations"][types, mbs, tps, algos] * float(factor)).tolist()

    def predict_stage_memory_helper(self, config, stage_index, ops=None, recompute_ops=None, tp_size=None,
                                    dp_size=None, base_batch_size=None, num_stages_behind=None, algo_list=None):
        """aceso_cost_model.py:747-767 (memo with the reference's key)."""
        if ops is None:
            st = config.stages[stage_index]
            ops, recompute_ops, tp_size, dp_size = st.ops, st.recompute_ops, st.tp_size, st.dp_size
            base_batch_size = getattr(st, "base_bs", config.micro_bs)
            algo_list, num_stages_behind = st.algo, st.num_stages_behind
        key = f"ops{ops[0]}{len(ops)}tp{tp_size}dp{dp_size}rc{recompute_ops}algo{algo_list}bs{base_batch_size}stage{num_stages_behind}"
        self.stage_memory_visit += 1
        if self.stage_memory_set.get(key) is not None:
            self.stage_memory_hit += 1
            return self.stage_memory_set[key]
        v = self.predict_stage_memory(ops, recompute_ops, tp_size, dp_size, base_batch_size, num_stages_behind, algo_list)
        self.stage_memory_set[key] = v
        return v

    def clear_memo(self):
        """Empties the two memo tables and their counters (the reference keeps them for the life of its process,
        aceso_cost_model.py:743-791; a host that runs many searches in one process clears them in between)."""
        self.stage_memory_set, self.stage_memory_visit, self.stage_memory_hit = {}, 0, 0
        self.stage_time_set, self.stage_time_visit, self.stage_time_hit = {}, 0, 0

    def predict_stage_time_helper(self, config, stage_index):
        """aceso_cost_model.py:773-791."""
        st = config.stages[stage_index]
        key = f"ops{st.ops[0]}{len(st.ops)}tp{st.tp_size}dp{st.dp_size}rc{st.recompute_ops}algo{st.algo}bs{config.micro_bs}"
        self.stage_time_visit += 1
        if self.stage_time_set.get(key) is not None:
            self.stage_time_hit += 1
            return self.stage_time_set[key]
        v = self.predict_stage_time(st.ops, st.recompute_ops, st.tp_size, st.dp_size, config.micro_bs, st.algo)
        self.stage_time_set[key] = v
        return v

    def _next_recompute_op_group(self, ops, op_groups, exceed_memory):
        """aceso_cost_model.py:794-820."""
        best_size, best_name = 0, None
        flags = self.graph.flags
        for name, g in op_groups.items():
            if (not g["recomputed"] and g["sum_size"] > best_size and
                    not (int(flags[self._type_index[name]]) & og.F_NO_RECOMPUTE)):
                best_size, best_name = g["sum_size"], name
        if best_size == 0:
            return None, None
        g = op_groups[best_name]
        g["recomputed"] = True
        nxt = g["index"][0] + 1
        if nxt >= len(ops):
            return None, None
        op_groups[ops[nxt]]["recomputed"] = True
        if best_size < exceed_memory:
            return g["index"], g["activation_size"]
        saved_size, index = 0, 0
        while saved_size <= exceed_memory and index < len(g["activation_size"]):
            saved_size += g["activation_size"][index]
            index += 1
        return list(g["index"][:index]), list(g["activation_size"][:index])

    def check_recompute(self, ops, base_batch_size, tp_size, dp_size, num_stages_behind, algo_list):
        """Greedy choice of recomputed ops until the stage fits the memory limit
        (aceso_cost_model.py:822-872): check_recompute_batch for one stage."""
        return self.check_recompute_batch([(ops, base_batch_size, tp_size, dp_size, num_stages_behind, algo_list)])[0]

    @staticmethod
    def _mark_recompute(rc, idx_group):
        """aceso_cost_model.py:852-859: the chosen ops and the op after each."""
        for si in idx_group:
            if si < 0:
                break
            rc[si] = 1
            if si < len(rc) - 1:
                rc[si + 1] = 1

    def check_recompute_batch(self, queries, memo=None, starts=None):
        """check_recompute for many stages at once, identical to calling it one by one.
        queries: [(ops, micro_bs, tp_size, dp_size, num_stages_behind, algo_list)]; returns the recompute lists.
        `memo` (default: `self.reference_memo`): whether the starting memory goes through the reference's memo table;
        `starts`, a list, receives per query (memo key, starting memory as evaluated) -- both are for the evaluate-ahead
        of predict_value_after_move, which works off the table and applies it when a result is used.

        Which op group a greedy round takes (:794-806) depends only on the group sums and on which
        groups earlier rounds took, not on the memory figures; those only decide whether the round
        takes the whole group or a prefix of it (:809-820) and when the loop stops.  So instead of one
        launch per round, the states "after the next 1, 2, ... whole groups" of every stage still above
        the limit are evaluated together in one launch and the reference's bookkeeping (:861-867) is
        replayed over the records in order; only a round that takes a prefix leaves that chain and
        asks for another launch.  Three launches are typical where the reference's loop makes a dozen
        stage evaluations."""
        args = self.settings
        n = len(queries)
        use_memo = self.reference_memo if memo is None else memo
        if not args.flex_recompute:
            if starts is not None:
                starts.extend((None, None) for _ in queries)
            return [[1] * len(q[0]) for q in queries]
        rcs = [[0] * len(q[0]) for q in queries]
        if n == 0:
            return rcs
        limit = args.memory_limit

        def query(k, rc):
            q = queries[k]
            return (q[0], rc, q[2], q[3], q[1], q[4], q[5])

        def build_groups(k):
            # (:835-848; the activation sizes are get_activation_size's table entries, looked up for the whole stage at
            # once: this loop is the host's largest share of a check_recompute call)
            ops, micro_bs, tp_size, dp_size, nsb, algo_list = queries[k]
            sizes = self._activation_sizes(ops, micro_bs, tp_size, dp_size, algo_list, nsb + 1)
            groups = {}
            for index, name in enumerate(ops):
                g = groups.get(name)
                if g is None:
                    g = groups[name] = {"index": [], "activation_size": [], "recomputed": False, "sum_size": 0}
                sz = sizes[index]
                g["index"].append(index)
                g["activation_size"].append(sz)
                g["sum_size"] += sz
            return groups

        def chain_of(k, groups, want, stale):
            """The states after the next 1, 2, ... whole-group rounds of stage k (on a copy of the "taken" marks):
            (recompute lists, group lengths)."""
            ops = queries[k][0]
            trial = {name: dict(g) for name, g in groups.items()}
            cur, states, chain, gain = bytearray(rcs[k]), [], [], 0.0
            while True:
                idx, sizes = self._next_recompute_op_group(ops, trial, math.inf)
                if idx is None:
                    break
                cur = bytearray(cur)
                self._mark_recompute(cur, idx)
                chain.append(len(idx))
                states.append(cur)
                gain += sum(sizes)
                # enough groups to get below the limit by their own sizes; after a prefix round (whose
                # effect is not known yet) the loop mostly ends, so one group ahead; a later launch continues if needed
                if stale or gain > want or len(chain) >= 16:
                    break
            return states, chain

        rec = self._stage_records([query(k, rcs[k]) for k in range(n)])
        state, pending = [], []
        for k, (ops, micro_bs, tp_size, dp_size, nsb, algo_list) in enumerate(queries):
            mw, mg, mo, ma, mp, mr = self._memory_breakdown(rec[k].tolist(), nsb)
            stage_memory = mw + mg + mo + ma + mp + mr
            if use_memo or starts is not None:
                # :828 asks predict_stage_memory_helper, whose table is keyed by the stage's first op NAME, its length and
                # its per-op lists (:759): a stage that shares those with one asked about earlier starts from that one's
                # memory, whatever its other ops are (possible where a model's layers differ, as T5's encoder and decoder)
                key = (f"ops{ops[0]}{len(ops)}tp{tp_size}dp{dp_size}rc{rcs[k]}algo{algo_list}bs{micro_bs}stage{nsb}")
                if starts is not None:
                    starts.append((key, stage_memory))
            if use_memo:
                self.stage_memory_visit += 1
                known = self.stage_memory_set.get(key)
                if known is not None:
                    self.stage_memory_hit += 1
                    stage_memory = known
                else:
                    self.stage_memory_set[key] = stage_memory
            stage_memory = stage_memory + args.peak_mem_in_backward
            # get_peak_activations of an all-zero recompute list is 0 (:421)
            st = {"mem": stage_memory, "saved": 0, "peak": 0, "groups": None, "stale": False}
            if stage_memory - limit > 0:
                st["groups"] = build_groups(k)
                pending.append(k)
            state.append(st)

        def account(st, r, nsb):
            new_saved, new_peak = float(r[R_SAVED]), float(r[R_PEAK])
            st["mem"] -= (new_saved - st["saved"]) * (nsb + 1)
            st["saved"] = new_saved
            st["mem"] += (new_peak - st["peak"])
            st["peak"] = new_peak

        while pending:
            launch, plan = [], {}
            for k in pending:
                st = state[k]
                states = [bytearray(rcs[k])] if st["stale"] else []  # a prefix round: its own state is not evaluated yet
                more, chain = chain_of(k, st["groups"], st["mem"] - limit, st["stale"])
                plan[k] = (len(launch), chain, int(st["stale"]))
                launch.extend(query(k, rc) for rc in states + more)
            rec = self._stage_records(launch) if launch else np.zeros((0, STAGE_REC))
            again = []
            for k in pending:
                st, ops, nsb = state[k], queries[k][0], queries[k][4]
                base, chain, off = plan[k]
                if st["stale"]:
                    account(st, rec[base], nsb)
                    st["stale"] = False
                j = 0
                while st["mem"] - limit > 0:
                    if j >= len(chain):
                        again.append(k)          # the evaluated chain is used up (or there was none): next launch
                        break
                    idx_group, _ = self._next_recompute_op_group(ops, st["groups"], st["mem"] - limit)
                    if idx_group is None:
                        break
                    self._mark_recompute(rcs[k], idx_group)
                    if len(idx_group) == chain[j]:
                        account(st, rec[base + off + j], nsb)
                        j += 1
                    else:
                        st["stale"] = True           # a prefix of the group: a state no launch has seen
                        again.append(k)
                        break
            # a stage whose chain was empty has no group left: _next_recompute_op_group returned None above
            pending = [k for k in again if state[k]["stale"] or self._has_open_group(queries[k][0], state[k]["groups"])]
        return rcs

    def _has_open_group(self, ops, groups) -> bool:
        """Whether _next_recompute_op_group would still return a group."""
        trial = {name: dict(g) for name, g in groups.items()}
        return self._next_recompute_op_group(ops, trial, math.inf)[0] is not None

    def update_recompute(self, config, stage_idx=None):
        """aceso_cost_model.py:874-883 (the stages are independent: all of them go through one
        check_recompute_batch)."""
        stages = [config.stages[k] for k in ([stage_idx] if stage_idx is not None else range(config.num_stages))]
        rcs = self.check_recompute_batch([(st.ops, config.micro_bs, st.tp_size, st.dp_size, st.num_stages_behind, st.algo)
                                          for st in stages])
        for st, rc in zip(stages, rcs):
            st.recompute_ops = rc

    def update_recompute_batch(self, configs) -> None:
        """update_recompute(config) for every stage of every plan, in lockstep on the GPU."""
        qs, where = [], []
        for c in configs:
            for st in c.stages:
                qs.append((st.ops, c.micro_bs, st.tp_size, st.dp_size, st.num_stages_behind, st.algo))
                where.append(st)
        for st, rc in zip(where, self.check_recompute_batch(qs)):
            st.recompute_ops = rc

    def update_recompute_arrays(self, batch: PlanBatch, on_device: Optional[bool] = None) -> PlanBatch:
        """update_recompute for every stage of every plan of an encoded batch, without Python objects:
        a copy of the batch with the recompute bits check_recompute chooses (see recompute.py).
        `on_device` (default: yes, with the GPU evaluator): upload the batch, run the greedy loop with its
        selection in the device kernels, download the result -- the same bits as the loop with the numpy
        selection (`on_device=False`), some 30 times sooner for 16,384 plans."""
        from .recompute import update_recompute_arrays, update_recompute_device
        ev = self.evaluator
        if on_device is None:
            on_device = hasattr(ev, "handle")        # the library's handle: the GPU evaluator
        if not on_device or batch.n_plans == 0:
            return update_recompute_arrays(self, batch)
        return ev.download(update_recompute_device(self, ev.upload(batch)))

    def update_recompute_device(self, dbatch):
        """update_recompute_arrays for a batch that lives on the device (evaluator.DeviceBatch in, a new one out)."""
        from .recompute import update_recompute_device
        return update_recompute_device(self, dbatch)

    def generate_initial_config(self, num_stages, args):
        """aceso_utils.py:710-721: the search's starting plan for `args.initial_point` (balance, imbalance_gpu,
        imbalance_op, test, or the path of a plan file) on this model's op list; unscored."""
        from .initial_plans import generate_initial_config
        return generate_initial_config(num_stages, args, self.graph.ops)

    def predict_value_after_move(self, config, bottleneck, partner, num_ops_moved, metric, inc_gpus=False,
                                 dec_gpus=False, dim=None):
        """aceso_cost_model.py:693-739."""
        st = config.stages[bottleneck]
        if self.look_ahead > 0 and not inc_gpus and not dec_gpus and partner is not None and bottleneck != partner:
            ahead = self._scan_step(st, config.micro_bs, bottleneck < partner, num_ops_moved, metric)
            if ahead is not None:
                return ahead
        ops, tp_size, dp_size = list(st.ops), list(st.tp_size), list(st.dp_size)
        algo_list, recompute_ops = list(st.algo), list(st.recompute_ops)
        if num_ops_moved > 0:
            sl = slice(None, -num_ops_moved) if bottleneck < partner else slice(num_ops_moved, None)
            ops, tp_size, dp_size, algo_list = ops[sl], tp_size[sl], dp_size[sl], algo_list[sl]
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
            recompute_ops = self.check_recompute(ops, config.micro_bs, tp_size, dp_size, st.num_stages_behind, algo_list)
        if metric in ["time", "time_with_efficiency"]:
            value = self.predict_stage_time(ops, recompute_ops, tp_size, dp_size, config.micro_bs, algo_list)
        elif metric == "memory":
            value = self.predict_stage_memory(ops, recompute_ops, tp_size, dp_size, config.micro_bs,
                                              st.num_stages_behind, algo_list)
        else:
            raise RuntimeError(f"metric {metric} not implemented.")
        return value, recompute_ops

    # ---- predict_value_after_move over a scan of op counts ------------------------------------------------------------
    # The reference's op migration (aceso_prims.py:168-185, :252-271) asks predict_value_after_move for the same stage
    # with 0, 1, 2, ... ops taken off one end until a value falls below its goal, and again from 0 for the next goal.
    # One such call is a check_recompute (two or three launches) and a stage evaluation, each for ONE stage: launch
    # latency, not scoring.  Once a scan is recognised (the same stage contents, the next op count) the coming op counts
    # are evaluated together, a window that doubles while the scan goes on, and the later calls are answered from that.
    # What a call returns and what it leaves in the memo table are the same as without: a result evaluated ahead is
    # computed off the table (from the stage's own memory) and the table is consulted and written when the result is
    # used; where the table then holds another starting memory for the key, the result is dropped and the call takes
    # the ordinary path.

    _SCANS_KEPT = 16

    def _scan_entry(self, key, count, evaluate):
        """The scan with this key and what was evaluated ahead for op count `count`: (scan, entry), entry None when the
        call is to take the ordinary path.  `evaluate(scan, step)` fills scan["ahead"] for `scan["window"]` op counts
        from `count` on, `step` apart; it is called when `count` continues the scan and is not there yet."""
        scan = self._scans.get(key)
        if scan is None:
            if len(self._scans) >= self._SCANS_KEPT:
                del self._scans[next(iter(self._scans))]
            self._scans[key] = {"last": count, "window": 0, "ahead": {}, "dropped": False}
            return None, None
        if count <= 0:
            scan["last"] = count
            return scan, None
        entry = scan["ahead"].get(count)
        if entry is not None:
            scan["last"] = count
            return scan, entry
        step = count - scan["last"]
        scan["last"] = count
        if not 0 < step <= 8 or scan["dropped"]:
            scan["window"] = 0
            return scan, None
        scan["window"] = min(max(4, 2 * scan["window"]), self.look_ahead)
        try:
            evaluate(scan, step)
        except (KeyError, ValueError, TypeError, IndexError, RuntimeError, ArithmeticError):
            # whatever a later op count's stage raises belongs to the call that asks for it (if one ever does): this
            # call takes the ordinary path, and so do the rest of the scan's
            scan["dropped"] = True
            return scan, None
        return scan, scan["ahead"].get(count)

    def _scan_step(self, st, micro_bs, to_the_right, num_ops_moved, metric):
        """predict_value_after_move(..., num_ops_moved, metric) from a result evaluated ahead: (value, recompute list),
        or None when the call is to take the ordinary path."""
        if metric in ("time", "time_with_efficiency"):
            on_time = True
        elif metric == "memory":
            on_time = False
        else:
            return None
        a = self.settings
        try:
            key = (tuple(st.ops), bytes(st.tp_size), bytes(st.dp_size), bytes(st.algo), micro_bs, st.num_stages_behind,
                   to_the_right, on_time, a.memory_limit, a.flex_recompute, a.peak_mem_in_backward)
        except (ValueError, TypeError):           # a size beyond a byte: not worth a second encoding
            return None
        scan, entry = self._scan_entry(key, num_ops_moved,
                                       lambda sc, step: self._scan_ahead(sc, st, micro_bs, to_the_right, num_ops_moved, step, on_time))
        if entry is None:
            return None
        rc, value, memo_key, start = entry
        if memo_key is not None and self.reference_memo:
            known = self.stage_memory_set.get(memo_key)
            if known is not None and known != start:
                # check_recompute would start elsewhere (see check_recompute_batch); the keys of a scan's other op counts
                # tend to be taken likewise: nothing more is evaluated ahead for this stage
                self.scan_ahead_dropped += 1
                scan["dropped"] = True
                return None
            self.stage_memory_visit += 1
            if known is not None:
                self.stage_memory_hit += 1
            else:
                self.stage_memory_set[memo_key] = start
        self.scan_ahead_used += 1
        return value, list(rc)

    def _scan_ahead(self, scan, st, micro_bs, to_the_right, first, step, on_time):
        """Evaluate `scan["window"]` op counts from `first` on, `step` apart, for stage `st`."""
        n, nsb = len(st.ops), st.num_stages_behind
        counts = [k for k in range(first, first + step * scan["window"], step) if k < n]
        if not counts:
            return
        ops, tp_size, dp_size, algo = list(st.ops), list(st.tp_size), list(st.dp_size), list(st.algo)
        parts = []
        for k in counts:
            sl = slice(None, -k) if to_the_right else slice(k, None)
            parts.append((ops[sl], tp_size[sl], dp_size[sl], algo[sl]))
        starts = []
        rcs = self.check_recompute_batch([(o, micro_bs, t, d, nsb, g) for o, t, d, g in parts], memo=False, starts=starts)
        # (predict_stage_time evaluates with no stage behind, predict_stage_memory with the stage's own count)
        rec = self._stage_records([(o, rc, t, d, micro_bs, 0 if on_time else nsb, g)
                                   for (o, t, d, g), rc in zip(parts, rcs)])
        for j, k in enumerate(counts):
            r = rec[j].tolist()
            if on_time:
                value = self._stage_time_of(r)
            else:
                mw, mg, mo, ma, mp, mr = self._memory_breakdown(r, nsb)
                value = mw + mg + mo + ma + mp + mr
            scan["ahead"][k] = (bytes(rcs[j]), value, starts[j][0], starts[j][1])
        self.scan_ahead_evaluated += len(counts)

    def _delta_scan_step(self, config, st, longest_stage, right, num_ops_moved, decrease):
        """wrap_predict_delta_time from a result evaluated ahead (the op migration asks for 1, 2, 3, ... moved ops of one
        stage in turn when --predict-delta-time is on, aceso_prims.py:174-177), or None for the ordinary path."""
        try:
            nb = None
            if not decrease:
                other = config.stages[longest_stage + 1] if right else config.stages[longest_stage - 1]
                nb = (other.tp_size[0], other.dp_size[0]) if right else (other.tp_size[-1], other.dp_size[-1])
            key = ("delta", tuple(st.ops), bytes(st.recompute_ops), bytes(st.tp_size), bytes(st.dp_size), bytes(st.algo),
                   config.micro_bs, right, decrease, nb)
        except (ValueError, TypeError, IndexError):
            return None

        def evaluate(scan, step):
            n = len(st.ops)
            counts = [k for k in range(num_ops_moved, num_ops_moved + step * scan["window"], step) if k < n]
            queries = []
            for k in counts:
                sl = slice(n - k, None) if right else slice(0, k)
                if decrease:
                    rc, tp, dp = list(st.recompute_ops[sl]), st.tp_size[sl], st.dp_size[sl]
                else:
                    rc, tp, dp = [0] * k, [nb[0]] * k, [nb[1]] * k
                queries.append((st.ops[sl], rc, tp, dp, config.micro_bs, 0, st.algo[sl]))
            rec = self._stage_records(queries)
            for j, k in enumerate(counts):
                scan["ahead"][k] = self._stage_time_of(rec[j].tolist(), delta=True, on_the_right=right, decrease=decrease)
            self.scan_ahead_evaluated += len(counts)

        scan, value = self._scan_entry(key, num_ops_moved, evaluate)
        if value is not None:
            self.scan_ahead_used += 1
        return value

    def wrap_predict_delta_time(self, config, longest_stage, shortest_stage, num_ops_moved, decrease=True):
        """aceso_cost_model.py:885-922."""
        st = config.stages[longest_stage]
        num_ops = len(st.ops)
        if longest_stage == shortest_stage:
            raise RuntimeError("")
        right = longest_stage < shortest_stage
        if self.look_ahead > 0 and 0 < num_ops_moved < num_ops:
            ahead = self._delta_scan_step(config, st, longest_stage, right, num_ops_moved, decrease)
            if ahead is not None:
                return ahead
        sl = slice(num_ops - num_ops_moved, None) if right else slice(0, num_ops_moved)
        ops, algo_list = st.ops[sl], st.algo[sl]
        if decrease:
            recompute_ops, tp_size, dp_size = list(st.recompute_ops[sl]), st.tp_size[sl], st.dp_size[sl]
        else:
            nb = config.stages[longest_stage + 1] if right else config.stages[longest_stage - 1]
            recompute_ops = [0 for _ in range(num_ops_moved)]
            tp_size = [nb.tp_size[0] if right else nb.tp_size[-1] for _ in range(num_ops_moved)]
            dp_size = [nb.dp_size[0] if right else nb.dp_size[-1] for _ in range(num_ops_moved)]
        return self.predict_stage_time(ops, recompute_ops, tp_size, dp_size, config.micro_bs, algo_list,
                                       delta=True, on_the_right=right, decrease=decrease)


# ---- module-level API with the reference's names -------------------------------------------------
args = None
_model: Optional[CostModel] = None


def configure(new_args, device="cuda:0"):
    """Give the module the argparse namespace the reference reads at import (aceso_cost_model.py:10)."""
    global args, _device
    args = new_args
    _device = device


_device = "cuda:0"


def _m() -> CostModel:
    if _model is None:
        raise RuntimeError("read_profiled_time() has not been called")
    return _model


def read_profiled_time(model_name, model_size, time_path):
    """aceso_cost_model.py:27: load the profile database; returns the number of op types."""
    global _model
    if args is None:
        raise RuntimeError("call configure(args) first")
    if _model is not None:
        _model.close()
    _model = CostModel.from_directory(args, model_name, model_size, time_path, device=_device)
    return len(_model.db.op_names)


def predict_time_breakdown(config, print_time=False, print_memory=False):
    return _m().predict_time_breakdown(config, print_time, print_memory)


def predict_time_breakdown_batch(configs):
    return _m().predict_time_breakdown_batch(configs)


def predict_stage_time(ops, recompute_ops, tp_size, dp_size, base_batch_size, algo_list, delta=False,
                       on_the_right=False, decrease=True):
    return _m().predict_stage_time(ops, recompute_ops, tp_size, dp_size, base_batch_size, algo_list, delta,
                                   on_the_right, decrease)


def predict_stage_memory(ops, recompute_ops, tp_size, dp_size, base_batch_size, num_stages_behind, algo_list,
                         breakdown=False):
    return _m().predict_stage_memory(ops, recompute_ops, tp_size, dp_size, base_batch_size, num_stages_behind,
                                     algo_list, breakdown)


def predict_value_after_move(config, bottleneck, partner, num_ops_moved, metric, inc_gpus=False, dec_gpus=False, dim=None):
    return _m().predict_value_after_move(config, bottleneck, partner, num_ops_moved, metric, inc_gpus, dec_gpus, dim)


def wrap_predict_delta_time(config, longest_stage, shortest_stage, num_ops_moved, decrease=True):
    return _m().wrap_predict_delta_time(config, longest_stage, shortest_stage, num_ops_moved, decrease)


def predict_stage_time_helper(config, stage_index):
    return _m().predict_stage_time_helper(config, stage_index)


def predict_stage_memory_helper(config, stage_index, ops=None, recompute_ops=None, tp_size=None, dp_size=None,
                                base_batch_size=None, num_stages_behind=None, algo_list=None):
    return _m().predict_stage_memory_helper(config, stage_index, ops, recompute_ops, tp_size, dp_size,
                                            base_batch_size, num_stages_behind, algo_list)


def check_recompute(ops, base_batch_size, tp_size, dp_size, num_stages_behind, algo_list):
    return _m().check_recompute(ops, base_batch_size, tp_size, dp_size, num_stages_behind, algo_list)


def update_recompute(config, stage_idx=None):
    return _m().update_recompute(config, stage_idx)


def get_reserved_memory_list(config):
    return _m().get_reserved_memory_list(config)


def get_activation_size(op_name, mbs, tp, algo_index=0):
    return _m().get_activation_size(op_name, mbs, tp, algo_index)


def reference_arg_parser():
    """The flags of the reference's command lines that the cost model reads (aceso_utils.py:359-453), with its
    defaults; flags of the search itself are accepted and ignored."""
    import argparse
    ap = argparse.ArgumentParser(allow_abbrev=False)
    ap.add_argument("--model-name", type=str, default=None)
    ap.add_argument("--model-size", type=str, default=None)
    ap.add_argument("--num-layers", type=int, default=None)
    ap.add_argument("--global-batch-size", type=int, default=None)
    ap.add_argument("--micro-batch-size", type=int, nargs="+", default=None)
    ap.add_argument("--num-nodes", type=int, required=True)
    ap.add_argument("--num-gpus-per-node", type=int, required=True)
    ap.add_argument("--memory-limit", type=int, default=28000)
    ap.add_argument("--max-tp", type=int, default=None)
    ap.add_argument("--profiled-time-path", type=str, required=True, help="with the trailing /")
    ap.add_argument("--memory-pred-type", type=str, default="MAX")
    ap.add_argument("--initial-point", type=str, default="balance")
    ap.add_argument("--init-dim", type=str, default="tp")
    ap.add_argument("--do-not-consider-shared-tensor-space", action="store_false", dest="consider_shared_space")
    ap.add_argument("--do-not-consider-reserved-space", action="store_false", dest="consider_reserved_space")
    ap.add_argument("--do-not-use-flex-recompute", action="store_false", dest="flex_recompute")
    ap.add_argument("--peak-mem-in-backward", type=int, default=0)
    ap.add_argument("--consider-collective-memory", action="store_true")
    ap.add_argument("--save-to-csv", type=str, default=None)
    return ap


def main(argv=None, device="cuda:0") -> int:
    """`python -m superscaler_amd.aceso_cost_model`: what the reference's module does when run as a script
    (aceso_cost_model.py:926-932) -- read the plan file named by --initial-point, print its time and memory
    breakdown, write the per-stage csv if --save-to-csv names one.  Takes the reference's flags."""
    import json
    from .plan import config_from_json, save_config_info_to_csv
    ns, _ignored = reference_arg_parser().parse_known_args(argv)
    ns.num_gpus = ns.num_nodes * ns.num_gpus_per_node
    with open(ns.initial_point) as f:
        config_dict = json.load(f)
    # (aceso_utils.py:473-497: the plan file names the model; defaults of the micro-batch sizes by model)
    ns.model_name, ns.model_size = config_dict["model_name"], config_dict["model_size"]
    if ns.model_name not in ("resnet", "gpt", "t5", "scale-layer"):
        raise RuntimeError(f"model {ns.model_name} is not supported yet.")
    if ns.micro_batch_size is None:
        ns.micro_batch_size = [16, 32, 48, 64] if ns.model_name == "resnet" else [1, 2, 4, 8]
    if ns.num_layers is None:
        from .plan import GPT_CONFIGS, T5_CONFIGS
        if ns.model_name == "gpt":
            ns.num_layers = GPT_CONFIGS[ns.model_size][0]
        elif ns.model_name == "t5":
            ns.num_layers = T5_CONFIGS[ns.model_size][0]
        elif ns.model_name == "scale-layer":
            raise RuntimeError("should provide --num-layers for scale-layer exp")
    configure(ns, device)
    read_profiled_time(config_dict["model_name"], config_dict["model_size"], ns.profiled_time_path)
    try:
        config = config_from_json(config_dict, _m().graph.ops)
        predict_time_breakdown(config, print_time=True, print_memory=True)
        if ns.save_to_csv is not None:
            save_config_info_to_csv(config, get_reserved_memory_list(config), ns.save_to_csv)
    finally:
        _m().close()
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
