"""ctypes front end of the C oracle (oracle/aceso_oracle.c) -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this file.

`COracle(orc, full_op_list, global_batch_size)` takes a loaded Python oracle (oracle/aceso_oracle.py)
and flattens its state into the dense tables the C code reads, using the Python oracle's own
functions for everything the reference resolves through names, strings and dicts:
  * per op name: the shared-buffer / layer-start predicates (aceso_cost_model.py:386-388, :412);
  * get_op_spec (model_ops_info.py:92-150) per (op, algo, side), recognised as one of four layouts
    and verified against the Python function for every tp, dp in 1..8 x 1..1024;
  * get_reshard_time (aceso_cost_model.py:247-260) per (collective, group size, table entry),
    NaN where it raises KeyError.
Plans go in as plain arrays (stages, per-op tp / dp / algo / recompute).
"""
import ctypes
import math
import os
import subprocess

import numpy as np

from .aceso_oracle import Oracle, get_op_spec

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libaceso_oracle.so")
PRIMS = ["all_reduce", "all_gather", "reduce_scatter", "all_to_all"]
MAX_STAGES = 16


def build(verbose=False):
    """gcc -> oracle/libaceso_oracle.so (IEEE doubles, no contraction, OpenMP over plans)."""
    cmd = ["gcc", "-O2", "-std=c11", "-fPIC", "-shared", "-ffp-contract=off", "-fopenmp",
           os.path.join(HERE, "aceso_oracle.c"), "-o", LIB_PATH, "-lm"]
    if verbose:
        print(" ".join(cmd))
    subprocess.run(cmd, check=True)
    return LIB_PATH


class _Db(ctypes.Structure):
    _fields_ = [("n_types", ctypes.c_int32), ("n_mbs", ctypes.c_int32), ("n_tp", ctypes.c_int32), ("n_algo", ctypes.c_int32),
                ("mbs_values", ctypes.c_void_p), ("field", ctypes.c_void_p * 8), ("type_flags", ctypes.c_void_p),
                ("spec_kind", ctypes.c_void_p), ("reshard_ms", ctypes.c_void_p),
                ("intra_band", ctypes.c_void_p), ("inter_band", ctypes.c_void_p),
                ("n_intra", ctypes.c_int32), ("n_inter", ctypes.c_int32),
                ("resharding", ctypes.c_int32), ("shared_space", ctypes.c_int32), ("reserved_space", ctypes.c_int32),
                ("pred_min", ctypes.c_int32), ("gpus_per_node", ctypes.c_int32), ("global_bs", ctypes.c_int32),
                ("main_params", ctypes.c_double), ("optimizer", ctypes.c_double), ("memory_limit", ctypes.c_double),
                ("collective_memory", ctypes.c_int32)]


class _Plans(ctypes.Structure):
    _fields_ = [("n_plans", ctypes.c_int64), ("n_ops", ctypes.c_int32), ("type_of_pos", ctypes.c_void_p),
                ("num_stages", ctypes.c_void_p), ("micro_bs", ctypes.c_void_p), ("stage_len", ctypes.c_void_p),
                ("tp_log", ctypes.c_void_p), ("dp_log", ctypes.c_void_p), ("algo", ctypes.c_void_p), ("rc", ctypes.c_void_p)]


_KINDS = [lambda tp, dp: {"R": tp, "V": 1, "dims": [1, dp, 1]},
          lambda tp, dp: {"R": tp, "V": 1, "dims": [dp, 1, 1]},
          lambda tp, dp: {"R": 1, "V": 1, "dims": [1, dp, tp]},
          lambda tp, dp: {"R": 1, "V": 1, "dims": [dp, tp, 1]}]


def _spec_kind(name, algo, input_spec):
    """Which of the four layouts get_op_spec returns for this (op, algo, side); checked on a grid."""
    probe = get_op_spec(name, 2, 4, algo, input_spec)
    if probe is None:
        kind = -1
    else:
        kind = next(k for k, f in enumerate(_KINDS) if f(2, 4) == probe)
    for tp in (1, 2, 4, 8):
        for dp in (1, 2, 4, 8, 16, 64, 1024):
            got = get_op_spec(name, tp, dp, algo, input_spec)
            assert got == (None if kind < 0 else _KINDS[kind](tp, dp)), (name, algo, input_spec, tp, dp)
    return kind


class COracle:
    def __init__(self, orc: Oracle, full_op_list, global_batch_size: int):
        if not os.path.exists(LIB_PATH):
            build()
        self.lib = ctypes.CDLL(LIB_PATH)
        self.lib.orc_score.restype = ctypes.c_int
        self.lib.orc_score.argtypes = [ctypes.POINTER(_Db), ctypes.POINTER(_Plans), ctypes.c_int] + [ctypes.c_void_p] * 6 + [ctypes.c_int]
        args = orc.args
        if args.support_comm_predict:
            raise NotImplementedError("support_comm_predict only changes a printed column: not restated in C")
        names = list(orc.op_list)
        self.type_index = {n: k for k, n in enumerate(names)}
        self.full_op_list = list(full_op_list)
        self.type_of_pos = np.array([self.type_index[n] for n in self.full_op_list], dtype=np.int32)
        some = orc.compute_fwd_time[names[0]]
        n_mbs, n_tp, n_algo = len(some), len(some[0]), len(some[0][0])
        self.shape = (len(names), n_mbs, n_tp, n_algo)
        self._keep = []

        def dense(attr):
            a = np.array([getattr(orc, attr)[n] for n in names], dtype=np.float64).reshape(self.shape)
            a = np.ascontiguousarray(a)
            self._keep.append(a)
            return a

        fields = [dense(f) for f in Oracle.FIELDS]
        flags = np.zeros(len(names), dtype=np.uint8)
        for k, n in enumerate(names):
            flags[k] = (1 if n == "enc-attention-dropout" else 0) | (2 if orc._zero_act(n) else 0) | (4 if orc._layer_start(n) else 0)
        spec = np.zeros((len(names), n_algo, 2), dtype=np.int8)
        for k, n in enumerate(names):
            for a in range(n_algo):
                spec[k, a, 0] = _spec_kind(n, a, False)
                spec[k, a, 1] = _spec_kind(n, a, True)
        # get_reshard_time of every input size, per collective and group size
        rt = np.full((4, 4) + self.shape, np.nan)
        in_sz = fields[2]
        if args.resharding:
            cache = {}
            for pi, prim in enumerate(PRIMS):
                for lg in range(1, 4):
                    for idx in np.ndindex(*self.shape):
                        key = (pi, lg, float(in_sz[idx]))
                        if key not in cache:
                            try:
                                cache[key] = float(orc.get_reshard_time(prim, 1 << lg, float(in_sz[idx])))
                            except KeyError:
                                cache[key] = math.nan
                        rt[(pi, lg) + idx] = cache[key]
        mbs_values = np.array(list(args.micro_batch_size), dtype=np.int32)
        intra = np.array(orc.intra_band, dtype=np.float64)
        inter = np.array(orc.inter_band, dtype=np.float64)
        self._keep += [flags, spec, rt, mbs_values, intra, inter, self.type_of_pos]
        db = _Db()
        db.n_types, db.n_mbs, db.n_tp, db.n_algo = self.shape
        db.mbs_values = mbs_values.ctypes.data
        for k in range(8):
            db.field[k] = fields[k].ctypes.data
        db.type_flags = flags.ctypes.data
        db.spec_kind = spec.ctypes.data
        db.reshard_ms = rt.ctypes.data
        db.intra_band, db.inter_band = intra.ctypes.data, inter.ctypes.data
        db.n_intra, db.n_inter = len(intra), len(inter)
        db.resharding = int(bool(args.resharding))
        db.shared_space = int(bool(args.consider_shared_space))
        db.reserved_space = int(bool(args.consider_reserved_space))
        if args.memory_pred_type not in ("MAX", "MIN"):
            raise RuntimeError(f"unknown args.memory_pred_type {args.memory_pred_type}")
        db.pred_min = int(args.memory_pred_type == "MIN")
        db.gpus_per_node = int(args.num_gpus_per_node)
        db.global_bs = int(global_batch_size)
        db.main_params, db.optimizer = float(args.memory_main_params), float(args.memory_optimizer)
        db.memory_limit = float(args.memory_limit)
        db.collective_memory = int(bool(args.consider_collective_memory))
        self.db = db

    def score_arrays(self, num_stages, micro_bs, stage_len, tp_log, dp_log, algo, rc, strict=False, lists=False,
                     threads=1, memory_limit=None):
        """Plain arrays in ([P], [P], [P,16], [P,N] x 4) -> (iter_ms, peak_mb, feasible, error[, time_list, memory_list])."""
        P, N = tp_log.shape
        assert N == len(self.type_of_pos)
        arrs = [np.ascontiguousarray(num_stages, dtype=np.int32), np.ascontiguousarray(micro_bs, dtype=np.int32),
                np.ascontiguousarray(stage_len, dtype=np.int32)] + \
               [np.ascontiguousarray(a, dtype=np.uint8) for a in (tp_log, dp_log, algo, rc)]
        pl = _Plans()
        pl.n_plans, pl.n_ops = P, N
        pl.type_of_pos = self.type_of_pos.ctypes.data
        (pl.num_stages, pl.micro_bs, pl.stage_len, pl.tp_log, pl.dp_log, pl.algo, pl.rc) = [a.ctypes.data for a in arrs]
        it, pk = np.empty(P), np.empty(P)
        fe, er = np.empty(P, dtype=np.uint8), np.empty(P, dtype=np.uint8)
        tl = np.full((P, MAX_STAGES), np.nan) if lists else None
        ml = np.full((P, MAX_STAGES), np.nan) if lists else None
        if memory_limit is not None:
            self.db.memory_limit = float(memory_limit)
        rc_ = self.lib.orc_score(ctypes.byref(self.db), ctypes.byref(pl), int(strict), it.ctypes.data, pk.ctypes.data,
                                 fe.ctypes.data, er.ctypes.data, tl.ctypes.data if lists else None,
                                 ml.ctypes.data if lists else None, int(threads))
        assert rc_ == 0
        return (it, pk, fe, er, tl, ml) if lists else (it, pk, fe, er)

    def score_configs(self, configs, **kw):
        """Config objects (stages with ops / tp_size / dp_size / algo / recompute_ops) -> score_arrays."""
        P, N = len(configs), len(self.full_op_list)
        S = np.zeros(P, dtype=np.int32)
        mb = np.zeros(P, dtype=np.int32)
        sl = np.zeros((P, MAX_STAGES), dtype=np.int32)
        tp, dp, al, rc = (np.zeros((P, N), dtype=np.uint8) for _ in range(4))
        for p, c in enumerate(configs):
            S[p], mb[p] = c.num_stages, c.micro_bs
            lo = 0
            for s, st in enumerate(c.stages):
                n = len(st.ops)
                assert list(st.ops) == self.full_op_list[lo:lo + n]
                sl[p, s] = n
                tp[p, lo:lo + n] = [int(math.log(t, 2)) for t in st.tp_size]
                dp[p, lo:lo + n] = [int(math.log(d, 2)) for d in st.dp_size]
                al[p, lo:lo + n] = st.algo
                rc[p, lo:lo + n] = st.recompute_ops
                lo += n
            assert lo == N
        return self.score_arrays(S, mb, sl, tp, dp, al, rc, **kw)
