"""Table compiler: profile database + op graph + settings -> the dense tables the HIP kernel
gathers from.

Everything in search/aceso_cost_model.py that involves a string, a dict probe, a logarithm or
an op name is evaluated here, once, on the host, with the reference's own arithmetic
(Python floats, math.log), so the device only ever adds, multiplies, divides and takes
maxima of table entries:

  row[type]  per op type, contiguous (staged in LDS as a unit):
     hot   [diag][code][6]   fwd us, bwd us, weights MB, activations MB (x1.5 / 0 rule of
                             :386-391 applied), fwd_reserved MB, bwd_reserved MB
     start [diag][code][3]   input MB, input/intra-node-bandwidth, input/inter-node-bandwidth
                             (:319-336 for the stage's first op, with the index quirks of :275-299)
     out   [mbs][tp][algo][2] output/intra-bandwidth, output/inter-bandwidth (indexed the way
                             :321-326 mixes the first op's tp with the last op's mbs and algo)
     z     [k][diag][code]   ms of collective k (one per (primitive, group size) in use) on this
                             op's input (:247-260, string keys resolved here)
  code = tp_log2 * n_algo + algo.  A "diag" is one way of turning an op's tp into its micro-batch
  index: micro_bs // dp with dp = stage_gpus / tp (:496) depends only on (micro_bs, stage_gpus,
  tp), so each (micro_bs, stage_gpus) pair maps to a tuple (mbs index for tp=1,2,4,8); equal
  tuples share a diag.  Entries whose micro-batch is not profiled are NaN (the reference
  raises KeyError there).
  pair_kinds[kind][glog][code_prev][code_cur]  byte: forward | backward << 4 collective table
     ids (0 = the all-zero table: nothing to do, last id = the all-NaN table: the reference would
     raise) for an adjacent op
     pair, from get_op_spec / get_reshard_primitives (model_ops_info.py:92-150, cost_model:185-245)
  stage_lut[mbs index][glog]  diag | per-tp mbs-index nibbles << 16 (0xF = not profiled).
     Unscorable (micro-batch, stage size) pairs point at diag n_diag, whose hot entries are all NaN.
  pos_info[i]  LDS slot of op i's row | slot of op i+1's row << 8 | kind of the (i, i+1) pair << 16 | flags << 24
"""
import ctypes
import math
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import numpy as np

from . import opgraph as og
from .profile_db import CostModelSettings, ProfileDB

ABI_VERSION = 8
MAX_STAGES = 16
STAGE_REC = 18
LDS_BYTES = 160 * 1024
F_RESHARDING, F_RESERVED_MIN, F_NO_RESERVED, F_COLLECTIVE_MEM = 1, 2, 4, 8

(R_FWD, R_BWD, R_IN_COMM, R_OUT_COMM, R_RECOMP, R_WEIGHTS, R_INPUTS, R_ACT, R_SAVED, R_PEAK,
 R_RESERVED, R_IDEAL_FWD, R_IDEAL_BWD, R_IDEAL_IN, R_IDEAL_OUT, R_STAGE_MS, R_STAGE_MB, R_RESHARD) = range(18)


class AceTablesStruct(ctypes.Structure):
    """ace_tables_t of include/ace_eval.h."""
    _fields_ = [
        ("abi_version", ctypes.c_int32), ("num_ops", ctypes.c_int32), ("num_types", ctypes.c_int32),
        ("n_mbs", ctypes.c_int32), ("n_tp", ctypes.c_int32), ("n_algo", ctypes.c_int32),
        ("n_diag", ctypes.c_int32), ("n_glog", ctypes.c_int32), ("n_z", ctypes.c_int32),
        ("n_pair_kinds", ctypes.c_int32), ("row_doubles", ctypes.c_int32),
        ("hot_off", ctypes.c_int32), ("start_off", ctypes.c_int32), ("out_off", ctypes.c_int32),
        ("z_off", ctypes.c_int32), ("z_table_doubles", ctypes.c_int32), ("n_windows", ctypes.c_int32),
        ("lds_row_bytes", ctypes.c_int32),
        ("flags", ctypes.c_int32), ("main_params", ctypes.c_double), ("optimizer", ctypes.c_double),
        ("rows", ctypes.c_void_p), ("pos_info", ctypes.c_void_p), ("pair_kinds", ctypes.c_void_p),
        ("stage_lut", ctypes.c_void_p), ("nb_minus_1", ctypes.c_void_p), ("win_pos", ctypes.c_void_p),
        ("win_row_begin", ctypes.c_void_p), ("win_rows", ctypes.c_void_p),
    ]


@dataclass
class CompiledTables:
    graph: og.OpGraph
    db: ProfileDB
    settings: CostModelSettings
    n_diag: int
    n_glog: int
    n_z: int
    n_pair_kinds: int
    row_doubles: int
    hot_off: int
    start_off: int
    out_off: int
    z_off: int
    z_table_doubles: int
    lds_row_bytes: int
    flags: int
    rows: np.ndarray            # float64 [n_types, row_doubles]
    pos_info: np.ndarray        # uint32 [N + 1]
    pair_kinds: np.ndarray      # uint8 [n_pk, n_glog, 8, 8]
    stage_lut: np.ndarray       # uint32 [n_mbs, 16]
    nb_minus_1: np.ndarray      # float64 [n_mbs]
    win_pos: np.ndarray         # int32 [n_win + 1]
    win_row_begin: np.ndarray   # int32 [n_win + 1]
    win_rows: np.ndarray        # uint32 [n_rows_total, 2]
    diag_tuples: List[Tuple[int, ...]]
    z_keys: List[Tuple[int, int]]   # (prim id, group size) per collective table

    @property
    def n_windows(self):
        return len(self.win_pos) - 1

    @property
    def C(self):
        return len(self.db.tp_list) * self.db.n_algo

    def as_struct(self) -> AceTablesStruct:
        db = self.db
        s = AceTablesStruct()
        s.abi_version = ABI_VERSION
        s.num_ops = self.graph.num_ops
        s.num_types = len(db.op_names)
        s.n_mbs, s.n_tp, s.n_algo = len(db.mbs_list), len(db.tp_list), db.n_algo
        s.n_diag, s.n_glog, s.n_z, s.n_pair_kinds = self.n_diag, self.n_glog, self.n_z, self.n_pair_kinds
        s.row_doubles = self.row_doubles
        s.hot_off, s.start_off, s.out_off, s.z_off = self.hot_off, self.start_off, self.out_off, self.z_off
        s.z_table_doubles = self.z_table_doubles
        s.n_windows = self.n_windows
        s.lds_row_bytes = self.lds_row_bytes
        s.flags = self.flags
        s.main_params = float(self.settings.memory_main_params)
        s.optimizer = float(self.settings.memory_optimizer)
        for name in ("rows", "pos_info", "pair_kinds", "stage_lut", "nb_minus_1", "win_pos",
                     "win_row_begin", "win_rows"):
            arr = getattr(self, name)
            assert arr.flags["C_CONTIGUOUS"]
            setattr(s, name, arr.ctypes.data)
        return s

    # what a (micro_bs index, log2 stage gpus) pair allows
    def allowed_tp_logs(self, bidx: int, glog: int) -> List[int]:
        mrow = int(self.stage_lut[bidx, glog]) >> 16
        return [t for t in range(len(self.db.tp_list)) if ((mrow >> (4 * t)) & 15) != 15]


def _mbs_tuple(db: ProfileDB, micro_bs: int, gpus: int) -> Tuple[Optional[int], ...]:
    """mbs index per tp for a stage of `gpus` devices: 15 = micro_bs // dp is not a profiled size
    (the reference raises KeyError), None = tp does not divide into the stage (never encoded)."""
    idx = {m: k for k, m in enumerate(db.mbs_list)}
    out = []
    for tp in db.tp_list:
        if tp > gpus or gpus % tp:
            out.append(None)
            continue
        dp = gpus // tp
        out.append(idx.get(micro_bs // dp, 15))   # aceso_cost_model.py:496, :22-25
    return tuple(out)


def _merge_diag(diags: List[List[Optional[int]]], tup) -> int:
    """Index of a diag compatible with `tup` (equal wherever both are defined), extended by
    tup's entries; a new diag if there is none."""
    for d, cur in enumerate(diags):
        if all(a is None or b is None or a == b for a, b in zip(cur, tup)):
            diags[d] = [b if a is None else a for a, b in zip(cur, tup)]
            return d
    diags.append(list(tup))
    return len(diags) - 1


def compile_tables(graph: og.OpGraph, db: ProfileDB, settings: CostModelSettings,
                   lds_budget: int = LDS_BYTES, max_glog: int = 16) -> CompiledTables:
    if list(db.op_names) != list(graph.type_names):
        raise ValueError("op graph and profile database list different op types")
    n_types, M, T, A = len(db.op_names), len(db.mbs_list), len(db.tp_list), db.n_algo
    if M > 15 or T > 4 or A not in (1, 2):
        raise ValueError("table geometry outside what the evaluator encodes (<=15 mbs, <=4 tp, 1-2 algos)")
    C = T * A
    CP = 8            # codes are 3 bits: pair-kind blocks are always 8 x 8
    tb = db.tables
    shared = settings.consider_shared_space

    # ---- diags and the stage LUT -----------------------------------------------------------
    diags: List[List[Optional[int]]] = []
    lut_diag = np.full((M, 16), -1, dtype=np.int64)
    lut_mrow = np.full((M, 16), 0xFFFF, dtype=np.int64)
    n_glog = 1
    for bi, mb in enumerate(db.mbs_list):
        for glog in range(min(16, max_glog)):
            tup = _mbs_tuple(db, mb, 1 << glog)
            if all(x is None or x == 15 for x in tup):
                continue
            lut_diag[bi, glog] = _merge_diag(diags, tup)
            word = 0
            for t in range(4):
                x = tup[t] if t < T else None
                word |= (15 if x is None else x) << (4 * t)
            lut_mrow[bi, glog] = word
            n_glog = max(n_glog, glog + 1)
    diag_tuples = [tuple(15 if x is None else x for x in d) for d in diags]
    n_real_diag = len(diag_tuples)
    if n_real_diag == 0 or n_real_diag > 200:
        raise ValueError("no scorable (micro-batch, stage size) combination")
    ND = n_real_diag

    # ---- adjacent-pair kinds and the collectives in use ----------------------------------------
    z_keys: List[Tuple[int, int]] = []

    ERR = 15   # placeholder while the number of real tables is still growing

    coll_mem = bool(getattr(settings, "consider_collective_memory", False) and settings.resharding
                    and settings.consider_reserved_space)

    def z_id(prim, n):
        if prim == og.P_NONE or (prim == og.P_SPLIT and not coll_mem):
            return 0          # nothing to pay: split is free (aceso_cost_model.py:257-258)
        name = og.PRIM_NAMES[prim]
        # (split costs no time but occupies memory, :262-266: with collective memory it gets a table of its own)
        if prim != og.P_SPLIT and (name not in db.collectives or n not in db.collectives[name]):
            return ERR        # KeyError in the reference (:251)
        if (prim, n) not in z_keys:
            if len(z_keys) >= 13:
                raise ValueError("more than 13 distinct (collective, group size) pairs")
            z_keys.append((prim, n))
        return z_keys.index((prim, n)) + 1

    pk_blocks: List[bytes] = []
    pk_arrays: List[np.ndarray] = []
    pk_of_pos = np.zeros(graph.num_ops + 1, dtype=np.int64)
    kinds = [og.spec_kinds(n) for n in db.op_names]
    pair_cache: Dict[Tuple[int, int], int] = {}
    zero_block = np.zeros((n_glog, CP, CP), dtype=np.uint8)

    def pair_block(tprev: int, tcur: int) -> np.ndarray:
        blk = np.zeros((n_glog, CP, CP), dtype=np.uint8)
        if not settings.resharding:
            return blk
        for glog in range(n_glog):
            g = 1 << glog
            for cp in range(C):
                tp0, a0 = db.tp_list[cp // A], cp % A
                if tp0 > g:
                    continue
                for cc in range(C):
                    tp1, a1 = db.tp_list[cc // A], cc % A
                    if tp1 > g:
                        continue
                    src = og.kind_layout(kinds[tprev][a0][1], tp0, g // tp0)
                    dst = og.kind_layout(kinds[tcur][a1][0], tp1, g // tp1)
                    try:
                        pf, pb, n = og.reshard_prims(src, dst)
                        blk[glog, cp, cc] = z_id(pf, n) | (z_id(pb, n) << 4)
                    except og.InconsistentSpecs:
                        blk[glog, cp, cc] = ERR | (ERR << 4)
        return blk

    def intern(blk: np.ndarray) -> int:
        key = blk.tobytes()
        if key in pk_blocks:
            return pk_blocks.index(key)
        pk_blocks.append(key)
        pk_arrays.append(blk)
        return len(pk_blocks) - 1

    intern(zero_block)     # kind 0: no resharding (also used for position 0)
    for i in range(1, graph.num_ops):
        key = (int(graph.type_of_pos[i - 1]), int(graph.type_of_pos[i]))
        if key not in pair_cache:
            pair_cache[key] = intern(pair_block(*key))
        pk_of_pos[i] = pair_cache[key]
    if len(pk_arrays) > 255:
        raise ValueError("more than 255 distinct adjacent-op spec pairings")
    pair_kinds = np.ascontiguousarray(np.stack(pk_arrays))
    # cost-table ids: 0 = all zeros, 1..len(z_keys) = real collectives, last = all NaN (errors);
    # no tables at all when nothing can ever be paid (resharding off: T5)
    use_z = bool(settings.resharding and (pair_kinds != 0).any())
    NZ = len(z_keys) + 2 if use_z else 0
    if use_z:
        lo, hi = pair_kinds & 15, pair_kinds >> 4
        lo = np.where(lo == ERR, NZ - 1, lo)
        hi = np.where(hi == ERR, NZ - 1, hi)
        pair_kinds = np.ascontiguousarray((lo | (hi << 4)).astype(np.uint8))
    else:
        pair_kinds = np.zeros((1, n_glog, CP, CP), dtype=np.uint8)
        pk_of_pos[:] = 0

    # ---- rows ------------------------------------------------------------------------------
    hot_off = 0
    start_off = hot_off + (ND + 1) * C * 6      # diag ND: all NaN, where unscorable (micro-batch, stage size) pairs point
    out_off = start_off + ND * C * 3
    out_off += out_off & 1                     # (16-byte aligned: its entries are read as pairs)
    z_off = out_off + M * T * A * 2
    z_table_doubles = 1
    while z_table_doubles < ND * C:
        z_table_doubles *= 2          # one collective's table, padded so its index is a shift
    # with collective memory a second set of tables follows: MB a collective occupies (get_reshard_memory :262-273)
    row_doubles = z_off + NZ * z_table_doubles * (2 if coll_mem else 1)
    row_doubles += row_doubles & 1
    if ND > 14:
        raise ValueError("more than 14 distinct micro-batch maps: a plan packs one 4-bit diag per stage")
    # stage LUT: [mbs][glog] -> diag | mrow << 16
    stage_lut = np.zeros((M, 16), dtype=np.uint32)
    for bi in range(M):
        for glog in range(16):
            d = int(lut_diag[bi, glog])
            if d < 0:
                stage_lut[bi, glog] = ND | (0xFFFF << 16)
            else:
                stage_lut[bi, glog] = d | (int(lut_mrow[bi, glog]) << 16)
    rows = np.zeros((n_types, row_doubles), dtype=np.float64)
    nan = math.nan
    reserved_on = settings.consider_reserved_space
    for ty, name in enumerate(db.op_names):
        fl = int(graph.flags[ty])
        hot = np.full((ND + 1, C, 6), nan)
        start = np.full((ND, C, 3), nan)
        z = np.full((max(NZ, 1), ND, C), nan)
        z[0] = 0.0
        zm = np.full((max(NZ, 1), ND, C), nan)
        zm[0] = 0.0
        for d, tup in enumerate(diag_tuples):
            for t in range(T):
                m = tup[t]
                if m == 15:
                    continue
                for a in range(A):
                    c = t * A + a
                    act = float(tb["activations"][ty, m, t, a])
                    if shared and (fl & og.F_ACT_X1_5):
                        act = act * 1.5
                    elif shared and (fl & og.F_ACT_ZERO):
                        act = 0.0
                    rf = float(tb["reserved_fwd"][ty, m, t, a]) if reserved_on else 0.0
                    rb = float(tb["reserved_bwd"][ty, m, t, a]) if reserved_on else 0.0
                    hot[d, c] = (float(tb["fwd"][ty, m, t, a]), float(tb["bwd"][ty, m, t, a]),
                                 float(tb["weights"][ty, m, t, a]), act, rf, rb)
                    insz = float(tb["input_size"][ty, m, t, a])
                    start[d, c] = (insz, db.p2p_time(insz, db.intra_band), db.p2p_time(insz, db.inter_band))
                    for k, (prim, n) in enumerate(z_keys):
                        z[k + 1, d, c] = db.reshard_time(og.PRIM_NAMES[prim], n, insz)
                        # get_reshard_memory: the data itself, times the group size for the gathering collectives
                        zm[k + 1, d, c] = insz * n if og.PRIM_NAMES[prim] in ("all_gather", "all_to_all") else insz
        out = np.zeros((M, T, A, 2))
        for m in range(M):
            for t in range(T):
                for a in range(A):
                    osz = float(tb["output_size"][ty, m, t, a])
                    out[m, t, a] = (db.p2p_time(osz, db.intra_band), db.p2p_time(osz, db.inter_band))
        rows[ty, hot_off:hot_off + hot.size] = hot.ravel()
        rows[ty, start_off:start_off + start.size] = start.ravel()
        rows[ty, out_off:out_off + out.size] = out.ravel()
        for k in range(NZ):
            rows[ty, z_off + k * z_table_doubles:z_off + (k + 1) * z_table_doubles] = nan if k == NZ - 1 else 0.0
            rows[ty, z_off + k * z_table_doubles:z_off + k * z_table_doubles + ND * C] = z[k].ravel()
            if coll_mem:
                o = z_off + (NZ + k) * z_table_doubles
                rows[ty, o:o + z_table_doubles] = nan if k == NZ - 1 else 0.0
                rows[ty, o:o + ND * C] = zm[k].ravel()

    # ---- LDS residency: one window if every row fits, else windows over op positions ----------
    row_bytes = row_doubles * 8
    rk_bytes = pair_kinds.size
    small = ((rk_bytes + 15) & ~15) + M * 16 * 8
    avail = (lds_budget - small) & ~15
    if avail < 2 * row_bytes:
        raise ValueError(f"one op type's row ({row_bytes} B) does not fit LDS twice ({avail} B available)")
    slots = avail // row_bytes
    if slots > 255:
        slots = 255
    pos_info = np.zeros(graph.num_ops + 1, dtype=np.uint32)
    win_pos, win_row_begin, win_rows = [0], [0], []
    tp = graph.type_of_pos
    i = 0
    N = graph.num_ops
    while i < N:
        # a window also holds the row of the op right after it (a stage that ends with the window's
        # last op opens the next stage there) and ends at a multiple of 4 ops (the kernel restages
        # between 4-op words) or at the last op
        slot_of: Dict[int, int] = {}
        j = i
        good = None
        while j < N:
            ty = int(tp[j])
            if ty not in slot_of:
                if len(slot_of) >= slots:
                    break
                slot_of[ty] = len(slot_of)
            j += 1
            if j == N:
                good = (j, dict(slot_of))
            elif j % 4 == 0:
                nt = int(tp[j])
                if nt in slot_of:
                    good = (j, dict(slot_of))
                elif len(slot_of) < slots:
                    snap = dict(slot_of)
                    snap[nt] = len(snap)
                    good = (j, snap)
        if good is None:
            raise ValueError("LDS too small for a 4-op window of this op graph")
        j, slot_of = good
        for k in range(i, j):
            own = slot_of[int(tp[k])]
            nxt = slot_of[int(tp[k + 1])] if k + 1 < N else own
            pos_info[k] = own | (nxt << 8)
        for ty, sl in slot_of.items():
            win_rows.append((ty, sl * row_bytes))
        win_row_begin.append(len(win_rows))
        win_pos.append(j)
        i = j
    win_pos[-1] = 0x7fffffff      # past every position the kernel walks (it walks 16 * ceil(N / 16)): no restaging after the last window
    lds_row_bytes = max(off for _, off in win_rows) + row_bytes

    # the (op k, op k + 1) pair, seen from position k
    normal = [not (shared and (int(graph.flags[t]) & (og.F_ACT_X1_5 | og.F_ACT_ZERO))) for t in range(n_types)]
    for k in range(N - 1):
        cur_t, next_t = int(tp[k]), int(tp[k + 1])
        fl = 0
        if normal[cur_t] and (int(graph.flags[next_t]) & og.F_LAYER_START):
            fl |= 1      # ordinary op right before a layer start: saved += 0, peak segment closes
        if normal[cur_t]:
            fl |= 2      # ordinary op: closes the last segment when the pair ends the stage
        pos_info[k] |= (int(pk_of_pos[k + 1]) << 16) | (fl << 24)

    flags = 0
    if settings.resharding and (pair_kinds != 0).any():
        flags |= F_RESHARDING
    if not settings.consider_reserved_space:
        flags |= F_NO_RESERVED
    elif settings.memory_pred_type == "MIN":
        flags |= F_RESERVED_MIN
    if coll_mem and (flags & F_RESHARDING):
        flags |= F_COLLECTIVE_MEM
    nbm1 = np.array([float(settings.global_batch_size // mb - 1) for mb in db.mbs_list], dtype=np.float64)
    return CompiledTables(
        graph=graph, db=db, settings=settings, n_diag=ND, n_glog=n_glog, n_z=NZ,
        n_pair_kinds=len(pk_arrays), row_doubles=row_doubles, hot_off=hot_off, start_off=start_off,
        out_off=out_off, z_off=z_off, z_table_doubles=z_table_doubles, lds_row_bytes=int(lds_row_bytes), flags=flags,
        rows=np.ascontiguousarray(rows), pos_info=np.ascontiguousarray(pos_info),
        pair_kinds=pair_kinds, stage_lut=np.ascontiguousarray(stage_lut), nb_minus_1=nbm1,
        win_pos=np.array(win_pos, dtype=np.int32), win_row_begin=np.array(win_row_begin, dtype=np.int32),
        win_rows=np.ascontiguousarray(np.array(win_rows, dtype=np.uint32).reshape(-1, 2)),
        diag_tuples=diag_tuples, z_keys=z_keys)
