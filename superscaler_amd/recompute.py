"""check_recompute for whole batches of encoded plans.

The reference chooses a stage's recomputed ops greedily (search/aceso_cost_model.py:822-872): while
the stage is above the memory limit, take the op name whose activations (summed over the stage,
times num_stages_behind + 1) are largest (get_next_recompute_op_group, :794-820), recompute all of
its occurrences -- or just enough of them -- together with the op after each, and re-evaluate the
saved / peak activations.  `update_recompute_arrays` runs that loop for every stage of every plan
of a PlanBatch at once: the selection is numpy over (stage, op type) matrices with the reference's
order of floating-point additions and its tie-breaks (dict insertion order = first appearance in
the stage), and every greedy round costs one single-stage-query launch for all stages still above
the limit.  Results are identical to calling check_recompute stage by stage.
"""
import numpy as np

from . import opgraph as og
from .plan import PlanBatch
from .tables import R_ACT, R_INPUTS, R_PEAK, R_RESERVED, R_SAVED, R_WEIGHTS


def _stage_table(codes: np.ndarray, hdr: np.ndarray):
    """Every stage of every plan: (plan, first op, one past the last op, stage index)."""
    P, N = codes.shape
    pp, pos = np.nonzero(codes & 16)                       # row-major: by plan, then by position
    first_of_plan = np.r_[True, pp[1:] != pp[:-1]]
    last_of_plan = np.r_[pp[1:] != pp[:-1], True]
    hi = np.where(last_of_plan, N, np.r_[pos[1:], N])
    start_idx = np.flatnonzero(first_of_plan)
    sidx = np.arange(len(pp)) - np.repeat(start_idx, np.diff(np.r_[start_idx, len(pp)]))
    return pp, pos, hi, sidx


def _stage_memory(cm, rec: np.ndarray, nsb: np.ndarray) -> np.ndarray:
    """predict_stage_memory (aceso_cost_model.py:517-539) on stage records, element-wise in the
    reference's order of operations."""
    args = cm.settings
    w = rec[:, R_WEIGHTS]
    mg = w
    mmp = w * args.memory_main_params
    mo = w * args.memory_optimizer
    x = rec[:, R_INPUTS] + rec[:, R_ACT] - rec[:, R_SAVED]
    ma = x * nsb
    mp = x + rec[:, R_PEAK]
    mr = rec[:, R_RESERVED] if args.consider_reserved_space else np.zeros_like(w)
    mw = w + mmp
    return mw + mg + mo + ma + mp + mr


def update_recompute_arrays(cm, batch: PlanBatch) -> PlanBatch:
    """A copy of `batch` whose recompute bits are what update_recompute (aceso_cost_model.py:874-883)
    would choose for every stage.  Raises KeyError / ValueError like the scoring calls do for plans
    outside the profile database."""
    args, tables = cm.settings, cm.tables
    codes = np.ascontiguousarray(batch.codes & np.uint8(0xF7))
    hdr = batch.hdr
    P, N = codes.shape
    if not args.flex_recompute:
        return PlanBatch(codes | np.uint8(8), hdr.copy())
    A = tables.db.n_algo
    a_shift = 1 if A == 2 else 0
    q_plan, q_lo, q_hi, q_s = _stage_table(codes, hdr)
    Q = len(q_plan)
    S = (hdr[:, 0] & 0xff).astype(np.int64)
    if Q != int(S.sum()) or not (codes[:, 0] & 16).all():
        raise ValueError("malformed encoding: stage bits do not match the stage counts")
    q_nsb = S[q_plan] - 1 - q_s
    q_bidx = ((hdr[q_plan, 0] >> 8) & 0xff).astype(np.int64)
    gword = hdr[q_plan, 1].astype(np.uint64) | (hdr[q_plan, 2].astype(np.uint64) << np.uint64(32))
    q_glog = ((gword >> (4 * q_s).astype(np.uint64)) & np.uint64(15)).astype(np.int64)

    def records(qsel):
        """Stage records of the selected stages with the current recompute bits."""
        h = np.zeros((len(qsel), 4), dtype=np.uint32)
        h[:, 0] = (q_nsb[qsel] + 1) | (q_bidx[qsel] << 8)
        h[:, 1] = q_glog[qsel]
        rg = np.stack([q_lo[qsel], q_hi[qsel]], axis=1).astype(np.uint32)
        status, rec0 = cm.evaluator.stage_records_host(PlanBatch(codes[q_plan[qsel]], h), rg)
        cm._raise_for_status(status)
        return rec0

    def all_records():
        """Stage records of every stage with all recompute bits cleared: one launch over the plans
        themselves (a stage's memory terms do not depend on its neighbours)."""
        status, rec = cm.evaluator.picked_records_host(PlanBatch(codes, hdr), q_plan, q_s)
        cm._raise_for_status(status)
        return rec

    mem = _stage_memory(cm, all_records(), q_nsb.astype(np.float64)) + args.peak_mem_in_backward
    act = np.flatnonzero(mem - args.memory_limit > 0)
    if len(act) == 0:
        return PlanBatch(codes, hdr.copy())

    # ---- op groups of the stages above the limit (aceso_cost_model.py:835-843) --------------------
    n_types = len(tables.db.op_names)
    type_of_pos = np.asarray(tables.graph.type_of_pos, dtype=np.int64)
    norec = (np.asarray(tables.graph.flags)[:n_types] & og.F_NO_RECOMPUTE) != 0
    lens = (q_hi - q_lo)[act]
    e_q = np.repeat(np.arange(len(act)), lens)                       # element -> active stage, in (stage, position) order
    e_pos = np.arange(int(lens.sum())) - np.repeat(np.cumsum(lens) - lens, lens) + np.repeat(q_lo[act], lens)
    e_type = type_of_pos[e_pos]
    e_code = (codes[q_plan[act][e_q], e_pos] & 7).astype(np.int64)
    e_tp, e_algo = e_code >> a_shift, e_code & (A - 1)
    mrow = (tables.stage_lut[q_bidx[act], q_glog[act]] >> 16).astype(np.int64)
    e_m = (mrow[e_q] >> (4 * e_tp)) & 15
    if (e_m >= len(tables.db.mbs_list)).any():
        raise KeyError("a stage's micro-batch size per replica is not in the profile database")
    e_size = tables.db.tables["activations"][e_type, e_m, e_tp, e_algo] * (q_nsb[act][e_q] + 1)
    nA = len(act)
    sum_size = np.zeros((nA, n_types))
    np.add.at(sum_size, (e_q, e_type), e_size)                        # unbuffered: adds in position order
    first_pos = np.full((nA, n_types), N, dtype=np.int64)
    np.minimum.at(first_pos, (e_q, e_type), e_pos)
    # the members of every (stage, type) group, in position order
    # (elements are in (stage, position) order already: a stable sort by (stage, type) keeps positions ascending)
    e_key = (e_q * n_types + e_type).astype(np.int32 if nA * n_types < 2 ** 31 else np.int64)
    order = np.argsort(e_key, kind="stable")
    g_pos, g_size = e_pos[order], e_size[order]
    g_key = e_key[order]
    g_start = np.full(nA * n_types, 0, dtype=np.int64)
    g_count = np.bincount(g_key, minlength=nA * n_types)
    g_start[1:] = np.cumsum(g_count)[:-1]

    recomputed = np.zeros((nA, n_types), dtype=bool)
    a_mem = mem[act].copy()
    a_saved = np.zeros(nA)
    a_peak = np.zeros(nA)           # get_peak_activations of an all-zero recompute list is 0 (:421)
    a_plan, a_lo, a_hi, a_nsb = q_plan[act], q_lo[act], q_hi[act], q_nsb[act]
    alive = np.ones(nA, dtype=bool)
    while alive.any():
        ids = np.flatnonzero(alive)
        exceed = a_mem[ids] - args.memory_limit
        # the group with the largest sum; ties go to the op name that appears first in the stage
        elig = ~recomputed[ids] & ~norec[None, :] & (sum_size[ids] > 0)
        masked = np.where(elig, sum_size[ids], -np.inf)
        best = masked.max(axis=1)
        found = best > 0
        pick_key = np.where(elig & (masked == best[:, None]), first_pos[ids], N + 1)
        T = pick_key.argmin(axis=1)
        alive[ids[~found]] = False
        ids, exceed, best, T = ids[found], exceed[found], best[found], T[found]
        if len(ids) == 0:
            break
        recomputed[ids, T] = True
        nxt = first_pos[ids, T] + 1
        inside = nxt < a_hi[ids]
        alive[ids[~inside]] = False                                   # ":805-806" returns None: the loop ends
        ids, exceed, best, T, nxt = ids[inside], exceed[inside], best[inside], T[inside], nxt[inside]
        if len(ids) == 0:
            break
        recomputed[ids, type_of_pos[nxt]] = True
        # how many members of the group: all of them, or the shortest prefix that saves more than the excess
        start, count = g_start[ids * n_types + T], g_count[ids * n_types + T]
        take = count.copy()
        partial = ~(best < exceed)
        if partial.any():
            saved = np.zeros(len(ids))
            index = np.zeros(len(ids), dtype=np.int64)
            for _ in range(int(count[partial].max())):
                go = partial & (saved <= exceed) & (index < count)
                if not go.any():
                    break
                saved[go] += g_size[start[go] + index[go]]
                index[go] += 1
            take[partial] = index[partial]
        m_q = np.repeat(np.arange(len(ids)), take)
        m_k = np.arange(int(take.sum())) - np.repeat(np.cumsum(take) - take, take)
        m_pos = g_pos[start[m_q] + m_k]
        rows = a_plan[ids][m_q]
        codes[rows, m_pos] |= 8
        follow = m_pos + 1 < a_hi[ids][m_q]
        codes[rows[follow], m_pos[follow] + 1] |= 8
        rec = records(act[ids])
        new_saved, new_peak = rec[:, R_SAVED], rec[:, R_PEAK]
        a_mem[ids] = a_mem[ids] - (new_saved - a_saved[ids]) * (a_nsb[ids] + 1)
        a_saved[ids] = new_saved
        a_mem[ids] = a_mem[ids] + (new_peak - a_peak[ids])
        a_peak[ids] = new_peak
        alive[ids[~(a_mem[ids] - args.memory_limit > 0)]] = False
    return PlanBatch(codes, hdr.copy())
