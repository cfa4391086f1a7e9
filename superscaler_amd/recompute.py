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


def update_recompute_device(cm, dbatch):
    """update_recompute for every stage of every plan of a device-resident batch (evaluator.DeviceBatch),
    without the plans ever visiting the host: the same greedy loop as `update_recompute_arrays`, with
    the selection done by the library's ace_recompute_groups / ace_recompute_select kernels and the
    memory bookkeeping by element-wise fp64 tensor operations (the reference's order of operations,
    one rounding each).  Returns a new DeviceBatch; bit-identical to the host form."""
    import ctypes
    import torch
    from .evaluator import AceRcTablesStruct, DeviceBatch, _check
    args, tables, ev = cm.settings, cm.tables, cm.evaluator
    if getattr(dbatch, "order", None) is not None:
        raise ValueError("update_recompute_device: the batch is stored in grouped order (group_by_depth)")
    dev = dbatch.hdr.device
    N, P = dbatch.num_ops, dbatch.n_plans
    G = (N + 15) // 16
    codes = dbatch.codes.clone()
    if not args.flex_recompute:
        codes |= 8
        if G * 16 != N:
            codes.view(G, P, 16)[G - 1, :, N - (G - 1) * 16:] = 0
        return DeviceBatch.from_device(codes, dbatch.hdr, N)
    codes &= 0xF7
    hdr = dbatch.hdr.to(torch.int64) & 0xFFFFFFFF
    # ---- every stage of every plan: (plan, first op, one past the last op, stage index) ----------
    rows = codes.permute(1, 0, 2).reshape(P, G * 16)[:, :N]
    idx = ((rows & 16) != 0).nonzero()                      # sorted by plan, then by position
    q_plan, q_lo = idx[:, 0].contiguous(), idx[:, 1].contiguous()
    Q = int(q_plan.numel())
    S = hdr[:, 0] & 0xff
    if Q != int(S.sum().item()) or not bool(((rows[:, 0] & 16) != 0).all().item()):
        raise ValueError("malformed encoding: stage bits do not match the stage counts")
    same_next = torch.cat([q_plan[1:] == q_plan[:-1], torch.zeros(1, dtype=torch.bool, device=dev)])
    q_hi = torch.where(same_next, torch.cat([q_lo[1:], q_lo.new_full((1,), N)]), q_lo.new_full((Q,), N))
    first = torch.cat([torch.ones(1, dtype=torch.bool, device=dev), q_plan[1:] != q_plan[:-1]])
    start_idx = first.nonzero().squeeze(1)
    counts = torch.diff(torch.cat([start_idx, start_idx.new_full((1,), Q)]))
    q_s = torch.arange(Q, device=dev) - torch.repeat_interleave(start_idx, counts)
    q_nsb = S[q_plan] - 1 - q_s
    q_bidx = (hdr[q_plan, 0] >> 8) & 0xff
    gword = hdr[q_plan, 1] | (hdr[q_plan, 2] << 32)
    q_glog = (gword >> (4 * q_s)) & 15

    # ---- all stages with the recompute bits cleared: one launch over the plans themselves ---------
    out = ev.score(DeviceBatch.from_device(codes, dbatch.hdr, N), breakdown=True)
    cm._raise_for_status(out[3].cpu().numpy())
    rec = out[4][q_plan, q_s]

    def stage_memory(r, nsb):
        w = r[:, R_WEIGHTS]
        x = r[:, R_INPUTS] + r[:, R_ACT] - r[:, R_SAVED]
        mr = r[:, R_RESERVED] if args.consider_reserved_space else torch.zeros_like(w)
        return (w + w * args.memory_main_params) + w + w * args.memory_optimizer + x * nsb + (x + r[:, R_PEAK]) + mr

    mem = stage_memory(rec, q_nsb.to(torch.float64)) + args.peak_mem_in_backward
    act = (mem - args.memory_limit > 0).nonzero().squeeze(1)
    nA = int(act.numel())
    if nA == 0:
        return DeviceBatch.from_device(codes, dbatch.hdr, N)

    # ---- device tables of the selection kernels ----------------------------------------------------
    n_types = len(tables.db.op_names)
    act_tab = np.ascontiguousarray(tables.db.tables["activations"], dtype=np.float64)
    d_act = torch.from_numpy(act_tab).to(dev)
    d_types = torch.from_numpy(np.ascontiguousarray(tables.graph.type_of_pos, dtype=np.int32)).to(dev)
    norec = ((np.asarray(tables.graph.flags)[:n_types] & og.F_NO_RECOMPUTE) != 0).astype(np.uint8)
    d_norec = torch.from_numpy(norec).to(dev)
    lut = torch.from_numpy(np.ascontiguousarray(tables.stage_lut).astype(np.int64)).to(dev)
    t = AceRcTablesStruct(codes.data_ptr(), P, d_types.data_ptr(), d_act.data_ptr(), d_norec.data_ptr(), N, n_types,
                          act_tab.shape[1], act_tab.shape[2], act_tab.shape[3])
    a_plan = q_plan[act].to(torch.int32).contiguous()
    a_lo, a_hi = q_lo[act].to(torch.int32).contiguous(), q_hi[act].to(torch.int32).contiguous()
    a_nsb = q_nsb[act].to(torch.int32).contiguous()
    a_mrow = (lut[q_bidx[act], q_glog[act]] >> 16).to(torch.int32).contiguous()      # (bit pattern of the uint32)
    sum_size = torch.zeros((nA, n_types), dtype=torch.float64, device=dev)
    first_pos = torch.full((nA, n_types), N, dtype=torch.int32, device=dev)
    bad = torch.zeros(nA, dtype=torch.int32, device=dev)
    stream = ev._stream()
    with ev.device_context():
        _check(ev.lib, ev.lib.ace_recompute_groups(ctypes.byref(t), nA, a_plan.data_ptr(), a_lo.data_ptr(), a_hi.data_ptr(),
                                                   a_nsb.data_ptr(), a_mrow.data_ptr(), sum_size.data_ptr(),
                                                   first_pos.data_ptr(), bad.data_ptr(), stream), "ace_recompute_groups")
    if bool(bad.any().item()):
        raise KeyError("a stage's micro-batch size per replica is not in the profile database")
    recomputed = torch.zeros((nA, n_types), dtype=torch.uint8, device=dev)
    a_mem = mem[act].contiguous()
    a_saved = torch.zeros(nA, dtype=torch.float64, device=dev)
    a_peak = torch.zeros(nA, dtype=torch.float64, device=dev)     # get_peak_activations of an all-zero list is 0 (:421)
    alive = torch.ones(nA, dtype=torch.uint8, device=dev)
    q_hdr = torch.zeros((nA, 4), dtype=torch.int32, device=dev)
    q_hdr[:, 0] = ((a_nsb.to(torch.int64) + 1) | (q_bidx[act] << 8)).to(torch.int32)
    q_hdr[:, 1] = q_glog[act].to(torch.int32)
    q_rng = torch.stack([a_lo, a_hi], dim=1).contiguous()
    nsb1 = (a_nsb + 1).to(torch.float64)
    while True:
        with ev.device_context():
            _check(ev.lib, ev.lib.ace_recompute_select(ctypes.byref(t), codes.data_ptr(), nA, a_plan.data_ptr(), a_lo.data_ptr(),
                                                       a_hi.data_ptr(), a_nsb.data_ptr(), a_mrow.data_ptr(), sum_size.data_ptr(),
                                                       first_pos.data_ptr(), recomputed.data_ptr(), a_mem.data_ptr(),
                                                       float(args.memory_limit), alive.data_ptr(), stream), "ace_recompute_select")
        ids = alive.nonzero().squeeze(1)
        if ids.numel() == 0:
            break
        # re-evaluate the stages that were changed: their plans' columns, as single-stage queries
        sub = DeviceBatch.from_device(codes.index_select(1, a_plan[ids].to(torch.int64)).contiguous(), q_hdr[ids].contiguous(),
                                      N, ranges=q_rng[ids].contiguous())
        r = ev.score(sub, breakdown=True)[4][:, 0, :]
        new_saved, new_peak = r[:, R_SAVED], r[:, R_PEAK]
        m = a_mem[ids] - (new_saved - a_saved[ids]) * nsb1[ids]
        a_saved[ids] = new_saved
        m = m + (new_peak - a_peak[ids])
        a_peak[ids] = new_peak
        a_mem[ids] = m
        alive[ids] = (m - args.memory_limit > 0).to(torch.uint8)
    return DeviceBatch.from_device(codes, dbatch.hdr, N)
