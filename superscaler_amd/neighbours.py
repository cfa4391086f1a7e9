"""Neighbour generation in array form and a batched local search on top of it.

The reference's move primitives (search/aceso_prims.py:812-826: op migration `dec_op`, `inc/dec_tp`,
`inc/dec_dp`, `inc/dec_mbs`, recompute and algorithm fine-tuning) rebuild Python objects with
copy.deepcopy for every candidate.  Here a move is a byte edit on a copy of the base plan's code
row / header, so thousands of neighbours of one plan are produced with a few numpy operations and
scored by one kernel launch.  The search policy of the reference (aceso_policy.py) is not
reproduced: `hill_climb` is a plain best-neighbour descent used to exercise the batched path.
"""
from typing import Tuple

import numpy as np

from . import opgraph as og
from .plan import PlanBatch
from .tables import CompiledTables


def _stage_bounds(codes_row: np.ndarray):
    starts = np.flatnonzero(codes_row & 16)
    return starts, np.append(starts[1:], len(codes_row))


def _set_header(hdr_row, S, bidx, glogs, gpn):
    gword, cross, till = 0, 0, 0
    for s in range(S):
        gword |= int(glogs[s]) << (4 * s)
        if till % gpn == 0 and till > 0:
            cross |= 1 << s
        till += 1 << int(glogs[s])
        if till % gpn == 0:
            cross |= 1 << (16 + s)
    hdr_row[0] = S | (bidx << 8)
    hdr_row[1] = gword & 0xFFFFFFFF
    hdr_row[2] = gword >> 32
    hdr_row[3] = cross


# edit operations of a move descriptor (uint32[4]: template | op << 16, p0, p1, unused)
OP_NONE, OP_MIGRATE, OP_TP_STEP, OP_RC_TOGGLE, OP_ALGO_TOGGLE = 0, 1, 2, 3, 4


def sample_moves(base: PlanBatch, tables: CompiledTables, n: int, rng: np.random.Generator,
                 max_move: int = 8) -> Tuple[PlanBatch, np.ndarray]:
    """n single-move neighbours of base plan 0 as (templates, moves).  A neighbour is one template row
    (0 = the base plan; the others carry a changed header: micro-batch steps and device moves between
    stages) plus at most one edit of its code bytes, described by four words:
        template | op << 16,  p0,  p1,  0
        OP_MIGRATE      p0 = cut | new cut << 16, p1 = tp (log2) the moved ops take
        OP_TP_STEP      p0 = first op | one past the last << 16, p1 = 1 (tp up) or 0 (tp down)
        OP_RC_TOGGLE    p0 = first op | one past the last << 16
        OP_ALGO_TOGGLE  p0 = op position
    Moves that would leave the profiled grid become (template 0, OP_NONE): a copy of the base plan.
    `apply_moves_host` (numpy) and the library's ace_apply_moves (on the device) expand them."""
    A = tables.db.n_algo
    N = tables.graph.num_ops
    if N >= 65536:
        raise ValueError("move descriptors hold 16-bit op positions")
    gpn = tables.settings.num_gpus_per_node
    row0, hdr0 = base.codes[0], base.hdr[0]
    S = int(hdr0[0] & 0xff)
    bidx = int(hdr0[0] >> 8) & 0xff
    gword = int(hdr0[1]) | (int(hdr0[2]) << 32)
    glogs = np.array([(gword >> (4 * s)) & 15 for s in range(S)], dtype=np.int64)
    starts, ends = _stage_bounds(row0)
    tunable = (tables.graph.flags[tables.graph.type_of_pos] & og.F_TUNABLE) != 0
    M = len(tables.db.mbs_list)
    tp0 = ((row0 & 7) // A).astype(np.int64)
    stage_of_pos = np.cumsum((row0 >> 4) & 1) - 1
    kinds = rng.integers(0, 6, size=n)
    moves = np.zeros((n, 4), dtype=np.uint32)
    t_codes, t_hdr = [row0.copy()], [hdr0.copy()]

    def allowed(b, gl):
        return tables.allowed_tp_logs(b, gl)

    def ok_bits(b, gl):
        return sum(1 << t for t in allowed(b, gl))

    # kind 0, op migration: move a stage boundary by up to max_move ops; the ops that change stage
    # take the tp of the op they now follow / precede in the receiving stage
    rows = np.flatnonzero(kinds == 0)
    if S > 1 and len(rows):
        j = rng.integers(1, S, size=len(rows))
        d = rng.integers(1, max_move + 1, size=len(rows)) * np.where(rng.random(len(rows)) < 0.5, 1, -1)
        cut = starts[j]
        new_cut = cut + d
        good = (new_cut > starts[j - 1]) & (new_cut < ends[j])
        rows, cut, new_cut, d = rows[good], cut[good], new_cut[good], d[good]
        ref = np.where(d > 0, tp0[cut - 1], tp0[cut])        # stage j-1 grows to the right / stage j to the left
        moves[rows, 0] = OP_MIGRATE << 16
        moves[rows, 1] = cut | (new_cut << 16)
        moves[rows, 2] = ref

    # kind 1, tp <-> dp inside one stage: all ops one step up or down, if the stage allows it
    rows = np.flatnonzero(kinds == 1)
    if len(rows):
        s = rng.integers(0, S, size=len(rows))
        step = np.where(rng.random(len(rows)) < 0.5, 1, -1)
        # a stage's ops may sit on different tp: the move is legal iff every tp value present has a legal target
        bits = np.array([ok_bits(bidx, int(g)) for g in glogs], dtype=np.int64)
        present = np.array([sum(1 << int(v) for v in np.unique(tp0[starts[k]:ends[k]])) for k in range(S)], dtype=np.int64)
        want = np.where(step > 0, present[s] << 1, present[s] >> 1)
        lost = (step < 0) & ((present[s] & 1) == 1)                      # tp = 1 cannot go down
        good = ((want & ~bits[s]) == 0) & ~lost
        rows, s, step = rows[good], s[good], step[good]
        moves[rows, 0] = OP_TP_STEP << 16
        moves[rows, 1] = starts[s] | (ends[s] << 16)
        moves[rows, 2] = (step > 0).astype(np.uint32)

    # kind 2, micro-batch size one step up or down, if every op stays on the profiled grid: a header-only template
    rows = np.flatnonzero(kinds == 2)
    if len(rows):
        up = rng.random(len(rows)) < 0.5
        for sign, sel in ((1, up), (-1, ~up)):
            b2 = bidx + sign
            if not 0 <= b2 < M or not sel.any():
                continue
            bits = np.array([ok_bits(b2, int(g)) for g in glogs], dtype=np.int64)[stage_of_pos]
            if (((bits >> tp0) & 1) == 1).all():
                h = hdr0.copy()
                h[0] = S | (b2 << 8)
                t_codes.append(row0.copy())
                t_hdr.append(h)
                moves[rows[sel], 0] = len(t_codes) - 1

    # kind 3, recompute: toggle a short run of ops
    rows = np.flatnonzero(kinds == 3)
    if len(rows):
        lo = rng.integers(0, N, size=len(rows))
        hi = np.minimum(N, lo + rng.integers(1, 14, size=len(rows)))
        moves[rows, 0] = OP_RC_TOGGLE << 16
        moves[rows, 1] = lo | (hi << 16)

    # kind 4, partition algorithm of one tunable op
    rows = np.flatnonzero(kinds == 4)
    if A == 2 and len(rows):
        cand = np.flatnonzero(tunable)
        moves[rows, 0] = OP_ALGO_TOGGLE << 16
        moves[rows, 1] = cand[rng.integers(0, len(cand), size=len(rows))]

    # kind 5, move half of stage a's devices to a stage b that has exactly that many (sizes stay powers
    # of two and the total is unchanged); few distinct (a, b) pairs, each a template of its own
    rows = np.flatnonzero(kinds == 5)
    if S > 1 and len(rows):
        a = rng.integers(0, S, size=len(rows))
        b = (a + rng.integers(1, S, size=len(rows))) % S
        for pa, pb in sorted({(int(x), int(y)) for x, y in zip(a, b)}):
            if glogs[pa] - 1 != glogs[pb]:
                continue
            g2 = glogs.copy()
            g2[pa] -= 1
            g2[pb] += 1
            row = row0.copy()
            good = True
            for st in (pa, pb):
                ok = allowed(bidx, int(g2[st]))
                if not ok:
                    good = False
                    break
                lo, hi = int(starts[st]), int(ends[st])
                t = np.clip(tp0[lo:hi], min(ok), max(ok))
                if not np.all(np.isin(t, ok)):
                    good = False
                    break
                row[lo:hi] = (row[lo:hi] & 0xF8) | (t * A + (row[lo:hi] & (A - 1))).astype(np.uint8)
            if not good:
                continue
            h = hdr0.copy()
            _set_header(h, S, bidx, g2, gpn)
            t_codes.append(row)
            t_hdr.append(h)
            moves[rows[(a == pa) & (b == pb)], 0] = len(t_codes) - 1
    return PlanBatch(np.stack(t_codes), np.stack(t_hdr)), moves


# ---- the reference's own primitives as descriptors --------------------------------------------------------------
# What search/aceso_prims.py's primitives do to a plan, before the update_recompute() call each of them ends with
# (CostModel.update_recompute_arrays / update_recompute_device on the expanded batch; check_recompute does not look at
# the recompute bits a stage had, so re-choosing them for every stage of a plan whose other stages already carry
# check_recompute's choice gives what the primitive's own call on the touched stages gives).  Which stage, partner,
# count or direction to try is the caller's policy (aceso_policy.py, the goal loops of prim_mig_op, the producer /
# consumer choice of prim_tp_dp), made from predict_value_after_move / wrap_predict_delta_time as in the reference.

def _plan_fields(base: PlanBatch, p: int = 0):
    row, hdr = base.codes[p], base.hdr[p]
    S = int(hdr[0] & 0xff)
    gword = int(hdr[1]) | (int(hdr[2]) << 32)
    glogs = np.array([(gword >> (4 * s)) & 15 for s in range(S)], dtype=np.int64)
    starts, ends = _stage_bounds(row)
    return row, hdr, S, int(hdr[0] >> 8) & 0xff, glogs, starts, ends


def migrate_ops_move(base: PlanBatch, n_algo: int, stage: int, partner: int, num_ops: int, template: int = 0) -> np.ndarray:
    """action_move_once (aceso_prims.py:66-134): the last `num_ops` ops of `stage` go to the stage on its right
    (partner > stage) or its first `num_ops` to the stage on its left; they take the tp (and with it the dp) of the
    receiving stage's nearest op (:91-92, :112-113) and keep their algorithm.  One descriptor (uint32[4])."""
    row, _, S, _, _, starts, ends = _plan_fields(base, template)
    if not (0 <= stage < S and 0 <= partner < S and abs(stage - partner) == 1):
        raise ValueError("op migration goes to an adjacent stage")
    if not 0 < num_ops < ends[stage] - starts[stage]:
        raise ValueError("the stage must keep at least one op")       # (:84-86 returns the plan unchanged)
    tp = (row & 7) // n_algo
    if stage < partner:
        cut = int(starts[partner])
        new_cut, ref = cut - num_ops, int(tp[cut])
    else:
        cut = int(starts[stage])
        new_cut, ref = cut + num_ops, int(tp[cut - 1])
    return np.array([template | (OP_MIGRATE << 16), cut | (new_cut << 16), ref, 0], dtype=np.uint32)


def stage_tp_step_move(base: PlanBatch, stage: int, up: bool, template: int = 0) -> np.ndarray:
    """prim_tp_dp_exchange (aceso_prims.py:772-797): every op of `stage` one tp step up (dp halves) or down (dp
    doubles) on the same devices.  The caller checks the legality conditions of :781 / :786-789.  One descriptor."""
    _, _, S, _, _, starts, ends = _plan_fields(base, template)
    if not 0 <= stage < S:
        raise ValueError("no such stage")
    return np.array([template | (OP_TP_STEP << 16), int(starts[stage]) | (int(ends[stage]) << 16), 1 if up else 0, 0],
                    dtype=np.uint32)


def device_steps_template(base: PlanBatch, tables: CompiledTables, steps, p: int = 0):
    """prim_tp_dp (aceso_prims.py:377-485): devices move between stages; `steps` lists (stage, "tp" | "dp", +1 | -1)
    for the producer (its tp or dp halves, :312-321) and the consumers (doubles, :302-310).  A dp step only changes the
    stage's device count; a tp step also moves every op of the stage one tp index.  Returns (code row, header) of the
    resulting plan, to be used as a template row (op OP_NONE)."""
    row, hdr, S, bidx, glogs, starts, ends = _plan_fields(base, p)
    A = tables.db.n_algo
    row, glogs = row.copy(), glogs.copy()
    for stage, dim, sign in steps:
        if dim not in ("tp", "dp") or sign not in (1, -1) or not 0 <= stage < S:
            raise ValueError(f"bad step {(stage, dim, sign)}")
        glogs[stage] += sign
        if dim == "tp":
            lo, hi = int(starts[stage]), int(ends[stage])
            t = (row[lo:hi] & 7).astype(np.int64) // A + sign
            if t.min() < 0 or t.max() >= len(tables.db.tp_list):
                raise ValueError("tp step leaves the profiled sizes")
            row[lo:hi] = (row[lo:hi] & 0xF8) | (t * A + (row[lo:hi] & (A - 1))).astype(np.uint8)
    if glogs.min() < 0:
        raise ValueError("a stage would lose its last device")
    h = hdr.copy()
    _set_header(h, S, bidx, glogs, tables.settings.num_gpus_per_node)
    return row, h


def micro_batch_template(base: PlanBatch, tables: CompiledTables, micro_bs: int, tp_per_stage, p: int = 0):
    """prim_mbs (aceso_prims.py:544-580): the next micro-batch size, every stage uniformly on the tp size
    best_total_gpu_time (:509-542) chose for it (`tp_per_stage`, sizes).  Returns (code row, header)."""
    row, hdr, S, _, glogs, starts, ends = _plan_fields(base, p)
    A = tables.db.n_algo
    row = row.copy()
    for s in range(S):
        t = tables.db.tp_list.index(int(tp_per_stage[s]))
        lo, hi = int(starts[s]), int(ends[s])
        row[lo:hi] = (row[lo:hi] & 0xF8) | (np.uint8(t * A) + (row[lo:hi] & (A - 1))).astype(np.uint8)
    h = hdr.copy()
    h[0] = S | (tables.db.mbs_list.index(int(micro_bs)) << 8)
    return row, h


def apply_moves_host(templates: PlanBatch, moves: np.ndarray, n_algo: int) -> PlanBatch:
    """Expand move descriptors into plans with numpy (masks over a [neighbours, ops] byte matrix)."""
    A = np.uint8(n_algo)
    tmpl = (moves[:, 0] & 0xffff).astype(np.int64)
    op = (moves[:, 0] >> 16).astype(np.int64)
    codes = templates.codes[tmpl]
    hdr = templates.hdr[tmpl]
    N = codes.shape[1]
    pos = np.arange(N)
    lo16, hi16 = (moves[:, 1] & 0xffff).astype(np.int64), (moves[:, 1] >> 16).astype(np.int64)

    def with_tp(seg, t):
        """The code bytes `seg` with their tp replaced by t (algo, recompute and stage bits kept)."""
        return (seg & np.uint8(0xF8)) | (np.asarray(t).astype(np.uint8) * A + (seg & np.uint8(A - 1)))

    rows = np.flatnonzero(op == OP_MIGRATE)
    if len(rows):
        cut, new_cut = lo16[rows], hi16[rows]
        moved = (pos[None, :] >= np.minimum(cut, new_cut)[:, None]) & (pos[None, :] < np.maximum(cut, new_cut)[:, None])
        sub = codes[rows]
        sub[np.arange(len(rows)), cut] &= 0xEF
        sub = np.where(moved, with_tp(sub, moves[rows, 2][:, None]), sub)
        sub[np.arange(len(rows)), new_cut] |= 16
        codes[rows] = sub
    rows = np.flatnonzero(op == OP_TP_STEP)
    if len(rows):
        inside = (pos[None, :] >= lo16[rows][:, None]) & (pos[None, :] < hi16[rows][:, None])
        sub = codes[rows]
        t = ((sub & 7) // A).astype(np.int64) + np.where(moves[rows, 2] == 1, 1, -1)[:, None]
        codes[rows] = np.where(inside, with_tp(sub, t.clip(0, 7)), sub)
    rows = np.flatnonzero(op == OP_RC_TOGGLE)
    if len(rows):
        run = (pos[None, :] >= lo16[rows][:, None]) & (pos[None, :] < hi16[rows][:, None])
        codes[rows] ^= (run * np.uint8(8)).astype(np.uint8)
    rows = np.flatnonzero(op == OP_ALGO_TOGGLE)
    if len(rows):
        codes[rows, moves[rows, 1].astype(np.int64)] ^= 1
    return PlanBatch(codes, hdr)


def make_neighbours(base: PlanBatch, tables: CompiledTables, n: int, rng: np.random.Generator,
                    max_move: int = 8) -> PlanBatch:
    """n single-move neighbours of base plan 0 (moves that would leave the profiled grid are replaced
    by a copy of the base plan, so the batch always has n valid rows)."""
    templates, moves = sample_moves(base, tables, n, rng, max_move)
    return apply_moves_host(templates, moves, tables.db.n_algo)


class VisitedPlans:
    """The search's visited set (aceso_search.py:47,105 over aceso_utils.py:831-844) in array form.

    The reference keys on the config_details string: per-stage op counts, tp, dp, recompute flags,
    algos and the micro-batch size.  For one op graph the encoded bytes of a plan (its code row and
    the first three header words; the fourth, the cross-node bits, follows from them) carry exactly
    that information, so two plans have the same string iff these bytes are equal."""

    def __init__(self):
        self._seen = set()

    def __len__(self):
        return len(self._seen)

    @staticmethod
    def keys(batch: PlanBatch) -> np.ndarray:
        """One fixed-size bytes key per plan (a numpy void array; equal keys = equal plans)."""
        raw = np.concatenate([np.ascontiguousarray(batch.codes),
                              np.ascontiguousarray(batch.hdr[:, :3]).view(np.uint8).reshape(batch.n_plans, 12)], axis=1)
        return np.ascontiguousarray(raw).view(np.dtype((np.void, raw.shape[1]))).ravel()

    def unseen(self, batch: PlanBatch) -> np.ndarray:
        """Mask of the plans that were not marked before and do not repeat an earlier row of this batch."""
        keys = self.keys(batch)
        _, first = np.unique(keys, return_index=True)
        mask = np.zeros(batch.n_plans, dtype=bool)
        mask[first] = True
        if self._seen:
            for p in np.flatnonzero(mask):
                if keys[p].tobytes() in self._seen:
                    mask[p] = False
        return mask

    def mark(self, batch: PlanBatch, rows=None) -> None:
        keys = self.keys(batch)
        for p in (range(batch.n_plans) if rows is None else rows):
            self._seen.add(keys[int(p)].tobytes())


_K0, _K1, _K2 = np.uint64(0x9E3779B97F4A7C15), np.uint64(0xBF58476D1CE4E5B9), np.uint64(0x94D049BB133111EB)


def _key_word(a, b, c, d, idx):
    """The library's per-word mixing (two rounds of the splitmix64 finaliser), on uint64 arrays."""
    u = np.uint64
    x = ((b << u(32)) | a) + _K0 * (u(2) * idx + u(1))
    y = ((d << u(32)) | c) ^ (x >> u(29))
    x = (x ^ (x >> u(30))) * _K1
    x = (x ^ (x >> u(27))) * _K2
    x = x ^ (x >> u(31))
    y = (y + x) * _K1
    y = (y ^ (y >> u(27))) * _K2
    return x ^ y ^ (y >> u(31))


_J0, _J1, _J2 = np.uint64(0xD6E8FEB86659FD93), np.uint64(0xFF51AFD7ED558CCD), np.uint64(0xC4CEB9FE1A85EC53)


def _key_word2(a, b, c, d, idx):
    """The second mixing function of the library's 128-bit plan keys."""
    u = np.uint64
    x = ((d << u(32)) | b) + _J0 * (u(2) * idx + u(1))
    y = ((c << u(32)) | a) ^ (x >> u(31))
    x = (x ^ (x >> u(32))) * _J1
    x = (x ^ (x >> u(29))) * _J2
    x = x ^ (x >> u(32))
    y = (y + x) * _J1
    y = (y ^ (y >> u(29))) * _J2
    return x ^ y ^ (y >> u(32))


def plan_keys_host(batch: PlanBatch) -> np.ndarray:
    """The 128-bit plan keys ace_apply_moves writes, computed on the host (uint64[n_plans, 2])."""
    P, N = batch.codes.shape
    G = (N + 15) // 16
    padded = np.zeros((P, G * 16), dtype=np.uint8)
    padded[:, :N] = batch.codes
    w = padded.view(np.uint32).reshape(P, G, 4).astype(np.uint64)
    idx = (np.arange(G, dtype=np.uint64) + np.uint64(1))[None, :]
    h = batch.hdr.astype(np.uint64)
    zero = np.zeros(P, dtype=np.uint64)
    keys = np.empty((P, 2), dtype=np.uint64)
    with np.errstate(over="ignore"):
        for col, mix in enumerate((_key_word, _key_word2)):
            keys[:, col] = np.bitwise_xor.reduce(mix(w[:, :, 0], w[:, :, 1], w[:, :, 2], w[:, :, 3], idx), axis=1)
            keys[:, col] ^= mix(h[:, 0], h[:, 1], h[:, 2], zero, np.uint64(0))
    return keys


KEY128 = np.dtype([("a", "<u8"), ("b", "<u8")])


def as_key128(keys) -> np.ndarray:
    """uint64[n, 2] (what ace_apply_moves / plan_keys_host give) as one 128-bit record per plan."""
    k = np.asarray(keys)
    if k.dtype == KEY128:
        return k
    k = np.ascontiguousarray(k, dtype=np.uint64)
    if k.ndim != 2 or k.shape[1] != 2:
        raise ValueError("plan keys are pairs of 64-bit words")
    return k.view(KEY128).ravel()


class VisitedKeys:
    """A visited set over 128-bit plan keys (for neighbours that only exist on the device): two sorted
    arrays, a large one and a small one that takes the new keys and is folded into the large one
    when it has grown (so marking costs a merge of the small array only).  Two plans are taken for the
    same plan when both 64-bit halves of their keys agree; the reference's sets compare the plans' full
    strings (aceso_utils.py:831-850)."""

    SMALL_LIMIT = 65536

    def __init__(self):
        self._sorted = np.empty(0, dtype=KEY128)
        self._small = np.empty(0, dtype=KEY128)

    def __len__(self):
        return len(self._sorted) + len(self._small)

    @staticmethod
    def _absent(sorted_keys: np.ndarray, keys: np.ndarray) -> np.ndarray:
        if len(sorted_keys) == 0:
            return np.ones(len(keys), dtype=bool)
        pos = np.searchsorted(sorted_keys, keys)
        return sorted_keys[np.minimum(pos, len(sorted_keys) - 1)] != keys

    def unseen(self, keys: np.ndarray) -> np.ndarray:
        """Mask of the keys not marked before that do not repeat an earlier entry of `keys`."""
        keys = as_key128(keys)
        _, first = np.unique(keys, return_index=True)
        mask = np.zeros(len(keys), dtype=bool)
        mask[first] = True
        cand = np.flatnonzero(mask)
        ok = self._absent(self._sorted, keys[cand]) & self._absent(self._small, keys[cand])
        mask[cand[~ok]] = False
        return mask

    def mark(self, keys: np.ndarray) -> None:
        k = np.unique(as_key128(keys))
        k = k[self._absent(self._sorted, k)]              # (the two arrays stay disjoint: __len__ is their sum)
        self._small = np.union1d(self._small, k)
        if len(self._small) > self.SMALL_LIMIT:
            self._sorted = np.union1d(self._sorted, self._small)
            self._small = np.empty(0, dtype=KEY128)


def hill_climb(cm, start: PlanBatch, steps: int, n_neighbours: int, seed: int = 0, max_move: int = 8,
               on_step=None, visited: VisitedPlans = None, greedy_recompute: bool = False,
               device_moves: bool = False) -> Tuple[PlanBatch, float, float]:
    """Best-neighbour descent: at every step n_neighbours single-move neighbours of the current plan
    are scored in one launch and the fastest feasible one replaces it if it is faster.  With a
    `visited` set, neighbours seen in an earlier step (or twice in one step) are dropped before
    scoring, as aceso_search.py:47 does.  With `greedy_recompute` every neighbour's recompute bits are
    replaced by check_recompute's choice before it is scored, as the reference's primitives do
    (aceso_prims.py:107-108).  With `device_moves` the neighbours never exist on the host: the move
    descriptors (16 bytes each) are expanded by the library on the device and only the winner is
    rebuilt here; `visited` is then a VisitedKeys (128-bit keys of the plan bytes, computed by the
    same kernel, before any recompute bits are re-chosen) and `greedy_recompute` runs check_recompute's
    loop on the device as well (CostModel.update_recompute_device).
    Returns (plan, iteration ms, peak MB)."""
    if device_moves and isinstance(visited, VisitedPlans):
        raise ValueError("device_moves: use a VisitedKeys set")
    rng = np.random.default_rng(seed)
    tables = cm.tables
    ev = cm.evaluator
    cur = start.slice(0, 1)
    it, pk, fe, st = ev.score_host(cur)
    cur_t = float(it[0]) if fe[0] else float("inf")
    cur_m = float(pk[0])
    if visited is not None:
        visited.mark(plan_keys_host(cur) if device_moves else cur)
    for step in range(steps):
        if device_moves:
            templates, moves = sample_moves(cur, tables, n_neighbours, rng, max_move)
            if visited is None:
                # equal descriptors are equal plans: keep one of each (template < 2^16, op < 2^8, p1 < 2^8)
                packed = (moves[:, 0] | (moves[:, 2] << 24)).astype(np.uint64) | (moves[:, 1].astype(np.uint64) << np.uint64(32))
                # (first occurrences, in the order they were drawn: among neighbours of equal time the earliest wins,
                # as it does when the duplicates are scored too)
                moves = moves[np.sort(np.unique(packed, return_index=True)[1])]
                d = ev.apply_moves(templates, moves)
            else:
                d, keys = ev.apply_moves(templates, moves, with_keys=True)
                keys = as_key128(keys.cpu().numpy().view(np.uint64))
                keep = np.flatnonzero(visited.unseen(keys))
                if len(keep) == 0:
                    if on_step is not None:
                        on_step(step, cur_t, cur_m)
                    continue
                visited.mark(keys[keep])
                moves = moves[keep]
                d = ev.select(d, ev._torch.from_numpy(keep).to(d.hdr.device))
            if greedy_recompute:
                d = cm.update_recompute_device(d)
            it, pk, fe, st = ev.score(d)
            idx, val, cnt = ev.topk(it, fe, 1)
            if int(cnt.item()) == 1 and float(val[0].item()) < cur_t:
                best_i = int(idx[0].item())
                cur = ev.download(d, idx[:1]) if greedy_recompute else \
                    apply_moves_host(templates, moves[best_i:best_i + 1], tables.db.n_algo)
                cur_t, cur_m = float(val[0].item()), float(pk[best_i].item())
            if on_step is not None:
                on_step(step, cur_t, cur_m)
            continue
        nb = make_neighbours(cur, tables, n_neighbours, rng, max_move)
        if visited is not None:
            keep = np.flatnonzero(visited.unseen(nb))
            if len(keep) == 0:
                if on_step is not None:
                    on_step(step, cur_t, cur_m)
                continue
            nb = PlanBatch(np.ascontiguousarray(nb.codes[keep]), np.ascontiguousarray(nb.hdr[keep]))
            visited.mark(nb)
        if greedy_recompute:
            nb = cm.update_recompute_arrays(nb)
        d = ev.upload(nb, validate=False)
        it, pk, fe, st = ev.score(d)
        idx, val, cnt = ev.topk(it, fe, 1)
        if int(cnt.item()) == 1:
            best_i, best_t = int(idx[0].item()), float(val[0].item())
            if best_t < cur_t:
                cur = nb.slice(best_i, best_i + 1)
                cur_t, cur_m = best_t, float(pk[best_i].item())
        if on_step is not None:
            on_step(step, cur_t, cur_m)
    return cur, cur_t, cur_m
