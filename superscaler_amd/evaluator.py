"""ctypes binding of libace_eval.so and the torch-side plumbing (device buffers, streams).

`PlanEvaluator` owns one ace_handle_t (tables resident on the device).  It never computes a
score itself: if the HIP library is missing or no GPU is present it raises.
"""
import ctypes
import os
from typing import Optional

import numpy as np

from .plan import PlanBatch, validate_batch
from .tables import ABI_VERSION, MAX_STAGES, STAGE_REC, AceTablesStruct, CompiledTables

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libace_eval.so")
_lib = None

EXPORTS = ["ace_abi_version", "ace_strerror", "ace_last_hip_error", "ace_create", "ace_destroy",
           "ace_score_batch", "ace_score_batch_static", "ace_reserve", "ace_topk_workspace_bytes", "ace_topk", "ace_time_score_kernel", "ace_apply_moves",
           "ace_recompute_groups", "ace_recompute_select", "ace_group_keys", "ace_gather_plans"]


class AceBatchStruct(ctypes.Structure):
    _fields_ = [("d_codes", ctypes.c_void_p), ("d_hdr", ctypes.c_void_p), ("d_range", ctypes.c_void_p),
                ("n_plans", ctypes.c_size_t), ("d_order", ctypes.c_void_p)]


class AceRcTablesStruct(ctypes.Structure):
    _fields_ = [("d_codes", ctypes.c_void_p), ("n_plans", ctypes.c_size_t), ("d_type_of_pos", ctypes.c_void_p),
                ("d_activations", ctypes.c_void_p), ("d_no_recompute", ctypes.c_void_p), ("num_ops", ctypes.c_int32),
                ("num_types", ctypes.c_int32), ("n_mbs", ctypes.c_int32), ("n_tp", ctypes.c_int32), ("n_algo", ctypes.c_int32)]


class AceError(RuntimeError):
    pass


def load_library():
    """dlopen the in-tree HIP library; no fallback of any kind."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise AceError(f"{_LIB_PATH} is missing: build it with `python -m superscaler_amd.build` "
                       "(there is no CPU fallback for plan scoring)")
    lib = ctypes.CDLL(_LIB_PATH)
    lib.ace_abi_version.restype = ctypes.c_int
    lib.ace_strerror.restype = ctypes.c_char_p
    lib.ace_strerror.argtypes = [ctypes.c_int]
    lib.ace_last_hip_error.restype = ctypes.c_char_p
    lib.ace_create.restype = ctypes.c_int
    lib.ace_create.argtypes = [ctypes.POINTER(AceTablesStruct), ctypes.POINTER(ctypes.c_void_p)]
    lib.ace_destroy.restype = None
    lib.ace_destroy.argtypes = [ctypes.c_void_p]
    lib.ace_score_batch.restype = ctypes.c_int
    lib.ace_score_batch.argtypes = [ctypes.c_void_p, ctypes.POINTER(AceBatchStruct), ctypes.c_double, ctypes.c_int,
                                    ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                    ctypes.c_void_p, ctypes.c_void_p]
    lib.ace_score_batch_static.restype = ctypes.c_int
    lib.ace_score_batch_static.argtypes = [ctypes.c_void_p, ctypes.POINTER(AceBatchStruct), ctypes.c_double, ctypes.c_int,
                                           ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    lib.ace_reserve.restype = ctypes.c_int
    lib.ace_reserve.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    lib.ace_topk_workspace_bytes.restype = ctypes.c_size_t
    lib.ace_topk_workspace_bytes.argtypes = [ctypes.c_size_t, ctypes.c_int]
    lib.ace_topk.restype = ctypes.c_int
    lib.ace_topk.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int,
                             ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
                             ctypes.c_void_p]
    lib.ace_time_score_kernel.restype = ctypes.c_int
    lib.ace_time_score_kernel.argtypes = [ctypes.c_void_p, ctypes.POINTER(AceBatchStruct), ctypes.c_double,
                                          ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                          ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(ctypes.c_double)]
    lib.ace_apply_moves.restype = ctypes.c_int
    lib.ace_apply_moves.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t,
                                    ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    lib.ace_group_keys.restype = ctypes.c_int
    lib.ace_group_keys.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    lib.ace_gather_plans.restype = ctypes.c_int
    lib.ace_gather_plans.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_size_t, ctypes.c_int] + [ctypes.c_void_p] * 3
    lib.ace_recompute_groups.restype = ctypes.c_int
    lib.ace_recompute_groups.argtypes = [ctypes.POINTER(AceRcTablesStruct), ctypes.c_int] + [ctypes.c_void_p] * 9
    lib.ace_recompute_select.restype = ctypes.c_int
    lib.ace_recompute_select.argtypes = ([ctypes.POINTER(AceRcTablesStruct), ctypes.c_void_p, ctypes.c_int] +
                                         [ctypes.c_void_p] * 9 + [ctypes.c_double, ctypes.c_void_p, ctypes.c_void_p])
    if lib.ace_abi_version() != ABI_VERSION:
        raise AceError("libace_eval.so has a different ABI version")
    _lib = lib
    return lib


def _check(lib, rc, what):
    if rc != 0:
        msg = lib.ace_strerror(rc).decode()
        hip = lib.ace_last_hip_error().decode()
        raise AceError(f"{what}: {msg}" + (f" ({hip})" if hip and rc == -3 else ""))


WAVE = 64            # lanes of a wavefront
WAVES_PER_GROUP = 16  # wavefronts of the scoring kernel's large workgroup
_SNAKE = np.array([0, 1, 2, 3, 7, 6, 5, 4, 8, 9, 10, 11, 15, 14, 13, 12])


def deal_slots(n_plans: int) -> np.ndarray:
    """For a batch sorted from deep to shallow: which sorted position goes into each storage slot.
    The sorted plans are cut into wavefronts of 64 and the wavefronts are dealt round-robin to the
    workgroups of 16, so that every workgroup (every CU) gets the same mix of deep and shallow
    wavefronts; inside a workgroup they are laid out boustrophedon, because wavefront w runs on SIMD
    w % 4 and the four SIMDs should get equal shares too.  The last n_plans % 64 plans keep their place."""
    full = n_plans // WAVE
    groups = (full + WAVES_PER_GROUP - 1) // WAVES_PER_GROUP
    chunk = np.arange(full)
    if groups > 1:
        dealt = []
        for b in range(groups):
            mine = chunk[b::groups]                       # deepest ... shallowest wavefront of this workgroup
            dealt.append(mine[_SNAKE] if len(mine) == WAVES_PER_GROUP else mine)
        chunk = np.concatenate(dealt)
    slots = (chunk[:, None] * WAVE + np.arange(WAVE)[None, :]).reshape(-1)
    return np.concatenate([slots, np.arange(full * WAVE, n_plans)])


def depth_order(batch: PlanBatch) -> np.ndarray:
    """Storage order for a batch: perm[i] = the caller's index of the plan stored in slot i.  The plans
    are sorted (stably) by pipeline depth, deepest first, and by the positions of their first two
    stage boundaries, so that plans that close their stages at the same ops share a wavefront; the
    wavefronts are then dealt to the workgroups (deal_slots)."""
    S = (batch.hdr[:, 0] & 0xff).astype(np.int64)
    P, N = batch.codes.shape
    if N < 2:
        perm = np.argsort(-S, kind="stable")
    else:
        cuts = (batch.codes[:, 1:] & 16) != 0
        c1 = cuts.argmax(axis=1) + 1
        c1[~cuts.any(axis=1)] = 0
        cuts[np.arange(P), c1 - 1] &= (c1 == 0)
        c2 = cuts.argmax(axis=1) + 1
        c2[~cuts.any(axis=1)] = 0
        perm = np.lexsort((c2, c1, -S))
    return perm[deal_slots(P)]


def pack_small_inputs(buf: np.ndarray, batch: PlanBatch, ranges) -> int:
    """Lay a small batch out for the kernel in `buf` (uint8): codes [ceil(N/16)][P][16] (zero padded), then the
    headers uint32 [P][4], then the ranges uint32 [P][2] if given.  Returns the number of bytes used."""
    P, N = batch.codes.shape
    G = (N + 15) // 16
    off_hdr = G * P * 16
    off_rng = off_hdr + P * 16
    n_in = off_rng + (P * 8 if ranges is not None else 0)
    lay = buf[:off_hdr].reshape(G, P, 16)
    full = N // 16
    if full:
        lay[:full] = batch.codes[:, :full * 16].reshape(P, full, 16).transpose(1, 0, 2)
    if full < G:
        lay[full, :, :N - full * 16] = batch.codes[:, full * 16:]
        lay[full, :, N - full * 16:] = 0
    buf[off_hdr:off_rng].view(np.uint32).reshape(P, 4)[...] = batch.hdr
    if ranges is not None:
        buf[off_rng:n_in].view(np.uint32).reshape(P, 2)[...] = ranges
    return n_in


class DeviceBatch:
    """A PlanBatch resident in HBM in the layout the kernel streams."""

    def __init__(self, batch: PlanBatch, device="cuda:0", ranges: Optional[np.ndarray] = None, staging=None,
                 group_by_depth: bool = False):
        """`staging`: a pinned uint8 host tensor of at least P * N bytes; the plan bytes then go through
        it and the copy to the device does not block the host (the caller must not reuse the tensor
        before that copy has completed).
        `group_by_depth`: store the plans sorted by pipeline depth (deepest first) and position of the
        first two stage boundaries, with the permutation alongside (`order`), so that the lanes of a
        wavefront close their stages together; results still come back in the caller's order."""
        import torch
        self.n_plans = batch.n_plans
        self.num_ops = batch.num_ops
        P, N = batch.codes.shape
        G = (N + 15) // 16
        host_codes, host_hdr = batch.codes, batch.hdr
        self.order = None
        if group_by_depth and P > 1:
            perm = depth_order(batch)
            host_codes, host_hdr = host_codes[perm], host_hdr[perm]
            if ranges is not None:
                ranges = np.asarray(ranges)[perm]
            self.order = torch.from_numpy(perm.astype(np.int32)).to(device)
        pinned = getattr(batch, "pinned_tensors", None) if host_codes is batch.codes else None
        if pinned is not None:
            # the plans were produced in page-locked memory (PlanEvaluator.pinned_plan_batch): the copy to the device reads
            # them where they are, no staging copy on the host
            codes = pinned[0].to(device, non_blocking=True)
        elif staging is not None:
            stage = staging[:P * N].view(P, N)
            stage.copy_(torch.from_numpy(np.ascontiguousarray(host_codes)))
            codes = stage.to(device, non_blocking=True)
        else:
            codes = torch.from_numpy(np.ascontiguousarray(host_codes)).to(device)
        if G * 16 != N:
            codes = torch.nn.functional.pad(codes, (0, G * 16 - N))
        # [P, G, 16] -> [G, P, 16]: plan-minor, sixteen ops per 16-byte word
        self.codes = codes.view(P, G, 16).permute(1, 0, 2).contiguous()
        if pinned is not None:
            self.hdr = pinned[1].to(device, non_blocking=True)
        else:
            self.hdr = torch.from_numpy(np.ascontiguousarray(host_hdr).view(np.int32)).to(device)
        self.ranges = None
        if ranges is not None:
            r = np.ascontiguousarray(ranges, dtype=np.uint32)
            assert r.shape == (P, 2)
            self.ranges = torch.from_numpy(r.view(np.int32)).to(device)
        self.struct = AceBatchStruct(self.codes.data_ptr(), self.hdr.data_ptr(),
                                     self.ranges.data_ptr() if self.ranges is not None else None, P,
                                     self.order.data_ptr() if self.order is not None else None)

    @classmethod
    def from_device(cls, codes, hdr, num_ops: int, ranges=None, order=None):
        """Wrap tensors that are already on the device in the kernel's layout: codes uint8 [G, P, 16], hdr int32
        [P, 4], ranges (single-stage queries) int32 [P, 2] or None, order int32 [P] (result index of the plan in
        each slot) or None."""
        self = cls.__new__(cls)
        self.n_plans, self.num_ops = int(hdr.shape[0]), int(num_ops)
        self.codes, self.hdr, self.ranges, self.order = codes, hdr, ranges, order
        self.struct = AceBatchStruct(codes.data_ptr(), hdr.data_ptr(), ranges.data_ptr() if ranges is not None else None,
                                     self.n_plans, order.data_ptr() if order is not None else None)
        return self

    @property
    def bytes_moved_per_plan(self):
        return self.codes.shape[0] * 16 + 16 + (4 if self.order is not None else 0)


class PlanEvaluator:
    def __init__(self, tables: CompiledTables, device="cuda:0"):
        import torch
        if not torch.cuda.is_available():
            raise AceError("no GPU visible: plan scoring runs on the HIP kernels only")
        self.lib = load_library()
        self.tables = tables
        self.device = torch.device(device)
        self._torch = torch
        with torch.cuda.device(self.device):
            ts = tables.as_struct()
            h = ctypes.c_void_p()
            _check(self.lib, self.lib.ace_create(ctypes.byref(ts), ctypes.byref(h)), "ace_create")
        self.handle = h
        self._deal_cache = {}
        self._topk_ws = None
        self._small = None
        self._graphs_alive = 0

    def close(self):
        if getattr(self, "handle", None):
            self.lib.ace_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def upload(self, batch: PlanBatch, validate: bool = True, ranges: Optional[np.ndarray] = None,
               staging=None, group_by_depth: bool = False) -> DeviceBatch:
        """`validate` checks the encoding on the host first (a clear message instead of per-plan status
        bytes; the kernel itself is safe for any byte content).  `group_by_depth`: see DeviceBatch."""
        if validate and ranges is None:
            msg = validate_batch(batch, self.tables)
            if msg:
                raise ValueError(msg)
        return DeviceBatch(batch, self.device, ranges, staging, group_by_depth)

    def pinned_plan_batch(self, n_plans: int) -> PlanBatch:
        """An empty PlanBatch (codes uint8 [n_plans, N], hdr uint32 [n_plans, 4]) whose arrays live in page-locked host
        memory: a producer that writes its plans there (synth.make_plans(out=...), neighbours on the host, a reader of
        plan files) hands them to upload() / score_stream() without the host-side staging copy, so the transfer runs at
        the bus's rate.  The caller must not rewrite the arrays while an upload of them is in flight."""
        torch = self._torch
        N = self.tables.graph.num_ops
        tc = torch.empty((n_plans, N), dtype=torch.uint8, pin_memory=True)
        th = torch.empty((n_plans, 4), dtype=torch.int32, pin_memory=True)
        b = PlanBatch(tc.numpy(), th.numpy().view(np.uint32))
        b.pinned_tensors = (tc, th)
        return b

    def device_context(self):
        """Context manager that makes this evaluator's GPU the current one (for raw library calls)."""
        return self._torch.cuda.device(self.device)

    def _stream(self):
        return ctypes.c_void_p(self._torch.cuda.current_stream(self.device).cuda_stream)

    def score(self, dbatch: DeviceBatch, memory_limit: Optional[float] = None, strict: bool = False,
              breakdown: bool = False, out=None):
        """Launch the scoring kernel; returns device tensors (iter_ms, peak_mb, feasible, status[, stage records
        [P, 16, STAGE_REC]; [P, 1, STAGE_REC] for single-stage queries])."""
        torch = self._torch
        P = dbatch.n_plans
        limit = float(self.tables.settings.memory_limit if memory_limit is None else memory_limit)
        if out is None:
            it = torch.empty(P, dtype=torch.float64, device=self.device)
            pk = torch.empty(P, dtype=torch.float64, device=self.device)
            fe = torch.empty(P, dtype=torch.uint8, device=self.device)
            st = torch.empty(P, dtype=torch.uint8, device=self.device)
        else:
            it, pk, fe, st = out
        breakdown = breakdown or dbatch.ranges is not None
        # (plain scoring with every row resident uses the handle's workspace, which the library reallocates for a larger
        # batch -- unless a captured step holds its address: then ace_reserve() has fixed it and the call is refused)
        # (a single-stage query has one record)
        n_rec = 1 if dbatch.ranges is not None else MAX_STAGES
        rec = torch.zeros((P, n_rec, STAGE_REC), dtype=torch.float64, device=self.device) if breakdown else None
        with torch.cuda.device(self.device):
            rc = self.lib.ace_score_batch(self.handle, ctypes.byref(dbatch.struct), limit, int(strict),
                                          it.data_ptr(), pk.data_ptr(), fe.data_ptr(), st.data_ptr(),
                                          rec.data_ptr() if breakdown else None, self._stream())
        _check(self.lib, rc, "ace_score_batch")
        return (it, pk, fe, st, rec) if breakdown else (it, pk, fe, st)

    def reserve(self, max_plans: int, fixed: bool = False):
        """Size the handle's scoring workspace for batches of up to `max_plans` plans now; `fixed`: a later, larger
        batch is refused (AceError) instead of reallocating it (what a captured step needs)."""
        with self._torch.cuda.device(self.device):
            _check(self.lib, self.lib.ace_reserve(self.handle, int(max_plans), int(fixed)), "ace_reserve")

    def topk(self, iter_ms, feasible, k: int):
        """Device-wide top-k: (indices int64[k], times f64[k], count)."""
        torch = self._torch
        n = iter_ms.numel()
        need = self.lib.ace_topk_workspace_bytes(n, k)
        if self._topk_ws is None or self._topk_ws.numel() < need:
            # (a captured step keeps its own reference to the workspace it recorded, so the old one stays alive for it)
            self._topk_ws = torch.empty(need, dtype=torch.uint8, device=self.device)
        idx = torch.empty(k, dtype=torch.int64, device=self.device)
        val = torch.empty(k, dtype=torch.float64, device=self.device)
        cnt = torch.empty(1, dtype=torch.int32, device=self.device)
        with torch.cuda.device(self.device):
            rc = self.lib.ace_topk(self.handle, iter_ms.data_ptr(), feasible.data_ptr(), n, k, idx.data_ptr(),
                                   val.data_ptr(), cnt.data_ptr(), self._topk_ws.data_ptr(), self._topk_ws.numel(),
                                   self._stream())
        _check(self.lib, rc, "ace_topk")
        return idx, val, cnt

    def capture_step(self, dbatch: DeviceBatch, k: int, memory_limit: Optional[float] = None, strict: bool = False):
        """Score + top-k of a resident batch recorded once in a HIP graph (the library's launches record into a
        capturing stream as they are; nothing in them clears memory with a memset node).  Returns a StepGraph:
        `replay()` runs the recorded launches again on the batch's current bytes and returns the same output
        tensors ((iter_ms, peak_mb, feasible, status), (indices, times, count)).  For a batch that is scored
        again and again after edits in place; the seventeen launches of a step then cost one submission."""
        return StepGraph(self, dbatch, k, memory_limit, strict)

    def time_score_kernel(self, dbatch: DeviceBatch, reps: int, memory_limit: Optional[float] = None) -> float:
        """Average scoring-kernel duration in ms over `reps` back-to-back launches (hipEvents on the
        launch stream)."""
        torch = self._torch
        P = dbatch.n_plans
        limit = float(self.tables.settings.memory_limit if memory_limit is None else memory_limit)
        it = torch.empty(P, dtype=torch.float64, device=self.device)
        pk = torch.empty(P, dtype=torch.float64, device=self.device)
        fe = torch.empty(P, dtype=torch.uint8, device=self.device)
        ms = ctypes.c_double()
        with torch.cuda.device(self.device):
            rc = self.lib.ace_time_score_kernel(self.handle, ctypes.byref(dbatch.struct), limit, 0, it.data_ptr(),
                                                pk.data_ptr(), fe.data_ptr(), reps, self._stream(), ctypes.byref(ms))
        _check(self.lib, rc, "ace_time_score_kernel")
        return ms.value

    def score_stream(self, batches, k: int, memory_limit: Optional[float] = None, strict: bool = False):
        """Score host-resident batches one after the other while the next one is uploaded: uploads go
        through two pinned staging buffers on a second stream (same priority), scoring and the
        per-batch top-k run on the current stream.  Plans are not validated on the host: malformed or
        unscorable ones come back infeasible.  Returns (global plan indices, times) of the k fastest
        feasible plans over all batches (ascending, ties -> lower global index) and the number of
        plans seen."""
        torch = self._torch
        copy_stream = torch.cuda.Stream(device=self.device)
        main = torch.cuda.current_stream(self.device)
        best_idx = np.empty(0, dtype=np.int64)
        best_val = np.empty(0, dtype=np.float64)
        offset = 0
        it = iter(batches)
        staging = [None, None]
        turn = [0]

        def upload(b):
            # buffer `turn` was last used two batches ago, and that batch has been scored and synchronised
            # (plans that already sit in page-locked memory need no staging buffer)
            need = b.n_plans * b.num_ops
            if getattr(b, "pinned_tensors", None) is None and (staging[turn[0]] is None or staging[turn[0]].numel() < need):
                staging[turn[0]] = torch.empty(need, dtype=torch.uint8, pin_memory=True)
            with torch.cuda.stream(copy_stream):
                d = self.upload(b, validate=False, staging=staging[turn[0]])
                ev = torch.cuda.Event()
                ev.record(copy_stream)
            turn[0] ^= 1
            return d, ev

        nxt = next(it, None)
        pending = upload(nxt) if nxt is not None else None
        while pending is not None:
            d, ready = pending
            nxt = next(it, None)
            pending = upload(nxt) if nxt is not None else None     # overlaps with the scoring below
            main.wait_event(ready)
            t, pk, fe, st = self.score(d, memory_limit, strict)
            idx, val, cnt = self.topk(t, fe, k)
            n = int(cnt.item())                                      # synchronises this batch
            best_idx = np.concatenate([best_idx, idx[:n].cpu().numpy() + offset])
            best_val = np.concatenate([best_val, val[:n].cpu().numpy()])
            order = np.lexsort((best_idx, best_val))[:k]
            best_idx, best_val = best_idx[order], best_val[order]
            offset += d.n_plans
            del d
        return best_idx, best_val, offset

    def apply_moves(self, templates: PlanBatch, moves: np.ndarray, with_keys: bool = False):
        """Expand move descriptors (neighbours.sample_moves) into a device-resident batch: only the
        templates and 16 bytes per neighbour cross the bus.  With `with_keys` also returns a device
        tensor int64[n] holding a 64-bit key of every plan's bytes (neighbours.plan_keys_host computes
        the same keys from a PlanBatch)."""
        torch = self._torch
        T, N = templates.codes.shape
        G = (N + 15) // 16
        n = int(moves.shape[0])
        tc = np.zeros((T, G * 16), dtype=np.uint8)
        tc[:, :N] = templates.codes
        d_tc = torch.from_numpy(tc).to(self.device)
        d_th = torch.from_numpy(np.ascontiguousarray(templates.hdr).view(np.int32)).to(self.device)
        d_mv = torch.from_numpy(np.ascontiguousarray(moves, dtype=np.uint32).view(np.int32)).to(self.device)
        codes = torch.empty((G, n, 16), dtype=torch.uint8, device=self.device)
        hdr = torch.empty((n, 4), dtype=torch.int32, device=self.device)
        keys = torch.zeros((n, 2), dtype=torch.int64, device=self.device) if with_keys else None
        with torch.cuda.device(self.device):
            rc = self.lib.ace_apply_moves(d_tc.data_ptr(), d_th.data_ptr(), T, d_mv.data_ptr(), n, N,
                                          self.tables.db.n_algo, codes.data_ptr(), hdr.data_ptr(),
                                          keys.data_ptr() if with_keys else None, self._stream())
        _check(self.lib, rc, "ace_apply_moves")
        d = DeviceBatch.from_device(codes, hdr, N)
        return (d, keys) if with_keys else d

    def select(self, d: DeviceBatch, index) -> DeviceBatch:
        """The plans `index` (device int64 tensor) of a device-resident batch, as a new batch."""
        if d.order is not None:
            raise ValueError("select: the batch is stored in grouped order (group_by_depth)")
        return DeviceBatch.from_device(d.codes.index_select(1, index).contiguous(), d.hdr.index_select(0, index).contiguous(),
                                       d.num_ops)

    def download(self, d: DeviceBatch, index=None) -> PlanBatch:
        """A device-resident batch (or its plans `index`, a device int64 tensor) as a host PlanBatch."""
        if index is not None:
            d = self.select(d, index)
        if d.order is not None:
            raise ValueError("download: the batch is stored in grouped order (group_by_depth)")
        G, P, _ = d.codes.shape
        codes = d.codes.permute(1, 0, 2).reshape(P, G * 16)[:, :d.num_ops].contiguous().cpu().numpy()
        return PlanBatch(codes, d.hdr.cpu().numpy().view(np.uint32).copy())

    def group(self, d: DeviceBatch) -> DeviceBatch:
        """A copy of a device-resident batch in grouped storage order (see DeviceBatch), made on the
        device: sort keys from the library (ace_group_keys), a stable sort, one gather of the plan
        bytes.  Worth it for a batch that is scored more than once; results of the copy come back in the
        order of `d`.  Equal to upload(batch, group_by_depth=True) of the same plans."""
        torch = self._torch
        if d.order is not None or d.ranges is not None:
            raise ValueError("group: a plain batch in its own order is expected")
        P = d.n_plans
        keys = torch.empty(P, dtype=torch.int64, device=self.device)
        with self.device_context():
            _check(self.lib, self.lib.ace_group_keys(d.codes.data_ptr(), d.hdr.data_ptr(), P, d.num_ops, keys.data_ptr(),
                                                     self._stream()), "ace_group_keys")
        by_key = torch.sort(keys, stable=True).indices       # (keys are below 2^48: signed order = unsigned order)
        slots = self._deal_cache.get(P)
        if slots is None:
            slots = torch.from_numpy(deal_slots(P)).to(self.device)
            self._deal_cache = {P: slots}
        perm = by_key.index_select(0, slots).to(torch.int32)
        codes, hdr = torch.empty_like(d.codes), torch.empty_like(d.hdr)
        with self.device_context():
            _check(self.lib, self.lib.ace_gather_plans(d.codes.data_ptr(), d.hdr.data_ptr(), perm.data_ptr(), P, d.num_ops,
                                                       codes.data_ptr(), hdr.data_ptr(), self._stream()), "ace_gather_plans")
        return DeviceBatch.from_device(codes, hdr, d.num_ops, order=perm)

    def stage_records_host(self, batch: PlanBatch, ranges: np.ndarray):
        """Single-stage queries: (status, stage record 0 of every query) as numpy arrays."""
        out = self.score(self.upload(batch, ranges=ranges), breakdown=True)
        return out[3].cpu().numpy(), out[4][:, 0, :].cpu().numpy()

    def picked_records_host(self, batch: PlanBatch, plan_idx: np.ndarray, stage_idx: np.ndarray):
        """Whole plans: (status of every plan, the stage records [plan_idx[k], stage_idx[k]]) as numpy arrays
        (picked on the device, so only those records cross the bus)."""
        torch = self._torch
        out = self.score(self.upload(batch), breakdown=True)
        pick = out[4][torch.from_numpy(np.ascontiguousarray(plan_idx)).to(self.device),
                      torch.from_numpy(np.ascontiguousarray(stage_idx)).to(self.device)]
        return out[3].cpu().numpy(), pick.cpu().numpy()

    # ---- small host-in / host-out calls ------------------------------------------------------------
    # The reference's search calls the cost model for one plan or one stage at a time, so the time of such
    # a call is what a host-side search sees.  Small batches therefore go through one pinned buffer each
    # way: the plans are laid out for the kernel on the host in page-locked memory, which the kernel reads
    # and writes where it is.
    SMALL_IO_BYTES = 1 << 20

    def _small_io(self):
        if self._small is None:
            torch = self._torch
            n = self.SMALL_IO_BYTES
            h_in = torch.empty(n, dtype=torch.uint8, pin_memory=True)
            h_out = torch.empty(n, dtype=torch.uint8, pin_memory=True)
            self._small = (h_in, h_in.numpy(), h_out, h_out.numpy())
        return self._small

    def _score_small(self, batch: PlanBatch, limit: float, strict: bool, breakdown: bool, ranges):
        """score_host for a batch whose inputs and outputs fit SMALL_IO_BYTES; None if they do not."""
        P, N = batch.codes.shape
        G = (N + 15) // 16
        breakdown = breakdown or ranges is not None
        off_hdr = G * P * 16
        off_rng = off_hdr + P * 16
        n_in = off_rng + (P * 8 if ranges is not None else 0)
        n_rec = 1 if ranges is not None else MAX_STAGES          # a single-stage query has one record
        rec_bytes = P * n_rec * STAGE_REC * 8 if breakdown else 0
        off_fe = 16 * P + rec_bytes
        n_out = off_fe + 2 * P
        if n_in > self.SMALL_IO_BYTES or n_out > self.SMALL_IO_BYTES:
            return None
        # the kernel reads the plans from, and writes its results to, page-locked host memory directly (the device sees it
        # at the same address): a kilobyte each way over the bus costs less than two copies and their bookkeeping
        # (measured: 5 to 12 us of a 70 to 140 us call)
        h_in, np_in, h_out, np_out = self._small_io()
        pack_small_inputs(np_in, batch, ranges)
        if breakdown:
            np_out[16 * P:off_fe] = 0
        base_in, base_out = h_in.data_ptr(), h_out.data_ptr()
        struct = AceBatchStruct(base_in, base_in + off_hdr, base_in + off_rng if ranges is not None else None, P, None)
        with self._torch.cuda.device(self.device):
            rc = self.lib.ace_score_batch(self.handle, ctypes.byref(struct), limit, int(strict), base_out, base_out + 8 * P,
                                          base_out + off_fe, base_out + off_fe + P,
                                          base_out + 16 * P if breakdown else None, self._stream())
        _check(self.lib, rc, "ace_score_batch")
        self._torch.cuda.current_stream(self.device).synchronize()
        f64 = np_out[:off_fe].view(np.float64)
        out = (f64[:P].copy(), f64[P:2 * P].copy(), np_out[off_fe:off_fe + P].copy(), np_out[off_fe + P:n_out].copy())
        if breakdown:
            out += (f64[2 * P:].reshape(P, n_rec, STAGE_REC).copy(),)
        return out

    # convenience: host in, host out
    def score_host(self, batch: PlanBatch, memory_limit=None, strict=False, breakdown=False, ranges=None,
                   group_by_depth: bool = False):
        if ranges is None:
            msg = validate_batch(batch, self.tables)
            if msg:
                raise ValueError(msg)
        if not group_by_depth and batch.n_plans <= 4096:
            limit = float(self.tables.settings.memory_limit if memory_limit is None else memory_limit)
            out = self._score_small(batch, limit, strict, breakdown, ranges)
            if out is not None:
                return out
        d = self.upload(batch, validate=False, ranges=ranges, group_by_depth=group_by_depth)
        out = self.score(d, memory_limit, strict, breakdown)
        self._torch.cuda.synchronize(self.device)
        return tuple(None if t is None else t.cpu().numpy() for t in out)


class StepGraph:
    """See PlanEvaluator.capture_step."""

    def __init__(self, ev: PlanEvaluator, dbatch: DeviceBatch, k: int, memory_limit=None, strict=False):
        torch = ev._torch
        self.batch = dbatch                       # the graph holds its addresses
        P = dbatch.n_plans
        self.scores = (torch.empty(P, dtype=torch.float64, device=ev.device), torch.empty(P, dtype=torch.float64, device=ev.device),
                       torch.empty(P, dtype=torch.uint8, device=ev.device), torch.empty(P, dtype=torch.uint8, device=ev.device))
        # one eager step on a side stream first: the handle's workspace and the top-k workspace are allocated
        # there, never inside the capture
        side = torch.cuda.Stream(device=ev.device)
        side.wait_stream(torch.cuda.current_stream(ev.device))
        with torch.cuda.stream(side):
            ev.score(dbatch, memory_limit, strict, out=self.scores)
            ev.topk(self.scores[0], self.scores[2], k)
        torch.cuda.current_stream(ev.device).wait_stream(side)
        torch.cuda.synchronize(ev.device)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            ev.score(dbatch, memory_limit, strict, out=self.scores)
            self.top = ev.topk(self.scores[0], self.scores[2], k)
        self._topk_ws = ev._topk_ws               # the recorded launches write into it: it must outlive a larger topk()
        self._ev = ev
        ev._graphs_alive += 1
        ev.reserve(0, fixed=True)                 # the handle's workspace may not move while the graph lives

    def replay(self):
        if self._ev is None or not self._ev.handle:
            raise AceError("the captured step was released, or its evaluator closed")
        self.graph.replay()
        return self.scores, self.top

    def release(self):
        """Forget the recorded launches (the evaluator may then score larger batches again)."""
        if self._ev is not None:
            self._ev._graphs_alive -= 1
            if self._ev._graphs_alive == 0 and self._ev.handle:
                self._ev.reserve(0, fixed=False)
            self._ev = None
            self.graph = None
            self._topk_ws = None

    def __del__(self):
        try:
            self.release()
        except Exception:
            pass
