"""Shared test plumbing: build the oracle from the same database / settings the product
compiles its tables from, score batches with the oracle, load the CPU emulation build."""
import ctypes
import os
import subprocess

import numpy as np

from oracle.aceso_oracle import Oracle, Settings
from oracle.aceso_oracle import Config as OConfig, StageInfo as OStage

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_FIELD = {"fwd": "compute_fwd_time", "bwd": "compute_bwd_time", "input_size": "input_size",
                "output_size": "output_size", "weights": "weights", "activations": "activations",
                "reserved_fwd": "reserved_fwd", "reserved_bwd": "reserved_bwd"}


def oracle_for(tables):
    """An Oracle holding exactly the data `tables` was compiled from."""
    st, db = tables.settings, tables.db
    s = Settings(model_name=st.model_name, micro_batch_size=list(st.micro_batch_size),
                 num_gpus_per_node=st.num_gpus_per_node, memory_limit=st.memory_limit, max_tp=st.max_tp,
                 consider_shared_space=st.consider_shared_space,
                 consider_reserved_space=st.consider_reserved_space, flex_recompute=st.flex_recompute,
                 peak_mem_in_backward=st.peak_mem_in_backward, memory_pred_type=st.memory_pred_type,
                 consider_collective_memory=bool(getattr(st, "consider_collective_memory", False)))
    s.resharding = st.resharding
    orc = Oracle(s)
    orc.load_dense(db.op_names, {ORACLE_FIELD[k]: v.tolist() for k, v in db.tables.items()},
                   db.collectives, db.intra_band, db.inter_band)
    return orc


def oracle_config(batch, p, tables):
    return batch.to_config(p, tables, cls_config=OConfig, cls_stage=OStage)


def oracle_scores(orc, batch, tables, idx=None, strict=False):
    """(iter_ms, peak_mb, feasible, configs) for the selected plans."""
    idx = range(batch.n_plans) if idx is None else idx
    it, pk, fe, cfgs = [], [], [], []
    for p in idx:
        c = oracle_config(batch, p, tables)
        t, m, f = orc.score(c, strict=strict)
        it.append(t); pk.append(m); fe.append(int(f)); cfgs.append(c)
    return np.array(it), np.array(pk), np.array(fe, dtype=np.uint8), cfgs


_emu = None


def emu_lib():
    """The bounds-checked CPU build of the kernel's state machine (tests/emu/ace_emu.cpp)."""
    global _emu
    if _emu is None:
        so = os.path.join(ROOT, "tests", "emu", "libace_emu.so")
        src = os.path.join(ROOT, "tests", "emu", "ace_emu.cpp")
        hdrs = [os.path.join(ROOT, "superscaler_amd", "csrc", h) for h in ("ace_plan_state.h", "ace_score_loop.h")]
        if (not os.path.exists(so)) or os.path.getmtime(so) < max(os.path.getmtime(f) for f in [src] + hdrs):
            subprocess.run(["g++", "-O2", "-std=c++17", "-ffp-contract=off", "-shared", "-fPIC",
                            "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROOT, "superscaler_amd", "csrc"),
                            src, "-o", so], check=True)
        _emu = ctypes.CDLL(so)
        _emu.ace_emu_score.restype = ctypes.c_int
        _emu.ace_emu_kernel.restype = ctypes.c_int
    return _emu


def emu_score(tables, batch, memory_limit=None, strict=False, breakdown=False, ranges=None, defer=True):
    lib = emu_lib()
    ts = tables.as_struct()
    P = batch.n_plans
    codes = np.ascontiguousarray(batch.codes)
    hdr = np.ascontiguousarray(batch.hdr)
    it = np.zeros(P); pk = np.zeros(P)
    fe = np.zeros(P, dtype=np.uint8); st = np.zeros(P, dtype=np.uint8)
    rec = np.zeros((P, 1 if ranges is not None else 16, 18)) if (breakdown or ranges is not None) else None
    limit = tables.settings.memory_limit if memory_limit is None else memory_limit
    if ranges is not None:
        ranges = np.ascontiguousarray(ranges, dtype=np.uint32)
        breakdown = True
    rc = lib.ace_emu_score(ctypes.byref(ts), codes.ctypes.data_as(ctypes.c_void_p), hdr.ctypes.data_as(ctypes.c_void_p),
                           ranges.ctypes.data_as(ctypes.c_void_p) if ranges is not None else None, ctypes.c_longlong(P), ctypes.c_double(limit), ctypes.c_int(int(strict)), ctypes.c_int(int(defer)),
                           it.ctypes.data_as(ctypes.c_void_p), pk.ctypes.data_as(ctypes.c_void_p),
                           fe.ctypes.data_as(ctypes.c_void_p), st.ctypes.data_as(ctypes.c_void_p),
                           rec.ctypes.data_as(ctypes.c_void_p) if breakdown else None)
    assert rc == 0
    return it, pk, fe, st, rec


def kernel_layout(codes):
    """uint8 [P][N] -> [ceil(N / 16)][P][16], zero padded: the layout the scoring kernel reads."""
    P, N = codes.shape
    G = (N + 15) // 16
    out = np.zeros((P, G * 16), dtype=np.uint8)
    out[:, :N] = codes
    return np.ascontiguousarray(out.reshape(P, G, 16).transpose(1, 0, 2))


def emu_kernel_score(tables, batch, memory_limit=None, strict=False, breakdown=False, ranges=None, raw_codes=None, order=None):
    """The scoring kernel's own loop (csrc/ace_score_loop.h) on the CPU with guard pages behind every array:
    an out-of-range index ends the process with SIGSEGV, so call this from a child process.
    `raw_codes`: a [G][P][16] array to use as is (e.g. with junk in the padding bytes)."""
    lib = emu_lib()
    ts = tables.as_struct()
    P = batch.n_plans
    codes = kernel_layout(batch.codes) if raw_codes is None else np.ascontiguousarray(raw_codes)
    hdr = np.ascontiguousarray(batch.hdr)
    it = np.zeros(P); pk = np.zeros(P)
    fe = np.zeros(P, dtype=np.uint8); st = np.zeros(P, dtype=np.uint8)
    if ranges is not None:
        ranges = np.ascontiguousarray(ranges, dtype=np.uint32)
        breakdown = True
    rec = np.zeros((P, 1 if ranges is not None else 16, 18)) if breakdown else None
    limit = tables.settings.memory_limit if memory_limit is None else memory_limit
    vp = ctypes.c_void_p
    if order is not None:
        order = np.ascontiguousarray(order, dtype=np.uint32)
    rc = lib.ace_emu_kernel(ctypes.byref(ts), codes.ctypes.data_as(vp), hdr.ctypes.data_as(vp),
                            ranges.ctypes.data_as(vp) if ranges is not None else None,
                            order.ctypes.data_as(vp) if order is not None else None, ctypes.c_longlong(P),
                            ctypes.c_double(limit), ctypes.c_int(int(strict)), it.ctypes.data_as(vp), pk.ctypes.data_as(vp),
                            fe.ctypes.data_as(vp), st.ctypes.data_as(vp), rec.ctypes.data_as(vp) if breakdown else None)
    assert rc == 0
    return it, pk, fe, st, rec


def plan_arrays(batch, tables):
    """A PlanBatch as the plain arrays the C oracle takes: (num_stages, micro_bs, stage_len[P,16],
    tp_log, dp_log, algo, rc [P,N])."""
    codes, hdr = batch.codes, batch.hdr
    P, N = codes.shape
    A = tables.db.n_algo
    c = codes & 7
    tp_log, algo, rc = (c // A).astype(np.uint8), (c % A).astype(np.uint8), ((codes >> 3) & 1).astype(np.uint8)
    ns = ((codes >> 4) & 1).astype(np.int64)
    stage = np.cumsum(ns, axis=1) - 1
    S = (hdr[:, 0] & 0xff).astype(np.int32)
    micro_bs = np.asarray(tables.db.mbs_list, dtype=np.int32)[(hdr[:, 0] >> 8) & 0xff]
    gword = hdr[:, 1].astype(np.uint64) | (hdr[:, 2].astype(np.uint64) << np.uint64(32))
    glog = ((gword[:, None] >> (4 * np.clip(stage, 0, 15)).astype(np.uint64)) & np.uint64(15)).astype(np.int64)
    dp_log = (glog - tp_log).astype(np.uint8)
    stage_len = np.zeros((P, 16), dtype=np.int32)
    np.add.at(stage_len, (np.repeat(np.arange(P), N), np.clip(stage, 0, 15).ravel()), 1)
    return S, micro_bs, stage_len, tp_log, dp_log, algo, rc


_c_oracles = {}


def c_oracle_for(tables):
    """The C oracle loaded with exactly the data `tables` was compiled from (through the Python oracle)."""
    from oracle.c_oracle import COracle
    key = id(tables)
    if key not in _c_oracles:
        _c_oracles[key] = (COracle(oracle_for(tables), tables.graph.ops, tables.settings.global_batch_size), tables)
    return _c_oracles[key][0]


def c_oracle_scores(tables, batch, strict=False, threads=1, memory_limit=None, lists=False):
    return c_oracle_for(tables).score_arrays(*plan_arrays(batch, tables), strict=strict, threads=threads,
                                             memory_limit=memory_limit, lists=lists)


class EmuEvaluator:
    """Test double with PlanEvaluator.score_host's signature, backed by tests/emu."""

    def __init__(self, tables):
        self.tables = tables

    def score_host(self, batch, memory_limit=None, strict=False, breakdown=False, ranges=None):
        it, pk, fe, st, rec = emu_score(self.tables, batch, memory_limit, strict, breakdown, ranges)
        return (it, pk, fe, st, rec) if (breakdown or ranges is not None) else (it, pk, fe, st)

    def stage_records_host(self, batch, ranges):
        out = emu_score(self.tables, batch, None, False, True, ranges)
        return out[3], out[4][:, 0, :]

    def picked_records_host(self, batch, plan_idx, stage_idx):
        out = emu_score(self.tables, batch, None, False, True, None)
        return out[3], out[4][plan_idx, stage_idx]

    def close(self):
        pass


class EmuDeviceEvaluator(EmuEvaluator):
    """Test double for the device-resident calls of PlanEvaluator, on CPU tensors: `score` runs the kernel's
    own loop behind guard pages (tests/emu), `lib` offers ace_recompute_groups / ace_recompute_select from
    the host build of csrc/ace_edit_kernels.h.  A wrong index ends the process: use it in a child process."""

    def __init__(self, tables):
        import contextlib
        import types
        import torch
        super().__init__(tables)
        self._torch = torch
        self.device = torch.device("cpu")
        emu = emu_lib()
        vp = ctypes.c_void_p
        emu.ace_emu_rc_groups.restype = ctypes.c_int
        emu.ace_emu_rc_groups.argtypes = [vp, ctypes.c_int] + [vp] * 9
        emu.ace_emu_rc_select.restype = ctypes.c_int
        emu.ace_emu_rc_select.argtypes = [vp, vp, ctypes.c_int] + [vp] * 9 + [ctypes.c_double, vp, vp]
        self.lib = types.SimpleNamespace(ace_recompute_groups=lambda t, *a: emu.ace_emu_rc_groups(ctypes.cast(t, vp), *a),
                                         ace_recompute_select=lambda t, *a: emu.ace_emu_rc_select(ctypes.cast(t, vp), *a),
                                         ace_strerror=lambda code: b"emulation error")
        self.device_context = contextlib.nullcontext

    def _stream(self):
        return None

    def upload(self, batch, validate=True, ranges=None, staging=None):
        from superscaler_amd.evaluator import DeviceBatch
        return DeviceBatch(batch, "cpu", ranges)

    def score(self, dbatch, memory_limit=None, strict=False, breakdown=False, out=None):
        torch = self._torch
        from superscaler_amd.plan import PlanBatch
        P, N = dbatch.n_plans, dbatch.num_ops
        stub = PlanBatch(np.zeros((P, N), dtype=np.uint8), dbatch.hdr.numpy().view(np.uint32).copy())
        rg = dbatch.ranges.numpy().view(np.uint32) if dbatch.ranges is not None else None
        order = dbatch.order.numpy().view(np.uint32) if getattr(dbatch, "order", None) is not None else None
        it, pk, fe, st, rec = emu_kernel_score(self.tables, stub, memory_limit, strict, breakdown, rg,
                                               raw_codes=dbatch.codes.contiguous().numpy(), order=order)
        return (torch.from_numpy(it), torch.from_numpy(pk), torch.from_numpy(fe), torch.from_numpy(st),
                torch.from_numpy(rec) if rec is not None else None)



def odd_workloads():
    """Small workloads at the corners of the table geometry: one tp, one micro-batch size, 16 ops (one full
    group, no padding), six micro-batch sizes with deep pipelines (rows in windows), stages wider than a node,
    short ResNets with one row per op."""
    from superscaler_amd.synth import Workload
    return [
        Workload("gpt_1tp_1mbs", "gpt", 1, 256, 128, 0, [1], 1, 1, 8, 2000.0, [1], 32, 0.5, seed=1),
        Workload("gpt_16ops", "gpt", 1, 256, 128, 0, [1, 2], 2, 2, 8, 200.0, [1, 2], 64, 0.5, seed=2),
        Workload("gpt_wide_stages", "gpt", 2, 512, 256, 0, [2, 4], 8, 2, 64, 500.0, [1, 2, 4, 8], 64, 0.4, seed=3),
        Workload("gpt_6mbs_64gpus", "gpt", 1, 256, 128, 0, [1, 2, 4, 8, 16, 32], 64, 8, 128, 100.0, [1, 2, 4, 8, 16], 64, 0.6, seed=4),
        Workload("gpt_3tp", "gpt", 3, 256, 128, 0, [4], 4, 4, 16, 300.0, [1, 2, 4], 64, 0.2, seed=5),
        Workload("t5_1layer", "t5", 1, 256, 64, 32, [1, 2], 4, 4, 16, 300.0, [1, 2, 4], 64, 0.5, seed=6),
        Workload("t5_1tp", "t5", 2, 256, 64, 32, [8], 2, 1, 16, 300.0, [1, 2], 64, 0.5, seed=7),
        Workload("resnet_1111", "resnet", None, 32, 64, 0, [1, 2, 4], 4, 4, 32, 300.0, [1, 2, 4], 64, 0.5, conv=True,
                 resnet_blocks=(1, 1, 1, 1), seed=8),
        Workload("resnet_16gpus", "resnet", None, 32, 64, 0, [2], 16, 8, 32, 100.0, [1, 4, 16], 64, 0.5, conv=True,
                 resnet_blocks=(2, 1, 1, 2), seed=9),
        Workload("resnet_2tp", "resnet", None, 64, 64, 0, [1, 2, 4, 8], 8, 2, 64, 100.0, [1, 8], 64, 0.9, conv=True,
                 resnet_blocks=(1, 2, 3, 1), seed=10),
    ]
