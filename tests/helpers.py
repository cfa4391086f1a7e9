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
                 peak_mem_in_backward=st.peak_mem_in_backward, memory_pred_type=st.memory_pred_type)
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
        hdr = os.path.join(ROOT, "superscaler_amd", "csrc", "ace_plan_state.h")
        if (not os.path.exists(so)) or os.path.getmtime(so) < max(os.path.getmtime(src), os.path.getmtime(hdr)):
            subprocess.run(["g++", "-O2", "-std=c++17", "-ffp-contract=off", "-shared", "-fPIC",
                            "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROOT, "superscaler_amd", "csrc"),
                            src, "-o", so], check=True)
        _emu = ctypes.CDLL(so)
        _emu.ace_emu_score.restype = ctypes.c_int
    return _emu


def emu_score(tables, batch, memory_limit=None, strict=False, breakdown=False, ranges=None, defer=True):
    lib = emu_lib()
    ts = tables.as_struct()
    P = batch.n_plans
    codes = np.ascontiguousarray(batch.codes)
    hdr = np.ascontiguousarray(batch.hdr)
    it = np.zeros(P); pk = np.zeros(P)
    fe = np.zeros(P, dtype=np.uint8); st = np.zeros(P, dtype=np.uint8)
    rec = np.zeros((P, 16, 18)) if (breakdown or ranges is not None) else None
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
