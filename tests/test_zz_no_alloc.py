"""ace_score_batch_static -- the scoring entry point that allocates nothing -- against ace_score_batch, through the
C ABI: two calls in a row, the second on a smaller batch, must both give ace_score_batch's bytes (the static
scratch keeps the first call's records); too large a batch is refused.  Collected last by name."""
import ctypes

import numpy as np
import pytest

from superscaler_amd import synth

pytestmark = pytest.mark.gpu


def _outputs(ev, torch, P):
    return (torch.full((P,), -1.0, dtype=torch.float64, device=ev.device), torch.full((P,), -1.0, dtype=torch.float64, device=ev.device),
            torch.full((P,), 9, dtype=torch.uint8, device=ev.device), torch.full((P,), 9, dtype=torch.uint8, device=ev.device))


def _raw_call(ev, torch, entry, d, limit, outs):
    it, pk, fe, st = outs
    stream = ctypes.c_void_p(torch.cuda.current_stream(ev.device).cuda_stream)
    with ev.device_context():
        if entry == "static":
            rc = ev.lib.ace_score_batch_static(ev.handle, ctypes.byref(d.struct), limit, 0, it.data_ptr(), pk.data_ptr(),
                                               fe.data_ptr(), st.data_ptr(), stream)
        else:
            rc = ev.lib.ace_score_batch(ev.handle, ctypes.byref(d.struct), limit, 0, it.data_ptr(), pk.data_ptr(),
                                        fe.data_ptr(), st.data_ptr(), None, stream)
    assert rc == 0, ev.lib.ace_strerror(rc)
    torch.cuda.synchronize()


def _raw_scores(ev, torch, entry, d, limit):
    outs = _outputs(ev, torch, d.n_plans)
    _raw_call(ev, torch, entry, d, limit, outs)
    return [t.cpu().numpy() for t in outs]


@pytest.mark.parametrize("name,sizes", [("gpt3_13b", (16384, 5000)), ("gpt3_1_3b", (3000, 64)), ("wresnet_1b", (2048, 700))])
def test_static_entry_point_equals_score_batch(name, sizes):
    import torch
    from superscaler_amd.evaluator import PlanEvaluator
    w = synth.WORKLOADS[name]
    tables = synth.make_tables(w)
    limit = float(tables.settings.memory_limit)
    ev = PlanEvaluator(tables)          # the handle the static entry point is called on: ace_score_batch never runs on it
    ref = PlanEvaluator(tables)         # a second handle, for what ace_score_batch returns
    try:
        batches = [synth.make_plans(w, tables, n_plans=n, seed_offset=40 + k) for k, n in enumerate(sizes)]
        dev = [ev.upload(b) for b in batches]
        want = [_raw_scores(ref, torch, "plain", ref.upload(b), limit) for b in batches]
        # the handle has no workspace of its own and may not get one: a call that allocated would fail with ACE_EFIXED
        with ev.device_context():
            assert ev.lib.ace_reserve(ev.handle, 0, 1) == 0
        outs = [_outputs(ev, torch, d.n_plans) for d in dev]
        torch.cuda.synchronize()
        free0 = torch.cuda.mem_get_info()[0]
        for d, o in zip(dev, outs):                                              # two calls in a row, the second smaller
            _raw_call(ev, torch, "static", d, limit, o)
        # outputs were allocated beforehand: the device's free memory is what it was
        assert torch.cuda.mem_get_info()[0] == free0
        got = [[t.cpu().numpy() for t in o] for o in outs]
        for g, x in zip(got, want):
            for a, b in zip(g, x):
                assert np.array_equal(a, b, equal_nan=True)
        assert got[0][2].any() and (got[0][3] == 0).all()
        # the second call again after the first (records of the larger batch are still in the scratch)
        again = _raw_scores(ev, torch, "static", dev[1], limit)
        assert all(np.array_equal(a, b, equal_nan=True) for a, b in zip(again, want[1]))
        # the plain entry point on this handle would have to allocate its workspace now: refused, as fixed above
        o = _outputs(ev, torch, dev[0].n_plans)
        with ev.device_context():
            rc = ev.lib.ace_score_batch(ev.handle, ctypes.byref(dev[0].struct), limit, 0, o[0].data_ptr(), o[1].data_ptr(),
                                        o[2].data_ptr(), o[3].data_ptr(), None, None)
        assert rc == -6, rc
        # beyond the stated maximum: refused, nothing launched
        big = ev.upload(synth.make_plans(w, tables, n_plans=16385, seed_offset=44))
        it = torch.zeros(16385, dtype=torch.float64, device=ev.device)
        fe = torch.zeros(16385, dtype=torch.uint8, device=ev.device)
        with ev.device_context():
            rc = ev.lib.ace_score_batch_static(ev.handle, ctypes.byref(big.struct), limit, 0, it.data_ptr(), it.data_ptr(),
                                               fe.data_ptr(), None, None)
        assert rc == -2 and ev.lib.ace_strerror(rc)
    finally:
        ev.close()
        ref.close()
