"""ace_score_batch_static -- the scoring entry point that allocates nothing -- against ace_score_batch, through the
C ABI: two calls in a row, the second on a smaller batch, must both give ace_score_batch's bytes (the static
scratch keeps the first call's records); too large a batch is refused.  Collected last by name."""
import ctypes

import numpy as np
import pytest

from superscaler_amd import synth

pytestmark = pytest.mark.gpu


def _raw_scores(ev, torch, entry, d, limit):
    P = d.n_plans
    it = torch.full((P,), -1.0, dtype=torch.float64, device=ev.device)
    pk = torch.full((P,), -1.0, dtype=torch.float64, device=ev.device)
    fe = torch.full((P,), 9, dtype=torch.uint8, device=ev.device)
    st = torch.full((P,), 9, dtype=torch.uint8, device=ev.device)
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
    return [t.cpu().numpy() for t in (it, pk, fe, st)]


@pytest.mark.parametrize("name,sizes", [("gpt3_13b", (16384, 5000)), ("gpt3_1_3b", (3000, 64)), ("wresnet_1b", (2048, 700))])
def test_static_entry_point_equals_score_batch(name, sizes):
    import torch
    from superscaler_amd.evaluator import PlanEvaluator
    w = synth.WORKLOADS[name]
    tables = synth.make_tables(w)
    limit = float(tables.settings.memory_limit)
    ev = PlanEvaluator(tables)
    try:
        batches = [synth.make_plans(w, tables, n_plans=n, seed_offset=40 + k) for k, n in enumerate(sizes)]
        dev = [ev.upload(b) for b in batches]
        want = [_raw_scores(ev, torch, "plain", d, limit) for d in dev]
        free0 = torch.cuda.mem_get_info()[0]
        got = [_raw_scores(ev, torch, "static", d, limit) for d in dev]          # two calls in a row, the second smaller
        for g, x in zip(got, want):
            for a, b in zip(g, x):
                assert np.array_equal(a, b, equal_nan=True)
        assert got[0][2].any() and (got[0][3] == 0).all()
        # the second call again after the first (records of the larger batch are still in the scratch)
        again = _raw_scores(ev, torch, "static", dev[1], limit)
        assert all(np.array_equal(a, b, equal_nan=True) for a, b in zip(again, want[1]))
        # (outputs of _raw_scores are the only tensors made in between: at most a few MiB of cached blocks)
        assert free0 - torch.cuda.mem_get_info()[0] < (8 << 20)
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
