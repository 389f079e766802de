"""The entry point that allocates nothing, mmsim_eval_batch_static, against mmsim_eval_batch.

Both are called through the C ABI on the same inputs; every result array must be identical (the two
share the packing code and the kernels, only the home of the device buffers differs).  Two calls in a
row, the second with a smaller input, so that what the first call left in the static scratch would
show if anything that must start at zero were not cleared.  Collected last (file name): a failure
here must not hide the other tests.
"""
import numpy as np
import pytest

from mms_amd import _lib, engine as E
from mms_amd.synthetic import make_config

pytestmark = pytest.mark.gpu


def _same(a, b, where):
    assert a.keys() == b.keys(), where
    for k in a:
        if a[k].dtype.kind == "f":
            assert np.array_equal(a[k].view(np.uint64), b[k].view(np.uint64)), f"{k} differs {where}"
        else:
            assert np.array_equal(a[k], b[k]), f"{k} differs {where}"


def _both(eng, dws, table, packed, flags, where):
    print(f"no-alloc entry point: {where}, flags {flags}", flush=True)
    got = E.eval_batch(eng, dws, table, packed, flags, static=True)
    ref = E.eval_batch(eng, dws, table, packed, flags, static=False)
    _same(got, ref, where)
    return got


def test_static_entry_point_equals_the_allocating_one_on_two_calls_in_a_row():
    eng = E.Engine.default()
    counts = _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS
    # first call: configuration 2, all 64 placements x 2 seeds, counts and per-request outputs
    cfg = make_config(2, 64)
    table = E.LatencyTable(cfg.profiles, cfg.batch_sizes)
    streams = [cfg.stream(s) for s in cfg.base_seeds[:2]]
    dws = [E.DeviceWorkload(eng, s.tstamps[:3000], s.model_ids[:3000], s.slos[:3000], cfg.num_models)
           for s in streams]
    big = _both(eng, dws, table, E.pack_placements(cfg.placements, table), counts | _lib.WANT_PER_REQUEST,
                "cfg 2, 64 placements x 2 seeds x 3000 requests")
    assert big["n_good"].sum() > 0
    # second call, smaller: 9 placements x 1 seed x a shorter stream, counts only, then scores only
    few = E.pack_placements(cfg.placements[5:14], table)
    dw1 = [E.DeviceWorkload(eng, streams[0].tstamps[:700], streams[0].model_ids[:700],
                            streams[0].slos[:700], cfg.num_models)]
    small = _both(eng, dw1, table, few, counts, "cfg 2, 9 placements x 1 seed x 700 requests")
    assert small["n_good"].sum() > 0
    _both(eng, dw1, table, few, 0, "scores only")
    # the batching simulator shares the scratch
    cfg5 = make_config(5, 24)
    t5 = E.LatencyTable(cfg5.profiles, cfg5.batch_sizes)
    s5 = cfg5.stream(0)
    dw5 = [E.DeviceWorkload(eng, s5.tstamps[:2000], s5.model_ids[:2000], s5.slos[:2000], cfg5.num_models)]
    _both(eng, dw5, t5, E.pack_placements(cfg5.placements, t5), _lib.BATCHING | counts, "cfg 5, 24 placements, batching")
    # and the first input again: same answer as before
    again = E.eval_batch(eng, dws, table, E.pack_placements(cfg.placements, table),
                         counts | _lib.WANT_PER_REQUEST, static=True)
    _same(again, big, "first input again")


def test_static_entry_point_refuses_what_does_not_fit():
    eng = E.Engine.default()
    cfg = make_config(2, 64)
    table = E.LatencyTable(cfg.profiles, cfg.batch_sizes)
    st = cfg.stream(0)
    dw = [E.DeviceWorkload(eng, st.tstamps, st.model_ids, st.slos, cfg.num_models)]
    packed = E.pack_placements(cfg.placements, table)
    # per-request outputs of 512 placements x 9.6k requests: 512 * 9600 * 9 bytes = 44 MB, beyond the scratch
    with pytest.raises(_lib.MmsimError) as err:
        E.eval_batch(eng, dw, table, E.pack_placements(cfg.placements * 8, table), _lib.WANT_PER_REQUEST, static=True)
    assert err.value.code == _lib.E_NOMEM and str(_lib.STATIC_SCRATCH_BYTES) in str(err.value)
    # the scratch is usable afterwards
    got = E.eval_batch(eng, dw, table, packed, 0, static=True)
    ref = E.eval_batch(eng, dw, table, packed, 0, static=False)
    _same(got, ref, "after a refusal")
