"""Inputs beyond the limits of the compiled kernels (MMSIM_MAX_* in include/mmsim.h) and the one
input the batching kernel does not simulate: every one is refused with an error code and a message,
or reported in status[], and the context works afterwards.  No kernel is launched for a refused batch."""
import numpy as np
import pytest

from mms_amd import _lib, engine as E
from mms_amd.placement_policy.base_policy import ModelPlacement
from mms_amd.profiling import ParallelConfig, synthetic_profile
from oracle import oracle_c

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def eng():
    return E.Engine.default()


def _stream(M, R=200, seed=0):
    rng = np.random.default_rng(seed)
    return (np.cumsum(rng.exponential(0.01, R)), rng.integers(0, M, R).astype(np.int32),
            np.full(R, 1.0, np.float32))


def _refused(eng, profiles, sols, code, text, flags=0, batch_sizes=(1,), M=None, extra_configs=()):
    M = len(profiles) if M is None else M
    table = E.LatencyTable(profiles, list(batch_sizes))
    for c in extra_configs:
        table.config_id(c)
    dw = E.DeviceWorkload(eng, *_stream(M), M)
    with pytest.raises(_lib.MmsimError) as err:
        E.Batch(eng, [dw], table, E.pack_placements(sols, table), flags)
    assert err.value.code == code, str(err.value)
    assert text in str(err.value), str(err.value)
    dw.close()


def _still_works(eng):
    pcs = [ParallelConfig(1, 1, 2)]
    profiles = [synthetic_profile(f"m{m}", 0.1, pcs) for m in range(2)]
    table = E.LatencyTable(profiles, [1])
    sols = [ModelPlacement(pcs, [[0, 1]])]
    t, m, s = _stream(2)
    dw = E.DeviceWorkload(eng, t, m, s, 2)
    out = E.evaluate(eng, [dw], table, sols, 0)
    lat, pp = table.arrays()
    ref = oracle_c.eval_placements(t, m, s, lat, pp, [1], *E.pack_placements(sols, table), want_counts=True)
    assert np.array_equal(out["n_good"][0], ref["n_good"])
    dw.close()


def test_more_than_32_stages(eng):
    pcs = [ParallelConfig(1, 1, 33)]
    profiles = [synthetic_profile("m0", 0.1, pcs)]
    _refused(eng, profiles, [ModelPlacement(pcs, [[0]])], _lib.E_UNSUPPORTED, "more than 32 pipeline stages")
    _still_works(eng)


def test_more_than_64_replicas_of_a_model(eng):
    pc = ParallelConfig(1, 1, 1)
    profiles = [synthetic_profile(f"m{m}", 0.1, [pc]) for m in range(2)]
    ok = ModelPlacement([pc] * 64, [[0]] * 64)                   # 64 replicas are simulated
    table = E.LatencyTable(profiles, [1])
    t, m, s = _stream(2)
    dw = E.DeviceWorkload(eng, t, m, s, 2)
    flags = _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS
    out = E.evaluate(eng, [dw], table, [ok], flags)
    lat, pp = table.arrays()
    ref = oracle_c.eval_placements(t, m, s, lat, pp, [1], *E.pack_placements([ok], table), want_counts=True)
    assert np.array_equal(out["n_good"][0], ref["n_good"])
    assert np.array_equal(out["group_num_requests"][0], ref["group_num_requests"])
    dw.close()
    _refused(eng, profiles, [ModelPlacement([pc] * 65, [[0]] * 65)], _lib.E_UNSUPPORTED, "more than 64 replicas")


def test_more_than_254_groups(eng):
    pc = ParallelConfig(1, 1, 1)
    profiles = [synthetic_profile(f"m{m}", 0.1, [pc]) for m in range(8)]
    rows = [[g % 8] for g in range(255)]
    _refused(eng, profiles, [ModelPlacement([pc] * 255, rows)], _lib.E_UNSUPPORTED, "more than 254 groups")


def test_more_than_255_clock_slots(eng):
    pc = ParallelConfig(1, 1, 16)
    profiles = [synthetic_profile(f"m{m}", 0.1, [pc]) for m in range(16)]
    _refused(eng, profiles, [ModelPlacement([pc] * 16, [[g] for g in range(16)])], _lib.E_UNSUPPORTED,
             "more than 255 pipeline stages in total")


def test_more_than_255_configurations(eng):
    pcs = [ParallelConfig(1, op, 1) for op in range(1, 257)]
    profiles = [synthetic_profile("m0", 0.1, pcs[:1])]
    _refused(eng, profiles, [ModelPlacement(pcs[:1], [[0]])], _lib.E_UNSUPPORTED,
             "more than 255 parallel configurations", extra_configs=pcs)


def test_latency_rows_longer_than_the_descriptor_can_index(eng):
    pcs = [ParallelConfig(1, op, 32) for op in range(1, 34)]        # 33 configurations x 32 stages > 1022 entries
    profiles = [synthetic_profile("m0", 0.1, pcs)]
    # (per-stage latencies must differ, or the table shrinks to one entry per configuration)
    profiles[0].para_dict[pcs[0]].latency[1][0] *= 2
    _refused(eng, profiles, [ModelPlacement(pcs[:1], [[0]])], _lib.E_UNSUPPORTED,
             "more than 1022 pipeline stages in total", extra_configs=pcs)


def test_more_than_16_batch_sizes_and_sizes_without_a_latency_column(eng):
    pc = ParallelConfig(1, 1, 1)
    sizes = [1 << k for k in range(17)]
    profiles = [synthetic_profile("m0", 0.1, [pc], batch_sizes=sizes)]
    _refused(eng, profiles, [ModelPlacement([pc], [[0]])], _lib.E_UNSUPPORTED, "more than 16 batch sizes",
             flags=_lib.BATCHING, batch_sizes=sizes)
    # the latency column of a size is floor(log2(size)) (controller.py:668): 8 needs column 3 of a 2-column table
    profiles = [synthetic_profile("m0", 0.1, [pc], batch_sizes=[1, 8])]
    _refused(eng, profiles, [ModelPlacement([pc], [[0]])], _lib.E_INVALID, "must index a latency column",
             flags=_lib.BATCHING, batch_sizes=[1, 8])
    _still_works(eng)


def test_state_that_does_not_fit_in_lds(eng):
    """Per-wavefront state grows with models (replica bounds, queue heads) and clock slots; beyond the CU's LDS
    the batch is refused."""
    pc = ParallelConfig(1, 1, 15)
    M = 60000
    prof = synthetic_profile("m", 0.1, [pc])
    table = E.LatencyTable([prof] * M, [1])
    sols = [ModelPlacement([pc] * 17, [[g] for g in range(17)])]      # 255 clock slots x 512 bytes + M bytes of bounds
    dw = E.DeviceWorkload(eng, *_stream(M), M)
    for flags, text in ((0, "does not fit in LDS"), (_lib.BATCHING, "does not fit in LDS")):
        with pytest.raises(_lib.MmsimError) as err:
            E.Batch(eng, [dw], table, E.pack_placements(sols, table), flags)
        assert err.value.code == _lib.E_UNSUPPORTED and text in str(err.value), str(err.value)
    dw.close()
    _still_works(eng)


def test_more_items_than_one_workgroup_can_own(eng, opts):
    """The scheduled launch gives a workgroup at most 256 (tile, stream) items; forced to one workgroup, 257 tiles
    are refused (and run fine with the workgroups the library would choose)."""
    pc = ParallelConfig(1, 1, 1)
    profiles = [synthetic_profile(f"m{m}", 0.1, [pc]) for m in range(2)]
    sols = [ModelPlacement([pc], [[b % 2]]) for b in range(257 * 64)]
    opts(request_loop=1, sched_groups=1)
    _refused(eng, profiles, sols, _lib.E_UNSUPPORTED, "too many (tile, stream) pairs")
    opts(request_loop=1, sched_groups=0)
    table = E.LatencyTable(profiles, [1])
    t, m, s = _stream(2, R=300)
    dw = E.DeviceWorkload(eng, t, m, s, 2)
    out = E.evaluate(eng, [dw], table, sols, 0)
    lat, pp = table.arrays()
    ref = oracle_c.eval_placements(t, m, s, lat, pp, [1], *E.pack_placements(sols[:2], table), want_counts=True)
    assert np.array_equal(out["n_good"][0][:2], ref["n_good"]) and np.array_equal(out["n_good"][0][2:4], ref["n_good"])
    dw.close()


def test_options_are_validated(eng):
    for bad in (dict(request_loop=2), dict(waves_per_cu=9), dict(batching_lanes=12), dict(segment_requests=-5),
                dict(batching_lds_tables=4)):
        with pytest.raises(_lib.MmsimError) as err:
            eng.set_options(**bad)
        assert err.value.code == _lib.E_INVALID and "options" in str(err.value)
    eng.set_options()
    with pytest.raises(TypeError):
        eng.set_options(no_such_field=1)
    _still_works(eng)


def test_a_simulation_whose_replica_clocks_are_all_infinite_is_reported(eng):
    """Batching simulator: a model whose only replica has an infinite latency (no profile for the group's
    configuration) is accepted once under an infinite SLO, after which the group's clock is infinite and the next
    request of the model finds no replica to choose.  The reference then indexes its arrays with -1
    (controller.py:760-778); here that simulation is marked MMSIM_E_UNSUPPORTED in status[], the others of the batch
    are unaffected, and the kernel ends normally."""
    pa, pb = ParallelConfig(1, 1, 1), ParallelConfig(1, 1, 2)
    sizes = [1, 2]
    profiles = [synthetic_profile("m0", 0.1, [pb], batch_sizes=sizes),          # model 0 has no profile for pa
                synthetic_profile("m1", 0.1, [pa, pb], batch_sizes=sizes)]
    table = E.LatencyTable(profiles, sizes)
    sols = [ModelPlacement([pb], [[0, 1]]), ModelPlacement([pa, pb], [[0, 1], [1]]), ModelPlacement([pa], [[1]])]
    packed = E.pack_placements(sols, table)
    R = 120
    t = np.arange(R) * 0.05
    m = (np.arange(R) % 2).astype(np.int32)
    s = np.full(R, np.inf, np.float32)
    dw = E.DeviceWorkload(eng, t, m, s, 2)
    flags = _lib.BATCHING | _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS
    batch = E.Batch(eng, [dw], table, packed, flags)
    batch.run()
    batch.sync()
    with pytest.raises(_lib.MmsimError) as err:       # by default a failed simulation is an error that names it
        batch.fetch()
    assert err.value.code == _lib.E_UNSUPPORTED and "(0, 1)" in str(err.value)
    out = batch.fetch(allow_failed=True)
    batch.close()
    assert list(out["status"][0]) == [0, _lib.E_UNSUPPORTED, 0]
    lat, pp = table.arrays()
    for b in (0, 2):                                  # the healthy simulations of the batch equal the oracle's
        one = E.pack_placements([sols[b]], table)
        ref = oracle_c.eval_placements(t, m, s, lat, pp, sizes, *one, batching=True, want_counts=True)
        assert out["n_good"][0, b] == ref["n_good"][0]
        assert np.array_equal(out["model_num_good"][0, b], ref["model_num_good"][0])
        g = len(sols[b].group_configs)
        assert np.array_equal(out["group_num_requests"][0, b][:g], ref["group_num_requests"][0][:g])
    # the single-placement entry point has no status array: the call fails with the code
    m2g = np.array([[0], [-1]], np.int32)
    g2m = np.array([[0, -1]], np.int32)
    lat1 = np.full((2, 1, 1, 2), np.inf, np.float32)
    fin, good = np.zeros(R), np.zeros(R, bool)
    with pytest.raises(_lib.MmsimError) as err:
        E.simulate_requests_mixed_batching(eng, fin, good, t, np.zeros(R, np.int32), s, m2g, g2m,
                                           np.ones(1, np.int32), lat1, sizes)
    assert err.value.code == _lib.E_UNSUPPORTED
    dw.close()
    _still_works(eng)
