"""Size-independent properties of the plain simulator at the headline configuration's full
placement count (16384 candidates of configuration 4, one arrival seed, ~1M requests each):
results must not depend on where a placement sits in the batch, on what shares its wavefront,
or on how often the batch is run; counts must be consistent with each other."""
import numpy as np
import pytest

from mms_amd import _lib, engine as E
from mms_amd.synthetic import make_config

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def eng():
    return E.Engine.default()


def _scores(eng, cfg, table, dw, sols, flags=0):
    batch = E.Batch(eng, [dw], table, E.pack_placements(sols, table), flags)
    batch.run()
    batch.sync()
    out = batch.fetch()
    batch.close()
    return out


def test_full_size_position_independence_and_consistency(eng):
    cfg = make_config(4)
    st = cfg.stream(0)
    table = E.LatencyTable(cfg.profiles, cfg.batch_sizes)
    dw = E.DeviceWorkload(eng, st.tstamps, st.model_ids, st.slos, cfg.num_models)
    sols = cfg.placements
    B = len(sols)
    assert B == 16384
    base = _scores(eng, cfg, table, dw, sols)

    # 1. any permutation of the candidate list gives every placement the same result
    perm = np.random.default_rng(5).permutation(B)
    shuffled = _scores(eng, cfg, table, dw, [sols[i] for i in perm])
    assert np.array_equal(shuffled["n_good"][0], base["n_good"][0][perm])
    assert np.array_equal(shuffled["latency_sum"][0], base["latency_sum"][0][perm])

    # 2. a placement evaluated in a small batch (other wavefront mates, other LDS layout) agrees
    pick = perm[:200]
    small = _scores(eng, cfg, table, dw, [sols[i] for i in pick])
    assert np.array_equal(small["n_good"][0], base["n_good"][0][pick])
    assert np.array_equal(small["latency_sum"][0], base["latency_sum"][0][pick])

    # 3. counts are consistent: goodput = sum of per-model goods = sum of per-group goods, and every
    #    request of a hosted model is dispatched to exactly one group (a subset, all outputs on)
    sub = [sols[i] for i in pick[:128]]
    full = _scores(eng, cfg, table, dw, sub, _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS)
    assert np.array_equal(full["n_good"][0], base["n_good"][0][pick[:128]])
    assert np.array_equal(full["model_num_good"][0].sum(axis=1), full["n_good"][0])
    assert np.array_equal(full["group_num_good"][0].sum(axis=1), full["n_good"][0])
    per_model = np.bincount(st.model_ids[st.model_ids >= 0], minlength=cfg.num_models)
    for k, pl in enumerate(sub):
        hosted = np.zeros(cfg.num_models, bool)
        for ms in pl.group_models:
            hosted[list(ms)] = True
        assert full["group_num_requests"][0][k].sum() == per_model[hosted].sum()
        assert np.all(full["model_num_good"][0][k][~hosted] == 0)
    assert np.all(full["n_good"][0] <= len(st.tstamps))

    # 4. with an infinite SLO nothing hosted is dropped
    inf_dw = E.DeviceWorkload(eng, st.tstamps, st.model_ids, np.full(len(st.slos), np.inf, np.float32), cfg.num_models)
    lax = _scores(eng, cfg, table, inf_dw, sub)
    for k, pl in enumerate(sub):
        hosted = np.zeros(cfg.num_models, bool)
        for ms in pl.group_models:
            hosted[list(ms)] = True
        assert lax["n_good"][0][k] == per_model[hosted].sum()
