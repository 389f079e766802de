"""Shared helpers of the parity tests: run the same packed inputs through the
CPU oracle and through libmmsim and compare to the bar (bit-exact counts,
flags and finish times; latency sums to 1e-12 relative)."""
import numpy as np

from oracle import oracle_c


def oracle_batch(stream, table, packed, batching=False, want_per_request=False):
    """CPU oracle on one stream for every placement of a packed batch."""
    lat, pp = table.arrays()
    num_groups, group_cfg, gm_off, gm_idx = packed
    return oracle_c.eval_placements(
        stream.tstamps, stream.model_ids, stream.slos, lat, pp, table.batch_sizes, num_groups,
        group_cfg, gm_off, gm_idx, batching=batching, want_counts=True,
        want_per_request=want_per_request)


def assert_batch_matches(gpu, ref, seed_index, num_groups, per_request=False, where=""):
    """gpu: dict from engine.Batch.fetch() ([n_seeds][B][...]); ref: oracle dict ([B][...])."""
    s = seed_index
    assert np.array_equal(gpu["n_good"][s], ref["n_good"]), f"n_good differs {where}"
    if "model_num_good" in gpu:
        assert np.array_equal(gpu["model_num_requests"][s], ref["model_num_requests"]), f"model_num_requests {where}"
        assert np.array_equal(gpu["model_num_good"][s], ref["model_num_good"]), f"model_num_good {where}"
    if "group_num_requests" in gpu:
        assert np.array_equal(gpu["group_num_requests"][s], ref["group_num_requests"]), f"group_num_requests {where}"
        assert np.array_equal(gpu["group_num_good"][s], ref["group_num_good"]), f"group_num_good {where}"
    if per_request:
        R = ref["finish"].shape[1]
        assert np.array_equal(gpu["good"][s][:, :R], ref["good"]), f"good flags differ {where}"
        # bar: 1e-12 relative; the arithmetic is the same fp64 sequence, so demand identical bits
        assert np.array_equal(gpu["finish"][s][:, :R].view(np.uint64), ref["finish"].view(np.uint64)), \
            f"finish differs {where}"
    # streaming fp64 sum in arrival order on both sides -> identical
    assert np.array_equal(gpu["latency_sum"][s], ref["latency_sum"]), f"latency_sum differs {where}"
