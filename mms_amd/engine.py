"""Python side of the C ABI: packs placements and profiles into the flat
arrays ``libmmsim`` takes and turns its results back into numpy arrays.

The packing is the batched form of the reference's per-placement table build
(``approximate_one_case_one_placement``, alpa_serve/simulator/controller.py:
412-476).  That code fills ``stage_latency[model][group][stage]`` for every
placement; the value depends only on the group's ParallelConfig, so here a
latency table is built once per distinct ParallelConfig (``LatencyTable``) and a
placement is reduced to "which config does each group use, which models does
it host".
"""
import ctypes as C
from contextlib import contextmanager
from itertools import chain
from typing import List, Sequence

import numpy as np

from mms_amd import _lib
from mms_amd.util import FIXED_OVERHEAD, STAGE_PENALTY


class Engine:
    """One libmmsim context (one GPU, one stream)."""

    _default = None

    def __init__(self, device: int = 0):
        self.lib = _lib.load()
        self._h = C.c_void_p()
        _lib.check(self.lib.mmsim_ctx_create(device, C.byref(self._h)))
        self.device = device

    @classmethod
    def default(cls):
        if cls._default is None:
            cls._default = cls(0)
        return cls._default

    def device_info(self):
        info = _lib.DeviceInfo()
        _lib.check(self.lib.mmsim_ctx_device_info(self._h, C.byref(info)))
        return {"name": info.name.decode(), "arch": info.arch.decode(),
                "compute_units": info.compute_units, "clock_khz": info.clock_khz,
                "lds_bytes_per_block": info.lds_bytes_per_block, "hbm_bytes": info.hbm_bytes}

    def make_options(self, **fields):
        """An ``mmsim_options`` with the library's defaults and ``fields`` changed."""
        opt = _lib.Options()
        self.lib.mmsim_options_default(C.byref(opt))
        names = {f[0] for f in _lib.Options._fields_} - {"struct_size", "reserved"}
        for k, v in fields.items():
            if k not in names:
                raise TypeError(f"mmsim_options has no field {k!r}")
            setattr(opt, k, int(v))
        return opt

    def set_options(self, **fields):
        """Options of every batch this context makes from now on (``mmsim_ctx_set_options``);
        without arguments: the defaults."""
        opt = self.make_options(**fields)
        _lib.check(self.lib.mmsim_ctx_set_options(self._h, C.byref(opt)))
        self._options = dict(fields)

    @contextmanager
    def options(self, **fields):
        """``with engine.options(request_loop=1): ...`` -- the fields on top of what is set now, put back afterwards."""
        before = dict(getattr(self, "_options", {}))
        self.set_options(**{**before, **fields})
        try:
            yield self
        finally:
            self.set_options(**before)

    def close(self):
        if self._h:
            self.lib.mmsim_ctx_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class DeviceWorkload:
    """A request stream resident in HBM (arrivals f64, model ids i32, SLOs f32)."""

    def __init__(self, engine: Engine, tstamps, model_ids, slos, num_models: int):
        self.engine = engine
        ts = _lib.carray(tstamps, np.float64)
        mid = _lib.carray(model_ids, np.int32)
        sl = _lib.carray(slos, np.float32)
        assert len(ts) == len(mid) == len(sl)
        self.R = len(ts)
        self.M = int(num_models)
        self._h = C.c_void_p()
        _lib.check(engine.lib.mmsim_workload_create(
            engine._h, self.R, self.M, _lib.ptr(ts, C.c_double), _lib.ptr(mid, C.c_int32),
            _lib.ptr(sl, C.c_float), C.byref(self._h)))

    def close(self):
        if self._h:
            self.engine.lib.mmsim_workload_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class LatencyTable:
    """cfg_lat[M][C][Smax][NB] float32 for a growing set of ParallelConfigs.

    Entry values follow controller.py:456-459 / :472-474 exactly: the Python
    float product ``latency[bs][k] * (1 + 0.009 * len(latency[1]))`` rounded to
    float32 on store; a config a model has no profile for gives +inf
    (:461, :476).
    """

    def __init__(self, prof_ress: Sequence, batch_sizes: Sequence[int] = (1,)):
        self.prof_ress = list(prof_ress)
        self.batch_sizes = [int(b) for b in batch_sizes]
        assert self.batch_sizes[0] == 1
        self.configs = []
        self.index = {}
        self._arrays = None

    def config_id(self, cfg) -> int:
        i = self.index.get(cfg)
        if i is None:
            i = self.index[cfg] = len(self.configs)
            self.configs.append(cfg)
            self._arrays = None
        return i

    def arrays(self):
        if self._arrays is None:
            M, Cn, NB = len(self.prof_ress), max(len(self.configs), 1), len(self.batch_sizes)
            smax = max([int(c.pp) for c in self.configs] or [1])
            lat = np.zeros((M, Cn, smax, NB), np.float32)
            pp = np.ones(Cn, np.int32)
            with np.errstate(over="ignore"):
                for c, cfg in enumerate(self.configs):
                    pp[c] = cfg.pp
                    for m, prof in enumerate(self.prof_ress):
                        entry = prof.para_dict.get(cfg, None)
                        if not entry:
                            lat[m, c] = np.inf
                            continue
                        scale = 1 + STAGE_PENALTY * len(entry.latency[1])
                        for k in range(cfg.pp):
                            for b, bs in enumerate(self.batch_sizes):
                                lat[m, c, k, b] = entry.latency[bs][k] * scale
            self._arrays = (lat, pp)
        return self._arrays


def pack_placements(sols: Sequence, table: LatencyTable):
    """ModelPlacement list -> (num_groups[B], group_cfg[B][Gmax], gm_off[B][Gmax+1], gm_idx)."""
    B = len(sols)
    num_groups = np.fromiter((len(s.group_configs) for s in sols), np.int32, B)
    Gmax = max(int(num_groups.max()) if B else 1, 1)
    # two flat passes over all groups of all placements, scattered into the padded [B][Gmax] arrays row by row
    total_groups = int(num_groups.sum()) if B else 0
    has = np.arange(Gmax)[None, :] < num_groups[:, None]
    group_cfg = np.zeros((B, Gmax), np.int32)
    sizes = np.zeros((B, Gmax), np.int64)
    group_cfg[has] = np.fromiter(map(table.config_id, chain.from_iterable(s.group_configs for s in sols)),
                                 np.int32, total_groups)
    sizes[has] = np.fromiter(map(len, chain.from_iterable(s.group_models for s in sols)), np.int64, total_groups)
    gm_off = np.zeros((B, Gmax + 1), np.int64)
    np.cumsum(sizes, axis=1, out=gm_off[:, 1:])
    per_sol = gm_off[:, -1].copy()
    base = np.zeros(B, np.int64)
    np.cumsum(per_sol[:-1], out=base[1:])
    gm_off += base[:, None]
    total = int(per_sol.sum())
    gm_idx = np.fromiter(chain.from_iterable(chain.from_iterable(s.group_models) for s in sols),
                         np.int32, total)
    return num_groups, group_cfg, gm_off, gm_idx


def _result_arrays(flags, n_seeds, B, M, Gmax, Rmax):
    """Caller-owned result arrays for L = n_seeds * B simulations and the mmsim_result that points at them."""
    L = B * n_seeds
    out = {"n_good": np.zeros(L, np.int64), "latency_sum": np.zeros(L, np.float64),
           "status": np.zeros(L, np.int32)}
    r = _lib.Result()
    r.n_good = _lib.ptr(out["n_good"], C.c_int64)
    r.latency_sum = _lib.ptr(out["latency_sum"], C.c_double)
    r.status = _lib.ptr(out["status"], C.c_int32)
    if flags & _lib.WANT_MODEL_COUNTS:
        out["model_num_requests"] = np.zeros((L, M), np.int32)
        out["model_num_good"] = np.zeros((L, M), np.int32)
        r.model_num_requests = _lib.ptr(out["model_num_requests"], C.c_int32)
        r.model_num_good = _lib.ptr(out["model_num_good"], C.c_int32)
    if flags & _lib.WANT_GROUP_COUNTS:
        out["group_num_requests"] = np.zeros((L, Gmax), np.int32)
        out["group_num_good"] = np.zeros((L, Gmax), np.int32)
        r.group_num_requests = _lib.ptr(out["group_num_requests"], C.c_int32)
        r.group_num_good = _lib.ptr(out["group_num_good"], C.c_int32)
    if flags & _lib.WANT_PER_REQUEST:
        out["finish"] = np.zeros((L, Rmax), np.float64)
        out["good"] = np.zeros((L, Rmax), np.uint8)
        r.finish = _lib.ptr(out["finish"], C.c_double)
        r.good = _lib.ptr(out["good"], C.c_uint8)
    if flags & _lib.WANT_OP_COUNT:
        out["fp_ops"] = np.zeros(L, np.int64)
        r.fp_ops = _lib.ptr(out["fp_ops"], C.c_int64)
    return out, r


def check_status(status, what="simulation"):
    """Raises ``MmsimError`` when a simulation's ``status`` is not 0: such a simulation ran out of idle-event
    slots (``E_OVERFLOW``) or met an input the batching simulator does not support (``E_UNSUPPORTED``), and its
    counts and per-request outputs are partly unwritten."""
    status = np.asarray(status)
    bad = np.flatnonzero(status.reshape(-1) != 0)
    if bad.size:
        code = int(status.reshape(-1)[bad[0]])
        names = ", ".join(str(tuple(int(x) for x in np.unravel_index(i, status.shape))) for i in bad[:8])
        why = {_lib.E_OVERFLOW: "ran out of idle-event slots",
               _lib.E_UNSUPPORTED: "met an input the batching simulator does not support (all replica clocks infinite)"
               }.get(code, "failed")
        raise _lib.MmsimError(code, f"{bad.size} {what}(s) {why}; their results are invalid: {names}"
                                    f"{' ...' if bad.size > 8 else ''} (pass allow_failed=True to read status[] instead)")


def _shape_results(out, n_seeds, B, allow_failed=False):
    L = n_seeds * B
    if "good" in out:
        out["good"] = out["good"].astype(bool)
    for k in list(out):
        if out[k].ndim >= 1 and out[k].shape[0] == L:
            out[k] = out[k].reshape((n_seeds, B) + out[k].shape[1:])
    if not allow_failed:
        check_status(out["status"], "simulation (seed, placement)")
    return out


def _abi_inputs(workloads, table, packed, fixed_overhead):
    """The mmsim_tables / mmsim_placements / workload-handle arguments of the batch entry points.
    Returns (tables, placements, handles, keep): `keep` holds the arrays the structs point into."""
    num_groups, group_cfg, gm_off, gm_idx = packed
    lat, pp = table.arrays()
    bss = _lib.carray(table.batch_sizes, np.int32)
    B, Gmax = group_cfg.shape
    t = _lib.Tables(lat.shape[0], lat.shape[1], lat.shape[2], lat.shape[3],
                    _lib.ptr(lat, C.c_float), _lib.ptr(pp, C.c_int32), _lib.ptr(bss, C.c_int32),
                    float(fixed_overhead))
    num_groups = _lib.carray(num_groups, np.int32)
    group_cfg = _lib.carray(group_cfg, np.int32)
    gm_off = _lib.carray(gm_off, np.int64)
    gm_idx = _lib.carray(gm_idx, np.int32)
    p = _lib.Placements(B, Gmax, _lib.ptr(num_groups, C.c_int32),
                        _lib.ptr(group_cfg, C.c_int32), _lib.ptr(gm_off, C.c_int64),
                        _lib.ptr(gm_idx, C.c_int32))
    wl = (C.c_void_p * len(workloads))(*[w._h for w in workloads])
    return t, p, wl, (lat, pp, bss, num_groups, group_cfg, gm_off, gm_idx)


def eval_batch(engine: "Engine", workloads, table: "LatencyTable", packed, flags: int = 0,
               fixed_overhead: float = FIXED_OVERHEAD, static: bool = False, allow_failed: bool = False):
    """One call of ``mmsim_eval_batch`` (create + run + sync + fetch + destroy inside the library), or of
    ``mmsim_eval_batch_static`` -- the same without any device allocation, for batches that fit the
    library's static device scratch.  Result arrays are [n_seeds][B][...]."""
    workloads = list(workloads)
    t, p, wl, keep = _abi_inputs(workloads, table, packed, fixed_overhead)
    n_seeds, B, Gmax = len(workloads), p.B, p.Gmax
    out, r = _result_arrays(flags, n_seeds, B, t.M, Gmax, max(w.R for w in workloads))
    fn = engine.lib.mmsim_eval_batch_static if static else engine.lib.mmsim_eval_batch
    _lib.check(fn(engine._h, wl, n_seeds, C.byref(t), C.byref(p), int(flags), C.byref(r)))
    del keep
    return _shape_results(out, n_seeds, B, allow_failed)


def evaluate_successors(engine: "Engine", workloads, table: "LatencyTable", bases: Sequence, parent, group, model,
                        flags: int = 0, normalize: bool = True, fixed_overhead: float = FIXED_OVERHEAD):
    """One call of ``mmsim_eval_successors``: the placements ``bases`` followed by their successors, successor k
    being ``bases[parent[k]].add_model(group[k], model[k])`` (``.normalize()`` with ``normalize``), built inside
    the library instead of as Python objects.  Result arrays are [n_seeds][len(bases) + len(parent)][...]; the
    per-group counts of a successor are in its own (normalized) group order."""
    workloads = list(workloads)
    t, p, wl, keep = _abi_inputs(workloads, table, pack_placements(bases, table), fixed_overhead)
    par, grp, mod = (_lib.carray(x, np.int32) for x in (parent, group, model))
    assert len(par) == len(grp) == len(mod)
    sc = _lib.Successors(len(par), _lib.ptr(par, C.c_int32), _lib.ptr(grp, C.c_int32), _lib.ptr(mod, C.c_int32),
                         1 if normalize else 0)
    n_seeds, B = len(workloads), p.B + len(par)
    out, r = _result_arrays(flags, n_seeds, B, t.M, p.Gmax, max(w.R for w in workloads))
    _lib.check(engine.lib.mmsim_eval_successors(engine._h, wl, n_seeds, C.byref(t), C.byref(p), C.byref(sc),
                                                int(flags), C.byref(r)))
    del keep
    return _shape_results(out, n_seeds, B)


def eval_pairs(engine: "Engine", workloads, table: "LatencyTable", packed, stream_of, flags: int = 0,
               fixed_overhead: float = FIXED_OVERHEAD, allow_failed: bool = False):
    """One call of ``mmsim_eval_pairs``: placement b on ``workloads[stream_of[b]]`` only.
    Result arrays are [B][...].  A simulation that failed (``status[b] != 0``) raises unless
    ``allow_failed``."""
    workloads = list(workloads)
    t, p, wl, keep = _abi_inputs(workloads, table, packed, fixed_overhead)
    so = _lib.carray(stream_of, np.int32)
    assert len(so) == p.B
    out, r = _result_arrays(flags, 1, p.B, t.M, p.Gmax, max(w.R for w in workloads))
    _lib.check(engine.lib.mmsim_eval_pairs(engine._h, wl, len(workloads), C.byref(t), C.byref(p),
                                           _lib.ptr(so, C.c_int32), int(flags), C.byref(r)))
    del keep
    if not allow_failed:
        check_status(out["status"])
    if "good" in out:
        out["good"] = out["good"].astype(bool)
    return out


class Batch:
    """Device-resident batch of placements x seeds; run() may be repeated."""

    def __init__(self, engine: Engine, workloads: Sequence[DeviceWorkload], table: LatencyTable,
                 packed, flags: int, fixed_overhead: float = FIXED_OVERHEAD, options=None):
        """``options``: dict of ``mmsim_options`` fields for this batch only (default: the engine's)."""
        self.engine = engine
        self.workloads = list(workloads)
        self.flags = int(flags)
        t, p, wl, keep = _abi_inputs(self.workloads, table, packed, fixed_overhead)
        self.B, self.Gmax, self.M = p.B, p.Gmax, t.M
        self.n_seeds = len(self.workloads)
        self.Rmax = max(w.R for w in self.workloads)
        self._h = C.c_void_p()
        opt = C.byref(engine.make_options(**options)) if options is not None else None
        _lib.check(engine.lib.mmsim_batch_create_ex(engine._h, wl, self.n_seeds, C.byref(t), C.byref(p),
                                                    self.flags, opt, C.byref(self._h)))

    def run(self):
        _lib.check(self.engine.lib.mmsim_batch_run(self._h))

    def sync(self) -> float:
        """Waits for the run; returns the simulation kernel's time in ms (HIP events)."""
        ms = C.c_float(0)
        _lib.check(self.engine.lib.mmsim_batch_sync(self._h, C.byref(ms)))
        return ms.value

    def info(self):
        bi = _lib.BatchInfo()
        _lib.check(self.engine.lib.mmsim_batch_get_info(self._h, C.byref(bi)))
        return {f[0]: getattr(bi, f[0]) for f in bi._fields_}

    def kernel_name(self) -> str:
        """The kernel template instance run() launches, as a profiler prints it."""
        buf = C.create_string_buffer(256)
        _lib.check(self.engine.lib.mmsim_batch_kernel_name(self._h, buf, len(buf)))
        return buf.value.decode()

    def fetch(self, per_request=True, allow_failed=False):
        """Results of the last run.  ``per_request=False`` leaves finish / good of a
        ``WANT_PER_REQUEST`` batch on the device (for ``model_stats``).  A simulation that
        failed (``status != 0``: batching simulator only) raises ``MmsimError`` naming it,
        unless ``allow_failed``, in which case the caller reads ``out["status"]``."""
        flags = self.flags if per_request else self.flags & ~_lib.WANT_PER_REQUEST
        out, r = _result_arrays(flags, self.n_seeds, self.B, self.M, self.Gmax, self.Rmax)
        _lib.check(self.engine.lib.mmsim_batch_fetch(self._h, C.byref(r)))
        return _shape_results(out, self.n_seeds, self.B, allow_failed)

    def model_stats(self, skip):
        """Per (simulation, model) statistics of the last run's per-request outputs, computed on
        the device (``mmsim_batch_model_stats``; workload.py:308-354).  ``skip[s]`` requests are
        trimmed at either end of stream ``s``.  Arrays are [n_seeds][B][M]."""
        L = self.n_seeds * self.B
        out = {f[0]: np.zeros((L, self.M), np.int32 if f[1] is _lib._p_i32 else np.float64)
               for f in _lib.ModelStats._fields_}
        r = _lib.ModelStats(*[_lib.ptr(out[f[0]], f[1]._type_) for f in _lib.ModelStats._fields_])
        wl = (C.c_void_p * self.n_seeds)(*[w._h for w in self.workloads])
        sk = (C.c_int64 * self.n_seeds)(*[int(x) for x in skip])
        _lib.check(self.engine.lib.mmsim_batch_model_stats(self._h, wl, self.n_seeds, sk, C.byref(r)))
        return {k: v.reshape(self.n_seeds, self.B, self.M) for k, v in out.items()}

    def close(self):
        if self._h:
            self.engine.lib.mmsim_batch_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def evaluate(engine: Engine, workloads: Sequence[DeviceWorkload], table: LatencyTable, sols: Sequence,
             flags: int = 0, fixed_overhead: float = FIXED_OVERHEAD):
    """One-shot: pack, upload, simulate, fetch (one call of ``mmsim_eval_batch``).  Result arrays are
    [n_seeds][B][...].  A batching simulation that runs out of idle-event slots is simulated again with more
    inside that call; ``Batch`` reports it in ``status`` instead."""
    return eval_batch(engine, workloads, table, pack_placements(sols, table), flags, fixed_overhead)


def simulate_requests_mixed(engine: Engine, finish, good, tstamps, model_ids, slos, m_id2g_id,
                            num_stages, stage_latency, num_requests=None,
                            fixed_overhead: float = FIXED_OVERHEAD):
    """Same call as the reference's numba kernel (controller.py:561-628):
    fills ``finish``/``good`` in place and returns the four count arrays."""
    ts = _lib.carray(tstamps, np.float64)
    R = len(ts) if num_requests is None else int(num_requests)
    mid = _lib.carray(model_ids, np.int32)
    sl = _lib.carray(slos, np.float32)
    m2g = _lib.carray(m_id2g_id, np.int32)
    ns = _lib.carray(num_stages, np.int32)
    lat = _lib.carray(stage_latency, np.float32)
    M, G = m2g.shape
    assert lat.shape[:2] == (M, G)
    S = lat.shape[2]
    fin = np.empty(R, np.float64)
    gd = np.empty(R, np.uint8)
    counts = [np.zeros(M, np.int32), np.zeros(M, np.int32), np.zeros(G, np.int32), np.zeros(G, np.int32)]
    _lib.check(engine.lib.mmsim_simulate_requests_mixed(
        engine._h, _lib.ptr(fin, C.c_double), _lib.ptr(gd, C.c_uint8), _lib.ptr(ts, C.c_double),
        _lib.ptr(mid, C.c_int32), _lib.ptr(sl, C.c_float), _lib.ptr(m2g, C.c_int32),
        _lib.ptr(ns, C.c_int32), _lib.ptr(lat, C.c_float), R, M, G, S, float(fixed_overhead),
        *[_lib.ptr(c, C.c_int32) for c in counts]))
    finish[:R] = fin
    good[:R] = gd.astype(bool)
    return tuple(counts)


def simulate_requests(engine: Engine, finish, good, tstamps, model_ids, slos, m_id2g_id,
                      group_max_latency, group_sum_latency, num_requests=None,
                      fixed_overhead: float = FIXED_OVERHEAD):
    """Same call as the reference's scalar-clock kernel (controller.py:506-558):
    fills ``finish``/``good`` in place and returns the four count arrays."""
    ts = _lib.carray(tstamps, np.float64)
    R = len(ts) if num_requests is None else int(num_requests)
    mid = _lib.carray(model_ids, np.int32)
    sl = _lib.carray(slos, np.float32)
    m2g = _lib.carray(m_id2g_id, np.int32)
    gmax = _lib.carray(group_max_latency, np.float32)
    gsum = _lib.carray(group_sum_latency, np.float32)
    M, G = m2g.shape
    assert gmax.shape == (M, G) and gsum.shape == (M, G)
    fin = np.empty(R, np.float64)
    gd = np.empty(R, np.uint8)
    counts = [np.zeros(M, np.int32), np.zeros(M, np.int32), np.zeros(G, np.int32), np.zeros(G, np.int32)]
    _lib.check(engine.lib.mmsim_simulate_requests(
        engine._h, _lib.ptr(fin, C.c_double), _lib.ptr(gd, C.c_uint8), _lib.ptr(ts, C.c_double),
        _lib.ptr(mid, C.c_int32), _lib.ptr(sl, C.c_float), _lib.ptr(m2g, C.c_int32),
        _lib.ptr(gmax, C.c_float), _lib.ptr(gsum, C.c_float), R, M, G, float(fixed_overhead),
        *[_lib.ptr(c, C.c_int32) for c in counts]))
    finish[:R] = fin
    good[:R] = gd.astype(bool)
    return tuple(counts)


def simulate_requests_mixed_batching(engine: Engine, finish, good, tstamps, model_ids, slos, m_id2g_id,
                                     g_id2m_id, num_stages, stage_latency, batch_sizes,
                                     num_requests=None, fixed_overhead: float = FIXED_OVERHEAD):
    """Same call as the reference's batching loop (controller.py:631-798);
    ``stage_latency`` is [M][G][Smax][NB] with one column per batch size."""
    ts = _lib.carray(tstamps, np.float64)
    R = len(ts) if num_requests is None else int(num_requests)
    mid = _lib.carray(model_ids, np.int32)
    sl = _lib.carray(slos, np.float32)
    m2g = _lib.carray(m_id2g_id, np.int32)
    g2m = _lib.carray(g_id2m_id, np.int32)
    ns = _lib.carray(num_stages, np.int32)
    lat = _lib.carray(stage_latency, np.float32)
    bss = _lib.carray(batch_sizes, np.int32)
    M, G = m2g.shape
    assert lat.shape[:2] == (M, G) and lat.shape[3] == len(bss)
    S = lat.shape[2]
    fin = np.empty(R, np.float64)
    gd = np.empty(R, np.uint8)
    counts = [np.zeros(M, np.int32), np.zeros(M, np.int32), np.zeros(G, np.int32), np.zeros(G, np.int32)]
    _lib.check(engine.lib.mmsim_simulate_requests_mixed_batching(
        engine._h, _lib.ptr(fin, C.c_double), _lib.ptr(gd, C.c_uint8), _lib.ptr(ts, C.c_double),
        _lib.ptr(mid, C.c_int32), _lib.ptr(sl, C.c_float), _lib.ptr(m2g, C.c_int32),
        _lib.ptr(g2m, C.c_int32), _lib.ptr(ns, C.c_int32), _lib.ptr(lat, C.c_float),
        _lib.ptr(bss, C.c_int32), R, M, G, S, len(bss), float(fixed_overhead),
        *[_lib.ptr(c, C.c_int32) for c in counts]))
    finish[:R] = fin
    good[:R] = gd.astype(bool)
    return tuple(counts)
