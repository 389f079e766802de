"""ctypes binding of ``libmmsim_oracle.so`` -- TEST INFRASTRUCTURE ONLY.

Builds the library from ``mmsim_oracle.c`` on demand with gcc
(``-O2 -ffp-contract=off``) when it is missing or older than its source.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmmsim_oracle.so")
_SRC = os.path.join(_HERE, "mmsim_oracle.c")
_lib = None


def build(force=False):
    stale = (not os.path.exists(_SO) or
             (os.path.exists(_SRC) and os.path.getmtime(_SRC) > os.path.getmtime(_SO)))
    if force or stale:
        subprocess.check_call(["make", "-C", _HERE, "-B", "libmmsim_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_SO)
        for name in ("oracle_simulate_requests_mixed", "oracle_simulate_requests",
                     "oracle_simulate_requests_mixed_batching", "oracle_eval_placements"):
            getattr(_lib, name).restype = C.c_int
    return _lib


def _p(a, t):
    return None if a is None else a.ctypes.data_as(C.POINTER(t))


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


def simulate_requests_mixed(tstamps, model_ids, slos, m2g, num_stages, lat, fixed_overhead=0.011):
    """lat float32 [M][G][S].  Returns finish, good(bool), counts(4), fp_ops."""
    ts, mid, sl = _c(tstamps, np.float64), _c(model_ids, np.int32), _c(slos, np.float32)
    m2g, ns, lat = _c(m2g, np.int32), _c(num_stages, np.int32), _c(lat, np.float32)
    M, G = m2g.shape
    S = lat.shape[2]
    R = len(ts)
    finish, good = np.empty(R, np.float64), np.empty(R, np.uint8)
    cnt = [np.zeros(M, np.int32), np.zeros(M, np.int32), np.zeros(G, np.int32), np.zeros(G, np.int32)]
    ops = C.c_int64(0)
    rc = lib().oracle_simulate_requests_mixed(
        _p(finish, C.c_double), _p(good, C.c_uint8), _p(ts, C.c_double), _p(mid, C.c_int32),
        _p(sl, C.c_float), _p(m2g, C.c_int32), _p(ns, C.c_int32), _p(lat, C.c_float),
        C.c_int64(R), C.c_int32(M), C.c_int32(G), C.c_int32(S), C.c_double(fixed_overhead),
        *[_p(c, C.c_int32) for c in cnt], C.byref(ops))
    assert rc == 0, rc
    return finish, good.astype(bool), tuple(cnt), ops.value


def simulate_requests(tstamps, model_ids, slos, m2g, gmax, gsum, fixed_overhead=0.011):
    ts, mid, sl = _c(tstamps, np.float64), _c(model_ids, np.int32), _c(slos, np.float32)
    m2g, gmax, gsum = _c(m2g, np.int32), _c(gmax, np.float32), _c(gsum, np.float32)
    M, G = m2g.shape
    R = len(ts)
    finish, good = np.empty(R, np.float64), np.empty(R, np.uint8)
    cnt = [np.zeros(M, np.int32), np.zeros(M, np.int32), np.zeros(G, np.int32), np.zeros(G, np.int32)]
    rc = lib().oracle_simulate_requests(
        _p(finish, C.c_double), _p(good, C.c_uint8), _p(ts, C.c_double), _p(mid, C.c_int32),
        _p(sl, C.c_float), _p(m2g, C.c_int32), _p(gmax, C.c_float), _p(gsum, C.c_float),
        C.c_int64(R), C.c_int32(M), C.c_int32(G), C.c_double(fixed_overhead),
        *[_p(c, C.c_int32) for c in cnt])
    assert rc == 0, rc
    return finish, good.astype(bool), tuple(cnt)


def simulate_requests_mixed_batching(tstamps, model_ids, slos, m2g, g2m, num_stages, lat,
                                     batch_sizes, fixed_overhead=0.011):
    """lat float32 [M][G][S][NB].  Returns finish, good, counts(4), max_heap_len."""
    ts, mid, sl = _c(tstamps, np.float64), _c(model_ids, np.int32), _c(slos, np.float32)
    m2g, g2m = _c(m2g, np.int32), _c(g2m, np.int32)
    ns, lat, bss = _c(num_stages, np.int32), _c(lat, np.float32), _c(batch_sizes, np.int32)
    M, G = m2g.shape
    S, NB = lat.shape[2], lat.shape[3]
    assert NB == len(bss)
    R = len(ts)
    finish, good = np.full(R, np.nan, np.float64), np.full(R, 255, np.uint8)
    cnt = [np.zeros(M, np.int32), np.zeros(M, np.int32), np.zeros(G, np.int32), np.zeros(G, np.int32)]
    mh = C.c_int64(0)
    rc = lib().oracle_simulate_requests_mixed_batching(
        _p(finish, C.c_double), _p(good, C.c_uint8), _p(ts, C.c_double), _p(mid, C.c_int32),
        _p(sl, C.c_float), _p(m2g, C.c_int32), _p(g2m, C.c_int32), _p(ns, C.c_int32),
        _p(lat, C.c_float), _p(bss, C.c_int32),
        C.c_int64(R), C.c_int32(M), C.c_int32(G), C.c_int32(S), C.c_int32(NB),
        C.c_double(fixed_overhead), *[_p(c, C.c_int32) for c in cnt], C.byref(mh), None)
    assert rc == 0, rc
    assert not (good == 255).any()
    return finish, good.astype(bool), tuple(cnt), mh.value


def eval_placements(tstamps, model_ids, slos, cfg_lat, cfg_pp, batch_sizes, num_groups, group_cfg,
                    gm_off, gm_idx, batching=False, fixed_overhead=0.011, want_counts=True,
                    want_per_request=False):
    """Sequential evaluation of B packed placements on one request stream.

    cfg_lat float32 [M][C][Smax][NB]; group_cfg int32 [B][Gmax]; gm_off int64 [B][Gmax+1].
    Returns dict with n_good[B], latency_sum[B], optional counts and per-request arrays, fp_ops.
    """
    ts, mid, sl = _c(tstamps, np.float64), _c(model_ids, np.int32), _c(slos, np.float32)
    cfg_lat, cfg_pp = _c(cfg_lat, np.float32), _c(cfg_pp, np.int32)
    bss = _c(batch_sizes, np.int32)
    ng, gc = _c(num_groups, np.int32), _c(group_cfg, np.int32)
    off, idx = _c(gm_off, np.int64), _c(gm_idx, np.int32)
    M, Cn, Smax, NB = cfg_lat.shape
    B, Gmax = gc.shape
    R = len(ts)
    out = {"n_good": np.zeros(B, np.int64), "latency_sum": np.zeros(B, np.float64)}
    mr = mg = gr = gg = fin = gd = None
    if want_counts:
        mr, mg = np.zeros((B, M), np.int32), np.zeros((B, M), np.int32)
        gr, gg = np.zeros((B, Gmax), np.int32), np.zeros((B, Gmax), np.int32)
    if want_per_request:
        fin, gd = np.zeros((B, R), np.float64), np.zeros((B, R), np.uint8)
    ops = C.c_int64(0)
    rc = lib().oracle_eval_placements(
        C.c_int64(R), C.c_int32(M), _p(ts, C.c_double), _p(mid, C.c_int32), _p(sl, C.c_float),
        _p(cfg_lat, C.c_float), _p(cfg_pp, C.c_int32), C.c_int32(Cn), C.c_int32(Smax), C.c_int32(NB),
        _p(bss, C.c_int32), C.c_double(fixed_overhead),
        C.c_int32(B), C.c_int32(Gmax), _p(ng, C.c_int32), _p(gc, C.c_int32),
        _p(off, C.c_int64), _p(idx, C.c_int32), C.c_int32(1 if batching else 0),
        _p(out["n_good"], C.c_int64), _p(out["latency_sum"], C.c_double),
        _p(mr, C.c_int32), _p(mg, C.c_int32), _p(gr, C.c_int32), _p(gg, C.c_int32),
        _p(fin, C.c_double), _p(gd, C.c_uint8), C.byref(ops))
    assert rc == 0, rc
    out.update(model_num_requests=mr, model_num_good=mg, group_num_requests=gr,
               group_num_good=gg, finish=fin, good=None if gd is None else gd.astype(bool),
               fp_ops=ops.value)
    return out
