"""Seeded random tiny simulator inputs shared by the oracle and parity tests."""
import numpy as np


def random_case(seed, max_m=4, max_g=3, max_s=3, max_r=50, nb=1, p_unknown=0.05,
                p_inf_row=0.05, p_odd_slo=0.05, tie_prob=0.2, load=1.0, inf_slo=True, p_member=0.6):
    """Returns dict(tstamps, model_ids, slos, m2g, g2m, num_stages, lat[M][G][S][nb])."""
    rng = np.random.default_rng(seed)
    M = int(rng.integers(1, max_m + 1))
    G = int(rng.integers(1, max_g + 1))
    num_stages = rng.integers(1, max_s + 1, size=G).astype(np.int32)
    S = int(num_stages.max())
    R = int(rng.integers(0, max_r + 1))
    member = rng.random((G, M)) < p_member
    m2g = np.full((M, G), -1, np.int32)
    g2m = np.full((G, M), -1, np.int32)
    for m in range(M):
        gs = [g for g in range(G) if member[g, m]]
        m2g[m, :len(gs)] = gs
    for g in range(G):
        ms = [m for m in range(M) if member[g, m]]
        g2m[g, :len(ms)] = ms
    base = rng.uniform(0.01, 0.3, size=(M, G, S, 1))
    steps = [1, 2, 4, 8, 16] + [16 + k for k in range(1, 12)]   # slow growth past 16 so that large batches can form
    growth = 1 + 0.15 * (np.array(steps[:nb]) - 1).reshape(1, 1, 1, nb)
    jitter = rng.uniform(0.9, 1.1, size=(M, G, S, nb))
    lat = (base * growth * jitter).astype(np.float32)
    for m in range(M):
        for g in range(G):
            if rng.random() < p_inf_row:
                lat[m, g] = np.inf
    gaps = rng.exponential(0.08 / load, size=R)
    gaps[rng.random(R) < tie_prob] = 0.0
    tstamps = np.cumsum(gaps)
    model_ids = rng.integers(0, M, size=R).astype(np.int32)
    model_ids[rng.random(R) < p_unknown] = -1
    slos = (rng.uniform(0.1, 1.5, size=R)).astype(np.float32)
    odd = rng.random(R) < p_odd_slo
    odd_values = [np.inf, np.nan, 0.0] if inf_slo else [np.nan, 0.0]
    slos[odd] = rng.choice(np.array(odd_values, np.float32), size=int(odd.sum()))
    return dict(tstamps=tstamps, model_ids=model_ids, slos=slos, m2g=m2g, g2m=g2m,
                num_stages=num_stages, lat=lat, M=M, G=G, S=S, R=R)
