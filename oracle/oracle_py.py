"""Second, independently written restatement of the simulator request loops.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).  Pure Python over
numpy scalars, meant for small inputs: it exists so that two restatements
written separately (this one and ``mmsim_oracle.c``) can be required to agree
bit for bit on thousands of random cases.  It keeps Python-level data
structures (lists as FIFOs, ``heapq``) where the C version keeps arrays.

Reference behaviour restated here:
  simulate_mixed           alpa_serve/simulator/controller.py:561-628
  simulate_scalar_clock    alpa_serve/simulator/controller.py:506-558
  simulate_mixed_batching  alpa_serve/simulator/controller.py:631-798
  build_tables             alpa_serve/simulator/controller.py:412-476
"""
import heapq
import math

import numpy as np

INF = 1e100
OVERHEAD = 0.011


def _f64(x):
    return float(np.float64(x))


def build_tables(group_configs, group_models, prof_ress, batch_sizes=(1,), penalty_per_stage=0.009):
    """Placement -> (m_id2g_id, g_id2m_id, num_stages, stage_latency[M][G][S][NB] as float32).

    controller.py:412-476.  Missing config -> whole row +inf.
    """
    M, G = len(prof_ress), len(group_configs)
    m2g = np.full((M, max(G, 1)), -1, np.int32)
    fill = [0] * M
    for g, ms in enumerate(group_models):
        for m in ms:
            m2g[m][fill[m]] = g
            fill[m] += 1
    g2m = np.full((max(G, 1), M), -1, np.int32)
    cnt = [0] * max(G, 1)
    for m in range(M):
        for g in m2g[m]:
            if g >= 0:
                g2m[g][cnt[g]] = m
                cnt[g] += 1
    num_stages = np.array([c.pp for c in group_configs], np.int32)
    S = int(num_stages.max()) if G else 1
    lat = np.zeros((M, max(G, 1), S, len(batch_sizes)), np.float32)
    for m in range(M):
        for g in range(G):
            entry = prof_ress[m].para_dict.get(group_configs[g])
            if not entry:
                lat[m, g] = np.inf
                continue
            scale = 1 + penalty_per_stage * len(entry.latency[1])
            for k in range(num_stages[g]):
                for b, bs in enumerate(batch_sizes):
                    lat[m, g, k, b] = entry.latency[bs][k] * scale
    return m2g, g2m, num_stages, lat


def simulate_mixed(tstamps, model_ids, slos, m2g, num_stages, lat):
    """lat: float32 [M][G][S].  Returns finish, good, (mreq, mgood, greq, ggood)."""
    R = len(tstamps)
    M, G = m2g.shape
    clocks = [[0.0] * int(lat.shape[2]) for _ in range(G)]
    finish = np.zeros(R, np.float64)
    good = np.zeros(R, bool)
    mreq, mgood = np.zeros(M, np.int32), np.zeros(M, np.int32)
    greq, ggood = np.zeros(G, np.int32), np.zeros(G, np.int32)
    for i in range(R):
        now, m, slo = _f64(tstamps[i]), int(model_ids[i]), _f64(slos[i])
        finish[i], good[i] = now, False
        if m < 0:
            continue
        mreq[m] += 1
        row = []                       # replica groups, "-1 terminated"
        for g in m2g[m]:
            if g < 0:
                break
            row.append(int(g))
        pick, best = -1, INF
        for g in row:
            c = clocks[g][num_stages[g] - 1]
            if c < best:
                pick, best = g, c
        if pick < 0:
            continue
        t = now
        trail = []
        for k in range(num_stages[pick]):
            t = (clocks[pick][k] if clocks[pick][k] > t else t) + _f64(lat[m, pick, k])
            trail.append(t)
        done = t + OVERHEAD
        greq[pick] += 1
        if done - now <= slo:
            finish[i], good[i] = done, True
            clocks[pick][:len(trail)] = trail
            ggood[pick] += 1
            mgood[m] += 1
    return finish, good, (mreq, mgood, greq, ggood)


def simulate_scalar_clock(tstamps, model_ids, slos, m2g, gmax, gsum):
    """Legacy one-clock-per-group variant; gmax/gsum float32 [M][G]."""
    R = len(tstamps)
    M, G = m2g.shape
    clock = [0.0] * G
    finish = np.zeros(R, np.float64)
    good = np.zeros(R, bool)
    mreq, mgood = np.zeros(M, np.int32), np.zeros(M, np.int32)
    greq, ggood = np.zeros(G, np.int32), np.zeros(G, np.int32)
    for i in range(R):
        now, m, slo = _f64(tstamps[i]), int(model_ids[i]), _f64(slos[i])
        finish[i], good[i] = now, False
        if m < 0:
            continue
        mreq[m] += 1
        pick, best = -1, INF
        for g in m2g[m]:
            if g < 0:
                break
            if clock[g] < best:
                pick, best = int(g), clock[g]
        if pick < 0:
            continue
        begin = clock[pick] if clock[pick] > now else now
        done = begin + _f64(gsum[m, pick]) + OVERHEAD
        greq[pick] += 1
        if done - now <= slo:
            finish[i], good[i] = done, True
            clock[pick] = begin + _f64(gmax[m, pick])
            ggood[pick] += 1
            mgood[m] += 1
    return finish, good, (mreq, mgood, greq, ggood)


class _BatchingSim:
    """State machine of the batching simulator (controller.py:631-798)."""

    def __init__(self, tstamps, model_ids, slos, m2g, g2m, num_stages, lat, batch_sizes):
        self.ts = [float(x) for x in tstamps]
        self.mid = [int(x) for x in model_ids]
        self.slo = [_f64(x) for x in slos]
        self.m2g, self.g2m = m2g, g2m
        self.ns = [int(x) for x in num_stages]
        self.lat = lat                      # float32 [M][G][S][NB]
        self.bss = list(batch_sizes)
        R, (M, G) = len(self.ts), m2g.shape
        self.finish = np.zeros(R, np.float64)
        self.good = np.zeros(R, bool)
        self.mreq, self.mgood = np.zeros(M, np.int32), np.zeros(M, np.int32)
        self.greq, self.ggood = np.zeros(G, np.int32), np.zeros(G, np.int32)
        self.clk = [[0.0] * int(lat.shape[2]) for _ in range(G)]
        self.idle_at = [0.0] * G
        self.fifo = [[] for _ in range(M)]
        self.events = []                    # heap of (idle time, group)
        self.max_events = 0

    def oldest_waiting_model(self, g):
        pick, best = -1, INF
        for m in self.g2m[g]:
            if m < 0:
                break
            q = self.fifo[m]
            if q and self.ts[q[0]] < best:
                pick, best = int(m), self.ts[q[0]]
        return pick

    def meets(self, t0, g, m, col, deadline):
        t = t0
        for k in range(self.ns[g]):
            c = self.clk[g][k]
            t = (c if c >= t else t) + _f64(self.lat[m, g, k, col])
        return t + OVERHEAD <= deadline

    def serve(self, t0, m, g):
        while True:
            q = self.fifo[m]
            head = None
            while q:
                r = q.pop(0)
                if self.meets(t0, g, m, 0, self.ts[r] + self.slo[r]):
                    head = r
                    break
                self.greq[g] += 1
                self.finish[r], self.good[r] = self.ts[r], False
            if head is None:
                m = self.oldest_waiting_model(g)
                if m == -1:
                    return
                continue
            size = 1
            for bs in self.bss[1:]:
                if bs - 1 > len(q):
                    break
                if not self.meets(t0, g, m, int(math.log2(bs)), self.ts[head] + self.slo[head]):
                    break
                size = bs
            members = [head] + [q.pop(0) for _ in range(size - 1)]
            col = int(math.log2(size))
            t = t0 + OVERHEAD
            trail = []
            for k in range(self.ns[g]):
                c = self.clk[g][k]
                t = (c if c > t else t) + _f64(self.lat[m, g, k, col])
                trail.append(t)
            for r in members:
                self.finish[r], self.good[r] = t, True
            self.clk[g][:len(trail)] = trail
            self.idle_at[g] = trail[0]
            heapq.heappush(self.events, (trail[0], g))
            self.max_events = max(self.max_events, len(self.events))
            self.greq[g] += size
            self.ggood[g] += size
            self.mgood[m] += size
            return

    def run(self):
        for i, now in enumerate(self.ts):
            while self.events and self.events[0][0] <= now:
                when, g = heapq.heappop(self.events)
                m = self.oldest_waiting_model(g)
                if m == -1:
                    break
                self.serve(when, m, g)
            m = self.mid[i]
            if m < 0 or self.m2g[m][0] < 0:
                self.finish[i], self.good[i] = now, False
                continue
            pick, best = -1, INF
            for g in self.m2g[m]:
                if g < 0:
                    break
                c = self.clk[g][self.ns[g] - 1]
                if c < best:
                    pick, best = int(g), c
            self.fifo[m].append(i)
            self.mreq[m] += 1
            if now >= self.idle_at[pick]:
                self.serve(now, m, pick)
        while self.events:
            when, g = heapq.heappop(self.events)
            m = self.oldest_waiting_model(g)
            if m != -1:
                self.serve(when, m, g)
        assert all(not q for q in self.fifo)
        return self.finish, self.good, (self.mreq, self.mgood, self.greq, self.ggood)


def simulate_mixed_batching(tstamps, model_ids, slos, m2g, g2m, num_stages, lat, batch_sizes):
    sim = _BatchingSim(tstamps, model_ids, slos, m2g, g2m, num_stages, lat, batch_sizes)
    out = sim.run()
    return out + (sim.max_events,)
