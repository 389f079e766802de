// Batching request-loop simulation for gfx950.
//
// Restates the reference's simulate_requests_mixed_batching
// (alpa_serve/simulator/controller.py:631-798) with one simulation per
// (placement, arrival seed) and all simulations of a wavefront walking the same
// request stream.  The outer loop over arrivals is in lockstep; what happens
// between two arrivals (idle groups picking up queued requests, dropping
// requests that can no longer meet their deadline, growing a batch) differs
// per simulation and runs as divergent loops, so a wavefront pays for every
// simulation's trips.  These loops are bound by latency and instruction issue,
// not by lanes, and a simulation's state takes about 2 KB of LDS.  Hence narrow
// tiles: a wavefront carries 64, 32, 16 or 8 simulations ("lanes" below),
// whichever puts most wavefronts on a CU; with 8, each simulation is worked on
// by an octet of lanes that hold the same state, take the same branches and
// split the scans among them.
//
// State of a lane:
//   * stage clocks clk[slot][lane] in LDS, as in the plain simulator; a
//     group's "idle since" time is its first-stage clock (the reference keeps
//     a separate array that always holds the same value, :727 and :725);
//   * one FIFO per model.  A model's queue only ever holds a contiguous run
//     of that model's arrivals, so it is a (head, tail) window into the
//     seed's arrivals regrouped by model; tail is the number of arrivals so
//     far (the same for every lane that hosts the model) and head[m][lane]
//     lives in LDS, together with the dense rank of the head request's
//     arrival time (hrank[m][lane]) so that "whose head arrived first" is
//     decided without touching global memory;
//   * the pending idle events, a multiset of (time, group) that the
//     reference keeps in a heap (:728, :739-740): an unsorted array of slots
//     per lane in LDS, in chunks of eight, with the earliest time of every
//     chunk kept beside it and a stack of the free slots.  Popping the
//     lexicographic minimum reads the chunk minima and then one chunk; adding
//     an event takes a slot off the stack.  If a lane would need more slots
//     than were provisioned it is flagged MMSIM_E_OVERFLOW and stops; its
//     results are then reported as invalid.
//
// Arithmetic follows the reference: deadlines are arrival + (double)slo,
// check_slo adds the fixed overhead last (:666-672) while a committed batch
// adds it first (:715), batch growth tests the FIRST request's deadline only
// (:693-702).

#include "mmsim_internal.h"

namespace mmsim {

namespace {

__device__ __forceinline__ int uniform_i(int v) { return __builtin_amdgcn_readfirstlane(v); }
// max of two doubles that are never NaN: one v_max_f64 without the input quieting that the generic
// fmax lowering adds
__device__ __forceinline__ double max_nn(double x, double y) {
    double r;
    asm("v_max_f64 %0, %1, %2" : "=v"(r) : "v"(x), "v"(y));
    return r;
}
__device__ __forceinline__ int ilog2i(int v) { return 31 - __clz(v); }

// ---- octet primitives.  An octet is eight consecutive lanes that work on one simulation; its lanes are
// always converged when they call these (they hold the same state and take the same branches).
// <octet primitives>
__device__ __forceinline__ int lane_id() { return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }
// bit j = the predicate of lane j of the octet
__device__ __forceinline__ uint32_t oct_ballot(bool p) {
    const uint64_t b = __builtin_amdgcn_ballot_w64(p);
    return (uint32_t)(b >> (lane_id() & 56)) & 0xFFu;
}
// exchange with the lane whose index differs in bit 0, bit 1, or with the mirror lane of the octet:
// three rounds of it reach all eight lanes
template <int STEP>
__device__ __forceinline__ uint32_t oct_swap(uint32_t v) {
    constexpr int ctrl = STEP == 0 ? 0xB1 /* quad_perm 1,0,3,2 */ : STEP == 1 ? 0x4E /* quad_perm 2,3,0,1 */ : 0x141 /* row_half_mirror */;
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, ctrl, 0xF, 0xF, false);
}
template <int STEP>
__device__ __forceinline__ double oct_swap(double v) {
    return __hiloint2double((int)oct_swap<STEP>((uint32_t)__double2hiint(v)), (int)oct_swap<STEP>((uint32_t)__double2loint(v)));
}
template <int STEP>
__device__ __forceinline__ uint64_t oct_swap(uint64_t v) {
    return ((uint64_t)oct_swap<STEP>((uint32_t)(v >> 32)) << 32) | oct_swap<STEP>((uint32_t)v);
}
// the value of lane k of the octet (k may differ from lane to lane)
__device__ __forceinline__ uint32_t oct_get(uint32_t v, int k) {
    return (uint32_t)__builtin_amdgcn_ds_bpermute(((lane_id() & 56) | k) << 2, (int)v);
}
__device__ __forceinline__ double oct_get(double v, int k) {
    return __hiloint2double((int)oct_get((uint32_t)__double2hiint(v), k), (int)oct_get((uint32_t)__double2loint(v), k));
}
__device__ __forceinline__ float oct_get(float v, int k) { return __uint_as_float(oct_get(__float_as_uint(v), k)); }
// the value of the octet's first lane: the first lane of each quad to its quad, then the lanes of the octet's second
// quad take the lane four below (two DPP moves, no trip through the LDS crossbar)
__device__ __forceinline__ uint32_t oct_first(uint32_t v) {
    const int q = __builtin_amdgcn_update_dpp(0, (int)v, 0x00 /* quad_perm 0,0,0,0 */, 0xF, 0xF, false);
    return (uint32_t)__builtin_amdgcn_update_dpp(q, q, 0x114 /* row_shr:4 */, 0xF, 0xA /* lanes 4-7 and 12-15 of a row */, false);
}
__device__ __forceinline__ double oct_first(double v) {
    return __hiloint2double((int)oct_first((uint32_t)__double2hiint(v)), (int)oct_first((uint32_t)__double2loint(v)));
}
// The lanes of an octet run in lockstep; this marks the places where that matters (all have read a
// value before any of them overwrites it).  No instruction.
__device__ __forceinline__ void oct_sync() { __builtin_amdgcn_wave_barrier(); }
// </octet primitives>
// Minimum over the octet, in all of its lanes.  One DPP instruction per step: v_min_u32_dpp d, d, d =
// min(d of the lane the pattern names, d); a DPP operand needs two wait states after the write of its
// register (s_nop 1).
__device__ __forceinline__ uint32_t oct_min(uint32_t v) {
    asm("s_nop 1\n"
        "v_min_u32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n"
        "s_nop 1\n"
        "v_min_u32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n"
        "s_nop 1\n"
        "v_min_u32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n"
        : "+v"(v));
    return v;
}
// 64 bits: the smallest high word, then the smallest low word among the lanes that have it
__device__ __forceinline__ uint64_t oct_min(uint64_t v) {
    const uint32_t hi = (uint32_t)(v >> 32), lo = (uint32_t)v;
    const uint32_t mh = oct_min(hi);
    const uint32_t ml = oct_min(hi == mh ? lo : 0xFFFFFFFFu);
    return ((uint64_t)mh << 32) | ml;
}
// Doubles that are never negative nor NaN (clocks and event times: they start at +0 and only ever
// grow by latencies >= 0; +inf is allowed) order as their bit patterns do.
__device__ __forceinline__ double oct_min(double v) {
    return __longlong_as_double((long long)oct_min((uint64_t)__double_as_longlong(v)));
}
// sum over the octet, in all of its lanes (the same order of additions in every lane)
__device__ __forceinline__ double oct_sum(double v) {
    v += oct_swap<0>(v);
    v += oct_swap<1>(v);
    return v + oct_swap<2>(v);
}

typedef volatile __attribute__((address_space(3))) uint32_t lds_vu32;
__device__ __forceinline__ lds_vu32 *as_lds_vu32(void *p) { return (lds_vu32 *)p; }

// NBT: latency columns held in registers (the table's NB columns, rounded up to 4, 8 or 16).
// LATLDS / G2MLDS: the latency table / the lists of each group's models are read from their LDS
// copies.  These are compile-time choices so that every LDS access is a DS instruction: through a
// generic pointer the compiler may fold a constant of the index (the 31 of 31 - clz(batch size)) into
// the instruction's offset field, and the hardware picks the aperture from the base register alone,
// which then lies below the LDS aperture for a table at the start of LDS.
// OCT: tiles of eight simulations, each worked on by an octet of consecutive lanes (lane = 8 * simulation
// + helper).  The lanes of an octet hold the same state and take the same branches; the scans (event
// slots, models of a group, replicas, heads' deadlines, latency columns) are split among them.
// UNIF: every (model, configuration) has the same latencies in all of its stages, and the table holds them
// once (a row of NB columns per configuration): a pass over a group's stages loads its latency once.
// SH (octets only): at most 64 event slots per simulation.  Which slots are in use is a 64-bit mask in registers
// and lane c of an octet keeps the earliest time of chunk c in a register: neither the free-slot stack nor the
// chunk minima are read from LDS.
template <int NBT, bool LATLDS, bool G2MLDS, bool OCT, bool UNIF, bool SH>
__global__ __launch_bounds__(kMaxWavesPerBlockBatching *kWave) void sim_batching_kernel(const BatchingArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];

    const int W = (int)(blockDim.x >> 6);
    const int wv = uniform_i((int)(threadIdx.x >> 6));
    const int lane = (int)(threadIdx.x & 63);
    const unsigned grid_seeds = a.paired ? 1u : (unsigned)a.n_seeds;
    const int tile = (int)(blockIdx.x / grid_seeds) * W + wv;
    // paired batches: the tile's own stream; otherwise every tile on every stream
    const int seed = a.paired ? (tile < a.tiles ? a.tile_seed[tile] : 0) : (int)(blockIdx.x % grid_seeds);
    const bool want_model = (a.flags & MMSIM_WANT_MODEL_COUNTS) != 0;
    const bool want_group = (a.flags & MMSIM_WANT_GROUP_COUNTS) != 0;
    const bool want_req = (a.flags & MMSIM_WANT_PER_REQUEST) != 0;
    const int M = a.M, Gmax = a.Gmax, NB = a.NB;
    // simulations per wavefront (64, 32, 16 or 8): pitch of the per-simulation LDS arrays.  Octets mean 8: a constant
    // there, so that the index arithmetic is shifts, not multiplications
    const int LS = OCT ? 8 : a.lane_stride;
    const int sl = OCT ? lane >> 3 : lane;  // this lane's simulation within the tile
    const int oj = OCT ? lane & 7 : 0;      // this lane's place in its octet
    const int fill = OCT ? kWave : LS;      // lanes that fill the wavefront's shared LDS arrays

    // ---- LDS: [latency table, shared, if it fits][per wavefront: group descriptors | clocks | event times |
    //      chunk minima | queue heads | head ranks | event groups | free slots | arrivals per model | offsets of
    //      the models' arrival lists | batch sizes | models of each group, if they fit]
    const int nch = a.heap_cap >> 3;         // chunks of eight event slots
    const int nch8 = (nch + 7) & ~7;         // chunk minima are read eight at a time; the spare ones stay +inf
    float *lat_lds = reinterpret_cast<float *>(lds_raw);
    if (a.lat_lds_bytes > 0) {
        const int n = M * a.lat_row * NB;
        for (int i = (int)threadIdx.x; i < n; i += (int)blockDim.x) lat_lds[i] = a.lat[i];
    }
    unsigned char *mine = lds_raw + a.lat_lds_bytes + wv * a.wave_lds_bytes;
    // (octet tiles get a group's descriptor with the replica lists and keep no copy of the table: the replicas past
    // the eighth of a model, rare, are looked up in global memory)
    uint32_t *ginfo = reinterpret_cast<uint32_t *>(mine) + sl;
    size_t o = OCT ? 0 : (size_t)(Gmax + 1) * LS * 4;
    double *clk = reinterpret_cast<double *>(mine + o) + sl;
    o += (size_t)a.nslots * LS * 8;
    double *ev_t = reinterpret_cast<double *>(mine + o) + sl;
    o += (size_t)a.heap_cap * LS * 8;
    double *cm_t = reinterpret_cast<double *>(mine + o) + sl;  // earliest event time of each chunk (not with SH)
    if constexpr (!SH) o += (size_t)nch8 * LS * 8;
    uint32_t *head = reinterpret_cast<uint32_t *>(mine + o) + sl;
    o += (size_t)M * LS * 4;
    int32_t *hrank = reinterpret_cast<int32_t *>(mine + o) + sl;  // rank of the arrival at head[m] (already known before it arrives)
    o += (size_t)M * LS * 4;
    uint32_t *ev_g = reinterpret_cast<uint32_t *>(mine + o) + sl;
    o += (size_t)a.heap_cap * LS * 4;
    uint16_t *fstack = reinterpret_cast<uint16_t *>(mine + o) + sl;  // free event slots, the next one to use on top (not with SH)
    if constexpr (!SH) o += (size_t)a.heap_cap * LS * 2;
    // [M], same for all lanes; written by lane 0 and read by all, hence volatile (and spelled as an LDS
    // pointer: volatile accesses are not rewritten from generic to LDS by the compiler)
    lds_vu32 *arrived = as_lds_vu32(mine + o);
    o += ((size_t)M * 4 + 15) & ~(size_t)15;
    int64_t *mq_off = reinterpret_cast<int64_t *>(mine + o);  // [M+1] this seed's offsets into mq
    o += ((size_t)(M + 1) * 8 + 15) & ~(size_t)15;
    int32_t *bsz = reinterpret_cast<int32_t *>(mine + o);  // [NB] batch sizes
    o += ((size_t)NB * 4 + 15) & ~(size_t)15;
    uint16_t *g2m_off_lds = reinterpret_cast<uint16_t *>(mine + o) + sl;  // [Gmax+1][64]
    o += (size_t)(Gmax + 1) * LS * 2;
    uint16_t *g2m_idx_lds = reinterpret_cast<uint16_t *>(mine + o) + sl;  // [members_max][64]

    bool sizes_pow2 = true;  // wave-uniform: batch size q is 1 << q
    for (int q = 0; q < NB; ++q) sizes_pow2 = sizes_pow2 && a.batch_sizes[q] == (1 << q);

    const bool live = tile < a.tiles;
    const bool sim = sl < LS;  // the other lanes of a narrow tile only help fetching requests
    if (live && sim) {
        const uint32_t *gsrc = a.ginfo + (size_t)tile * (Gmax + 1) * kWave + sl;
        if constexpr (!OCT)
            for (int g = 0; g <= Gmax; ++g) ginfo[g * LS] = gsrc[g * kWave];
        for (int s = 0; s < a.nslots; ++s) clk[s * LS] = 0.0;
        for (int e = 0; e < a.heap_cap; ++e) {  // free event slots never win a minimum scan
            ev_t[e * LS] = __builtin_inf();
            ev_g[e * LS] = 0xFFFFFFFFu;
            if constexpr (!SH) fstack[e * LS] = (uint16_t)(a.heap_cap - 1 - e);  // slot 0 is used first, so events gather in the first chunks
        }
        if constexpr (!SH)
            for (int c = 0; c < nch8; ++c) cm_t[c * LS] = __builtin_inf();
        {
            const int64_t *mo = a.mq_off + (size_t)seed * (M + 1);
            for (int m = lane; m <= M; m += fill) mq_off[m] = mo[m];
            for (int q = lane; q < NB; q += fill) bsz[q] = a.batch_sizes[q];
            for (int m = 0; m < M; ++m) {
                head[m * LS] = 0u;
                hrank[m * LS] = a.mq[mo[m]].rank;  // of the model's first arrival (the padding entry if it has none)
            }
        }
        for (int m = lane; m < M; m += fill) arrived[m] = 0u;
        if (a.g2m_in_lds) {
            const uint16_t *osrc = a.g2m_off + (size_t)tile * (Gmax + 1) * kWave + sl;
            const uint16_t *isrc = a.g2m_idx + (size_t)tile * a.members_max * kWave + sl;
            for (int g = 0; g <= Gmax; ++g) g2m_off_lds[g * LS] = osrc[g * kWave];
            for (int x = 0; x < a.members_max; ++x) g2m_idx_lds[x * LS] = isrc[(size_t)x * kWave];
        }
    }
    __syncthreads();  // the latency table is complete; wavefronts run independently from here
    if (!live) return;

    const int wave = a.paired ? tile : seed * a.tiles + tile;  // where this (tile, stream) pair's results go
    const int64_t off = a.stream_off[seed];
    const int64_t R = a.stream_off[seed + 1] - off;
    const Req *__restrict__ reqs = a.streams + off;
    const uint64_t *__restrict__ rep_tile = a.rep8 + (size_t)tile * M * kWave + sl;
    // octets: the row of a model holds a descriptor per lane (the j-th replica's group for lane 8 * simulation + j)
    const uint32_t *__restrict__ repd_tile = reinterpret_cast<const uint32_t *>(a.rep8) + (size_t)tile * M * 2 * kWave + lane;
    auto row_of = [&](int mx) -> uint64_t {
        const size_t mr = (size_t)(mx < 0 ? 0 : mx);
        if constexpr (OCT) return repd_tile[mr * 2 * kWave];
        return rep_tile[mr * kWave];
    };
    const uint8_t *__restrict__ repx_tile = a.repx + (size_t)tile * M * a.rep_extra * kWave + sl;
    const uint16_t *g2m_off_glb = a.g2m_off + (size_t)tile * (Gmax + 1) * kWave + sl;
    const uint16_t *g2m_idx_glb = a.g2m_idx + (size_t)tile * a.members_max * kWave + sl;
    auto g2m_off_at = [&](uint32_t g) -> int { return G2MLDS ? g2m_off_lds[g * LS] : g2m_off_glb[(size_t)g * kWave]; };
    auto g2m_idx_at = [&](int x) -> int { return G2MLDS ? g2m_idx_lds[x * LS] : g2m_idx_glb[(size_t)x * kWave]; };
    auto lat_at = [&](uint32_t i) -> float { return LATLDS ? lat_lds[i] : a.lat[i]; };
    int32_t *model_good = a.model_good + (size_t)wave * M * kWave + sl;
    int32_t *group_req = a.group_req + (size_t)wave * Gmax * kWave + sl;
    int32_t *group_good = a.group_good + (size_t)wave * Gmax * kWave + sl;
    double *fin_out = a.finish + (size_t)wave * a.Rmax * kWave + sl;
    uint8_t *good_out = a.good + (size_t)wave * a.Rmax * kWave + sl;
    const double overhead = a.fixed_overhead;

    int32_t n_good = 0;
    double lat_sum = 0.0;
    int nfree = a.heap_cap;  // free event slots of this lane (heap_cap - nfree events are pending)
    uint64_t used = 0;       // SH: bit e = event slot e holds an event
    double my_cm = __builtin_inf();  // SH: the earliest event time of chunk oj (this lane's place in its octet)
    static_assert(!SH || OCT, "registers for the event slots' bookkeeping go with octets");
    double next_due = __builtin_inf();  // the earliest of them (+inf if none): arrivals before it skip the event list
    int dead = sim ? 0 : 1;  // nonzero: this lane simulates nothing (more): out of event slots, unsupported input, or a spare lane of a narrow tile

    const uint32_t none = (uint32_t)Gmax;
    Req blk_req = {0.0, -1, 0.0f};  // this lane's request of the current block of 64
    uint64_t g8_next = 0;          // replica list (eight group bytes) of the next request's model, fetched ahead

    // :654-664 -- among the models of group g with a waiting request, the one whose head arrived first
    auto select_model = [&](uint32_t g) -> int {
        const int lo = g2m_off_at(g), hi = g2m_off_at(g + 1u);
        if constexpr (OCT) {
            // The models of the group are dealt to the lanes of the octet (model x to lane x mod 8), two per lane
            // and round so that their reads overlap; every lane keeps the smallest key of its own models and the
            // octet takes one minimum at the end.  The key orders by rank of the head's arrival, then by place in
            // the list.
            constexpr int kPerLane = 2;
            uint64_t best = ~0ull;
            for (int xb = lo; xb < hi; xb += 8 * kPerLane) {
                int mm[kPerLane];
                uint32_t rk[kPerLane], hd[kPerLane], ar[kPerLane];
#pragma unroll
                for (int u = 0; u < kPerLane; ++u) {
                    const int x = xb + 8 * u + oj;
                    mm[u] = g2m_idx_at(x < hi ? x : hi - 1);
                }
#pragma unroll
                for (int u = 0; u < kPerLane; ++u) {
                    rk[u] = (uint32_t)hrank[mm[u] * LS];
                    hd[u] = head[mm[u] * LS];
                    ar[u] = arrived[mm[u]];
                }
#pragma unroll
                for (int u = 0; u < kPerLane; ++u) {
                    const int x = xb + 8 * u + oj;
                    const bool waiting = x < hi && (int)(ar[u] - hd[u]) > 0;
                    const uint64_t key = waiting ? ((uint64_t)rk[u] << 32) | ((uint64_t)(uint32_t)(x - lo) << 16) | (uint32_t)mm[u] : ~0ull;
                    best = key < best ? key : best;
                }
            }
            best = oct_min(best);
            return best == ~0ull ? -1 : (int)(best & 0xFFFFu);
        }
        int min_rank = 0x7FFFFFFF;
        int pick = -1;
        for (int x0 = lo; x0 < hi; x0 += 4) {  // four models at a time: their reads overlap
            int mm[4], rk[4];
            uint32_t hd[4], ar[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) mm[u] = g2m_idx_at(x0 + u < hi ? x0 + u : hi - 1);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                rk[u] = hrank[mm[u] * LS];
                hd[u] = head[mm[u] * LS];
                ar[u] = arrived[mm[u]];
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
                // strictly earlier arrival; ties keep the earlier-listed model
                if (x0 + u < hi && (int)(ar[u] - hd[u]) > 0 && rk[u] < min_rank) {
                    min_rank = rk[u];
                    pick = mm[u];
                }
        }
        return pick;
    };

    // :666-672 without the final "+ overhead <= deadline": the time a batch started at t0 leaves the
    // group's last stage, for every latency column at once (one pass over the stages, four stages per
    // round of LDS reads)
    auto batch_times = [&](double t0, const double *gclk, int stages, uint32_t lat_mg, double(&tb)[NBT]) {
#pragma unroll
        for (int b = 0; b < NBT; ++b) tb[b] = t0;
        float lu[NBT];
        if constexpr (UNIF) {
#pragma unroll
            for (int b = 0; b < NBT; ++b) lu[b] = lat_at(lat_mg + (uint32_t)(b < NB ? b : NB - 1));
        }
        for (int k0 = 0; k0 < stages; k0 += 4) {
            double c[4];
            float l[4][NBT];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int k = k0 + u < stages ? k0 + u : stages - 1;
                c[u] = gclk[k * LS];
#pragma unroll
                for (int b = 0; b < NBT; ++b) l[u][b] = UNIF ? lu[b] : lat_at(lat_mg + (uint32_t)(k * NB + (b < NB ? b : NB - 1)));
            }
#pragma unroll
            for (int u = 1; u < 4; ++u)
                if (!(k0 + u < stages)) {  // past the last stage: max(-inf, t) + 0 leaves t as it is
                    c[u] = -__builtin_inf();
#pragma unroll
                    for (int b = 0; b < NBT; ++b) l[u][b] = 0.0f;
                }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
#pragma unroll
                for (int b = 0; b < NBT; ++b) tb[b] = max_nn(c[u], tb[b]) + (double)l[u][b];
            }
        }
    };

    // the same for one latency column (the octet's lanes take one column each)
    // c0: the group's clocks of the first four stages, read by the caller (they do not change before the commit, which
    // uses them again); lu: with UNIF, the column's latency; l0: otherwise, the column's latencies of the first four
    // stages as read here (the commit takes them from the lane that had its column)
    auto batch_time_col = [&](double t0, const double *gclk, int stages, uint32_t lat_mg, int col, const double(&c0)[4],
                              float lu, float(&l0)[4]) -> double {
        double t = t0;
        for (int k0 = 0; k0 < stages; k0 += 4) {
            double c[4];
            float l[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int k = k0 + u < stages ? k0 + u : stages - 1;
                c[u] = k0 == 0 ? c0[u] : gclk[k * LS];
                l[u] = UNIF ? lu : lat_at(lat_mg + (uint32_t)(k * NB + col));
            }
            if (k0 == 0) {
#pragma unroll
                for (int u = 0; u < 4; ++u) l0[u] = l[u];
            }
#pragma unroll
            for (int u = 1; u < 4; ++u)
                if (!(k0 + u < stages)) {
                    c[u] = -__builtin_inf();
                    l[u] = 0.0f;
                }
#pragma unroll
            for (int u = 0; u < 4; ++u) t = max_nn(c[u], t) + (double)l[u];
        }
        return t;
    };
    constexpr bool COOP = OCT && NBT <= 8;  // batch attempts split over the octet (one latency column per lane)

    // :706-732 with :674-704 inlined; the reference's recursion on "nothing servable" is the outer loop
    // d: the group's descriptor (its index is desc_group(d))
    auto handle = [&](double t0, int m, uint32_t d) {
        const uint32_t g = desc_group(d);
        const int stages = (int)desc_stages_m1(d) + 1;
        double *gclk = clk + (desc_last_slot(d) - desc_stages_m1(d)) * LS;
        // COOP: the clocks of the group's first four stages (the same for every queue tried below)
        double c0[4] = {0.0, 0.0, 0.0, 0.0};
        if constexpr (COOP) {
#pragma unroll
            for (int u = 0; u < 4; ++u) c0[u] = gclk[(u < stages ? u : stages - 1) * LS];
        }
        for (;;) {
            const uint32_t lat_mg = ((uint32_t)m * (uint32_t)a.lat_row + desc_lat_off(d)) * (uint32_t)NB;  // the (model, group) rows of the table
            const int64_t base = mq_off[m];
            const uint32_t arr = arrived[m];  // does not change while a lane is in here
            uint32_t h = head[m * LS];        // arr - h > 0: the caller saw a waiting request
            if constexpr (OCT) oct_sync();
            // drop heads that cannot meet their deadline even alone (:677-686).  The finish time of a
            // batch of one does not depend on which request it is, so it is computed once; the
            // deadlines of up to eight heads are fetched together, the first eight ahead of that pass.
            int64_t q0 = base + h;
            int avail = (int)(arr - h) < 8 ? (int)(arr - h) : 8;
            bool found = false;
            int64_t first = 0;
            double deadline = 0.0, first_t = 0.0;
            int bs = 1;
            // COOP: what this lane fetched of the queue (entry q0 + oj: arrival time, deadline, index, rank; and the
            // rank of entry q0 + oj + 8), the head that leads the batch, the first four stages as batch_time_col read them
            double2 hv = {0.0, 0.0};
            int2 ir = {0, 0};
            int32_t rank8 = 0;
            int kfirst = 0;
            float l0[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            if constexpr (COOP) {
                // lane j of the octet takes entry j from the head of the queue on -- all of it, whether it has arrived
                // yet or not, so that a batch made of these eight needs no further fetch -- and latency column j
                const MqEntry *ep = &a.mq[q0 + oj];
                hv = *reinterpret_cast<const double2 *>(ep);
                ir = *reinterpret_cast<const int2 *>(&ep->idx);
                rank8 = ep[8].rank;
                const int mycol = oj < NB ? oj : NB - 1;
                float lu = 0.0f;
                if constexpr (UNIF) lu = lat_at(lat_mg + (uint32_t)mycol);
                const double tcol = batch_time_col(t0, gclk, stages, lat_mg, mycol, c0, lu, l0);
                const double alone = oct_first(tcol) + overhead;  // check_slo(..., batch size 1, deadline) == (alone <= deadline)
                for (;;) {
                    const uint32_t pass = oct_ballot(oj < avail && alone <= hv.y);
                    const int k = pass ? __ffs((int)pass) - 1 : avail;  // the heads before k are dropped
                    if (oj < k) {
                        if (want_req) {
                            fin_out[(size_t)ir.x * kWave] = hv.x;
                            good_out[(size_t)ir.x * kWave] = 0;
                        }
                    }
                    if (want_group && oj == 0) group_req[g * kWave] += k;
                    if (pass) {
                        found = true;
                        kfirst = k;
                        first = q0 + k;
                        deadline = oct_get(hv.y, k);
                        h += (uint32_t)(k + 1);
                        break;
                    }
                    h += (uint32_t)avail;
                    if (h == arr) break;
                    q0 = base + h;
                    avail = (int)(arr - h) < 8 ? (int)(arr - h) : 8;
                    ep = &a.mq[q0 + oj];
                    hv = *reinterpret_cast<const double2 *>(ep);
                    ir = *reinterpret_cast<const int2 *>(&ep->idx);
                    rank8 = ep[8].rank;
                }
                if (found) {
                    // grow the batch while the first request still meets its deadline (:693-702): lane b tests
                    // batch size b, the batch is the last size before the first one that fails.  When the sizes are
                    // 1, 2, 4, ... (size b is 1 << b and has latency column b) nothing needs to be looked up.
                    const int cand = sizes_pow2 ? 1 << (oj < NB ? oj : NB - 1) : bsz[oj < NB ? oj : NB - 1];
                    const double tc = sizes_pow2 ? tcol : oct_get(tcol, ilog2i(cand));
                    const bool ok = oj == 0 || (oj < NB && cand - 1 <= (int)(arr - h) && (tc + overhead) <= deadline);
                    const uint32_t fail = ~oct_ballot(ok) & 0xFFu;
                    const int nb_ok = fail ? __ffs((int)fail) - 1 : 8;
                    bs = sizes_pow2 ? 1 << (nb_ok - 1) : bsz[nb_ok - 1];
                }
            } else {
            double dl[8], tq[8];  // deadlines and arrival times (one 16-byte load per head)
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const double2 v = *reinterpret_cast<const double2 *>(&a.mq[q0 + (k < avail ? k : avail - 1)]);
                tq[k] = v.x;
                dl[k] = v.y;
            }
            double tb[NBT];
            batch_times(t0, gclk, stages, lat_mg, tb);
            const double alone = tb[0] + overhead;  // check_slo(..., batch size 1, deadline) == (alone <= deadline)
            for (;;) {
                for (int k = 0; k < avail; ++k) {
                    h += 1u;
                    if (alone <= dl[k]) {
                        found = true;
                        first = q0 + k;
                        deadline = dl[k];
                        first_t = tq[k];
                        break;
                    }
                    if (want_group && oj == 0) group_req[g * kWave] += 1;
                    if (want_req) {
                        const MqEntry e = a.mq[q0 + k];
                        fin_out[(size_t)e.idx * kWave] = e.t;
                        good_out[(size_t)e.idx * kWave] = 0;
                    }
                }
                if (found || h == arr) break;
                q0 = base + h;
                avail = (int)(arr - h) < 8 ? (int)(arr - h) : 8;
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const double2 v = *reinterpret_cast<const double2 *>(&a.mq[q0 + (k < avail ? k : avail - 1)]);
                    tq[k] = v.x;
                    dl[k] = v.y;
                }
            }
            if (found) {
                // grow the batch while the first request still meets its deadline (:693-702)
                for (int b = 1; b < NB; ++b) {
                    const int cand = bsz[b];
                    if (cand - 1 > (int)(arr - h)) break;
                    const int col = ilog2i(cand);
                    double tc = tb[0];
#pragma unroll
                    for (int x = 1; x < NBT; ++x) tc = col == x ? tb[x] : tc;
                    if (!((tc + overhead) <= deadline)) break;
                    bs = cand;
                }
            }
            }
            if (!found) {  // :709-713
                head[m * LS] = h;
                // the rank of this model's next arrival is not needed to pick another model (this one has
                // nothing waiting), so its fetch overlaps the selection
                const int32_t next_rank = a.mq[base + h].rank;
                const int m_next = select_model(g);
                hrank[m * LS] = next_rank;
                m = m_next;
                if (m < 0) return;
                continue;
            }
            // run it (:715-732).  The rank of the arrival after the batch: one of the sixteen the octet fetched, or
            // fetched while the stages are walked
            const int col = ilog2i(bs);
            int32_t next_rank;
            if constexpr (COOP) {
                const int kb = kfirst + bs;  // batches of sixteen and more reach past what was fetched
                next_rank = kb < 16 ? (int32_t)oct_get((uint32_t)(kb < 8 ? ir.y : rank8), kb & 7) : a.mq[first + bs].rank;
            } else {
                next_rank = a.mq[first + bs].rank;
            }
            double t = t0 + overhead;
            double idle_at = 0.0;
            float lu = 0.0f;  // UNIF: the latency of every stage at this batch size
            if constexpr (UNIF && COOP) {
                lu = oct_get(l0[0], col);
            } else if constexpr (UNIF) {
                lu = lat_at(lat_mg + (uint32_t)col);
            }
            for (int k0 = 0; k0 < stages; k0 += 4) {
                double c[4];
                float l[4];
                if (COOP && k0 == 0) {  // as batch_time_col read them; the latencies are those of the lane that took this column
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        c[u] = c0[u];
                        l[u] = UNIF ? lu : oct_get(l0[u], col);
                    }
                } else {
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const int k = k0 + u < stages ? k0 + u : stages - 1;
                        c[u] = gclk[k * LS];
                        l[u] = UNIF ? lu : lat_at(lat_mg + (uint32_t)(k * NB + col));
                    }
                }
                if constexpr (OCT) oct_sync();
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    if (k0 + u < stages) {
                        t = max_nn(t, c[u]) + (double)l[u];
                        gclk[(k0 + u) * LS] = t;
                        if (k0 + u == 0) idle_at = t;
                    }
            }
            head[m * LS] = h + (uint32_t)(bs - 1);  // the batch is the arrivals first .. first+bs-1 of the model
            hrank[m * LS] = next_rank;
            if constexpr (COOP) {
                // the batch is the entries kfirst .. kfirst + bs - 1 of those fetched: each lane accounts for its own
                // (the octet's latency sums are added up at the end)
                if (oj >= kfirst && oj < kfirst + bs) {
                    lat_sum += t - hv.x;
                    if (want_req) {
                        fin_out[(size_t)ir.x * kWave] = t;
                        good_out[(size_t)ir.x * kWave] = 1;
                    }
                }
                for (int u = 8 - kfirst; u < bs; ++u) {  // members behind those eight (heads were dropped first): rare
                    const MqEntry e = a.mq[first + u];
                    if (oj == 0) {
                        lat_sum += t - e.t;
                        if (want_req) {
                            fin_out[(size_t)e.idx * kWave] = t;
                            good_out[(size_t)e.idx * kWave] = 1;
                        }
                    }
                }
            } else {
            lat_sum += t - first_t;  // the first member's arrival time came with its deadline
            if (want_req) {
                const int32_t r = a.mq[first].idx;
                fin_out[(size_t)r * kWave] = t;
                good_out[(size_t)r * kWave] = 1;
            }
            for (int u0 = 1; u0 < bs; u0 += 8) {  // arrival times of up to eight more members fetched together
                double at[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) at[k] = a.mq[first + (u0 + k < bs ? u0 + k : bs - 1)].t;
                for (int k = 0; k < 8 && u0 + k < bs; ++k) {
                    lat_sum += t - at[k];
                    if (want_req) {
                        const int32_t r = a.mq[first + u0 + k].idx;
                        fin_out[(size_t)r * kWave] = t;
                        good_out[(size_t)r * kWave] = 1;
                    }
                }
            }
            }
            n_good += bs;
            if (want_group && oj == 0) {  // the lanes of an octet would all add
                group_req[g * kWave] += bs;
                group_good[g * kWave] += bs;
            }
            if (want_model && oj == 0) model_good[(size_t)m * kWave] += bs;
            if (nfree == 0) {
                dead = MMSIM_E_OVERFLOW;
                return;
            }
            nfree -= 1;
            int slot;
            if constexpr (SH) {
                slot = __ffsll((long long)~used) - 1;  // the lowest free slot: events gather in the first chunks
                used |= 1ull << slot;
                if (oj == (slot >> 3)) my_cm = fmin(my_cm, idle_at);
            } else {
                slot = fstack[nfree * LS];
                double *cm = cm_t + (slot >> 3) * LS;
                *cm = fmin(*cm, idle_at);
            }
            ev_t[slot * LS] = idle_at;
            ev_g[slot * LS] = d;  // the descriptor, not the index: it orders like the index and saves the look-up when the event is due
            next_due = fmin(next_due, idle_at);
            return;
        }
    };

    // earliest event time (+inf if there is no event), the chunk that holds it (the first such chunk),
    // and the earliest time among the other chunks
    auto chunk_scan = [&](double &T, int &cj, double &others) {
        T = __builtin_inf();
        others = __builtin_inf();
        cj = 0;
        if constexpr (SH) {
            // at most eight chunks, their minima in the octet's registers; the earliest time of all is next_due, which
            // is kept exact.  The earliest of the other chunks is left to pop_event, which computes it while it waits
            // for the chunk's slots.
            T = next_due;
            cj = __ffs((int)oct_ballot(my_cm == T)) - 1;  // -1: there is no event (T is +inf, and so are the minima: 0)
            cj = cj < 0 ? 0 : cj;
            return;
        }
        if constexpr (OCT) {
            for (int c0 = 0; c0 < nch; c0 += 8) {  // one chunk minimum per lane
                const double v = cm_t[(c0 + oj) * LS];
                const double mn = oct_min(v);
                const int first = __ffs((int)oct_ballot(v == mn)) - 1;
                const double rest = oct_min(oj == first ? __builtin_inf() : v);
                if (mn < T) {
                    others = T < rest ? T : rest;  // the previous earliest is now one of the others
                    T = mn;
                    cj = c0 + first;
                } else {
                    others = mn < others ? mn : others;
                }
            }
            return;
        }
        for (int c0 = 0; c0 < nch; c0 += 8) {
            double v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = cm_t[(c0 + u) * LS];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (v[u] < T) {
                    others = T;  // the previous earliest is the earliest of the others so far
                    T = v[u];
                    cj = c0 + u;
                } else {
                    others = v[u] < others ? v[u] : others;
                }
        }
    };
    // removes the lexicographically smallest (time, group) event, whose time T and chunk cj chunk_scan
    // found (others as returned by it); returns its word (the group's descriptor, which orders like the group's
    // index) and sets next_due to the earliest time left
    // SH: the same in one piece, for the time T and chunk cj that chunk_scan gave
    auto pop_event = [&](double T, int cj) -> uint32_t {
        uint32_t bg = 0xFFFFFFFFu;
        int be = cj << 3;
        const uint32_t tied = oct_ballot(my_cm == T);
        const bool tie = (tied & (tied - 1u)) != 0;
        if (tie) {  // several chunks hold an event at time T: the smallest group among all of them (rare)
            for (int c = 0; c < nch; ++c) {
                if (!((tied >> c) & 1u)) continue;
                for (int u = 0; u < 8; ++u) {
                    const int e = (c << 3) + u;
                    const uint32_t g = ev_g[e * LS];
                    if (ev_t[e * LS] == T && g < bg) {
                        bg = g;
                        be = e;
                    }
                }
            }
            cj = be >> 3;
        }
        const int e = (cj << 3) + oj;  // one slot of the chunk per lane
        const double t = ev_t[e * LS];
        const uint32_t g = ev_g[e * LS];
        const double others = oct_min(oj == cj ? __builtin_inf() : my_cm);  // (with a tie: T again, whichever chunk was taken)
        if (!tie) {
            bg = oct_min(t == T ? g : 0xFFFFFFFFu);
            be = (cj << 3) + __ffs((int)oct_ballot(t == T && g == bg)) - 1;
        }
        const double left = oct_min(e == be ? __builtin_inf() : t);  // earliest time left in the chunk
        ev_t[be * LS] = __builtin_inf();
        ev_g[be * LS] = 0xFFFFFFFFu;
        if (oj == cj) my_cm = left;
        used &= ~(1ull << be);
        nfree += 1;
        next_due = left < others ? left : others;
        return bg;
    };
    auto take_event = [&](double T, int cj, double others) -> uint32_t {
        if constexpr (SH) return pop_event(T, cj);
        uint32_t bg = 0xFFFFFFFFu;
        int be = cj << 3;
        if (others == T) {
            // several chunks hold an event at time T: the smallest group among all of them (rare)
            for (int c = 0; c < nch; ++c) {
                if (cm_t[c * LS] != T) continue;
                for (int u = 0; u < 8; ++u) {
                    const int e = (c << 3) + u;
                    const uint32_t g = ev_g[e * LS];
                    if (ev_t[e * LS] == T && g < bg) {
                        bg = g;
                        be = e;
                    }
                }
            }
            cj = be >> 3;
        }
        if constexpr (OCT) {
            // one slot of the chunk per lane
            const int e = (cj << 3) + oj;
            const double t = ev_t[e * LS];
            if (others != T) {
                const uint32_t g = ev_g[e * LS];
                bg = oct_min(t == T ? g : 0xFFFFFFFFu);
                be = (cj << 3) + __ffs((int)oct_ballot(t == T && g == bg)) - 1;
            }
            const double left = oct_min(e == be ? __builtin_inf() : t);  // earliest time left in the chunk
            ev_t[be * LS] = __builtin_inf();
            ev_g[be * LS] = 0xFFFFFFFFu;
            cm_t[cj * LS] = left;
            fstack[nfree * LS] = (uint16_t)be;
            nfree += 1;
            next_due = left < others ? left : others;
            return bg;
        }
        double t[8];
        uint32_t g[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            t[u] = ev_t[((cj << 3) + u) * LS];
            g[u] = ev_g[((cj << 3) + u) * LS];
        }
        if (others != T) {
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (t[u] == T && g[u] < bg) {
                    bg = g[u];
                    be = (cj << 3) + u;
                }
        }
        double left = __builtin_inf();  // earliest time left in the chunk
#pragma unroll
        for (int u = 0; u < 8; ++u) left = ((cj << 3) + u != be && t[u] < left) ? t[u] : left;
        ev_t[be * LS] = __builtin_inf();
        ev_g[be * LS] = 0xFFFFFFFFu;
        cm_t[cj * LS] = left;
        fstack[nfree * LS] = (uint16_t)be;
        nfree += 1;
        next_due = left < others ? left : others;
        return bg;
    };

    for (int64_t i0 = 0; i0 < R; i0 += kWave) {
    {
        const int64_t at = i0 + lane < R ? i0 + lane : R - 1;
        blk_req = reqs[at];
        g8_next = row_of(__builtin_amdgcn_readlane(blk_req.m, 0));
    }
    const int nj = R - i0 < kWave ? (int)(R - i0) : kWave;
    for (int j = 0; j < nj; ++j) {
        const int64_t i = i0 + j;
        const double tstamp = __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(blk_req.t), j),
                                               __builtin_amdgcn_readlane(__double2loint(blk_req.t), j));
        const int m = __builtin_amdgcn_readlane(blk_req.m, j);
        // the replica list of this request's model was fetched during the previous request; start the next one's
        const uint64_t g8 = g8_next;
        if (j != kWave - 1) {  // the first request of a block gets its list when the block is fetched
            const int mn = __builtin_amdgcn_readlane(blk_req.m, j + 1);
            g8_next = row_of(mn);
        }

        // ---- idle events that are due (:739-744)
        if (!dead && next_due <= tstamp) {
            for (;;) {
                double ti, others;
                int cj;
                chunk_scan(ti, cj, others);
                if (!(ti <= tstamp)) {  // also: no event left
                    next_due = ti;
                    break;
                }
                const uint32_t d = take_event(ti, cj, others);  // sets next_due; handle() lowers it when it adds an earlier event
                const int m2 = select_model(desc_group(d));
                if (m2 < 0) break;  // the popped event is dropped, later due events stay (:742-743)
                handle(ti, m2, d);
                if (dead || !(next_due <= tstamp)) break;
            }
        }

        // ---- the arrival (:746-778)
        bool queued = false;
        uint32_t gsel = none;
        if constexpr (OCT) {
            // One replica per lane: the lane's word is the descriptor of that replica's group.  The clocks of its
            // last and of its first stage and the model's arrival count are read together; the first of the smallest
            // last-stage clocks wins, as in a scan with "<" (:760-770), and whether that group is idle (:776) is one
            // bit of a ballot over the first-stage clocks.
            const uint32_t dj = (uint32_t)g8;
            const bool valid = (int32_t)dj >= 0 && m >= 0;
            const uint32_t last = desc_last_slot(dj);
            const double c = clk[last * LS];                             // slot 0 for a lane without a replica: not used
            const double cf = clk[(last - desc_stages_m1(dj)) * LS];
            uint32_t seen = 0;
            if (m >= 0) seen = arrived[m];
            const uint32_t vb = oct_ballot(valid);
            uint32_t dsel = kEmpty;  // the chosen group's descriptor, once it is needed
            int selj = -1;           // the lane of the octet whose replica was chosen
            bool ready = false;
            if ((vb & 1u) && !dead) {
                double best = 1e100;
                const double mn = oct_min(valid ? c : __builtin_inf());
                if (mn < best) {
                    best = mn;
                    selj = __ffs((int)oct_ballot(valid && c == mn)) - 1;
                    ready = ((oct_ballot(tstamp >= cf) >> selj) & 1u) != 0;
                }
                if (vb >> 7)  // the list may go on
                    for (int x = 0; x < a.rep_extra; ++x) {
                        const uint32_t g = repx_tile[((size_t)m * a.rep_extra + x) * kWave];
                        if (g == none) break;
                        const uint32_t d2 = a.ginfo[((size_t)tile * (Gmax + 1) + g) * kWave + sl];
                        const double c2 = clk[desc_last_slot(d2) * LS];
                        if (c2 < best) {
                            best = c2;
                            selj = -1;
                            dsel = d2;
                            ready = tstamp >= clk[(desc_last_slot(d2) - desc_stages_m1(d2)) * LS];
                        }
                    }
                queued = true;
            }
            if (m >= 0) {
                // every lane sees the same arrival count and writes the same count + 1; lanes that do not host m never
                // read it (a wavefront's LDS accesses are carried out in program order)
                __builtin_amdgcn_wave_barrier();
                arrived[m] = seen + 1u;
                __builtin_amdgcn_wave_barrier();
            }
            if (!queued) {
                if (want_req && !dead) {
                    fin_out[(size_t)i * kWave] = tstamp;
                    good_out[(size_t)i * kWave] = 0;
                }
            } else if (selj < 0 && dsel == kEmpty) {
                // every replica's clock is infinite (only after a batch with infinite latency was accepted under an
                // infinite SLO): the reference's g_id stays -1 here, which its arrays take as "the last group"
                // (controller.py:760-778); that accident is not reproduced
                dead = MMSIM_E_UNSUPPORTED;
            } else if (ready) {  // :776-778
                if (selj >= 0) dsel = oct_get(dj, selj);
                handle(tstamp, m, dsel);
            }
            continue;
        }
        if (m >= 0) {
            const bool hosted = (uint32_t)(g8 & 0xFFu) != none;
            if (hosted && !dead) {
                // group with the strictly smallest last-stage clock (:760-770)
                double best = 1e100;
                bool more = true;  // the list may go on
                for (int j0 = 0; j0 < kPackedReplicas && more; j0 += 4) {  // four replicas at a time: their reads overlap
                    uint32_t g[4], d[4];
                    double c[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) g[u] = (uint32_t)(g8 >> (8 * (j0 + u))) & 0xFFu;
#pragma unroll
                    for (int u = 0; u < 4; ++u) d[u] = ginfo[g[u] * LS];  // the empty row for unused bytes
#pragma unroll
                    for (int u = 0; u < 4; ++u) c[u] = clk[desc_last_slot(d[u]) * LS];
#pragma unroll
                    for (int u = 0; u < 4; ++u)
                        if (g[u] != none && c[u] < best) {
                            best = c[u];
                            gsel = g[u];
                        }
                    more = g[3] != none;
                }
                for (int j = 0; more && j < a.rep_extra; ++j) {
                    const uint32_t g = repx_tile[((size_t)m * a.rep_extra + j) * kWave];
                    if (g == none) break;
                    const double c = clk[desc_last_slot(ginfo[g * LS]) * LS];
                    if (c < best) {
                        best = c;
                        gsel = g;
                    }
                }
                queued = true;
            }
        }
        if (m >= 0) {
            // every lane sees the same arrival count; lanes that do not host m never read it
            // (all lanes read the same count and write the same count + 1: no lane needs to be singled out, and
            // a wavefront's LDS accesses are carried out in program order)
            __builtin_amdgcn_wave_barrier();
            const uint32_t seen = arrived[m];
            arrived[m] = seen + 1u;
            __builtin_amdgcn_wave_barrier();
        }
        if (!queued) {
            if (want_req && !dead) {
                fin_out[(size_t)i * kWave] = tstamp;
                good_out[(size_t)i * kWave] = 0;
            }
        } else if (gsel == none) {
            // every replica's clock is infinite (only after a batch with infinite latency was accepted under an
            // infinite SLO): the reference's g_id stays -1 here, which its arrays take as "the last group"
            // (controller.py:760-778); that accident is not reproduced
            dead = MMSIM_E_UNSUPPORTED;
        } else {
            const uint32_t d = ginfo[gsel * LS];
            const double idle_since = clk[(desc_last_slot(d) - desc_stages_m1(d)) * LS];
            if (tstamp >= idle_since) handle(tstamp, m, d);  // :776-778
        }
    }
    }
    // ---- drain (:781-787)
    while (!dead && nfree < a.heap_cap) {
        double ti, others;
        int cj;
        chunk_scan(ti, cj, others);
        const uint32_t d = take_event(ti, cj, others);
        const int m2 = select_model(desc_group(d));
        if (m2 < 0) continue;
        handle(ti, m2, d);
    }

    if constexpr (COOP) lat_sum = oct_sum(lat_sum);  // each lane summed the batch members it had fetched
    if (oj == 0) {
        const size_t out = (size_t)wave * kWave + sl;
        a.n_good[out] = n_good;
        a.lat_sum[out] = lat_sum;
        a.status[out] = dead;
    }
}

}  // namespace

hipError_t launch_sim_batching(const BatchingArgs &args, int wpb, size_t lds_bytes, hipStream_t stream,
                               std::string *err) {
    hipError_t e = hipSuccess;
    if (wpb < 1 || wpb > kMaxWavesPerBlockBatching || args.NB > kMaxLatencyColumns || (args.heap_cap & 7) != 0) {
        e = hipErrorInvalidValue;
    } else {
        const bool ll = args.lat_lds_bytes > 0, gl = args.g2m_in_lds != 0;
        const bool oct = args.lane_stride == 8, unif = args.uniform_stages != 0;
        const bool small_heap = oct && args.heap_cap <= 64;
        void (*kern)(const BatchingArgs) = nullptr;
#define MMSIM_PICK4(NBT, O, U, S)                                                                               \
    (ll ? (gl ? sim_batching_kernel<NBT, true, true, O, U, S> : sim_batching_kernel<NBT, true, false, O, U, S>) \
        : (gl ? sim_batching_kernel<NBT, false, true, O, U, S> : sim_batching_kernel<NBT, false, false, O, U, S>))
#define MMSIM_PICK3(NBT, O, S) (unif ? MMSIM_PICK4(NBT, O, true, S) : MMSIM_PICK4(NBT, O, false, S))
#define MMSIM_PICK(NBT) kern = !oct ? MMSIM_PICK3(NBT, false, false) : small_heap ? MMSIM_PICK3(NBT, true, true) : MMSIM_PICK3(NBT, true, false)
        if (args.NB <= 4)
            MMSIM_PICK(4);
        else if (args.NB <= 8)
            MMSIM_PICK(8);
        else
            MMSIM_PICK(16);
#undef MMSIM_PICK
#undef MMSIM_PICK3
#undef MMSIM_PICK4
        if (lds_bytes > 64 * 1024)
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)lds_bytes);
        if (e == hipSuccess) {
            const unsigned tile_groups = (unsigned)((args.tiles + wpb - 1) / wpb);
            hipLaunchKernelGGL(kern, dim3(tile_groups * (unsigned)(args.paired ? 1 : args.n_seeds)), dim3(wpb * kWave), lds_bytes, stream, args);
            e = hipGetLastError();
        }
    }
    if (e != hipSuccess && err) *err = std::string("sim_batching launch: ") + hipGetErrorString(e);
    return e;
}

// The template instance launch_sim_batching picks for these arguments, as profilers print it.
std::string sim_batching_kernel_name(const BatchingArgs &args) {
    const int nbt = args.NB <= 4 ? 4 : args.NB <= 8 ? 8 : 16;
    auto tf = [](bool v) { return v ? "true" : "false"; };
    return "sim_batching_kernel<" + std::to_string(nbt) + ", " + tf(args.lat_lds_bytes > 0) + ", " + tf(args.g2m_in_lds != 0) +
           ", " + tf(args.lane_stride == 8) + ", " + tf(args.uniform_stages != 0) + ", " +
           tf(args.lane_stride == 8 && args.heap_cap <= 64) + ">";
}

}  // namespace mmsim
