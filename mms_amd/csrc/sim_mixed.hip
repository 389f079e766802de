// Plain (non-batching) request-loop simulation for gfx950.
//
// Restates the reference's simulate_requests_mixed
// (alpa_serve/simulator/controller.py:561-628) for a whole batch of candidate
// placements at once.  One lane simulates one (placement, arrival seed) pair;
// the 64 lanes of a wavefront hold 64 placements that walk the SAME request
// stream in lockstep, so everything that depends only on the request
// (arrival time, model id, SLO) is wave-uniform and is fetched with scalar
// loads, while everything that depends on the placement is per lane:
//
//   * per-lane stage clocks live in LDS as clk[slot][lane] (8 bytes each).
//     The slots of a lane are its groups' pipeline stages laid end to end;
//     the bank an access hits depends on the lane only, so any per-lane slot
//     choice is conflict free.
//   * the replicas of the request's model are 32-bit descriptors
//     rep[tile][model][j][lane] (coalesced 256-byte rows), listed in the
//     order the reference scans them; a descriptor carries the group's first
//     slot, stage count, latency-table column and group index.
//   * group choice (strictly smallest last-stage clock, first listed wins
//     ties) and the SLO decision are selects / exec-masked stores, with
//     wave-uniform early exits when no lane has another replica or stage.
//
// Arithmetic is fp64 add / max / sub / compare in the reference's order;
// fp32 operands (latencies, SLOs) are widened first.  Compiled with
// -ffp-contract=off (there is no multiply to contract anyway).
//
// Workgroup = one wavefront.  Lanes never exchange data, so there are no
// barriers.  blockIdx.x = tile * n_seeds + seed, which puts the waves that
// read the same stream on the same XCD when n_seeds is a multiple of 8.

#include "mmsim_internal.h"

namespace mmsim {

namespace {

template <int N>
struct ChunkFor {
    // requests whose descriptors are fetched ahead as one group; bounded so
    // that the descriptor registers of a chunk stay within ~64 VGPRs
    static constexpr int value = N <= 8 ? 8 : (N <= 16 ? 4 : (N <= 32 ? 2 : 1));
};

template <int SMAX, int RMAX>
__global__ __launch_bounds__(kWave) void sim_mixed_kernel(const MixedArgs a) {
    extern __shared__ double lds_clk[];  // [nslots][64] then optional group counters

    const int lane = threadIdx.x;
    const int seed = blockIdx.x % a.n_seeds;
    const int tile = blockIdx.x / a.n_seeds;
    const int wave = seed * a.tiles + tile;
    const bool want_model = (a.flags & MMSIM_WANT_MODEL_COUNTS) != 0;
    const bool want_group = (a.flags & MMSIM_WANT_GROUP_COUNTS) != 0;
    const bool want_req = (a.flags & MMSIM_WANT_PER_REQUEST) != 0;
    const bool want_ops = (a.flags & MMSIM_WANT_OP_COUNT) != 0;

    double *clk = lds_clk + lane;  // clk[slot * 64]
    for (int s = 0; s < a.nslots; ++s) clk[s * kWave] = 0.0;
    uint32_t *gcnt = reinterpret_cast<uint32_t *>(lds_clk + (size_t)a.nslots * kWave) + lane;
    if (want_group)
        for (int g = 0; g < 2 * a.Gmax; ++g) gcnt[g * kWave] = 0u;

    const int64_t off = a.stream_off[seed];
    const int64_t R = a.stream_off[seed + 1] - off;
    const Req *__restrict__ reqs = a.streams + off;
    const uint32_t *__restrict__ rep_tile = a.rep + (size_t)tile * a.M * RMAX * kWave + lane;
    const int32_t *__restrict__ rmax_tile = a.rmax + (size_t)tile * a.M;
    const float *__restrict__ lat = a.lat;
    int32_t *model_good = a.model_good + (size_t)wave * a.M * kWave + lane;
    double *fin_out = a.finish + (size_t)wave * a.Rmax * kWave + lane;
    uint8_t *good_out = a.good + (size_t)wave * a.Rmax * kWave + lane;

    int32_t n_good = 0;
    double lat_sum = 0.0;
    int64_t fp_ops = 0;

    constexpr int CH = ChunkFor<RMAX>::value;

    for (int64_t base = 0; base < R; base += CH) {
        Req rq[CH];
        int32_t nrep[CH];
        uint32_t desc[CH][RMAX];
#pragma unroll
        for (int u = 0; u < CH; ++u) {
            const int64_t i = base + u < R ? base + u : R - 1;
            rq[u] = reqs[i];
        }
#pragma unroll
        for (int u = 0; u < CH; ++u) {
            const bool live = base + u < R && rq[u].m >= 0;
            nrep[u] = live ? rmax_tile[rq[u].m] : 0;
        }
#pragma unroll
        for (int u = 0; u < CH; ++u) {
            const uint32_t *row = rep_tile + (size_t)(rq[u].m < 0 ? 0 : rq[u].m) * RMAX * kWave;
#pragma unroll
            for (int j = 0; j < RMAX; ++j) desc[u][j] = j < nrep[u] ? row[j * kWave] : kEmpty;
        }

#pragma unroll
        for (int u = 0; u < CH; ++u) {
            if (base + u >= R) break;
            const double tstamp = rq[u].t;
            const int32_t m = rq[u].m;
            const double slo = (double)rq[u].slo;

            // ---- choose the replica group: strictly smallest last-stage clock (:590-598)
            double best = 1e100;
            uint32_t sel = kEmpty;
            int nvalid = 0;
#pragma unroll
            for (int j = 0; j < RMAX; ++j) {
                if (j >= nrep[u]) break;  // wave-uniform
                const uint32_t d = desc[u][j];
                const bool valid = d != kEmpty;
                nvalid += valid ? 1 : 0;
                const uint32_t last = valid ? desc_slot0(d) + desc_stages(d) - 1u : 0u;
                const double c = clk[last * kWave];
                const bool better = valid && c < best;
                best = better ? c : best;
                sel = better ? d : sel;
            }
            const bool has = sel != kEmpty;
            const int S = has ? (int)desc_stages(sel) : 0;
            const uint32_t slot0 = has ? desc_slot0(sel) : 0u;
            const float *lrow = lat + ((size_t)(m < 0 ? 0 : m) * a.C + (has ? desc_cfg(sel) : 0u)) * a.lat_stride;
            double *gclk = clk + slot0 * kWave;

            // ---- walk the pipeline stages (:605-608)
            double t = tstamp;
            double tmp[SMAX];
            int kdone = 0;  // wave-uniform: stages walked by the deepest lane
#pragma unroll
            for (int k = 0; k < SMAX; ++k) {
                const bool active = k < S;
                if (__ballot(active) == 0ull) break;
                kdone = k + 1;
                if (active) {
                    const double c = gclk[k * kWave];
                    const double l = (double)lrow[k];
                    t = (c > t ? c : t) + l;
                    tmp[k] = t;
                }
            }
            const double finish_time = t + a.fixed_overhead;  // :610
            const double latency = finish_time - tstamp;
            const bool acc = has && latency <= slo;  // :613

            if (acc) {  // :614-619
                n_good += 1;
                lat_sum += latency;
            }
#pragma unroll
            for (int k = 0; k < SMAX; ++k) {
                if (k >= kdone) break;
                if (acc && k < S) gclk[k * kWave] = tmp[k];
            }
            if (want_group && has) {  // :611, :618
                const uint32_t g = desc_group(sel);
                gcnt[g * kWave] += 1u;
                if (acc) gcnt[(a.Gmax + g) * kWave] += 1u;
            }
            if (want_ops && has) fp_ops += 2 * S + nvalid + 3;
            if (want_model && m >= 0) model_good[(size_t)m * kWave] += acc ? 1 : 0;
            if (want_req) {
                fin_out[(base + u) * kWave] = acc ? finish_time : tstamp;
                good_out[(base + u) * kWave] = acc ? 1 : 0;
            }
        }
    }

    const size_t out = (size_t)seed * a.tiles * kWave + (size_t)tile * kWave + lane;
    a.n_good[out] = n_good;
    a.lat_sum[out] = lat_sum;
    if (want_ops) a.fp_ops[out] = fp_ops;
    if (want_group) {
        int32_t *greq = a.group_req + (size_t)wave * a.Gmax * kWave + lane;
        int32_t *ggood = a.group_good + (size_t)wave * a.Gmax * kWave + lane;
        for (int g = 0; g < a.Gmax; ++g) {
            greq[g * kWave] = (int32_t)gcnt[g * kWave];
            ggood[g * kWave] = (int32_t)gcnt[(a.Gmax + g) * kWave];
        }
    }
}

template <int SMAX, int RMAX>
hipError_t launch_one(const MixedArgs &args, size_t lds_bytes, hipStream_t stream) {
    auto kern = sim_mixed_kernel<SMAX, RMAX>;
    if (lds_bytes > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (e != hipSuccess) return e;
    }
    const dim3 grid((unsigned)(args.tiles * args.n_seeds));
    hipLaunchKernelGGL(kern, grid, dim3(kWave), lds_bytes, stream, args);
    return hipGetLastError();
}

template <int SMAX>
hipError_t launch_r(const MixedArgs &args, int rb, size_t lds_bytes, hipStream_t stream) {
    switch (rb) {
        case 1: return launch_one<SMAX, 1>(args, lds_bytes, stream);
        case 2: return launch_one<SMAX, 2>(args, lds_bytes, stream);
        case 4: return launch_one<SMAX, 4>(args, lds_bytes, stream);
        case 8: return launch_one<SMAX, 8>(args, lds_bytes, stream);
        case 16: return launch_one<SMAX, 16>(args, lds_bytes, stream);
        case 64: return launch_one<SMAX, 64>(args, lds_bytes, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

int smax_bucket_for(int smax) {
    for (int b : {1, 4, 8, 16, 32})
        if (smax <= b) return b;
    return -1;
}

int rmax_bucket_for(int rmax) {
    for (int b : {1, 2, 4, 8, 16, 64})
        if (rmax <= b) return b;
    return -1;
}

hipError_t launch_sim_mixed(const MixedArgs &args, int sb, int rb, size_t lds_bytes, hipStream_t stream,
                            std::string *err) {
    hipError_t e;
    switch (sb) {
        case 1: e = launch_r<1>(args, rb, lds_bytes, stream); break;
        case 4: e = launch_r<4>(args, rb, lds_bytes, stream); break;
        case 8: e = launch_r<8>(args, rb, lds_bytes, stream); break;
        case 16: e = launch_r<16>(args, rb, lds_bytes, stream); break;
        case 32: e = launch_r<32>(args, rb, lds_bytes, stream); break;
        default: e = hipErrorInvalidValue; break;
    }
    if (e != hipSuccess && err) *err = std::string("sim_mixed launch: ") + hipGetErrorString(e);
    return e;
}

}  // namespace mmsim
