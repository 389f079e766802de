// Serving statistics of the per-request outputs, computed where they lie in device memory
// (Workload.compute_stats, workload.py:308-354): per (simulation, model) the number of accepted
// requests inside the window that the warm-up trimming leaves, the arrival times of the first and
// the last of them, and the mean, standard deviation, 90th and 99th percentile of their latencies.
//
// One workgroup per (wavefront of simulations, model): lane = simulation, as in the simulators, so
// finish[wave][request][64] is read a coalesced row at a time.  The requests of a model are the same
// for every lane (the per-model lists of the stream), only `good` differs.  The workgroup's eight
// wavefronts take contiguous slices of the model's requests and count into the same histograms.
//
// Percentiles are order statistics: sorted[int(q * n)] (workload.py:344-346), found exactly with a
// radix selection on the bit pattern of the latency (positive doubles order as their bits do): eight
// passes of eight bits, most significant first, each lane counting into its own 256 bins in LDS the
// elements that match the digits it has fixed so far.  Both percentiles are selected in the same
// passes (two histograms).  The first pass also counts and sums (n decides the two ranks), the
// second one sums the squared deviations.  Sums are compensated (Neumaier), so mean and deviation
// are within a few ulp of the exact value, as numpy's pairwise sums are; they are not bit-equal to
// numpy's.
#include "mmsim_internal.h"

namespace mmsim {
namespace {

constexpr int kBins = 256;
constexpr int kUnroll = 8;
constexpr int kStatsWaves = 8;  // wavefronts of a workgroup; they share one pair of histograms

struct Accum {
    double sum = 0.0, comp = 0.0;
    __device__ void add(double x) {  // Neumaier's compensated sum
        const double t = sum + x;
        comp += (fabs(sum) >= fabs(x)) ? (sum - t) + x : (x - t) + sum;
        sum = t;
    }
    __device__ double value() const { return sum + comp; }
};

// Finds the bin that holds rank k of a lane's histogram column (read only: every wavefront of the
// workgroup does the same search and must find the same bin).
__device__ inline void pick_bin(const uint32_t *col, uint32_t &k, uint64_t &prefix, int shift) {
    uint32_t cum = 0, before = 0, sel = 0;
    bool found = false;
#pragma unroll 8
    for (int bin = 0; bin < kBins; ++bin) {
        const uint32_t c = col[bin * kWave];
        if (!found && cum + c > k) {
            found = true;
            sel = (uint32_t)bin;
            before = cum;
        }
        cum += c;
    }
    prefix |= (uint64_t)sel << shift;
    k -= before;
}

// What a wavefront found in its slice of a model's requests, handed to the others through LDS.
struct Partial {
    double sum[kStatsWaves][kWave], comp[kStatsWaves][kWave], first[kStatsWaves][kWave], last[kStatsWaves][kWave];
    int32_t n[kStatsWaves][kWave];
};

__global__ __launch_bounds__(kStatsWaves *kWave) void model_stats_kernel(StatsArgs a) {
    extern __shared__ uint32_t hist[];  // [2][kBins][64], then Partial
    Partial &part = *reinterpret_cast<Partial *>(hist + 2 * kBins * kWave);
    const int lane = threadIdx.x % kWave, wv = threadIdx.x / kWave;
    const int wave = blockIdx.x;
    const int m = blockIdx.y;
    const int stream = a.paired ? a.tile_seed[wave] : wave / a.tiles;
    const MqEntry *__restrict__ q = a.mq[stream];
    const int64_t lo = a.lo[stream], hi = a.hi[stream];
    // a model's entries are in stream order: cut [e0, e1) down to the requests of the window [lo, hi)
    auto first_at_least = [&](int64_t b0, int64_t b1, int64_t v) {
        while (b0 < b1) {
            const int64_t mid = b0 + (b1 - b0) / 2;
            if ((int64_t)q[mid].idx < v) b0 = mid + 1; else b1 = mid;
        }
        return b0;
    };
    const int64_t m0 = a.mq_off[(size_t)stream * (a.M + 1) + m], m1 = a.mq_off[(size_t)stream * (a.M + 1) + m + 1];
    const int64_t e0 = first_at_least(m0, m1, lo), e1 = first_at_least(e0, m1, hi);
    // the wavefronts of the workgroup share the model's requests in contiguous slices, in order
    const int64_t per = (e1 - e0 + kStatsWaves - 1) / kStatsWaves;
    const int64_t s0 = std::min(e1, e0 + wv * per), s1 = std::min(e1, s0 + per);

    uint32_t *col0 = hist + lane, *col1 = hist + kBins * kWave + lane;
    auto clear = [&]() {  // each wavefront clears its share of the bins
        for (int bin = wv; bin < kBins; bin += kStatsWaves) col0[bin * kWave] = col1[bin * kWave] = 0;
    };
    clear();
    __syncthreads();

    const size_t base = (size_t)wave * (size_t)a.Rmax * kWave + lane;
    const double *__restrict__ fin = a.finish + base;
    const uint8_t *__restrict__ gd = a.good + base;

    int32_t n = 0;
    double first = 0.0, last = 0.0, mean = 0.0, lat_sum = 0.0, dev_sum = 0.0;
    Accum acc;
    uint64_t pre0 = 0, pre1 = 0;
    uint32_t k0 = 0, k1 = 0;

    for (int pass = 0; pass < 8; ++pass) {
        const int shift = 56 - 8 * pass;
        const uint64_t fixed = pass == 0 ? 0ull : ~0ull << (shift + 8);  // digits the earlier passes have fixed
        auto take = [&](bool ok, double lat, double t) {
            if (!ok) return;
            const uint64_t bits = (uint64_t)__double_as_longlong(lat);
            if (pass == 0) {
                if (n == 0) first = t;
                last = t;
                n += 1;
                acc.add(lat);
            } else if (pass == 1) {
                const double d = lat - mean;
                acc.add(d * d);
            }
            const uint32_t bin = (uint32_t)(bits >> shift) & (kBins - 1);
            if ((bits & fixed) == pre0) atomicAdd(&col0[bin * kWave], 1u);
            if ((bits & fixed) == pre1) atomicAdd(&col1[bin * kWave], 1u);
        };
        // A block's rows are fetched together, and the entries of the next block (clamped to the slice) while
        // this one is counted: the loop is bound by memory latency.
        int32_t idx[kUnroll];
        double t[kUnroll];
        auto entries = [&](int64_t e) {
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const int64_t at = std::min(e + u, s1 - 1);
                idx[u] = q[at].idx;
                t[u] = q[at].t;
            }
        };
        if (s0 < s1) entries(s0);
        for (int64_t e = s0; e < s1; e += kUnroll) {
            double f[kUnroll], at_t[kUnroll];
            uint8_t g[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const size_t row = (size_t)idx[u] * kWave;
                f[u] = fin[row];
                g[u] = gd[row];
                at_t[u] = t[u];
            }
            entries(e + kUnroll);
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) take(e + u < s1 && g[u] != 0, f[u] - at_t[u], at_t[u]);
        }
        if (pass <= 1) {  // the slices' counts and compensated sums, added up in slice order by every wavefront
            part.sum[wv][lane] = acc.sum;
            part.comp[wv][lane] = acc.comp;
            if (pass == 0) {
                part.n[wv][lane] = n;
                part.first[wv][lane] = first;
                part.last[wv][lane] = last;
            }
        }
        __syncthreads();
        if (pass <= 1) {
            Accum all;
            int32_t count = 0;
            for (int w = 0; w < kStatsWaves; ++w) {
                all.add(part.sum[w][lane]);
                all.add(part.comp[w][lane]);
                if (pass == 0 && part.n[w][lane] > 0) {
                    if (count == 0) first = part.first[w][lane];
                    last = part.last[w][lane];
                    count += part.n[w][lane];
                }
            }
            if (pass == 0) {
                n = count;
                lat_sum = all.value();
                mean = n > 0 ? lat_sum / (double)n : 0.0;
                k0 = (uint32_t)(int32_t)(0.90 * (double)n);  // int(0.90 * len(sorted_latency)), workload.py:345
                k1 = (uint32_t)(int32_t)(0.99 * (double)n);
            } else {
                dev_sum = all.value();
            }
            acc = Accum();
        }
        pick_bin(col0, k0, pre0, shift);
        pick_bin(col1, k1, pre1, shift);
        __syncthreads();  // everyone has read the bins (and the partial sums)
        clear();
        __syncthreads();
    }

    if (wv != 0) return;
    const size_t o = ((size_t)wave * a.M + m) * kWave + lane;
    a.model_req[o] = (int32_t)(e1 - e0);
    a.model_good[o] = n;
    a.first_start[o] = first;
    a.last_start[o] = last;
    a.latency_sum[o] = n > 0 ? lat_sum : 0.0;
    a.latency_mean[o] = mean;  // a model without accepted requests reports the latencies [0] (workload.py:340-342)
    a.latency_std[o] = n > 0 ? sqrt(dev_sum / (double)n) : 0.0;
    a.latency_p90[o] = n > 0 ? __longlong_as_double((long long)pre0) : 0.0;
    a.latency_p99[o] = n > 0 ? __longlong_as_double((long long)pre1) : 0.0;
}

}  // namespace

hipError_t launch_model_stats(const StatsArgs &args, int waves, hipStream_t stream, std::string *err) {
    constexpr size_t lds = 2 * kBins * kWave * sizeof(uint32_t) + sizeof(Partial);
    if (waves <= 0 || args.M <= 0) return hipSuccess;
    if (args.M > 65535) {
        if (err) *err = "model_stats_kernel: more than 65535 models";
        return hipErrorInvalidValue;
    }
    hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void *>(model_stats_kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (rc != hipSuccess) {
        if (err) *err = "model_stats_kernel: cannot raise the LDS limit";
        return rc;
    }
    hipLaunchKernelGGL(model_stats_kernel, dim3((unsigned)waves, (unsigned)args.M), dim3(kStatsWaves * kWave), lds, stream, args);
    return hipGetLastError();
}

}  // namespace mmsim
