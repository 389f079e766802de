// Serving statistics of the per-request outputs, computed where they lie in device memory
// (Workload.compute_stats, workload.py:308-354): per (simulation, model) the number of accepted
// requests inside the window that the warm-up trimming leaves, the arrival times of the first and
// the last of them, and the mean, standard deviation, 90th and 99th percentile of their latencies.
//
// One workgroup of 1024 threads per (simulation, model); its threads share the model's requests, which
// the per-model lists of the stream name (index and arrival time).  The first pass gathers the model's
// latencies out of the simulation's column of finish[wave][request][64] / good (one 8-byte element per
// 512-byte row: read once; simulations of one wavefront run side by side, so the rows are shared in L2)
// into a contiguous scratch row, all ones for requests that were not accepted, and counts, sums and bins
// the top byte on the way; every thread later reads back only what it wrote itself.
//
// Percentiles are order statistics: sorted[int(q * n)] (workload.py:344-346), found exactly with a
// radix selection on a 64-bit key that orders like the latency (its bit pattern with the sign handled): eight
// passes of eight bits, most significant first, counting into 256 bins in LDS the elements that match
// the digits fixed so far; both percentiles in the same passes (two histograms).  Latencies are spread
// out, so after two or three digits only a handful of elements still match: once no more than 1024 do
// (for either percentile), they are collected in LDS and ranked there directly, which ends the
// selection in one more sweep instead of up to six (equal latencies by the thousand, as an idle system
// produces, simply run all eight passes).  The first pass also
// counts and sums (n decides the two ranks), the second one sums the squared deviations.  Sums are
// compensated (Neumaier) per thread and added up in a fixed order, so mean and deviation are within a
// few ulp of the exact value, as numpy's pairwise sums are; they are not bit-equal to numpy's.
#include "mmsim_internal.h"

namespace mmsim {
namespace {

constexpr int kBins = 256;

struct Accum {
    double sum = 0.0, comp = 0.0;
    __device__ void add(double x) {  // Neumaier's compensated sum
        const double t = sum + x;
        comp += (fabs(sum) >= fabs(x)) ? (sum - t) + x : (x - t) + sum;
        sum = t;
    }
    __device__ double value() const { return sum + comp; }
};

constexpr int kStatsThreads = 1024;
constexpr int kSmallSelect = 1024;  // candidates that are ranked directly in LDS
// Latencies are selected by a 64-bit key that orders like the double (sign flipped for positive values, all bits
// for negative ones: the batching simulator can finish a request before it arrived, when a group that became idle
// earlier picks it up with its old idle time, controller.py:739-744, :715-720).  All ones is the key of a NaN
// pattern and marks requests that were not accepted.
constexpr uint64_t kNotAccepted = ~0ull;
__device__ inline uint64_t key_of(double v) {
    const uint64_t bits = (uint64_t)__double_as_longlong(v);
    return bits ^ ((uint64_t)((long long)bits >> 63) | 0x8000000000000000ull);
}
__device__ inline double value_of(uint64_t key) {
    const uint64_t bits = (key >> 63) ? key ^ 0x8000000000000000ull : ~key;
    return __longlong_as_double((long long)bits);
}

__device__ inline Accum wave_sum(Accum v) {  // lanes of a wavefront, fixed order
    for (int d = 32; d > 0; d >>= 1) {
        const double s2 = __shfl_down(v.sum, d), c2 = __shfl_down(v.comp, d);
        v.add(s2);
        v.add(c2);
    }
    return v;
}

__global__ __launch_bounds__(kStatsThreads) void model_stats_kernel(StatsArgs a) {
    __shared__ uint32_t hist[2][kBins];
    __shared__ double part_sum[kStatsThreads / kWave], part_comp[kStatsThreads / kWave];
    __shared__ int32_t part_n[kStatsThreads / kWave];
    __shared__ long long part_first[kStatsThreads / kWave], part_last[kStatsThreads / kWave];
    __shared__ uint64_t sh_pre[2];
    __shared__ uint32_t sh_k[2], sh_cand[2], sh_cnt[2];
    __shared__ uint64_t cand[2][kSmallSelect];
    __shared__ double sh_total;
    const int tid = threadIdx.x, wv = tid / kWave, ln = tid % kWave;
    const int row = blockIdx.x, sim = a.sim0 + row, m = blockIdx.y;  // row: the simulation's scratch row in this launch
    const int stream = a.sim_stream[sim];
    const MqEntry *__restrict__ q = a.mq[stream];
    const int64_t lo = a.lo[stream], hi = a.hi[stream];
    auto first_at_least = [&](int64_t b0, int64_t b1, int64_t v) {
        while (b0 < b1) {
            const int64_t mid = b0 + (b1 - b0) / 2;
            if ((int64_t)q[mid].idx < v) b0 = mid + 1; else b1 = mid;
        }
        return b0;
    };
    const int64_t m0 = a.mq_off[(size_t)stream * (a.M + 1) + m], m1 = a.mq_off[(size_t)stream * (a.M + 1) + m + 1];
    const int64_t e0 = first_at_least(m0, m1, lo), e1 = first_at_least(e0, m1, hi);
    const double *__restrict__ fin = a.finish + a.sim_base[sim];
    const uint8_t *__restrict__ gd = a.good + a.sim_base[sim];
    uint64_t *__restrict__ scr = a.scratch + (size_t)row * (size_t)a.scratch_pitch;

    for (int b = tid; b < 2 * kBins; b += kStatsThreads) (&hist[0][0])[b] = 0;
    __syncthreads();

    // pass 0: gather, count, sum, first and last accepted request, top byte
    int32_t n = 0;
    long long first_e = 0x7FFFFFFFFFFFFFFFll, last_e = -1;
    Accum acc;
    for (int64_t e = e0 + tid; e < e1; e += kStatsThreads) {
        const size_t row = (size_t)q[e].idx * kWave;
        const bool ok = gd[row] != 0;
        const double lat = fin[row] - q[e].t;
        const uint64_t bits = ok ? key_of(lat) : kNotAccepted;
        scr[e] = bits;
        if (ok) {
            n += 1;
            acc.add(lat);
            first_e = e < first_e ? e : first_e;
            last_e = e > last_e ? e : last_e;
            atomicAdd(&hist[0][(uint32_t)(bits >> 56)], 1u);
        }
    }
    auto block_sum = [&](Accum v) -> double {  // the workgroup's compensated sum, added up in a fixed order; in every thread
        v = wave_sum(v);
        if (ln == 0) {
            part_sum[wv] = v.sum;
            part_comp[wv] = v.comp;
        }
        __syncthreads();
        if (tid == 0) {
            Accum all;
            for (int w = 0; w < kStatsThreads / kWave; ++w) {
                all.add(part_sum[w]);
                all.add(part_comp[w]);
            }
            sh_total = all.value();
        }
        __syncthreads();
        return sh_total;
    };
    const double lat_sum = block_sum(acc);
    for (int d = 32; d > 0; d >>= 1) {
        n += __shfl_down(n, d);
        const long long f2 = __shfl_down(first_e, d), l2 = __shfl_down(last_e, d);
        first_e = f2 < first_e ? f2 : first_e;
        last_e = l2 > last_e ? l2 : last_e;
    }
    if (ln == 0) {
        part_n[wv] = n;
        part_first[wv] = first_e;
        part_last[wv] = last_e;
    }
    __syncthreads();
    n = 0;
    first_e = 0x7FFFFFFFFFFFFFFFll;
    last_e = -1;
    for (int w = 0; w < kStatsThreads / kWave; ++w) {
        n += part_n[w];
        first_e = part_first[w] < first_e ? part_first[w] : first_e;
        last_e = part_last[w] > last_e ? part_last[w] : last_e;
    }
    const double mean = n > 0 ? lat_sum / (double)n : 0.0;
    double dev_sum = 0.0;

    if (tid == 0) {
        sh_pre[0] = sh_pre[1] = 0;
        sh_k[0] = (uint32_t)(int32_t)(0.90 * (double)n);  // int(0.90 * len(sorted_latency)), workload.py:345
        sh_k[1] = (uint32_t)(int32_t)(0.99 * (double)n);
    }
    __syncthreads();
    for (int pass = 0; pass < 8; ++pass) {
        const int shift = 56 - 8 * pass;
        if (pass > 0) {
            const uint64_t fixed = ~0ull << (shift + 8);
            const uint64_t pre0 = sh_pre[0], pre1 = sh_pre[1];
            Accum dev;
            for (int64_t e = e0 + tid; e < e1; e += kStatsThreads) {
                const uint64_t bits = scr[e];
                if (bits == kNotAccepted) continue;
                if (pass == 1) {
                    const double d = value_of(bits) - mean;
                    dev.add(d * d);
                }
                const uint32_t bin = (uint32_t)(bits >> shift) & (kBins - 1);
                if ((bits & fixed) == pre0) atomicAdd(&hist[0][bin], 1u);
                if ((bits & fixed) == pre1) atomicAdd(&hist[1][bin], 1u);
            }
            if (pass == 1) dev_sum = block_sum(dev);
        }
        __syncthreads();
        if (tid < 2) {  // thread h finds the bin that holds rank k of histogram h (pass 0: both ranks in histogram 0)
            const uint32_t *hh = hist[pass == 0 ? 0 : tid];
            uint32_t k = sh_k[tid], cum = 0, sel = 0, before = 0;
            bool found = false;
            for (int bin = 0; bin < kBins; ++bin) {
                const uint32_t c = hh[bin];
                if (!found && cum + c > k) {
                    found = true;
                    sel = (uint32_t)bin;
                    before = cum;
                }
                cum += c;
            }
            sh_pre[tid] |= (uint64_t)sel << shift;
            sh_k[tid] = k - before;
            sh_cand[tid] = found ? hh[sel] : 0u;  // elements that match the digits fixed so far
            sh_cnt[tid] = 0;
        }
        __syncthreads();
        if (pass >= 1 && pass < 7 && sh_cand[0] <= (uint32_t)kSmallSelect && sh_cand[1] <= (uint32_t)kSmallSelect) {
            // few candidates left: collect them (in any order) and rank them directly; rank sh_k among the
            // candidates of a percentile is its order statistic (equal keys are told apart by their place)
            const uint64_t fixed = ~0ull << shift;
            const uint64_t pre0 = sh_pre[0], pre1 = sh_pre[1];
            for (int64_t e = e0 + tid; e < e1; e += kStatsThreads) {
                const uint64_t bits = scr[e];
                if (bits == kNotAccepted) continue;
                if ((bits & fixed) == pre0) cand[0][atomicAdd(&sh_cnt[0], 1u)] = bits;
                if ((bits & fixed) == pre1) cand[1][atomicAdd(&sh_cnt[1], 1u)] = bits;
            }
            __syncthreads();
            for (int h = 0; h < 2; ++h) {
                const uint32_t c = sh_cnt[h];
                if ((uint32_t)tid < c) {
                    const uint64_t mine = cand[h][tid];
                    uint32_t rank = 0;
                    for (uint32_t j = 0; j < c; ++j) {
                        const uint64_t other = cand[h][j];
                        rank += (other < mine || (other == mine && j < (uint32_t)tid)) ? 1u : 0u;
                    }
                    if (rank == sh_k[h]) sh_pre[h] = mine;
                }
            }
            __syncthreads();
            break;
        }
        for (int b = tid; b < 2 * kBins; b += kStatsThreads) (&hist[0][0])[b] = 0;
        __syncthreads();
    }

    if (tid != 0) return;
    const size_t o = (size_t)sim * a.M + m;
    a.model_req[o] = (int32_t)(e1 - e0);
    a.model_good[o] = n;
    a.first_start[o] = n > 0 ? q[first_e].t : 0.0;
    a.last_start[o] = n > 0 ? q[last_e].t : 0.0;
    a.latency_sum[o] = n > 0 ? lat_sum : 0.0;
    a.latency_mean[o] = mean;
    a.latency_std[o] = n > 0 ? sqrt(dev_sum / (double)n) : 0.0;
    a.latency_p90[o] = n > 0 ? value_of(sh_pre[0]) : 0.0;
    a.latency_p99[o] = n > 0 ? value_of(sh_pre[1]) : 0.0;
}

}  // namespace

hipError_t launch_model_stats(const StatsArgs &args, int n_sims, hipStream_t stream, std::string *err) {
    if (n_sims <= 0 || args.M <= 0) return hipSuccess;
    if (args.M > 65535) {
        if (err) *err = "model_stats_kernel: more than 65535 models";
        return hipErrorInvalidValue;
    }
    hipLaunchKernelGGL(model_stats_kernel, dim3((unsigned)n_sims, (unsigned)args.M), dim3(kStatsThreads), 0, stream, args);
    return hipGetLastError();
}

}  // namespace mmsim
