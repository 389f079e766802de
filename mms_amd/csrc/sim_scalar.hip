// Scalar-clock request loop for gfx950.
//
// Restates the reference's simulate_requests (alpa_serve/simulator/controller.py:506-558), the variant
// that approximate_one_case_one_placement runs with mixed=False: one clock per group, a request
// finishes at max(clock, arrival) + the sum of the group's stage latencies + the fixed overhead and,
// if accepted, moves the clock to max(clock, arrival) + the largest stage latency.  No public caller of
// the reference passes mixed=False (controller.py:410), so this is a single-placement entry point
// only: one wavefront fetches 64 requests at a time, hands them out with v_readlane, and all of its
// lanes carry the same state; lane 0 writes the results.

#include "mmsim_internal.h"

namespace mmsim {

namespace {

__global__ __launch_bounds__(kWave) void sim_scalar_kernel(const ScalarArgs a) {
    __shared__ double clk[MMSIM_MAX_GROUPS];
    const int lane = (int)threadIdx.x;
    for (int g = lane; g < a.G; g += kWave) clk[g] = 0.0;
    __syncthreads();
    for (int64_t i0 = 0; i0 < a.R; i0 += kWave) {
        const int64_t at = i0 + lane < a.R ? i0 + lane : a.R - 1;
        const double my_t = a.tstamps[at];
        const int my_m = a.model_ids[at];
        const float my_slo = a.slos[at];
        const int n = (int)(a.R - i0 < kWave ? a.R - i0 : kWave);
        for (int k = 0; k < n; ++k) {
            const double tstamp = __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(my_t), k),
                                                   __builtin_amdgcn_readlane(__double2loint(my_t), k));
            const int m = __builtin_amdgcn_readlane(my_m, k);
            const double slo = (double)__int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_slo), k));
            double finish = tstamp;
            bool good = false;
            if (m >= 0) {  // :522-526
                if (lane == 0) a.model_req[m] += 1;
                // the group with the strictly smallest clock, first listed wins ties (:529-536)
                int g_id = -1;
                double min_clock = __builtin_inf();
                const int32_t *row = a.m_id2g_id + (size_t)m * a.G;
                for (int j = 0; j < a.G; ++j) {
                    const int g = row[j];
                    if (g < 0) break;
                    const double c = clk[g];
                    if (c < min_clock) {
                        min_clock = c;
                        g_id = g;
                    }
                }
                if (g_id >= 0) {  // :543-555
                    const double c = clk[g_id];
                    const double start_time = c > tstamp ? c : tstamp;
                    const double finish_time = start_time + (double)a.group_sum_latency[(size_t)m * a.G + g_id] + a.fixed_overhead;
                    if (lane == 0) a.group_req[g_id] += 1;
                    if (finish_time - tstamp <= slo) {
                        finish = finish_time;
                        good = true;
                        clk[g_id] = start_time + (double)a.group_max_latency[(size_t)m * a.G + g_id];
                        if (lane == 0) {
                            a.group_good[g_id] += 1;
                            a.model_good[m] += 1;
                        }
                    }
                }
            }
            if (lane == 0) {
                a.finish[i0 + k] = finish;
                a.good[i0 + k] = good ? 1 : 0;
            }
        }
    }
}

}  // namespace

hipError_t launch_sim_scalar(const ScalarArgs &args, hipStream_t stream, std::string *err) {
    hipLaunchKernelGGL(sim_scalar_kernel, dim3(1), dim3(kWave), 0, stream, args);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess && err) *err = std::string("sim_scalar launch: ") + hipGetErrorString(e);
    return e;
}

}  // namespace mmsim
