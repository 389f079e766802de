// Internal declarations shared by the host API and the kernel launchers of libmmsim.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>
#include <vector>

#include "../../include/mmsim.h"

namespace mmsim {

// One request as the kernels read it: 16 bytes, so a wavefront fetches a
// request with one scalar 128-bit load.
struct __attribute__((aligned(16))) Req {
    double t;
    int32_t m;
    float slo;
};
static_assert(sizeof(Req) == 16, "Req must be 16 bytes");

// Replica descriptor: one 32-bit word per (placement, model, replica).
//   bits  0..7   first clock slot of the group (slots are the placement's
//                pipeline stages laid end to end)
//   bits  8..12  stages of the group minus one
//   bits 13..20  configuration index (column of the latency table)
//   bits 21..28  group index within the placement
// kEmpty marks "no such replica".
constexpr uint32_t kEmpty = 0xFFFFFFFFu;
__host__ __device__ inline uint32_t pack_desc(uint32_t slot0, uint32_t stages, uint32_t cfg, uint32_t group) {
    return slot0 | ((stages - 1u) << 8) | (cfg << 13) | (group << 21);
}
__host__ __device__ inline uint32_t desc_slot0(uint32_t d) { return d & 0xFFu; }
__host__ __device__ inline uint32_t desc_stages(uint32_t d) { return ((d >> 8) & 0x1Fu) + 1u; }
__host__ __device__ inline uint32_t desc_cfg(uint32_t d) { return (d >> 13) & 0xFFu; }
__host__ __device__ inline uint32_t desc_group(uint32_t d) { return (d >> 21) & 0xFFu; }

constexpr int kWave = 64;

// Arguments of the plain (non-batching) simulation kernel.
struct MixedArgs {
    const Req *streams;          // all seeds' requests, back to back
    const int64_t *stream_off;   // [n_seeds+1] element offsets into streams
    const uint32_t *rep;         // [tiles][M][rmax_bucket][64] replica descriptors
    const int32_t *rmax;         // [tiles][M] most replicas of model m over the tile's lanes
    const float *lat;            // [M][C][lat_stride] stage latencies (batch size 1)
    int32_t M, C, lat_stride;
    int32_t n_seeds, B, tiles, nslots, Gmax;
    int64_t Rmax;                // longest stream (row pitch of per-request outputs)
    double fixed_overhead;
    uint32_t flags;
    // outputs
    int32_t *n_good;             // [n_seeds][tiles*64]
    double *lat_sum;             // [n_seeds][tiles*64]
    int32_t *model_good;         // [waves][M][64]
    int32_t *group_req;          // [waves][Gmax][64]
    int32_t *group_good;         // [waves][Gmax][64]
    double *finish;              // [waves][Rmax][64]
    uint8_t *good;               // [waves][Rmax][64]
    int64_t *fp_ops;             // [n_seeds][tiles*64]
};

// Picks the compiled (stage, replica) bucket and launches.  Returns a HIP error.
hipError_t launch_sim_mixed(const MixedArgs &args, int smax, int rmax_bucket, size_t lds_bytes,
                            hipStream_t stream, std::string *err);
// Smallest compiled bucket >= value, or -1.
int smax_bucket_for(int smax);
int rmax_bucket_for(int rmax);

}  // namespace mmsim
