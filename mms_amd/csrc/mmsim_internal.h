// Internal declarations shared by the host API and the kernel launchers of libmmsim.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>
#include <vector>

#include "../../include/mmsim.h"

namespace mmsim {

// One request as the kernels read it: 16 bytes, so a block of 64 requests is
// one coalesced 1 KiB load per wavefront.
struct __attribute__((aligned(16))) Req {
    double t;
    int32_t m;
    float slo;
};
static_assert(sizeof(Req) == 16, "Req must be 16 bytes");

// Group descriptor: one 32-bit word per (placement, group).  The plain simulator
// reads a model's replicas as descriptors; the batching simulator keeps a per
// lane table of them in LDS and lists replicas as group indices.
//   bits  0..7   clock slot of the group's LAST pipeline stage (slots are the
//                placement's pipeline stages laid end to end)
//   bits  8..12  stages of the group minus one
//   bits 13..22  offset of the group's configuration inside a model's row of
//                the compact latency table
//   bits 23..30  group index within the placement
// kEmpty (sign bit set, slot field 0) marks "no such group".
//
// The replicas of a model are listed as group indices, one byte each, eight to
// a 64-bit word per (placement, model); unused bytes hold the index of the
// extra, empty descriptor row (num_groups_max).
constexpr uint32_t kEmpty = 0x80000000u;
__host__ __device__ inline uint32_t pack_desc(uint32_t slot0, uint32_t stages, uint32_t lat_off, uint32_t group) {
    return (slot0 + stages - 1u) | ((stages - 1u) << 8) | (lat_off << 13) | (group << 23);
}
__host__ __device__ inline uint32_t desc_last_slot(uint32_t d) { return d & 0xFFu; }
__host__ __device__ inline uint32_t desc_stages_m1(uint32_t d) { return (d >> 8) & 0x1Fu; }
__host__ __device__ inline uint32_t desc_lat_off(uint32_t d) { return (d >> 13) & 0x3FFu; }
__host__ __device__ inline uint32_t desc_group(uint32_t d) { return (d >> 23) & 0xFFu; }
constexpr int kMaxLatRow = 1023;  // floats per model in the compact latency table
constexpr int kPackedReplicas = 8;

constexpr int kWave = 64;
constexpr int kStageBytes = kWave * (int)sizeof(Req);  // one staged block of requests

// Arguments of the plain (non-batching) simulation kernel.
struct MixedArgs {
    const Req *streams;          // all seeds' requests, back to back
    const int64_t *stream_off;   // [n_seeds+1] element offsets into streams
    const uint4 *rep32;          // [tiles][M][2][64] descriptors of the first 8 replicas, four to a 16-byte word
    const uint32_t *repx32;      // [tiles][M][rep_extra][64] descriptors of replicas 8, 9, ...
    const uint8_t *rmax;         // [tiles][M] most replicas of model m over the tile's lanes
    const float *lat;            // [M][lat_row] compact stage latencies (batch size 1)
    int32_t M, lat_row, rep_extra;
    int32_t n_seeds, B, tiles, nslots, Gmax;
    int32_t lat_in_lds;          // 1: the block keeps a copy of lat in LDS
    int32_t uniform_stages;      // 1: all stages of a (model, config) have the same latency; lat is [M][C]
    int32_t pow2_depths;         // 1: every group of the batch has 1, 2, 4, 8 or 16 stages
    int32_t wave_lds_bytes;      // LDS bytes of one wavefront's private region
    int32_t rmax_lds_bytes;      // M rounded up to 16
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

// Arguments of the batching simulation kernel.  Replica lists and group
// descriptors are shared with the plain kernel; on top come, per seed, the
// arrivals regrouped by model (a model's FIFO is always a window of that list)
// and, per lane, the models of each group.
struct BatchingArgs {
    const Req *streams;          // all seeds' requests, back to back
    const int64_t *stream_off;   // [n_seeds+1]
    const int64_t *mq_off;       // [n_seeds][M+1] offsets into mq_* of the arrivals of each model
    const double *mq_t;          // arrival time of each model-ordered arrival
    const double *mq_dl;         // its deadline: arrival + (double)slo
    const int32_t *mq_idx;       // its index in the seed's stream
    const uint64_t *rep8;        // as in MixedArgs
    const uint8_t *repx;
    const uint32_t *ginfo;       // [tiles][Gmax+1][64]
    const uint16_t *g2m_off;     // [tiles][Gmax+1][64] start of each group's model list
    const uint16_t *g2m_idx;     // [tiles][members_max][64] model ids, ascending per group
    const float *lat;            // [M][lat_row][NB]
    const int32_t *batch_sizes;  // [NB]
    int32_t M, lat_row, NB, rep_extra, members_max, heap_cap;
    int32_t n_seeds, B, tiles, nslots, Gmax;
    int32_t wave_lds_bytes;
    int64_t Rmax;
    double fixed_overhead;
    uint32_t flags;
    // outputs
    int32_t *n_good;             // [n_seeds][tiles*64]
    double *lat_sum;             // [n_seeds][tiles*64]
    int32_t *status;             // [n_seeds][tiles*64] 0 or MMSIM_E_OVERFLOW
    int32_t *model_good;         // [waves][M][64]
    int32_t *group_req;          // [waves][Gmax][64]
    int32_t *group_good;         // [waves][Gmax][64]
    double *finish;              // [waves][Rmax][64]
    uint8_t *good;               // [waves][Rmax][64]
};
hipError_t launch_sim_batching(const BatchingArgs &args, int waves_per_block, size_t lds_bytes, hipStream_t stream,
                               std::string *err);

// Launches the plain simulator with `waves_per_block` wavefronts per workgroup.
hipError_t launch_sim_mixed(const MixedArgs &args, int smax_bucket, int waves_per_block, size_t lds_bytes,
                            hipStream_t stream, std::string *err);
// Smallest compiled stage bucket >= value, or -1.
int smax_bucket_for(int smax);
constexpr int kMaxWavesPerBlock = 8;          // plain simulator
constexpr int kMaxWavesPerBlockBatching = 4;  // batching simulator

}  // namespace mmsim
