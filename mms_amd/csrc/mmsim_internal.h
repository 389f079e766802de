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

// One arrival in a seed's arrivals regrouped by model (batching simulator): a model's FIFO is always
// a window of that list.  rank is the dense rank of the arrival time among the seed's arrival times,
// so comparing ranks is comparing times (the reference compares times, ties keep the earlier-listed
// model) without fetching them.
struct __attribute__((aligned(32))) MqEntry {
    double t;      // arrival time
    double dl;     // deadline: arrival + (double)slo
    int32_t idx;   // index in the seed's stream
    int32_t rank;
    int32_t pad[2];
};
static_assert(sizeof(MqEntry) == 32, "MqEntry must be 32 bytes");
constexpr int kMqPadding = 16;  // zeroed entries behind the last stream's lists

// Group descriptor of the batching simulator: one 32-bit word per (placement,
// group), kept per lane in LDS; replicas are listed as group indices.
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

// Replica descriptor of the plain simulator: one 32-bit word per (tile, model,
// replica, lane), made for the lane that reads it, so that the hot loop gets
// its LDS addresses with one AND:
//   bits  3..17  LDS byte address (relative to the workgroup's dynamic LDS,
//                8-byte aligned, so bits 0..2 are free) of the clock of the
//                group's LAST stage, for this lane
//   bits  0..2   stages - 1, low three bits
//   bits 28..29  stages - 1, high two bits
//   bits 18..27  index of the group's LAST-stage latency in the model's row of
//                the compact latency table
//   bit  31      "no such replica"; the address then names the lane's clock
//                that is +inf forever, so it never wins the choice (chunked
//                loop), or the entry repeats the lane's first one, which
//                wins every tie against its copies (loop over runs, which
//                keeps no +inf clock; a lane without any replica names its
//                first clock slot and is told by this bit)
constexpr uint32_t kRepAddrMask = 0x3FFF8u;
__host__ __device__ inline uint32_t pack_rep(uint32_t last_clock_addr, uint32_t stages, uint32_t lat_last) {
    const uint32_t sm1 = stages - 1u;
    return last_clock_addr | (sm1 & 7u) | ((sm1 >> 3) << 28) | (lat_last << 18);
}
__host__ __device__ inline uint32_t rep_addr(uint32_t d) { return d & kRepAddrMask; }
__host__ __device__ inline uint32_t rep_stages_m1(uint32_t d) { return (d & 7u) | ((d >> 25) & 0x18u); }
__host__ __device__ inline uint32_t rep_lat_last(uint32_t d) { return (d >> 18) & 0x3FFu; }
constexpr int kSlotBytes = 64 * 8;  // one clock slot: 64 lanes x f64

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
    const int32_t *tile_seed;    // paired batches: the one stream each tile is simulated on (see `paired`)
    int32_t paired;              // 1: every tile has its own stream and results are laid out as for one seed;
                                 // 0: every tile is simulated on every stream
    int32_t slot_rows;           // row pitch of slot_cnt (most slots of any tile)
    int32_t state_rows;          // row pitch of state
    double *state;               // [waves][state_rows][64] clocks parked between segments (scheduled launch)
    // Scheduled launch (loop over runs): workgroup w owns the items wg_off[w] .. wg_off[w+1]-1, an item being one
    // (tile, stream) pair cut into segments of seg_requests requests; its wavefronts take turns on them.
    const int32_t *wg_off;       // [workgroups + 1]
    const int32_t *item_tile;    // [items]
    const int32_t *item_seed;    // [items]
    const int32_t *item_nslots;  // [items] clock slots of the item's tile
    const int32_t *item_bytes;   // [items] LDS bytes a wavefront needs to simulate the item
    const int32_t *item_nseg;    // [items] segments of the item's stream (at least 1)
    const int32_t *part_off;     // [workgroups][kMaxWavesPerBlock] byte offset of each wavefront's LDS region behind the
                                 //   schedule state, -1: that wavefront has none and leaves at once
    const int32_t *part_bytes;   // [workgroups][kMaxWavesPerBlock] size of that region
    int32_t sched_groups;        // workgroups of the scheduled launch
    int32_t seg_requests;        // requests per segment, a multiple of 64
    int32_t sched_lds_bytes;     // LDS bytes of the schedule state (behind the latency table)
    int32_t sched_spin_limit;    // a wavefront leaves after waiting this many times in a row for an item to be handed back
    int32_t lat_in_lds;          // 1: the block keeps a copy of lat in LDS
    int32_t uniform_stages;      // 1: all stages of a (model, config) have the same latency; lat is [M][C]
    int32_t pow2_depths;         // 1: every group of the batch has 1, 2, 4, 8 or 16 stages
    int32_t lat_lds_bytes;       // LDS bytes of the shared latency table (0 if it stays in global memory)
    int32_t wave_lds_bytes;      // LDS bytes of one wavefront's private region
    int32_t rmax_lds_bytes;      // M rounded up to 16
    int64_t Rmax;                // longest stream (row pitch of per-request outputs)
    double fixed_overhead;
    uint32_t flags;
    // outputs
    int32_t *n_good;             // [n_seeds][tiles*64]
    double *lat_sum;             // [n_seeds][tiles*64]
    int32_t *model_good;         // [waves][M][64]
    double *finish;              // [waves][Rmax][64]
    uint8_t *good;               // [waves][Rmax][64]
    int64_t *fp_ops;             // [n_seeds][tiles*64]
    int32_t *error;              // set to 1 if the kernel finds its LDS layout assumption broken
    int32_t model_lds;           // 1: per-model counters [M][64] live in LDS behind the slot counters (small batches,
                                 // where LDS is not what limits the wavefronts per CU); 0: relaxed adds to model_good
    // Per-group counts are kept per clock slot: the row of a group's last stage holds, per lane, its requests (low half)
    // and accepted requests (high half); the host knows which slot is which group's last.
    int32_t group_lds;           // 1: a row of 64-bit counters per clock slot in LDS behind the clocks, one add per request,
                                 // added to slot_cnt when the turn ends (small batches); 0: counts per lane in registers,
                                 // added to slot_cnt when the lane's group changes
    unsigned long long *slot_cnt;  // [waves][slot_rows][64], zeroed by the host before the launch
    int32_t runs;                // 1: the request loop walks runs of equal models (streams whose requests mostly repeat the
                                 // model of the one before); 0: fixed chunks of four requests
    int32_t skip_ahead;          // 1: requests that every lane must reject are found a block at a time and not simulated (scores only)
    int32_t xcd_map;             // 1: all seeds of a tile group on one XCD (see sim_mixed.hip); 0: seeds innermost
};

// LDS layout of the plain simulator, shared by the kernel and by the host code
// that bakes LDS addresses into the replica descriptors:
//   [latency table][wavefront 0][wavefront 1]...
//   wavefront: [64 staged requests (chunked loop only)][replica bounds u8[M]]
//              [clocks: nslots+1 rows of 64 f64][slot counters: nslots rows of 64 u64][model counters]
// Row nslots of the clocks is the +inf row that empty descriptors point at.
// rmax_lds_bytes is M rounded up to 16.
__host__ __device__ inline uint32_t mixed_clock_offset(int32_t rmax_lds_bytes, bool runs) {
    return (uint32_t)((runs ? 0 : kStageBytes) + rmax_lds_bytes);  // the loop over runs keeps its requests in registers
}
constexpr int kMaxGroupItems = 256;   // items one workgroup of a scheduled launch can own
constexpr int kSchedLdsBytes = 1024;  // LDS reserved for its schedule state

// Arguments of the batching simulation kernel.  Replica lists and group
// descriptors are shared with the plain kernel; on top come, per seed, the
// arrivals regrouped by model (a model's FIFO is always a window of that list)
// and, per lane, the models of each group.
struct BatchingArgs {
    const Req *streams;          // all seeds' requests, back to back
    const int64_t *stream_off;   // [n_seeds+1]
    const int64_t *mq_off;       // [n_seeds][M+1] offsets into mq of the arrivals of each model
    const MqEntry *mq;           // model-ordered arrivals of all seeds, plus kMqPadding zeroed entries at the end
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
    int32_t lat_lds_bytes;       // > 0: the workgroup keeps a copy of lat in LDS (that many bytes, 16-aligned)
    int32_t g2m_in_lds;          // 1: each wavefront keeps its g2m_off / g2m_idx rows in LDS
    int32_t lane_stride;         // 64, 32 or 16: lanes of a wavefront that simulate; pitch of the per-lane LDS arrays
    int32_t uniform_stages;      // 1: a configuration's stages all have the same latencies and lat holds them once ([M][lat_row][NB], one row per configuration)
    const int32_t *tile_seed;    // as in MixedArgs
    int32_t paired;
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
// Arguments of the scalar-clock request loop (one placement, device pointers).
struct ScalarArgs {
    const double *tstamps;            // [R]
    const int32_t *model_ids;         // [R]
    const float *slos;                // [R]
    const int32_t *m_id2g_id;         // [M][G], -1 terminated rows
    const float *group_max_latency;   // [M][G]
    const float *group_sum_latency;   // [M][G]
    int64_t R;
    int32_t M, G;
    double fixed_overhead;
    double *finish;                   // [R]
    uint8_t *good;                    // [R]
    int32_t *model_req, *model_good;  // [M], zeroed by the caller
    int32_t *group_req, *group_good;  // [G], zeroed by the caller
};
// Arguments of the statistics kernel: the per-request outputs of a batch and, per stream, its arrivals
// regrouped by model and the window of request indices that the warm-up trimming leaves.  One launch
// handles the simulations sim0 .. sim0 + n - 1, one scratch row each.
struct StatsArgs {
    const double *finish;           // [waves][Rmax][64]
    const uint8_t *good;            // [waves][Rmax][64]
    const MqEntry *const *mq;       // [n_streams] model-ordered arrivals of each stream
    const int64_t *mq_off;          // [n_streams][M+1]
    const int64_t *lo, *hi;         // [n_streams] window [lo, hi) of request indices
    const int32_t *sim_stream;      // [n_sims] stream of each simulation
    const int64_t *sim_base;        // [n_sims] wave * Rmax * 64 + lane: where its column of finish / good starts
    uint64_t *scratch;              // [rows][scratch_pitch] latencies of a stream's requests in model order (all ones: not accepted)
    int64_t scratch_pitch;
    int32_t M, sim0;
    // outputs, [n_sims][M]
    int32_t *model_req, *model_good;
    double *first_start, *last_start, *latency_sum, *latency_mean, *latency_std, *latency_p90, *latency_p99;
};
hipError_t launch_model_stats(const StatsArgs &args, int n, hipStream_t stream, std::string *err);
constexpr int64_t kStatsScratchBytes = (int64_t)1 << 30;  // scratch rows of one launch (more simulations take several launches)

hipError_t launch_sim_scalar(const ScalarArgs &args, hipStream_t stream, std::string *err);

hipError_t launch_sim_batching(const BatchingArgs &args, int waves_per_block, size_t lds_bytes, hipStream_t stream,
                               std::string *err);

// Launches the plain simulator with `waves_per_block` wavefronts per workgroup.
hipError_t launch_sim_mixed(const MixedArgs &args, int smax_bucket, int waves_per_block, size_t lds_bytes,
                            hipStream_t stream, std::string *err);
std::string sim_mixed_kernel_name(const MixedArgs &args, int smax_bucket);
std::string sim_batching_kernel_name(const BatchingArgs &args);
// Smallest compiled stage bucket >= value, or -1.
int smax_bucket_for(int smax);
constexpr int kMaxWavesPerBlock = 8;          // plain simulator
constexpr int kMaxWavesPerBlockBatching = 4;  // batching simulator
constexpr int kMaxLatencyColumns = MMSIM_MAX_BATCH_SIZES;  // batching simulator: batch sizes below 2^16

}  // namespace mmsim
