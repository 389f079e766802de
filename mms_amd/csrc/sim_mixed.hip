// Plain (non-batching) request-loop simulation for gfx950.
//
// Restates the reference's simulate_requests_mixed
// (alpa_serve/simulator/controller.py:561-628) for a whole batch of candidate
// placements at once.  One lane simulates one (placement, arrival seed) pair;
// the 64 lanes of a wavefront hold 64 placements that walk the SAME request
// stream in lockstep, so everything that depends only on the request
// (arrival time, model id, SLO) is wave-uniform, while everything that depends
// on the placement is per lane.  Nothing in a request's dependency chain
// touches global memory:
//
//   * requests are fetched 64 at a time with one coalesced 1 KiB load per
//     wavefront, one block ahead, into registers (lane j holds request j);
//   * the replicas of the request's model are 32-bit descriptors made for the
//     lane that reads them (LDS address of the group's last-stage clock,
//     stage count, index of its last-stage latency), eight per (tile, model,
//     lane) in two 16-byte words rep32[tile][model][2][lane] (two coalesced
//     1 KiB loads, listed in the order the reference scans them).
//     Missing replicas point at a clock that is +inf forever (chunked loop)
//     or repeat the lane's first replica, which wins every tie against its
//     copies (loop over runs), so the scan itself needs no validity test;
//   * per-lane stage clocks live in LDS as clk[slot][lane] (8 bytes each);
//     the slots of a lane are its groups' pipeline stages laid end to end.
//     The bank an access hits depends on the lane only, so any per-lane
//     group or slot choice is conflict free;
//   * stage latencies live in a compact table lat[model][config stage] that
//     the workgroup keeps in LDS (shared by its wavefronts).  When every
//     (model, config) has one latency for all its stages the table shrinks
//     to lat[model][config] and the per-stage latency reads disappear.
//
// A request therefore costs two dependent LDS round trips: (1) last-stage
// clock and last-stage latency of every listed replica, (2) the stage clocks
// of the chosen group; single-stage placements need only the first.
// Group choice (strictly smallest last-stage clock, first listed wins ties)
// is a tournament of selects; stage walk, SLO decision and commit are one
// hand-scheduled inline-asm block (walk_asm.inc), with a C++ version for the
// shapes the block is not generated for.
//
// Two request loops (template argument RUNS, chosen by the host from how often
// a stream's requests repeat the model of the one before):
//   * chunks: the block is parked in LDS; four requests at a time are read
//     back with broadcast reads and their descriptors fetched one chunk
//     ahead (always eight loads per chunk, so the wait counters let the
//     fetch overlap the current chunk);
//   * runs (bursty streams): the block is cut into runs of equal models with
//     one ballot; descriptors are fetched once per run, one run ahead, and
//     the request simulated is read out of the lanes' registers with
//     v_readlane.  Clocks change only when a request is accepted, so the
//     chosen group is kept from request to request while no lane of the
//     wavefront has accepted anything, and with scores as the only output the
//     requests that every lane must then reject are found for the whole block
//     at once and not simulated at all (see the loop).
// One wavefront per SIMD issues at most one instruction every four cycles,
// whatever its kind, so the loops are written for few instructions and few
// per-lane branches.
//
// A lane whose request cannot meet its SLO even if it only had to wait for
// the chosen group's last stage skips the walk: with t >= arrival at every
// stage and rounding monotone,
//   fl(fl(fl(max(arrival, clk_last) + lat_last) + overhead) - arrival)
// never exceeds the latency the full walk would produce, so "that bound > slo"
// implies the reference's reject.  It only shortens the walk of the
// wavefront; results are identical.
//
// Arithmetic is fp64 add / max / sub / compare in the reference's order;
// fp32 operands (latencies, SLOs) are widened first.  Arrival times and
// latencies are never NaN and latencies never negative (the host rejects
// them), so the hardware max is an exact select.  Compiled with
// -ffp-contract=off; there is no multiply anyway.
//
// Workgroup = up to 4 wavefronts that share only the read-only latency
// table; after the single barrier that publishes it, wavefronts run
// independently (lanes never exchange data).
// Workgroups go to the eight XCDs round-robin by blockIdx.x, and each XCD has
// its own L2.  A request costs a wavefront 16 bytes of its stream but 2 KiB of
// its tile's descriptor rows, so the mapping keeps the descriptors together:
// blockIdx.x = ((tile_group / 8) * n_seeds + seed) * 8 + tile_group % 8, i.e.
// all seeds of a tile group run on one XCD and an XCD sees one eighth of the
// descriptor tables (a.xcd_map; the grid is padded to whole rounds of eight
// tile groups, the padding workgroups leave at once).  With a.xcd_map == 0
// blockIdx.x = tile_group * n_seeds + seed.

#include "mmsim_internal.h"
#include "walk_asm.inc"

namespace mmsim {

namespace {

__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// max of two doubles that are never NaN: one v_max_f64 without the input
// quieting the generic fmax lowering adds.
__device__ __forceinline__ double vmax(double x, double y) {
    double r;
    asm("v_max_f64 %0, %1, %2" : "=v"(r) : "v"(x), "v"(y));
    return r;
}

__device__ __forceinline__ double vmin(double x, double y) {
    double r;
    asm("v_min_f64 %0, %1, %2" : "=v"(r) : "v"(x), "v"(y));
    return r;
}

// Smallest values of x and of y over the 64 lanes, as scalars: butterflies inside rows of 16 lanes, then the
// row results carried to the last lane (row_bcast15 into rows 1 and 3, row_bcast31 into rows 2 and 3).
// One DPP instruction per step and value: v_min_u32_dpp d, d, d = min(d of the lane the pattern names, d),
// lanes the row mask leaves out keep d.  A DPP operand needs two wait states after the write of its
// register; the two independent chains and one s_nop give them.  All lanes must be active.
__device__ __forceinline__ void wave_min2_u32(uint32_t &x, uint32_t &y) {
#define MMSIM_MIN_STEP(PATTERN)                         \
    "s_nop 1\n"                                         \
    "v_min_u32_dpp %0, %0, %0 " PATTERN " bank_mask:0xf\n" \
    "v_min_u32_dpp %1, %1, %1 " PATTERN " bank_mask:0xf\n"
    asm volatile(MMSIM_MIN_STEP("quad_perm:[1,0,3,2] row_mask:0xf")
                 MMSIM_MIN_STEP("quad_perm:[2,3,0,1] row_mask:0xf")
                 MMSIM_MIN_STEP("row_half_mirror row_mask:0xf")
                 MMSIM_MIN_STEP("row_mirror row_mask:0xf")
                 MMSIM_MIN_STEP("row_bcast:15 row_mask:0xa")
                 MMSIM_MIN_STEP("row_bcast:31 row_mask:0xc")
                 "s_nop 1\n"
                 : "+v"(x), "+v"(y));
#undef MMSIM_MIN_STEP
    x = (uint32_t)__builtin_amdgcn_readlane((int)x, 63);
    y = (uint32_t)__builtin_amdgcn_readlane((int)y, 63);
}

// LDS accesses by byte address (the replica descriptors carry addresses, not pointers).
__device__ __forceinline__ double lds_f64(uint32_t addr) {
    return *reinterpret_cast<const __attribute__((address_space(3))) double *>(addr);
}
__device__ __forceinline__ float lds_f32(uint32_t addr) {
    return *reinterpret_cast<const __attribute__((address_space(3))) float *>(addr);
}
__device__ __forceinline__ void lds_set_f64(uint32_t addr, double v) {
    *reinterpret_cast<__attribute__((address_space(3))) double *>(addr) = v;
}

// 64-bit LDS add that returns nothing (the wavefront does not wait for it; LDS operations of a wavefront stay in order)
__device__ __forceinline__ void lds_add_u64(uint32_t addr, unsigned long long v) {
    asm volatile("ds_add_u64 %0, %1" : : "v"(addr), "v"(v) : "memory");
}

// 32-bit LDS byte address of a pointer into shared memory (for ds_* in inline asm).
__device__ __forceinline__ uint32_t lds_addr(const void *p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void *)p;
}

template <int I>
struct Idx {
    static constexpr int value = I;
};

// f(Idx<0>), f(Idx<1>), ... while f returns true, at most N times.  Compile-time
// recursion: every array index inside f is a constant, arrays stay in registers.
template <int I, int N, typename F>
__device__ __forceinline__ void static_while(F &&f) {
    if constexpr (I < N) {
        if (f(Idx<I>{})) static_while<I + 1, N>(static_cast<F &&>(f));
    }
}

// if (c(0)) { b(0); if (c(1)) { b(1); ... } } with per-lane conditions.
template <int I, int N, typename C, typename B>
__device__ __forceinline__ void static_nest(C &&c, B &&b) {
    if constexpr (I < N) {
        if (c(Idx<I>{})) {
            b(Idx<I>{});
            static_nest<I + 1, N>(static_cast<C &&>(c), static_cast<B &&>(b));
        }
    }
}

// Stage walk in blocks [0,1) [1,2) [2,4) [4,8) ...: one wave-uniform test per
// block ("does any lane reach this depth?"), nested per-lane ifs inside.
template <int LO, int HI, int N, typename C, typename B>
__device__ __forceinline__ void walk_blocks(C &&c, B &&b) {
    if constexpr (LO < N) {
        if (__ballot(c(Idx<LO>{})) != 0ull) {
            static_nest<LO, (HI < N ? HI : N)>(static_cast<C &&>(c), static_cast<B &&>(b));
            walk_blocks<HI, 2 * HI, N>(static_cast<C &&>(c), static_cast<B &&>(b));
        }
    }
}

// Chunked request loop (streams whose requests rarely repeat the model of the one before): requests whose
// descriptors and fields are fetched ahead together.  The fetch of a chunk has the time the previous
// chunk takes to arrive; four requests cover the latency of the descriptor loads.
constexpr int kChunk = 4;
struct Chunk {
    int m[kChunk];        // wave-uniform model id (or -1)
    int nrep[kChunk];     // wave-uniform replica bound of the tile for that model
    double t[kChunk];     // arrival time (same in every lane)
    float slo[kChunk];    // SLO (same in every lane)
    uint4 da[kChunk];     // per-lane descriptors of replicas 0..3
    uint4 db[kChunk];     // per-lane descriptors of replicas 4..7
};

template <int J>
__device__ __forceinline__ uint32_t pick_desc(const uint4 &a, const uint4 &b) {
    if constexpr (J == 0) return a.x;
    if constexpr (J == 1) return a.y;
    if constexpr (J == 2) return a.z;
    if constexpr (J == 3) return a.w;
    if constexpr (J == 4) return b.x;
    if constexpr (J == 5) return b.y;
    if constexpr (J == 6) return b.z;
    return b.w;
}

// Schedule state of one workgroup (in LDS behind the latency table): one word per item, twice the segment
// the item is at, plus one while a wavefront is simulating that segment.  A wavefront takes an item by
// compare-and-swap on its word and hands it back with a plain atomic store, so there is no lock to hold.
struct SchedLds {
    uint32_t item[kMaxGroupItems];
};
static_assert(sizeof(SchedLds) <= kSchedLdsBytes, "schedule state outgrew its LDS reservation");

// SMAX: most stages of a group (bucket).  LATLDS: the latency table is kept in LDS.  UNIFORM: one
// latency per (model, configuration).  POW2: every group has 1, 2, 4, 8 or 16 stages.  OUT: what the
// request loop produces beyond goodput and latency sum (a.flags says which of it): 0 nothing, 1
// per-model / per-group counts kept in registers and global rows, 2 the same counts kept in LDS (small
// batches), 3 also per-request results and operation counts; a level's loop carries no trace of the
// higher levels' outputs.  RUNS: the loop walks runs of equal models (bursty
// streams) instead of fixed chunks of four requests.
template <int SMAX, bool LATLDS, bool UNIFORM, bool POW2, int OUT, bool RUNS>
__global__ __launch_bounds__(kMaxWavesPerBlock *kWave) void sim_mixed_kernel(const MixedArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    constexpr int RREG = kPackedReplicas;

    const int W = (int)(blockDim.x >> 6);
    const int wv = uniform((int)(threadIdx.x >> 6));
    const int lane = (int)(threadIdx.x & 63);
    constexpr bool STATS = OUT > 0;
    const bool want_model = STATS && (a.flags & MMSIM_WANT_MODEL_COUNTS) != 0;
    const bool want_group = STATS && (a.flags & MMSIM_WANT_GROUP_COUNTS) != 0;
    const bool want_req = OUT == 3 && (a.flags & MMSIM_WANT_PER_REQUEST) != 0;
    const bool want_ops = OUT == 3 && (a.flags & MMSIM_WANT_OP_COUNT) != 0;
    constexpr bool pow2 = POW2;
    // The loop over runs is launched as a schedule (see the top of the file): its descriptors hold clock
    // addresses relative to the wavefront's clock rows, wherever in LDS they are this time.
    constexpr bool SCHED = RUNS;

    // ---- LDS: [latency table][schedule state (SCHED)][per wavefront: request block (chunked loop) | replica
    //            bounds | clocks (chunked loop: +inf row last) | slot counters | model counters].
    if (lds_addr(lds_raw) != 0u) {  // the descriptors assume the dynamic LDS starts at address 0
        if (threadIdx.x == 0) *a.error = 1;
        return;
    }
    // Loop over runs with one latency per (model, configuration): a run's model row of the latency table (at most
    // 64 entries, the host sees to that) travels in a register, one entry per lane, and the latencies of the run's
    // listed replicas are gathered from it across the lanes once per run; the table is not needed in LDS then (LDS
    // decides how many wavefronts a CU gets), and a replica scan ends with the tournament instead of a dependent
    // read of the winner's latency.
    constexpr bool RUNLAT = RUNS && UNIFORM;
    constexpr bool TABLE_LDS = LATLDS && !RUNLAT;
    float *lat_lds = reinterpret_cast<float *>(lds_raw);
    const int lat_floats = TABLE_LDS ? a.M * a.lat_row : 0;
    for (int i = (int)threadIdx.x; i < lat_floats; i += (int)blockDim.x) lat_lds[i] = a.lat[i];

    // Which (tile, stream) pairs this wavefront simulates, and where its LDS region is.
    SchedLds *sched = reinterpret_cast<SchedLds *>(lds_raw + a.lat_lds_bytes);
    int item0 = 0, n_items = 0;      // SCHED: this workgroup's items are item0 .. item0 + n_items - 1
    int part_off = -1, part_bytes = 0;  // SCHED: this wavefront's LDS region (offset behind the schedule state), -1: none
    int tile = 0, seed = 0;
    bool live = true;
    if constexpr (SCHED) {
        item0 = a.wg_off[blockIdx.x];
        n_items = a.wg_off[blockIdx.x + 1] - item0;
        part_off = a.part_off[(size_t)blockIdx.x * kMaxWavesPerBlock + wv];
        part_bytes = a.part_bytes[(size_t)blockIdx.x * kMaxWavesPerBlock + wv];
        for (int k = (int)threadIdx.x; k < n_items; k += (int)blockDim.x) sched->item[k] = 0u;
        live = wv < kMaxWavesPerBlock && part_off >= 0;
    } else {
        const unsigned grid_seeds = a.paired ? 1u : (unsigned)a.n_seeds;
        const unsigned bq = a.xcd_map ? blockIdx.x >> 3 : blockIdx.x;
        seed = (int)(bq % grid_seeds);
        const int tgroup = a.xcd_map ? (int)(bq / grid_seeds) * 8 + (int)(blockIdx.x & 7u) : (int)(bq / grid_seeds);
        tile = tgroup * W + wv;
        live = tile < a.tiles;
        if (a.paired && live) seed = a.tile_seed[tile];
    }
    unsigned char *mine = lds_raw + a.lat_lds_bytes + (SCHED ? a.sched_lds_bytes + part_off : wv * a.wave_lds_bytes);
    uint8_t *rmax_lds = mine + (RUNS ? 0 : kStageBytes);
    const uint32_t clk_off = (uint32_t)(mine - lds_raw) + mixed_clock_offset(a.rmax_lds_bytes, RUNS);
    double *clk = reinterpret_cast<double *>(lds_raw + clk_off) + lane;
    const uint32_t rel_base = SCHED ? clk_off : 0u;  // what turns a descriptor's clock address into an LDS address
    // Counter homes: output level 1 keeps no counters in LDS (its request loop carries no code for them)
    // Level 2 is compiled for counters in LDS and keeps both kinds, wanted or not (the host provides the room), so
    // that its request loop tests no flag; level 3 looks at the arguments.
    const bool group_lds = OUT == 2 || (OUT == 3 && want_group && a.group_lds != 0);  // a 64-bit counter per (clock slot, lane) in LDS
    const bool group_regs = want_group && !group_lds;  // counts per lane in registers, added to global rows when the group changes
    const bool model_lds = OUT == 2 || (OUT == 3 && want_model && a.model_lds != 0);
    if constexpr (!SCHED) {
        if (live)
            for (int i = lane; i < a.M; i += kWave) rmax_lds[i] = a.rmax[(size_t)tile * a.M + i];
    }
    __syncthreads();
    if (!live) return;  // a wavefront without work: padding of the last workgroup, or no LDS region in this schedule

    const float *lat_base = TABLE_LDS ? lat_lds : a.lat;
    const double overhead = a.fixed_overhead;

  for (int spins = 0;;) {  // SCHED: one turn per (item, segment) this wavefront is given; otherwise a single turn
    int seg = 0, item_k = 0;
    if constexpr (SCHED) {
        // Take the item of this workgroup that is furthest behind among those that fit this wavefront's LDS
        // region and that nobody is simulating right now (ties: the largest, so that the large regions serve
        // the large items).  One lane looks and claims the item with a compare-and-swap; if another
        // wavefront was faster it looks again.
        int got = -1;  // -1: nothing left for this wavefront, -2: what is left is being simulated by others right now
        if (lane == 0) {
            for (int tries = 0; tries < 64; ++tries) {
                int best = -1, best_bytes = -1;
                uint32_t best_word = 0xFFFFFFFFu;
                bool pending = false;
                for (int k = 0; k < n_items; ++k) {
                    const uint32_t w = __hip_atomic_load(&sched->item[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    const int sg = (int)(w >> 1), nsg = a.item_nseg[item0 + k];
                    const int bytes = a.item_bytes[item0 + k];
                    if (sg >= nsg || bytes > part_bytes) continue;
                    if (w & 1u) {  // worth waiting for only if a segment follows the one being simulated
                        if (sg + 1 < nsg) pending = true;
                        continue;
                    }
                    if (w < best_word || (w == best_word && bytes > best_bytes)) {
                        best = k;
                        best_word = w;
                        best_bytes = bytes;
                    }
                }
                if (best < 0) {
                    got = pending ? -2 : -1;
                    break;
                }
                uint32_t expect = best_word;
                if (__hip_atomic_compare_exchange_strong(&sched->item[best], &expect, best_word | 1u, __ATOMIC_ACQUIRE,
                                                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)) {
                    got = best;
                    break;
                }
                got = -2;  // lost the race for that item: look again (or, after many losses, sleep first)
            }
        }
        got = uniform(got);
        if (got == -1) break;
        if (got == -2) {
            // Everything left for this wavefront is in another wavefront's hands.  Wait a little for a segment to
            // end; a wavefront that has waited long leaves: no item depends on it (an item is either being
            // simulated or was just handed back by a wavefront that is about to look for work itself).
            __builtin_amdgcn_s_sleep(127);
            if (++spins > a.sched_spin_limit) break;
            continue;
        }
        spins = 0;
        item_k = got;
        tile = a.item_tile[item0 + item_k];
        seed = a.item_seed[item0 + item_k];
        seg = uniform((int)(__hip_atomic_load(&sched->item[item_k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) >> 1));
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");  // the state another wavefront parked for this item
        for (int i = lane; i < a.M; i += kWave) rmax_lds[i] = a.rmax[(size_t)tile * a.M + i];
    }
    const int nslots = SCHED ? a.item_nslots[item0 + item_k] : a.nslots;
    // Slot counters (group_lds): one row per clock row, behind the clocks.  The counter of the group whose last-stage
    // clock is at LDS address x is at x + cnt_rel: requests in the low half, accepted requests in the high half.
    // (the loop over runs has no +inf row behind its clocks)
    const uint32_t cnt_rel = (uint32_t)(nslots + (RUNS ? 0 : 1)) * kSlotBytes;
    unsigned long long *scnt = reinterpret_cast<unsigned long long *>(lds_raw + clk_off + cnt_rel) + lane;  // [nslots][64]
    uint32_t *mcnt = reinterpret_cast<uint32_t *>(lds_raw + clk_off + cnt_rel + (group_lds ? nslots * kSlotBytes : 0)) + lane;  // [M][64] accepted requests per model

    const int wave = a.paired ? tile : seed * a.tiles + tile;  // where this (tile, stream) pair's results go
    const size_t out = (size_t)wave * kWave + lane;
    const int64_t off = a.stream_off[seed];
    const int64_t R = a.stream_off[seed + 1] - off;
    // This turn simulates requests [r0, r1) of the stream.  Segments other than the first pick up the lane's
    // state where the wavefront that simulated the segment before parked it.
    const int64_t r0 = SCHED ? (int64_t)seg * a.seg_requests : 0;
    const int64_t r1 = SCHED && r0 + a.seg_requests < R ? r0 + a.seg_requests : R;
    const bool resume = seg > 0;
    const bool last_seg = r1 >= R;
    double *saved = a.state + (size_t)wave * a.state_rows * kWave + lane;

    int32_t n_good = 0;
    double lat_sum = 0.0;
    int64_t fp_ops = 0;
    if (resume) {
        for (int s = 0; s < nslots; ++s) clk[s * kWave] = saved[(size_t)s * kWave];
        n_good = a.n_good[out];
        lat_sum = a.lat_sum[out];
        if (want_ops) fp_ops = a.fp_ops[out];
    } else {
        for (int s = 0; s < nslots; ++s) clk[s * kWave] = 0.0;
    }
    if constexpr (!RUNS) clk[nslots * kWave] = __builtin_inf();
    if (group_lds)
        for (int s = 0; s < nslots; ++s) scnt[s * kWave] = 0ull;  // of this turn; added to slot_cnt when it ends

    int32_t *model_good = a.model_good + (size_t)wave * a.M * kWave + lane;
    if (model_lds)
        for (int m = 0; m < a.M; ++m) mcnt[m * kWave] = resume && want_model ? (uint32_t)model_good[(size_t)m * kWave] : 0u;

    const int4 *__restrict__ reqs4 = reinterpret_cast<const int4 *>(a.streams + off);
    const uint4 *__restrict__ rep_tile = a.rep32 + (size_t)tile * a.M * 2 * kWave + lane;
    const uint32_t *__restrict__ repx_tile = a.repx32 + (size_t)tile * a.M * a.rep_extra * kWave + lane;
    double *fin_out = a.finish + (size_t)wave * a.Rmax * kWave + lane;
    uint8_t *good_out = a.good + (size_t)wave * a.Rmax * kWave + lane;

    // the group chosen for the last request, kept while it stays valid (see the request loop)
    int ch_model = -2;        // wave-uniform: model the choice was made for
    bool ch_stale = true;     // wave-uniform: some lane accepted a request since
    double ch_best = __builtin_inf(), ch_l_last = 0.0;  // its last-stage clock and the model's last-stage latency there
    int ch_sm1 = -1;          // its stages - 1, or -1: the lane has no replica to send the request to
    uint32_t ch_last = 0, ch_first = 0;  // LDS addresses of its last and first stage clocks
    int ch_lrow = 0;          // where its stage latencies start in the model's row of the latency table
    constexpr bool SKIP = RUNS && OUT <= 2;  // per-request outputs and operation counts need every request
    bool ch_looked = false;   // wave-uniform: the block has been searched for requests that the current choice rejects
    uint64_t skip = 0;        // wave-uniform: requests of the block that every lane rejects while nobody accepts

    // Per-group counts without LDS (group_regs).  A lane's group changes only when the choice is made anew, and
    // between two choices every request the wavefront handles (simulated or passed over) goes to that group, so a
    // lane keeps, for its current group, how many requests of this turn had been handled (the request's place in the
    // stream, wave-uniform) and where its own count of accepted requests stood when it chose the group, and adds
    // the differences to the global row of the group's last
    // clock slot when its group changes (one 64-bit relaxed add, requests in the low half, accepted requests in the
    // high half; nobody waits for it; every counter has one owner).
    uint32_t pg_addr = 0xFFFFFFFFu, pg_req0 = 0;  // LDS address of the group's last-stage clock (or none); requests handled then
    int32_t pg_good0 = 0;                         // n_good then
    unsigned long long *slot_cnt = a.slot_cnt + (size_t)wave * a.slot_rows * kWave;
    auto flush_group = [&](uint32_t handled) {  // handled: requests of this turn handled so far (wave-uniform)
        const uint32_t reqs = handled - pg_req0, goods = (uint32_t)(n_good - pg_good0);
        if (pg_addr != 0xFFFFFFFFu && reqs != 0)
            __hip_atomic_fetch_add(&slot_cnt[(pg_addr - clk_off) >> 3], ((unsigned long long)goods << 32) | reqs,
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };
    // Per-model counts in global rows (no LDS for them): in the loop over runs a lane's accepted requests of a run
    // are the growth of n_good over the run, added once at its end.
    const bool model_per_run = RUNS && want_model && !model_lds;

    // One request for the whole wavefront: `at` is its place in the stream, m / n the model and the tile's
    // replica bound for it (wave-uniform), da / db this lane's descriptors of the model's replicas.
    // Where the scan of a request's first four replicas reads: the last-stage clocks and the last-stage latencies.
    // Worked out ahead of the request (it depends on the descriptors only), while the request before waits for LDS.
    // (LDS byte addresses; used with the latency table in LDS only.)  The empty statement at the end keeps the
    // compiler from moving the arithmetic to where the addresses are used, which is after the wait.
    struct ScanAddr {
        uint32_t c[4];
        uint32_t l[4];
    };
    auto scan_addr = [&](ScanAddr &sa, const uint4 &da, int m) {
        const uint32_t lrow_m = lds_addr(lat_lds) + (uint32_t)(m < 0 ? 0 : m) * (uint32_t)a.lat_row * 4u;
        static_while<0, 4>([&](auto J) {
            constexpr int j = decltype(J)::value;
            const uint32_t d = pick_desc<j>(da, da);
            sa.c[j] = rep_addr(d) + rel_base;
            sa.l[j] = lrow_m + rep_lat_last(d) * 4u;
            return true;
        });
        asm volatile("" : "+v"(sa.c[0]), "+v"(sa.c[1]), "+v"(sa.c[2]), "+v"(sa.c[3]), "+v"(sa.l[0]), "+v"(sa.l[1]),
                          "+v"(sa.l[2]), "+v"(sa.l[3]));
    };
    const ScanAddr no_addr{};
    auto nothing = []() {};
    // Loop over runs: LDS addresses of the last-stage clocks of the run's listed replicas, worked out once per run
    // (they depend on the descriptors only) and pinned there.
    uint32_t run_ca[RREG] = {};
    float run_l[RREG] = {};  // RUNLAT: their last-stage latencies

    // (PLAIN: the caller has seen that the tile lists one to four replicas for the model: the scan has no case to
    // tell, reads where `sa` says, and calls `meanwhile` once its reads are under way)
    auto simulate = [&](int64_t at, int m, int n, const uint4 &da, const uint4 &db, double tstamp, double slo,
                        auto PLAIN, const ScanAddr &sa, auto &&meanwhile) -> uint64_t {
        constexpr bool plain_scan = decltype(PLAIN)::value != 0;
        const float *lrow_m = lat_base + (size_t)(m < 0 ? 0 : m) * a.lat_row;

        // ---- choose the replica group: strictly smallest last-stage clock (:590-598).
        //      One LDS round trip fetches, for every listed replica, the clock of its last
        //      stage and the latency of its last stage (needed by the early-reject bound).
        // Strictly smallest clock, first listed wins ties: a tournament whose left side wins ties
        // picks the same entry as the reference's left-to-right scan, in log2 dependent steps.
        // Entries past a lane's own replicas are empty descriptors, whose clock reads +inf (chunked loop) or what
        // the lane's first entry reads (loop over runs).
        struct Cand {
            double c;
            uint32_t d;
            float l;
        };
        auto first_min = [](const Cand &x, const Cand &y) {
            const bool right = y.c < x.c;
            return Cand{vmin(x.c, y.c), right ? y.d : x.d, right ? y.l : x.l};
        };
        auto scan = [&](Cand &win, auto J0) {  // entries J0 .. J0 + 3
            constexpr int j0 = decltype(J0)::value, nj = 4;
            Cand k[nj];
            static_while<0, nj>([&](auto J) {
                constexpr int j = decltype(J)::value;
                k[j].d = pick_desc<j0 + j>(da, db);
                if constexpr (plain_scan) {
                    k[j].c = lds_f64(sa.c[j]);
                    k[j].l = lds_f32(sa.l[j]);
                } else if constexpr (RUNS) {
                    k[j].c = lds_f64(run_ca[j0 + j]);
                    k[j].l = RUNLAT ? run_l[j0 + j] : 0.0f;  // (otherwise the winner's latency is read after the tournament, one read for eight)
                } else {
                    k[j].c = lds_f64(rep_addr(k[j].d) + rel_base);
                    k[j].l = lrow_m[rep_lat_last(k[j].d)];
                }
                return true;
            });
            if constexpr (plain_scan) meanwhile();
            const Cand a01 = first_min(k[0], k[1]), a23 = first_min(k[2], k[3]);
            win = first_min(a01, a23);
        };
        // Clocks change only when a request is accepted, so while no lane of the wavefront has
        // accepted anything since the last scan, a request for the same model finds the same group
        // in every lane: the choice is kept from request to request (bursts make most requests
        // repeat the model of the one before, and most of a burst is rejected).
        if (!RUNS || m != ch_model || ch_stale) {  // the chunked loop always scans
            Cand win{__builtin_inf(), kEmpty, 0.0f};
            // The loop over runs serves bursty streams of well-replicated models: it fetches eight entries at once
            // when the tile lists more than four.  The chunked loop serves streams of many models with few replicas
            // each: one to four listed replicas are its straight path, entries 4-7 a second step off that path.
            auto beyond_eight = [&]() {  // rare: more than 8 replicas, read the rest on demand
                const uint32_t *row = repx_tile + (size_t)m * a.rep_extra * kWave;
                for (int j = RREG; j < n; ++j) {
                    const uint32_t d = row[(size_t)(j - RREG) * kWave];
                    win = first_min(win, Cand{lds_f64(rep_addr(d) + rel_base), d, lrow_m[rep_lat_last(d)]});
                }
            };
            if constexpr (RUNS) {
                if (__builtin_expect(n > 4, 0)) {
                    Cand more;
                    scan(win, Idx<0>{});
                    scan(more, Idx<4>{});
                    win = first_min(win, more);  // the final of the tournament of eight: entries 0-3 against 4-7
                    if (n > RREG) beyond_eight();
                } else if (OUT != 3 || n > 0) {  // (runs without a listed replica are passed over as a whole, see the loop)
                    scan(win, Idx<0>{});
                }
            } else if constexpr (plain_scan) {
                scan(win, Idx<0>{});
            } else {
                if (__builtin_expect(n > 0, 1)) scan(win, Idx<0>{});
                if (__builtin_expect(n > 4, 0)) {
                    Cand more;
                    scan(more, Idx<4>{});
                    win = first_min(win, more);
                    if (n > RREG) beyond_eight();
                }
            }
            if constexpr (RUNS && !RUNLAT) win.l = lrow_m[rep_lat_last(win.d)];
            // a clock that is infinite (a group that served a request with infinite latency) is never
            // chosen (:590-598: "tmp < min_device_clock" with min_device_clock starting at inf)
            ch_model = m;
            ch_looked = false;
            ch_best = win.c;
            ch_l_last = (double)win.l;
            // what the walk needs of the chosen group, worked out once per choice
            // (chunked loop: an empty descriptor points at the +inf row, so the clock alone tells whether a group was
            // found; loop over runs: the empty entries of a lane repeat its first entry and lose every tie to it, so
            // an empty entry wins only where the lane lists no replica at all)
            const bool found = win.c < 1e100 && (!RUNS || (int32_t)win.d >= 0);
            const int stages_m1 = (int)rep_stages_m1(win.d);
            ch_sm1 = found ? stages_m1 : -1;
            ch_last = rep_addr(win.d) + rel_base;
            ch_first = ch_last - (uint32_t)stages_m1 * kSlotBytes;  // (read by walking lanes only)
            ch_lrow = found ? (int)rep_lat_last(win.d) - stages_m1 : 0;
            if (group_regs) {  // requests handled up to here went to the group chosen before (:611, :618)
                const uint32_t now = found ? ch_last : 0xFFFFFFFFu;
                if (now != pg_addr) {
                    flush_group((uint32_t)(at - r0));
                    pg_addr = now;
                    pg_req0 = (uint32_t)(at - r0);
                    pg_good0 = n_good;
                }
            }
        }
        const double best = ch_best;
        const bool has = ch_sm1 >= 0;
        const int sm1 = ch_sm1;
        const uint32_t last_addr = ch_last;    // only used when the lane has a replica
        const uint32_t first_addr = ch_first;
        const float *lrow = lrow_m + ch_lrow;
        const double l_last = ch_l_last;

        double finish_time;
        bool acc = false;
        uint64_t acc_mask = 0;  // wave-uniform: lanes that accepted the request
        // Nobody asks which lane accepted or when it finished: scores only, and the counts of the loop over runs
        // without counters in LDS (they come from the growth of n_good, per run and per choice of group).
        constexpr bool LEAN = OUT == 0 || (OUT == 1 && RUNS);
        bool asm_walk = false;
        if constexpr (SMAX == 1) {
            // ---- single-stage groups: the clock read for the choice is the whole pipeline (:605-619)
            const double t = vmax(tstamp, best) + l_last;
            finish_time = t + overhead;
            const double latency = finish_time - tstamp;
            acc = has && latency <= slo;
            if (acc) {
                lds_set_f64(last_addr, t);
                n_good += 1;
                lat_sum += latency;
            }
        } else {
            // ---- lanes that cannot make the SLO even with an otherwise idle pipeline skip the walk
            const double bound = ((vmax(tstamp, best) + l_last) + overhead) - tstamp;
            const int walk = !(bound > slo) ? sm1 : -1;  // stages - 1 of lanes that walk (no per-lane branch; -1 without a replica)
            if constexpr ((LATLDS || RUNLAT) && (SMAX == 4 || SMAX == 16)) {
                // ---- stage walk, SLO decision and commit (:605-619) as one hand-scheduled block
                uint64_t saved_exec, mask1, mask2, mask4, mask8;  // masks: scratch of the power-of-two walk
                int accepted;
                double latency;
                const uint32_t cb_addr = first_addr;
#define MMSIM_WALK(NAME, LATNAME, LATVAL, TSREG)                                                                    \
asm volatile(NAME##_TEXT                                                                                        \
     : [sv] "=&s"(saved_exec), [acc] "=&v"(accepted), [fin] "=&v"(finish_time), [lat] "=&v"(latency),   \
       [ng] "+v"(n_good), [ls] "+v"(lat_sum), [m1] "=&s"(mask1), [m2] "=&s"(mask2), [m4] "=&s"(mask4),  \
       [m8] "=&s"(mask8), [am] "=&s"(acc_mask)                                                          \
     : [walk] "v"(walk), [cb] "v"(cb_addr), [LATNAME] "v"(LATVAL), [ts] TSREG(tstamp), [slo] "v"(slo),  \
       [oh] "s"(overhead)                                                                               \
     : "vcc", "scc", "memory", NAME##_CLOBBERS)
// (the loop over runs has the arrival time in scalar registers, read out of the block with v_readlane)
#define MMSIM_WALK_TS(NAME, LATNAME, LATVAL)                   \
    do {                                                       \
        if constexpr (RUNS)                                    \
            MMSIM_WALK(NAME, LATNAME, LATVAL, "s");            \
        else                                                   \
            MMSIM_WALK(NAME, LATNAME, LATVAL, "v");            \
    } while (0)
#define MMSIM_WALK_PICK(NAME, LATNAME, LATVAL)                 \
    do {                                                       \
        if constexpr (LEAN)                                    \
            MMSIM_WALK_TS(NAME##_LEAN, LATNAME, LATVAL);       \
        else                                                   \
            MMSIM_WALK_TS(NAME, LATNAME, LATVAL);              \
    } while (0)
                if constexpr (UNIFORM) {
                    if (pow2) {
                        if constexpr (SMAX == 4)
                            MMSIM_WALK_PICK(MMSIM_WALK_PU4, lc, l_last);
                        else
                            MMSIM_WALK_PICK(MMSIM_WALK_PU16, lc, l_last);
                    } else {
                        if constexpr (SMAX == 4)
                            MMSIM_WALK_PICK(MMSIM_WALK_U4, lc, l_last);
                        else
                            MMSIM_WALK_PICK(MMSIM_WALK_U16, lc, l_last);
                    }
                } else {
                    const uint32_t lb = lds_addr(lrow);
                    if (pow2) {
                        if constexpr (SMAX == 4)
                            MMSIM_WALK_PICK(MMSIM_WALK_PN4, lb, lb);
                        else
                            MMSIM_WALK_PICK(MMSIM_WALK_PN16, lb, lb);
                    } else {
                        if constexpr (SMAX == 4)
                            MMSIM_WALK_PICK(MMSIM_WALK_N4, lb, lb);
                        else
                            MMSIM_WALK_PICK(MMSIM_WALK_N16, lb, lb);
                    }
                }
#undef MMSIM_WALK_PICK
#undef MMSIM_WALK_TS
#undef MMSIM_WALK
                if constexpr (!LEAN) acc = accepted != 0;
                asm_walk = true;
            } else {
                // ---- the same in plain C++ (other stage buckets, latency table in global memory):
                //      fetch, then the dependent chain (:605-608)
                double *gclk = reinterpret_cast<double *>(lds_raw + first_addr);
                double cv[SMAX];
                float lv[SMAX];
                walk_blocks<0, 1, SMAX>(
                    [&](auto K) { return decltype(K)::value <= walk; },
                    [&](auto K) {
                        constexpr int k = decltype(K)::value;
                        cv[k] = gclk[k * kWave];
                        if (!UNIFORM) lv[k] = lrow[k];
                    });
                double t = tstamp;
                walk_blocks<0, 1, SMAX>(
                    [&](auto K) { return decltype(K)::value <= walk; },
                    [&](auto K) {
                        constexpr int k = decltype(K)::value;
                        t = vmax(t, cv[k]) + (UNIFORM ? l_last : (double)lv[k]);
                        cv[k] = t;
                    });
                finish_time = t + overhead;  // :610
                const double latency = finish_time - tstamp;
                acc = walk >= 0 && latency <= slo;  // :613
                if (acc) {  // :614-619
                    n_good += 1;
                    lat_sum += latency;
                }
                const int commit = acc ? walk : -1;
                walk_blocks<0, 1, SMAX>(
                    [&](auto K) { return decltype(K)::value <= commit; },
                    [&](auto K) {
                        constexpr int k = decltype(K)::value;
                        gclk[k * kWave] = cv[k];
                    });
            }
        }
        if constexpr (RUNS) {
            if (!asm_walk) acc_mask = __ballot(acc);
            ch_stale = acc_mask != 0ull;
        }
        if (group_regs) {
            // counted when the lane's group changes (above)
        } else if (group_lds && has) {  // :611, :618
            lds_add_u64(last_addr + cnt_rel, acc ? 0x100000001ull : 1ull);
        }
        if (want_ops) {
            asm volatile("" ::: "memory");  // keep this a wave-uniform branch, off the common path
            int nvalid = 0;
            static_while<0, RREG>([&](auto J) {
                constexpr int j = decltype(J)::value;
                nvalid += (j < n && (int32_t)pick_desc<j>(da, db) >= 0) ? 1 : 0;
                return true;
            });
            if (n > RREG) {
                const uint32_t *row = repx_tile + (size_t)m * a.rep_extra * kWave;
                for (int j = RREG; j < n; ++j) nvalid += (int32_t)row[(size_t)(j - RREG) * kWave] >= 0 ? 1 : 0;
            }
            if (has) fp_ops += 2 * (sm1 + 1) + nvalid + 3;
        }
        if (model_lds) {  // an LDS add that returns nothing (a request of an unknown model is accepted by nobody: adds 0 to row 0)
            __hip_atomic_fetch_add(&mcnt[(m < 0 ? 0 : m) * kWave], acc ? 1u : 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
        } else if (want_model && !model_per_run && m >= 0 && acc) {  // one owner per counter: a relaxed add that nobody waits for
            __hip_atomic_fetch_add(&model_good[(size_t)m * kWave], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (want_req) {
            fin_out[at * kWave] = acc ? finish_time : tstamp;
            good_out[at * kWave] = acc ? 1 : 0;
        }
        return acc_mask;
    };

    int4 ahead = make_int4(0, 0, -1, 0);  // this lane's request of the next block
    if (R > 0) ahead = reqs4[r0 + lane < R ? r0 + lane : R - 1];

    if constexpr (RUNS) {
        // Descriptors of the run about to start (fetched while the run before it is simulated).
        uint4 nda = make_uint4(kEmpty, kEmpty, kEmpty, kEmpty), ndb = nda;
        float nlat = 0.0f;  // RUNLAT: entry `lane` of the model's row of the latency table
        const int lat_lane = lane < a.lat_row ? lane : 0;
        // (the second half of a row, replicas 4-7, is only read by runs whose tile lists more than four replicas
        // for the model; the other runs load the first half twice -- the second load hits the line the first one
        // just brought in -- which costs no branch and no memory traffic)
        auto fetch_run = [&](int model, bool more_than_four) {  // model < 0: any row will do, nothing is simulated
            const uint4 *row = rep_tile + (size_t)(model < 0 ? 0 : model) * (2 * kWave);
            nda = row[0];
            ndb = row[more_than_four ? kWave : 0];
            if constexpr (RUNLAT) nlat = a.lat[(size_t)(model < 0 ? 0 : model) * a.lat_row + lat_lane];
        };
        {
            const int z0 = __builtin_amdgcn_readlane(ahead.z, 0);
            fetch_run(r0 < r1 ? z0 : -1, true);
        }

        for (int64_t blk = r0; blk < r1; blk += kWave) {
            // Lane j holds request j of the block; the request being simulated is read out of these
            // registers with v_readlane.  The model word also carries the tile's replica bound.
            const int nblk = (int)(r1 - blk < kWave ? r1 - blk : kWave);  // requests in this block
            int4 r = ahead;
            {
                const bool ok = lane < nblk && r.z >= 0;
                const int bound = (int)rmax_lds[ok ? r.z : 0];
                r.z = ok ? (r.z | (bound << 24)) : -1;
            }
            {
                const int64_t nx = blk + kWave + lane;
                ahead = reqs4[nx < R ? nx : R - 1];
            }
            // Bursts make most requests repeat the model of the one before: the block is cut into runs of
            // equal model words, and descriptors are fetched once per run.
            const int before = __builtin_amdgcn_ds_bpermute(((lane - 1) & 63) << 2, r.z);
            const uint64_t starts = __ballot(lane < nblk && (lane == 0 || r.z != before)) | 1ull;
            const uint64_t valid = nblk == kWave ? ~0ull : ((1ull << nblk) - 1ull);
            if constexpr (SKIP) {
                skip = 0;
                ch_looked = false;
            }

            for (int s0 = 0; s0 < nblk;) {
                const uint64_t later = starts & (s0 >= 63 ? 0ull : (~0ull << (s0 + 1)));
                const int s1 = later ? (int)__builtin_ctzll(later) : nblk;  // the run is requests [s0, s1)
                const uint4 da = nda, db = ndb;
                const float lat_row_here = nlat;
                {   // the run after this one: of this block, or the first of the next block
                    int zn = -1;
                    if (s1 < nblk)
                        zn = __builtin_amdgcn_readlane(r.z, s1);
                    else if (blk + kWave < r1)
                        zn = __builtin_amdgcn_readlane(ahead.z, 0);
                    // (a word of this block carries the tile's replica bound; the first word of the next block does
                    // not yet, so its row is fetched whole)
                    fetch_run(zn < 0 ? -1 : (zn & 0xFFFFFF), s1 >= nblk || (zn >> 24) > 4);
                }
                const int w = __builtin_amdgcn_readlane(r.z, s0);
                const int m = w >= 0 ? (w & 0xFFFFFF) : -1;  // wave-uniform model id (or -1)
                const int n = w >= 0 ? (w >> 24) : 0;        // replica bound of the tile; 0: nothing to simulate
                if constexpr (OUT != 3) {
                    // no lane of the tile hosts the model (or the stream names a model that does not exist): nothing
                    // changes and nothing is counted, whatever the requests are
                    if (n == 0) {
                        if (group_regs) pg_req0 += (uint32_t)(s1 - s0);  // (not requests of the group the lane counts for)
                        s0 = s1;
                        continue;
                    }
                }
                const uint64_t run = (s1 >= 64 ? ~0ull : ((1ull << s1) - 1ull)) & (~0ull << s0) & valid;
                const int32_t good_before = n_good;  // model_per_run
                static_while<0, RREG>([&](auto J) {
                    constexpr int j = decltype(J)::value;
                    run_ca[j] = rep_addr(pick_desc<j>(da, db)) + rel_base;
                    return true;
                });
                asm volatile("" : "+v"(run_ca[0]), "+v"(run_ca[1]), "+v"(run_ca[2]), "+v"(run_ca[3]), "+v"(run_ca[4]),
                                  "+v"(run_ca[5]), "+v"(run_ca[6]), "+v"(run_ca[7]));
                if constexpr (RUNLAT) {
                    auto gather = [&](auto J) {
                        constexpr int j = decltype(J)::value;
                        run_l[j] = __int_as_float(__builtin_amdgcn_ds_bpermute(
                            (int)(rep_lat_last(pick_desc<j>(da, db)) << 2), __float_as_int(lat_row_here)));
                        return true;
                    };
                    static_while<0, 4>(gather);
                    if (n > 4) static_while<4, RREG>(gather);
                }

                auto request = [&](int i) {
                    return simulate(blk + i, m, n, da, db,
                                    __hiloint2double(__builtin_amdgcn_readlane(r.y, i), __builtin_amdgcn_readlane(r.x, i)),
                                    (double)__int_as_float(__builtin_amdgcn_readlane(r.w, i)), Idx<0>{}, no_addr, nothing);
                };

                if constexpr (SKIP) {
                    uint64_t later = run & (~1ull << s0);  // requests of the run that follow the one being simulated
                    for (int i = s0;;) {
                        const uint64_t accepted = request(i);
                        // Nobody accepted: until somebody does, a request of this model is rejected by every lane
                        // (before any walk) if  fl(fl(fl(max(t, best) + l_last) + overhead) - t) > slo  in every
                        // lane.  For t <= best in every lane the left side is fl(C - t) with
                        // C = fl(fl(best + l_last) + overhead), and rounding is monotone, so any lower bound of
                        // the smallest C of the wavefront decides for all lanes at once (and any lower bound of
                        // the smallest best guards t <= best): the bounds are the smallest high words over the
                        // lanes, low words zero (non-negative doubles order like their high words).  Lane j
                        // tests request j of the block, and the requests found are not simulated: a rejected
                        // request changes nothing and counts only as a request of the group its lane would
                        // have chosen (:611), which is the group kept from the request before.
                        if (accepted) {
                            skip = 0;
                        } else if (a.skip_ahead && !ch_looked && later) {
                            ch_looked = true;
                            const bool chosen = ch_sm1 >= 0;
                            const uint32_t none = 0x7FF00000u;  // high word of +inf
                            uint32_t chi = chosen ? (uint32_t)__double2hiint((ch_best + ch_l_last) + overhead) : none;
                            uint32_t bhi = chosen ? (uint32_t)__double2hiint(ch_best) : none;
                            wave_min2_u32(chi, bhi);
                            const double clow = __hiloint2double((int)chi, 0);
                            const double blow = __hiloint2double((int)bhi, 0);
                            const double tj = __hiloint2double(r.y, r.x);
                            const bool rejected = r.z == w && tj <= blow && (clow - tj) > (double)__int_as_float(r.w);
                            skip |= __ballot(rejected);
                        }
                        const uint64_t todo = later & ~skip;
                        const int next = todo ? (int)__builtin_ctzll(todo) : 64;
                        if constexpr (OUT == 2) {
                            // requests of the run that are passed over for good
                            const int passed = __builtin_popcountll(next < 64 ? later & ~(~0ull << next) : later);
                            if (group_lds && passed > 0 && ch_sm1 >= 0)
                                lds_add_u64(ch_last + cnt_rel, (unsigned long long)passed);
                        }
                        if (!todo) break;
                        later &= ~1ull << next;
                        i = next;
                    }
                } else {
                    for (int i = s0; i < s1; ++i) request(i);
                }
                if (model_per_run && m >= 0) {  // one owner per counter: a relaxed add that nobody waits for
                    const int32_t grown = n_good - good_before;
                    if (grown != 0)
                        __hip_atomic_fetch_add(&model_good[(size_t)m * kWave], grown, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                s0 = s1;
            }
        }
    } else {
        int4 *stage4 = reinterpret_cast<int4 *>(mine);
        for (int64_t blk = r0; blk < r1; blk += kWave) {
            {   // park this block's requests; the model word also carries the tile's replica bound
                int4 r = ahead;
                const bool ok = blk + lane < r1 && r.z >= 0;
                const int bound = (int)rmax_lds[ok ? r.z : 0];
                r.z = ok ? (r.z | (bound << 24)) : -1;
                stage4[lane] = r;
            }
            {
                const int64_t nx = blk + kWave + lane;
                ahead = reqs4[nx < R ? nx : R - 1];
            }
            const int nblk = (int)(r1 - blk < kWave ? r1 - blk : kWave);  // requests in this block

            // Always 2 * kChunk loads per chunk, whatever the requests are, so that the wait counters let
            // the fetch of the next chunk overlap the simulation of this one.
            auto load_chunk = [&](Chunk &c, int cb) {
                int4 r[kChunk];
                static_while<0, kChunk>([&](auto U) {
                    constexpr int u = decltype(U)::value;
                    r[u] = stage4[cb + u];  // broadcast read; cb + u < 64
                    return true;
                });
                static_while<0, kChunk>([&](auto U) {
                    constexpr int u = decltype(U)::value;
                    const int w = uniform(r[u].z);
                    const bool ok = w >= 0;
                    const int m = ok ? (w & 0xFFFFFF) : -1;
                    c.m[u] = m;
                    c.nrep[u] = ok ? (w >> 24) : 0;  // 0: nothing to simulate (unknown model or no replica in the tile)
                    c.t[u] = __hiloint2double(r[u].y, r[u].x);
                    c.slo[u] = __int_as_float(r[u].w);
                    const uint4 *row = rep_tile + (size_t)(ok ? m : 0) * (2 * kWave);
                    c.da[u] = row[0];
                    c.db[u] = row[kWave];
                    return true;
                });
            };

            Chunk cur, nxt;
            load_chunk(cur, 0);
            for (int cb = 0; cb < nblk; cb += kChunk) {
                const bool more = cb + kChunk < nblk;
                load_chunk(nxt, more ? cb + kChunk : cb);
                // Single-stage groups: the usual chunk -- four requests, each of a model with one to four listed
                // replicas -- is simulated as straight-line code (no test between its requests, so that the fetches
                // of the next chunk and the address arithmetic of the next request fill the waits of the dependent
                // chain); any other chunk goes the general way.  (With the walk blocks of the deeper buckets, which
                // branch inside, the second copy of the loop body costs more than it gains: measured.)
                bool usual = SMAX == 1 && LATLDS && cb + kChunk <= nblk;
                static_while<0, kChunk>([&](auto U) {
                    constexpr int u = decltype(U)::value;
                    usual = usual && (unsigned)(cur.nrep[u] - 1) < 4u;
                    return true;
                });
                if (__builtin_expect(usual, 1)) {
                    ScanAddr sa[2];
                    scan_addr(sa[0], cur.da[0], cur.m[0]);
                    static_while<0, kChunk>([&](auto U) {
                        constexpr int u = decltype(U)::value;
                        simulate(blk + cb + u, cur.m[u], cur.nrep[u], cur.da[u], cur.db[u], cur.t[u], (double)cur.slo[u], Idx<1>{},
                                 sa[u & 1], [&]() {
                                     if constexpr (u + 1 < kChunk) scan_addr(sa[(u + 1) & 1], cur.da[u + 1], cur.m[u + 1]);
                                 });
                        return true;
                    });
                } else {
                    static_while<0, kChunk>([&](auto U) {
                        constexpr int u = decltype(U)::value;
                        if (cb + u >= nblk) return false;
                        simulate(blk + cb + u, cur.m[u], cur.nrep[u], cur.da[u], cur.db[u], cur.t[u], (double)cur.slo[u], Idx<0>{},
                                 no_addr, nothing);
                        return true;
                    });
                }
                cur = nxt;
            }
        }
    }

    a.n_good[out] = n_good;
    a.lat_sum[out] = lat_sum;
    if (want_ops) a.fp_ops[out] = fp_ops;
    if (!last_seg)
        for (int s = 0; s < nslots; ++s) saved[(size_t)s * kWave] = clk[s * kWave];
    if (model_lds && want_model)
        for (int m = 0; m < a.M; ++m) model_good[(size_t)m * kWave] = (int32_t)mcnt[m * kWave];
    if (group_regs) flush_group((uint32_t)(r1 - r0));
    if (group_lds && want_group) {  // one owner per counter at a time (segments of an item follow one another)
        for (int s = 0; s < nslots; ++s) {
            const unsigned long long v = scnt[s * kWave];
            if (v != 0ull) __hip_atomic_fetch_add(&slot_cnt[s * kWave + lane], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if constexpr (SCHED) {
        // hand the item back: its parked state must be visible to whichever wavefront takes its next segment
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        if (lane == 0) {
            __hip_atomic_store(&sched->item[item_k], (uint32_t)(seg + 1) << 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
            if (last_seg) atomicAdd(a.error + 1, 1);  // items completed: the host checks that none is missing
        }
    } else {
        break;
    }
  }
}

template <int SMAX, bool LATLDS, bool UNIFORM, bool POW2, int OUT, bool RUNS>
hipError_t launch_kernel(const MixedArgs &args, int wpb, size_t lds_bytes, hipStream_t stream) {
    auto kern = sim_mixed_kernel<SMAX, LATLDS, UNIFORM, POW2, OUT, RUNS>;
    if (lds_bytes > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (e != hipSuccess) return e;
    }
    unsigned blocks;
    if (RUNS) {
        blocks = (unsigned)args.sched_groups;
    } else {
        const unsigned tile_groups = (unsigned)((args.tiles + wpb - 1) / wpb);
        blocks = (args.xcd_map ? ((tile_groups + 7u) & ~7u) : tile_groups) * (unsigned)(args.paired ? 1 : args.n_seeds);
    }
    const dim3 grid(blocks);
    hipLaunchKernelGGL(kern, grid, dim3(wpb * kWave), lds_bytes, stream, args);
    return hipGetLastError();
}

template <int SMAX, bool LATLDS, bool UNIFORM, bool POW2, int OUT>
hipError_t launch_one(const MixedArgs &args, int wpb, size_t lds_bytes, hipStream_t stream) {
    return args.runs ? launch_kernel<SMAX, LATLDS, UNIFORM, POW2, OUT, true>(args, wpb, lds_bytes, stream)
                     : launch_kernel<SMAX, LATLDS, UNIFORM, POW2, OUT, false>(args, wpb, lds_bytes, stream);
}

// The specialisations that pay are compiled for the usual case (latency table in LDS); with the
// table in global memory only the general kernels exist.
template <int SMAX, bool UNIFORM>
hipError_t launch_u(const MixedArgs &args, int wpb, size_t lds_bytes, hipStream_t stream) {
    // what the request loop has to produce: 0 scores only, 1 also per-model / per-group counts without counters in
    // LDS, 2 counts with counters in LDS (small batches), 3 anything
    const bool lds_counters = args.group_lds && args.model_lds;  // both or neither, unless per-request outputs are asked for
    const int out = (args.flags & (MMSIM_WANT_PER_REQUEST | MMSIM_WANT_OP_COUNT)) ? 3
                    : (args.flags & (MMSIM_WANT_MODEL_COUNTS | MMSIM_WANT_GROUP_COUNTS)) ? (lds_counters ? 2 : 1) : 0;
    if (!args.lat_in_lds) return launch_one<SMAX, false, UNIFORM, false, 3>(args, wpb, lds_bytes, stream);
    if constexpr (SMAX == 4 || SMAX == 16) {  // the stage buckets with a hand-scheduled walk
        if (args.pow2_depths)
            return out == 3   ? launch_one<SMAX, true, UNIFORM, true, 3>(args, wpb, lds_bytes, stream)
                   : out == 2 ? launch_one<SMAX, true, UNIFORM, true, 2>(args, wpb, lds_bytes, stream)
                   : out == 1 ? launch_one<SMAX, true, UNIFORM, true, 1>(args, wpb, lds_bytes, stream)
                              : launch_one<SMAX, true, UNIFORM, true, 0>(args, wpb, lds_bytes, stream);
    }
    return out == 3   ? launch_one<SMAX, true, UNIFORM, false, 3>(args, wpb, lds_bytes, stream)
           : out == 2 ? launch_one<SMAX, true, UNIFORM, false, 2>(args, wpb, lds_bytes, stream)
           : out == 1 ? launch_one<SMAX, true, UNIFORM, false, 1>(args, wpb, lds_bytes, stream)
                      : launch_one<SMAX, true, UNIFORM, false, 0>(args, wpb, lds_bytes, stream);
}

template <int SMAX>
hipError_t launch_s(const MixedArgs &args, int wpb, size_t lds_bytes, hipStream_t stream) {
    return args.uniform_stages ? launch_u<SMAX, true>(args, wpb, lds_bytes, stream)
                               : launch_u<SMAX, false>(args, wpb, lds_bytes, stream);
}

}  // namespace

int smax_bucket_for(int smax) {
    for (int b : {1, 4, 16, 32})
        if (smax <= b) return b;
    return -1;
}

// The template instance launch_sim_mixed picks for these arguments, as profilers print it (same choices as
// launch_u / launch_s above).
std::string sim_mixed_kernel_name(const MixedArgs &args, int sb) {
    const bool lds_counters = args.group_lds && args.model_lds;  // both or neither, unless per-request outputs are asked for
    int out = (args.flags & (MMSIM_WANT_PER_REQUEST | MMSIM_WANT_OP_COUNT)) ? 3
              : (args.flags & (MMSIM_WANT_MODEL_COUNTS | MMSIM_WANT_GROUP_COUNTS)) ? (lds_counters ? 2 : 1) : 0;
    bool latlds = args.lat_in_lds != 0, pow2 = latlds && (sb == 4 || sb == 16) && args.pow2_depths;
    if (!latlds) out = 3;
    auto tf = [](bool v) { return v ? "true" : "false"; };
    return "sim_mixed_kernel<" + std::to_string(sb) + ", " + tf(latlds) + ", " + tf(args.uniform_stages != 0) + ", " + tf(pow2) +
           ", " + std::to_string(out) + ", " + tf(args.runs != 0) + ">";
}

hipError_t launch_sim_mixed(const MixedArgs &args, int sb, int wpb, size_t lds_bytes, hipStream_t stream,
                            std::string *err) {
    hipError_t e;
    if (wpb < 1 || wpb > kMaxWavesPerBlock) {
        e = hipErrorInvalidValue;
    } else {
        switch (sb) {
            case 1: e = launch_s<1>(args, wpb, lds_bytes, stream); break;
            case 4: e = launch_s<4>(args, wpb, lds_bytes, stream); break;
            case 16: e = launch_s<16>(args, wpb, lds_bytes, stream); break;
            case 32: e = launch_s<32>(args, wpb, lds_bytes, stream); break;
            default: e = hipErrorInvalidValue; break;
        }
    }
    if (e != hipSuccess && err) *err = std::string("sim_mixed launch: ") + hipGetErrorString(e);
    return e;
}

}  // namespace mmsim
