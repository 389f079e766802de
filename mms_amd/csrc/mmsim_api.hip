// Host side of libmmsim: handles, validation, packing of placements into the
// device layout the kernels read, launches, result unpacking.
//
// The packing restates the table build of approximate_one_case_one_placement
// (alpa_serve/simulator/controller.py:412-476) in the factored form the
// kernels use: instead of stage_latency[M][G][Smax] per placement, one latency
// table per distinct parallel configuration plus, per (placement, model), the
// ordered list of replica groups (m_id2g_id, :418-422).

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <chrono>
#include <cstring>
#include <functional>
#include <limits>
#include <memory>
#include <mutex>
#include <atomic>
#include <new>
#include <thread>

#include "mmsim_internal.h"

using namespace mmsim;

namespace {

thread_local std::string g_last_error;

int fail(int code, const std::string &msg) {
    g_last_error = msg;
    return code;
}

int hip_fail(hipError_t e, const char *what) {
    return fail(e == hipErrorOutOfMemory ? MMSIM_E_NOMEM : MMSIM_E_HIP,
                std::string(what) + ": " + hipGetErrorString(e));
}

#define HIP_TRY(expr)                                      \
    do {                                                   \
        hipError_t e__ = (expr);                           \
        if (e__ != hipSuccess) return hip_fail(e__, #expr); \
    } while (0)

// Device memory for a batch comes either from hipMalloc or, while g_arena is set (mmsim_eval_batch_static), from
// a bump allocator over the library's static device scratch: such buffers are never freed one by one.
struct Arena {
    unsigned char *base = nullptr;
    size_t cap = 0, used = 0;
    bool overflow = false;
};
thread_local Arena *g_arena = nullptr;

template <typename T>
struct DevBuf {
    T *p = nullptr;
    size_t n = 0;
    bool owned = true;
    DevBuf() = default;
    DevBuf(const DevBuf &) = delete;
    DevBuf &operator=(const DevBuf &) = delete;
    ~DevBuf() { release(); }
    void release() {
        if (p && owned) (void)hipFree(p);
        p = nullptr;
        n = 0;
        owned = true;
    }
    hipError_t alloc(size_t count) {
        release();
        n = count;
        const size_t bytes = std::max<size_t>(count, 1) * sizeof(T);
        if (Arena *ar = g_arena) {
            const size_t rounded = (bytes + 255) & ~(size_t)255;
            if (rounded > ar->cap - ar->used) {
                ar->overflow = true;
                n = 0;
                return hipErrorOutOfMemory;
            }
            p = reinterpret_cast<T *>(ar->base + ar->used);
            ar->used += rounded;
            owned = false;
            return hipSuccess;
        }
        return hipMalloc(reinterpret_cast<void **>(&p), bytes);
    }
    size_t bytes() const { return n * sizeof(T); }
};

}  // namespace

// Device scratch of mmsim_eval_batch_static: every device table and result buffer of one batch is carved out
// of this array, so that entry point never allocates.  Each GPU the library runs on holds its own copy at its
// own address until the process ends; host code only ever uses the address hipGetSymbolAddress returned for
// the current device (kept in the context), never the array's name.
static __device__ __align__(256) unsigned char scratch[MMSIM_STATIC_SCRATCH_BYTES];
constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static unsigned char *g_scratch_ptr[kMaxDevices] = {};  // per device, filled by the first context made on it

struct mmsim_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    hipDeviceProp_t prop{};
    int max_lds = 0;
    unsigned char *scratch = nullptr;     // this device's copy of the static scratch (mmsim_eval_batch_static)
    hipEvent_t ev_static[2] = {};         // timing events of batches that live in the static scratch
    mmsim_options opt{};                  // what batches made without options of their own use (mmsim_ctx_set_options)
};

std::atomic<uint64_t> g_next_workload_id{1};

struct mmsim_workload {
    mmsim_ctx *ctx = nullptr;
    uint64_t id = 0;  // unique per mmsim_workload_create: a batch remembers which streams it was made from
    int64_t R = 0;
    int32_t M = 0;
    DevBuf<Req> reqs;
    std::vector<int32_t> model_num_requests;  // requests per model id (placement independent)
    int64_t repeats = 0;                      // requests with the model of the request before
    // arrivals regrouped by model (batching simulator): offsets per model, then per arrival
    // its time, its deadline time + (double)slo and its index in the stream
    std::vector<int64_t> mq_off;
    DevBuf<MqEntry> mq;
};

// Ordered replica lists per (placement, model): the rows of m_id2g_id.
struct RepLists {
    int32_t B = 0, M = 0, Gmax = 0;
    std::vector<int32_t> num_groups;  // [B]
    std::vector<int32_t> group_cfg;   // [B][Gmax]
    std::vector<int64_t> off;         // [B*M+1]
    std::vector<int32_t> grp;         // group index per replica
    // models of each group in the order the batching simulator scans them (g_id2m_id);
    // left empty, they are derived from the replica lists as the reference does (:424-430)
    std::vector<int64_t> g2m_off;     // [B*Gmax+1]
    std::vector<int32_t> g2m_m;
};

struct mmsim_batch {
    mmsim_ctx *ctx = nullptr;
    uint32_t flags = 0;
    int32_t n_seeds = 0, B = 0, M = 0, Gmax = 0, tiles = 0, waves = 0;
    int32_t smax_bucket = 0, rmax_all = 0, nslots = 0, waves_per_block = 1;
    size_t lds_bytes = 0;
    int64_t Rmax = 0, Rtotal = 0;
    std::vector<int64_t> wl_R;                           // [n_seeds] stream lengths
    std::vector<uint64_t> wl_id;                         // [n_seeds] ids of the workloads the batch was made from
    std::vector<std::vector<int32_t>> wl_model_requests;  // [n_seeds][M] requests per model of each stream
    std::vector<int32_t> pos;  // pos[placement] = tile * 64 + lane it is simulated on
    // Paired batch (mmsim_eval_pairs): placement p is simulated on stream stream_of[p] only; a tile holds
    // placements of one stream, and results are laid out as for a single seed.
    bool paired = false;
    std::vector<int32_t> stream_of;   // [B]
    DevBuf<int32_t> tile_seed;        // [tiles]
    int32_t out_seeds = 1;            // seeds of the result layout: n_seeds, or 1 for a paired batch
    size_t wave_bytes = 0;     // LDS bytes of one wavefront's region (chunked loop, batching simulator)
    // Plain simulator, loop over runs: one launch of `sched_groups` workgroups, each owning a set of (tile, stream)
    // items that its wavefronts simulate segment by segment (clocks parked in `state` between segments).
    int32_t sched_groups = 0, sched_waves = 0, seg_requests = 0, max_nseg = 1;
    DevBuf<int32_t> plan;      // wg_off | item_tile | item_seed | item_nslots | item_bytes | item_nseg | part_off | part_bytes
    DevBuf<double> state;

    DevBuf<Req> streams;
    DevBuf<int64_t> stream_off;
    DevBuf<uint32_t> rep32, repx32;
    DevBuf<uint64_t> rep8;
    DevBuf<uint8_t> repx;
    DevBuf<uint8_t> rmax;
    DevBuf<int32_t> kerr;
    DevBuf<uint32_t> ginfo;
    DevBuf<float> lat;
    DevBuf<int32_t> n_good;
    DevBuf<double> lat_sum;
    DevBuf<int32_t> model_good, group_req, group_good;
    DevBuf<unsigned long long> slot_cnt;      // plain simulator: per-group counts by last clock slot [waves][nslots][64]
    std::vector<int16_t> group_last_slot;     // [B][Gmax] last clock slot of each group, -1: no such group
    int32_t group_by_slot = 0, slot_rows = 0; // group_by_slot: the group counts are in slot_cnt (else in group_req / group_good)
    int32_t group_lds = 0;                    // the kernel keeps the slot counters in LDS while it runs
    DevBuf<double> finish;
    DevBuf<uint8_t> good;
    DevBuf<int64_t> fp_ops;
    // batching simulator
    DevBuf<int64_t> mq_off;
    DevBuf<MqEntry> mq;
    DevBuf<int32_t> status, batch_sizes;
    DevBuf<uint16_t> g2m_off, g2m_idx;
    DevBuf<float> lat_nb;
    std::vector<uint8_t> hosted;  // [B][M] model has a replica (batching: decides model_num_requests)
    BatchingArgs bargs{};
    // device buffers of mmsim_batch_model_stats, made by its first call and kept for the next ones
    DevBuf<const MqEntry *> st_mq;
    DevBuf<int64_t> st_i64;   // mq_off | lo | hi | sim_base
    DevBuf<int32_t> st_i32;   // sim_stream | model_req | model_good
    DevBuf<double> st_f64;    // the seven double results
    DevBuf<uint64_t> st_scratch;

    MixedArgs args{};
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    bool own_events = true;  // false: the context's events (batch in the static scratch)
    bool ran = false;
    mmsim_options opt{};     // the options the batch was built with

    ~mmsim_batch() {
        if (own_events && ev_start) (void)hipEventDestroy(ev_start);
        if (own_events && ev_stop) (void)hipEventDestroy(ev_stop);
    }
};

namespace {

int check_tables(const mmsim_tables *t) {
    if (!t || !t->cfg_lat || !t->cfg_pp) return fail(MMSIM_E_INVALID, "tables: null pointer");
    if (t->M < 1 || t->C < 1 || t->Smax < 1 || t->NB < 1) return fail(MMSIM_E_INVALID, "tables: M, C, Smax, NB must be >= 1");
    if (t->M > 0xFFFFFF) return fail(MMSIM_E_UNSUPPORTED, "more than 16777215 models");
    if (t->C > 255) return fail(MMSIM_E_UNSUPPORTED, "tables: more than 255 parallel configurations");
    if (t->Smax > MMSIM_MAX_STAGES) return fail(MMSIM_E_UNSUPPORTED, "tables: more than 32 pipeline stages");
    for (int c = 0; c < t->C; ++c)
        if (t->cfg_pp[c] < 1 || t->cfg_pp[c] > t->Smax)
            return fail(MMSIM_E_INVALID, "tables: cfg_pp[c] outside 1..Smax");
    if (t->NB > 1 && (!t->batch_sizes || t->batch_sizes[0] != 1))
        return fail(MMSIM_E_INVALID, "tables: batch_sizes[0] must be 1");
    if (!(t->fixed_overhead == t->fixed_overhead)) return fail(MMSIM_E_INVALID, "tables: fixed_overhead is NaN");
    return MMSIM_OK;
}

int check_options(const mmsim_options *o) {
    if (!o) return MMSIM_OK;
    if (o->struct_size != (int32_t)sizeof(mmsim_options))
        return fail(MMSIM_E_INVALID, "options: struct_size is not sizeof(mmsim_options); start from mmsim_options_default");
    auto tri = [](int32_t v) { return v >= -1 && v <= 1; };
    if (!tri(o->request_loop) || !tri(o->counts_in_lds) || !tri(o->tile_order_by_slots) || !tri(o->skip_ahead) || !tri(o->xcd_map))
        return fail(MMSIM_E_INVALID, "options: a -1 / 0 / 1 switch has another value");
    if (o->waves_per_cu < 0 || o->waves_per_cu > kMaxWavesPerBlock) return fail(MMSIM_E_INVALID, "options: waves_per_cu outside 0..8");
    if (o->sched_groups < 0 || o->segment_requests < 0 || o->sched_spin_limit < -1 || o->batching_event_slots < 0 ||
        o->stats_scratch_bytes < 0)
        return fail(MMSIM_E_INVALID, "options: negative value");
    if (o->batching_lanes != 0 && o->batching_lanes != 8 && o->batching_lanes != 16 && o->batching_lanes != 32 && o->batching_lanes != 64)
        return fail(MMSIM_E_INVALID, "options: batching_lanes must be 0, 8, 16, 32 or 64");
    if (o->batching_lds_tables < -1 || o->batching_lds_tables > 3) return fail(MMSIM_E_INVALID, "options: batching_lds_tables outside -1..3");
    return MMSIM_OK;
}

// Runs fn(lo, hi) on slices of [0, n) on up to 16 host threads (one slice per thread; the caller's
// slices write disjoint memory).  Small ranges run on the calling thread.
template <class F>
void parallel_slices(int64_t n, int64_t min_per_thread, F &&fn) {
    int64_t threads = std::min<int64_t>(16, std::max(1u, std::thread::hardware_concurrency()));
    threads = std::min<int64_t>(threads, n / std::max<int64_t>(1, min_per_thread));
    if (threads <= 1) {
        fn((int64_t)0, n);
        return;
    }
    const int64_t per = (n + threads - 1) / threads;
    std::vector<std::thread> pool;
    for (int64_t lo = per; lo < n; lo += per) pool.emplace_back([&fn, lo, per, n] { fn(lo, std::min(n, lo + per)); });
    fn((int64_t)0, std::min(n, per));
    for (std::thread &th : pool) th.join();
}

// group -> models CSR of the C ABI into ordered per-(placement, model) replica lists
int lists_from_placements(const mmsim_placements *p, int32_t M, int32_t C, RepLists *out) {
    if (!p || !p->num_groups || !p->group_cfg || !p->gm_off) return fail(MMSIM_E_INVALID, "placements: null pointer");
    if (p->B < 1 || p->Gmax < 1) return fail(MMSIM_E_INVALID, "placements: B and Gmax must be >= 1");
    if (p->Gmax > MMSIM_MAX_GROUPS) return fail(MMSIM_E_UNSUPPORTED, "placements: more than 254 groups");
    out->B = p->B;
    out->M = M;
    out->Gmax = p->Gmax;
    out->num_groups.assign(p->num_groups, p->num_groups + p->B);
    out->group_cfg.assign(p->group_cfg, p->group_cfg + (size_t)p->B * p->Gmax);
    out->off.assign((size_t)p->B * M + 1, 0);
    for (int32_t b = 0; b < p->B; ++b) {
        const int32_t G = p->num_groups[b];
        if (G < 0 || G > p->Gmax) return fail(MMSIM_E_INVALID, "placements: num_groups[b] outside 0..Gmax");
        const int64_t *off = p->gm_off + (size_t)b * (p->Gmax + 1);
        for (int32_t g = 0; g < G; ++g) {
            const int32_t c = p->group_cfg[(size_t)b * p->Gmax + g];
            if (c < 0 || c >= C) return fail(MMSIM_E_INVALID, "placements: group_cfg outside 0..C-1");
            if (off[g + 1] < off[g]) return fail(MMSIM_E_INVALID, "placements: gm_off not monotone");
            if (off[g + 1] > off[g] && !p->gm_idx) return fail(MMSIM_E_INVALID, "placements: gm_idx is null");
            for (int64_t x = off[g]; x < off[g + 1]; ++x) {
                const int32_t m = p->gm_idx[x];
                if (m < 0 || m >= M) return fail(MMSIM_E_INVALID, "placements: model index outside 0..M-1");
                out->off[(size_t)b * M + m + 1] += 1;
            }
        }
    }
    for (size_t i = 1; i < out->off.size(); ++i) out->off[i] += out->off[i - 1];
    out->grp.assign((size_t)out->off.back(), 0);
    std::vector<int64_t> fill(out->off.begin(), out->off.end() - 1);
    for (int32_t b = 0; b < p->B; ++b) {
        const int64_t *off = p->gm_off + (size_t)b * (p->Gmax + 1);
        for (int32_t g = 0; g < p->num_groups[b]; ++g)  // ascending group index = reference order (:419-422)
            for (int64_t x = off[g]; x < off[g + 1]; ++x) out->grp[(size_t)fill[(size_t)b * M + p->gm_idx[x]]++] = g;
    }
    return MMSIM_OK;
}

// Base placements followed by their successors ("parent + one more replica"), as one placement list.
// With normalize the successor is what ModelPlacement.add_model(group, model).normalize() gives
// (alpa_serve/placement_policy/base_policy.py:24-35): the models of every group ascending, the groups in
// the (stable) order of their model tuples, each group keeping its configuration.
struct ExpandedPlacements {
    std::vector<int32_t> num_groups, group_cfg, gm_idx;
    std::vector<int64_t> gm_off;
    mmsim_placements view{};
};

int expand_successors(const mmsim_placements *base, const mmsim_successors *sc, int32_t M, ExpandedPlacements *out) {
    if (!base || !base->num_groups || !base->group_cfg || !base->gm_off) return fail(MMSIM_E_INVALID, "placements: null pointer");
    if (base->B < 1 || base->Gmax < 1) return fail(MMSIM_E_INVALID, "placements: B and Gmax must be >= 1");
    if (!sc || sc->n < 0 || (sc->n > 0 && (!sc->parent || !sc->group || !sc->model)))
        return fail(MMSIM_E_INVALID, "successors: null pointer or negative count");
    const int32_t B0 = base->B, Gmax = base->Gmax;
    const int64_t total = (int64_t)B0 + sc->n;
    if (total > 0x7FFFFFFF) return fail(MMSIM_E_UNSUPPORTED, "successors: too many placements");
    int64_t members = 0;  // entries of gm_idx
    for (int32_t b = 0; b < B0; ++b) {
        const int32_t G = base->num_groups[b];
        if (G < 0 || G > Gmax) return fail(MMSIM_E_INVALID, "placements: num_groups[b] outside 0..Gmax");
        const int64_t *off = base->gm_off + (size_t)b * (Gmax + 1);
        for (int32_t g = 0; g < G; ++g)
            if (off[g + 1] < off[g]) return fail(MMSIM_E_INVALID, "placements: gm_off not monotone");
        if (G > 0 && off[G] > off[0] && !base->gm_idx) return fail(MMSIM_E_INVALID, "placements: gm_idx is null");
        members += G > 0 ? off[G] - off[0] : 0;
    }
    for (int32_t k = 0; k < sc->n; ++k) {
        const int32_t p = sc->parent[k];
        if (p < 0 || p >= B0) return fail(MMSIM_E_INVALID, "successors: parent outside 0..B-1");
        if (sc->group[k] < 0 || sc->group[k] >= base->num_groups[p]) return fail(MMSIM_E_INVALID, "successors: group outside the parent's groups");
        if (sc->model[k] < 0 || sc->model[k] >= M) return fail(MMSIM_E_INVALID, "successors: model index outside 0..M-1");
        const int64_t *off = base->gm_off + (size_t)p * (Gmax + 1);
        members += (base->num_groups[p] > 0 ? off[base->num_groups[p]] - off[0] : 0) + 1;
    }
    out->num_groups.resize((size_t)total);
    out->group_cfg.assign((size_t)total * Gmax, 0);
    out->gm_off.assign((size_t)total * (Gmax + 1), 0);
    out->gm_idx.resize((size_t)members);
    int64_t at = 0;
    for (int32_t b = 0; b < B0; ++b) {  // the base placements as they are
        const int32_t G = base->num_groups[b];
        const int64_t *off = base->gm_off + (size_t)b * (Gmax + 1);
        out->num_groups[(size_t)b] = G;
        int64_t *dst = out->gm_off.data() + (size_t)b * (Gmax + 1);
        for (int32_t g = 0; g < G; ++g) {
            out->group_cfg[(size_t)b * Gmax + g] = base->group_cfg[(size_t)b * Gmax + g];
            dst[g] = at;
            for (int64_t x = off[g]; x < off[g + 1]; ++x) out->gm_idx[(size_t)at++] = base->gm_idx[x];
        }
        for (int32_t g = G; g <= Gmax; ++g) dst[g] = at;
    }
    parallel_slices(sc->n, 256, [&](int64_t k0, int64_t k1) {
        // where each successor's members start: the parents' sizes are known, so slices write disjoint ranges
        int64_t pos = at;
        for (int64_t k = 0; k < k0; ++k) {
            const int32_t p = sc->parent[k];
            const int64_t *off = base->gm_off + (size_t)p * (Gmax + 1);
            pos += (base->num_groups[p] > 0 ? off[base->num_groups[p]] - off[0] : 0) + 1;
        }
        std::vector<std::vector<int32_t>> rows;
        std::vector<int32_t> order;
        for (int64_t k = k0; k < k1; ++k) {
            const int32_t p = sc->parent[k], G = base->num_groups[p];
            const int64_t *off = base->gm_off + (size_t)p * (Gmax + 1);
            rows.resize((size_t)G);
            order.resize((size_t)G);
            for (int32_t g = 0; g < G; ++g) {
                rows[(size_t)g].assign(base->gm_idx + off[g], base->gm_idx + off[g + 1]);
                if (g == sc->group[k]) rows[(size_t)g].push_back(sc->model[k]);
                if (sc->normalize) std::sort(rows[(size_t)g].begin(), rows[(size_t)g].end());
                order[(size_t)g] = g;
            }
            if (sc->normalize)
                std::stable_sort(order.begin(), order.end(), [&](int32_t x, int32_t y) { return rows[(size_t)x] < rows[(size_t)y]; });
            const size_t q = (size_t)B0 + (size_t)k;
            out->num_groups[q] = G;
            int64_t *dst = out->gm_off.data() + q * (Gmax + 1);
            for (int32_t g = 0; g < G; ++g) {
                const int32_t src = order[(size_t)g];
                out->group_cfg[q * Gmax + g] = base->group_cfg[(size_t)p * Gmax + src];
                dst[g] = pos;
                for (int32_t m : rows[(size_t)src]) out->gm_idx[(size_t)pos++] = m;
            }
            for (int32_t g = G; g <= Gmax; ++g) dst[g] = pos;
        }
    });
    out->view.B = (int32_t)total;
    out->view.Gmax = Gmax;
    out->view.num_groups = out->num_groups.data();
    out->view.group_cfg = out->group_cfg.data();
    out->view.gm_off = out->gm_off.data();
    out->view.gm_idx = out->gm_idx.data();
    return MMSIM_OK;
}

// Builds every device table of a batch from replica lists and launches nothing.
int build_batch(mmsim_ctx *ctx, const mmsim_workload *const *wls, int32_t n_seeds, const mmsim_tables *t,
                const RepLists &rl, uint32_t flags, mmsim_batch **out, const int32_t *stream_of = nullptr,
                const mmsim_options *options = nullptr) {
    const mmsim_options &o = options ? *options : ctx->opt;
    // MMSIM_TIMING=1 prints the host time of each phase of the packing (diagnostics)
    const bool timing = std::getenv("MMSIM_TIMING") != nullptr;
    auto t_last = std::chrono::steady_clock::now();
    auto phase = [&](const char *name) {
        if (!timing) return;
        const auto now = std::chrono::steady_clock::now();
        std::fprintf(stderr, "[mmsim] build_batch %-28s %8.3f ms\n", name, std::chrono::duration<double, std::milli>(now - t_last).count());
        t_last = now;
    };

    const bool batching = (flags & MMSIM_BATCHING) != 0;
    if (batching && (flags & MMSIM_WANT_OP_COUNT)) return fail(MMSIM_E_UNSUPPORTED, "operation counts are only available for the plain simulator");
    if (batching) {
        if (!t->batch_sizes || t->batch_sizes[0] != 1) return fail(MMSIM_E_INVALID, "tables: batch_sizes[0] must be 1");
        for (int b = 0; b < t->NB; ++b) {
            if (t->batch_sizes[b] < 1) return fail(MMSIM_E_INVALID, "tables: batch size < 1");
            int col = 0;
            for (int v = t->batch_sizes[b]; v > 1; v >>= 1) ++col;
            if (col >= t->NB) return fail(MMSIM_E_INVALID, "tables: floor(log2(batch size)) must index a latency column");
        }
        if (t->M > 65535) return fail(MMSIM_E_UNSUPPORTED, "batching simulator: more than 65535 models");
        if (t->NB > MMSIM_MAX_BATCH_SIZES) return fail(MMSIM_E_UNSUPPORTED, "batching simulator: more than 16 batch sizes");
    }
    const int32_t M = t->M, C = t->C, B = rl.B, Gmax = rl.Gmax;
    if (n_seeds < 1 || !wls) return fail(MMSIM_E_INVALID, "need at least one workload");
    for (int s = 0; s < n_seeds; ++s) {
        if (!wls[s]) return fail(MMSIM_E_INVALID, "null workload");
        if (wls[s]->ctx != ctx) return fail(MMSIM_E_INVALID, "workload belongs to another context");
        if (wls[s]->M != M) return fail(MMSIM_E_INVALID, "workload and tables disagree on the number of models");
    }
    std::unique_ptr<mmsim_batch> b(new (std::nothrow) mmsim_batch);
    if (!b) return fail(MMSIM_E_NOMEM, "host allocation failed");
    b->ctx = ctx;
    b->opt = o;
    b->flags = flags;
    b->n_seeds = n_seeds;
    b->B = B;
    b->M = M;
    b->Gmax = Gmax;
    for (int s = 0; s < n_seeds; ++s) {  // copied: the batch does not depend on the workloads outliving it
        b->wl_R.push_back(wls[s]->R);
        b->wl_id.push_back(wls[s]->id);
        b->wl_model_requests.push_back(wls[s]->model_num_requests);
    }
    b->paired = stream_of != nullptr;
    b->out_seeds = b->paired ? 1 : n_seeds;
    if (b->paired) {
        b->stream_of.assign(stream_of, stream_of + B);
        for (int32_t p = 0; p < B; ++p)
            if (stream_of[p] < 0 || stream_of[p] >= n_seeds) return fail(MMSIM_E_INVALID, "stream_of names a stream outside 0..n_streams-1");
    }

    // ---- per placement: slot layout; per (placement, model): replica count
    int smax = 1, rmax_all = 1, nslots = 1;
    bool pow2_depths = true;  // every group has 1, 2, 4, 8 or 16 stages
    std::vector<uint8_t> slot0((size_t)B * Gmax, 0);
    std::vector<int32_t> slots_of(B, 0);  // clock slots placement p needs
    // A placement's clock slots are laid out shallowest group first, groups that host no model before all others:
    // the walk for power-of-two depths lets every walking lane read as many clock rows as the deepest walking lane
    // of its wavefront, and a lane whose deepest group comes last then reads past its own slots only by what the
    // tile's deepest group has on its own deepest (nothing, where a tile's placements are equally deep).
    std::vector<uint8_t> group_hosts((size_t)B * Gmax, 0);
    for (int32_t p = 0; p < B; ++p)
        for (int64_t x = rl.off[(size_t)p * M]; x < rl.off[(size_t)(p + 1) * M]; ++x) {
            const int32_t g = rl.grp[(size_t)x];
            if (g >= 0 && g < rl.num_groups[p]) group_hosts[(size_t)p * Gmax + g] = 1;
        }
    for (int32_t p = 0; p < B; ++p) {
        int s = 0;
        int32_t by_depth[MMSIM_MAX_GROUPS];  // the groups by (hosts anything ? stages : 0), a counting sort
        const int32_t ng = rl.num_groups[p];
        {
            constexpr int kKeys = 34;  // 0, 1 .. 32 stages, more (refused below)
            uint8_t key[MMSIM_MAX_GROUPS];
            int32_t first[kKeys + 1] = {};
            for (int32_t g = 0; g < ng; ++g) {
                const int pp = t->cfg_pp[rl.group_cfg[(size_t)p * Gmax + g]];
                key[g] = (uint8_t)(group_hosts[(size_t)p * Gmax + g] ? std::min(pp, kKeys - 1) : 0);
                first[key[g] + 1] += 1;
            }
            for (int k = 0; k < kKeys; ++k) first[k + 1] += first[k];
            for (int32_t g = 0; g < ng; ++g) by_depth[first[key[g]]++] = g;
        }
        for (int32_t k = 0; k < ng; ++k) {
            const int32_t g = by_depth[k];
            const int pp = t->cfg_pp[rl.group_cfg[(size_t)p * Gmax + g]];
            if (s + pp > MMSIM_MAX_SLOTS)
                return fail(MMSIM_E_UNSUPPORTED, "placement has more than 255 pipeline stages in total");
            slot0[(size_t)p * Gmax + g] = (uint8_t)s;
            s += pp;
            smax = std::max(smax, pp);
            if ((pp & (pp - 1)) != 0 || pp > 16) pow2_depths = false;
        }
        nslots = std::max(nslots, s);
        slots_of[p] = std::max(s, 1);
        for (int32_t m = 0; m < M; ++m)
            rmax_all = std::max<int64_t>(rmax_all, rl.off[(size_t)p * M + m + 1] - rl.off[(size_t)p * M + m]);
    }
    if (rmax_all > MMSIM_MAX_REPLICAS) return fail(MMSIM_E_UNSUPPORTED, "a model has more than 64 replicas in one placement");
    b->smax_bucket = smax_bucket_for(smax);
    b->rmax_all = rmax_all;
    if (b->smax_bucket < 0) return fail(MMSIM_E_UNSUPPORTED, "no kernel bucket for this many pipeline stages");
    b->nslots = nslots;

    phase("slots and replica counts");
    // ---- compact batch-size-1 latency table.  General form: row of model m = its stage
    //      latencies for configuration 0, then configuration 1, ... (the cfg_pp[c] real
    //      stages only).  When every (model, config) has one latency for all its stages the
    //      row is just one value per configuration.
    bool uniform_stages = true;  // (the batching kernel reads every batch size's column: all of them must agree)
    for (int32_t m = 0; m < M && uniform_stages; ++m)
        for (int c = 0; c < C && uniform_stages; ++c) {
            const float *row = t->cfg_lat + ((size_t)m * C + c) * t->Smax * t->NB;
            for (int k = 1; k < t->cfg_pp[c]; ++k)
                if (std::memcmp(&row[(size_t)k * t->NB], &row[0], sizeof(float) * (batching ? (size_t)t->NB : 1)) != 0) uniform_stages = false;
        }
    std::vector<int32_t> lat_off(C + 1, 0);
    for (int c = 0; c < C; ++c) lat_off[c + 1] = lat_off[c] + (uniform_stages ? 1 : t->cfg_pp[c]);
    const int32_t lat_row = lat_off[C] + 1;  // one extra entry per model: +inf, the latency of "no such replica"
    if (lat_row > kMaxLatRow) return fail(MMSIM_E_UNSUPPORTED, "configurations have more than 1022 pipeline stages in total");
    std::vector<float> lat((size_t)M * lat_row, std::numeric_limits<float>::infinity());
    for (int32_t m = 0; m < M; ++m)
        for (int c = 0; c < C; ++c)
            for (int k = 0; k < (uniform_stages ? 1 : t->cfg_pp[c]); ++k) {
                const float v = t->cfg_lat[(((size_t)m * C + c) * t->Smax + k) * t->NB];
                if (v != v) return fail(MMSIM_E_INVALID, "tables: a stage latency is NaN");
                if (v < 0.0f) return fail(MMSIM_E_INVALID, "tables: a stage latency is negative");
                lat[(size_t)m * lat_row + lat_off[c] + k] = v;
            }

    // ---- which request loop: bursty streams (most requests repeat the model of the one before) get the loop over runs
    bool runs = false;
    if (!batching) {
        int64_t rep = 0, tot = 0;
        for (int s = 0; s < n_seeds; ++s) {
            rep += wls[s]->repeats;
            tot += wls[s]->R;
        }
        runs = 5 * rep > 4 * tot;  // four in five (measured: at three in four the chunked loop is still ahead)
        if (o.request_loop >= 0) runs = o.request_loop != 0;
        // (with one latency per (model, configuration) the loop over runs keeps a model's row of the table in a
        // register, one entry per lane, and no table in LDS)
        if (uniform_stages && lat_row > kWave) runs = false;
    }

    phase("latency table, loop choice");
    // ---- LDS budget
    const int32_t rmax_lds_bytes = (M + 15) & ~15;
    size_t wave_bytes = 0, lat_bytes = 0, lds_tail = 0, sched_bytes = 0;
    int lat_in_lds = 1;
    int wpb = 0;
    int heap_cap = 0, heap_min = 0, heap_pref = 0;  // batching simulator: event slots per lane (chosen, least, preferred)
    std::function<size_t(int, int)> batching_bytes_for;
    int blanes = kWave;  // batching simulator: lanes of a wavefront that simulate
    // Wavefronts per workgroup: no more than it takes to give every CU its share of the
    // batch (a small batch is spread over the CUs, one wavefront per workgroup), and
    // no more than fit in LDS.  Option waves_per_cu (1..8) sets the number instead.
    int wpb_cap = kMaxWavesPerBlock;
    {
        const int64_t waves_total = (int64_t)((B + kWave - 1) / kWave) * b->out_seeds;
        const int64_t cus = std::max(1, ctx->prop.multiProcessorCount);
        wpb_cap = (int)std::min<int64_t>(wpb_cap, std::max<int64_t>(1, (waves_total + cus - 1) / cus));
    }
    if (o.waves_per_cu > 0) wpb_cap = std::min(kMaxWavesPerBlock, o.waves_per_cu);
    // plain simulator, per wavefront: request block | replica bounds | clocks (chunked loop: one extra row that stays
    // +inf; loop over runs: as many rows more as the walk of the tile reads past its slots, see tile_tail)
    // | slot counters | model counters; the latency table is shared by the workgroup
    size_t model_lds_bytes = 0;  // per-model counters [M][64] in LDS (decided below)
    bool group_in_lds = false;   // a 64-bit counter per (clock slot, lane) in LDS (decided below)
    auto mixed_wave_bytes = [&](int ns, int tail_rows = 0) {
        const size_t behind = (group_in_lds ? (size_t)ns * kSlotBytes : 0) + model_lds_bytes;  // what follows the clocks
        const size_t slack = runs ? std::max((size_t)tail_rows * kSlotBytes, behind) : (size_t)kSlotBytes + behind;
        return ((size_t)mixed_clock_offset(rmax_lds_bytes, runs) + (size_t)ns * kSlotBytes + slack + 15) & ~(size_t)15;
    };
    if (!batching) {
        wave_bytes = mixed_wave_bytes(nslots);  // of the largest placement
        lat_bytes = runs && uniform_stages ? 0 : (lat.size() * sizeof(float) + 15) & ~(size_t)15;  // (see above)
        sched_bytes = runs ? (size_t)kSchedLdsBytes : 0;
        if (lat_bytes + sched_bytes + wave_bytes > (size_t)ctx->max_lds) {
            lat_in_lds = 0;
            lat_bytes = 0;
        }
        if (sched_bytes + wave_bytes > (size_t)ctx->max_lds) return fail(MMSIM_E_UNSUPPORTED, "per-wavefront state does not fit in LDS (too many stages/groups/models)");
        if ((size_t)ctx->max_lds > (size_t)kRepAddrMask) return fail(MMSIM_E_UNSUPPORTED, "LDS is larger than the descriptor's address field");
        // The walk for power-of-two depths lets every walking lane read as many clock rows as the deepest
        // one (up to 15 past its own group); the rows after the last wavefront's clocks must exist.  If that
        // tail does not fit beside even one wavefront, the general walk is used.
        lds_tail = pow2_depths ? (size_t)(b->smax_bucket - 1) * kSlotBytes : 0;
        if (lat_bytes + sched_bytes + wave_bytes + lds_tail > (size_t)ctx->max_lds) {
            lds_tail = 0;
            pow2_depths = false;
        }
        // Per-model and per-group counters.  In LDS (a row of 64-bit counters per clock slot, a row of 32-bit counters
        // per model) they cost one LDS add each per request, but the rows can cost a CU wavefronts (configuration 4:
        // 32 KB more per wavefront).  Without LDS the group counts are kept per lane in registers and added to global
        // rows when the lane's group changes, and accepted requests are added to global per-model rows, which a lone
        // wavefront has to wait behind (small batches: about 300 cycles per request).  So the counters go to LDS, both
        // kinds together, when that does not lower the wavefronts a CU gets.  Option counts_in_lds = 0 / 1 forces the
        // choice.  With per-request outputs or operation counts (the general kernel) each kind goes to LDS if
        // it fits at all.
        const size_t room = (size_t)ctx->max_lds - lat_bytes - sched_bytes - lds_tail;
        const size_t model_rows = (size_t)M * kWave * sizeof(uint32_t);
        if (flags & (MMSIM_WANT_PER_REQUEST | MMSIM_WANT_OP_COUNT)) {
            group_in_lds = (flags & MMSIM_WANT_GROUP_COUNTS) != 0;
            wave_bytes = mixed_wave_bytes(nslots);
            if (group_in_lds && wave_bytes > room) {
                group_in_lds = false;
                wave_bytes = mixed_wave_bytes(nslots);
            }
            if ((flags & MMSIM_WANT_MODEL_COUNTS) && wave_bytes + model_rows <= room) {
                model_lds_bytes = model_rows;
                wave_bytes = mixed_wave_bytes(nslots);
            }
        } else if (flags & (MMSIM_WANT_MODEL_COUNTS | MMSIM_WANT_GROUP_COUNTS)) {
            group_in_lds = false;
            const size_t without = std::min<size_t>(wpb_cap, room / mixed_wave_bytes(nslots));
            group_in_lds = true;
            model_lds_bytes = model_rows;
            const size_t with = std::min<size_t>(wpb_cap, room / mixed_wave_bytes(nslots));
            bool in_lds = with >= 1 && with >= without;
            if (o.counts_in_lds >= 0) in_lds = with >= 1 && o.counts_in_lds != 0;
            if (!in_lds) {
                group_in_lds = false;
                model_lds_bytes = 0;
            }
            wave_bytes = mixed_wave_bytes(nslots);
        } else {
            group_in_lds = false;
        }
    } else {
        // per wavefront: descriptors | clocks | event times | chunk minima | queue heads | head ranks | event
        // groups | free slots | arrivals per model | offsets of the models' arrival lists | batch sizes.
        // Event slots: the reference's heap holds about one entry per group plus a few stale ones (most
        // seen: G+3); min(2*G+8, G+16) are provisioned if that fits, never less than G+4, always a multiple
        // of eight (the kernel keeps them in chunks of eight).
        auto bytes_for = [&](int lanes, int slots) {
            const size_t nch8 = (size_t)((slots / 8 + 7) & ~7);
            // (octet tiles with at most 64 event slots keep the free slots and the chunk minima in registers)
            const bool in_regs = lanes == 8 && slots <= 64;
            return ((lanes == 8 ? 0 : (size_t)(Gmax + 1) * lanes * 4) + (size_t)nslots * lanes * 8 + (size_t)2 * M * lanes * 4 +
                    (size_t)slots * lanes * (8 + 4 + (in_regs ? 0 : 2)) + (in_regs ? 0 : nch8 * lanes * 8) +
                    (((size_t)M * 4 + 15) & ~(size_t)15) + (((size_t)(M + 1) * 8 + 15) & ~(size_t)15) +
                    (((size_t)t->NB * 4 + 15) & ~(size_t)15) + 15) & ~(size_t)15;
        };
        heap_min = (Gmax + 4 + 7) & ~7;
        heap_pref = std::max(heap_min, std::min(2 * Gmax + 8, Gmax + 16) & ~7);
        // Option batching_event_slots fixes the number of event slots per simulation (a multiple of eight; fewer than
        // the simulation needs makes it stop with MMSIM_E_OVERFLOW: used to test that path)
        if (o.batching_event_slots > 0) heap_pref = heap_min = std::max(8, o.batching_event_slots & ~7);
        auto size_for = [&](int lanes) {
            for (heap_cap = heap_pref; heap_cap >= heap_min; heap_cap -= 8) {
                wave_bytes = bytes_for(lanes, heap_cap);
                if (wave_bytes <= (size_t)ctx->max_lds) break;
            }
        };
        // Simulations per wavefront.  The loops between two arrivals run per lane and are bound by
        // latency (LDS and memory round trips), so a wavefront takes nearly as long with 8 simulations
        // as with 64 while its LDS footprint grows with their number: narrow tiles (32, 16 or 8 lanes
        // simulate, the others only help fetching requests) put more wavefronts on a CU, and that is
        // what hides the latency.  The widest tile that still gives every SIMD two wavefronts is used.
        blanes = kWave;
        if (o.batching_lanes > 0) {
            blanes = o.batching_lanes;
        } else {
            const int64_t cus = std::max(1, ctx->prop.multiProcessorCount);
            for (;;) {
                size_for(blanes);
                const int64_t per_cu = heap_cap >= heap_min ? (int64_t)ctx->max_lds / (int64_t)wave_bytes : 0;
                const int64_t waves = (int64_t)((B + blanes - 1) / blanes) * b->out_seeds;
                if (blanes == 8 || (per_cu >= 8 && waves >= 8 * cus)) break;
                blanes /= 2;
            }
        }
        size_for(blanes);
        if (heap_cap < heap_min) return fail(MMSIM_E_UNSUPPORTED, "batching simulator: per-wavefront state does not fit in LDS (too many models/stages/groups)");
        batching_bytes_for = bytes_for;
        wpb = (int)std::min<size_t>(kMaxWavesPerBlockBatching, (size_t)ctx->max_lds / wave_bytes);
    }

    std::vector<int32_t> tile_nslots;  // most clock slots of a placement of each tile
    std::vector<int32_t> tile_stream;  // paired batches: the stream of each tile
    phase("LDS budget");
    // ---- lane assignment.  A wavefront walks as many pipeline stages as its deepest
    //      lane needs, so placements are ordered by depth before they are cut into
    //      tiles of 64: first by their deepest group, then by the expected depth of a
    //      request (request-count weighted depth of the deepest group hosting each model).
    {
        std::vector<double> weight(M, 0.0);
        for (int s = 0; s < n_seeds; ++s)
            for (int32_t m = 0; m < M; ++m) weight[m] += (double)wls[s]->model_num_requests[m];
        std::vector<int32_t> deepest(B, 0);
        std::vector<double> expected(B, 0.0);
        std::atomic<bool> bad_group{false};
        parallel_slices(B, 512, [&](int64_t p0, int64_t p1) {
            std::vector<int32_t> depth_of(M);
            for (int64_t p = p0; p < p1; ++p) {
                std::fill(depth_of.begin(), depth_of.end(), 0);
                for (int32_t m = 0; m < M; ++m)
                    for (int64_t x = rl.off[(size_t)p * M + m]; x < rl.off[(size_t)p * M + m + 1]; ++x) {
                        const int32_t g = rl.grp[(size_t)x];
                        if (g < 0 || g >= rl.num_groups[p]) {
                            bad_group = true;
                            return;
                        }
                        depth_of[m] = std::max(depth_of[m], t->cfg_pp[rl.group_cfg[(size_t)p * Gmax + g]]);
                    }
                for (int32_t m = 0; m < M; ++m) {
                    deepest[p] = std::max(deepest[p], depth_of[m]);
                    expected[p] += weight[m] * depth_of[m];
                }
            }
        });
        if (bad_group) return fail(MMSIM_E_INVALID, "replica list names a group that does not exist");
        // Deepest first: their wavefronts take longest.  The loop over runs sizes a wavefront's LDS region by the
        // clock slots of its own tile, so there placements with similar slot counts share a tile
        // (option tile_order_by_slots = 0: by expected depth only).
        bool by_slots = runs;
        if (o.tile_order_by_slots >= 0) by_slots = runs && o.tile_order_by_slots != 0;
        std::vector<int32_t> order(B);
        for (int32_t p = 0; p < B; ++p) order[p] = p;
        std::stable_sort(order.begin(), order.end(), [&](int32_t x, int32_t y) {
            if (b->paired && stream_of[x] != stream_of[y]) return stream_of[x] < stream_of[y];
            if (deepest[x] != deepest[y]) return deepest[x] > deepest[y];
            if (by_slots && slots_of[x] != slots_of[y]) return slots_of[x] > slots_of[y];
            return expected[x] > expected[y];
        });
        const int32_t tl = batching ? blanes : kWave;  // placements per tile
        b->pos.assign(B, 0);
        int32_t tile = -1, in_tile = tl;
        for (int32_t k = 0; k < B; ++k) {
            const int32_t p = order[k];
            if (in_tile == tl || (b->paired && stream_of[p] != tile_stream.back())) {  // a tile holds one stream's placements
                ++tile;
                in_tile = 0;
                tile_nslots.push_back(1);
                tile_stream.push_back(b->paired ? stream_of[p] : 0);
            }
            b->pos[p] = tile * kWave + in_tile++;
            tile_nslots[tile] = std::max(tile_nslots[tile], slots_of[p]);
        }
        b->tiles = tile + 1;
        b->waves = b->paired ? b->tiles : b->tiles * n_seeds;
        if (batching) {
            b->waves_per_block = std::min(wpb, b->tiles);
            b->wave_bytes = wave_bytes;
            b->lds_bytes = (size_t)b->waves_per_block * wave_bytes;
        } else if (!runs) {
            // chunked loop: every wavefront gets the region of the largest placement; as many wavefronts per
            // workgroup as fit (beyond one per SIMD only the same number on every SIMD pays)
            int w = (int)std::min<size_t>(wpb_cap, ((size_t)ctx->max_lds - lat_bytes - lds_tail) / wave_bytes);
            if (w > 4) w = w == 8 ? 8 : 4;
            b->waves_per_block = std::max(1, std::min(w, b->tiles));
            b->wave_bytes = wave_bytes;
            b->lds_bytes = lat_bytes + (size_t)b->waves_per_block * wave_bytes + lds_tail;
        }
    }

    phase("lane assignment");
    // ---- loop over runs: the schedule.  An item is one (tile, stream) pair; it needs an LDS region as large as its
    //      tile's clock slots ask for.  Items are dealt to at most one workgroup per CU, tiles staying on one XCD (a
    //      workgroup goes to XCD blockIdx % 8; the tile's descriptor rows then live in one L2), largest first in
    //      snake order so that every workgroup gets a similar mix.  A workgroup's LDS is cut into regions sized for
    //      its largest items, one wavefront per region, as many as fit (up to 8: two per SIMD); its wavefronts then
    //      take the items in turns, a segment of the stream at a time, always the item that is furthest behind, so
    //      that all items of a workgroup finish together however many regions there are.
    std::vector<int32_t> plan;
    if (!batching && runs) {
        // Rows the walk of a tile can read past the tile's clock slots (power-of-two walk: every walking lane reads
        // as many rows as the deepest walking lane, from its own group's first slot on).  They are part of the
        // item's region, so that the reads stay inside the workgroup's LDS wherever the region lies; what is read
        // there is never used.
        std::vector<int32_t> tile_tail(b->tiles, 0);
        if (pow2_depths && lds_tail > 0) {
            std::vector<int32_t> deepest_of(b->tiles, 0), reach(b->tiles, 0);
            for (int pass = 0; pass < 2; ++pass)
                for (int32_t p = 0; p < B; ++p) {
                    const int tile = b->pos[p] / kWave;
                    for (int32_t g = 0; g < rl.num_groups[p]; ++g) {
                        if (!group_hosts[(size_t)p * Gmax + g]) continue;
                        if (pass == 0)
                            deepest_of[tile] = std::max(deepest_of[tile], (int32_t)t->cfg_pp[rl.group_cfg[(size_t)p * Gmax + g]]);
                        else
                            reach[tile] = std::max(reach[tile], (int32_t)slot0[(size_t)p * Gmax + g] + deepest_of[tile]);
                    }
                }
            for (int32_t t2 = 0; t2 < b->tiles; ++t2) tile_tail[t2] = std::max(0, reach[t2] - tile_nslots[t2]);
        }
        lds_tail = 0;  // (the chunked loop keeps one tail behind the last wavefront's region instead)
        struct Item { int32_t tile, seed, bytes; };
        const int64_t n_items = (int64_t)b->waves;
        const int64_t cus = std::max(1, ctx->prop.multiProcessorCount);
        int64_t groups = std::min<int64_t>(cus, n_items);
        if (o.sched_groups > 0) groups = std::min<int64_t>(n_items, o.sched_groups);
        if (n_items > groups * kMaxGroupItems) return fail(MMSIM_E_UNSUPPORTED, "too many (tile, stream) pairs for one launch; split the batch");
        std::vector<int32_t> tile_bytes(b->tiles);
        for (int32_t t2 = 0; t2 < b->tiles; ++t2) tile_bytes[t2] = (int32_t)mixed_wave_bytes(tile_nslots[t2], tile_tail[t2]);
        std::vector<int32_t> torder(b->tiles);
        for (int32_t t2 = 0; t2 < b->tiles; ++t2) torder[t2] = t2;
        std::stable_sort(torder.begin(), torder.end(), [&](int32_t x, int32_t y) { return tile_bytes[x] > tile_bytes[y]; });
        const int nx = groups >= 8 ? 8 : 1;  // XCDs that get workgroups of their own
        std::vector<std::vector<Item>> per_xcd(nx);
        for (int32_t i = 0; i < b->tiles; ++i) {
            const int r = i % (2 * nx), x = r < nx ? r : 2 * nx - 1 - r;
            if (b->paired)
                per_xcd[x].push_back(Item{torder[i], tile_stream[torder[i]], tile_bytes[torder[i]]});
            else
                for (int s2 = 0; s2 < n_seeds; ++s2) per_xcd[x].push_back(Item{torder[i], s2, tile_bytes[torder[i]]});
        }
        std::vector<std::vector<Item>> per_group((size_t)groups);
        for (int x = 0; x < nx; ++x) {
            std::vector<int64_t> mine;  // this XCD's workgroups
            for (int64_t w = x; w < groups; w += nx) mine.push_back(w);
            std::stable_sort(per_xcd[x].begin(), per_xcd[x].end(), [](const Item &u, const Item &v) { return u.bytes > v.bytes; });
            const int64_t gx = (int64_t)mine.size();
            for (size_t i = 0; i < per_xcd[x].size(); ++i) {
                const int64_t r = (int64_t)(i % (size_t)(2 * gx)), at = r < gx ? r : 2 * gx - 1 - r;
                per_group[(size_t)mine[(size_t)at]].push_back(per_xcd[x][i]);
            }
        }
        // The schedule state is one word per item of a workgroup (never more than the kSchedLdsBytes the budget above
        // set aside).
        {
            size_t most = 1;
            for (const auto &its : per_group) most = std::max(most, its.size());
            sched_bytes = std::min<size_t>(kSchedLdsBytes, (most * sizeof(uint32_t) + 15) & ~(size_t)15);
        }
        const size_t cap = (size_t)ctx->max_lds - lat_bytes - sched_bytes;
        int max_regions = kMaxWavesPerBlock;
        if (o.waves_per_cu > 0) max_regions = std::min(kMaxWavesPerBlock, o.waves_per_cu);
        int64_t seg_requests = 16384;
        if (o.segment_requests > 0) seg_requests = std::max<int64_t>(kWave, (int64_t)o.segment_requests & ~(int64_t)(kWave - 1));
        std::vector<int32_t> wg_off(groups + 1, 0), part_off((size_t)groups * kMaxWavesPerBlock, -1), part_bytes((size_t)groups * kMaxWavesPerBlock, 0);
        bool shared = false;  // some workgroup has more items than regions: streams are cut into segments
        size_t lds_used = 0;
        int waves_max = 1;
        for (int64_t w = 0; w < groups; ++w) {
            const auto &its = per_group[(size_t)w];  // largest first
            if ((int64_t)its.size() > kMaxGroupItems) return fail(MMSIM_E_UNSUPPORTED, "too many (tile, stream) pairs for one workgroup; split the batch");
            wg_off[w + 1] = wg_off[w] + (int32_t)its.size();
            size_t used = 0;
            int regions = 0;
            for (size_t i = 0; i < its.size() && regions < max_regions; ++i)
                if (used + (size_t)its[i].bytes <= cap) {  // an item too large for what is left: smaller ones may still fit
                    part_off[(size_t)w * kMaxWavesPerBlock + regions] = (int32_t)used;
                    part_bytes[(size_t)w * kMaxWavesPerBlock + regions] = its[i].bytes;
                    used += (size_t)its[i].bytes;
                    ++regions;
                }
            // Wavefronts k and k + 4 of a workgroup share a SIMD.  Regions come out largest first; with more than
            // four, the second wavefronts of the SIMDs get theirs smallest first, so that the largest items meet
            // the smallest ones: where every item has a wavefront of its own, the wavefront of a small item ends
            // early and leaves the SIMD to the large one, and the four SIMDs end at about the same time.
            for (int k = 4, l = regions - 1; k < l; ++k, --l) {
                std::swap(part_off[(size_t)w * kMaxWavesPerBlock + k], part_off[(size_t)w * kMaxWavesPerBlock + l]);
                std::swap(part_bytes[(size_t)w * kMaxWavesPerBlock + k], part_bytes[(size_t)w * kMaxWavesPerBlock + l]);
            }
            if ((int)its.size() > regions) shared = true;
            lds_used = std::max(lds_used, used);
            waves_max = std::max(waves_max, regions);
        }
        int64_t rmin = b->wl_R.empty() ? 0 : b->wl_R[0];
        for (int s2 = 0; s2 < n_seeds; ++s2) rmin = std::min(rmin, b->wl_R[(size_t)s2]);
        if (!shared) seg_requests = 0x7FFFFFC0;  // every item has a wavefront of its own: one segment
        int32_t max_nseg = 1;
        const size_t total = (size_t)wg_off[groups];
        plan.assign((size_t)(groups + 1) + 5 * total + 2 * (size_t)groups * kMaxWavesPerBlock, 0);
        int32_t *p_off = plan.data(), *p_tile = p_off + groups + 1, *p_seed = p_tile + total, *p_ns = p_seed + total,
                *p_bytes = p_ns + total, *p_nseg = p_bytes + total, *p_poff = p_nseg + total, *p_pbytes = p_poff + (size_t)groups * kMaxWavesPerBlock;
        std::copy(wg_off.begin(), wg_off.end(), p_off);
        for (int64_t w = 0; w < groups; ++w)
            for (size_t i = 0; i < per_group[(size_t)w].size(); ++i) {
                const Item &it = per_group[(size_t)w][i];
                const size_t at = (size_t)wg_off[w] + i;
                const int64_t Rs = b->wl_R[(size_t)it.seed];
                const int64_t ns = std::max<int64_t>(1, (Rs + seg_requests - 1) / seg_requests);
                if (ns > 60000) return fail(MMSIM_E_INVALID, "option segment_requests is too small for these streams");
                p_tile[at] = it.tile;
                p_seed[at] = it.seed;
                p_ns[at] = tile_nslots[it.tile];
                p_bytes[at] = it.bytes;
                p_nseg[at] = (int32_t)ns;
                max_nseg = std::max(max_nseg, (int32_t)ns);
            }
        std::copy(part_off.begin(), part_off.end(), p_poff);
        std::copy(part_bytes.begin(), part_bytes.end(), p_pbytes);
        b->sched_groups = (int32_t)groups;
        b->sched_waves = waves_max;
        b->seg_requests = (int32_t)seg_requests;
        b->max_nseg = max_nseg;
        b->waves_per_block = waves_max;
        b->wave_bytes = 0;
        b->lds_bytes = lat_bytes + sched_bytes + lds_used + lds_tail;
    }

    phase("schedule");
    // ---- per lane group descriptors [tiles][Gmax+1][64]; row Gmax stays empty
    std::vector<uint32_t> ginfo((size_t)b->tiles * (Gmax + 1) * kWave, kEmpty);
    for (int32_t p = 0; p < B; ++p) {
        const int tile = b->pos[p] / kWave, lane = b->pos[p] % kWave;
        for (int32_t g = 0; g < rl.num_groups[p]; ++g) {
            const int32_t c = rl.group_cfg[(size_t)p * Gmax + g];
            ginfo[((size_t)tile * (Gmax + 1) + g) * kWave + lane] =
                pack_desc(slot0[(size_t)p * Gmax + g], (uint32_t)t->cfg_pp[c], (uint32_t)lat_off[c], (uint32_t)g);
        }
    }
    // ---- replica lists.  Plain simulator: descriptors, the first 8 as [tiles][M][2][64] x (4 x u32),
    //      the rest [tiles][M][RX][64] x u32, missing entries empty.  Batching simulator: group
    //      indices, first 8 packed [tiles][M][64] x u64, the rest [tiles][M][RX][64] x u8, missing
    //      entries name the empty descriptor row Gmax.
    const int RX = std::max(rmax_all - kPackedReplicas, 0);
    const uint64_t none8 = 0x0101010101010101ull * (uint64_t)Gmax;
    std::vector<uint32_t> rep32, repx32;
    std::vector<uint64_t> rep8;
    std::vector<uint8_t> repx;
    // Tiles of eight simulations (octets): a row of rep8 is read as 64 descriptors instead, one per lane of the
    // wavefront -- lane 8 * simulation + j holds the descriptor of the j-th replica (kEmpty: none); the second half
    // of the row is not used.
    const bool octets = batching && blanes == 8;
    if (batching) {
        rep8.assign((size_t)b->tiles * M * kWave, octets ? ((uint64_t)kEmpty << 32 | kEmpty) : none8);
        repx.assign((size_t)b->tiles * M * RX * kWave, (uint8_t)Gmax);
    } else {
        rep32.resize((size_t)b->tiles * M * 2 * kWave * 4);
        repx32.resize((size_t)b->tiles * M * RX * kWave);
    }
    // LDS byte address of clock slot `slot` of the lane that simulates position `ps` (plain simulator);
    // slot < 0 names the lane's +inf clock.
    // The loop over runs takes addresses relative to the wavefront's clock rows (its LDS region moves from turn to
    // turn) and sizes the rows by the tile; the chunked loop takes LDS addresses, every region as large as the largest.
    // The loop over runs has no +inf row (LDS decides how many wavefronts a CU gets there): the missing entries of a
    // lane that lists replicas repeat its first entry, flagged empty -- a copy never beats the entry it copies, since
    // a tie goes to the entry listed first -- and those of a lane that lists none name its first clock slot; the
    // kernel tells by the flag that such a lane found nothing.
    auto clock_addr = [&](int ps, int slot) {
        const int tile = ps / kWave, lane = ps % kWave;
        const uint32_t base = runs ? 0u : (uint32_t)(lat_bytes + (size_t)(tile % b->waves_per_block) * b->wave_bytes + mixed_clock_offset(rmax_lds_bytes, false));
        const int inf_slot = runs ? 0 : nslots;
        return base + (uint32_t)(slot < 0 ? inf_slot : slot) * kSlotBytes + (uint32_t)lane * (uint32_t)sizeof(double);
    };
    if (!batching) {  // missing replicas: the +inf clock (see above) and the +inf latency, flagged empty
        const uint32_t inf_lat = (uint32_t)lat_off[C] << 18;
        parallel_slices(b->tiles, 8, [&](int64_t t0, int64_t t1) {
            for (int64_t tile = t0; tile < t1; ++tile) {
                uint32_t lane_word[kWave];
                for (int lane = 0; lane < kWave; ++lane) lane_word[lane] = kEmpty | clock_addr((int)tile * kWave + lane, -1) | inf_lat;
                uint32_t *dst = rep32.data() + (size_t)tile * M * 2 * kWave * 4;
                for (size_t i = 0; i < (size_t)M * 2 * kWave * 4; ++i) dst[i] = lane_word[(i / 4) % kWave];
                uint32_t *dx = repx32.data() + (size_t)tile * M * RX * kWave;
                for (size_t i = 0; i < (size_t)M * RX * kWave; ++i) dx[i] = lane_word[i % kWave];
            }
        });
    }
    std::vector<int32_t> tile_begin;
    std::vector<uint8_t> rmax((size_t)b->tiles * M, 0);
    // (by tile: the placements of a tile write that tile's rows only)
    std::vector<int32_t> by_tile(B);
    {
        std::vector<int32_t> at((size_t)b->tiles + 1, 0);
        for (int32_t p = 0; p < B; ++p) at[(size_t)(b->pos[p] / kWave) + 1] += 1;
        for (int32_t k = 0; k < b->tiles; ++k) at[(size_t)k + 1] += at[(size_t)k];
        std::vector<int32_t> fill(at.begin(), at.end() - 1);
        for (int32_t p = 0; p < B; ++p) by_tile[(size_t)fill[(size_t)(b->pos[p] / kWave)]++] = p;
        tile_begin = std::move(at);
    }
    parallel_slices(b->tiles, 8, [&](int64_t t0, int64_t t1) {
    for (int64_t k = tile_begin[(size_t)t0]; k < tile_begin[(size_t)t1]; ++k) {
        const int32_t p = by_tile[(size_t)k];
        const int tile = b->pos[p] / kWave, lane = b->pos[p] % kWave;
        for (int32_t m = 0; m < M; ++m) {
            const int64_t lo = rl.off[(size_t)p * M + m], hi = rl.off[(size_t)p * M + m + 1];
            uint8_t &rm = rmax[(size_t)tile * M + m];
            rm = std::max<uint8_t>(rm, (uint8_t)(hi - lo));
            uint64_t word = none8;
            uint32_t first_desc = 0;
            for (int64_t x = lo; x < hi; ++x) {
                const int32_t g = rl.grp[(size_t)x];
                const int j = (int)(x - lo);
                if (batching) {
                    if (j < kPackedReplicas && octets)
                        reinterpret_cast<uint32_t *>(rep8.data())[((size_t)tile * M + m) * 2 * kWave + (size_t)lane * 8 + (size_t)j] =
                            ginfo[((size_t)tile * (Gmax + 1) + g) * kWave + lane];
                    else if (j < kPackedReplicas)
                        word = (word & ~(0xFFull << (8 * j))) | ((uint64_t)g << (8 * j));
                    else
                        repx[(((size_t)tile * M + m) * RX + (size_t)(j - kPackedReplicas)) * kWave + lane] = (uint8_t)g;
                } else {
                    const int32_t c = rl.group_cfg[(size_t)p * Gmax + g];
                    const int pp = t->cfg_pp[c];
                    const uint32_t d = pack_rep(clock_addr(b->pos[p], slot0[(size_t)p * Gmax + g] + pp - 1), (uint32_t)pp,
                                                (uint32_t)(lat_off[c] + (uniform_stages ? 0 : pp - 1)));
                    if (j == 0) first_desc = d;
                    if (j < kPackedReplicas)  // word j/4 of the lane, component j%4
                        rep32[((((size_t)tile * M + m) * 2 + (size_t)(j / 4)) * kWave + lane) * 4 + (size_t)(j % 4)] = d;
                    else
                        repx32[(((size_t)tile * M + m) * RX + (size_t)(j - kPackedReplicas)) * kWave + lane] = d;
                }
            }
            if (!batching && runs && hi > lo)  // (see clock_addr)
                for (int j = (int)(hi - lo); j < kPackedReplicas + RX; ++j) {
                    if (j < kPackedReplicas)
                        rep32[((((size_t)tile * M + m) * 2 + (size_t)(j / 4)) * kWave + lane) * 4 + (size_t)(j % 4)] = first_desc | kEmpty;
                    else
                        repx32[(((size_t)tile * M + m) * RX + (size_t)(j - kPackedReplicas)) * kWave + lane] = first_desc | kEmpty;
                }
            if (batching && !octets) rep8[((size_t)tile * M + m) * kWave + lane] = word;
        }
    }
    });

    phase("descriptors");
    // ---- batching simulator: models of each group, full latency table, which models a lane hosts
    std::vector<uint16_t> g2m_off, g2m_idx;
    std::vector<float> lat_nb;
    int members_max = 1;
    if (batching) {
        b->hosted.assign((size_t)B * M, 0);
        std::vector<std::vector<int32_t>> lists(Gmax);
        std::vector<std::vector<int32_t>> all((size_t)B * Gmax);
        for (int32_t p = 0; p < B; ++p) {
            size_t total = 0;
            for (int32_t g = 0; g < rl.num_groups[p]; ++g) {
                std::vector<int32_t> &dst = all[(size_t)p * Gmax + g];
                if (!rl.g2m_off.empty())
                    dst.assign(rl.g2m_m.begin() + rl.g2m_off[(size_t)p * Gmax + g], rl.g2m_m.begin() + rl.g2m_off[(size_t)p * Gmax + g + 1]);
                total += dst.size();
            }
            for (int32_t m = 0; m < M; ++m) {
                const int64_t lo = rl.off[(size_t)p * M + m], hi = rl.off[(size_t)p * M + m + 1];
                b->hosted[(size_t)p * M + m] = hi > lo;
                if (rl.g2m_off.empty())  // ascending model id within a group, as :424-430 builds it
                    for (int64_t x = lo; x < hi; ++x) {
                        all[(size_t)p * Gmax + rl.grp[(size_t)x]].push_back(m);
                        ++total;
                    }
            }
            if (total > 65535) return fail(MMSIM_E_UNSUPPORTED, "batching simulator: more than 65535 (group, model) pairs in a placement");
            members_max = std::max<int>(members_max, (int)total);
        }
        g2m_off.assign((size_t)b->tiles * (Gmax + 1) * kWave, 0);
        g2m_idx.assign((size_t)b->tiles * members_max * kWave, 0);
        for (int32_t p = 0; p < B; ++p) {
            const int tile = b->pos[p] / kWave, lane = b->pos[p] % kWave;
            uint16_t at = 0;
            for (int32_t g = 0; g <= Gmax; ++g) {
                g2m_off[((size_t)tile * (Gmax + 1) + g) * kWave + lane] = at;
                if (g < rl.num_groups[p])
                    for (int32_t m : all[(size_t)p * Gmax + g]) {
                        if (m < 0 || m >= M) return fail(MMSIM_E_INVALID, "group model list names a model outside 0..M-1");
                        g2m_idx[((size_t)tile * members_max + at) * kWave + lane] = (uint16_t)m;
                        ++at;
                    }
            }
        }
        lat_nb.resize((size_t)M * lat_row * t->NB);
        for (int32_t m = 0; m < M; ++m)
            for (int c = 0; c < C; ++c)
                for (int k = 0; k < (uniform_stages ? 1 : t->cfg_pp[c]); ++k)
                    for (int q = 0; q < t->NB; ++q) {
                        const float v = t->cfg_lat[(((size_t)m * C + c) * t->Smax + k) * t->NB + q];
                        if (v != v || v < 0.0f) return fail(MMSIM_E_INVALID, "tables: a stage latency is NaN or negative");
                        lat_nb[((size_t)m * lat_row + lat_off[c] + k) * t->NB + q] = v;
                    }
    }

    // ---- batching simulator: keep the latency table (per workgroup) and the models of each group (per
    //      wavefront) in LDS when they fit; they are read in the innermost loops.  Wavefronts per
    //      workgroup (up to one per SIMD) come first: the loops are bound by latency, so a CU with an
    //      idle SIMD loses more than one that reads these tables through the caches.
    size_t batching_lat_lds = 0;
    int batching_g2m_lds = 0;
    if (batching) {
        const size_t lat_b = (lat_nb.size() * sizeof(float) + 15) & ~(size_t)15;
        const size_t g2m_b = ((size_t)(Gmax + 1) * blanes * 2 + (size_t)members_max * blanes * 2 + 15) & ~(size_t)15;
        const size_t cap = (size_t)ctx->max_lds;
        const int tiles_here = std::max(1, b->tiles);
        // Fewer event slots (down to G+8) are accepted when that puts more wavefronts on a CU.
        const int wpb_max = kMaxWavesPerBlockBatching;
        const int heap_try_min = std::min(heap_cap, std::max(heap_min, (Gmax + 8 + 7) & ~7));
        int best_w = 0, best_total = 0, best_heap = heap_cap;
        // option batching_lds_tables (bit 0: latency table, bit 1: group lists) fixes which tables may go to LDS
        const int allowed = o.batching_lds_tables >= 0 ? (o.batching_lds_tables & 3) : 3;
        for (int hc = heap_cap; hc >= heap_try_min; hc -= 8) {
            const size_t wb = batching_bytes_for(blanes, hc);
            for (int per_cu = 1; per_cu <= 2; ++per_cu)  // workgroups meant to share a CU (each gets that share of LDS)
                for (int opt = 0; opt < 4; ++opt) {      // both, lists only, table only, neither: the first that gives most wavefronts
                    // (the lists before the table: a selection reads them in two dependent steps, while the table is
                    // read beside the queue's entries, which come from memory anyway; measured 2.19 s against 2.42 s)
                    const bool want_lat = opt == 0 || opt == 2, want_g2m = opt < 2;
                    if ((want_lat && !(allowed & 1)) || (want_g2m && !(allowed & 2))) continue;
                    const size_t per = wb + (want_g2m ? g2m_b : 0), shared = want_lat ? lat_b : 0;
                    if (shared + per > cap / per_cu) continue;
                    const int w = (int)std::min<size_t>(std::min(wpb_max, tiles_here), (cap / per_cu - shared) / per);
                    if (per_cu * w > best_total) {
                        best_total = per_cu * w;
                        best_w = w;
                        best_heap = hc;
                        batching_lat_lds = shared;
                        batching_g2m_lds = want_g2m ? 1 : 0;
                    }
                }
        }
        heap_cap = best_heap;
        wave_bytes = batching_bytes_for(blanes, heap_cap);
        wpb = std::max(1, best_w);
        if (batching_g2m_lds) wave_bytes += g2m_b;
        b->waves_per_block = std::min(wpb, b->tiles);
        b->wave_bytes = wave_bytes;
        b->lds_bytes = batching_lat_lds + (size_t)b->waves_per_block * wave_bytes;
    }

    phase("batching tables");
    // ---- request streams back to back
    std::vector<int64_t> soff(n_seeds + 1, 0);
    for (int s = 0; s < n_seeds; ++s) {
        soff[s + 1] = soff[s] + wls[s]->R;
        b->Rmax = std::max(b->Rmax, wls[s]->R);
    }
    b->Rtotal = soff[n_seeds];

    hipStream_t st = ctx->stream;
    HIP_TRY(hipSetDevice(ctx->device));
    HIP_TRY(b->streams.alloc((size_t)b->Rtotal));
    for (int s = 0; s < n_seeds; ++s)
        if (wls[s]->R > 0)
            HIP_TRY(hipMemcpyAsync(b->streams.p + soff[s], wls[s]->reqs.p, sizeof(Req) * (size_t)wls[s]->R,
                                   hipMemcpyDeviceToDevice, st));
    HIP_TRY(b->stream_off.alloc(soff.size()));
    HIP_TRY(hipMemcpyAsync(b->stream_off.p, soff.data(), sizeof(int64_t) * soff.size(), hipMemcpyHostToDevice, st));
    if (batching) {
        HIP_TRY(b->rep8.alloc(rep8.size()));
        HIP_TRY(hipMemcpyAsync(b->rep8.p, rep8.data(), sizeof(uint64_t) * rep8.size(), hipMemcpyHostToDevice, st));
        HIP_TRY(b->repx.alloc(repx.size()));
        if (!repx.empty()) HIP_TRY(hipMemcpyAsync(b->repx.p, repx.data(), repx.size(), hipMemcpyHostToDevice, st));
        HIP_TRY(b->ginfo.alloc(ginfo.size()));
        HIP_TRY(hipMemcpyAsync(b->ginfo.p, ginfo.data(), sizeof(uint32_t) * ginfo.size(), hipMemcpyHostToDevice, st));
    } else {
        HIP_TRY(b->rep32.alloc(rep32.size()));
        HIP_TRY(hipMemcpyAsync(b->rep32.p, rep32.data(), sizeof(uint32_t) * rep32.size(), hipMemcpyHostToDevice, st));
        HIP_TRY(b->repx32.alloc(repx32.size()));
        if (!repx32.empty())
            HIP_TRY(hipMemcpyAsync(b->repx32.p, repx32.data(), sizeof(uint32_t) * repx32.size(), hipMemcpyHostToDevice, st));
    }
    if (b->paired) {
        HIP_TRY(b->tile_seed.alloc(tile_stream.size()));
        HIP_TRY(hipMemcpyAsync(b->tile_seed.p, tile_stream.data(), sizeof(int32_t) * tile_stream.size(), hipMemcpyHostToDevice, st));
    }
    HIP_TRY(b->kerr.alloc(32));
    HIP_TRY(hipMemsetAsync(b->kerr.p, 0, 32 * sizeof(int32_t), st));
    HIP_TRY(b->rmax.alloc(rmax.size()));
    HIP_TRY(hipMemcpyAsync(b->rmax.p, rmax.data(), rmax.size(), hipMemcpyHostToDevice, st));
    HIP_TRY(b->lat.alloc(lat.size()));
    HIP_TRY(hipMemcpyAsync(b->lat.p, lat.data(), sizeof(float) * lat.size(), hipMemcpyHostToDevice, st));

    if (batching) {
        std::vector<int64_t> mqo((size_t)n_seeds * (M + 1));
        int64_t total = 0;
        for (int s = 0; s < n_seeds; ++s) {
            for (int32_t m = 0; m <= M; ++m) mqo[(size_t)s * (M + 1) + m] = total + wls[s]->mq_off[m];
            total += wls[s]->mq_off[M];
        }
        // padding entries: the kernel looks one entry past a popped head, and fetches the sixteen entries from a
        // queue's head on at once, whether they have arrived or not
        HIP_TRY(b->mq.alloc((size_t)total + kMqPadding));
        HIP_TRY(hipMemsetAsync(b->mq.p + total, 0, sizeof(MqEntry) * kMqPadding, st));
        int64_t at = 0;
        for (int s = 0; s < n_seeds; ++s) {
            const size_t n = (size_t)wls[s]->mq_off[M];
            if (n > 0) {
                HIP_TRY(hipMemcpyAsync(b->mq.p + at, wls[s]->mq.p, sizeof(MqEntry) * n, hipMemcpyDeviceToDevice, st));
            }
            at += (int64_t)n;
        }
        HIP_TRY(b->mq_off.alloc(mqo.size()));
        HIP_TRY(hipMemcpyAsync(b->mq_off.p, mqo.data(), sizeof(int64_t) * mqo.size(), hipMemcpyHostToDevice, st));
        HIP_TRY(b->g2m_off.alloc(g2m_off.size()));
        HIP_TRY(hipMemcpyAsync(b->g2m_off.p, g2m_off.data(), sizeof(uint16_t) * g2m_off.size(), hipMemcpyHostToDevice, st));
        HIP_TRY(b->g2m_idx.alloc(g2m_idx.size()));
        HIP_TRY(hipMemcpyAsync(b->g2m_idx.p, g2m_idx.data(), sizeof(uint16_t) * g2m_idx.size(), hipMemcpyHostToDevice, st));
        HIP_TRY(b->lat_nb.alloc(lat_nb.size()));
        HIP_TRY(hipMemcpyAsync(b->lat_nb.p, lat_nb.data(), sizeof(float) * lat_nb.size(), hipMemcpyHostToDevice, st));
        HIP_TRY(b->batch_sizes.alloc((size_t)t->NB));
        HIP_TRY(hipMemcpyAsync(b->batch_sizes.p, t->batch_sizes, sizeof(int32_t) * (size_t)t->NB, hipMemcpyHostToDevice, st));
    }
    const size_t lanes_padded = (size_t)b->waves * kWave;
    HIP_TRY(b->status.alloc(lanes_padded));
    HIP_TRY(b->n_good.alloc(lanes_padded));
    HIP_TRY(b->lat_sum.alloc(lanes_padded));
    if (flags & MMSIM_WANT_MODEL_COUNTS) HIP_TRY(b->model_good.alloc(lanes_padded * M));
    if (batching && (flags & MMSIM_WANT_GROUP_COUNTS)) {
        HIP_TRY(b->group_req.alloc(lanes_padded * Gmax));
        HIP_TRY(b->group_good.alloc(lanes_padded * Gmax));
    }
    if (!batching && (flags & MMSIM_WANT_GROUP_COUNTS)) {
        b->group_by_slot = 1;
        b->group_lds = group_in_lds ? 1 : 0;
        b->slot_rows = nslots;
        HIP_TRY(b->slot_cnt.alloc(lanes_padded * (size_t)nslots));
        b->group_last_slot.assign((size_t)B * Gmax, -1);
        for (int32_t p = 0; p < B; ++p)
            for (int32_t g = 0; g < rl.num_groups[p]; ++g)
                b->group_last_slot[(size_t)p * Gmax + g] =
                    (int16_t)(slot0[(size_t)p * Gmax + g] + t->cfg_pp[rl.group_cfg[(size_t)p * Gmax + g]] - 1);
    }
    if (flags & MMSIM_WANT_PER_REQUEST) {
        HIP_TRY(b->finish.alloc(lanes_padded * (size_t)b->Rmax));
        HIP_TRY(b->good.alloc(lanes_padded * (size_t)b->Rmax));
    }
    if (flags & MMSIM_WANT_OP_COUNT) HIP_TRY(b->fp_ops.alloc(lanes_padded));
    if (g_arena) {
        b->own_events = false;
        b->ev_start = ctx->ev_static[0];
        b->ev_stop = ctx->ev_static[1];
    } else {
        HIP_TRY(hipEventCreate(&b->ev_start));
        HIP_TRY(hipEventCreate(&b->ev_stop));
    }
    HIP_TRY(hipStreamSynchronize(st));  // host staging vectors go out of scope below

    phase("streams + uploads");
    // ---- loop over runs: the schedule's tables, and room to park clocks between segments
    if (!plan.empty()) {
        HIP_TRY(b->plan.alloc(plan.size()));
        HIP_TRY(hipMemcpy(b->plan.p, plan.data(), sizeof(int32_t) * plan.size(), hipMemcpyHostToDevice));
        if (b->max_nseg > 1) HIP_TRY(b->state.alloc((size_t)b->waves * nslots * kWave));
    }

    MixedArgs &a = b->args;
    a.state = b->state.p;
    a.state_rows = nslots;
    a.slot_rows = nslots;
    if (!plan.empty()) {
        const size_t groups = (size_t)b->sched_groups, total = (size_t)plan[groups];
        a.wg_off = b->plan.p;
        a.item_tile = a.wg_off + groups + 1;
        a.item_seed = a.item_tile + total;
        a.item_nslots = a.item_seed + total;
        a.item_bytes = a.item_nslots + total;
        a.item_nseg = a.item_bytes + total;
        a.part_off = a.item_nseg + total;
        a.part_bytes = a.part_off + groups * kMaxWavesPerBlock;
    }
    a.tile_seed = b->tile_seed.p;
    a.paired = b->paired ? 1 : 0;
    a.sched_groups = b->sched_groups;
    a.seg_requests = b->seg_requests;
    a.sched_lds_bytes = (int32_t)sched_bytes;
    a.sched_spin_limit = 20000;  // waits of 127 x 64 cycles: about 70 ms, several segments
    if (o.sched_spin_limit >= 0) a.sched_spin_limit = o.sched_spin_limit;
    a.streams = b->streams.p;
    a.stream_off = b->stream_off.p;
    a.rep32 = reinterpret_cast<const uint4 *>(b->rep32.p);
    a.repx32 = b->repx32.p;
    a.rmax = b->rmax.p;
    a.lat_lds_bytes = (int32_t)lat_bytes;
    a.error = b->kerr.p;
    a.lat = b->lat.p;
    a.M = M;
    a.lat_row = lat_row;
    a.rep_extra = RX;
    a.lat_in_lds = lat_in_lds;
    a.uniform_stages = uniform_stages ? 1 : 0;
    a.pow2_depths = pow2_depths ? 1 : 0;
    a.wave_lds_bytes = (int32_t)wave_bytes;
    a.rmax_lds_bytes = rmax_lds_bytes;
    a.n_seeds = n_seeds;
    a.B = B;
    a.tiles = b->tiles;
    a.nslots = nslots;
    a.Gmax = Gmax;
    a.Rmax = b->Rmax;
    a.fixed_overhead = t->fixed_overhead;
    a.flags = flags;
    a.n_good = b->n_good.p;
    a.lat_sum = b->lat_sum.p;
    a.model_good = b->model_good.p;
    a.model_lds = model_lds_bytes ? 1 : 0;
    a.group_lds = b->group_lds;
    a.slot_cnt = b->slot_cnt.p;
    a.xcd_map = 1;
    a.runs = runs ? 1 : 0;
    a.skip_ahead = o.skip_ahead >= 0 ? (o.skip_ahead ? 1 : 0) : 1;
    if (o.xcd_map >= 0) a.xcd_map = o.xcd_map ? 1 : 0;
    a.finish = b->finish.p;
    a.good = b->good.p;
    a.fp_ops = b->fp_ops.p;
    if (batching) {
        BatchingArgs &q = b->bargs;
        q.streams = b->streams.p;
        q.stream_off = b->stream_off.p;
        q.mq_off = b->mq_off.p;
        q.mq = b->mq.p;
        q.rep8 = b->rep8.p;
        q.repx = b->repx.p;
        q.ginfo = b->ginfo.p;
        q.g2m_off = b->g2m_off.p;
        q.g2m_idx = b->g2m_idx.p;
        q.lat = b->lat_nb.p;
        q.batch_sizes = b->batch_sizes.p;
        q.M = M;
        q.lat_row = lat_row;
        q.NB = t->NB;
        q.rep_extra = RX;
        q.members_max = members_max;
        q.heap_cap = heap_cap;
        q.n_seeds = n_seeds;
        q.B = B;
        q.tiles = b->tiles;
        q.nslots = nslots;
        q.Gmax = Gmax;
        q.wave_lds_bytes = (int32_t)wave_bytes;
        q.lat_lds_bytes = (int32_t)batching_lat_lds;
        q.g2m_in_lds = batching_g2m_lds;
        q.lane_stride = blanes;
        q.uniform_stages = uniform_stages ? 1 : 0;
        q.tile_seed = b->tile_seed.p;
        q.paired = b->paired ? 1 : 0;
        q.Rmax = b->Rmax;
        q.fixed_overhead = t->fixed_overhead;
        q.flags = flags;
        q.n_good = b->n_good.p;
        q.lat_sum = b->lat_sum.p;
        q.status = b->status.p;
        q.model_good = b->model_good.p;
        q.group_req = b->group_req.p;
        q.group_good = b->group_good.p;
        q.finish = b->finish.p;
        q.good = b->good.p;
    }
    phase("schedule tables, kernel args");
    *out = b.release();
    return MMSIM_OK;
}

}  // namespace

extern "C" {

int mmsim_abi_version(void) { return MMSIM_ABI_VERSION; }

const char *mmsim_last_error(void) { return g_last_error.c_str(); }

void mmsim_options_default(mmsim_options *o) {
    if (!o) return;
    std::memset(o, 0, sizeof(*o));
    o->struct_size = (int32_t)sizeof(mmsim_options);
    o->request_loop = o->counts_in_lds = o->tile_order_by_slots = o->sched_spin_limit = -1;
    o->skip_ahead = o->xcd_map = o->batching_lds_tables = -1;
}

int mmsim_ctx_set_options(mmsim_ctx *ctx, const mmsim_options *options) {
    if (!ctx) return fail(MMSIM_E_INVALID, "ctx_set_options: null context");
    int rc = check_options(options);
    if (rc) return rc;
    if (options)
        ctx->opt = *options;
    else
        mmsim_options_default(&ctx->opt);
    return MMSIM_OK;
}

int mmsim_ctx_create(int device, mmsim_ctx **out) {
    if (!out) return fail(MMSIM_E_INVALID, "ctx_create: out is null");
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count < 1)
        return fail(MMSIM_E_HIP, std::string("no usable HIP device: ") + (e != hipSuccess ? hipGetErrorString(e) : "device count is 0"));
    if (device < 0 || device >= count) return fail(MMSIM_E_INVALID, "ctx_create: device ordinal out of range");
    std::unique_ptr<mmsim_ctx> c(new (std::nothrow) mmsim_ctx);
    if (!c) return fail(MMSIM_E_NOMEM, "host allocation failed");
    c->device = device;
    mmsim_options_default(&c->opt);
    HIP_TRY(hipSetDevice(device));
    HIP_TRY(hipGetDeviceProperties(&c->prop, device));
    if (std::strncmp(c->prop.gcnArchName, "gfx950", 6) != 0)
        return fail(MMSIM_E_UNSUPPORTED, std::string("libmmsim is built for gfx950 only, device is ") + c->prop.gcnArchName);
    int lds = 0;
    if (hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerBlock, device) != hipSuccess || lds <= 0)
        lds = (int)c->prop.sharedMemPerBlock;
    c->max_lds = lds;
    HIP_TRY(hipStreamCreate(&c->stream));  // default priority, like every stream of the library
    HIP_TRY(hipEventCreate(&c->ev_static[0]));
    HIP_TRY(hipEventCreate(&c->ev_static[1]));
    {   // address of this device's copy of the static scratch: once per device, with that device current
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        if (device < kMaxDevices && g_scratch_ptr[device]) {
            c->scratch = g_scratch_ptr[device];
        } else {
            void *sp = nullptr;
            HIP_TRY(hipGetSymbolAddress(&sp, HIP_SYMBOL(scratch)));
            if (!sp) return fail(MMSIM_E_HIP, "ctx_create: the static scratch has no device address");
            c->scratch = static_cast<unsigned char *>(sp);
            if (device < kMaxDevices) g_scratch_ptr[device] = c->scratch;
        }
    }
    *out = c.release();
    return MMSIM_OK;
}

void mmsim_ctx_destroy(mmsim_ctx *ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    if (ctx->stream) {
        (void)hipStreamSynchronize(ctx->stream);
        (void)hipStreamDestroy(ctx->stream);
    }
    for (hipEvent_t e : ctx->ev_static)
        if (e) (void)hipEventDestroy(e);
    delete ctx;
}

int mmsim_ctx_device_info(mmsim_ctx *ctx, mmsim_device_info *out) {
    if (!ctx || !out) return fail(MMSIM_E_INVALID, "device_info: null pointer");
    std::memset(out, 0, sizeof(*out));
    std::snprintf(out->name, sizeof(out->name), "%s", ctx->prop.name);
    std::snprintf(out->arch, sizeof(out->arch), "%s", ctx->prop.gcnArchName);
    out->compute_units = ctx->prop.multiProcessorCount;
    out->clock_khz = ctx->prop.clockRate;
    out->lds_bytes_per_block = ctx->max_lds;
    out->hbm_bytes = (int64_t)ctx->prop.totalGlobalMem;
    return MMSIM_OK;
}

int mmsim_workload_create(mmsim_ctx *ctx, int64_t R, int32_t M, const double *tstamps, const int32_t *model_ids,
                          const float *slos, mmsim_workload **out) {
    if (!ctx || !out) return fail(MMSIM_E_INVALID, "workload_create: null pointer");
    *out = nullptr;
    if (R < 0 || M < 1) return fail(MMSIM_E_INVALID, "workload_create: R must be >= 0 and M >= 1");
    if (R > 0 && (!tstamps || !model_ids || !slos)) return fail(MMSIM_E_INVALID, "workload_create: null array");
    if (R > 0x7FFFFFFF) return fail(MMSIM_E_UNSUPPORTED, "workload_create: more than 2^31-1 requests");
    std::unique_ptr<mmsim_workload> w(new (std::nothrow) mmsim_workload);
    if (!w) return fail(MMSIM_E_NOMEM, "host allocation failed");
    w->ctx = ctx;
    w->id = g_next_workload_id.fetch_add(1);
    w->R = R;
    w->M = M;
    w->model_num_requests.assign(M, 0);
    std::vector<Req> host((size_t)R);
    bool sorted = true;
    for (int64_t i = 0; i < R; ++i) {
        if (model_ids[i] >= M) return fail(MMSIM_E_INVALID, "workload_create: model id >= M");
        if (tstamps[i] != tstamps[i]) return fail(MMSIM_E_INVALID, "workload_create: arrival time is NaN");
        host[i].t = tstamps[i];
        host[i].m = model_ids[i] < 0 ? -1 : model_ids[i];
        host[i].slo = slos[i];
        if (model_ids[i] >= 0) w->model_num_requests[model_ids[i]] += 1;
        if (i > 0 && host[i].m == host[i - 1].m) w->repeats += 1;
        if (i > 0 && tstamps[i] < tstamps[i - 1]) sorted = false;
    }
    w->mq_off.assign((size_t)M + 1, 0);
    for (int32_t m = 0; m < M; ++m) w->mq_off[m + 1] = w->mq_off[m] + w->model_num_requests[m];
    const size_t known = (size_t)w->mq_off[M];
    std::vector<MqEntry> mq(known);
    {
        // dense rank of every arrival time: one pass over a sorted stream (the normal case), a sort otherwise
        std::vector<int32_t> rank((size_t)R, 0);
        if (sorted) {
            for (int64_t i = 1; i < R; ++i) rank[(size_t)i] = rank[(size_t)i - 1] + (tstamps[i] != tstamps[i - 1] ? 1 : 0);
        } else {
            std::vector<int32_t> order((size_t)R);
            for (int64_t i = 0; i < R; ++i) order[(size_t)i] = (int32_t)i;
            std::stable_sort(order.begin(), order.end(), [&](int32_t x, int32_t y) { return tstamps[x] < tstamps[y]; });
            int32_t r = 0;
            for (int64_t k = 0; k < R; ++k) {
                if (k > 0 && tstamps[order[(size_t)k]] != tstamps[order[(size_t)k - 1]]) ++r;
                rank[(size_t)order[(size_t)k]] = r;
            }
        }
        std::vector<int64_t> fill(w->mq_off.begin(), w->mq_off.end() - 1);
        for (int64_t i = 0; i < R; ++i)
            if (model_ids[i] >= 0) {
                MqEntry &e = mq[(size_t)fill[model_ids[i]]++];
                e.t = tstamps[i];
                e.dl = tstamps[i] + (double)slos[i];  // controller.py:679
                e.idx = (int32_t)i;
                e.rank = rank[(size_t)i];
                e.pad[0] = e.pad[1] = 0;
            }
    }
    HIP_TRY(hipSetDevice(ctx->device));
    HIP_TRY(w->reqs.alloc((size_t)R));
    HIP_TRY(w->mq.alloc(known));
    if (R > 0) {
        HIP_TRY(hipMemcpyAsync(w->reqs.p, host.data(), sizeof(Req) * (size_t)R, hipMemcpyHostToDevice, ctx->stream));
        if (known > 0) {
            HIP_TRY(hipMemcpyAsync(w->mq.p, mq.data(), sizeof(MqEntry) * known, hipMemcpyHostToDevice, ctx->stream));
        }
        HIP_TRY(hipStreamSynchronize(ctx->stream));
    }
    *out = w.release();
    return MMSIM_OK;
}

void mmsim_workload_destroy(mmsim_workload *wl) {
    if (!wl) return;
    if (wl->ctx) (void)hipSetDevice(wl->ctx->device);
    delete wl;
}

int mmsim_batch_create_ex(mmsim_ctx *ctx, const mmsim_workload *const *workloads, int32_t n_seeds,
                          const mmsim_tables *tables, const mmsim_placements *placements, uint32_t flags,
                          const mmsim_options *options, mmsim_batch **out) {
    if (!ctx || !out) return fail(MMSIM_E_INVALID, "batch_create: null pointer");
    *out = nullptr;
    int rc = check_tables(tables);
    if (rc) return rc;
    rc = check_options(options);
    if (rc) return rc;
    RepLists rl;
    rc = lists_from_placements(placements, tables->M, tables->C, &rl);
    if (rc) return rc;
    return build_batch(ctx, workloads, n_seeds, tables, rl, flags, out, nullptr, options);
}

int mmsim_batch_create(mmsim_ctx *ctx, const mmsim_workload *const *workloads, int32_t n_seeds,
                       const mmsim_tables *tables, const mmsim_placements *placements, uint32_t flags,
                       mmsim_batch **out) {
    return mmsim_batch_create_ex(ctx, workloads, n_seeds, tables, placements, flags, nullptr, out);
}

int mmsim_batch_run(mmsim_batch *b) {
    if (!b) return fail(MMSIM_E_INVALID, "batch_run: null batch");
    mmsim_ctx *ctx = b->ctx;
    HIP_TRY(hipSetDevice(ctx->device));
    if (b->flags & MMSIM_WANT_MODEL_COUNTS)
        HIP_TRY(hipMemsetAsync(b->model_good.p, 0, b->model_good.bytes(), ctx->stream));
    if (b->group_by_slot) {
        HIP_TRY(hipMemsetAsync(b->slot_cnt.p, 0, b->slot_cnt.bytes(), ctx->stream));
    }
    if ((b->flags & MMSIM_BATCHING) && (b->flags & MMSIM_WANT_GROUP_COUNTS)) {
        HIP_TRY(hipMemsetAsync(b->group_req.p, 0, b->group_req.bytes(), ctx->stream));
        HIP_TRY(hipMemsetAsync(b->group_good.p, 0, b->group_good.bytes(), ctx->stream));
    }
    if (b->sched_groups > 0) HIP_TRY(hipMemsetAsync(b->kerr.p + 1, 0, sizeof(int32_t), ctx->stream));  // items completed
    HIP_TRY(hipEventRecord(b->ev_start, ctx->stream));
    std::string err;
    if (b->flags & MMSIM_BATCHING) {
        if (launch_sim_batching(b->bargs, b->waves_per_block, b->lds_bytes, ctx->stream, &err) != hipSuccess) return fail(MMSIM_E_HIP, err);
    } else {
        if (launch_sim_mixed(b->args, b->smax_bucket, b->waves_per_block, b->lds_bytes, ctx->stream, &err) != hipSuccess)
            return fail(MMSIM_E_HIP, err);
    }
    HIP_TRY(hipEventRecord(b->ev_stop, ctx->stream));
    b->ran = true;
    return MMSIM_OK;
}

int mmsim_batch_sync(mmsim_batch *b, float *kernel_ms) {
    if (!b) return fail(MMSIM_E_INVALID, "batch_sync: null batch");
    if (!b->ran) return fail(MMSIM_E_INVALID, "batch_sync: batch was never run");
    HIP_TRY(hipSetDevice(b->ctx->device));
    HIP_TRY(hipEventSynchronize(b->ev_stop));
    if (kernel_ms) HIP_TRY(hipEventElapsedTime(kernel_ms, b->ev_start, b->ev_stop));
    return MMSIM_OK;
}

int mmsim_batch_fetch(mmsim_batch *b, mmsim_result *out) {
    if (!b || !out) return fail(MMSIM_E_INVALID, "batch_fetch: null pointer");
    if (!b->ran) return fail(MMSIM_E_INVALID, "batch_fetch: batch was never run");
    if (!out->n_good || !out->latency_sum) return fail(MMSIM_E_INVALID, "batch_fetch: n_good and latency_sum are required");
    const bool wm = b->flags & MMSIM_WANT_MODEL_COUNTS, wg = b->flags & MMSIM_WANT_GROUP_COUNTS,
               wr = (b->flags & MMSIM_WANT_PER_REQUEST) && out->finish && out->good;  // left on the device if not asked for
    if (wm && (!out->model_num_requests || !out->model_num_good)) return fail(MMSIM_E_INVALID, "batch_fetch: model count arrays missing");
    if (wg && (!out->group_num_requests || !out->group_num_good)) return fail(MMSIM_E_INVALID, "batch_fetch: group count arrays missing");
    HIP_TRY(hipSetDevice(b->ctx->device));
    HIP_TRY(hipStreamSynchronize(b->ctx->stream));

    if (!(b->flags & MMSIM_BATCHING)) {
        int32_t kerrs[32] = {};
        HIP_TRY(hipMemcpy(kerrs, b->kerr.p, sizeof(kerrs), hipMemcpyDeviceToHost));
        const int32_t kerr = kerrs[0];
        if (kerr == 1) return fail(MMSIM_E_HIP, "simulation kernel: dynamic LDS does not start at address 0; results are invalid");
        if (kerr != 0) return fail(MMSIM_E_HIP, "simulation kernel: unexpected error flag; results are invalid");
        if (b->sched_groups > 0 && kerrs[1] != b->waves)
            return fail(MMSIM_E_HIP, "simulation kernel: the schedule completed " + std::to_string(kerrs[1]) + " of " +
                                         std::to_string(b->waves) + " (tile, stream) items; results are invalid");
    }
    const int32_t B = b->B, M = b->M, Gmax = b->Gmax, tiles = b->tiles;
    const size_t lanes_padded = (size_t)b->waves * kWave;
    std::vector<int32_t> ng(lanes_padded);
    std::vector<double> ls(lanes_padded);
    HIP_TRY(hipMemcpy(ng.data(), b->n_good.p, sizeof(int32_t) * lanes_padded, hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(ls.data(), b->lat_sum.p, sizeof(double) * lanes_padded, hipMemcpyDeviceToHost));
    std::vector<int32_t> st_host;
    int any_bad = 0;
    if (b->flags & MMSIM_BATCHING) {
        st_host.resize(lanes_padded);
        HIP_TRY(hipMemcpy(st_host.data(), b->status.p, sizeof(int32_t) * lanes_padded, hipMemcpyDeviceToHost));
    }
    std::vector<int64_t> ops;
    if (b->flags & MMSIM_WANT_OP_COUNT) {
        if (!out->fp_ops) return fail(MMSIM_E_INVALID, "batch_fetch: fp_ops array missing");
        ops.resize(lanes_padded);
        HIP_TRY(hipMemcpy(ops.data(), b->fp_ops.p, sizeof(int64_t) * lanes_padded, hipMemcpyDeviceToHost));
    }
    for (int s = 0; s < b->out_seeds; ++s)
        for (int32_t p = 0; p < B; ++p) {
            const size_t src = (size_t)s * tiles * kWave + b->pos[p];
            out->n_good[(size_t)s * B + p] = ng[src];
            out->latency_sum[(size_t)s * B + p] = ls[src];
            if (out->status) out->status[(size_t)s * B + p] = st_host.empty() ? 0 : st_host[src];
            if (!st_host.empty() && st_host[src] != 0) any_bad = st_host[src];
            if (!ops.empty()) out->fp_ops[(size_t)s * B + p] = ops[src];
        }
    // device rows are [wave][x][64] with wave = seed*tiles + tile; lane l of a seed is placement l
    auto unpack_i32 = [&](const DevBuf<int32_t> &dev, int32_t width, int32_t *dst) -> int {
        std::vector<int32_t> h(dev.n);
        HIP_TRY(hipMemcpy(h.data(), dev.p, dev.bytes(), hipMemcpyDeviceToHost));
        for (int s = 0; s < b->out_seeds; ++s)
            for (int32_t p = 0; p < B; ++p) {
                const size_t wave = (size_t)s * tiles + b->pos[p] / kWave;
                for (int32_t x = 0; x < width; ++x)
                    dst[((size_t)s * B + p) * width + x] = h[(wave * width + x) * kWave + b->pos[p] % kWave];
            }
        return MMSIM_OK;
    };
    if (wm) {
        int rc = unpack_i32(b->model_good, M, out->model_num_good);
        if (rc) return rc;
        for (int s = 0; s < b->out_seeds; ++s)
            for (int32_t p = 0; p < B; ++p)
                for (int32_t m = 0; m < M; ++m)  // the batching loop only counts requests of hosted models (:754-757, :773)
                    out->model_num_requests[((size_t)s * B + p) * M + m] =
                        (b->hosted.empty() || b->hosted[(size_t)p * M + m]) ? b->wl_model_requests[(size_t)(b->paired ? b->stream_of[p] : s)][m] : 0;
    }
    if (wg && b->group_by_slot) {  // counted per last clock slot of the group: map slots back to groups
        std::vector<unsigned long long> h(b->slot_cnt.n);
        HIP_TRY(hipMemcpy(h.data(), b->slot_cnt.p, b->slot_cnt.bytes(), hipMemcpyDeviceToHost));
        const size_t rows = (size_t)b->slot_rows;
        for (int s = 0; s < b->out_seeds; ++s)
            for (int32_t p = 0; p < B; ++p) {
                const size_t wave = (size_t)s * tiles + b->pos[p] / kWave;
                for (int32_t g = 0; g < Gmax; ++g) {
                    const int slot = b->group_last_slot[(size_t)p * Gmax + g];
                    const unsigned long long v = slot < 0 ? 0ull : h[(wave * rows + slot) * kWave + b->pos[p] % kWave];
                    out->group_num_requests[((size_t)s * B + p) * Gmax + g] = (int32_t)(v & 0xFFFFFFFFull);
                    out->group_num_good[((size_t)s * B + p) * Gmax + g] = (int32_t)(v >> 32);
                }
            }
    } else if (wg) {
        int rc = unpack_i32(b->group_req, Gmax, out->group_num_requests);
        if (rc) return rc;
        rc = unpack_i32(b->group_good, Gmax, out->group_num_good);
        if (rc) return rc;
    }
    if (wr && b->Rmax > 0) {
        const size_t Rm = (size_t)b->Rmax;
        std::vector<double> hf(Rm * kWave);
        std::vector<uint8_t> hg(Rm * kWave);
        std::vector<int32_t> owner((size_t)tiles * kWave, -1);  // placement simulated on each lane
        for (int32_t p = 0; p < B; ++p) owner[b->pos[p]] = p;
        for (int s = 0; s < b->out_seeds; ++s)
            for (int32_t tile = 0; tile < tiles; ++tile) {
                const size_t wave = (size_t)s * tiles + tile;
                HIP_TRY(hipMemcpy(hf.data(), b->finish.p + wave * Rm * kWave, sizeof(double) * Rm * kWave, hipMemcpyDeviceToHost));
                HIP_TRY(hipMemcpy(hg.data(), b->good.p + wave * Rm * kWave, Rm * kWave, hipMemcpyDeviceToHost));
                for (int l = 0; l < kWave; ++l) {
                    const int32_t p = owner[(size_t)tile * kWave + l];
                    if (p < 0) continue;
                    const size_t Rs = (size_t)b->wl_R[(size_t)(b->paired ? b->stream_of[p] : s)];
                    const size_t row = ((size_t)s * B + (size_t)p) * Rm;
                    for (size_t i = 0; i < Rs; ++i) {
                        out->finish[row + i] = hf[i * kWave + l];
                        out->good[row + i] = hg[i * kWave + l];
                    }
                }
            }
    }
    if (any_bad && !out->status)
        return fail(any_bad, any_bad == MMSIM_E_OVERFLOW
                                 ? "a simulation ran out of idle-event slots; its results are invalid (pass status[] to see which)"
                                 : "a simulation hit an input the batching simulator does not support (all replica clocks infinite)");
    return MMSIM_OK;
}

int mmsim_batch_model_stats(mmsim_batch *b, const mmsim_workload *const *workloads, int32_t n_streams,
                            const int64_t *skip, mmsim_model_stats *out) {
    if (!b || !workloads || !skip || !out) return fail(MMSIM_E_INVALID, "batch_model_stats: null pointer");
    if (!b->ran) return fail(MMSIM_E_INVALID, "batch_model_stats: batch was never run");
    if (!(b->flags & MMSIM_WANT_PER_REQUEST))
        return fail(MMSIM_E_INVALID, "batch_model_stats: the batch was created without MMSIM_WANT_PER_REQUEST");
    if (n_streams != b->n_seeds) return fail(MMSIM_E_INVALID, "batch_model_stats: pass the request streams the batch was created with");
    if (!out->model_num_requests || !out->model_num_good || !out->first_start || !out->last_start || !out->latency_sum ||
        !out->latency_mean || !out->latency_std || !out->latency_p90 || !out->latency_p99)
        return fail(MMSIM_E_INVALID, "batch_model_stats: every result array is required");
    const int32_t B = b->B, M = b->M, tiles = b->tiles;
    std::vector<const MqEntry *> mq((size_t)n_streams);
    std::vector<int64_t> mqo((size_t)n_streams * (M + 1)), lo((size_t)n_streams), hi((size_t)n_streams);
    for (int s = 0; s < n_streams; ++s) {
        const mmsim_workload *w = workloads[s];
        if (!w || w->ctx != b->ctx || w->id != b->wl_id[(size_t)s] || w->M != M || w->R != b->wl_R[(size_t)s])
            return fail(MMSIM_E_INVALID, "batch_model_stats: pass the request streams the batch was created with "
                                         "(the same workload objects, in the same order, still alive)");
        if (skip[s] < 0) return fail(MMSIM_E_INVALID, "batch_model_stats: negative skip");
        mq[(size_t)s] = w->mq.p;
        for (int32_t m = 0; m <= M; ++m) mqo[(size_t)s * (M + 1) + m] = w->mq_off[(size_t)m];
        lo[(size_t)s] = std::min<int64_t>(skip[s], w->R);   // start[skip:-skip], workload.py:315-318
        hi[(size_t)s] = std::max<int64_t>(lo[(size_t)s], w->R - skip[s]);
    }
    HIP_TRY(hipSetDevice(b->ctx->device));
    hipStream_t st = b->ctx->stream;
    // one workgroup per (simulation, model), results already in the caller's layout; a launch needs a scratch row
    // of 8 bytes per request for each of its simulations, so many simulations take several launches
    const int64_t n_sims = (int64_t)b->out_seeds * B;
    int64_t pitch = 1;
    for (int s = 0; s < n_streams; ++s) pitch = std::max<int64_t>(pitch, workloads[s]->mq_off[(size_t)M]);
    const int64_t scratch_bytes = b->opt.stats_scratch_bytes > 0 ? b->opt.stats_scratch_bytes : kStatsScratchBytes;
    const int64_t rows = std::max<int64_t>(1, std::min<int64_t>(n_sims, scratch_bytes / (pitch * (int64_t)sizeof(uint64_t))));
    std::vector<int32_t> sim_stream((size_t)n_sims);
    std::vector<int64_t> sim_base((size_t)n_sims);
    for (int s = 0; s < b->out_seeds; ++s)
        for (int32_t p = 0; p < B; ++p) {
            const size_t sim = (size_t)s * B + p;
            const int64_t wave = (int64_t)s * tiles + b->pos[p] / kWave;
            sim_stream[sim] = b->paired ? b->stream_of[p] : s;
            sim_base[sim] = wave * b->Rmax * kWave + b->pos[p] % kWave;
        }
    const size_t cells = (size_t)n_sims * (size_t)M;
    // (the buffers belong to the batch: the first call makes them, later calls allocate nothing)
    DevBuf<const MqEntry *> &d_mq = b->st_mq;
    DevBuf<int64_t> &d_i64 = b->st_i64;
    DevBuf<int32_t> &d_i32 = b->st_i32;
    DevBuf<double> &d_f64 = b->st_f64;
    DevBuf<uint64_t> &d_scratch = b->st_scratch;
    if (d_mq.n < mq.size()) HIP_TRY(d_mq.alloc(mq.size()));
    if (d_i64.n < mqo.size() + 2 * (size_t)n_streams + (size_t)n_sims) HIP_TRY(d_i64.alloc(mqo.size() + 2 * (size_t)n_streams + (size_t)n_sims));
    if (d_i32.n < (size_t)n_sims + 2 * cells) HIP_TRY(d_i32.alloc((size_t)n_sims + 2 * cells));
    if (d_f64.n < 7 * cells) HIP_TRY(d_f64.alloc(7 * cells));
    if (d_scratch.n < (size_t)rows * (size_t)pitch) HIP_TRY(d_scratch.alloc((size_t)rows * (size_t)pitch));
    HIP_TRY(hipMemcpyAsync(d_mq.p, mq.data(), sizeof(mq[0]) * mq.size(), hipMemcpyHostToDevice, st));
    int64_t *i64 = d_i64.p;
    std::vector<int64_t> up;  // one upload: mq_off | lo | hi | sim_base (alive until the stream is waited for below)
    up.reserve(mqo.size() + 2 * lo.size() + sim_base.size());
    up.insert(up.end(), mqo.begin(), mqo.end());
    up.insert(up.end(), lo.begin(), lo.end());
    up.insert(up.end(), hi.begin(), hi.end());
    up.insert(up.end(), sim_base.begin(), sim_base.end());
    HIP_TRY(hipMemcpyAsync(i64, up.data(), sizeof(int64_t) * up.size(), hipMemcpyHostToDevice, st));
    HIP_TRY(hipMemcpyAsync(d_i32.p, sim_stream.data(), sizeof(int32_t) * sim_stream.size(), hipMemcpyHostToDevice, st));
    StatsArgs f{};
    f.finish = b->finish.p;
    f.good = b->good.p;
    f.mq = d_mq.p;
    f.mq_off = i64;
    f.lo = i64 + mqo.size();
    f.hi = f.lo + n_streams;
    f.sim_base = f.hi + n_streams;
    f.sim_stream = d_i32.p;
    f.scratch = d_scratch.p;
    f.scratch_pitch = pitch;
    f.M = M;
    f.model_req = d_i32.p + n_sims;
    f.model_good = f.model_req + cells;
    double *d = d_f64.p;
    double **slots[7] = {&f.first_start, &f.last_start, &f.latency_sum, &f.latency_mean, &f.latency_std, &f.latency_p90, &f.latency_p99};
    for (int k = 0; k < 7; ++k) *slots[k] = d + (size_t)k * cells;
    for (int64_t sim0 = 0; sim0 < n_sims; sim0 += rows) {  // launches on one stream: the scratch rows are reused in order
        f.sim0 = (int32_t)sim0;
        std::string err;
        hipError_t e = launch_model_stats(f, (int)std::min<int64_t>(rows, n_sims - sim0), st, &err);
        if (e != hipSuccess) return fail(MMSIM_E_HIP, err.empty() ? std::string("model_stats launch: ") + hipGetErrorString(e) : err);
    }
    // two copies back (the integer results, the double results), then into the caller's arrays
    std::vector<int32_t> h_i32(2 * cells);
    std::vector<double> h_f64(7 * cells);
    HIP_TRY(hipMemcpyAsync(h_i32.data(), f.model_req, sizeof(int32_t) * 2 * cells, hipMemcpyDeviceToHost, st));
    HIP_TRY(hipMemcpyAsync(h_f64.data(), d, sizeof(double) * 7 * cells, hipMemcpyDeviceToHost, st));
    HIP_TRY(hipStreamSynchronize(st));
    std::memcpy(out->model_num_requests, h_i32.data(), sizeof(int32_t) * cells);
    std::memcpy(out->model_num_good, h_i32.data() + cells, sizeof(int32_t) * cells);
    double *const o64[7] = {out->first_start, out->last_start, out->latency_sum, out->latency_mean,
                            out->latency_std, out->latency_p90, out->latency_p99};
    for (int k = 0; k < 7; ++k) std::memcpy(o64[k], h_f64.data() + (size_t)k * cells, sizeof(double) * cells);
    return MMSIM_OK;
}

void mmsim_batch_destroy(mmsim_batch *b) {
    if (!b) return;
    if (b->ctx) {
        (void)hipSetDevice(b->ctx->device);
        (void)hipStreamSynchronize(b->ctx->stream);
    }
    delete b;
}

int mmsim_batch_get_info(const mmsim_batch *b, mmsim_batch_info *out) {
    if (!b || !out) return fail(MMSIM_E_INVALID, "batch_get_info: null pointer");
    out->lanes = b->B * b->out_seeds;
    out->waves = b->waves;
    out->n_seeds = b->n_seeds;
    out->B = b->B;
    out->smax_bucket = b->smax_bucket;
    out->max_replicas = b->rmax_all;
    out->slots = b->nslots;
    out->lds_bytes = (int32_t)b->lds_bytes;
    out->requests_total = b->Rtotal;
    out->table_bytes = (int64_t)(b->rep32.bytes() + b->repx32.bytes() + b->rep8.bytes() + b->repx.bytes() + b->ginfo.bytes() +
                                 b->rmax.bytes() + b->lat.bytes() + b->lat_nb.bytes());
    out->stream_bytes = (int64_t)b->streams.bytes();
    out->workgroups = b->sched_groups;
    out->segments = b->max_nseg;
    out->launches = 1;
    out->waves_per_group = b->waves_per_block;
    out->event_slots = (b->flags & MMSIM_BATCHING) ? b->bargs.heap_cap : 0;
    out->reserved = 0;
    return MMSIM_OK;
}

int mmsim_batch_kernel_name(const mmsim_batch *b, char *buf, size_t size) {
    if (!b || !buf || size == 0) return fail(MMSIM_E_INVALID, "batch_kernel_name: null pointer or empty buffer");
    const std::string name = (b->flags & MMSIM_BATCHING) ? sim_batching_kernel_name(b->bargs)
                                                         : sim_mixed_kernel_name(b->args, b->smax_bucket);
    std::snprintf(buf, size, "%s", name.c_str());
    return MMSIM_OK;
}

namespace {

// One-call evaluation with the given options (nullptr: the context's): every placement on every stream, or, with
// stream_of, placement b on workloads[stream_of[b]] only.  event_slots (optional) receives the event slots per
// simulation that the batching simulator was given.
int eval_once(mmsim_ctx *ctx, const mmsim_workload *const *workloads, int32_t n_streams, const mmsim_tables *tables,
              const mmsim_placements *placements, const int32_t *stream_of, uint32_t flags, const mmsim_options *options,
              mmsim_result *out, int *event_slots) {
    int rc = check_tables(tables);
    if (rc) return rc;
    rc = check_options(options);
    if (rc) return rc;
    RepLists rl;
    rc = lists_from_placements(placements, tables->M, tables->C, &rl);
    if (rc) return rc;
    mmsim_batch *b = nullptr;
    rc = build_batch(ctx, workloads, n_streams, tables, rl, flags, &b, stream_of, options);
    if (rc == MMSIM_OK && event_slots) *event_slots = b->bargs.heap_cap;
    if (rc == MMSIM_OK) rc = mmsim_batch_run(b);
    if (rc == MMSIM_OK) rc = mmsim_batch_sync(b, nullptr);
    if (rc == MMSIM_OK) rc = mmsim_batch_fetch(b, out);
    mmsim_batch_destroy(b);
    return rc;
}

// The batching simulator gives every simulation a fixed number of idle-event slots (what the reference's heap is
// seen to need, and what fits in LDS); a simulation that needs more stops with MMSIM_E_OVERFLOW.  Those are
// simulated again here, alone and with twice the slots, until they fit or LDS says no (they then keep that status).
int eval_with_retry(mmsim_ctx *ctx, const mmsim_workload *const *workloads, int32_t n_streams, const mmsim_tables *tables,
                    const mmsim_placements *placements, const int32_t *stream_of, uint32_t flags, mmsim_result *out) {
    const bool watch = (flags & MMSIM_BATCHING) != 0 && placements && n_streams > 0 && placements->B > 0;
    const int32_t rows = stream_of ? 1 : n_streams;  // simulations per placement
    std::vector<int32_t> own_status;
    mmsim_result res = *out;
    if (watch && !res.status) {
        own_status.assign((size_t)rows * placements->B, 0);
        res.status = own_status.data();
    }
    int slots = 0;
    int rc = eval_once(ctx, workloads, n_streams, tables, placements, stream_of, flags, nullptr, &res, &slots);
    if (rc != MMSIM_OK || !watch) return rc;
    const int32_t B = placements->B, Gmax = placements->Gmax, M = tables->M;
    const size_t G1 = (size_t)Gmax + 1;
    int64_t Rmax = 0;
    for (int s = 0; s < n_streams; ++s) Rmax = std::max(Rmax, workloads[s]->R);
    for (int round = 0; round < 8; ++round) {
        std::vector<int32_t> again;
        for (int32_t p = 0; p < B; ++p)
            for (int s = 0; s < rows; ++s)
                if (res.status[(size_t)s * B + p] == MMSIM_E_OVERFLOW) {
                    again.push_back(p);
                    break;
                }
        if (again.empty()) break;
        slots *= 2;
        const int32_t B2 = (int32_t)again.size();
        std::vector<int32_t> ng(B2), gc((size_t)B2 * Gmax), idx, so(B2, 0);
        std::vector<int64_t> off((size_t)B2 * G1);
        for (int32_t k = 0; k < B2; ++k) {
            const int32_t p = again[k];
            ng[k] = placements->num_groups[p];
            if (stream_of) so[k] = stream_of[p];
            std::copy(placements->group_cfg + (size_t)p * Gmax, placements->group_cfg + (size_t)(p + 1) * Gmax, gc.begin() + (size_t)k * Gmax);
            for (size_t g = 0; g < G1; ++g) {
                const int64_t lo = placements->gm_off[(size_t)p * G1 + g];
                off[(size_t)k * G1 + g] = (int64_t)idx.size();
                if (g < (size_t)ng[k]) idx.insert(idx.end(), placements->gm_idx + lo, placements->gm_idx + placements->gm_off[(size_t)p * G1 + g + 1]);
            }
        }
        if (idx.empty()) idx.push_back(0);
        const mmsim_placements sub = {B2, Gmax, ng.data(), gc.data(), off.data(), idx.data()};
        const size_t L2 = (size_t)rows * B2;
        std::vector<int64_t> n_good(L2);
        std::vector<double> lat_sum(L2), finish;
        std::vector<int32_t> mreq, mgood, greq, ggood, status(L2);
        std::vector<uint8_t> good;
        mmsim_result r2{};
        r2.n_good = n_good.data();
        r2.latency_sum = lat_sum.data();
        r2.status = status.data();
        if (flags & MMSIM_WANT_MODEL_COUNTS) {
            mreq.resize(L2 * M), mgood.resize(L2 * M);
            r2.model_num_requests = mreq.data(), r2.model_num_good = mgood.data();
        }
        if (flags & MMSIM_WANT_GROUP_COUNTS) {
            greq.resize(L2 * Gmax), ggood.resize(L2 * Gmax);
            r2.group_num_requests = greq.data(), r2.group_num_good = ggood.data();
        }
        if ((flags & MMSIM_WANT_PER_REQUEST) && res.finish && res.good) {
            finish.resize(L2 * (size_t)Rmax), good.resize(L2 * (size_t)Rmax);
            r2.finish = finish.data(), r2.good = good.data();
        }
        mmsim_options o = ctx->opt;
        o.batching_event_slots = slots;
        if (eval_once(ctx, workloads, n_streams, tables, &sub, stream_of ? so.data() : nullptr, flags, &o, &r2, nullptr) != MMSIM_OK)
            break;  // (does not fit in LDS)
        for (int32_t k = 0; k < B2; ++k)
            for (int s = 0; s < rows; ++s) {
                const size_t src = (size_t)s * B2 + k, dst = (size_t)s * B + again[k];
                if (res.n_good) res.n_good[dst] = n_good[src];
                if (res.latency_sum) res.latency_sum[dst] = lat_sum[src];
                res.status[dst] = status[src];
                if (r2.model_num_requests && res.model_num_requests) std::copy(&mreq[src * M], &mreq[src * M] + M, res.model_num_requests + dst * M);
                if (r2.model_num_good && res.model_num_good) std::copy(&mgood[src * M], &mgood[src * M] + M, res.model_num_good + dst * M);
                if (r2.group_num_requests && res.group_num_requests) std::copy(&greq[src * Gmax], &greq[src * Gmax] + Gmax, res.group_num_requests + dst * Gmax);
                if (r2.group_num_good && res.group_num_good) std::copy(&ggood[src * Gmax], &ggood[src * Gmax] + Gmax, res.group_num_good + dst * Gmax);
                if (r2.finish) {
                    std::copy(&finish[src * (size_t)Rmax], &finish[src * (size_t)Rmax] + Rmax, res.finish + dst * (size_t)Rmax);
                    std::copy(&good[src * (size_t)Rmax], &good[src * (size_t)Rmax] + Rmax, res.good + dst * (size_t)Rmax);
                }
            }
    }
    return MMSIM_OK;
}

}  // namespace

int mmsim_eval_batch(mmsim_ctx *ctx, const mmsim_workload *const *workloads, int32_t n_seeds,
                     const mmsim_tables *tables, const mmsim_placements *placements, uint32_t flags,
                     mmsim_result *out) {
    if (!ctx || !out) return fail(MMSIM_E_INVALID, "eval_batch: null pointer");
    return eval_with_retry(ctx, workloads, n_seeds, tables, placements, nullptr, flags, out);
}

int mmsim_eval_successors(mmsim_ctx *ctx, const mmsim_workload *const *workloads, int32_t n_seeds,
                          const mmsim_tables *tables, const mmsim_placements *base, const mmsim_successors *successors,
                          uint32_t flags, mmsim_result *out) {
    if (!ctx || !out) return fail(MMSIM_E_INVALID, "eval_successors: null pointer");
    int rc = check_tables(tables);
    if (rc) return rc;
    ExpandedPlacements all;
    rc = expand_successors(base, successors, tables->M, &all);
    if (rc) return rc;
    return mmsim_eval_batch(ctx, workloads, n_seeds, tables, &all.view, flags, out);
}

int mmsim_eval_pairs(mmsim_ctx *ctx, const mmsim_workload *const *workloads, int32_t n_streams,
                     const mmsim_tables *tables, const mmsim_placements *placements, const int32_t *stream_of,
                     uint32_t flags, mmsim_result *out) {
    if (!ctx || !out || !stream_of) return fail(MMSIM_E_INVALID, "eval_pairs: null pointer");
    return eval_with_retry(ctx, workloads, n_streams, tables, placements, stream_of, flags, out);
}

int mmsim_eval_batch_static(mmsim_ctx *ctx, const mmsim_workload *const *workloads, int32_t n_seeds,
                            const mmsim_tables *tables, const mmsim_placements *placements, uint32_t flags,
                            mmsim_result *out) {
    if (!ctx || !out) return fail(MMSIM_E_INVALID, "eval_batch_static: null pointer");
    if (!ctx->scratch) return fail(MMSIM_E_HIP, "eval_batch_static: the context has no static scratch");
    int rc = check_tables(tables);
    if (rc) return rc;
    RepLists rl;
    rc = lists_from_placements(placements, tables->M, tables->C, &rl);
    if (rc) return rc;
    // Every device buffer of the batch is carved out of the device's static scratch (nothing is allocated or
    // freed on the device); the scratch keeps the last call's contents, and what must start at zero is
    // cleared by build_batch / mmsim_batch_run as for any batch.
    Arena arena;
    arena.base = ctx->scratch;
    arena.cap = MMSIM_STATIC_SCRATCH_BYTES;
    mmsim_batch *b = nullptr;
    g_arena = &arena;
    rc = build_batch(ctx, workloads, n_seeds, tables, rl, flags, &b);
    g_arena = nullptr;
    if (rc != MMSIM_OK && arena.overflow)
        return fail(MMSIM_E_NOMEM, "eval_batch_static: the batch (placements x models x seeds, streams, requested outputs) "
                                   "needs more device scratch than the static " +
                                       std::to_string((size_t)MMSIM_STATIC_SCRATCH_BYTES) + " bytes; use mmsim_eval_batch");
    if (rc == MMSIM_OK) rc = mmsim_batch_run(b);
    if (rc == MMSIM_OK) rc = mmsim_batch_sync(b, nullptr);
    if (rc == MMSIM_OK) rc = mmsim_batch_fetch(b, out);
    mmsim_batch_destroy(b);  // frees nothing on the device: the buffers belong to the scratch
    return rc;
}

int mmsim_simulate_requests_mixed(mmsim_ctx *ctx, double *finish, uint8_t *good, const double *tstamps,
                                  const int32_t *model_ids, const float *slos, const int32_t *m_id2g_id,
                                  const int32_t *num_stages, const float *stage_latency, int64_t num_requests,
                                  int32_t M, int32_t G, int32_t Smax, double fixed_overhead,
                                  int32_t *model_num_requests, int32_t *model_num_good_requests,
                                  int32_t *group_num_requests, int32_t *group_num_good_requests) {
    if (!ctx) return fail(MMSIM_E_INVALID, "simulate_requests_mixed: null context");
    if (M < 1 || G < 1 || Smax < 1 || num_requests < 0) return fail(MMSIM_E_INVALID, "simulate_requests_mixed: bad size");
    if (!m_id2g_id || !num_stages || !stage_latency || !model_num_requests || !model_num_good_requests ||
        !group_num_requests || !group_num_good_requests || (num_requests > 0 && (!finish || !good)))
        return fail(MMSIM_E_INVALID, "simulate_requests_mixed: null pointer");
    if (G > MMSIM_MAX_GROUPS) return fail(MMSIM_E_UNSUPPORTED, "simulate_requests_mixed: more than 254 groups");
    // every group is its own latency-table column
    mmsim_tables t{};
    t.M = M;
    t.C = G;
    t.Smax = Smax;
    t.NB = 1;
    t.cfg_lat = stage_latency;
    t.cfg_pp = num_stages;
    t.batch_sizes = nullptr;
    t.fixed_overhead = fixed_overhead;
    int rc = check_tables(&t);
    if (rc) return rc;
    RepLists rl;
    rl.B = 1;
    rl.M = M;
    rl.Gmax = G;
    rl.num_groups.assign(1, G);
    rl.group_cfg.resize(G);
    for (int g = 0; g < G; ++g) rl.group_cfg[g] = g;
    rl.off.assign((size_t)M + 1, 0);
    for (int32_t m = 0; m < M; ++m)
        for (int32_t j = 0; j < G; ++j) {
            const int32_t g = m_id2g_id[(size_t)m * G + j];
            if (g < 0) break;
            if (g >= G) return fail(MMSIM_E_INVALID, "simulate_requests_mixed: m_id2g_id names a group >= G");
            rl.grp.push_back(g);
            rl.off[m + 1] += 1;
        }
    for (int32_t m = 0; m < M; ++m) rl.off[m + 1] += rl.off[m];

    mmsim_workload *wl = nullptr;
    rc = mmsim_workload_create(ctx, num_requests, M, tstamps, model_ids, slos, &wl);
    if (rc) return rc;
    mmsim_batch *b = nullptr;
    const mmsim_workload *wls[1] = {wl};
    const uint32_t flags = MMSIM_WANT_MODEL_COUNTS | MMSIM_WANT_GROUP_COUNTS | MMSIM_WANT_PER_REQUEST;
    rc = build_batch(ctx, wls, 1, &t, rl, flags, &b);
    if (rc == MMSIM_OK) rc = mmsim_batch_run(b);
    if (rc == MMSIM_OK) rc = mmsim_batch_sync(b, nullptr);
    if (rc == MMSIM_OK) {
        int64_t ng = 0;
        double ls = 0.0;
        mmsim_result r{};
        r.n_good = &ng;
        r.latency_sum = &ls;
        r.model_num_requests = model_num_requests;
        r.model_num_good = model_num_good_requests;
        r.group_num_requests = group_num_requests;
        r.group_num_good = group_num_good_requests;
        r.finish = finish;
        r.good = good;
        rc = mmsim_batch_fetch(b, &r);
    }
    mmsim_batch_destroy(b);
    mmsim_workload_destroy(wl);
    return rc;
}

int mmsim_simulate_requests(mmsim_ctx *ctx, double *finish, uint8_t *good, const double *tstamps,
                            const int32_t *model_ids, const float *slos, const int32_t *m_id2g_id,
                            const float *group_max_latency, const float *group_sum_latency, int64_t num_requests,
                            int32_t M, int32_t G, double fixed_overhead,
                            int32_t *model_num_requests, int32_t *model_num_good_requests,
                            int32_t *group_num_requests, int32_t *group_num_good_requests) {
    if (!ctx) return fail(MMSIM_E_INVALID, "simulate_requests: null context");
    if (M < 1 || G < 1 || num_requests < 0) return fail(MMSIM_E_INVALID, "simulate_requests: bad size");
    if (!m_id2g_id || !group_max_latency || !group_sum_latency || !model_num_requests || !model_num_good_requests ||
        !group_num_requests || !group_num_good_requests ||
        (num_requests > 0 && (!finish || !good || !tstamps || !model_ids || !slos)))
        return fail(MMSIM_E_INVALID, "simulate_requests: null pointer");
    if (G > MMSIM_MAX_GROUPS) return fail(MMSIM_E_UNSUPPORTED, "simulate_requests: more than 254 groups");
    for (size_t i = 0; i < (size_t)M * G; ++i) {
        if (m_id2g_id[i] >= G) return fail(MMSIM_E_INVALID, "simulate_requests: m_id2g_id names a group >= G");
        if (group_max_latency[i] != group_max_latency[i] || group_sum_latency[i] != group_sum_latency[i] ||
            group_max_latency[i] < 0.0f || group_sum_latency[i] < 0.0f)
            return fail(MMSIM_E_INVALID, "simulate_requests: a latency is NaN or negative");
    }
    for (int64_t i = 0; i < num_requests; ++i) {
        if (tstamps[i] != tstamps[i]) return fail(MMSIM_E_INVALID, "simulate_requests: an arrival time is NaN");
        if (model_ids[i] >= M) return fail(MMSIM_E_INVALID, "simulate_requests: a request names a model >= M");
    }
    std::memset(model_num_requests, 0, sizeof(int32_t) * (size_t)M);
    std::memset(model_num_good_requests, 0, sizeof(int32_t) * (size_t)M);
    std::memset(group_num_requests, 0, sizeof(int32_t) * (size_t)G);
    std::memset(group_num_good_requests, 0, sizeof(int32_t) * (size_t)G);
    if (num_requests == 0) return MMSIM_OK;

    HIP_TRY(hipSetDevice(ctx->device));
    hipStream_t st = ctx->stream;
    const size_t R = (size_t)num_requests, MG = (size_t)M * G;
    DevBuf<double> d_t, d_fin;
    DevBuf<int32_t> d_m, d_m2g, d_cnt;
    DevBuf<float> d_slo, d_max, d_sum;
    DevBuf<uint8_t> d_good;
    HIP_TRY(d_t.alloc(R));
    HIP_TRY(d_fin.alloc(R));
    HIP_TRY(d_m.alloc(R));
    HIP_TRY(d_slo.alloc(R));
    HIP_TRY(d_good.alloc(R));
    HIP_TRY(d_m2g.alloc(MG));
    HIP_TRY(d_max.alloc(MG));
    HIP_TRY(d_sum.alloc(MG));
    HIP_TRY(d_cnt.alloc(2 * (size_t)M + 2 * (size_t)G));
    HIP_TRY(hipMemcpyAsync(d_t.p, tstamps, sizeof(double) * R, hipMemcpyHostToDevice, st));
    HIP_TRY(hipMemcpyAsync(d_m.p, model_ids, sizeof(int32_t) * R, hipMemcpyHostToDevice, st));
    HIP_TRY(hipMemcpyAsync(d_slo.p, slos, sizeof(float) * R, hipMemcpyHostToDevice, st));
    HIP_TRY(hipMemcpyAsync(d_m2g.p, m_id2g_id, sizeof(int32_t) * MG, hipMemcpyHostToDevice, st));
    HIP_TRY(hipMemcpyAsync(d_max.p, group_max_latency, sizeof(float) * MG, hipMemcpyHostToDevice, st));
    HIP_TRY(hipMemcpyAsync(d_sum.p, group_sum_latency, sizeof(float) * MG, hipMemcpyHostToDevice, st));
    HIP_TRY(hipMemsetAsync(d_cnt.p, 0, d_cnt.bytes(), st));
    ScalarArgs a{};
    a.tstamps = d_t.p;
    a.model_ids = d_m.p;
    a.slos = d_slo.p;
    a.m_id2g_id = d_m2g.p;
    a.group_max_latency = d_max.p;
    a.group_sum_latency = d_sum.p;
    a.R = num_requests;
    a.M = M;
    a.G = G;
    a.fixed_overhead = fixed_overhead;
    a.finish = d_fin.p;
    a.good = d_good.p;
    a.model_req = d_cnt.p;
    a.model_good = d_cnt.p + M;
    a.group_req = d_cnt.p + 2 * (size_t)M;
    a.group_good = d_cnt.p + 2 * (size_t)M + G;
    std::string err;
    if (launch_sim_scalar(a, st, &err) != hipSuccess) return fail(MMSIM_E_HIP, err);
    HIP_TRY(hipMemcpyAsync(finish, d_fin.p, sizeof(double) * R, hipMemcpyDeviceToHost, st));
    HIP_TRY(hipMemcpyAsync(good, d_good.p, R, hipMemcpyDeviceToHost, st));
    std::vector<int32_t> cnt(2 * (size_t)M + 2 * (size_t)G);
    HIP_TRY(hipMemcpyAsync(cnt.data(), d_cnt.p, d_cnt.bytes(), hipMemcpyDeviceToHost, st));
    HIP_TRY(hipStreamSynchronize(st));
    std::memcpy(model_num_requests, cnt.data(), sizeof(int32_t) * (size_t)M);
    std::memcpy(model_num_good_requests, cnt.data() + M, sizeof(int32_t) * (size_t)M);
    std::memcpy(group_num_requests, cnt.data() + 2 * (size_t)M, sizeof(int32_t) * (size_t)G);
    std::memcpy(group_num_good_requests, cnt.data() + 2 * (size_t)M + G, sizeof(int32_t) * (size_t)G);
    return MMSIM_OK;
}

int mmsim_simulate_requests_mixed_batching(mmsim_ctx *ctx, double *finish, uint8_t *good, const double *tstamps,
                                           const int32_t *model_ids, const float *slos, const int32_t *m_id2g_id,
                                           const int32_t *g_id2m_id, const int32_t *num_stages,
                                           const float *stage_latency, const int32_t *batch_sizes, int64_t num_requests,
                                           int32_t M, int32_t G, int32_t Smax, int32_t NB, double fixed_overhead,
                                           int32_t *model_num_requests, int32_t *model_num_good_requests,
                                           int32_t *group_num_requests, int32_t *group_num_good_requests) {
    if (!ctx) return fail(MMSIM_E_INVALID, "simulate_requests_mixed_batching: null context");
    if (M < 1 || G < 1 || Smax < 1 || NB < 1 || num_requests < 0)
        return fail(MMSIM_E_INVALID, "simulate_requests_mixed_batching: bad size");
    if (!m_id2g_id || !g_id2m_id || !num_stages || !stage_latency || !batch_sizes || !model_num_requests ||
        !model_num_good_requests || !group_num_requests || !group_num_good_requests ||
        (num_requests > 0 && (!finish || !good)))
        return fail(MMSIM_E_INVALID, "simulate_requests_mixed_batching: null pointer");
    if (G > MMSIM_MAX_GROUPS) return fail(MMSIM_E_UNSUPPORTED, "simulate_requests_mixed_batching: more than 254 groups");
    mmsim_tables t{};
    t.M = M;
    t.C = G;  // every group is its own latency-table column
    t.Smax = Smax;
    t.NB = NB;
    t.cfg_lat = stage_latency;
    t.cfg_pp = num_stages;
    t.batch_sizes = batch_sizes;
    t.fixed_overhead = fixed_overhead;
    int rc = check_tables(&t);
    if (rc) return rc;
    RepLists rl;
    rl.B = 1;
    rl.M = M;
    rl.Gmax = G;
    rl.num_groups.assign(1, G);
    rl.group_cfg.resize(G);
    for (int g = 0; g < G; ++g) rl.group_cfg[g] = g;
    rl.off.assign((size_t)M + 1, 0);
    for (int32_t m = 0; m < M; ++m)
        for (int32_t j = 0; j < G; ++j) {
            const int32_t g = m_id2g_id[(size_t)m * G + j];
            if (g < 0) break;
            if (g >= G) return fail(MMSIM_E_INVALID, "simulate_requests_mixed_batching: m_id2g_id names a group >= G");
            rl.grp.push_back(g);
            rl.off[m + 1] += 1;
        }
    for (int32_t m = 0; m < M; ++m) rl.off[m + 1] += rl.off[m];
    rl.g2m_off.assign((size_t)G + 1, 0);
    for (int32_t g = 0; g < G; ++g) {
        for (int32_t j = 0; j < M; ++j) {
            const int32_t m = g_id2m_id[(size_t)g * M + j];
            if (m < 0) break;
            if (m >= M) return fail(MMSIM_E_INVALID, "simulate_requests_mixed_batching: g_id2m_id names a model >= M");
            rl.g2m_m.push_back(m);
        }
        rl.g2m_off[g + 1] = (int64_t)rl.g2m_m.size();
    }

    mmsim_workload *wl = nullptr;
    rc = mmsim_workload_create(ctx, num_requests, M, tstamps, model_ids, slos, &wl);
    if (rc) return rc;
    const mmsim_workload *wls[1] = {wl};
    const uint32_t flags = MMSIM_BATCHING | MMSIM_WANT_MODEL_COUNTS | MMSIM_WANT_GROUP_COUNTS | MMSIM_WANT_PER_REQUEST;
    // (a simulation that runs out of idle-event slots is run again with twice as many, as in mmsim_eval_batch)
    mmsim_options o = ctx->opt;
    for (int attempt = 0; attempt < 8; ++attempt) {
        mmsim_batch *b = nullptr;
        rc = build_batch(ctx, wls, 1, &t, rl, flags, &b, nullptr, &o);
        if (rc == MMSIM_OK) o.batching_event_slots = 2 * b->bargs.heap_cap;
        if (rc == MMSIM_OK) rc = mmsim_batch_run(b);
        if (rc == MMSIM_OK) rc = mmsim_batch_sync(b, nullptr);
        if (rc == MMSIM_OK) {
            int64_t ng = 0;
            double ls = 0.0;
            mmsim_result r{};
            r.n_good = &ng;
            r.latency_sum = &ls;
            r.model_num_requests = model_num_requests;
            r.model_num_good = model_num_good_requests;
            r.group_num_requests = group_num_requests;
            r.group_num_good = group_num_good_requests;
            r.finish = finish;
            r.good = good;
            rc = mmsim_batch_fetch(b, &r);
        }
        mmsim_batch_destroy(b);
        if (rc != MMSIM_E_OVERFLOW) break;
    }
    mmsim_workload_destroy(wl);
    return rc;
}

}  // extern "C"
