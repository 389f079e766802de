/*
 * libmmsim -- MI355X (gfx950) evaluation of candidate model placements with
 * AlpaServe's approximate serving simulator.
 *
 * Plain C ABI: opaque handles, plain pointers and sizes, integer status codes.
 * Every entry point returns MMSIM_OK (0) or a negative MMSIM_E_* code; a
 * human-readable message for the last failure on the calling thread is
 * available from mmsim_last_error().  No entry point retains a host pointer
 * after it returns.  A context and the objects made from it must be used by
 * one thread at a time.  There is no CPU fallback: without a usable HIP
 * device mmsim_ctx_create fails.
 *
 * What each entry point stands in for in the reference (alpa-projects/mms):
 *
 *   mmsim_simulate_requests_mixed
 *       the numba kernel simulate_requests_mixed, same argument list
 *       (alpa_serve/simulator/controller.py:561-628; called at :491-494).
 *   mmsim_simulate_requests_mixed_batching
 *       simulate_requests_mixed_batching, same argument list
 *       (alpa_serve/simulator/controller.py:631-798; called at :486-489).
 *   mmsim_simulate_requests
 *       the numba kernel simulate_requests (one clock per group), same
 *       argument list (alpa_serve/simulator/controller.py:506-558; called at
 *       :496-499 when mixed is False, which no caller of the reference passes).
 *   mmsim_workload_create
 *       the per-workload arrays approximate_one_case derives once and caches:
 *       arrivals, model_ids (int32) and slos (float32)
 *       (alpa_serve/simulator/controller.py:321-339).
 *   mmsim_batch_create / _run / _sync / _fetch, mmsim_eval_batch
 *       the loop "for sol in sols: approximate_one_case(...)" of
 *       PlacementEvaluator.get_scores / get_stats
 *       (alpa_serve/placement_policy/base_policy.py:175-189, 191-264), i.e.
 *       approximate_one_case_one_placement's table build
 *       (controller.py:412-476) plus the request loop for every placement
 *       of the list, and the reductions of the fast-stats epilogue
 *       (controller.py:393-403: number of good requests, sum of latencies).
 */
#ifndef MMSIM_H_
#define MMSIM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MMSIM_ABI_VERSION 1

enum {
    MMSIM_OK = 0,
    MMSIM_E_INVALID = -1,     /* bad argument (null pointer, negative size, index out of range) */
    MMSIM_E_UNSUPPORTED = -2, /* shape outside the compiled kernel buckets                      */
    MMSIM_E_HIP = -3,         /* a HIP runtime call failed                                      */
    MMSIM_E_NOMEM = -4,       /* host or device allocation failed                               */
    MMSIM_E_OVERFLOW = -5     /* a lane ran out of idle-event slots (batching); see status[]    */
};

/* Limits of the compiled kernels. */
#define MMSIM_MAX_STAGES 32        /* pipeline stages of one group                */
#define MMSIM_MAX_REPLICAS 64      /* groups hosting one model in one placement   */
#define MMSIM_MAX_GROUPS 254       /* groups of one placement                     */
#define MMSIM_MAX_SLOTS 255        /* sum of pipeline stages over a placement     */
#define MMSIM_MAX_CONFIGS 255      /* distinct parallel configurations            */
#define MMSIM_MAX_BATCH_SIZES 16   /* batch sizes (batching simulator)            */

typedef struct mmsim_ctx mmsim_ctx;
typedef struct mmsim_workload mmsim_workload;
typedef struct mmsim_batch mmsim_batch;

int mmsim_abi_version(void);
const char *mmsim_last_error(void);

/* Binds a context to HIP device `device` and creates its stream. */
int mmsim_ctx_create(int device, mmsim_ctx **out);
void mmsim_ctx_destroy(mmsim_ctx *ctx);

/*
 * Tuning options of the launch plan.  The reference keeps its simulator knobs
 * as module constants (alpa_serve/simulator/controller.py:432, 517, 575, 644;
 * alpa_serve/util.py:11-13); here they are explicit, defaulted parameters.
 * Fill the struct with mmsim_options_default() and change what is needed:
 * -1 (switches) or 0 (numbers) means "let the library decide".  No option
 * changes a result; they move work between kernels, wavefronts and memories,
 * and exist for measurements and for tests that must reach every code path.
 */
typedef struct {
    int32_t struct_size;          /* sizeof(mmsim_options), set by mmsim_options_default                      */
    int32_t request_loop;         /* plain simulator: 1 = loop over runs of equal models (scheduled launch),
                                     0 = chunks of four requests; -1: runs when at least four in five requests
                                     of the batch's streams repeat the model of the request before.  A latency
                                     table with one latency per (model, configuration) and more than 63
                                     configurations takes the chunks whatever this says                        */
    int32_t waves_per_cu;         /* 1..8: most wavefronts per workgroup of the plain simulator; 0: as many as fit */
    int32_t counts_in_lds;        /* counts of the plain simulator: 1 = counters in LDS, 0 = in registers and
                                     global rows; -1: LDS when that does not cost a CU wavefronts              */
    int32_t tile_order_by_slots;  /* loop over runs: 0 = tiles composed by pipeline depth only; -1 / 1: by clock
                                     slots as well                                                              */
    int32_t sched_groups;         /* workgroups of the scheduled launch; 0: one per CU                          */
    int32_t segment_requests;     /* requests per turn of an item in the scheduled launch; 0: 16384             */
    int32_t sched_spin_limit;     /* looks in a row after which a wavefront that finds only busy items leaves;
                                     -1: 20000                                                                  */
    int32_t skip_ahead;           /* loop over runs: 0 = simulate every request; -1 / 1: requests that every lane
                                     of a wavefront must reject are not simulated                              */
    int32_t xcd_map;              /* chunked loop: 0 = seeds innermost in the workgroup numbering; -1 / 1: all
                                     seeds of a tile group on one XCD                                           */
    int32_t batching_lanes;       /* batching simulator: 8, 16, 32 or 64 simulations per wavefront; 0: the widest
                                     that still gives a CU eight wavefronts                                    */
    int32_t batching_event_slots; /* batching simulator: idle-event slots per simulation (a multiple of eight);
                                     0: from the group count.  Too few makes a simulation stop with
                                     MMSIM_E_OVERFLOW (the one-call entry points then try again with more)     */
    int32_t batching_lds_tables;  /* batching simulator: bit 0 latency table, bit 1 models of each group may be
                                     copied to LDS; -1: both, subject to fit                                    */
    int32_t reserved;
    int64_t stats_scratch_bytes;  /* scratch of one launch of mmsim_batch_model_stats; 0: 1 GiB                 */
} mmsim_options;
void mmsim_options_default(mmsim_options *options);
/* Options for every batch the context makes from now on without options of its own (mmsim_batch_create,
 * mmsim_eval_batch, mmsim_eval_pairs, mmsim_eval_batch_static, the single-placement calls); NULL restores the
 * defaults. */
int mmsim_ctx_set_options(mmsim_ctx *ctx, const mmsim_options *options);

typedef struct {
    char name[128];
    char arch[64];
    int32_t compute_units;
    int32_t clock_khz;
    int32_t lds_bytes_per_block;
    int64_t hbm_bytes;
} mmsim_device_info;
int mmsim_ctx_device_info(mmsim_ctx *ctx, mmsim_device_info *out);

/*
 * One request stream (one arrival seed), copied to device memory.
 *   tstamps   [R] arrival times in the order the requests are to be processed
 *   model_ids [R] model index in [0, M) or negative for "not registered"
 *   slos      [R] float32 seconds; +inf = never dropped, NaN = always dropped
 * Streams are generated on the host by design: the reference draws them from
 * numpy's legacy Mersenne-Twister / rejection-sampled gamma stream
 * (alpa_serve/simulator/workload.py:135-155), which is sequential per model
 * and goes through the host's libm; a device generator could not reproduce
 * those arrivals bit for bit, and a stream is made once per search.
 */
int mmsim_workload_create(mmsim_ctx *ctx, int64_t R, int32_t M,
                          const double *tstamps, const int32_t *model_ids,
                          const float *slos, mmsim_workload **out);
void mmsim_workload_destroy(mmsim_workload *wl);

/*
 * Latency table shared by all placements of a batch: what
 * approximate_one_case_one_placement computes per (model, group) depends only
 * on the group's parallel configuration, so it is given once per distinct
 * configuration.
 *   cfg_lat [M][C][Smax][NB]  float32( stage latency * (1 + 0.009*pp) ), or
 *                             +inf for a configuration the model has no
 *                             profile for; entries k >= cfg_pp[c] are ignored
 *   cfg_pp  [C]               pipeline stages of configuration c (1..Smax)
 *   batch_sizes [NB]          batch sizes, batch_sizes[0] == 1; only column 0
 *                             is used without MMSIM_BATCHING
 */
typedef struct {
    int32_t M, C, Smax, NB;
    const float *cfg_lat;
    const int32_t *cfg_pp;
    const int32_t *batch_sizes;
    double fixed_overhead; /* 0.011 in the reference */
} mmsim_tables;

/*
 * B candidate placements.  Placement b has num_groups[b] groups; group g uses
 * configuration group_cfg[b*Gmax+g] and hosts the models
 *   gm_idx[ gm_off[b*(Gmax+1)+g] .. gm_off[b*(Gmax+1)+g+1] )
 * in the order given (the order of ModelPlacement.group_models[g]).
 */
typedef struct {
    int32_t B, Gmax;
    const int32_t *num_groups;
    const int32_t *group_cfg;
    const int64_t *gm_off;
    const int32_t *gm_idx;
} mmsim_placements;

/* flags */
#define MMSIM_BATCHING 1u          /* batching simulator instead of the plain one */
#define MMSIM_WANT_MODEL_COUNTS 2u /* fill model_num_requests / model_num_good     */
#define MMSIM_WANT_GROUP_COUNTS 4u /* fill group_num_requests / group_num_good     */
#define MMSIM_WANT_PER_REQUEST 8u  /* fill finish / good for every request         */
#define MMSIM_WANT_OP_COUNT 16u    /* fill fp_ops (plain simulator only)            */

/*
 * Results, caller-allocated.  Simulation ("lane") l = seed * B + b.
 * Pointers not asked for by the flags may be null.
 */
typedef struct {
    int64_t *n_good;             /* [L]        accepted requests                                    */
    double *latency_sum;         /* [L]        sum of (finish - arrival) over requests in arrival order */
    int32_t *model_num_requests; /* [L][M]     */
    int32_t *model_num_good;     /* [L][M]     */
    int32_t *group_num_requests; /* [L][Gmax]  */
    int32_t *group_num_good;     /* [L][Gmax]  */
    double *finish;              /* [L][Rmax]  Rmax = longest stream of the batch; row tail unspecified */
    uint8_t *good;               /* [L][Rmax]  both may be NULL: the per-request outputs then stay on the
                                               device (mmsim_batch_model_stats reads them there) */
    int32_t *status;             /* [L]        0, or MMSIM_E_OVERFLOW for a lane whose results are invalid */
    int64_t *fp_ops;             /* [L]        sum over dispatched requests of 2*stages + replicas + 3:
                                               the fp64 max/add/compare operations the reference's loop
                                               performs (controller.py:590-613) */
} mmsim_result;

/* Packs the placements, uploads them and allocates device result buffers.  The
 * batch copies what it needs of the workloads for mmsim_batch_run / _fetch:
 * they may be destroyed before it (mmsim_batch_model_stats is the exception,
 * see there). */
int mmsim_batch_create(mmsim_ctx *ctx, const mmsim_workload *const *workloads, int32_t n_seeds,
                       const mmsim_tables *tables, const mmsim_placements *placements,
                       uint32_t flags, mmsim_batch **out);
/* The same with options for this batch only (NULL: the context's). */
int mmsim_batch_create_ex(mmsim_ctx *ctx, const mmsim_workload *const *workloads, int32_t n_seeds,
                          const mmsim_tables *tables, const mmsim_placements *placements,
                          uint32_t flags, const mmsim_options *options, mmsim_batch **out);
/* Enqueues the simulation kernels on the context's stream (asynchronous). */
int mmsim_batch_run(mmsim_batch *batch);
/* Waits for the last run.  kernel_ms (optional) receives the time between HIP
 * events recorded on the stream right before and after the simulation kernel. */
int mmsim_batch_sync(mmsim_batch *batch, float *kernel_ms);
/* Copies results of the last completed run into caller memory. */
int mmsim_batch_fetch(mmsim_batch *batch, mmsim_result *out);

/* Serving statistics per (simulation, model), computed on the device from the
 * per-request outputs of the last run, which stay there: what
 * Workload.compute_stats (alpa_serve/simulator/workload.py:308-354) derives
 * from start / finish / good, start being the arrival times.  All arrays are
 * [L][M], L as in mmsim_result; all are required.
 *
 * Only requests skip[s] <= i < R_s - skip[s] of stream s count (the caller
 * computes skip as workload.py:313 does: int(warmup / (last - first arrival) *
 * R); 0 keeps every request).  Of the accepted requests of a model inside that
 * window: their number, the arrival times of the first and the last one
 * (throughput = number / (last - first), :337), the sum, mean and standard
 * deviation of their latencies finish - arrival (np.mean / np.std, :349) and
 * the order statistics sorted[int(0.90 * n)], sorted[int(0.99 * n)] (:344-346).
 * A model none of whose requests was accepted reports 0 for all of them, as
 * the reference's latency = [0] does (:340-342).
 *
 * Counts, times and the two percentiles are exact.  Sum, mean and deviation
 * are compensated sums: sum and mean within 1e-14 relative of the exact value,
 * hence within 1e-12 of numpy's pairwise sums, but not bit-equal to them; a
 * deviation far below the mean (nearly equal latencies) is exact to 1e-12 of
 * the mean, not of itself -- in numpy as well.
 *
 * The batch must have been created with MMSIM_WANT_PER_REQUEST and run;
 * `workloads` are the n_streams workload objects it was created with, in the
 * same order and not destroyed in between (their per-model request lists are
 * read; the batch keeps no copy of them, and it checks that these are the
 * objects it was made from: any other stream, even one of the same length, is
 * refused with MMSIM_E_INVALID).  Call mmsim_batch_fetch as well to learn of
 * simulations that failed. */
typedef struct {
    int32_t *model_num_requests; /* requests of the model inside the window     */
    int32_t *model_num_good;     /* accepted ones among them                     */
    double *first_start;         /* arrival of the first accepted request        */
    double *last_start;          /* arrival of the last accepted request         */
    double *latency_sum;
    double *latency_mean;
    double *latency_std;
    double *latency_p90;
    double *latency_p99;
} mmsim_model_stats;
int mmsim_batch_model_stats(mmsim_batch *batch, const mmsim_workload *const *workloads, int32_t n_streams,
                            const int64_t *skip, mmsim_model_stats *out);
void mmsim_batch_destroy(mmsim_batch *batch);

/*
 * Like mmsim_eval_batch, but placement b is simulated on workloads[stream_of[b]]
 * only: B simulations, results laid out [B][...] (finish / good rows are Rmax
 * long, Rmax the longest of the streams).  This is the loop over the segments
 * of a ModelPlacementWithReplacement in approximate_one_case
 * (alpa_serve/simulator/controller.py:345-391): every (start time, placement)
 * pair is simulated on its own slice of the arrivals from idle clocks; here all
 * segments of all candidates are lanes of one launch.
 */
int mmsim_eval_pairs(mmsim_ctx *ctx, const mmsim_workload *const *workloads, int32_t n_streams,
                     const mmsim_tables *tables, const mmsim_placements *placements,
                     const int32_t *stream_of, uint32_t flags, mmsim_result *out);

/*
 * mmsim_eval_batch for candidates given as "a placement plus one more replica":
 * what the searches of the reference build one Python object at a time with
 * sol.add_model(group, model).normalize() before they score the list
 * (alpa_serve/placement_policy/base_policy.py:392, :453-458; ModelPlacement.add_model
 * / normalize :24-35).  The batch holds the B base placements followed by the
 * n successors; successor k is base placement parent[k] with model[k] appended
 * to its group group[k].  With normalize != 0 the successor is then brought
 * into the form ModelPlacement.normalize() gives: the models of every group in
 * ascending order, the groups in the stable order of their model tuples (a
 * tuple that is a prefix of another comes first), every group keeping its
 * configuration.  The order of the groups decides which replica wins a clock
 * tie, so it is part of the result; the per-group counts of a successor are in
 * that order.  Results are laid out as for mmsim_eval_batch with B + n
 * placements: simulation l = seed * (B + n) + index, index < B for a base
 * placement and B + k for successor k.
 */
typedef struct {
    int32_t n;
    const int32_t *parent; /* [n] index of the base placement          */
    const int32_t *group;  /* [n] group of the parent that gets a replica */
    const int32_t *model;  /* [n] the model replicated                  */
    int32_t normalize;
} mmsim_successors;
int mmsim_eval_successors(mmsim_ctx *ctx, const mmsim_workload *const *workloads, int32_t n_seeds,
                          const mmsim_tables *tables, const mmsim_placements *base,
                          const mmsim_successors *successors, uint32_t flags, mmsim_result *out);

/*
 * mmsim_eval_batch without any device allocation or free.  It has no
 * counterpart in the reference; it is for callers that cannot allocate device
 * memory: tight search or serving loops, harnesses that forbid hipMalloc.
 * The call is synchronous and runs on the context's own stream (it copies,
 * clears and waits like mmsim_eval_batch, so it cannot itself be recorded
 * into a HIP graph).  Same arguments, results and error codes as
 * mmsim_eval_batch, bit for bit, but every device table and result buffer of
 * the batch lives in a static device array of MMSIM_STATIC_SCRATCH_BYTES that
 * the library holds on each GPU it runs on until the process ends: no
 * hipMalloc, no hipFree.  A batch that needs more (many placements x models,
 * several long streams, per-request outputs) is refused with MMSIM_E_NOMEM
 * and a message that names the limit.  All calls on one GPU share that GPU's
 * array: calls that overlap on one GPU race, from whichever contexts or
 * threads they come.  The workloads are inputs and stay the caller's.
 */
#define MMSIM_STATIC_SCRATCH_BYTES (32u << 20)
int mmsim_eval_batch_static(mmsim_ctx *ctx, const mmsim_workload *const *workloads, int32_t n_seeds,
                            const mmsim_tables *tables, const mmsim_placements *placements,
                            uint32_t flags, mmsim_result *out);

typedef struct {
    int32_t lanes, waves, n_seeds, B;
    int32_t smax_bucket, max_replicas, slots, lds_bytes;
    int64_t requests_total;   /* sum of stream lengths over seeds                     */
    int64_t table_bytes;      /* device bytes of the packed placement tables          */
    int64_t stream_bytes;     /* device bytes of the request streams                  */
    int32_t workgroups;       /* scheduled launch (bursty streams): workgroups, each owning a set of
                                 (64 placements, stream) items; 0 for the other launches            */
    int32_t segments;         /* pieces a stream is cut into so that a workgroup's items take turns  */
    int32_t launches;         /* kernel launches of one mmsim_batch_run                             */
    int32_t waves_per_group;  /* wavefronts of a workgroup that simulate side by side               */
    int32_t event_slots;      /* batching simulator: idle-event slots per simulation; 0 otherwise   */
    int32_t reserved;
} mmsim_batch_info;
int mmsim_batch_get_info(const mmsim_batch *batch, mmsim_batch_info *out);
/* Name of the kernel template instance mmsim_batch_run launches for this batch, as a profiler prints it
 * (e.g. "sim_mixed_kernel<16, true, true, true, 0, true>"); measurement aid, no counterpart in the reference. */
int mmsim_batch_kernel_name(const mmsim_batch *batch, char *buf, size_t size);

/* create + run + sync + fetch + destroy.  With MMSIM_BATCHING, a simulation that runs out of idle-event slots
 * (status MMSIM_E_OVERFLOW: the reference's heap of idle events has no bound, the kernel's list of them has) is
 * simulated again inside this call with twice the slots, until it fits or LDS cannot hold more; only then does it
 * keep that status.  mmsim_eval_pairs, mmsim_eval_successors and mmsim_simulate_requests_mixed_batching do the
 * same; a batch (mmsim_batch_fetch) reports the status and leaves the choice to the caller
 * (mmsim_options.batching_event_slots). */
int mmsim_eval_batch(mmsim_ctx *ctx, const mmsim_workload *const *workloads, int32_t n_seeds,
                     const mmsim_tables *tables, const mmsim_placements *placements,
                     uint32_t flags, mmsim_result *out);

/*
 * Single-placement calls with the argument lists of the reference's kernels.
 * finish [R] and good [R] are written for every request; the four count
 * arrays are zeroed and filled.  Layouts:
 *   m_id2g_id     [M][G]  replica groups of each model, -1 terminated
 *   g_id2m_id     [G][M]  models of each group, -1 terminated (batching only)
 *   num_stages    [G]
 *   stage_latency [M][G][Smax]        (plain)   float32
 *                 [M][G][Smax][NB]    (batching)
 */
int mmsim_simulate_requests_mixed(
    mmsim_ctx *ctx, double *finish, uint8_t *good, const double *tstamps,
    const int32_t *model_ids, const float *slos, const int32_t *m_id2g_id,
    const int32_t *num_stages, const float *stage_latency, int64_t num_requests,
    int32_t M, int32_t G, int32_t Smax, double fixed_overhead,
    int32_t *model_num_requests, int32_t *model_num_good_requests,
    int32_t *group_num_requests, int32_t *group_num_good_requests);

/* group_max_latency, group_sum_latency: [M][G] float32 (controller.py:433-443) */
int mmsim_simulate_requests(
    mmsim_ctx *ctx, double *finish, uint8_t *good, const double *tstamps,
    const int32_t *model_ids, const float *slos, const int32_t *m_id2g_id,
    const float *group_max_latency, const float *group_sum_latency, int64_t num_requests,
    int32_t M, int32_t G, double fixed_overhead,
    int32_t *model_num_requests, int32_t *model_num_good_requests,
    int32_t *group_num_requests, int32_t *group_num_good_requests);

int mmsim_simulate_requests_mixed_batching(
    mmsim_ctx *ctx, double *finish, uint8_t *good, const double *tstamps,
    const int32_t *model_ids, const float *slos, const int32_t *m_id2g_id,
    const int32_t *g_id2m_id, const int32_t *num_stages, const float *stage_latency,
    const int32_t *batch_sizes, int64_t num_requests,
    int32_t M, int32_t G, int32_t Smax, int32_t NB, double fixed_overhead,
    int32_t *model_num_requests, int32_t *model_num_good_requests,
    int32_t *group_num_requests, int32_t *group_num_good_requests);

#ifdef __cplusplus
}
#endif
#endif /* MMSIM_H_ */
