/*
 * CPU ORACLE -- test infrastructure, not product code.
 *
 * Plain-C restatement of the request loops of AlpaServe's approximate serving
 * simulator.  Only the tests, the smoke check and the benchmark's CPU-baseline
 * leg may build, load or call this file; the shipped library never does.
 *
 * Functions and the reference code each one follows:
 *   oracle_simulate_requests_mixed           alpa_serve/simulator/controller.py:561-628
 *   oracle_simulate_requests                 alpa_serve/simulator/controller.py:506-558
 *   oracle_simulate_requests_mixed_batching  alpa_serve/simulator/controller.py:631-798
 *   oracle_build_stage_latency               alpa_serve/simulator/controller.py:412-476 (table layout only;
 *                                            the fp64 product and fp32 rounding are done by the caller)
 *   oracle_eval_placements                   loop of PlacementEvaluator.get_scores,
 *                                            alpa_serve/placement_policy/base_policy.py:175-189
 *
 * Arithmetic: fp64 add / max / sub / compare on operands that are fp64
 * (arrival times, clocks) or fp32 promoted to fp64 (SLOs, stage latencies),
 * in the reference's operation order.  Build with -ffp-contract=off.
 *
 * Pinning status:
 *   simulate_requests_mixed, simulate_requests: pinned by closed forms, a
 *     hand-derived worked example, an independent Lindley recursion and an
 *     independently written Python restatement (tests/test_oracle_*.py).
 *   simulate_requests_mixed_batching: pinned by golden vectors written by the
 *     reference's own function (tests/golden/) plus the Python restatement.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_INF 1e100 /* alpa_serve/util.py:23 */

static inline double dmax(double a, double b) { return b > a ? b : a; }

/* ------------------------------------------------------------------------- */
/* controller.py:561-628                                                      */
int oracle_simulate_requests_mixed(
    double *finish, uint8_t *good, const double *tstamps,
    const int32_t *model_ids, const float *slos,
    const int32_t *m_id2g_id,     /* [M][G], -1 padded                      */
    const int32_t *num_stages,    /* [G]                                    */
    const float *stage_latency,   /* [M][G][Smax]                           */
    int64_t num_requests, int32_t M, int32_t G, int32_t Smax,
    double fixed_overhead,
    int32_t *model_num_requests, int32_t *model_num_good_requests, /* [M]   */
    int32_t *group_num_requests, int32_t *group_num_good_requests, /* [G]   */
    int64_t *fp_ops /* optional: adds 2*S_g + r_m + 3 per dispatched request */)
{
    double *clocks = (double *)calloc((size_t)(G > 0 ? G : 1) * (size_t)(Smax > 0 ? Smax : 1), sizeof(double));
    double *tmp = (double *)calloc((size_t)(Smax > 0 ? Smax : 1), sizeof(double));
    if (!clocks || !tmp) { free(clocks); free(tmp); return -1; }
    memset(model_num_requests, 0, sizeof(int32_t) * (size_t)M);
    memset(model_num_good_requests, 0, sizeof(int32_t) * (size_t)M);
    memset(group_num_requests, 0, sizeof(int32_t) * (size_t)G);
    memset(group_num_good_requests, 0, sizeof(int32_t) * (size_t)G);
    int64_t ops = 0;

    for (int64_t i = 0; i < num_requests; ++i) {
        const double tstamp = tstamps[i];
        const int32_t m = model_ids[i];
        const double slo = (double)slos[i];

        if (m < 0) { finish[i] = tstamp; good[i] = 0; continue; }       /* :582-585 */
        model_num_requests[m] += 1;                                     /* :587 */

        int32_t g = -1;                                                 /* :590-598 */
        double best = ORACLE_INF;
        int32_t r_m = 0;
        for (int32_t j = 0; j < G; ++j) {
            const int32_t cand = m_id2g_id[(size_t)m * G + j];
            if (cand < 0) break;
            ++r_m;
            const double c = clocks[(size_t)cand * Smax + (num_stages[cand] - 1)];
            if (c < best) { best = c; g = cand; }
        }
        if (g < 0) { finish[i] = tstamp; good[i] = 0; continue; }       /* :600-603 */

        const int32_t S = num_stages[g];
        const float *lat = stage_latency + ((size_t)m * G + g) * Smax;
        double *clk = clocks + (size_t)g * Smax;
        double t = tstamp;                                              /* :605-608 */
        for (int32_t k = 0; k < S; ++k) {
            t = dmax(t, clk[k]) + (double)lat[k];
            tmp[k] = t;
        }
        const double finish_time = t + fixed_overhead;                  /* :610 */
        group_num_requests[g] += 1;                                     /* :611 */
        ops += 2 * (int64_t)S + r_m + 3;

        if (finish_time - tstamp <= slo) {                              /* :613-619 */
            finish[i] = finish_time;
            good[i] = 1;
            for (int32_t k = 0; k < S; ++k) clk[k] = tmp[k];
            group_num_good_requests[g] += 1;
            model_num_good_requests[m] += 1;
        } else {                                                        /* :620-622 */
            finish[i] = tstamp;
            good[i] = 0;
        }
    }
    if (fp_ops) *fp_ops += ops;
    free(clocks);
    free(tmp);
    return 0;
}

/* ------------------------------------------------------------------------- */
/* controller.py:506-558 (one scalar clock per group; mixed=False)            */
int oracle_simulate_requests(
    double *finish, uint8_t *good, const double *tstamps,
    const int32_t *model_ids, const float *slos,
    const int32_t *m_id2g_id,          /* [M][G]                             */
    const float *group_max_latency,    /* [M][G]                             */
    const float *group_sum_latency,    /* [M][G]                             */
    int64_t num_requests, int32_t M, int32_t G, double fixed_overhead,
    int32_t *model_num_requests, int32_t *model_num_good_requests,
    int32_t *group_num_requests, int32_t *group_num_good_requests)
{
    double *clocks = (double *)calloc((size_t)(G > 0 ? G : 1), sizeof(double));
    if (!clocks) return -1;
    memset(model_num_requests, 0, sizeof(int32_t) * (size_t)M);
    memset(model_num_good_requests, 0, sizeof(int32_t) * (size_t)M);
    memset(group_num_requests, 0, sizeof(int32_t) * (size_t)G);
    memset(group_num_good_requests, 0, sizeof(int32_t) * (size_t)G);

    for (int64_t i = 0; i < num_requests; ++i) {
        const double tstamp = tstamps[i];
        const int32_t m = model_ids[i];
        const double slo = (double)slos[i];
        if (m < 0) { finish[i] = tstamp; good[i] = 0; continue; }
        model_num_requests[m] += 1;

        int32_t g = -1;
        double best = ORACLE_INF;
        for (int32_t j = 0; j < G; ++j) {
            const int32_t cand = m_id2g_id[(size_t)m * G + j];
            if (cand < 0) break;
            if (clocks[cand] < best) { best = clocks[cand]; g = cand; }
        }
        if (g < 0) { finish[i] = tstamp; good[i] = 0; continue; }

        const double start_time = dmax(clocks[g], tstamp);                /* :543 */
        const double finish_time =                                         /* :544 */
            start_time + (double)group_sum_latency[(size_t)m * G + g] + fixed_overhead;
        group_num_requests[g] += 1;
        if (finish_time - tstamp <= slo) {
            finish[i] = finish_time;
            good[i] = 1;
            clocks[g] = start_time + (double)group_max_latency[(size_t)m * G + g]; /* :550 */
            group_num_good_requests[g] += 1;
            model_num_good_requests[m] += 1;
        } else {
            finish[i] = tstamp;
            good[i] = 0;
        }
    }
    free(clocks);
    return 0;
}

/* ------------------------------------------------------------------------- */
/* controller.py:631-798 -- batching variant                                  */

typedef struct { double t; int32_t g; } idle_ev;

typedef struct {
    idle_ev *a;
    int64_t n, cap;
    int64_t max_n;
} ev_heap;

static inline int ev_less(idle_ev x, idle_ev y)
{   /* Python tuple order on (time, group) */
    return x.t < y.t || (x.t == y.t && x.g < y.g);
}

static int heap_push(ev_heap *h, idle_ev e)
{
    if (h->n == h->cap) {
        int64_t nc = h->cap ? h->cap * 2 : 64;
        idle_ev *na = (idle_ev *)realloc(h->a, sizeof(idle_ev) * (size_t)nc);
        if (!na) return -1;
        h->a = na; h->cap = nc;
    }
    int64_t i = h->n++;
    while (i > 0) {
        int64_t p = (i - 1) / 2;
        if (!ev_less(e, h->a[p])) break;
        h->a[i] = h->a[p];
        i = p;
    }
    h->a[i] = e;
    if (h->n > h->max_n) h->max_n = h->n;
    return 0;
}

static idle_ev heap_pop(ev_heap *h)
{
    idle_ev top = h->a[0];
    idle_ev last = h->a[--h->n];
    int64_t i = 0;
    for (;;) {
        int64_t c = 2 * i + 1;
        if (c >= h->n) break;
        if (c + 1 < h->n && ev_less(h->a[c + 1], h->a[c])) ++c;
        if (!ev_less(h->a[c], last)) break;
        h->a[i] = h->a[c];
        i = c;
    }
    if (h->n > 0) h->a[i] = last;
    return top;
}

typedef struct {
    /* inputs */
    double *finish; uint8_t *good;
    const double *tstamps; const float *slos;
    const int32_t *g_id2m_id; const int32_t *num_stages; const float *stage_latency;
    const int32_t *batch_sizes;
    int32_t M, G, Smax, NB;
    double fixed_overhead;
    /* state */
    double *clocks;            /* [G][Smax] */
    double *tmp;               /* [Smax]    */
    /* queue of model m = order[m][head[m] .. tail[m]) : request indices in arrival order */
    int64_t *order; int64_t *qbase; int64_t *head; int64_t *tail;
    ev_heap heap;
    int32_t *model_num_good_requests, *group_num_requests, *group_num_good_requests;
    int err;
    int64_t ops;   /* fp64 operations of check_slo calls, deadlines and commits (measurement only) */
} bsim;

static inline int64_t qlen(const bsim *s, int32_t m) { return s->tail[m] - s->head[m]; }
static inline int64_t qfront(const bsim *s, int32_t m) { return s->order[s->qbase[m] + s->head[m]]; }

static inline int ilog2_i32(int32_t v) { int r = 0; while (v > 1) { v >>= 1; ++r; } return r; }

/* :654-664 */
static int32_t b_select_model(const bsim *s, int32_t g)
{
    double min_arrival = ORACLE_INF;
    int32_t sel = -1;
    for (int32_t j = 0; j < s->M; ++j) {
        const int32_t m = s->g_id2m_id[(size_t)g * s->M + j];
        if (m < 0) break;
        if (qlen(s, m) > 0) {
            const double a = s->tstamps[qfront(s, m)];
            if (a < min_arrival) { min_arrival = a; sel = m; }
        }
    }
    return sel;
}

/* :666-672 ; lat points at stage_latency[m][g][0][b], stride NB between stages */
static int b_check_slo(const bsim *s, double tstamp, int32_t g, const float *lat, double deadline)
{
    double t = tstamp;
    const double *clk = s->clocks + (size_t)g * s->Smax;
    for (int32_t k = 0; k < s->num_stages[g]; ++k)
        t = dmax(clk[k], t) + (double)lat[(size_t)k * s->NB];
    return (t + s->fixed_overhead) <= deadline;
}

/* :706-732 with :674-704 inlined; recursion of the reference written as a loop */
static void b_handle(bsim *s, double tstamp, int32_t m, int32_t g)
{
    for (;;) {
        const float *lat_mg = s->stage_latency + (((size_t)m * s->G + g) * s->Smax) * s->NB;
        /* get_max_batch_under_slo :674-704 */
        int found = 0;
        int64_t first = -1;
        while (qlen(s, m) > 0) {
            const int64_t r = qfront(s, m);
            s->head[m] += 1;                                              /* pop(0) :678 */
            s->ops += 2 * (int64_t)s->num_stages[g] + 3;  /* deadline add, S max + S add, overhead add, compare */
            if (b_check_slo(s, tstamp, g, lat_mg, s->tstamps[r] + (double)s->slos[r])) {
                found = 1; first = r; break;
            }
            s->group_num_requests[g] += 1;                                /* :684-686 */
            s->finish[r] = s->tstamps[r];
            s->good[r] = 0;
        }
        if (!found) {                                                     /* :709-713 */
            const int32_t m2 = b_select_model(s, g);
            if (m2 == -1) return;
            m = m2;
            continue;
        }
        int32_t bs = 1;                                                   /* :693-702 */
        const double deadline = s->tstamps[first] + (double)s->slos[first];
        for (int32_t b = 1; b < s->NB; ++b) {
            const int32_t cand = s->batch_sizes[b];
            if ((int64_t)cand - 1 > qlen(s, m)) break;
            const int col = ilog2_i32(cand);
            if (col >= s->NB) { s->err = -2; return; }
            s->ops += 2 * (int64_t)s->num_stages[g] + 2;
            if (b_check_slo(s, tstamp, g, lat_mg + col, deadline)) bs = cand; else break;
        }
        /* :715-732 */
        const int col = ilog2_i32(bs);
        double t = tstamp + s->fixed_overhead;
        s->ops += 2 * (int64_t)s->num_stages[g] + 1;    /* the commit's overhead add and stage walk */
        double *clk = s->clocks + (size_t)g * s->Smax;
        const int32_t S = s->num_stages[g];
        for (int32_t k = 0; k < S; ++k) {
            t = dmax(t, clk[k]) + (double)lat_mg[(size_t)k * s->NB + col];
            s->tmp[k] = t;
        }
        s->finish[first] = t; s->good[first] = 1;
        for (int32_t u = 1; u < bs; ++u) {                                /* :704 */
            const int64_t r = qfront(s, m);
            s->head[m] += 1;
            s->finish[r] = t; s->good[r] = 1;
        }
        for (int32_t k = 0; k < S; ++k) clk[k] = s->tmp[k];
        idle_ev e; e.t = s->tmp[0]; e.g = g;                              /* :727-728 */
        if (heap_push(&s->heap, e)) { s->err = -1; return; }
        s->group_num_requests[g] += bs;
        s->group_num_good_requests[g] += bs;
        s->model_num_good_requests[m] += bs;
        return;
    }
}

int oracle_simulate_requests_mixed_batching(
    double *finish, uint8_t *good, const double *tstamps,
    const int32_t *model_ids, const float *slos,
    const int32_t *m_id2g_id,     /* [M][G]                                  */
    const int32_t *g_id2m_id,     /* [G][M]                                  */
    const int32_t *num_stages,    /* [G]                                     */
    const float *stage_latency,   /* [M][G][Smax][NB]                        */
    const int32_t *batch_sizes,   /* [NB], batch_sizes[0] == 1               */
    int64_t num_requests, int32_t M, int32_t G, int32_t Smax, int32_t NB,
    double fixed_overhead,
    int32_t *model_num_requests, int32_t *model_num_good_requests,
    int32_t *group_num_requests, int32_t *group_num_good_requests,
    int64_t *max_heap_len /* optional */,
    int64_t *fp_ops /* optional: adds the fp64 operations of every check_slo call (2*S + 2, + 1 for a head's
                       deadline) and of every committed batch (2*S + 1) */)
{
    bsim s;
    memset(&s, 0, sizeof(s));
    s.finish = finish; s.good = good; s.tstamps = tstamps; s.slos = slos;
    s.g_id2m_id = g_id2m_id; s.num_stages = num_stages; s.stage_latency = stage_latency;
    s.batch_sizes = batch_sizes;
    s.M = M; s.G = G; s.Smax = Smax; s.NB = NB; s.fixed_overhead = fixed_overhead;
    s.model_num_good_requests = model_num_good_requests;
    s.group_num_requests = group_num_requests;
    s.group_num_good_requests = group_num_good_requests;
    memset(model_num_requests, 0, sizeof(int32_t) * (size_t)M);
    memset(model_num_good_requests, 0, sizeof(int32_t) * (size_t)M);
    memset(group_num_requests, 0, sizeof(int32_t) * (size_t)G);
    memset(group_num_good_requests, 0, sizeof(int32_t) * (size_t)G);

    const size_t Mz = (size_t)(M > 0 ? M : 1), Gz = (size_t)(G > 0 ? G : 1), Sz = (size_t)(Smax > 0 ? Smax : 1);
    s.clocks = (double *)calloc(Gz * Sz, sizeof(double));
    s.tmp = (double *)calloc(Sz, sizeof(double));
    s.order = (int64_t *)calloc((size_t)(num_requests > 0 ? num_requests : 1), sizeof(int64_t));
    s.qbase = (int64_t *)calloc(Mz + 1, sizeof(int64_t));
    s.head = (int64_t *)calloc(Mz, sizeof(int64_t));
    s.tail = (int64_t *)calloc(Mz, sizeof(int64_t));
    int rc = 0;
    if (!s.clocks || !s.tmp || !s.order || !s.qbase || !s.head || !s.tail) { rc = -1; goto done; }

    /* A model's FIFO only ever holds a contiguous run of the requests of that
     * model that were enqueued, in arrival order: keep them in one array per
     * model (order[qbase[m] + slot]) with a head and a tail counter. */
    for (int64_t i = 0; i < num_requests; ++i)
        if (model_ids[i] >= 0) s.qbase[model_ids[i] + 1] += 1;
    for (int32_t m = 0; m < M; ++m) s.qbase[m + 1] += s.qbase[m];

    for (int64_t i = 0; i < num_requests; ++i) {                          /* :736-778 */
        const double tstamp = tstamps[i];
        while (s.heap.n > 0 && s.heap.a[0].t <= tstamp) {                 /* :739-744 */
            const idle_ev e = heap_pop(&s.heap);
            const int32_t m2 = b_select_model(&s, e.g);
            if (m2 == -1) break;
            b_handle(&s, e.t, m2, e.g);
            if (s.err) { rc = s.err; goto done; }
        }
        const int32_t m = model_ids[i];
        if (m < 0) { finish[i] = tstamp; good[i] = 0; continue; }        /* :748-751 */
        if (m_id2g_id[(size_t)m * G] < 0) {                               /* :754-757 */
            finish[i] = tstamp; good[i] = 0; continue;
        }
        int32_t g = -1;                                                   /* :760-770 */
        double best = ORACLE_INF;
        for (int32_t j = 0; j < G; ++j) {
            const int32_t cand = m_id2g_id[(size_t)m * G + j];
            if (cand < 0) break;
            const double c = s.clocks[(size_t)cand * Smax + (num_stages[cand] - 1)];
            if (c < best) { best = c; g = cand; }
        }
        /* enqueue :772-773 */
        s.order[s.qbase[m] + s.tail[m]] = i;
        s.tail[m] += 1;
        model_num_requests[m] += 1;
        if (g < 0) { rc = -3; goto done; } /* reference would index clocks[-1]; cannot occur for finite clocks */
        if (tstamp >= s.clocks[(size_t)g * Smax]) {                       /* :776-778 group_idle_tstamp[g] == clocks[g][0] */
            b_handle(&s, tstamp, m, g);
            if (s.err) { rc = s.err; goto done; }
        }
    }
    while (s.heap.n > 0) {                                                /* :781-787 */
        const idle_ev e = heap_pop(&s.heap);
        const int32_t m2 = b_select_model(&s, e.g);
        if (m2 == -1) continue;
        b_handle(&s, e.t, m2, e.g);
        if (s.err) { rc = s.err; goto done; }
    }
    for (int32_t m = 0; m < M; ++m)                                       /* :789-790 */
        if (qlen(&s, m) != 0) { rc = -4; break; }
    if (max_heap_len) *max_heap_len = s.heap.max_n;
    if (fp_ops) *fp_ops += s.ops;
done:
    free(s.clocks); free(s.tmp); free(s.order); free(s.qbase); free(s.head); free(s.tail);
    free(s.heap.a);
    return rc;
}

/* ------------------------------------------------------------------------- */
/* Placement -> per-placement tables, controller.py:412-476 (layout only).     */
/* cfg_lat[m][c][k][b] already holds float32(latency*(1+penalty)) or +inf.     */
void oracle_build_stage_latency(
    const float *cfg_lat, int32_t M, int32_t C, int32_t Smax_tab, int32_t NB,
    const int32_t *group_cfg, int32_t G, int32_t Smax,
    float *stage_latency /* [M][G][Smax][NB] */)
{
    for (int32_t m = 0; m < M; ++m)
        for (int32_t g = 0; g < G; ++g)
            for (int32_t k = 0; k < Smax; ++k)
                for (int32_t b = 0; b < NB; ++b)
                    stage_latency[(((size_t)m * G + g) * Smax + k) * NB + b] =
                        cfg_lat[(((size_t)m * C + group_cfg[g]) * Smax_tab + k) * NB + b];
}

/*
 * Evaluate a list of placements on one request stream, one after the other,
 * the way PlacementEvaluator.get_scores does (base_policy.py:175-189), from
 * the same packed inputs the shipped library takes.  Serves as the bounded
 * single-thread CPU baseline and as the batch-level parity checker.
 *
 * group membership is CSR: models of group g of placement b are
 *   gm_idx[gm_off[b*(Gmax+1)+g] .. gm_off[b*(Gmax+1)+g+1])
 */
int oracle_eval_placements(
    int64_t R, int32_t M, const double *tstamps, const int32_t *model_ids, const float *slos,
    const float *cfg_lat, const int32_t *cfg_pp, int32_t C, int32_t Smax_tab, int32_t NB,
    const int32_t *batch_sizes, double fixed_overhead,
    int32_t B, int32_t Gmax, const int32_t *num_groups, const int32_t *group_cfg /* [B][Gmax] */,
    const int64_t *gm_off /* [B][Gmax+1] */, const int32_t *gm_idx,
    int32_t batching,
    int64_t *n_good /* [B] */, double *latency_sum /* [B] */,
    int32_t *model_num_requests, int32_t *model_num_good /* [B][M] or NULL */,
    int32_t *group_num_requests, int32_t *group_num_good /* [B][Gmax] or NULL */,
    double *finish_out /* [B][R] or NULL */, uint8_t *good_out /* [B][R] or NULL */,
    int64_t *fp_ops /* optional */)
{
    double *finish = (double *)malloc(sizeof(double) * (size_t)(R > 0 ? R : 1));
    uint8_t *good = (uint8_t *)malloc((size_t)(R > 0 ? R : 1));
    int32_t *cnt = (int32_t *)malloc(sizeof(int32_t) * (2 * (size_t)M + 2 * (size_t)Gmax + 4));
    int rc = 0;
    if (!finish || !good || !cnt) { rc = -1; goto out; }
    for (int32_t b = 0; b < B && rc == 0; ++b) {
        const int32_t G = num_groups[b];
        const int32_t *gc = group_cfg + (size_t)b * Gmax;
        int32_t Smax = 1;
        for (int32_t g = 0; g < G; ++g) if (cfg_pp[gc[g]] > Smax) Smax = cfg_pp[gc[g]];
        if (Smax > Smax_tab) { rc = -5; break; }
        const int32_t Gz = G > 0 ? G : 1;
        int32_t *m2g = (int32_t *)malloc(sizeof(int32_t) * (size_t)M * Gz);
        int32_t *g2m = (int32_t *)malloc(sizeof(int32_t) * (size_t)Gz * M);
        int32_t *nrep = (int32_t *)calloc((size_t)M, sizeof(int32_t));
        int32_t *ninst = (int32_t *)calloc((size_t)Gz, sizeof(int32_t));
        int32_t *nst = (int32_t *)malloc(sizeof(int32_t) * (size_t)Gz);
        const int32_t NBu = batching ? NB : 1;
        float *sl = (float *)malloc(sizeof(float) * (size_t)M * Gz * Smax * NBu);
        if (!m2g || !g2m || !nrep || !ninst || !nst || !sl) rc = -1;
        if (rc == 0) {
            for (size_t x = 0; x < (size_t)M * Gz; ++x) { m2g[x] = -1; g2m[x] = -1; }
            const int64_t *off = gm_off + (size_t)b * (Gmax + 1);
            for (int32_t g = 0; g < G; ++g) {                               /* :418-422 */
                nst[g] = cfg_pp[gc[g]];
                for (int64_t x = off[g]; x < off[g + 1]; ++x) {
                    const int32_t m = gm_idx[x];
                    m2g[(size_t)m * Gz + nrep[m]++] = g;
                }
            }
            for (int32_t m = 0; m < M; ++m)                                 /* :424-430 */
                for (int32_t j = 0; j < Gz; ++j) {
                    const int32_t g = m2g[(size_t)m * Gz + j];
                    if (g >= 0) g2m[(size_t)g * M + ninst[g]++] = m;
                }
            for (int32_t m = 0; m < M; ++m)
                for (int32_t g = 0; g < G; ++g)
                    for (int32_t k = 0; k < Smax; ++k)
                        for (int32_t q = 0; q < NBu; ++q)
                            sl[(((size_t)m * Gz + g) * Smax + k) * NBu + q] =
                                cfg_lat[(((size_t)m * C + gc[g]) * Smax_tab + k) * NB + q];
            int32_t *mreq = cnt, *mgood = cnt + M, *greq = cnt + 2 * M, *ggood = cnt + 2 * M + Gmax;
            if (batching)
                rc = oracle_simulate_requests_mixed_batching(
                    finish, good, tstamps, model_ids, slos, m2g, g2m, nst, sl, batch_sizes,
                    R, M, Gz, Smax, NB, fixed_overhead, mreq, mgood, greq, ggood, NULL, fp_ops);
            else
                rc = oracle_simulate_requests_mixed(
                    finish, good, tstamps, model_ids, slos, m2g, nst, sl,
                    R, M, Gz, Smax, fixed_overhead, mreq, mgood, greq, ggood, fp_ops);
            if (rc == 0) {
                int64_t ng = 0; double ls = 0.0;
                for (int64_t i = 0; i < R; ++i) { ng += good[i]; ls += finish[i] - tstamps[i]; }
                n_good[b] = ng; latency_sum[b] = ls;
                if (model_num_requests) memcpy(model_num_requests + (size_t)b * M, mreq, sizeof(int32_t) * (size_t)M);
                if (model_num_good) memcpy(model_num_good + (size_t)b * M, mgood, sizeof(int32_t) * (size_t)M);
                if (group_num_requests) {
                    memset(group_num_requests + (size_t)b * Gmax, 0, sizeof(int32_t) * (size_t)Gmax);
                    memcpy(group_num_requests + (size_t)b * Gmax, greq, sizeof(int32_t) * (size_t)G);
                }
                if (group_num_good) {
                    memset(group_num_good + (size_t)b * Gmax, 0, sizeof(int32_t) * (size_t)Gmax);
                    memcpy(group_num_good + (size_t)b * Gmax, ggood, sizeof(int32_t) * (size_t)G);
                }
                if (finish_out) memcpy(finish_out + (size_t)b * R, finish, sizeof(double) * (size_t)R);
                if (good_out) memcpy(good_out + (size_t)b * R, good, (size_t)R);
            }
        }
        free(m2g); free(g2m); free(nrep); free(ninst); free(nst); free(sl);
    }
out:
    free(finish); free(good); free(cnt);
    return rc;
}
