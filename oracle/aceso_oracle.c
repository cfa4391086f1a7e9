/*
 * CPU oracle for the Aceso plan cost model in plain C -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load this file's
 * library; the product package never does.
 *
 * A restatement of the reference's scoring path, function by function, over dense arrays:
 *   search/aceso_cost_model.py  get_time_v3 (:301-356), intra/inter_node_band (:275-299),
 *   identical_spec / get_reshard_primitives (:185-245), get_recompute_time_v3 (:358-373),
 *   get_memory_v3 (:375-394), get_activations_v3 (:396-417), get_peak_activations (:419-447),
 *   get_reserved_memory (:449-485), predict_stage_memory (:514-539), predict_time_breakdown
 *   (:541-672: time_list, memory_list), and the callers' max / feasibility (aceso_search.py:66).
 * Every sum runs in the reference's order with the reference's association, in IEEE doubles
 * (compile without -ffast-math and with -ffp-contract=off), so results are bit-identical to the
 * reference's Python floats.  What the reference resolves through strings and dicts is handed
 * in as tables that the Python oracle (oracle/aceso_oracle.py) fills with its own functions:
 * per-type name predicates, get_op_spec's result per (type, algo, side) as one of four layouts,
 * and get_reshard_time per (collective, group size, table entry).
 *
 * Pinning: tests/test_oracle_c.py checks this file bit for bit against the Python oracle on
 * all synthetic workloads (incl. the error cases) and against the vectors the reference itself
 * wrote (the JSON files under tests/golden: time_list, memory_list of multi-stage plans).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

#define ORC_MAX_STAGES 16

enum { F_FWD, F_BWD, F_IN, F_OUT, F_W, F_ACT, F_RF, F_RB, F_COUNT };
enum { TF_DROPOUT = 1, TF_ZERO_ACT = 2, TF_LAYER_START = 4 };
enum { ORC_OK = 0, ORC_KEY_ERROR = 1, ORC_TYPE_ERROR = 2, ORC_INDEX_ERROR = 3 };

typedef struct orc_db {
    int32_t n_types, n_mbs, n_tp, n_algo;
    const int32_t *mbs_values;            /* [n_mbs] */
    const double *field[F_COUNT];         /* each [n_types][n_mbs][n_tp][n_algo] */
    const uint8_t *type_flags;            /* [n_types] TF_* */
    const int8_t *spec_kind;              /* [n_types][n_algo][2]: side 0 = output spec, 1 = input spec;
                                             -1 None, 0 {R=tp,[1,dp,1]}, 1 {R=tp,[dp,1,1]},
                                             2 {R=1,[1,dp,tp]}, 3 {R=1,[dp,tp,1]}  (model_ops_info.py:92-150) */
    const double *reshard_ms;             /* [4 prims][4 log2(group)][n_types][n_mbs][n_tp][n_algo];
                                             prims: all_reduce, all_gather, reduce_scatter, all_to_all;
                                             NaN where the reference raises KeyError */
    const double *intra_band, *inter_band;
    int32_t n_intra, n_inter;
    int32_t resharding, shared_space, reserved_space, pred_min;
    int32_t gpus_per_node, global_bs;
    double main_params, optimizer, memory_limit;
    int32_t collective_memory;            /* args.consider_collective_memory (:462) */
} orc_db;

typedef struct orc_plans {
    int64_t n_plans;
    int32_t n_ops;
    const int32_t *type_of_pos;           /* [n_ops] */
    const int32_t *num_stages;            /* [P] */
    const int32_t *micro_bs;              /* [P] */
    const int32_t *stage_len;             /* [P][16] ops per stage */
    const uint8_t *tp_log, *dp_log, *algo, *rc;   /* [P][n_ops] */
} orc_plans;

typedef struct { int R, V, dims[3]; int none; } spec_t;
enum { PRIM_NONE = -1, PRIM_ALL_REDUCE = 0, PRIM_ALL_GATHER = 1, PRIM_REDUCE_SCATTER = 2, PRIM_ALL_TO_ALL = 3, PRIM_SPLIT = 4 };

static size_t entry(const orc_db *db, int type, int m, int t, int a) {
    return (((size_t)type * db->n_mbs + m) * db->n_tp + t) * db->n_algo + a;
}

static int mbs_index(const orc_db *db, int mbs) {          /* :22-25, -1 = KeyError */
    for (int k = 0; k < db->n_mbs; ++k)
        if (db->mbs_values[k] == mbs) return k;
    return -1;
}

static double band(const double *b, int n, double data_size) {   /* :275-299 */
    if (data_size > 0) {
        int index = (int)(log(data_size) / log(2.0));       /* int(math.log(x, 2)): truncation toward zero */
        if (index >= 1) index -= 1;
        if (index >= n) return b[n - 1] * 0.001;
        if (index < 0) index += n;                           /* Python's negative index */
        if (index < 0) return NAN;                           /* ... which raises IndexError below -n */
        return b[index] * 0.001;
    }
    return 1;
}

static spec_t make_spec(int kind, int tp, int dp) {
    spec_t s;
    s.none = kind < 0;
    s.V = 1;
    s.R = (kind == 0 || kind == 1) ? tp : 1;
    s.dims[0] = s.dims[1] = s.dims[2] = 1;
    if (kind == 0) { s.dims[1] = dp; }
    else if (kind == 1) { s.dims[0] = dp; }
    else if (kind == 2) { s.dims[1] = dp; s.dims[2] = tp; }
    else if (kind == 3) { s.dims[0] = dp; s.dims[1] = tp; }
    return s;
}

static int identical_spec(const spec_t *a, const spec_t *b) {    /* :185-198 */
    if (a->none || b->none) return 1;
    int same = 1;
    if (a->R != b->R) same = 0;
    if (a->V != b->V) same = 0;
    for (int k = 0; k < 3; ++k)
        if (a->dims[k] != b->dims[k]) same = 0;
    return same;
}

/* :200-245; returns 0 when no rule matches (the reference then fails to unpack None: TypeError) */
static int reshard_primitives(const spec_t *in, const spec_t *req, int *fwd, int *bwd, int *ndev) {
    if (identical_spec(in, req)) { *fwd = PRIM_NONE; *bwd = PRIM_NONE; *ndev = 0; return 1; }
    if (in->R > req->R) {
        for (int k = 0; k < 3; ++k)
            if (in->dims[k] < req->dims[k]) { *fwd = PRIM_SPLIT; *bwd = PRIM_ALL_GATHER; *ndev = in->R / req->R; return 1; }
    } else if (in->V > req->V) {
        if (in->R < req->R) { *fwd = PRIM_ALL_REDUCE; *bwd = PRIM_NONE; *ndev = in->V / req->V; return 1; }
        for (int k = 0; k < 3; ++k)
            if (in->dims[k] < req->dims[k]) { *fwd = PRIM_REDUCE_SCATTER; *bwd = PRIM_ALL_GATHER; *ndev = in->V / req->V; return 1; }
    } else {
        for (int s = 0; s < 3; ++s) {
            if (in->dims[s] > req->dims[s]) {
                if (in->R < req->R) { *fwd = PRIM_ALL_GATHER; *bwd = PRIM_SPLIT; *ndev = in->dims[s] / req->dims[s]; return 1; }
                for (int d = 0; d < 3; ++d)
                    if (d != s && in->dims[d] < req->dims[d]) {
                        *fwd = PRIM_ALL_TO_ALL; *bwd = PRIM_ALL_TO_ALL; *ndev = in->dims[s] / req->dims[s];
                        return 1;
                    }
            }
        }
    }
    return 0;
}

/* get_reshard_time (:247-260) through the table the Python oracle filled; *err on KeyError */
static double reshard_time(const orc_db *db, int prim, int ndev, size_t e, int *err) {
    if (prim == PRIM_SPLIT) return 0;
    int lg = 0;
    while ((1 << lg) < ndev) ++lg;
    if (lg > 3 || (1 << lg) != ndev) { *err = ORC_KEY_ERROR; return 0; }
    size_t per = (size_t)db->n_types * db->n_mbs * db->n_tp * db->n_algo;
    double v = db->reshard_ms[((size_t)prim * 4 + lg) * per + e];
    if (v != v) { *err = ORC_KEY_ERROR; return 0; }
    return v;
}

typedef struct {
    const orc_db *db;
    const int32_t *types;       /* op types of the stage */
    const uint8_t *tp_log, *dp_log, *algo, *rc;
    int n;
    int micro_bs;
} stage_t;

/* mbs index of op i: get_mbs_index(base_batch_size // dp[i]) */
static int op_m(const stage_t *s, int i, int *err) {
    int m = mbs_index(s->db, s->micro_bs / (1 << s->dp_log[i]));
    if (m < 0) { *err = ORC_KEY_ERROR; return 0; }
    return m;
}

static void get_time_v3(const stage_t *s, int in_cross, int out_cross, double out[4], int *err) {   /* :301-356 */
    const orc_db *db = s->db;
    double fwd = 0, bwd = 0;
    if (s->n == 0) { out[0] = out[1] = out[2] = out[3] = 0; return; }
#define TPL(i) (s->tp_log[i])
#define DPL(i) (s->dp_log[i])
#define OPM(i) (op_m(s, i, err))
    for (int i = 0; i < s->n; ++i) {
        int m = OPM(i);
        if (m < 0) { *err = ORC_KEY_ERROR; m = 0; }
        size_t e = entry(db, s->types[i], m, TPL(i), s->algo[i]);
        fwd += db->field[F_FWD][e];
        bwd += db->field[F_BWD][e];
    }
    int in_m = OPM(0), out_m = OPM(s->n - 1);
    if (in_m < 0 || out_m < 0) { *err = ORC_KEY_ERROR; in_m = out_m = 0; }
    double in_sz = db->field[F_IN][entry(db, s->types[0], in_m, TPL(0), s->algo[0])];
    /* sic: the output size is indexed with tp[0], not tp[-1] (:322) */
    double out_sz = db->field[F_OUT][entry(db, s->types[s->n - 1], out_m, TPL(0), s->algo[s->n - 1])];
    double in_comm = in_cross ? in_sz / band(db->inter_band, db->n_inter, in_sz)
                              : in_sz / band(db->intra_band, db->n_intra, in_sz);
    double out_comm = out_cross ? out_sz / band(db->inter_band, db->n_inter, out_sz)
                                : out_sz / band(db->intra_band, db->n_intra, out_sz);
    double fwd_reshard = 0, bwd_reshard = 0;
    if (db->resharding) {
        for (int i = 1; i < s->n; ++i) {
            int tp_p = 1 << TPL(i - 1), dp_p = 1 << DPL(i - 1), tp_c = 1 << TPL(i), dp_c = 1 << DPL(i);
            spec_t prev = make_spec(db->spec_kind[((size_t)s->types[i - 1] * db->n_algo + s->algo[i - 1]) * 2 + 0], tp_p, dp_p);
            spec_t cur = make_spec(db->spec_kind[((size_t)s->types[i] * db->n_algo + s->algo[i]) * 2 + 1], tp_c, dp_c);
            int fp, bp, nd;
            if (!reshard_primitives(&prev, &cur, &fp, &bp, &nd)) { *err = ORC_TYPE_ERROR; continue; }
            int m = OPM(i);
            if (m < 0) { *err = ORC_KEY_ERROR; m = 0; }
            size_t e = entry(db, s->types[i], m, TPL(i), s->algo[i]);
            if (fp != PRIM_NONE) fwd_reshard += reshard_time(db, fp, nd, e, err);
            if (bp != PRIM_NONE) bwd_reshard += reshard_time(db, bp, nd, e, err);
        }
    }
    in_comm += fwd_reshard * 1000;
    out_comm += bwd_reshard * 1000;
    out[0] = fwd; out[1] = bwd; out[2] = in_comm; out[3] = out_comm;
#undef TPL
#undef DPL
#undef OPM
}

static int any_rc(const stage_t *s) {
    for (int i = 0; i < s->n; ++i)
        if (s->rc[i]) return 1;
    return 0;
}

static double get_recompute_time_v3(const stage_t *s, int *err) {   /* :358-373 */
    if (s->n == 0 || !any_rc(s)) return 0;
    double fwd = 0;
    for (int i = 0; i < s->n; ++i)
        if (s->rc[i] == 1)
            fwd += s->db->field[F_FWD][entry(s->db, s->types[i], op_m(s, i, err), s->tp_log[i], s->algo[i])];
    return fwd;
}

static void get_memory_v3(const stage_t *s, double *weights, double *inputs, double *activations, int *err) {   /* :375-394 */
    const orc_db *db = s->db;
    *inputs = db->field[F_IN][entry(db, s->types[0], op_m(s, 0, err), s->tp_log[0], s->algo[0])];
    double a = 0, w = 0;
    for (int i = 0; i < s->n; ++i) {
        size_t e = entry(db, s->types[i], op_m(s, i, err), s->tp_log[i], s->algo[i]);
        uint8_t fl = db->type_flags[s->types[i]];
        if (db->shared_space && (fl & TF_DROPOUT)) a += db->field[F_ACT][e] * 1.5;
        else if (db->shared_space && (fl & TF_ZERO_ACT)) a += 0;
        else a += db->field[F_ACT][e];
        w += db->field[F_W][e];
    }
    *weights = w;
    *activations = a;
}

static double get_activations_v3(const stage_t *s, int *err) {   /* :396-417 */
    const orc_db *db = s->db;
    if (s->n <= 1 || !any_rc(s)) return 0;
    double saved = 0;
    for (int i = 0; i < s->n - 1; ++i) {
        if (s->rc[i] == 1 && s->rc[i + 1] == 1) {
            size_t e = entry(db, s->types[i], op_m(s, i, err), s->tp_log[i], s->algo[i]);
            uint8_t fl = db->type_flags[s->types[i]];
            if (db->shared_space && (fl & TF_DROPOUT)) saved += db->field[F_ACT][e] * 1.5;
            else if (db->shared_space && (fl & TF_ZERO_ACT)) saved += 0;
            else if (db->type_flags[s->types[i + 1]] & TF_LAYER_START) saved += 0;
            else saved += db->field[F_ACT][e];
        }
    }
    return saved;
}

static double get_peak_activations(const stage_t *s, int *err) {   /* :419-447 */
    const orc_db *db = s->db;
    if (s->n <= 1 || !any_rc(s)) return 0;
    double saved = 0, best = 0;                              /* saved_list = [0]; max() at the end */
    for (int i = 0; i < s->n - 1; ++i) {
        if (s->rc[i] == 1 && s->rc[i + 1] == 1) {
            size_t e = entry(db, s->types[i], op_m(s, i, err), s->tp_log[i], s->algo[i]);
            uint8_t fl = db->type_flags[s->types[i]];
            if (db->shared_space && (fl & TF_ZERO_ACT)) saved += 0;
            else if (db->shared_space && (fl & TF_DROPOUT)) saved += db->field[F_ACT][e] * 1.5;
            else {
                saved += db->field[F_ACT][e];
                if ((db->type_flags[s->types[i + 1]] & TF_LAYER_START) || i + 1 == s->n - 1) {
                    if (saved > best) best = saved;
                    saved = 0;
                }
            }
        } else if (saved > 0) {
            if (saved > best) best = saved;
            saved = 0;
        }
    }
    return best;
}

static double get_reserved_memory(const stage_t *s, double memory_weights, int *err) {   /* :449-485 */
    const orc_db *db = s->db;
    double cur_f = 0, cur_b = 0;
    for (int i = 0; i < s->n - 1; ++i) {
        size_t e = entry(db, s->types[i], op_m(s, i, err), s->tp_log[i], s->algo[i]);
        if (db->field[F_RF][e] > cur_f) cur_f = db->field[F_RF][e];
        if (db->field[F_RB][e] > cur_b) cur_b = db->field[F_RB][e];
    }
    double max_collective = 0;
    if (db->collective_memory && db->resharding) {           /* :462-478, get_reshard_memory :262-273 */
        for (int i = 1; i < s->n; ++i) {
            int tp_p = 1 << s->tp_log[i - 1], dp_p = 1 << s->dp_log[i - 1], tp_c = 1 << s->tp_log[i], dp_c = 1 << s->dp_log[i];
            spec_t prev = make_spec(db->spec_kind[((size_t)s->types[i - 1] * db->n_algo + s->algo[i - 1]) * 2 + 0], tp_p, dp_p);
            spec_t cur = make_spec(db->spec_kind[((size_t)s->types[i] * db->n_algo + s->algo[i]) * 2 + 1], tp_c, dp_c);
            int fp, bp, nd;
            if (!reshard_primitives(&prev, &cur, &fp, &bp, &nd)) { *err = ORC_TYPE_ERROR; continue; }
            double sz = db->field[F_IN][entry(db, s->types[i], op_m(s, i, err), s->tp_log[i], s->algo[i])];
            int prims[2] = {fp, bp};
            for (int k = 0; k < 2; ++k) {
                if (prims[k] == PRIM_NONE) continue;
                double c = (prims[k] == PRIM_ALL_GATHER || prims[k] == PRIM_ALL_TO_ALL) ? sz * nd : sz;
                if (c > max_collective) max_collective = c;
            }
        }
    }
    if (!db->pred_min) {
        double a = cur_f + cur_b;
        return (a >= memory_weights ? a : memory_weights) + max_collective;   /* max(a, w): first wins ties */
    }
    double m = cur_f;                                        /* max(cur_f, cur_b, w, max_collective) */
    if (cur_b > m) m = cur_b;
    if (memory_weights > m) m = memory_weights;
    if (max_collective > m) m = max_collective;
    return m;
}

static double predict_stage_memory(const stage_t *s, int num_stages_behind, int *err) {   /* :514-539 */
    const orc_db *db = s->db;
    double memory_weights, inputs, activations;
    get_memory_v3(s, &memory_weights, &inputs, &activations, err);
    double memory_gradients = memory_weights;
    double memory_main_params = memory_weights * db->main_params;
    double memory_optimizer = memory_weights * db->optimizer;
    double saved = get_activations_v3(s, err);
    double peak = get_peak_activations(s, err);
    double memory_reserved = db->reserved_space ? get_reserved_memory(s, memory_weights, err) : 0;
    double memory_activations = (inputs + activations - saved) * num_stages_behind;
    double memory_peak = inputs + activations - saved + peak;
    memory_weights += memory_main_params;
    return memory_weights + memory_gradients + memory_optimizer + memory_activations + memory_peak + memory_reserved;
}

static void score_plan(const orc_db *db, const orc_plans *pl, int64_t p, int strict, double *iter_ms, double *peak_mb,
                       uint8_t *feasible, uint8_t *error, double *time_list, double *memory_list) {
    const int N = pl->n_ops;
    const int S = pl->num_stages[p];
    const int micro_bs = pl->micro_bs[p];
    int err = ORC_OK;
    double t_stage[ORC_MAX_STAGES], mem[ORC_MAX_STAGES];
    const int num_batches = db->global_bs / micro_bs;         /* :544 */
    int lo = 0, gpus_till_now = 0;
    for (int i = 0; i < S; ++i) {
        stage_t s;
        s.db = db;
        s.n = pl->stage_len[p * ORC_MAX_STAGES + i];
        s.types = pl->type_of_pos + lo;
        s.tp_log = pl->tp_log + p * N + lo;
        s.dp_log = pl->dp_log + p * N + lo;
        s.algo = pl->algo + p * N + lo;
        s.rc = pl->rc + p * N + lo;
        s.micro_bs = micro_bs;
        const int num_gpus = (1 << s.tp_log[0]) * (1 << s.dp_log[0]);          /* aceso_utils.py:104 */
        const int in_cross = (gpus_till_now % db->gpus_per_node) == 0 && gpus_till_now > 0;   /* :572 */
        gpus_till_now += num_gpus;
        const int out_cross = (gpus_till_now % db->gpus_per_node) == 0;         /* :574 */
        double t[4];
        get_time_v3(&s, in_cross, out_cross, t, &err);
        double recomp = get_recompute_time_v3(&s, &err);
        t_stage[i] = (t[0] + t[1] + t[2] + t[3] + recomp) / 1000;              /* :579 */
        mem[i] = predict_stage_memory(&s, S - 1 - i, &err);
        lo += s.n;
    }
    double sum_stage_time = 0;                                /* sum(_time_list) */
    for (int i = 0; i < S; ++i) sum_stage_time += t_stage[i];
    double max_t = 0, max_m = 0;
    for (int i = 0; i < S; ++i) {
        double ti = t_stage[i] * (num_batches - 1) + sum_stage_time;            /* :613-619 */
        if (time_list) time_list[p * ORC_MAX_STAGES + i] = ti;
        if (memory_list) memory_list[p * ORC_MAX_STAGES + i] = mem[i];
        if (i == 0 || ti > max_t) max_t = ti;
        if (i == 0 || mem[i] > max_m) max_m = mem[i];
    }
    if (!err && (max_t != max_t || max_m != max_m)) err = ORC_INDEX_ERROR;
    error[p] = (uint8_t)err;
    if (err) {
        iter_ms[p] = NAN; peak_mb[p] = NAN; feasible[p] = 0;
        return;
    }
    iter_ms[p] = max_t;
    peak_mb[p] = max_m;
    feasible[p] = strict ? (max_m < db->memory_limit) : (max_m <= db->memory_limit);
}

int orc_score(const orc_db *db, const orc_plans *pl, int strict, double *iter_ms, double *peak_mb, uint8_t *feasible,
              uint8_t *error, double *time_list, double *memory_list, int n_threads) {
    if (!db || !pl || !iter_ms || !peak_mb || !feasible || !error) return -1;
    if (n_threads < 1) n_threads = 1;
#pragma omp parallel for schedule(dynamic, 64) num_threads(n_threads)
    for (int64_t p = 0; p < pl->n_plans; ++p)
        score_plan(db, pl, p, strict, iter_ms, peak_mb, feasible, error, time_list, memory_list);
    return 0;
}
