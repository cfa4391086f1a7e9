/*
 * ace_eval.h -- C ABI of the MI355X batched plan evaluator (libace_eval.so).
 *
 * The reference (microsoft/SuperScaler, Aceso artifact) has no FFI on this path: the
 * boundary is the Python module search/aceso_cost_model.py, imported by
 * search/aceso_search.py:4, search/aceso_prims.py:7 and search/gen_megatron_plan.py:8.
 * Each entry point below names the reference function(s) it replaces.
 *
 * Conventions: plain pointers and sizes only; every "d_" pointer is DEVICE memory owned by
 * the caller (a torch tensor's data_ptr(), a hipMalloc'ed block ...); nothing allocated by
 * the library crosses the boundary except the opaque handle.  All calls return 0 or a
 * negative ACE_E* code; ace_strerror() names it.  Work is enqueued on the hipStream_t the
 * caller passes (as void*, NULL = the default stream); results are valid once that stream
 * has been synchronised.  One handle belongs to one device and must be created after any
 * fork() (the reference's search forks one process per pipeline depth).
 */
#ifndef ACE_EVAL_H
#define ACE_EVAL_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ACE_ABI_VERSION 8
#define ACE_MAX_STAGES 16      /* aceso_utils.py:502: end_num_stages = min(num_gpus, 16) */
#define ACE_STAGE_REC 18       /* doubles per stage record, see ACE_R_* */

enum {
    ACE_OK = 0,
    ACE_EINVAL = -1,      /* null pointer / bad size / bad table geometry */
    ACE_ETOOBIG = -2,     /* a single op type's table row exceeds LDS */
    ACE_EHIP = -3,        /* a HIP runtime call failed (ace_last_hip_error() says which) */
    ACE_ENOMEM = -4,
    ACE_EVERSION = -5,
    ACE_EFIXED = -6,      /* the call would have to reallocate a workspace that ace_reserve() fixed */
};

/* per-plan status bytes written by ace_score_batch */
enum {
    ACE_PLAN_OK = 0,
    ACE_PLAN_UNSCORABLE = 1,   /* the reference raises for this plan: micro_bs // dp is not a profiled
                                  micro-batch size (KeyError, aceso_cost_model.py:22-25), the specs of two
                                  adjacent ops of a stage are inconsistent (TypeError, :344) or a collective
                                  was never profiled for the group size (KeyError, :251).  Scores are NaN. */
    ACE_PLAN_MALFORMED = 3,    /* the encoding itself is inconsistent (stage bits vs num_stages ...) */
};

/* indices into a stage record (doubles); units as in the reference: us, MB */
enum {
    ACE_R_FWD = 0, ACE_R_BWD, ACE_R_IN_COMM, ACE_R_OUT_COMM, ACE_R_RECOMP,   /* get_time_v3 / get_recompute_time_v3 */
    ACE_R_WEIGHTS, ACE_R_INPUTS, ACE_R_ACT, ACE_R_SAVED, ACE_R_PEAK, ACE_R_RESERVED, /* get_memory_v3 ... get_reserved_memory */
    ACE_R_IDEAL_FWD, ACE_R_IDEAL_BWD, ACE_R_IDEAL_IN, ACE_R_IDEAL_OUT,       /* the tp=dp=1 pass, aceso_cost_model.py:588-592 */
    ACE_R_STAGE_MS, ACE_R_STAGE_MB,                                          /* stage time ms (:579), stage memory MB (:534) */
    ACE_R_RESHARD                                                            /* (fwd + bwd resharding) us, the print-only column of :355 */
};

/*
 * Compiled tables of one (model, profile database, settings) triple; built on the host by
 * superscaler_amd.tables.compile_tables().  All pointers are HOST memory, copied during
 * ace_create().  Replaces the module state read_profiled_time() fills
 * (aceso_cost_model.py:27-183) plus the per-call lookups get_op_spec / get_reshard_primitives
 * / get_reshard_time / intra_node_band / inter_node_band (:185-299), which are resolved into
 * these tables ahead of time.
 */
typedef struct ace_tables {
    int32_t abi_version;
    int32_t num_ops;        /* N: positions in the op sequence */
    int32_t num_types;      /* distinct op names (table rows) */
    int32_t n_mbs, n_tp, n_algo;
    int32_t n_diag;         /* distinct (micro_bs, stage gpus) -> per-tp micro-batch index maps, at most 14;
                               the hot sub-table holds n_diag + 1 (the last one all NaN) */
    int32_t n_glog;         /* stage device counts 2^0 .. 2^(n_glog-1) */
    int32_t n_z;            /* resharding cost tables: table 0 is all zeros (nothing to pay), then one per
                               (collective, group size) in use, the last one all NaN (the reference raises) */
    int32_t n_pair_kinds;   /* distinct adjacent-op spec pairings */
    int32_t row_doubles;    /* doubles per type row (even) */
    int32_t hot_off, start_off, out_off, z_off;   /* sub-table offsets inside a row, in doubles */
    int32_t z_table_doubles; /* doubles per resharding cost table (power of two >= n_diag * C) */
    int32_t n_windows;      /* >= 1; > 1 when the rows do not all fit in LDS */
    int32_t lds_row_bytes;  /* bytes of LDS reserved for resident rows */
    int32_t flags;          /* ACE_F_* */
    double main_params, optimizer;   /* aceso_utils.py:48-52 */
    const double *rows;            /* [num_types][row_doubles] */
    const uint32_t *pos_info;      /* [num_ops + 1]: LDS slot of the op's row | slot of the next op's row << 8 |
                                      kind of the (this op, next op) pair << 16 | flags << 24: bit 24 = an
                                      ordinary op followed by a layer start, bit 25 = an ordinary op
                                      (a slot is row_doubles * 8 bytes; the last entry is unused) */
    const uint8_t *pair_kinds;     /* [n_pair_kinds][n_glog][8][8] (first op's code, second op's code) */
    const uint32_t *stage_lut;     /* [n_mbs][16] by log2(stage gpus): diag | per-tp mbs-index nibbles << 16;
                                      diag n_diag = the all-NaN entries after the hot sub-table (a pair the
                                      reference raises KeyError for) */
    const double *nb_minus_1;      /* [n_mbs]: global_bs // micro_bs - 1 */
    const int32_t *win_pos;        /* [n_windows + 1] first position of each window (multiples of 4) */
    const int32_t *win_row_begin;  /* [n_windows + 1] into win_rows */
    const uint32_t *win_rows;      /* [..][2]: type id, LDS byte offset */
} ace_tables_t;

#define ACE_F_RESHARDING 1      /* args.resharding (aceso_utils.py:523-526) */
#define ACE_F_RESERVED_MIN 2    /* memory_pred_type == "MIN" (aceso_cost_model.py:482) */
#define ACE_F_NO_RESERVED 4     /* not consider_reserved_space (aceso_cost_model.py:525-528) */
#define ACE_F_COLLECTIVE_MEM 8   /* consider_collective_memory (aceso_cost_model.py:462-478): n_z more tables follow the
                                   n_z cost tables in every row, holding the MB each collective occupies
                                   (get_reshard_memory, :262-273) */

typedef struct ace_handle ace_handle_t;

/* A batch of plans, structure-of-arrays, resident in device memory.
 *  d_codes: uint8, one byte per (op, plan): bits 0-2 = tp_log2 * n_algo + algo, bit 3 = recompute,
 *           bit 4 = this op starts a pipeline stage.  Laid out [ceil(N/16)][n_plans][16]: sixteen
 *           consecutive ops of one plan are contiguous, consecutive plans follow each other, so a
 *           wavefront (one plan per lane) reads 1 KiB contiguous per load.
 *  d_hdr:   uint32[n_plans][4]: num_stages | micro-batch index << 8;  log2(stage gpus), 4 bits per
 *           stage (two words);  in-cross-node bit per stage | out-cross-node bits << 16
 *           (aceso_cost_model.py:572-574).
 * Replaces AcesoConfig / AcesoStageInfo (aceso_utils.py:58-89) as the scoring input. */
typedef struct ace_batch {
    const uint8_t *d_codes;
    const uint32_t *d_hdr;
    const uint32_t *d_range;   /* NULL, or uint32[n_plans][2] = (first op, one past the last op): each plan is ONE
                                  stage over that slice of the op sequence (bit 4 set on its first op only,
                                  num_stages field = num_stages_behind + 1).  The form of the single-stage queries
                                  predict_stage_time / predict_stage_memory (aceso_cost_model.py:493-539);
                                  results are read from stage record 0, so d_stage_out is required. */
    size_t n_plans;
    const uint32_t *d_order;   /* NULL, or uint32[n_plans]: slot i of d_codes / d_hdr / d_range holds the caller's plan
                                  d_order[i], and every result of that plan (d_iter_ms, d_peak_mb, d_feasible,
                                  d_status, d_stage_out) is written at index d_order[i].  Lets the caller store the
                                  plans in the order that suits the kernel -- lanes of a wavefront that close their
                                  stages at the same ops do not wait for each other, so grouping plans by pipeline
                                  depth (deepest first) and first stage boundaries is worth about a seventh of the
                                  kernel time on mixed batches -- and still get results in its own order.  Must be
                                  a permutation of 0 .. n_plans - 1 (entries >= n_plans are skipped). */
} ace_batch_t;

int ace_abi_version(void);
const char *ace_strerror(int code);
const char *ace_last_hip_error(void);

/* Upload tables to the current device.  Replaces read_profiled_time (aceso_cost_model.py:27). */
int ace_create(const ace_tables_t *tables, ace_handle_t **out);
void ace_destroy(ace_handle_t *h);

/* Score every plan of the batch: predict_time_breakdown (aceso_cost_model.py:541-672) followed by
 * the callers' reductions max(time_list), max(memory_list) and the feasibility test
 * max(memory_list) <= memory_limit (aceso_search.py:66; strict != 0 selects `<`,
 * gen_megatron_plan.py:111).
 *  d_iter_ms, d_peak_mb: double[n_plans];  d_feasible, d_status: uint8[n_plans] (d_status may be NULL)
 *  d_stage_out: NULL, or double[n_plans][ACE_MAX_STAGES][ACE_STAGE_REC] receiving the per-stage
 *  quantities predict_time_breakdown / predict_stage_time / predict_stage_memory are made of; for a
 *  batch of single-stage queries (batch->d_range) one record each: double[n_plans][ACE_STAGE_REC].
 * Plain scoring (no d_stage_out, no d_range) uses a workspace owned by the handle (80 bytes per plan
 * and stage, allocated on first use and grown when a larger batch arrives: that call allocates, unless
 * ace_reserve() sized or fixed it beforehand), so scoring calls on one handle must be stream-ordered with
 * respect to each other. */
int ace_score_batch(ace_handle_t *h, const ace_batch_t *batch, double memory_limit, int strict,
                    double *d_iter_ms, double *d_peak_mb, uint8_t *d_feasible, uint8_t *d_status,
                    double *d_stage_out, void *stream);

/* ace_score_batch for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): plain scoring (no d_stage_out, no batch->d_range) of at most
 * ACE_STATIC_MAX_PLANS plans, with the deferred-stage-tail records in a static device array of the library
 * (ACE_STATIC_MAX_PLANS * 1,280 bytes = 20 MiB, held by every GPU the library runs on until the process ends)
 * instead of the handle's workspace.  It calls no hipMalloc / hipFree and no allocating library routine, and
 * leaves the handle's workspace alone.  Same results as ace_score_batch, bit for bit.  Returns ACE_ETOOBIG for a
 * larger batch.  The array is shared by every call on that GPU, whichever handle or stream: calls that overlap
 * in time on one GPU race on it (order them on one stream, or with events); nothing in it has to be cleared
 * between calls (a launch reads back only the records it wrote itself).  The handle's device must be current.
 * No counterpart in the reference. */
#define ACE_STATIC_MAX_PLANS 16384
int ace_score_batch_static(ace_handle_t *h, const ace_batch_t *batch, double memory_limit, int strict,
                           double *d_iter_ms, double *d_peak_mb, uint8_t *d_feasible, uint8_t *d_status, void *stream);

/* Size the handle's workspace for plain scoring of batches of up to max_plans plans now (max_plans = 0: leave it as
 * it is), so that no later ace_score_batch / ace_time_score_kernel call of that size allocates.  With fixed != 0 a
 * later call that needs a larger workspace returns ACE_EFIXED instead of freeing and reallocating it (which would
 * synchronise the device in the middle of a stream, is invalid during stream capture and would leave a recorded
 * graph with the address of freed memory); fixed = 0 lets the workspace grow on demand again.  This call itself
 * may allocate: make it outside any capture.  No counterpart in the reference. */
int ace_reserve(ace_handle_t *h, size_t max_plans, int fixed);

/* The k feasible plans with the smallest iteration time, ascending, ties broken by the lower plan
 * index: the order sort_configs (aceso_utils.py:723-740) / gen_megatron_plan.py:131-135 produce.
 *  d_idx: int64[k], d_val: double[k]; entries past the number of feasible plans are -1 / +inf.
 *  d_workspace: device scratch of at least ace_topk_workspace_bytes(n, k) bytes.
 *  *d_count (int32, device, may be NULL) receives min(k, number of feasible plans). */
size_t ace_topk_workspace_bytes(size_t n, int k);
int ace_topk(ace_handle_t *h, const double *d_iter_ms, const uint8_t *d_feasible, size_t n, int k,
             int64_t *d_idx, double *d_val, int32_t *d_count, void *d_workspace, size_t workspace_bytes,
             void *stream);

/* Expand move descriptors into a batch of neighbour plans on the device, in the layout
 * ace_score_batch reads.  Replaces the per-candidate object rebuilding of the reference's move
 * primitives (search/aceso_prims.py:66-134 op migration, :357-375 tp / dp changes, :544-580
 * micro-batch steps, recompute and algorithm fine-tuning) for candidates that differ from a
 * template plan by one edit.
 *  d_template_codes: uint8[n_templates][16 * ceil(num_ops / 16)], one byte per op as in ace_batch_t,
 *                    plan-major (template 0 is normally the plan whose neighbours are wanted);
 *  d_template_hdr:   uint32[n_templates][4];
 *  d_moves:          uint32[n_moves][4] = template | op << 16, p0, p1, 0 with
 *                    op 0 copy; 1 migrate ops across a stage boundary (p0 = cut | new cut << 16, p1 = log2 tp
 *                    the moved ops take); 2 one tp step for the ops p0 = first | last + 1 << 16 (p1 = 1 up, 0 down);
 *                    3 toggle the recompute bit of the ops p0 = first | last + 1 << 16; 4 toggle the algorithm of op p0;
 *  d_codes_out:      uint8[ceil(num_ops / 16)][n_moves][16];  d_hdr_out: uint32[n_moves][4];
 *  d_keys_out:       NULL, or uint64[n_moves][2] that the CALLER HAS ZEROED: receives a 128-bit key of every
 *                    plan's bytes (equal plans -> equal keys; for visited sets, aceso_search.py:47,105; the reference's
 *                    sets hold the plans' full strings, aceso_utils.py:831-850: two distinct plans share a key with a
 *                    probability of about n^2 / 2^129 for n plans).
 * The caller decides which moves are legal; the kernel only edits bytes. */
int ace_apply_moves(const uint8_t *d_template_codes, const uint32_t *d_template_hdr, int n_templates,
                    const uint32_t *d_moves, size_t n_moves, int num_ops, int n_algo, uint8_t *d_codes_out,
                    uint32_t *d_hdr_out, uint64_t *d_keys_out, void *stream);

/* Sort keys for grouped storage (ace_batch_t.d_order) of a batch that is already on the device: d_keys[i]
 * (uint64[n_plans]) orders the plans by pipeline depth, deepest first, then by the positions of their first two
 * stage boundaries.  The caller sorts the keys (stably), deals the sorted wavefronts of 64 to the workgroups and
 * gathers d_codes / d_hdr into that order (superscaler_amd/evaluator.py: PlanEvaluator.group shows how).
 * d_codes: uint8[ceil(num_ops / 16)][n_plans][16], d_hdr: uint32[n_plans][4] as in ace_batch_t.
 * No counterpart in the reference, which scores one plan at a time. */
int ace_group_keys(const uint8_t *d_codes, const uint32_t *d_hdr, size_t n_plans, int num_ops, uint64_t *d_keys, void *stream);

/* Reorder a device-resident batch: slot i of the output holds plan d_perm[i] (uint32[n_plans]) of the input; the
 * same d_perm is then the d_order of the output batch.  Input and output must not overlap.
 * No counterpart in the reference. */
int ace_gather_plans(const uint8_t *d_codes_in, const uint32_t *d_hdr_in, const uint32_t *d_perm, size_t n_plans, int num_ops,
                     uint8_t *d_codes_out, uint32_t *d_hdr_out, void *stream);

/* The two steps of check_recompute's greedy loop (aceso_cost_model.py:822-872) that are not a stage
 * evaluation, for many encoded stages at once (one stage = the ops [lo, hi) of one plan of the batch).
 * The caller runs the loop: evaluate the stages (ace_score_batch with d_range), update their memory
 * (:861-867), call ace_recompute_select for those still above the limit, repeat. */
typedef struct ace_rc_tables {
    const uint8_t *d_codes;          /* the batch, uint8[ceil(num_ops / 16)][n_plans][16] */
    size_t n_plans;
    const int32_t *d_type_of_pos;    /* int32[num_ops]: op type (table row) of every position */
    const double *d_activations;     /* double[num_types][n_mbs][n_tp][n_algo]: the raw "activations" column
                                        (get_activation_size, aceso_cost_model.py:487-491) */
    const uint8_t *d_no_recompute;   /* uint8[num_types]: op names get_next_recompute_op_group never picks (:798) */
    int32_t num_ops, num_types, n_mbs, n_tp, n_algo;
} ace_rc_tables_t;

/* Op groups of every stage (:835-843).  d_plan / d_lo / d_hi / d_nsb: int32[n_stages] (plan index, first op,
 * one past the last op, num_stages_behind); d_mrow: uint32[n_stages], the micro-batch index of the stage per
 * tp (4 bits each, as in ace_tables_t.stage_lut).  d_sum_size: double[n_stages][num_types] ZEROED by the
 * caller; d_first_pos: int32[n_stages][num_types] FILLED WITH num_ops by the caller; d_bad: int32[n_stages]
 * zeroed by the caller, set where an op sits outside the profiled grid (the reference raises KeyError) or the
 * stage does not lie inside the batch (such a stage is left alone by both calls). */
int ace_recompute_groups(const ace_rc_tables_t *t, int n_stages, const int32_t *d_plan, const int32_t *d_lo,
                         const int32_t *d_hi, const int32_t *d_nsb, const uint32_t *d_mrow, double *d_sum_size,
                         int32_t *d_first_pos, int32_t *d_bad, void *stream);

/* One greedy round for every stage with d_alive[k] != 0: get_next_recompute_op_group (:794-820) on the
 * groups above and d_mem[k] - memory_limit, then the recompute bit of the chosen ops and of the op after each
 * (:852-859) is set in d_codes_rw (normally the same buffer as t->d_codes).  d_recomputed:
 * uint8[n_stages][num_types], zeroed before the first round; d_alive[k] is cleared where the loop ends. */
int ace_recompute_select(const ace_rc_tables_t *t, uint8_t *d_codes_rw, int n_stages, const int32_t *d_plan,
                         const int32_t *d_lo, const int32_t *d_hi, const int32_t *d_nsb, const uint32_t *d_mrow,
                         const double *d_sum_size, const int32_t *d_first_pos, uint8_t *d_recomputed, const double *d_mem,
                         double memory_limit, uint8_t *d_alive, void *stream);

/* Average duration in milliseconds of the `reps` scoring-kernel launches of one
 * ace_score_batch-equivalent call sequence, measured with hipEvents on `stream`
 * (for bench.py's roofline figure; not part of the reference). */
int ace_time_score_kernel(ace_handle_t *h, const ace_batch_t *batch, double memory_limit, int strict,
                          double *d_iter_ms, double *d_peak_mb, uint8_t *d_feasible, int reps,
                          void *stream, double *avg_ms);

#ifdef __cplusplus
}
#endif
#endif /* ACE_EVAL_H */
