// Bounds-checked CPU build of the per-plan state machine (superscaler_amd/csrc/ace_plan_state.h)
// -- TEST INFRASTRUCTURE ONLY.  It lets the CPU test-suite run the exact source the GPU kernel
// is made of (same header, compiled with ACE_HOST_EMU) against the oracle, with every "LDS"
// access checked for range and alignment, before anything is launched on a GPU.  The product
// library never links or loads this file.
#define ACE_HOST_EMU 1
#include "ace_edit_kernels.h"
#include "ace_score_loop.h"

#include <sys/mman.h>

#include <vector>

namespace {

template <bool BD, bool RANGED, bool DEFER = false, bool COLL = false>
void score_one(const ace_tables_t *t, const AceGeom &g, std::vector<unsigned char> &lds, uint32_t lds_bytes,
               const uint8_t *codes, ace_u4 h, ace_u2 range, double *rec, double &iter, double &peak, uint8_t &feas,
               uint8_t &st) {
    const size_t row_bytes = (size_t)t->row_doubles * 8;
    const uint32_t *pos = t->pos_info;
    AceLds view{lds.data(), lds_bytes};
    PlanState<BD, RANGED, DEFER, COLL> s;
    std::vector<double> ws(ACE_MAX_STAGES * ACE_WS_REC, __builtin_nan(""));
    if (DEFER) rec = ws.data();
    s.init(g, view, h, range);
    int w = 0, next_win = t->win_pos[0];
    for (int i = 0; i < g.N; ++i) {
        if (i == next_win) {
            // poison, then stage exactly the rows the window lists: a read of any other row yields NaN
            memset(lds.data(), 0xff, t->lds_row_bytes);
            for (int r = t->win_row_begin[w]; r < t->win_row_begin[w + 1]; ++r)
                memcpy(lds.data() + t->win_rows[2 * r + 1], t->rows + (size_t)t->win_rows[2 * r] * t->row_doubles, row_bytes);
            next_win = t->win_pos[++w];
        }
        if (!RANGED && i == 0) s.begin(g, view, 0, codes[0], pos[0]);
        const uint32_t nbyte = i + 1 < g.N ? codes[i + 1] : 0u;
        s.step(g, view, i, codes[i], nbyte, pair_bit(codes[i], nbyte), pos[i], i > 0 ? pos[i - 1] : 0u, i + 1 == g.N, rec);
    }
    if (DEFER) {
        s.replay_all(g, view, rec, s.s, codes[0] & 7u, pos[0] & 0xffu);
    }
    s.result(g, t->nb_minus_1[s.bidx], iter, peak, feas, st);
}

}  // namespace

extern "C" int ace_emu_score(const ace_tables_t *t, const uint8_t *codes /* [P][N] plan-major */,
                             const uint32_t *hdr /* [P][4] */, const uint32_t *range /* nullable [P][2] */,
                             long long P, double memory_limit, int strict, int defer, double *iter_ms, double *peak_mb,
                             uint8_t *feasible, uint8_t *status, double *stage_out /* nullable [P][16][18]; with ranges [P][18] */) {
    const int C = t->n_tp * t->n_algo;
    AceGeom g;
    memset(&g, 0, sizeof(g));
    g.N = t->num_ops; g.P = (int32_t)P; g.G = (t->num_ops + 15) / 16;
    g.C = C; g.A_shift = t->n_algo == 2 ? 1 : 0;
    g.n_mbs = t->n_mbs; g.n_tp = t->n_tp; g.n_algo = t->n_algo; g.n_glog = t->n_glog; g.n_pair_kinds = t->n_pair_kinds;
    g.hot_off = t->hot_off * 8u; g.start_off = t->start_off * 8u; g.out_off = t->out_off * 8u; g.z_off = t->z_off * 8u;
    g.z_shift = 3;
    while ((1 << (g.z_shift - 3)) < t->z_table_doubles) ++g.z_shift;
    g.zm_delta = (uint32_t)t->n_z << g.z_shift;
    const int32_t rk_bytes = t->n_pair_kinds * t->n_glog * 64;
    g.rk_lds_off = (uint32_t)t->lds_row_bytes;
    const uint32_t lds_bytes = ace_lds_layout(g.rk_lds_off, (uint32_t)rk_bytes, (uint32_t)t->n_mbs * 16u, &g.stg_lds_off, &g.lut2_lds_off);
    g.rk_kind_stride = (uint32_t)(t->n_glog * 64);
    g.row_bytes = (uint32_t)t->row_doubles * 8u;
    g.flags = t->flags; g.main_params = t->main_params; g.optimizer = t->optimizer;
    g.mem_limit = memory_limit; g.strict = strict ? 1 : 0;
    if (range && !stage_out) return -1;

    std::vector<unsigned char> lds(lds_bytes);
    for (long long p = 0; p < P; ++p) {
        memset(lds.data(), 0xff, lds.size());
        memcpy(lds.data() + g.rk_lds_off, t->pair_kinds, rk_bytes);
        memcpy(lds.data() + g.stg_lds_off, t->stage_lut, (size_t)t->n_mbs * 16 * 4);
        for (int j = 0; j < t->n_mbs * 16; ++j) {       // (as the kernel's staging loop fills this region)
            const uint32_t glog = (uint32_t)j & 15u, z_v = (t->stage_lut[j] & 15u) * (uint32_t)C * 8u;
            const ace_u2 e{z_v, ((glog < (uint32_t)t->n_glog ? glog : 0u) << 6) - z_v};
            memcpy(lds.data() + g.lut2_lds_off + 8 * j, &e, 8);
        }
        ace_u4 h;
        memcpy(&h, hdr + 4 * p, 16);
        ace_u2 rg{0u, 0u};
        if (range) memcpy(&rg, range + 2 * p, 8);
        double *rec = stage_out ? stage_out + (size_t)p * (range ? 1 : ACE_MAX_STAGES) * ACE_STAGE_REC : nullptr;
        const uint8_t *c = codes + (size_t)p * g.N;
        double iter, peak;
        uint8_t feas, st;
        const bool coll = (t->flags & ACE_F_COLLECTIVE_MEM) != 0;
        if (coll) {
            if (range) score_one<true, true, false, true>(t, g, lds, lds_bytes, c, h, rg, rec, iter, peak, feas, st);
            else if (stage_out) score_one<true, false, false, true>(t, g, lds, lds_bytes, c, h, rg, rec, iter, peak, feas, st);
            else score_one<false, false, false, true>(t, g, lds, lds_bytes, c, h, rg, rec, iter, peak, feas, st);
        }
        else if (range) score_one<true, true>(t, g, lds, lds_bytes, c, h, rg, rec, iter, peak, feas, st);
        else if (stage_out) score_one<true, false>(t, g, lds, lds_bytes, c, h, rg, rec, iter, peak, feas, st);
        else if (defer && t->n_windows == 1) score_one<false, false, true>(t, g, lds, lds_bytes, c, h, rg, rec, iter, peak, feas, st);
        else score_one<false, false>(t, g, lds, lds_bytes, c, h, rg, rec, iter, peak, feas, st);
        iter_ms[p] = iter; peak_mb[p] = peak; feasible[p] = feas;
        if (status) status[p] = st;
    }
    return 0;
}


// ------------------------------------------------------------------------------------------
// The kernel's own op loop (ace_score_loop.h) on the CPU, one lane per "workgroup", with every
// array the kernel reads or writes placed flush against an inaccessible page: an index past an
// array's end (or a page or more before its start) ends the process with SIGSEGV instead of
// going unnoticed.  Callers run this in a child process.
// ------------------------------------------------------------------------------------------
namespace {

struct GuardedPool {
    struct Map { void *base; size_t len; };
    std::vector<Map> maps;
    // a writable copy of `bytes` bytes of `src` (zeros if null) whose end (rounded up to `align` bytes, the
    // alignment the kernel's loads of that array need) touches a PROT_NONE page
    void *place(const void *src, size_t bytes, size_t align = 16) {
        const size_t pg = 4096, body = (bytes + pg - 1) / pg * pg + pg;
        unsigned char *m = (unsigned char *)mmap(nullptr, body + 2 * pg, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS, -1, 0);
        if (m == MAP_FAILED) { perror("mmap"); abort(); }
        mprotect(m, pg, PROT_NONE);
        mprotect(m + pg + body, pg, PROT_NONE);
        maps.push_back({m, body + 2 * pg});
        unsigned char *p = m + pg + body - ((bytes + align - 1) / align * align);
        if (src) memcpy(p, src, bytes);
        return p;
    }
    ~GuardedPool() { for (auto &m : maps) munmap(m.base, m.len); }
};

template <bool BD, bool RANGED, bool WIN, bool DEFER, bool COLL = false>
void run_lanes(const AceKernelArgs &a, unsigned char *lds, uint32_t lds_bytes) {
    for (long long p = 0; p < a.g.P; ++p) {
        memset(lds, 0xff, lds_bytes);
        ace_score_body<BD, RANGED, WIN, DEFER, 1, COLL>(a, lds, lds_bytes, 0, p, (uint32_t)a.g.P);
    }
}

}  // namespace

// codes: uint8 [G][P][16] (the kernel's layout).  Chooses the kernel variant as the library's launcher does.
extern "C" int ace_emu_kernel(const ace_tables_t *t, const uint8_t *codes, const uint32_t *hdr, const uint32_t *range,
                              const uint32_t *order /* nullable [P] */, long long P, double memory_limit, int strict,
                              double *iter_ms, double *peak_mb, uint8_t *feasible, uint8_t *status, double *stage_out) {
    if (range && !stage_out) return -1;
    AceKernelArgs a;
    memset(&a, 0, sizeof(a));
    AceGeom &g = a.g;
    const int C = t->n_tp * t->n_algo;
    g.N = t->num_ops; g.P = (int32_t)P; g.G = (t->num_ops + 15) / 16;
    g.C = C; g.A_shift = t->n_algo == 2 ? 1 : 0;
    g.n_mbs = t->n_mbs; g.n_tp = t->n_tp; g.n_algo = t->n_algo; g.n_glog = t->n_glog; g.n_pair_kinds = t->n_pair_kinds;
    g.hot_off = t->hot_off * 8u; g.start_off = t->start_off * 8u; g.out_off = t->out_off * 8u; g.z_off = t->z_off * 8u;
    g.z_shift = 3;
    while ((1 << (g.z_shift - 3)) < t->z_table_doubles) ++g.z_shift;
    g.zm_delta = (uint32_t)t->n_z << g.z_shift;
    a.rk_bytes = t->n_pair_kinds * t->n_glog * 64;
    g.rk_lds_off = (uint32_t)t->lds_row_bytes;
    a.stg_words = t->n_mbs * 16;
    const uint32_t lds_bytes = ace_lds_layout(g.rk_lds_off, (uint32_t)a.rk_bytes, (uint32_t)a.stg_words, &g.stg_lds_off, &g.lut2_lds_off);
    g.rk_kind_stride = (uint32_t)(t->n_glog * 64);
    g.row_bytes = (uint32_t)t->row_doubles * 8u;
    g.flags = t->flags; g.main_params = t->main_params; g.optimizer = t->optimizer;
    g.mem_limit = memory_limit; g.strict = strict ? 1 : 0;
    a.n_windows = t->n_windows; a.row_doubles = t->row_doubles;

    GuardedPool pool;
    const size_t G = (size_t)g.G, n_win_rows = (size_t)t->win_row_begin[t->n_windows];
    a.codes = (const ace_u4 *)pool.place(codes, G * (size_t)P * 16);
    a.hdr = (const ace_u4 *)pool.place(hdr, (size_t)P * 16);
    a.range = range ? (const ace_u2 *)pool.place(range, (size_t)P * 8, 8) : nullptr;
    a.order = order ? (const uint32_t *)pool.place(order, (size_t)P * 4, 4) : nullptr;
    a.rows = (const double *)pool.place(t->rows, (size_t)t->num_types * t->row_doubles * 8);
    // (the library uploads the num_ops + 1 descriptors into a zeroed array of 16 * G + 16)
    uint32_t *pos = (uint32_t *)pool.place(nullptr, (G * 16 + 16) * 4);
    memcpy(pos, t->pos_info, (size_t)(t->num_ops + 1) * 4);
    a.pos_info = pos;
    if (t->n_windows > 1 && t->num_types <= 256) {
        uint32_t *pt = (uint32_t *)pool.place(nullptr, (G * 16 + 16) * 4);
        ace_pos_types(t, pt, G * 16 + 16);
        a.pos_types = pt;
    }
    a.pair_kinds = (const uint8_t *)pool.place(t->pair_kinds, (size_t)a.rk_bytes, 4);
    a.stage_lut = (const uint32_t *)pool.place(t->stage_lut, (size_t)a.stg_words * 4, 4);
    a.nbm1 = (const double *)pool.place(t->nb_minus_1, (size_t)t->n_mbs * 8, 8);
    a.win_pos = (const int32_t *)pool.place(t->win_pos, (size_t)(t->n_windows + 1) * 4, 4);
    a.win_row_begin = (const int32_t *)pool.place(t->win_row_begin, (size_t)(t->n_windows + 1) * 4, 4);
    a.win_rows = (const uint32_t *)pool.place(t->win_rows, n_win_rows * 8, 4);
    // (what the library works out at ace_create: resident rows that lie in LDS as in global memory are staged as one block)
    if (t->n_windows == 1 && (t->row_doubles & 1) == 0) {
        bool flat = true;
        for (int r = 0; r < t->win_row_begin[1]; ++r)
            flat = flat && t->win_rows[2 * r] == (uint32_t)r && t->win_rows[2 * r + 1] == (uint32_t)r * (uint32_t)t->row_doubles * 8u;
        if (flat) a.flat_rows16 = t->win_row_begin[1] * (t->row_doubles / 2);
    }
    a.iter_ms = (double *)pool.place(iter_ms, (size_t)P * 8, 8);
    a.peak_mb = (double *)pool.place(peak_mb, (size_t)P * 8, 8);
    a.feasible = (uint8_t *)pool.place(feasible, (size_t)P, 1);
    a.status = status ? (uint8_t *)pool.place(status, (size_t)P, 1) : nullptr;
    const size_t rec_bytes = (size_t)P * (range ? 1 : ACE_MAX_STAGES) * ACE_STAGE_REC * 8;
    a.stage_out = stage_out ? (double *)pool.place(stage_out, rec_bytes, 8) : nullptr;   // (records of unused stages stay as the caller left them)
    unsigned char *lds = (unsigned char *)pool.place(nullptr, lds_bytes);
    const bool win = t->n_windows > 1;
    const bool coll = (t->flags & ACE_F_COLLECTIVE_MEM) != 0;
    const bool defer = !range && !stage_out && (!win || a.pos_types) && g.N < 32768 && !coll;
    if (defer) a.stage_ws = (double *)pool.place(nullptr, (size_t)P * ACE_MAX_STAGES * ACE_WS_REC * 8);

    if (coll) {
        if (range) { if (win) run_lanes<true, true, true, false, true>(a, lds, lds_bytes); else run_lanes<true, true, false, false, true>(a, lds, lds_bytes); }
        else if (stage_out) { if (win) run_lanes<true, false, true, false, true>(a, lds, lds_bytes); else run_lanes<true, false, false, false, true>(a, lds, lds_bytes); }
        else if (win) run_lanes<false, false, true, false, true>(a, lds, lds_bytes);
        else run_lanes<false, false, false, false, true>(a, lds, lds_bytes);
    }
    else if (range) { if (win) run_lanes<true, true, true, false>(a, lds, lds_bytes); else run_lanes<true, true, false, false>(a, lds, lds_bytes); }
    else if (stage_out) { if (win) run_lanes<true, false, true, false>(a, lds, lds_bytes); else run_lanes<true, false, false, false>(a, lds, lds_bytes); }
    else if (defer && win) run_lanes<false, false, true, true>(a, lds, lds_bytes);
    else if (defer) run_lanes<false, false, false, true>(a, lds, lds_bytes);
    else if (win) run_lanes<false, false, true, false>(a, lds, lds_bytes);
    else run_lanes<false, false, false, false>(a, lds, lds_bytes);

    memcpy(iter_ms, a.iter_ms, (size_t)P * 8);
    memcpy(peak_mb, a.peak_mb, (size_t)P * 8);
    memcpy(feasible, a.feasible, (size_t)P);
    if (status) memcpy(status, a.status, (size_t)P);
    if (stage_out) memcpy(stage_out, a.stage_out, rec_bytes);
    return 0;
}


// ------------------------------------------------------------------------------------------
// The plan-editing kernels (ace_edit_kernels.h) on the CPU, one call per work item, arrays behind
// guard pages as above.  Sizes follow the C ABI's documentation of ace_apply_moves /
// ace_recompute_groups / ace_recompute_select.
// ------------------------------------------------------------------------------------------
extern "C" int ace_emu_apply_moves(const uint8_t *tmpl_codes, const uint32_t *tmpl_hdr, int n_templates, const uint32_t *moves,
                                   long long n, int num_ops, int n_algo, uint8_t *codes_out, uint32_t *hdr_out,
                                   unsigned long long *keys_out) {
    GuardedPool pool;
    const int G = (num_ops + 15) / 16;
    const size_t cb = (size_t)G * 16;
    const ace_u4 *tc = (const ace_u4 *)pool.place(tmpl_codes, (size_t)n_templates * cb);
    const ace_u4 *th = (const ace_u4 *)pool.place(tmpl_hdr, (size_t)n_templates * 16);
    const ace_u4 *mv = (const ace_u4 *)pool.place(moves, (size_t)n * 16);
    ace_u4 *co = (ace_u4 *)pool.place(nullptr, (size_t)n * cb);
    ace_u4 *ho = (ace_u4 *)pool.place(nullptr, (size_t)n * 16);
    unsigned long long *ko = keys_out ? (unsigned long long *)pool.place(keys_out, (size_t)n * 16, 8) : nullptr;
    // (the library launches whole workgroups of 256: ids past n * G must fall out at the first test)
    const unsigned long long total = ((unsigned long long)n * G + 255) / 256 * 256;
    for (unsigned long long id = 0; id < total; ++id)
        apply_moves_body(id, tc, th, n_templates, mv, (unsigned long long)n, G, n_algo == 2 ? 1 : 0, co, ho, ko);
    memcpy(codes_out, co, (size_t)n * cb);
    memcpy(hdr_out, ho, (size_t)n * 16);
    if (keys_out) memcpy(keys_out, ko, (size_t)n * 16);
    return 0;
}

namespace {
struct RcHost {
    GuardedPool pool;
    RcTables k;
    uint8_t *codes;
    size_t code_bytes;
    const int32_t *plan, *lo, *hi, *nsb;
    const uint32_t *mrow;
    RcHost(const ace_rc_tables_t *t, int n, const int32_t *q_plan, const int32_t *q_lo, const int32_t *q_hi, const int32_t *q_nsb,
           const uint32_t *q_mrow) {
        code_bytes = (size_t)((t->num_ops + 15) / 16) * t->n_plans * 16;
        codes = (uint8_t *)pool.place(t->d_codes, code_bytes);
        k = RcTables{codes, (unsigned long long)t->n_plans,
                     (const int32_t *)pool.place(t->d_type_of_pos, (size_t)t->num_ops * 4, 4),
                     (const double *)pool.place(t->d_activations, (size_t)t->num_types * t->n_mbs * t->n_tp * t->n_algo * 8, 8),
                     (const uint8_t *)pool.place(t->d_no_recompute, (size_t)t->num_types, 1),
                     t->num_ops, t->num_types, t->n_mbs, t->n_tp, t->n_algo, t->n_algo == 2 ? 1 : 0};
        plan = (const int32_t *)pool.place(q_plan, (size_t)n * 4, 4);
        lo = (const int32_t *)pool.place(q_lo, (size_t)n * 4, 4);
        hi = (const int32_t *)pool.place(q_hi, (size_t)n * 4, 4);
        nsb = (const int32_t *)pool.place(q_nsb, (size_t)n * 4, 4);
        mrow = (const uint32_t *)pool.place(q_mrow, (size_t)n * 4, 4);
    }
};
}  // namespace

// (same parameter lists as ace_recompute_groups / ace_recompute_select, so a test double can stand in for the library)
extern "C" int ace_emu_rc_groups(const ace_rc_tables_t *t, int n, const int32_t *q_plan, const int32_t *q_lo, const int32_t *q_hi,
                                 const int32_t *q_nsb, const uint32_t *q_mrow, double *sum_size, int32_t *first_pos, int32_t *bad,
                                 void * /*stream*/) {
    RcHost h(t, n, q_plan, q_lo, q_hi, q_nsb, q_mrow);
    const size_t nt = (size_t)n * t->num_types;
    double *sum = (double *)h.pool.place(sum_size, nt * 8, 8);
    int32_t *first = (int32_t *)h.pool.place(first_pos, nt * 4, 4);
    int32_t *b = (int32_t *)h.pool.place(bad, (size_t)n * 4, 4);
    for (int a = 0; a < (n + 127) / 128 * 128; ++a)
        rc_groups_body(a, h.k, n, h.plan, h.lo, h.hi, h.nsb, h.mrow, sum, first, b);
    memcpy(sum_size, sum, nt * 8);
    memcpy(first_pos, first, nt * 4);
    memcpy(bad, b, (size_t)n * 4);
    return 0;
}

// (codes_rw must be t->d_codes, the usual call: the batch is edited in place)
extern "C" int ace_emu_rc_select(const ace_rc_tables_t *t, uint8_t *codes_rw, int n, const int32_t *q_plan, const int32_t *q_lo,
                                 const int32_t *q_hi, const int32_t *q_nsb, const uint32_t *q_mrow, const double *sum_size,
                                 const int32_t *first_pos, uint8_t *recomputed, const double *mem, double memory_limit,
                                 uint8_t *alive, void * /*stream*/) {
    if (codes_rw != t->d_codes) return -1;
    RcHost h(t, n, q_plan, q_lo, q_hi, q_nsb, q_mrow);
    const size_t nt = (size_t)n * t->num_types;
    const double *sum = (const double *)h.pool.place(sum_size, nt * 8, 8);
    const int32_t *first = (const int32_t *)h.pool.place(first_pos, nt * 4, 4);
    uint8_t *done = (uint8_t *)h.pool.place(recomputed, nt, 1);
    const double *m = (const double *)h.pool.place(mem, (size_t)n * 8, 8);
    uint8_t *al = (uint8_t *)h.pool.place(alive, (size_t)n, 1);
    for (int a = 0; a < (n + 127) / 128 * 128; ++a)
        rc_select_body(a, h.k, h.codes, n, h.plan, h.lo, h.hi, h.nsb, h.mrow, sum, first, done, m, memory_limit, al);
    memcpy(codes_rw, h.codes, h.code_bytes);
    memcpy(recomputed, done, nt);
    memcpy(alive, al, (size_t)n);
    return 0;
}

extern "C" int ace_emu_group_keys(const uint8_t *codes /* [G][P][16] */, const uint32_t *hdr, long long n, int num_ops,
                                  unsigned long long *keys) {
    GuardedPool pool;
    const int G = (num_ops + 15) / 16;
    const ace_u4 *c = (const ace_u4 *)pool.place(codes, (size_t)G * n * 16);
    const ace_u4 *h = (const ace_u4 *)pool.place(hdr, (size_t)n * 16);
    unsigned long long *k = (unsigned long long *)pool.place(nullptr, (size_t)n * 8, 8);
    for (unsigned long long p = 0; p < ((unsigned long long)n + 255) / 256 * 256; ++p)
        group_keys_body(p, c, h, (unsigned long long)n, G, num_ops, k);
    memcpy(keys, k, (size_t)n * 8);
    return 0;
}

extern "C" int ace_emu_gather_plans(const uint8_t *codes_in, const uint32_t *hdr_in, const uint32_t *perm, long long n, int num_ops,
                                    uint8_t *codes_out, uint32_t *hdr_out) {
    GuardedPool pool;
    const int G = (num_ops + 15) / 16;
    const ace_u4 *ci = (const ace_u4 *)pool.place(codes_in, (size_t)G * n * 16);
    const ace_u4 *hi = (const ace_u4 *)pool.place(hdr_in, (size_t)n * 16);
    const uint32_t *pm = (const uint32_t *)pool.place(perm, (size_t)n * 4, 4);
    ace_u4 *co = (ace_u4 *)pool.place(nullptr, (size_t)G * n * 16);
    ace_u4 *ho = (ace_u4 *)pool.place(nullptr, (size_t)n * 16);
    const unsigned long long total = ((unsigned long long)n * G + 255) / 256 * 256;
    for (unsigned long long id = 0; id < total; ++id) gather_plans_body(id, ci, hi, pm, (unsigned long long)n, G, co, ho);
    memcpy(codes_out, co, (size_t)G * n * 16);
    memcpy(hdr_out, ho, (size_t)n * 16);
    return 0;
}

