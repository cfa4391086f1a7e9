// Bounds-checked CPU build of the per-plan state machine (superscaler_amd/csrc/ace_plan_state.h)
// -- TEST INFRASTRUCTURE ONLY.  It lets the CPU test-suite run the exact source the GPU kernel
// is made of (same header, compiled with ACE_HOST_EMU) against the oracle, with every "LDS"
// access checked for range and alignment, before anything is launched on a GPU.  The product
// library never links or loads this file.
#define ACE_HOST_EMU 1
#include "ace_plan_state.h"

#include <vector>

namespace {

template <bool BD, bool RANGED, bool DEFER = false>
void score_one(const ace_tables_t *t, const AceGeom &g, std::vector<unsigned char> &lds, uint32_t lds_bytes,
               const uint8_t *codes, ace_u4 h, ace_u2 range, double *rec, double &iter, double &peak, uint8_t &feas,
               uint8_t &st) {
    const size_t row_bytes = (size_t)t->row_doubles * 8;
    const uint32_t *pos = t->pos_info;
    AceLds view{lds.data(), lds_bytes};
    PlanState<BD, RANGED, DEFER> s;
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
        const int n_st = s.s;
        for (int s2 = 0; s2 < n_st && s2 < ACE_MAX_STAGES; ++s2) s.replay(g, view, pos, rec, s2);
        s.s = n_st;              // replay() walks s again; result() checks the count of the op loop
    }
    s.result(g, t->nb_minus_1[s.bidx], iter, peak, feas, st);
}

}  // namespace

extern "C" int ace_emu_score(const ace_tables_t *t, const uint8_t *codes /* [P][N] plan-major */,
                             const uint32_t *hdr /* [P][4] */, const uint32_t *range /* nullable [P][2] */,
                             long long P, double memory_limit, int strict, int defer, double *iter_ms, double *peak_mb,
                             uint8_t *feasible, uint8_t *status, double *stage_out /* nullable [P][16][18] */) {
    const int C = t->n_tp * t->n_algo;
    AceGeom g;
    memset(&g, 0, sizeof(g));
    g.N = t->num_ops; g.P = (int32_t)P; g.G = (t->num_ops + 15) / 16;
    g.C = C; g.A_shift = t->n_algo == 2 ? 1 : 0;
    g.n_mbs = t->n_mbs; g.n_tp = t->n_tp; g.n_algo = t->n_algo; g.n_glog = t->n_glog; g.n_pair_kinds = t->n_pair_kinds;
    g.hot_off = t->hot_off * 8u; g.start_off = t->start_off * 8u; g.out_off = t->out_off * 8u; g.z_off = t->z_off * 8u;
    g.z_shift = 3;
    while ((1 << (g.z_shift - 3)) < t->z_table_doubles) ++g.z_shift;
    const int32_t rk_bytes = t->n_pair_kinds * t->n_glog * 64;
    g.rk_lds_off = (uint32_t)t->lds_row_bytes;
    g.stg_lds_off = (g.rk_lds_off + (uint32_t)rk_bytes + 15u) & ~15u;
    g.rk_kind_stride = (uint32_t)(t->n_glog * 64);
    g.row_bytes = (uint32_t)t->row_doubles * 8u;
    const uint32_t lds_bytes = g.stg_lds_off + (uint32_t)t->n_mbs * 16u * 4u;
    g.flags = t->flags; g.main_params = t->main_params; g.optimizer = t->optimizer;
    g.mem_limit = memory_limit; g.strict = strict ? 1 : 0;
    if (range && !stage_out) return -1;

    std::vector<unsigned char> lds(lds_bytes);
    for (long long p = 0; p < P; ++p) {
        memset(lds.data(), 0xff, lds.size());
        memcpy(lds.data() + g.rk_lds_off, t->pair_kinds, rk_bytes);
        memcpy(lds.data() + g.stg_lds_off, t->stage_lut, (size_t)t->n_mbs * 16 * 4);
        ace_u4 h;
        memcpy(&h, hdr + 4 * p, 16);
        ace_u2 rg{0u, 0u};
        if (range) memcpy(&rg, range + 2 * p, 8);
        double *rec = stage_out ? stage_out + (size_t)p * ACE_MAX_STAGES * ACE_STAGE_REC : nullptr;
        const uint8_t *c = codes + (size_t)p * g.N;
        double iter, peak;
        uint8_t feas, st;
        if (range) score_one<true, true>(t, g, lds, lds_bytes, c, h, rg, rec, iter, peak, feas, st);
        else if (stage_out) score_one<true, false>(t, g, lds, lds_bytes, c, h, rg, rec, iter, peak, feas, st);
        else if (defer && t->n_windows == 1) score_one<false, false, true>(t, g, lds, lds_bytes, c, h, rg, rec, iter, peak, feas, st);
        else score_one<false, false>(t, g, lds, lds_bytes, c, h, rg, rec, iter, peak, feas, st);
        iter_ms[p] = iter; peak_mb[p] = peak; feasible[p] = feas;
        if (status) status[p] = st;
    }
    return 0;
}
