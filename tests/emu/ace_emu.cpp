// Bounds-checked CPU build of the per-plan state machine (superscaler_amd/csrc/ace_plan_state.h)
// -- TEST INFRASTRUCTURE ONLY.  It lets the CPU test-suite run the exact source the GPU kernel
// is made of (same header, compiled with ACE_HOST_EMU) against the oracle, with every "LDS"
// access checked for range and alignment, before anything is launched on a GPU.  The product
// library never links or loads this file.
#define ACE_HOST_EMU 1
#include "ace_plan_state.h"

#include <vector>

extern "C" int ace_emu_score(const ace_tables_t *t, const uint8_t *codes /* [P][N] plan-major */,
                             const uint32_t *hdr /* [P][4] */, long long P, double memory_limit, int strict,
                             double *iter_ms, double *peak_mb, uint8_t *feasible, uint8_t *status,
                             double *stage_out /* nullable [P][16][18] */) {
    const int C = t->n_tp * t->n_algo;
    AceGeom g;
    memset(&g, 0, sizeof(g));
    g.N = t->num_ops; g.P = (int32_t)P; g.G = (t->num_ops + 15) / 16;
    g.C = C; g.A_shift = t->n_algo == 2 ? 1 : 0;
    g.n_mbs = t->n_mbs; g.n_tp = t->n_tp; g.n_algo = t->n_algo; g.n_glog = t->n_glog; g.n_pair_kinds = t->n_pair_kinds;
    g.hot_off = t->hot_off * 8u; g.start_off = t->start_off * 8u; g.out_off = t->out_off * 8u; g.z_off = t->z_off * 8u;
    g.z_stride = (uint32_t)(t->n_diag * C) * 8u;
    const int32_t rk_bytes = t->n_pair_kinds * t->n_glog * C * C;
    g.rk_lds_off = (uint32_t)t->lds_row_bytes;
    g.stg_lds_off = (g.rk_lds_off + (uint32_t)rk_bytes + 15u) & ~15u;
    const uint32_t lds_bytes = g.stg_lds_off + (uint32_t)t->n_mbs * 16u * 4u;
    g.flags = t->flags; g.main_params = t->main_params; g.optimizer = t->optimizer;
    g.mem_limit = memory_limit; g.strict = strict ? 1 : 0;
    const size_t row_bytes = (size_t)t->row_doubles * 8;

    std::vector<unsigned char> lds(lds_bytes);
    const ace_u4 *pos = reinterpret_cast<const ace_u4 *>(t->pos_info);
    for (long long p = 0; p < P; ++p) {
        // poison the row region so that a read of a row the window did not stage is caught as NaN
        memset(lds.data(), 0xff, lds.size());
        memcpy(lds.data() + g.rk_lds_off, t->pair_kinds, rk_bytes);
        memcpy(lds.data() + g.stg_lds_off, t->stage_lut, (size_t)t->n_mbs * 16 * 4);
        AceLds view{lds.data(), lds_bytes};
        ace_u4 h;
        memcpy(&h, hdr + 4 * p, 16);
        double *rec = stage_out ? stage_out + (size_t)p * ACE_MAX_STAGES * ACE_STAGE_REC : nullptr;
        int w = 0, next_win = t->win_pos[0];
        double iter, peak;
        uint8_t feas, st;
        if (stage_out) {
            PlanState<true> s;
            s.init(g, view, h);
            for (int i = 0; i < g.N; ++i) {
                if (i == next_win) {
                    memset(lds.data(), 0xff, t->lds_row_bytes);
                    for (int r = t->win_row_begin[w]; r < t->win_row_begin[w + 1]; ++r)
                        memcpy(lds.data() + t->win_rows[2 * r + 1], t->rows + (size_t)t->win_rows[2 * r] * t->row_doubles, row_bytes);
                    next_win = t->win_pos[++w];
                }
                s.step(g, view, codes[p * g.N + i], pos[i], rec);
            }
            s.finish(g, view, pos[g.N].y, rec);
            s.result(g, t->nb_minus_1[s.bidx], iter, peak, feas, st);
        } else {
            PlanState<false> s;
            s.init(g, view, h);
            for (int i = 0; i < g.N; ++i) {
                if (i == next_win) {
                    memset(lds.data(), 0xff, t->lds_row_bytes);
                    for (int r = t->win_row_begin[w]; r < t->win_row_begin[w + 1]; ++r)
                        memcpy(lds.data() + t->win_rows[2 * r + 1], t->rows + (size_t)t->win_rows[2 * r] * t->row_doubles, row_bytes);
                    next_win = t->win_pos[++w];
                }
                s.step(g, view, codes[p * g.N + i], pos[i], nullptr);
            }
            s.finish(g, view, pos[g.N].y, nullptr);
            s.result(g, t->nb_minus_1[s.bidx], iter, peak, feas, st);
        }
        iter_ms[p] = iter; peak_mb[p] = peak; feasible[p] = feas; if (status) status[p] = st;
    }
    return 0;
}
