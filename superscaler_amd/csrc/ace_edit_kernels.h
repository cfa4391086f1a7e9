// Kernels that edit or inspect plan bytes (move descriptors -> plans with 128-bit keys; the two
// selection steps of check_recompute's greedy loop), each as a function of its work-item index:
// the __global__ kernels in ace_eval.hip are one-line wrappers, and the host build of the tests
// (ACE_HOST_EMU) runs the same functions on the CPU with guard pages behind every array.
#pragma once
#include "ace_plan_state.h"

#ifdef ACE_HOST_EMU
#define ACE_ATOMIC_XOR(p, v) (*(p) ^= (v))
#else
#define ACE_ATOMIC_XOR(p, v) atomicXor((p), (v))
#endif

// One 64-bit value per (16-byte word, word index): two rounds of the splitmix64 finaliser.
ACE_HD unsigned long long plan_key_word(uint32_t a, uint32_t b, uint32_t c, uint32_t d, uint32_t idx) {
    unsigned long long x = ((unsigned long long)b << 32 | a) + 0x9E3779B97F4A7C15ull * (2ull * idx + 1ull);
    unsigned long long y = ((unsigned long long)d << 32 | c) ^ (x >> 29);
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    x ^= x >> 31;
    y = (y + x) * 0xBF58476D1CE4E5B9ull;
    y = (y ^ (y >> 27)) * 0x94D049BB133111EBull;
    return x ^ y ^ (y >> 31);
}

// The second half of a plan's 128-bit key: the same construction with other odd multipliers.
ACE_HD unsigned long long plan_key_word2(uint32_t a, uint32_t b, uint32_t c, uint32_t d, uint32_t idx) {
    unsigned long long x = ((unsigned long long)d << 32 | b) + 0xD6E8FEB86659FD93ull * (2ull * idx + 1ull);
    unsigned long long y = ((unsigned long long)c << 32 | a) ^ (x >> 31);
    x = (x ^ (x >> 32)) * 0xFF51AFD7ED558CCDull;
    x = (x ^ (x >> 29)) * 0xC4CEB9FE1A85EC53ull;
    x ^= x >> 32;
    y = (y + x) * 0xFF51AFD7ED558CCDull;
    y = (y ^ (y >> 29)) * 0xC4CEB9FE1A85EC53ull;
    return x ^ y ^ (y >> 32);
}

// ------------------------------------------------------------------------------------------
// Move descriptors -> plans: one thread writes one 16-byte word (16 ops) of one neighbour.
// ------------------------------------------------------------------------------------------
ACE_HD void apply_moves_body(unsigned long long id, const ace_u4 *tmpl_codes, const ace_u4 *tmpl_hdr, int n_templates,
                                                          const ace_u4 *moves, unsigned long long n, int G, int a_shift,
                                                          ace_u4 *codes_out, ace_u4 *hdr_out, unsigned long long *key_out) {
    if (id >= n * (unsigned long long)G) return;
    const unsigned long long k = id % n;              // consecutive lanes: consecutive neighbours of one word
    const int g = (int)(id / n);
    const ace_u4 mv = moves[k];
    uint32_t t = mv.x & 0xffffu;
    if (t >= (uint32_t)n_templates) t = 0;
    const uint32_t op = mv.x >> 16;
    const ace_u4 src = tmpl_codes[(size_t)t * G + g];
    if (g == 0) hdr_out[k] = tmpl_hdr[t];
    uint32_t w[4] = {src.x, src.y, src.z, src.w};
    const uint32_t lo16 = mv.y & 0xffffu, hi16 = mv.y >> 16;
    const uint32_t amask = (1u << a_shift) - 1u;      // algo bits of a code
    uint32_t lo = lo16, hi = hi16;                    // byte range [lo, hi) an edit covers
    if (op == 1u) { lo = lo16 < hi16 ? lo16 : hi16; hi = lo16 < hi16 ? hi16 : lo16; }
    if (op == 4u) { lo = lo16; hi = lo16 + 1u; }
    const uint32_t base = (uint32_t)g * 16u;
    const uint32_t hi_touch = op == 1u ? hi + 1u : hi;      // a migration also edits the byte at the far end
    if (op != 0u && lo < base + 16u && hi_touch > base) {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const uint32_t p = base + (uint32_t)j;
            uint32_t b = (w[j >> 2] >> (8 * (j & 3))) & 0xffu;
            const bool in = p >= lo && p < hi;
            if (op == 1u) {                            // migrate: cut = lo16, new cut = hi16, tp = mv.z
                if (p == lo16) b &= 0xEFu;
                if (in) b = ((b & 0xF8u) | ((mv.z << a_shift) + (b & amask))) & 0xffu;
                if (p == hi16) b |= 0x10u;
            } else if (op == 2u) {                     // every op of the stage one tp step up (mv.z = 1) or down
                if (in) {
                    int tp = (int)((b & 7u) >> a_shift) + (mv.z == 1u ? 1 : -1);
                    tp = tp < 0 ? 0 : (tp > 7 ? 7 : tp);
                    b = ((b & 0xF8u) | (((uint32_t)tp << a_shift) + (b & amask))) & 0xffu;
                }
            } else if (op == 3u) {                     // recompute toggle
                if (in) b ^= 8u;
            } else if (op == 4u) {                     // algorithm toggle
                if (in) b ^= 1u;
            }
            w[j >> 2] = (w[j >> 2] & ~(0xffu << (8 * (j & 3)))) | (b << (8 * (j & 3)));
        }
    }
    codes_out[(size_t)g * n + k] = ace_u4{w[0], w[1], w[2], w[3]};
    if (key_out) {
        // 128-bit key of the whole plan, two words per plan: each the XOR of one mixed value per 16-byte word (and one
        // for the header), from two different mixing functions
        unsigned long long hsh = plan_key_word(w[0], w[1], w[2], w[3], (uint32_t)g + 1u);
        unsigned long long hsh2 = plan_key_word2(w[0], w[1], w[2], w[3], (uint32_t)g + 1u);
        if (g == 0) {
            const ace_u4 hh = tmpl_hdr[t];
            hsh ^= plan_key_word(hh.x, hh.y, hh.z, 0u, 0u);      // (the fourth header word follows from the others)
            hsh2 ^= plan_key_word2(hh.x, hh.y, hh.z, 0u, 0u);
        }
        ACE_ATOMIC_XOR(&key_out[2 * k], hsh);
        ACE_ATOMIC_XOR(&key_out[2 * k + 1], hsh2);
    }
}

// ------------------------------------------------------------------------------------------
// check_recompute for encoded stages (aceso_cost_model.py:794-872): the two steps of its greedy
// loop that are not a stage evaluation.  One thread per stage; every sum runs over the stage's ops
// in position order, as the reference's lists do.
// ------------------------------------------------------------------------------------------
struct RcTables {
    const uint8_t *codes;          // [G][P][16], the batch being edited
    unsigned long long P;
    const int32_t *type_of_pos;    // [N]
    const double *act;             // activations [n_types][n_mbs][n_tp][n_algo] (raw table entries, :487-491)
    const uint8_t *norec;          // [n_types] never chosen for recomputation (:798)
    int32_t N, n_types, n_mbs, n_tp, n_algo, a_shift;
};

ACE_HD double rc_act_size(const RcTables &t, unsigned long long plan, int i, uint32_t mrow, int nsb,
                                              int *type_out, int *bad) {
    const uint32_t byte = t.codes[(((size_t)(i >> 4)) * t.P + plan) * 16 + (i & 15)];
    const uint32_t c = byte & 7u, tp = c >> t.a_shift, al = c & (uint32_t)(t.n_algo - 1);
    uint32_t m = (mrow >> (4u * tp)) & 15u;
    if (tp >= (uint32_t)t.n_tp || m >= (uint32_t)t.n_mbs) { *bad = 1; m = 0; }
    int type = t.type_of_pos[i];
    if (type < 0 || type >= t.n_types) { *bad = 1; type = 0; }
    *type_out = type;
    const uint32_t tpc = tp < (uint32_t)t.n_tp ? tp : 0u;
    return t.act[(((size_t)type * t.n_mbs + m) * t.n_tp + tpc) * t.n_algo + al] * (double)(nsb + 1);   // :841
}

// op groups of a stage (:835-843): per op name the sum of the activation sizes and the first position
ACE_HD void rc_groups_body(int a, RcTables t, int n, const int32_t *q_plan, const int32_t *q_lo, const int32_t *q_hi,
                                 const int32_t *q_nsb, const uint32_t *q_mrow, double *sum_size, int32_t *first_pos,
                                 int32_t *bad) {
    if (a >= n) return;
    double *sum = sum_size + (size_t)a * t.n_types;
    int32_t *first = first_pos + (size_t)a * t.n_types;
    int flag = 0;
    const int lo = q_lo[a], hi = q_hi[a];
    if (lo < 0 || hi > t.N || lo >= hi || q_plan[a] < 0 || (unsigned long long)q_plan[a] >= t.P) { bad[a] = 1; return; }
    for (int i = lo; i < hi; ++i) {
        int type;
        const double sz = rc_act_size(t, (unsigned long long)q_plan[a], i, q_mrow[a], q_nsb[a], &type, &flag);
        sum[type] += sz;
        if (i < first[type]) first[type] = i;
    }
    if (flag) bad[a] = 1;
}

// one round of the greedy loop for every stage still above the limit: get_next_recompute_op_group
// (:794-820) and the marking of the chosen ops and their successors (:852-859)
ACE_HD void rc_select_body(int a, RcTables t, uint8_t *codes_rw, int n, const int32_t *q_plan, const int32_t *q_lo,
                                 const int32_t *q_hi, const int32_t *q_nsb, const uint32_t *q_mrow, const double *sum_size,
                                 const int32_t *first_pos, uint8_t *recomputed, const double *mem, double memory_limit,
                                 uint8_t *alive) {
    if (a >= n || !alive[a]) return;
    const double *sum = sum_size + (size_t)a * t.n_types;
    const int32_t *first = first_pos + (size_t)a * t.n_types;
    uint8_t *done = recomputed + (size_t)a * t.n_types;
    // the largest group not yet taken; a tie goes to the op name that appears first in the stage (dict order)
    double best = 0.0;
    int T = -1, best_first = 0x7fffffff;
    for (int ty = 0; ty < t.n_types; ++ty) {
        const double s = sum[ty];
        const int f = first[ty];
        const bool open = !done[ty] && !t.norec[ty] && s > 0.0;
        const bool better = open && (s > best || (s == best && f < best_first));
        best = better ? s : best;
        best_first = better ? f : best_first;
        T = better ? ty : T;
    }
    const int lo = q_lo[a], hi = q_hi[a];
    // (a stage outside the plan: ace_recompute_groups has flagged it; nothing is touched)
    if (lo < 0 || hi > t.N || lo >= hi || q_plan[a] < 0 || (unsigned long long)q_plan[a] >= t.P) { alive[a] = 0; return; }
    if (T < 0) { alive[a] = 0; return; }                       // max_saved_size == 0
    done[T] = 1;
    const int nxt = first[T] + 1;
    if (nxt >= hi || nxt < lo) { alive[a] = 0; return; }        // :805-806
    const int tn = t.type_of_pos[nxt];
    if (tn >= 0 && tn < t.n_types) done[tn] = 1;
    const double exceed = mem[a] - memory_limit;
    const bool all = best < exceed;                              // :809
    const unsigned long long plan = (unsigned long long)q_plan[a];
    double saved = 0.0;
    int dummy = 0;
    for (int i = lo; i < hi; ++i) {
        if (t.type_of_pos[i] != T) continue;
        if (!all) {
            if (!(saved <= exceed)) break;                       // :814
            int type;
            saved += rc_act_size(t, plan, i, q_mrow[a], q_nsb[a], &type, &dummy);
        }
        codes_rw[(((size_t)(i >> 4)) * t.P + plan) * 16 + (i & 15)] |= 8u;
        if (i + 1 < hi) codes_rw[(((size_t)((i + 1) >> 4)) * t.P + plan) * 16 + ((i + 1) & 15)] |= 8u;
    }
}

// ------------------------------------------------------------------------------------------
// Sort key of a plan for grouped storage (ace_batch_t.d_order): pipeline depth (deepest first),
// then the positions of its first two stage boundaries.  One work item per plan.
// ------------------------------------------------------------------------------------------
ACE_HD void group_keys_body(unsigned long long p, const ace_u4 *codes, const ace_u4 *hdr, unsigned long long n, int G, int N,
                            unsigned long long *keys) {
    if (p >= n) return;
    const uint32_t S = hdr[p].x & 0xffu;
    uint32_t cut[2] = {0u, 0u};
    int found = 0;
    for (int g = 0; g < G && found < 2; ++g) {
        const ace_u4 w = codes[(size_t)g * n + p];
        const uint32_t words[4] = {w.x, w.y, w.z, w.w};
        for (int k = 0; k < 16 && found < 2; ++k) {
            const int i = g * 16 + k;
            if (i == 0 || i >= N) continue;                 // (the first op opens stage 0; padding bytes do not count)
            if ((words[k >> 2] >> (8 * (k & 3))) & 0x10u) cut[found++] = (uint32_t)i;
        }
    }
    // (positions are below 2^20: move descriptors and the kernels' range checks keep N under 65536 * 16)
    keys[p] = ((unsigned long long)(255u - S) << 40) | ((unsigned long long)(cut[0] & 0xfffffu) << 20) | (cut[1] & 0xfffffu);
}

// Reorder a batch: slot i of the output holds plan perm[i] of the input.  One work item per 16-byte
// word (16 ops of one plan); consecutive items write consecutive words.
ACE_HD void gather_plans_body(unsigned long long id, const ace_u4 *codes_in, const ace_u4 *hdr_in, const uint32_t *perm,
                              unsigned long long n, int G, ace_u4 *codes_out, ace_u4 *hdr_out) {
    if (id >= n * (unsigned long long)G) return;
    const unsigned long long i = id % n;
    const int g = (int)(id / n);
    unsigned long long src = perm[i];
    if (src >= n) src = i;                        // (not a permutation entry: the plan stays where it is)
    codes_out[(size_t)g * n + i] = codes_in[(size_t)g * n + src];
    if (g == 0) hdr_out[i] = hdr_in[src];
}
