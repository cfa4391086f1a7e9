// The scoring kernel's op loop, as a function of (workgroup, lane): the GPU kernel in ace_eval.hip
// is a one-line wrapper around ace_score_body(), and a host build (ACE_HOST_EMU, one lane per
// "workgroup") runs the very same loop on the CPU with every array behind guard pages, so that an
// index error shows up as a host fault in the CPU test-suite instead of a memory fault on the GPU.
#pragma once
#include "ace_plan_state.h"

#ifdef ACE_HOST_EMU
#define ACE_SYNC() ((void)0)
#define ACE_ANY(x) (x)
#else
#define ACE_SYNC() __syncthreads()
#define ACE_ANY(x) __any(x)
#endif

#ifndef ACE_HOST_EMU
#include "ace_score_loop_asm.inc"
#endif

struct AceKernelArgs {
    AceGeom g;
    const ace_u4 *codes;        // [G][P] 16 op bytes each
    const ace_u4 *hdr;          // [P]
    const ace_u2 *range;        // [P] (first op, one past the last op) or null
    const uint32_t *order;      // [P] result index of the plan in each slot, or null (slot i -> result i)
    const double *rows;         // [n_types][row_doubles]
    const uint32_t *pos_info;   // [N + 1], padded to 16 * G + 16 entries
    const uint32_t *pos_types;  // windowed rows: the same with each row's index in `rows` in place of its LDS slot (null: more than 256 rows)
    const ace_u4 *pos4;         // [16 * G + 16] per position: LDS address of its row's hot sub-table, of its cost tables, of the
                                //   32-bit pair-kind block of the (this, next) pair; bit 0: no layer start follows an ordinary op here, bit 1: ordinary op,
                                //   bits 8-15 / 16-23: this op's / the next op's row as the evaluation of the stage tails indexes rows
    const uint8_t *pair_kinds;  // -> LDS
    const uint32_t *stage_lut;  // -> LDS
    const double *nbm1;         // [n_mbs]
    const int32_t *win_pos;     // [n_windows + 1], multiples of 4
    const int32_t *win_row_begin;
    const uint32_t *win_rows;   // pairs (type, lds byte offset)
    const ace_u4 *win_dma;      // what the assembly op loop stages the windows from (see ace_score_loop_asm), or null
    int32_t n_windows, row_doubles, rk_bytes, stg_words;
    int32_t flat_rows16;        // rows resident and laid out in LDS as they lie in `rows`: their size in 16-byte pieces (else 0)
    double *iter_ms, *peak_mb;
    uint8_t *feasible, *status;
    double *stage_out;          // [P][ACE_MAX_STAGES][ACE_STAGE_REC], single-stage queries [P][ACE_STAGE_REC]
    double *stage_ws;           // [workgroup][ACE_MAX_STAGES][lanes of a workgroup][ACE_WS_REC] for deferred stage tails
};

// Windowed rows: the position descriptors (pos_info) with each row's index in `rows` where its LDS slot is (and the next
// position's where that one's is); positions past the last op read zero.  (Host side: what the library uploads as AceKernelArgs::pos_types.)
inline void ace_pos_types(const ace_tables_t *t, uint32_t *out, size_t entries) {
    const uint32_t row_bytes = (uint32_t)t->row_doubles * 8u;
    int w = 0;
    for (size_t i = 0; i < entries; ++i) {
        out[i] = 0u;
        if (i >= (size_t)t->num_ops) continue;
        while (w + 1 < t->n_windows && (size_t)t->win_pos[w + 1] <= i) ++w;
        const uint32_t info = t->pos_info[i], slot_off = (info & 0xffu) * row_bytes;
        uint32_t type = 0;
        for (int r = t->win_row_begin[w]; r < t->win_row_begin[w + 1]; ++r)
            if (t->win_rows[2 * r + 1] == slot_off) type = t->win_rows[2 * r];
        out[i] = (info & 0xffff0000u) | type;
    }
    // ... and the index of the next position's row in bits 8 to 15 (the last op: its own)
    for (size_t i = 0; i < entries && i < (size_t)t->num_ops; ++i)
        out[i] |= ((i + 1 < (size_t)t->num_ops ? out[i + 1] : out[i]) & 0xffu) << 8;
}

// Rows resident and laid out in LDS as they lie in global memory: one block copy with every lane busy, four loads in
// flight per lane (row by row, a lane has one load at a time and most lanes none).  The first four loads of a lane are
// asked for before the workgroup sorts its plans (stage_rows_first) and written after it (the sort's scratch space is
// where the rows go).
struct AceRowsFirst { ace_d2 v[4]; };
template <int BLOCK> ACE_HD AceRowsFirst stage_rows_first(const AceKernelArgs &a, int tid) {
    const ace_d2 *src = reinterpret_cast<const ace_d2 *>(a.rows);
    const int n = a.flat_rows16;
    AceRowsFirst f;
#pragma unroll
    for (int k = 0; k < 4; ++k) f.v[k] = tid + k * BLOCK < n ? src[tid + k * BLOCK] : ace_d2{0.0, 0.0};
    return f;
}
template <int BLOCK> ACE_HD void stage_rows_flat(const AceKernelArgs &a, unsigned char *lds_raw, int tid, const AceRowsFirst &f) {
    const ace_d2 *src = reinterpret_cast<const ace_d2 *>(a.rows);
    ace_d2 *dst = reinterpret_cast<ace_d2 *>(lds_raw);
    const int n = a.flat_rows16;
#pragma unroll
    for (int k = 0; k < 4; ++k)
        if (tid + k * BLOCK < n) dst[tid + k * BLOCK] = f.v[k];
    int j = tid + 4 * BLOCK;
    for (; j + 3 * BLOCK < n; j += 4 * BLOCK) {
        const ace_d2 v0 = src[j], v1 = src[j + BLOCK], v2 = src[j + 2 * BLOCK], v3 = src[j + 3 * BLOCK];
        dst[j] = v0; dst[j + BLOCK] = v1; dst[j + 2 * BLOCK] = v2; dst[j + 3 * BLOCK] = v3;
    }
    for (; j < n; j += BLOCK) dst[j] = src[j];
}

// Copy the rows window `w` needs from global memory into LDS (whole workgroup).
template <int BLOCK> ACE_HD void stage_window(const AceKernelArgs &a, unsigned char *lds_raw, int w, int tid) {
    const int rb = a.win_row_begin[w], re = a.win_row_begin[w + 1];
    const int n16 = a.row_doubles / 2;
    for (int r = rb; r < re; ++r) {
        const uint32_t type = a.win_rows[2 * r], off = a.win_rows[2 * r + 1];
        const ace_d2 *src = reinterpret_cast<const ace_d2 *>(a.rows + (size_t)type * a.row_doubles);
        ace_d2 *dst = reinterpret_cast<ace_d2 *>(lds_raw + off);
        for (int j = tid; j < n16; j += BLOCK) dst[j] = src[j];
    }
}

#ifndef ACE_HOST_EMU
// The op loop of the plain scoring kernel in gfx950 assembly (ace_score_loop_asm.inc; written by
// gen_score_loop_asm.py, which describes it): walks all ops of this lane's plan, parks every finished stage in the
// lane's workspace records like PlanState::stash(), and returns the number of stages closed.  LDS addresses in `pos4`
// are absolute: the caller checks that the workgroup's LDS array starts at address 0.
// WIN: the rows are windowed; the loop fetches its windows itself, from the records of a.win_dma (80 bytes per fetch
// event and wavefront, sixteen wavefronts: see the generator).
template <bool WIN>
__device__ __forceinline__ uint32_t ace_score_loop_asm(const AceKernelArgs &a, const AceGeom &g, uint64_t glogs, uint32_t lut2_lane,
                                                       uint32_t code_off, const double *rec_base, uint32_t rec_off, uint32_t ws_stride,
                                                       uint32_t prio, uint32_t wave) {
    uint32_t wsoff;         // the lane's record offset after the loop: rec_off + ws_stride * (stages closed)
    const uint64_t gstride = (uint64_t)(uint32_t)g.P * 16u;
    const uint32_t gs_lo = (uint32_t)gstride, gs_hi = (uint32_t)(gstride >> 32);
    const uint32_t pace = g.pace_lds_off + (wave & 3u) * 32u;     // this SIMD's eight arrival counters
    if (WIN) {
#define ACE_LOOP_ASM_RUN(TEXT)                                                                                          \
    asm volatile(TEXT : [wsoff] "=&v"(wsoff)                                                                               \
                 : [glogs] "v"(glogs), [lut2] "v"(lut2_lane), [codeoff] "v"(code_off), [recoff] "v"(rec_off),          \
                   [codes] "s"(a.codes), [pos] "s"(a.pos4), [n_ops] "s"(g.N), [recbase] "s"(rec_base), \
                   [gstride_lo] "s"(gs_lo), [gstride_hi] "s"(gs_hi), [wsstride] "s"(ws_stride), [prio] "s"(prio),       \
                   [dma] "s"(a.win_dma), [waveoff] "s"(wave * 80u)                                                      \
                 : ACE_LOOP_ASM_CLOBBERS)
        if (g.flags & ACE_F_RESHARDING) {
            if (g.flags & ACE_F_NO_RESERVED) ACE_LOOP_ASM_RUN(ACE_LOOP_ASM_WIN_RSH1_NONE);
            else if (g.flags & ACE_F_RESERVED_MIN) ACE_LOOP_ASM_RUN(ACE_LOOP_ASM_WIN_RSH1_MIN);
            else ACE_LOOP_ASM_RUN(ACE_LOOP_ASM_WIN_RSH1_MAX);
        } else {
            if (g.flags & ACE_F_NO_RESERVED) ACE_LOOP_ASM_RUN(ACE_LOOP_ASM_WIN_RSH0_NONE);
            else if (g.flags & ACE_F_RESERVED_MIN) ACE_LOOP_ASM_RUN(ACE_LOOP_ASM_WIN_RSH0_MIN);
            else ACE_LOOP_ASM_RUN(ACE_LOOP_ASM_WIN_RSH0_MAX);
        }
#undef ACE_LOOP_ASM_RUN
        return (wsoff - rec_off) / ws_stride;
    }
#define ACE_LOOP_ASM_RUN(TEXT)                                                                                          \
    asm volatile(TEXT : [wsoff] "=&v"(wsoff)                                                                               \
                 : [glogs] "v"(glogs), [lut2] "v"(lut2_lane), [codeoff] "v"(code_off), [recoff] "v"(rec_off),          \
                   [codes] "s"(a.codes), [pos] "s"(a.pos4), [n_ops] "s"(g.N), [recbase] "s"(rec_base), \
                   [gstride_lo] "s"(gs_lo), [gstride_hi] "s"(gs_hi), [wsstride] "s"(ws_stride),                         \
                   [pace] "s"(pace)                                                                                     \
                 : ACE_LOOP_ASM_CLOBBERS)
    if (g.flags & ACE_F_RESHARDING) {
        if (g.flags & ACE_F_NO_RESERVED) ACE_LOOP_ASM_RUN(ACE_LOOP_ASM_RSH1_NONE);
        else if (g.flags & ACE_F_RESERVED_MIN) ACE_LOOP_ASM_RUN(ACE_LOOP_ASM_RSH1_MIN);
        else ACE_LOOP_ASM_RUN(ACE_LOOP_ASM_RSH1_MAX);
    } else {
        if (g.flags & ACE_F_NO_RESERVED) ACE_LOOP_ASM_RUN(ACE_LOOP_ASM_RSH0_NONE);
        else if (g.flags & ACE_F_RESERVED_MIN) ACE_LOOP_ASM_RUN(ACE_LOOP_ASM_RSH0_MIN);
        else ACE_LOOP_ASM_RUN(ACE_LOOP_ASM_RSH0_MAX);
    }
#undef ACE_LOOP_ASM_RUN
    return (wsoff - rec_off) / ws_stride;
}
#endif

// BD: also write per-stage records.  RANGED: each plan is one stage over an op sub-range.
// WIN: the rows of all op types do not fit in LDS together; restage at window boundaries.
// DEFER: stage tails are stashed in the workspace and evaluated after the op loop, when all lanes
// are active again (together with WIN the boundary lookups of that evaluation read the rows in global memory,
// a.pos_types naming each position's row there).
// `tid` lane of workgroup `block` of `n_blocks`, BLOCK lanes each; `lds_raw`: the workgroup's LDS (`lds_bytes` long).
template <bool BD, bool RANGED, bool WIN, bool DEFER, int BLOCK, bool COLL = false>
ACE_HD void ace_score_body(const AceKernelArgs &a, unsigned char *lds_raw, uint32_t lds_bytes, int tid, long long block,
                           uint32_t n_blocks) {
    static_assert(!DEFER || (!BD && !RANGED && !COLL), "deferred stage tails: plain scoring only");
    // region offsets as absolute LDS addresses for the reads (see AceLds); the staging loops below
    // write through `lds_raw` with the plain offsets of a.g
    AceGeom g = a.g;
    const uint32_t lds_base = ace_lds_base(lds_raw);
    g.hot_off += lds_base; g.start_off += lds_base; g.out_off += lds_base; g.z_off += lds_base;
    g.rk_lds_off += lds_base; g.stg_lds_off += lds_base; g.lut2_lds_off += lds_base;
    if (g.lut2a_lds_off) g.lut2a_lds_off += lds_base;
    const long long slot = block * BLOCK + tid;                     // this lane's place in the batch (and in the workspace)
    AceRowsFirst rows_first;
    const bool flat = !WIN && a.flat_rows16 > 0;
    if (flat) rows_first = stage_rows_first<BLOCK>(a, tid);
    long long plan = slot;
    uint32_t prio = 0;                                              // issue priority of this wavefront in the op loop
#ifndef ACE_HOST_EMU
    if (!RANGED && BLOCK >= 128) {
        // The lanes of a wavefront walk the ops together, and every op at which one of them closes a stage takes all
        // of them through the stage-end code: so the workgroup deals its plans to its lanes by pipeline depth
        // (counting sort on the depth in the plan header, deepest first; plans of one depth in any order), and the
        // sorted wavefronts to the SIMDs in turn (wavefront w runs on SIMD w % 4) so that each SIMD gets the same
        // mix.  The wavefronts with the deeper plans get the higher issue priority: they have the most instructions
        // to issue and would otherwise be the last to finish, alone on their SIMDs.  Only which lane scores which
        // plan changes: results go to the plan's own index.  (Single-stage queries are left as they come: their
        // length, not a depth, is what would have to be sorted on.)
        unsigned int *cnt = reinterpret_cast<unsigned int *>(lds_raw);                  // 17 bins (nothing is staged yet)
        unsigned short *plan_of = reinterpret_cast<unsigned short *>(lds_raw + 128);     // [BLOCK]
        uint32_t depth = 0;                                                              // lanes past the batch: last
        if (slot < g.P) {
            depth = a.hdr[slot].x & 0xffu;
            depth = depth > 16u ? 16u : depth;
        }
        if (tid < 32) cnt[tid] = 0u;
        ACE_SYNC();
        const uint32_t rank = atomicAdd(&cnt[16u - depth], 1u);
        ACE_SYNC();
        uint32_t before = 0;
        for (uint32_t b = 0; b < 16u - depth; ++b) before += cnt[b];
        const uint32_t sorted = before + rank;
        // sorted wavefront q goes to wavefront q of the workgroup in rows of four, every second row reversed
        const uint32_t q = sorted >> 6;
        const uint32_t wave = (q & 4u) ? (q ^ 3u) : q;
        plan_of[(wave << 6) | (sorted & 63u)] = (unsigned short)tid;
        ACE_SYNC();
        plan = block * BLOCK + plan_of[tid];
        if (BLOCK >= 1024) {
            const uint32_t pw = (uint32_t)tid >> 6, qs = (pw & 4u) ? (pw ^ 3u) : pw;       // the sorted slice this wavefront walks
            prio = __builtin_amdgcn_readfirstlane(3u - (qs >> 2));
        }
        ACE_SYNC();
    }
#endif
    const bool in_batch = plan < g.P;
    const long long pl = in_batch ? plan : (long long)g.P - 1;      // plan this lane reads
    // where this lane's results go; a slot whose entry is not a valid index computes but writes nothing
    const long long out = a.order ? (long long)a.order[pl] : plan;
    const bool active = in_batch && out < g.P;

    // RANGED: the workgroup walks only the 16-op groups that hold an op of one of its queries (a single-stage
    // query covers a fraction of the sequence, and the walk is what such a call waits for)
    ace_u2 range{0u, 0u};
    int grp_begin = 0, grp_end = g.G;
    if (RANGED) {
        range = a.range[pl];
        // (what PlanState::init() makes of a malformed range)
        const bool ok = range.x < range.y && range.y <= (uint32_t)g.N;
        uint32_t lo = ok ? range.x : 0u, hi = ok ? range.y : 1u;
#ifndef ACE_HOST_EMU
        unsigned int *red = reinterpret_cast<unsigned int *>(lds_raw);     // two words, before anything is staged there
        if (tid == 0) { red[0] = 0xffffffffu; red[1] = 0u; }
        ACE_SYNC();
        atomicMin(&red[0], lo);
        atomicMax(&red[1], hi);
        ACE_SYNC();
        lo = red[0];
        hi = red[1];
        ACE_SYNC();
#endif
        grp_begin = (int)(lo >> 4);
        grp_end = (int)((hi + 15u) >> 4);
    }
    // the window that holds the first position walked
    int w0 = 0;
    if (RANGED && WIN)
        while (w0 + 1 < a.n_windows && a.win_pos[w0 + 1] <= (grp_begin << 4)) ++w0;

    // this lane's plan header and its first sixteen op bytes: asked for before the tables are staged, used after
    const ace_u4 h = a.hdr[pl];
    ace_u4 cw = a.codes[(size_t)grp_begin * g.P + pl];

    // small tables: pair kinds and the (micro-batch, stage gpus) LUT; without windows, every row
    // (four pair kinds per lane and turn: the table is a multiple of 64 bytes)
    for (int j = tid; j < (a.rk_bytes >> 2); j += BLOCK) {
        const uint32_t r4 = reinterpret_cast<const uint32_t *>(a.pair_kinds)[j];
        reinterpret_cast<uint32_t *>(lds_raw + a.g.rk_lds_off)[j] = r4;
        if (DEFER && a.g.pk32_lds_off) {
            uint32_t e[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t r = (r4 >> (8 * q)) & 0xffu;
                e[q] = ((r & 15u) << a.g.z_shift) | (((r >> 4) << a.g.z_shift) << 16);
            }
            // (entries 4j .. 4j + 3 of block j / 16; the blocks are ACE_PK32_BLOCK words apart)
            uint32_t *dst = reinterpret_cast<uint32_t *>(lds_raw + a.g.pk32_lds_off) + (4 * j + (j >> 4) * (int)(ACE_PK32_BLOCK - 64u));
#pragma unroll
            for (int q = 0; q < 4; ++q) dst[q] = e[q];
        }
    }
    for (int j = tid; j < a.stg_words; j += BLOCK) {
        const uint32_t w = a.stage_lut[j];
        reinterpret_cast<uint32_t *>(lds_raw + a.g.stg_lds_off)[j] = w;
        // entry j = micro-batch index * 16 + log2(stage size): byte offset of the stage's diag inside the cost sub-tables,
        // and the pair-kind block of the stage size relative to it (what PlanState::start_fast hands to the op loop)
        const uint32_t glog = (uint32_t)j & 15u;
        const uint32_t z_v = (w & 15u) * (uint32_t)a.g.C * 8u;
        const uint32_t gl = glog < (uint32_t)a.g.n_glog ? glog : 0u, rk = gl << 6;
        reinterpret_cast<ace_u2 *>(lds_raw + a.g.lut2_lds_off)[j] = ace_u2{z_v, rk - z_v};
        // (the assembly loop adds the pair-kind block offset to the op pair's own index, not to the diag's, and its blocks
        // are ACE_PK32_BLOCK words apart)
        if (DEFER && a.g.lut2a_lds_off) reinterpret_cast<ace_u2 *>(lds_raw + a.g.lut2a_lds_off)[j] = ace_u2{z_v, gl * ACE_PK32_BLOCK};
    }
    // (the assembly op loop over windowed rows fetches its windows itself, in a layout of its own)
#ifndef ACE_HOST_EMU
    const bool asm_loop = DEFER && lds_base == 0u && a.pos4 && a.g.lut2a_lds_off && (!WIN || (BLOCK == 1024 && a.win_dma));
#else
    const bool asm_loop = false;
#endif
    if (DEFER && a.g.pace_lds_off && tid < 32) reinterpret_cast<uint32_t *>(lds_raw + a.g.pace_lds_off)[tid] = 0u;
    if (flat) stage_rows_flat<BLOCK>(a, lds_raw, tid, rows_first);
    else if (!(WIN && asm_loop)) stage_window<BLOCK>(a, lds_raw, w0, tid);       // every row, or the first window's
    ACE_SYNC();

    AceLds lds = ace_make_lds(lds_raw, lds_bytes);
    lds.grows = reinterpret_cast<const unsigned char *>(a.rows);
    PlanState<BD, RANGED, DEFER, COLL, DEFER && WIN> st;
    st.init(g, lds, h, range);
    st.row_ids = a.pos_types;
    const double nbm1 = a.nbm1[st.bidx];
    // (a single-stage query has one record, a whole plan one per possible stage)
    const size_t rec_doubles = RANGED ? (size_t)ACE_STAGE_REC : (size_t)(ACE_MAX_STAGES * ACE_STAGE_REC);
    double *rec = (BD && a.stage_out && active) ? a.stage_out + (size_t)out * rec_doubles : nullptr;
    if (DEFER) {
        // per workgroup, stage-major: the records of one stage of the workgroup's lanes are adjacent (padded lanes own
        // a slot too), the sixteen stages of a workgroup follow each other
        rec = a.stage_ws + ((size_t)block * ACE_MAX_STAGES * BLOCK + (size_t)tid) * ACE_WS_REC;
        st.ws_stride = (uint32_t)BLOCK * (ACE_WS_REC / 2);
    }

    int w = w0 + 1;
    int next_win = WIN ? a.win_pos[w] : 0x7fffffff;
    const uint32_t first_code = cw.x & 7u;
    int grp_stop = grp_end;
#ifndef ACE_HOST_EMU
    if (asm_loop) {
        // the assembly form of the loop below (same operations per plan, same results)
        if (!(cw.x & 0x10u)) st.status = ACE_PLAN_MALFORMED;    // the first op must open a stage
        // (the loop looks each stage's offsets up in LDS, by the stage size's log2)
        st.s = (int)ace_score_loop_asm<WIN>(a, g, st.glogs, g.lut2a_lds_off + st.bidx * 128u, (uint32_t)pl * 16u,
                                            a.stage_ws + (size_t)block * ACE_MAX_STAGES * BLOCK * ACE_WS_REC,
                                            (uint32_t)tid * (ACE_WS_REC * 8u), (uint32_t)BLOCK * (ACE_WS_REC * 8u), prio,
                                            (uint32_t)__builtin_amdgcn_readfirstlane(tid >> 6));
        grp_stop = grp_begin;
    } else
#endif
    if (!RANGED) st.begin(g, lds, 0, cw.x & 0xffu, a.pos_info[0]);
    uint32_t pinfo = grp_begin ? a.pos_info[(grp_begin << 4) - 1] : 0u;    // descriptor of the previous group's last position
    for (int grp = grp_begin; grp < grp_stop; ++grp) {
        const int base = grp << 4;
        // the sixteen position descriptors of this group: scalar loads (the array is padded)
        const ace_u4 *ip = reinterpret_cast<const ace_u4 *>(a.pos_info + base);
        const ace_u4 i0 = ip[0], i1 = ip[1], i2 = ip[2], i3 = ip[3];
        const uint32_t infos[16] = {i0.x, i0.y, i0.z, i0.w, i1.x, i1.y, i1.z, i1.w,
                                    i2.x, i2.y, i2.z, i2.w, i3.x, i3.y, i3.z, i3.w};
        ace_u4 nxt = ace_u4{0u, 0u, 0u, 0u};
        if (grp + 1 < g.G) nxt = a.codes[(size_t)(grp + 1) * g.P + pl];
        uint32_t words[5] = {cw.x, cw.y, cw.z, cw.w, nxt.x};
        if (DEFER) {
            // whatever the caller left in the bytes past the last op reads as zero
#pragma unroll
            for (int j = 0; j < 5; ++j) {
                const int left = g.N - (base + 4 * j);          // code bytes of this word that belong to the plan
                words[j] &= left >= 4 ? 0xffffffffu : (left <= 0 ? 0u : ((1u << (8 * left)) - 1u));
            }
        }
        // pair_bit() of the sixteen (op, next op) pairs, four at a time: bit 0 of each byte
        uint32_t pairs[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t nw = (words[j] >> 8) | (words[j + 1] << 24);      // the next-op bytes of word j
            pairs[j] = ((words[j] & nw) >> 3) & ~(nw >> 4) & 0x01010101u;
        }
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            const int i = base + k;
            if (WIN && (k & 3) == 0 && i == next_win && w < a.n_windows) {
                // every lane of the workgroup reaches this point together (w < n_windows: the loop also
                // walks the padding positions of the last group, which must never restage)
                ACE_SYNC();
                stage_window<BLOCK>(a, lds_raw, w, tid);
                ACE_SYNC();
                ++w;
                next_win = a.win_pos[w];
            }
            // DEFER: positions past the last op are processed too (zeroed code bytes, padded descriptors):
            // the last stage was stashed at op N - 1, what follows lands in a stage nobody reads
            if (DEFER || i < g.N) {
                const uint32_t byte = (words[k >> 2] >> (8 * (k & 3))) & 0xffu;
                // (past the last op the code bytes are zero padding)
                const uint32_t nbyte = (words[(k + 1) >> 2] >> (8 * ((k + 1) & 3))) & 0xffu;
                const uint32_t pair = (pairs[k >> 2] >> (8 * (k & 3))) & 1u;
                st.step(g, lds, i, byte, nbyte, pair, infos[k], k ? infos[k - 1] : pinfo, i + 1 == g.N, rec);
            }
        }
        pinfo = infos[15];
        cw = nxt;
    }
    if (DEFER) {
        const int n_st = st.s;
        if (WIN) {
            // (row offsets as the rows lie in global memory)
            AceGeom gr = g;
            gr.start_off -= lds_base; gr.out_off -= lds_base;
            gr.row_bytes = (uint32_t)a.row_doubles * 8u;
            st.replay_all(gr, lds, rec, n_st, first_code, a.pos_types[0] & 0xffu);
        } else
            st.replay_all(g, lds, rec, n_st, first_code, a.pos_info[0] & 0xffu);
    }
    double iter, peak;
    uint8_t feas, stat;
    st.result(g, nbm1, iter, peak, feas, stat);
    if (active) {
        a.iter_ms[out] = iter;
        a.peak_mb[out] = peak;
        a.feasible[out] = feas;
        if (a.status) a.status[out] = stat;
    }
}
