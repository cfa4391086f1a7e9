// Per-plan scoring state machine of the batched Aceso plan evaluator.
//
// One instance scores one plan, op by op, in op order, with exactly the floating-point
// operations (and their association) of the reference's search/aceso_cost_model.py, so the
// results are bit-identical to the reference's Python floats:
//   begin()   head of the first stage
//   step()    one op: get_time_v3 sums (:307-313), resharding of the (previous, this) op pair
//             (:340-350), get_recompute_time_v3 (:365-371), get_memory_v3 (:382-392),
//             get_activations_v3 (:403-415), get_peak_activations (:428-445),
//             get_reserved_memory maxima (:453-460)
//   start_fast() / start_lookups()  stage head: per-stage lookup offsets; boundary input size /
//             p2p time (:319-331)
//   stash() / replay_all()  deferred stage tails: a finished stage's accumulators are parked in a
//             workspace and its tail is evaluated after the op loop
//   finish()  stage tail: output p2p (:321-336), stage time (:352-353, :579), stage memory
//             (predict_stage_memory :514-539, get_reserved_memory :480-483), running
//             sum / max for the 1F1B composition (:613-619)
//   result()  iteration time max_s(t_s*(nb-1) + sum t) and peak memory
//
// The same source is compiled by hipcc for gfx950 (one plan per lane, tables in LDS) and by
// g++ with ACE_HOST_EMU for a bounds-checked CPU build used only by tests.
#pragma once
#include <stdint.h>

#include "ace_eval.h"

#ifdef ACE_HOST_EMU
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#define ACE_HD inline
#define ACE_WAVE_ANY(x) (x)
struct AceLds {
    const unsigned char *base;
    uint32_t size;
    const unsigned char *grows = nullptr;     // the table rows as the caller holds them (behind the caller's guard pages)
    template <class T> T gld(uint32_t off) const {
        T v;
        memcpy(&v, grows + off, sizeof(T));
        return v;
    }
    template <class T> T ld(uint32_t off) const {
        if ((uint64_t)off + sizeof(T) > size || (off % (sizeof(T) > 16 ? 16 : sizeof(T))) != 0) {
            fprintf(stderr, "ace emu: LDS access out of bounds/misaligned: off=%u size=%zu lds=%u\n", off, sizeof(T), size);
            abort();
        }
        T v;
        memcpy(&v, base + off, sizeof(T));
        return v;
    }
};
static inline AceLds ace_make_lds(const unsigned char *base, uint32_t size) { return AceLds{base, size}; }
static inline uint32_t ace_lds_base(const unsigned char *) { return 0u; }   // host: offsets from `base`
static inline double ace_max(double a, double b) { return a > b ? a : b; }
#else
#define ACE_HD __device__ __forceinline__
#define ACE_WAVE_ANY(x) __any(x)
// LDS reads take the absolute LDS byte address.  The address of the workgroup's LDS array is a
// link-time constant (zero when the kernel has no other LDS variables) that the compiler cannot fold
// while it compiles; left inside per-lane address arithmetic it costs two or three vector
// instructions per op.  ace_lds_base() exposes it as a number, and the caller adds it to the
// wave-uniform region offsets once (scalar arithmetic), so per-lane address math never sees it.
struct AceLds {
    const unsigned char *grows;     // the table rows in global memory (replay of deferred stage tails over windowed rows)
    template <class T> ACE_HD T gld(uint32_t off) const {
        T v;
        __builtin_memcpy(&v, grows + off, sizeof(T));
        return v;
    }
    template <class T> ACE_HD T ld(uint32_t addr) const {
#if defined(__HIP_DEVICE_COMPILE__)
        typedef const unsigned char __attribute__((address_space(3))) *lptr;
        T v;
        __builtin_memcpy(&v, (lptr)(uintptr_t)addr, sizeof(T));
        return v;
#else
        (void)addr;
        return T{};             // (the host pass of the GPU build never runs this)
#endif
    }
};
ACE_HD AceLds ace_make_lds(const unsigned char *, uint32_t) { return AceLds{nullptr}; }
ACE_HD uint32_t ace_lds_base(const unsigned char *lds) {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef const unsigned char __attribute__((address_space(3))) *lptr;
    return (uint32_t)(uintptr_t)(lptr)lds;
#else
    (void)lds;
    return 0u;
#endif
}
// One v_max_f64.  fmax() makes the compiler quiet both operands first (two more instructions);
// table values are never signalling NaNs, and a NaN operand only occurs in plans that are
// reported as unscorable anyway.
ACE_HD double ace_max(double a, double b) {
    double r;
    asm("v_max_f64 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
#endif
ACE_HD bool ace_isnan(double a) { return a != a; }
// product of two values below 2^24 (a single full-rate instruction on the GPU)
#ifdef ACE_HOST_EMU
ACE_HD uint32_t ace_mul24(uint32_t a, uint32_t b) { return a * b; }
ACE_HD uint32_t ace_mad24(uint32_t a, uint32_t b, uint32_t c) { return a * b + c; }
ACE_HD double ace_fma(double a, double b, double c) { return std::fma(a, b, c); }
#else
ACE_HD uint32_t ace_mul24(uint32_t a, uint32_t b) { return __umul24(a, b); }
ACE_HD uint32_t ace_mad24(uint32_t a, uint32_t b, uint32_t c) {
    uint32_t r = __umul24(a, b) + c;
    asm("" : "+v"(r));          // one v_mad_u32_u24; without this the sum is re-associated into three instructions
    return r;
}
ACE_HD double ace_fma(double a, double b, double c) { return __builtin_fma(a, b, c); }
#endif
// 1.0 or 0.0 from a wave-uniform flag, built from integer words so that it stays in scalar registers
ACE_HD double ace_scalar_01(bool one) {
    uint32_t hi = one ? 0x3ff00000u : 0u;
#ifndef ACE_HOST_EMU
    asm("" : "+s"(hi));         // keeps the compiler from turning the product below into per-lane selects
#endif
    const uint64_t bits = (uint64_t)hi << 32;
    double d;
    __builtin_memcpy(&d, &bits, 8);
    return d;
}

struct alignas(16) ace_d2 { double x, y; };
struct alignas(16) ace_u4 { uint32_t x, y, z, w; };
struct alignas(8) ace_u2 { uint32_t x, y; };

#define ACE_HOT_STRIDE 48u     // bytes per (diag, code) entry of the hot sub-table
#define ACE_START_STRIDE 24u    // ... of the start sub-table: input MB, input / intra-node bandwidth, input / inter-node bandwidth

// Geometry and constants every lane reads (kernel arguments -> scalar registers).
struct AceGeom {
    int32_t N, P, G;            // ops, plans, 16-op groups
    int32_t C, A_shift;         // codes per diag (n_tp * n_algo), log2(n_algo)
    int32_t n_mbs, n_tp, n_algo, n_glog, n_pair_kinds;
    uint32_t hot_off, start_off, out_off, z_off;   // bytes inside a row
    uint32_t z_shift;           // log2(bytes of one resharding-cost table inside a row)
    uint32_t zm_delta;          // bytes from a cost table to the memory table of the same collective (ACE_F_COLLECTIVE_MEM)
    uint32_t rk_lds_off, stg_lds_off;              // LDS byte offsets of the pair-kind and stage LUT regions
    uint32_t lut2_lds_off;                         // ... of the per-(micro-batch, stage size) offset pairs (see ace_lds_layout)
    uint32_t pk32_lds_off;                         // ... of the pair-kind table in the assembly loop's form (0: LDS has no room for it)
    uint32_t pace_lds_off;                         // ... of the 4 x 8 arrival counters the assembly loop paces its wavefronts by
    uint32_t lut2a_lds_off;                        // ... of the assembly loop's own offset pairs (the block offset not relative; 0: none)
    uint32_t rk_kind_stride;    // bytes of one pair kind (n_glog * 64)
    uint32_t row_bytes;         // bytes of one op type's row
    int32_t flags;
    double main_params, optimizer, mem_limit;
    int32_t strict;
};

// position descriptor (wave-uniform), one word: bits 0-7 LDS slot of the op's row, 8-15 slot of the
// next op's row (while this op's window is resident), 16-23 kind of the (this op, next op) pair,
// bit 24: this is an ordinary op followed by a layer start, bit 25: this is an ordinary op
ACE_HD uint32_t info_row(const AceGeom &g, uint32_t i) { return (i & 0xffu) * g.row_bytes; }
ACE_HD uint32_t info_nextrow(const AceGeom &g, uint32_t i) { return ((i >> 8) & 0xffu) * g.row_bytes; }

#define ACE_PK32_BLOCK 65u      // words from one 64-entry block of the 32-bit pair-kind table to the next
#define ACE_WS_REC 10          // doubles per deferred stage record (see PlanState::stash)

// LDS regions behind the resident rows: pair kinds | stage LUT (one word per (micro-batch, stage size)) | per
// (micro-batch, stage size) two words: byte offset of the stage's diag inside the cost sub-tables, and the pair-kind block
// offset relative to it.  Returns the total LDS size.
#ifdef ACE_HOST_EMU
inline
#else
__host__ __device__ inline
#endif
uint32_t ace_lds_layout(uint32_t rk_off, uint32_t rk_bytes, uint32_t stg_words, uint32_t *stg_off, uint32_t *lut2_off) {
    *stg_off = (rk_off + rk_bytes + 15u) & ~15u;
    *lut2_off = (*stg_off + stg_words * 4u + 15u) & ~15u;
    return *lut2_off + stg_words * 8u;
}
// The assembly form of the op loop reads the pair kinds as 32-bit entries (one per byte of the table above: byte offset
// of the forward collective's cost table | that of the backward collective's << 16), placed behind everything else.
// Every block of 64 entries (one stage size of one pair kind) is followed by one unused entry: a block of 64 words
// spans all 64 LDS banks, and the lanes of a wavefront differ in their stage sizes, so without it lanes with the same
// (code, next code) and different stage sizes would read different words of one bank (ACE_PK32_BLOCK words per block).
#ifdef ACE_HOST_EMU
inline
#else
__host__ __device__ inline
#endif
uint32_t ace_lds_pk32(uint32_t lds_end, uint32_t rk_bytes, uint32_t *pk32_off) {
    *pk32_off = (lds_end + 15u) & ~15u;
    return *pk32_off + (rk_bytes / 64u) * ACE_PK32_BLOCK * 4u;
}

// COLL: consider_collective_memory (the tables carry ACE_F_COLLECTIVE_MEM).
// BD: per-stage records for the caller.  RANGED: one stage over an op sub-range.  DEFER: stage
// tails are not evaluated where the stage ends (where only the few lanes that cut at this op are
// active) but stashed to a per-plan workspace and replayed after the op loop with every lane busy.
// GROWS (with DEFER): the rows are windowed, so the evaluation of the stashed stages looks the stage boundaries up in
// the rows' global copy (its caller passes the geometry with row offsets as they are there).
template <bool BD, bool RANGED, bool DEFER = false, bool COLL = false, bool GROWS = false> struct PlanState {
    template <class T> ACE_HD static T row_ld(const AceLds &lds, uint32_t a) {
        if (GROWS) return lds.template gld<T>(a);
        return lds.template ld<T>(a);
    }

    // plan constants
    int S;
    uint32_t bidx;
    uint64_t glogs;
    uint32_t cross;
    uint32_t ideal_hot_v, ideal_start_v;
    int lo, hi;                 // RANGED: only ops lo <= i < hi belong to the plan (one stage)
    // stage state
    int s;
    uint32_t z_v, rk_v, mrow, dc_v;     // rk_v: pair-kind block offset of the stage MINUS z_v (see start_fast)
    uint32_t t_first;
    bool out_cross;
    double in_comm, inputs, id_in;
    // per-op accumulators (reset at every stage head)
    double fwd, bwd, rcs, W, A, saved, run, peak, rfm, rbm, rs_f, rs_b, mc;
    double id_fwd, id_bwd;
    bool lastclose;
    uint32_t replay_row;        // DEFER: row of the first op of the stage the replay decodes next (stages follow each other) ...
    uint32_t replay_code;       // ... and its code
    const uint32_t *row_ids;    // DEFER over windowed rows: per position, what stash() takes as `ids` (else the position's descriptor has them)
    uint64_t rk_all;            // per stage (4 bits each): the stage size as the pair-kind tables index it
    uint64_t diag_next, rk_next;   // diags / rk_all shifted down by the stages handed out so far
    uint32_t ws_stride;         // DEFER: 16-byte units between two stages of one plan in the workspace
    uint32_t ws_off;            // DEFER: 16-byte units from the plan's first slot to the slot of the current stage (fits: see ensure_stage_ws)
    uint64_t glogs_next;        // DEFER: glogs shifted down by the stages handed out so far
    uint32_t lut2_lane;         // DEFER: LDS address of the offset pairs of this plan's micro-batch size
    uint64_t diags;             // the diag of every stage, 4 bits each, looked up once per plan
    uint32_t r_next;            // collective ids of the (previous op, this op) pair, fetched one op ahead
    uint32_t pair_prev;         // pair_bit of the (previous op, this op) pair
    // plan accumulators
    double sum_t, max_t, max_mem;
    uint32_t status;

    ACE_HD void init(const AceGeom &g, const AceLds &lds, ace_u4 h, ace_u2 range) {
        S = (int)(h.x & 0xff);
        bidx = (h.x >> 8) & 0xff;
        glogs = (uint64_t)h.y | ((uint64_t)h.z << 32);
        cross = h.w;
        lo = RANGED ? (int)range.x : 0;
        hi = RANGED ? (int)range.y : g.N;
        s = -1;
        sum_t = 0.0; max_t = 0.0; max_mem = 0.0;
        status = 0;
        lastclose = false; replay_row = 0; replay_code = 0; r_next = 0; pair_prev = 0; row_ids = nullptr;
        ws_stride = ACE_WS_REC / 2;
        ws_off = 0;
        fwd = bwd = rcs = W = A = saved = run = peak = rfm = rbm = rs_f = rs_b = mc = 0.0;
        id_fwd = id_bwd = id_in = 0.0;
        in_comm = inputs = 0.0;
        z_v = rk_v = mrow = t_first = dc_v = 0;
        out_cross = false;
        ideal_hot_v = ideal_start_v = 0;
        if (bidx >= (uint32_t)g.n_mbs) { status = ACE_PLAN_MALFORMED; bidx = 0; }
        if (RANGED && (lo < 0 || hi > g.N || lo >= hi)) { status = ACE_PLAN_MALFORMED; lo = 0; hi = 1; }
        diags = 0;
        glogs_next = glogs;
        lut2_lane = g.lut2_lds_off + bidx * 128u;
        rk_all = 0; diag_next = 0; rk_next = 0;
        if (!DEFER) {
            // one LUT read per possible stage now, none where a stage begins (where few lanes are active)
            uint64_t rks = 0;
            stage_nibbles(g, lds, diags, rks);
            rewind(rks);
        }
        if (BD) {
            // the "ideal" pass uses tp = dp = 1 and micro-batch = micro_bs (aceso_cost_model.py:588-590):
            // the diag of (micro_bs, 1 gpu)
            uint32_t d = lds.ld<uint32_t>(g.stg_lds_off + (bidx * 16u + 0u) * 4u) & 15u;
            ideal_hot_v = ace_mul24(d, (uint32_t)g.C * ACE_HOT_STRIDE);
            ideal_start_v = ace_mul24(d, (uint32_t)g.C * ACE_START_STRIDE);
        }
    }

    // Per stage, four bits each (stage 0 lowest): the diag of the stage's (micro-batch, stage size) pair, and the stage
    // size as the pair-kind tables index it (a size outside the tables is unscorable anyway: block 0).
    ACE_HD void stage_nibbles(const AceGeom &g, const AceLds &lds, uint64_t &dg, uint64_t &rks) const {
        dg = 0; rks = 0;
        for (uint32_t k = 0; k < ACE_MAX_STAGES; ++k) {
            uint32_t glog = (uint32_t)(glogs >> (4u * k)) & 15u;
            uint32_t w = lds.ld<uint32_t>(g.stg_lds_off + (bidx * 16u + glog) * 4u);
            dg |= (uint64_t)(w & 15u) << (4u * k);
            rks |= (uint64_t)(glog < (uint32_t)g.n_glog ? glog : 0u) << (4u * k);
        }
    }

    // Start handing out the per-stage nibbles from stage 0 again (init; before the replay of stashed stages).
    ACE_HD void rewind(uint64_t rks) {
        rk_all = rks;
        diag_next = diags;
        rk_next = rks;
    }

    // Stage head, part 1: the per-stage offsets the op loop needs, accumulators back to zero.
    // `tail`: also what only finish() uses (one LDS read).
    ACE_HD void start_fast(const AceGeom &g, const AceLds &lds, bool tail) {
        ++s;
        if (DEFER) {
            // the op loop's two offsets of the next stage are READ, as one pair of words per (micro-batch, stage size): where
            // a stage ends a lane or two are active, but every vector instruction costs the whole wavefront an issue slot
            const uint32_t glog = (uint32_t)glogs_next & 15u;      // (past the sixteenth stage: zero, and result() refuses such a plan)
            glogs_next >>= 4;
            const ace_u2 zz = lds.ld<ace_u2>(lut2_lane + glog * 8u);
            z_v = zz.x;
            rk_v = zz.y;
            fwd = bwd = rcs = W = A = saved = run = peak = rfm = rbm = rs_f = rs_b = mc = 0.0;
            lastclose = false;
            r_next = 0;
            return;
        }
        // the next stage's nibbles sit at the bottom of diag_next / rk_next (stages come in order; past
        // the sixteenth they read zero, and such a plan is caught by result())
        const uint32_t d = (uint32_t)diag_next & 15u;
        const uint32_t rk = (uint32_t)rk_next & 15u;
        diag_next >>= 4;
        rk_next >>= 4;
        z_v = ace_mul24(d, (uint32_t)g.C * 8u);
        rk_v = (rk << 6) - z_v;      // relative to z_v, so that the op loop adds the same `zc` to both bases
        if (tail) {
            const uint32_t glog = (uint32_t)(glogs >> (4u * ((uint32_t)s & 15u))) & 15u;
            dc_v = ace_mul24(d, (uint32_t)g.C);
            mrow = lds.ld<uint32_t>(g.stg_lds_off + (bidx * 16u + glog) * 4u) >> 16;
        }
        fwd = bwd = rcs = W = A = saved = run = peak = rfm = rbm = rs_f = rs_b = mc = 0.0;
        lastclose = false;
        r_next = 0;             // a stage's first op pays no resharding
    }

    // Stage head, part 2: boundary input of the stage's first op (code `c`, row at LDS offset `row`).
    ACE_HD void start_lookups(const AceGeom &g, const AceLds &lds, uint32_t row, uint32_t c) {
        uint32_t sidx = (uint32_t)s & 15u;
        bool in_cross = (cross >> sidx) & 1u;
        out_cross = (cross >> (16u + sidx)) & 1u;
        t_first = c >> g.A_shift;
        uint32_t a = row + g.start_off + (dc_v + c) * ACE_START_STRIDE;
        inputs = row_ld<double>(lds, a);                                 // input size
        in_comm = row_ld<double>(lds, a + (in_cross ? 16u : 8u));        // size / inter- or intra-node bandwidth
        if (BD) {
            uint32_t ai = row + g.start_off + ideal_start_v + (c & (uint32_t)(g.n_algo - 1)) * ACE_START_STRIDE;
            id_in = lds.ld<double>(ai + (in_cross ? 16u : 8u));
            id_fwd = 0.0; id_bwd = 0.0;
        }
    }

    // The reserved-memory term of a stage (get_reserved_memory :480-483 with max_collective = 0).
    ACE_HD double reserved_term(const AceGeom &g) const {
        // (mc: the largest collective buffer, :480-483; without COLL the reference adds its integer 0)
        const double coll = COLL ? mc : 0.0;
        if (g.flags & ACE_F_NO_RESERVED) return 0.0;
        if (g.flags & ACE_F_RESERVED_MIN) return ace_max(ace_max(rfm, rbm), ace_max(W, coll));
        // (the sum below is never -0.0, so adding the reference's integer 0 would change nothing)
        return COLL ? ace_max(rfm + rbm, W) + coll : ace_max(rfm + rbm, W);
    }

    // DEFER: park the finished stage in the plan's workspace slot `s`: ten values in five 16-byte
    // stores (a store from a lane or two costs as much as one from sixty-four, so what can be
    // folded here without a table lookup is: fwd + bwd, the closed peak segment, the reserved term).
    // `ids`: row of the stage's last op | row of the op after it << 8, as replay's lookups index rows (LDS slots; for
    // windowed rows their indices in global memory).
    ACE_HD void stash(const AceGeom &g, double *ws, uint32_t i_last, uint32_t c_last, uint32_t c_next, bool prev_ordinary,
                      uint32_t ids) {
        if (ws == nullptr || s < 0 || s >= ACE_MAX_STAGES) return;
        // stages are stashed in order, once each: slot s of this plan is ws_off further on (a running
        // offset instead of s * ws_stride, which would be a slow 32-bit multiply per stage end)
        ace_d2 *r = reinterpret_cast<ace_d2 *>(ws) + ws_off;
        ws_off += ws_stride;
        // what the replay needs besides the sums.  Low word: code of the stage's last op * 8 + code of the op after it
        // (the next stage's first) in byte (position % 4); the other bytes are not read (the assembly form of the loop
        // stores its whole word of such bytes).  High word: position of the last op (16 bits) | ids << 16.
        uint64_t meta = ((uint64_t)((i_last & 0xffffu) | (ids << 16)) << 32) |
                        (uint64_t)(((c_last << 3) | c_next) << (8u * (i_last & 3u)));
        double meta_d;
        __builtin_memcpy(&meta_d, &meta, 8);
        const double fb = fwd + bwd;                                    // the first sum of :579
        // :439: max(peak, run) if the (previous op, last op) pair closes the last segment, i.e. if that pair is a
        // recompute pair and the previous op an ordinary one.  `run` is 0.0 unless that pair is a recompute pair
        // that continued the segment, so the wave-uniform half of the condition is all that has to be applied.
        const double peakc = ace_max(peak, run * ace_scalar_01(prev_ordinary));
        r[0] = ace_d2{fb, rcs}; r[1] = ace_d2{rs_f, rs_b}; r[2] = ace_d2{W, A}; r[3] = ace_d2{saved, peakc};
        r[4] = ace_d2{reserved_term(g), meta_d};
    }

    // DEFER: the evaluation of the stashed stages, in three steps per stage so that the caller can have the loads of
    // later stages in flight while it evaluates an earlier one: replay_load (the record), replay_lookups (decodes it
    // and reads the stage's boundary entries), replay_finish.  Stages in order; before stage 0, replay_code holds the
    // code of the plan's first op and replay_row the row of that op.
    struct Record { ace_d2 r[5]; };
    struct Lookups { double inputs, in_comm; ace_d2 oe; uint32_t lut, c_first, c_last; };

    ACE_HD void replay_load(const double *ws, int s2, Record &rec) const {
        // (every plan owns ACE_MAX_STAGES slots)
        const int sl = s2 < ACE_MAX_STAGES ? s2 : ACE_MAX_STAGES - 1;
        const ace_d2 *p = reinterpret_cast<const ace_d2 *>(ws) + (size_t)((uint32_t)sl * ws_stride);
#pragma unroll
        for (int j = 0; j < 5; ++j) rec.r[j] = p[j];
    }

    // `live`: the plan has a stage s2 (else the record is whatever the slot held: entry 0 of row 0 is looked up, and
    // the chain of first ops stays as it is).
    ACE_HD void replay_lookups(const AceGeom &g, const AceLds &lds, const Record &rec, int s2, bool live, Lookups &L) {
        uint64_t meta;
        __builtin_memcpy(&meta, &rec.r[4].y, 8);
        const uint32_t hi = (uint32_t)(meta >> 32);
        const uint32_t cc = ((uint32_t)meta >> (8u * (hi & 3u))) & 63u;
        uint32_t row_first = replay_row, row_last = (hi >> 16) & 0xffu;
        L.c_first = replay_code & 7u;
        L.c_last = cc >> 3;
        if (live) {
            replay_row = hi >> 24;
            replay_code = cc & 7u;
        } else {
            row_first = 0; row_last = 0; L.c_first = 0; L.c_last = 0;
        }
        const uint32_t sidx = (uint32_t)s2 & 15u;
        const uint32_t glog = (uint32_t)(glogs >> (4u * sidx)) & 15u;
        L.lut = lds.ld<uint32_t>(g.stg_lds_off + (bidx * 16u + glog) * 4u);
        const bool in_cross = (cross >> sidx) & 1u;
        const uint32_t dc = ace_mul24(L.lut & 15u, (uint32_t)g.C);
        const uint32_t a = row_first * g.row_bytes + g.start_off + (dc + L.c_first) * ACE_START_STRIDE;
        L.inputs = row_ld<double>(lds, a);                                  // input size
        L.in_comm = row_ld<double>(lds, a + (in_cross ? 16u : 8u));         // size / inter- or intra-node bandwidth
        L.oe = row_ld<ace_d2>(lds, out_entry_addr(g, row_last * g.row_bytes, L.c_last, L.c_first >> g.A_shift, L.lut >> 16));
    }

    // (the record and the looked-up values into the stage state: after this `rec` may be overwritten)
    ACE_HD void replay_take(const AceGeom &g, const Record &rec, const Lookups &L, int s2) {
        s = s2;
        dc_v = ace_mul24(L.lut & 15u, (uint32_t)g.C);
        mrow = L.lut >> 16;
        out_cross = (cross >> (16u + ((uint32_t)s2 & 15u))) & 1u;
        t_first = L.c_first >> g.A_shift;
        inputs = L.inputs;
        in_comm = L.in_comm;
        // finish_tail() recombines: (fb + 0) = fb; the peak is closed already; max(reserved + 0, W) = reserved
        fwd = rec.r[0].x; bwd = 0.0; rcs = rec.r[0].y; rs_f = rec.r[1].x; rs_b = rec.r[1].y; W = rec.r[2].x; A = rec.r[2].y;
        saved = rec.r[3].x; peak = rec.r[3].y; run = 0.0; lastclose = false; rfm = rec.r[4].x; rbm = 0.0;
    }

    // All stashed stages of a plan of n_st stages whose first op has code `code0` and row `row0`.  The records come from
    // memory (they were written up to a whole op loop ago) and waiting for them is most of what this costs: three are
    // in flight per lane (record s + 3 is asked for when stage s is taken), in three sets of registers used in turn;
    // a stage's boundary entries are looked up when its turn comes (LDS is idle by then).
    ACE_HD void replay_all(const AceGeom &g, const AceLds &lds, const double *ws, int n_st, uint32_t code0, uint32_t row0) {
        replay_code = code0;
        replay_row = row0;
        Record r[3];
        replay_load(ws, 0, r[0]);
        r[1] = r[0];
        r[2] = r[0];
        if (1 < n_st) replay_load(ws, 1, r[1]);
        if (2 < n_st) replay_load(ws, 2, r[2]);
        for (int base = 0; base < ACE_MAX_STAGES; base += 3) {
#pragma unroll
            for (int k = 0; k < 3; ++k) {
                const int s2 = base + k;
                if (!ACE_WAVE_ANY(s2 < n_st)) goto replayed;
                const bool live = s2 < n_st;
                Lookups lx;
                replay_lookups(g, lds, r[k], s2, live, lx);
                if (live) replay_take(g, r[k], lx, s2);
                // (only lanes that have the stage fetch it: the slot of a stage a plan does not have may never have been written)
                if (s2 + 3 < n_st) replay_load(ws, s2 + 3, r[k]);
                if (live) finish_tail(g, lds, 0u, lx.c_last, lx.oe, nullptr);
            }
        }
    replayed:
        s = n_st;               // (the evaluation walked s again; result() checks the count of the op loop)
    }

    // Address of output_size[ops[-1]][mbs[-1]][tp[0]][algo[-1]] (sic, aceso_cost_model.py:321-326) in the row at `lastrow`:
    // `c_last` the last op's code, `tf` the tp index of the stage's first op, `mr` the stage's row of micro-batch indices.
    ACE_HD static uint32_t out_entry_addr(const AceGeom &g, uint32_t lastrow, uint32_t c_last, uint32_t tf, uint32_t mr) {
        const uint32_t t_last = c_last >> g.A_shift;
        const uint32_t a_last = c_last & (uint32_t)(g.n_algo - 1);
        uint32_t m_last = (mr >> (4u * t_last)) & 15u;
        if (m_last >= (uint32_t)g.n_mbs) m_last = 0;   // only for plans whose sums are NaN already
        const uint32_t oidx = ((m_last * (uint32_t)g.n_tp + tf) << g.A_shift) + a_last;
        return lastrow + g.out_off + oidx * 16u;
    }

    // Stage tail; `lastrow` is the LDS offset of the row of the stage's last op, `c_last` its code.
    ACE_HD void finish(const AceGeom &g, const AceLds &lds, uint32_t lastrow, uint32_t c_last, double *rec) {
        const ace_d2 oe = row_ld<ace_d2>(lds, out_entry_addr(g, lastrow, c_last, t_first, mrow));
        finish_tail(g, lds, lastrow, c_last, oe, rec);
    }

    // ... with the output entry `oe` looked up already.
    ACE_HD void finish_tail(const AceGeom &g, const AceLds &lds, uint32_t lastrow, uint32_t c_last, ace_d2 oe, double *rec) {
        uint32_t a_last = c_last & (uint32_t)(g.n_algo - 1);
        double out_comm = out_cross ? oe.y : oe.x;
        double in_c = in_comm + rs_f * 1000.0;      // :352
        double out_c = out_comm + rs_b * 1000.0;    // :353
        double t = ((((fwd + bwd) + in_c) + out_c) + rcs) / 1000.0;   // :579
        sum_t += t;
        max_t = ace_max(max_t, t);
        if (lastclose) peak = ace_max(peak, run);   // :439 "i + 1 == len(ops) - 1" closes the last segment
        const double reserved = reserved_term(g);
        double mp = W * g.main_params;
        double opt = W * g.optimizer;
        double x = (inputs + A) - saved;
        double nsb = (double)(S - 1 - s);
        double mem_act = x * nsb;                   // :530
        double mem_peak = x + peak;                 // :531
        double wts = W + mp;                        // :533
        double mem = ((((wts + W) + opt) + mem_act) + mem_peak) + reserved;   // :534
        max_mem = ace_max(max_mem, mem);
        if (BD && rec != nullptr && s >= 0 && s < ACE_MAX_STAGES) {
            double *r = rec + (size_t)s * ACE_STAGE_REC;
            r[ACE_R_FWD] = fwd; r[ACE_R_BWD] = bwd; r[ACE_R_IN_COMM] = in_c; r[ACE_R_OUT_COMM] = out_c;
            r[ACE_R_RECOMP] = rcs; r[ACE_R_WEIGHTS] = W; r[ACE_R_INPUTS] = inputs; r[ACE_R_ACT] = A;
            r[ACE_R_SAVED] = saved; r[ACE_R_PEAK] = peak; r[ACE_R_RESERVED] = reserved;
            // ideal pass: output_size[ops[-1]][mbs index of micro_bs][tp index 0][algo[-1]]
            uint32_t iidx = ((bidx * (uint32_t)g.n_tp + 0u) << g.A_shift) + a_last;
            ace_d2 ie = lds.ld<ace_d2>(lastrow + g.out_off + iidx * 16u);
            r[ACE_R_IDEAL_FWD] = id_fwd; r[ACE_R_IDEAL_BWD] = id_bwd; r[ACE_R_IDEAL_IN] = id_in;
            r[ACE_R_IDEAL_OUT] = out_cross ? ie.y : ie.x;
            r[ACE_R_STAGE_MS] = t; r[ACE_R_STAGE_MB] = mem;
            r[ACE_R_RESHARD] = rs_f * 1000.0 + rs_b * 1000.0;   // print-only "reshard" column (:355)
        }
    }

    // Head of the plan's first stage (RANGED: of the queried stage); `byte` / `info` belong to its first op.
    ACE_HD void begin(const AceGeom &g, const AceLds &lds, int i, uint32_t byte, uint32_t info) {
        if (!(byte & 0x10u)) status = ACE_PLAN_MALFORMED;    // the first op must open a stage
        start_fast(g, lds, !DEFER);
        if (!DEFER) start_lookups(g, lds, info_row(g, info), byte & 7u);
    }

    // One op at position i.  `byte` is its code byte, `nbyte` the next op's (0 after the last op, where `plan_end` is set instead),
    // `pair` = pair_bit(byte, nbyte), `info` / `pinfo` this and the previous position's (wave-uniform) descriptors.  Everything that concerns the (this op, next op)
    // pair is handled here too, so nothing but the accumulators is carried from op to op; a stage
    // that ends with this op is closed (and the next one opened) in the middle of the step.
    ACE_HD void step(const AceGeom &g, const AceLds &lds, int i, uint32_t byte, uint32_t nbyte, uint32_t pair,
                     uint32_t info, uint32_t pinfo, bool plan_end, double *rec) {
        if (RANGED) {
            if (i < lo || i >= hi) return;
            if (i == lo) begin(g, lds, i, byte, info);
        }
        const uint32_t c = byte & 7u;
        const uint32_t nc = nbyte & 7u;
        const bool rc = (byte >> 3) & 1u;
        const uint32_t row = info_row(g, info);
        // entry index inside the diag's block, in 8-byte units: the hot entry is 48 bytes, the
        // collective-cost entry 8 bytes, so one multiply-add serves both addresses
        const uint32_t zc = ace_mad24(c, 8u, z_v);
        const uint32_t a = ace_mad24(zc, ACE_HOT_STRIDE / 8u, row + g.hot_off);
        ace_d2 e0 = lds.ld<ace_d2>(a);         // fwd us, bwd us
        ace_d2 e1 = lds.ld<ace_d2>(a + 16);    // weights MB, activations MB (shared-buffer rule applied)
        ace_d2 e2 = lds.ld<ace_d2>(a + 32);    // fwd / bwd reserved MB
        fwd += e0.x;
        bwd += e0.y;
        rcs = ace_fma((double)(int)rc, e0.x, rcs);   // rc is 0 or 1: the product is exact, one rounding as in "+="
        W += e1.x;
        A += e1.y;
        if (BD) {
            ace_d2 ie = lds.ld<ace_d2>(row + g.hot_off + ideal_hot_v + (c & (uint32_t)(g.n_algo - 1)) * ACE_HOT_STRIDE);
            id_fwd += ie.x;
            id_bwd += ie.y;
        }
        if (g.flags & ACE_F_RESHARDING) {
            // collective ids of the (previous, this) op pair, fetched while the previous op was
            // processed; id 0 is an all-zero cost table, so a pair that needs nothing (and a stage's
            // first op) adds 0.0, and the id past the last real table is all NaN (the reference raises there)
            const uint32_t r = r_next;
            const uint32_t pk = (info >> 16) & 0xffu;
            // (rk_v + zc = stage-size block * 64 + c * 8, and c * 8 + nc < 64: the [c][nc] entry of that block)
            r_next = lds.ld<uint8_t>((g.rk_lds_off + ace_mul24(pk, g.rk_kind_stride)) + ((rk_v + zc) + nc));
            const uint32_t za = (row + g.z_off) + zc;
            const uint32_t af = za + ((r & 15u) << g.z_shift), ab = za + ((r >> 4) << g.z_shift);
            rs_f += lds.ld<double>(af);
            rs_b += lds.ld<double>(ab);
            if (COLL) {
                // max_collective of get_reserved_memory (:462-478): the same pairs, the collectives' buffers
                mc = ace_max(mc, lds.ld<double>(af + g.zm_delta));
                mc = ace_max(mc, lds.ld<double>(ab + g.zm_delta));
            }
        }
        double rf_new = ace_max(rfm, e2.x), rb_new = ace_max(rbm, e2.y);
        // the stage ends with this op
        const bool last = RANGED ? (i + 1 == hi) : (((nbyte >> 4) & 1u) || plan_end);
        if (last) {
            // :439 "i + 1 == len(ops) - 1": the (previous, this) pair closes the last segment
            if (DEFER) stash(g, rec, (uint32_t)i, c, nc, (pinfo >> 25) & 1u, (GROWS ? row_ids[i] : info) & 0xffffu);
            else {
                lastclose = pair_prev & (pinfo >> 25) & 1u;
                finish(g, lds, row, c, rec);
            }
            if (!RANGED) {
                // (after the plan's last op this opens a stage that stays empty: s == S in the end)
                start_fast(g, lds, !DEFER);
                if (!DEFER && i + 1 < g.N) start_lookups(g, lds, info_nextrow(g, info), nc);
            }
            // the reserved maxima run over every op but the stage's last (get_reserved_memory :453-460):
            // the stage that ended took them as they were before this op, the new one starts from zero
            rf_new = 0.0;
            rb_new = 0.0;
        }
        rfm = rf_new;
        rbm = rb_new;
        // pair: (this op, next op) both recomputed and in one stage
        const bool savez = (info >> 24) & 1u;     // this is an ordinary op followed by a layer start
        // All of this is arithmetic on 0.0 / 1.0 factors instead of selects: x*1.0 and x+0.0 are exact,
        // so every value is the one the reference computes.  (After a stage end the accumulators
        // are zero and pair is false: nothing happens.)
        const double pairf = (double)(int)pair;
        const double keepf = pairf * ace_scalar_01(!savez);       // 1.0 iff the pair continues the running segment
        const double seg = ace_fma(pairf, e1.y, run);             // run + act              if pair
        saved = ace_fma(keepf, e1.y, saved);                      // saved += act           if pair and not savez
        const double closed = ace_fma(-keepf, seg, seg);          // seg if the segment closes here, else seg - seg = 0.0
        peak = ace_max(peak, closed);                             // max(peak, 0.0) leaves peak (>= 0) alone
        run = seg * keepf;                                        // 0.0 if closed, else seg
        pair_prev = pair;
    }

    ACE_HD void result(const AceGeom &g, double nbm1, double &iter_ms, double &peak_mb, uint8_t &feasible, uint8_t &st) {
        if (!RANGED && (s != S || S > ACE_MAX_STAGES)) status = ACE_PLAN_MALFORMED;   // every stage end also opened the next stage
        // max over stages of t_s*(nb-1) + sum(t): rounding is monotonic, so the maximum is attained
        // at the largest t_s and equals this expression bit for bit
        iter_ms = max_t * nbm1 + sum_t;
        peak_mb = max_mem;
        bool ok = status == 0 && !ace_isnan(iter_ms) && !ace_isnan(max_mem);
        if (!ok && status == 0) status = ACE_PLAN_UNSCORABLE;   // a table entry outside the profiled grid
        bool feas = g.strict ? (max_mem < g.mem_limit) : (max_mem <= g.mem_limit);
        feasible = (uint8_t)(ok && feas);
        st = (uint8_t)status;
        if (!ok) {
            iter_ms = __builtin_nan("");
            peak_mb = __builtin_nan("");
        }
    }
};

// 1 iff two consecutive ops (code bytes a, b) are both recomputed and b does not start a stage
ACE_HD uint32_t pair_bit(uint32_t a, uint32_t b) { return ((a & b) >> 3) & ~(b >> 4) & 1u; }

// byte k (0..15) of a 16-op group held in four 32-bit words
ACE_HD uint32_t group_byte(const uint32_t w[4], int k) { return (w[k >> 2] >> ((k & 3) * 8)) & 0xffu; }
