"""Writes ace_score_loop_asm.inc: the op loop of the plain scoring kernel (deferred stage tails) as gfx950 assembly.

    python3 superscaler_amd/csrc/gen_score_loop_asm.py

The loop is the one ace_score_body() runs in C++ (ace_score_loop.h, PlanState::step / stash / start_fast of
ace_plan_state.h, DEFER variant), written out by hand so that
  * the 0/1 factors of the recompute rules become execution masks: the recompute bit and the stage-start bit of an
    op are tested with one byte-select compare each (the recompute bit a step ahead), the recompute-pair mask is the
    AND of two consecutive recompute masks without the lanes whose next op starts a stage (scalar instructions), and
    the conditional additions run under the resulting lane mask (an addition that does not happen and an addition of
    +0.0 give the same bits);
  * the table reads of op k+1 are issued before op k's values are used (two alternating register sets);
  * every position-dependent address comes ready-made from a per-position table (four words per op position,
    read with scalar loads one 4-op word ahead) instead of being derived per op.
Floating-point operations and their order per plan are exactly those of the C++ loop, so results are bit-identical.
The loop ends with the plan's last op (every plan of a batch has the same number of ops; the mark planted behind the
last op closes the last stage for all lanes at once), not with the padding positions of the last 16-op group.

Pacing (rows resident): the wavefronts of a workgroup share the cache lines of their plans' code bytes (a line holds
the 16 bytes of eight neighbouring plans, which the depth sort deals to different wavefronts), and a wavefront of
deep plans needs twice the instructions per op of one with shallow plans: left alone they drift groups apart and every
line is fetched from memory twice.  So each SIMD counts, per 16-op group, how many of its four wavefronts have
entered it (eight LDS counters per SIMD, used in turn, never reset: the count modulo 4 is the rank); the two that enter
a group last run at issue priority 3 until their next group, the two that were first at 0.  The wavefronts of a
workgroup then walk within a group or two of each other.

The "_WIN" texts are for rows that do not fit in LDS together: the loop keeps its own windows of rows (only the parts
of a row it reads), consecutive windows in alternate halves of LDS.  At a window's first position all wavefronts of
the workgroup meet at a barrier, after which each issues its share of the LDS-direct loads of the window AFTER the
one being entered (Gen.fetch_event; the records come from ace_eval.hip's setup_windowed_asm), which therefore arrive
while the workgroup walks a whole window.

One text per (rows resident / windowed, resharding on / off, reserved-memory rule); each is a C string literal macro
that ace_score_loop.h pastes into an asm statement.  Register use: v28-v127 and s24-s99 belong to the loop; operands
live below.
"""
import os

HERE = os.path.dirname(os.path.abspath(__file__))

# ---- vector registers ---------------------------------------------------------------------------------------
FB, RCS = "v[32:33]", "v[34:35]"            # quad v[32:35]: stash record 0 = {fwd + bwd, recompute sum}
RSF, RSB = "v[36:37]", "v[38:39]"           # quad v[36:39]: record 1 = {resharding fwd, bwd}
W_, A_ = "v[40:41]", "v[42:43]"             # quad v[40:43]: record 2 = {weights, activations}
SAVED, PEAK = "v[44:45]", "v[46:47]"        # quad v[44:47]: record 3 = {saved, peak}
# record 4 = {reserved term, code*8 + next code of a word's ops, position word}: one quad per buffer of word-level values,
# so that the code word is stored from where the word's preparation wrote it
RESQ = ["v[48:51]", "v[56:59]"]
RES = ["v[48:49]", "v[56:57]"]
CN = ["v50", "v58"]
META = ["v51", "v59"]
FWD, BWD, RUN = "v[52:53]", "v[54:55]", "v[112:113]"
RFM = ["v[60:61]", "v[64:65]"]              # reserved maxima, alternating between consecutive ops
RBM = ["v[62:63]", "v[66:67]"]


def E(x):                                   # hot entry of an op: {fwd, bwd} {weights, act} {reserved fwd, bwd}
    b = 68 + 12 * x
    return dict(q0=f"v[{b}:{b+3}]", q1=f"v[{b+4}:{b+7}]", q2=f"v[{b+8}:{b+11}]", fwd=f"v[{b}:{b+1}]",
                bwd=f"v[{b+2}:{b+3}]", w=f"v[{b+4}:{b+5}]", act=f"v[{b+6}:{b+7}]", rf=f"v[{b+8}:{b+9}]",
                rb=f"v[{b+10}:{b+11}]")


def ZV(x):                                  # collective costs of an op's input: forward, backward
    b = 92 + 4 * x
    return f"v[{b}:{b+1}]", f"v[{b+2}:{b+3}]"


def R(x):                                   # cost-table byte offsets (forward | backward << 16) of an op pair
    return f"v{100 + x}"


WORD = [f"v{102 + j}" for j in range(4)]    # code words of the current 16-op group
NEXT = [f"v{106 + j}" for j in range(4)]    # ... of the next group


def D(y):                                   # per 4-op word: next-op bytes, code*8, code*8+next code, rc bit
    b = (110, 116)[y]
    r = (114, 118)[y]
    return dict(nw=f"v{b}", w8=f"v{b+1}", cn=CN[y], r8=f"v{r}")


ZV_, RK, ZVRK, WSOFF = "v120", "v121", "v[120:121]", "v122"   # WSOFF: byte offset of this lane's next stage record (it counts the stages)
PACE = "v123"                               # lane 0: what this group's arrival counter read before this wavefront was counted
# log2 of the plan's stage sizes, 4 bits each, next stage lowest; LDS address of the plan's micro-batch size in the table
# of (diag offset, pair-table block) per stage size
GLOGS, GLOGS_LO, LUT2 = "v[28:29]", "v28", "v30"
NZVRK = "v[124:125]"                         # ZVRK of the stage after the current one, read ahead
T0, T1, T01, T2 = "v126", "v127", "v[126:127]", "v33"

# ---- scalar registers ---------------------------------------------------------------------------------------
ALL = "s[24:25]"
CPTR, CPTR_LO, CPTR_HI = "s[26:27]", "s26", "s27"
GRP, K07, K08, POSBASE, LEFT, K1F = "s30", "s39", "s40", "s41", "s31", "s38"
PPTR, PPTR_LO, PPTR_HI = "s[36:37]", "s36", "s37"
M_P, M_ST, M_KP = "s[44:45]", "s[46:47]", "s[48:49]"
MRC = ["s[42:43]", "s[58:59]"]              # "recomputed" of the ops at even / odd positions: an op's is compared a step ahead (the pair mask is made of two)
MASK, PLANT = "s52", "s56"                   # padding mask and end-of-plan mark of one code word (scratch)
PREVFL = "s62"
NGRP = "s51"                                # number of 16-op groups
VMN = "s50"                                 # record stores issued since the load of the next group's code words
WSLIMIT = "s28"                             # WSOFF of a seventeenth stage, which no lane has room for
NEXTWIN, EVT, DMAOFF, ARRIVED = "s29", "s34", "s63", "s35"   # windowed rows: next window's first position, window index, ...
DMAPTR = "s[60:61]"
S0, S1, S2, S23 = "s96", "s97", "s98", "s[98:99]"


def P(y, q):                                # position entry q of the word in buffer y: hot, z, pair-table address, flags | rows << 8
    b = 64 + 16 * y + 4 * q
    return dict(hot=f"s{b}", z=f"s{b+1}", pk=f"s{b+2}", fl=f"s{b+3}")


def PBUF(y):
    return f"s[{64 + 16 * y}:{79 + 16 * y}]"


class Gen:
    def __init__(self, rsh, mode, win=False):
        self.rsh, self.mode, self.win, self.lines = rsh, mode, win, []

    def o(self, s):
        self.lines.append(s)

    def c(self, s):
        self.lines.append("; " + s)

    # -- pieces ------------------------------------------------------------------------------------------------
    def prep(self, y, wa, wb):
        d = D(y)
        self.c(f"word-level: next-op bytes, code*8, code*8+next code, recompute bit (buffer {y})")
        self.o(f"v_alignbit_b32 {d['nw']}, {wb}, {wa}, 8")
        self.o(f"v_and_b32 {d['w8']}, {K07}, {wa}")
        self.o(f"v_lshlrev_b32 {d['w8']}, 3, {d['w8']}")
        self.o(f"v_and_or_b32 {d['cn']}, {d['nw']}, {K07}, {d['w8']}")
        self.o(f"v_and_b32 {d['r8']}, {K08}, {wa}")

    def stage_fetch(self, dst):
        """Asks for z_v and the pair-table block of the plan's next stage: one 8-byte LDS read per lane, indexed by the
        next nibble of the plan's stage sizes."""
        self.o(f"v_and_b32 {T0}, 15, {GLOGS_LO}")
        self.o(f"v_lshl_add_u32 {T0}, {T0}, 3, {LUT2}")
        self.o(f"v_lshrrev_b64 {GLOGS}, 4, {GLOGS}")
        self.o(f"ds_read_b64 {dst}, {T0}")

    def issue(self, k1):
        """Address arithmetic and LDS reads of op k1 (0..16; 16 = first op of the next group)."""
        j1, b1 = k1 >> 2, k1 & 3
        y1, x1 = j1 & 1, k1 & 1
        d, p, e = D(y1), P(y1, b1), E(x1)
        sel = f"dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_{b1}"
        self.c(f"op {k1}: table reads")
        self.o(f"v_add_u32_sdwa {T0}, {ZV_}, {d['w8']} {sel}")
        self.o(f"v_mad_u32_u24 {T1}, {T0}, 6, {p['hot']}")
        self.o(f"ds_read_b128 {e['q0']}, {T1}")
        self.o(f"ds_read_b128 {e['q1']}, {T1} offset:16")
        self.o(f"ds_read_b128 {e['q2']}, {T1} offset:32")
        if not self.rsh:
            return
        self.o(f"v_add_u32_sdwa {T1}, {RK}, {d['cn']} {sel}")
        self.o(f"v_lshl_add_u32 {T1}, {T1}, 2, {p['pk']}")
        self.o(f"ds_read_b32 {R(1 - x1)}, {T1}")           # cost-table offsets of the (k1, k1 + 1) pair
        self.o(f"v_add_u32_e32 {T0}, {p['z']}, {T0}")
        self.o("s_waitcnt lgkmcnt(4)")                       # those of the (k1 - 1, k1) pair are in
        zf, zb = ZV(x1)
        wsel = "dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_"
        self.o(f"v_add_u32_sdwa {T1}, {T0}, {R(x1)} {wsel}0")
        self.o(f"v_add_u32_sdwa {T2}, {T0}, {R(x1)} {wsel}1")
        self.o(f"ds_read_b64 {zf}, {T1}")
        self.o(f"ds_read_b64 {zb}, {T2}")

    def fetch_event(self, L, pq):
        """Windowed rows, one fetch event: the wavefront's record {first position of the window after the one being
        entered, bit 0: wait for the fetch | number of loads << 8, address of the rows} and eight loads {byte offset in
        the rows, LDS address} (the second four go through s[pq:pq+7]); all wavefronts of the workgroup meet, then each
        issues its loads (LDS-direct, 1 KB each)."""
        self.o(f"s_mul_i32 {DMAOFF}, {EVT}, 1280")
        self.o(f"s_add_u32 {DMAOFF}, {DMAOFF}, %[waveoff]")
        self.o(f"s_load_dwordx4 s[96:99], {DMAPTR}, {DMAOFF}")
        self.o(f"s_add_u32 {DMAOFF}, {DMAOFF}, 16")
        self.o(f"s_load_dwordx8 s[52:59], {DMAPTR}, {DMAOFF}")
        self.o(f"s_add_u32 {DMAOFF}, {DMAOFF}, 32")
        self.o(f"s_load_dwordx8 s[{pq}:{pq + 7}], {DMAPTR}, {DMAOFF}")
        self.o("s_waitcnt vmcnt(0) lgkmcnt(0)")             # this wavefront's reads of the old rows and its loads so far have landed
        self.o("s_barrier")
        self.o(f"s_mov_b32 {ARRIVED}, 1")                   # (so have the next group's code words, if they were asked for)
        self.o(f"s_add_u32 {EVT}, {EVT}, 1")
        self.o(f"v_mbcnt_lo_u32_b32 {T0}, -1, 0")
        self.o(f"v_mbcnt_hi_u32_b32 {T0}, -1, {T0}")
        self.o(f"v_lshlrev_b32 {T0}, 4, {T0}")
        self.o(f"s_bfe_u32 {DMAOFF}, s97, 0x40008")         # number of loads
        for j in range(8):
            base = 52 + 2 * j if j < 4 else pq + 2 * (j - 4)
            self.o(f"s_cmp_le_u32 {DMAOFF}, {j}")
            self.o(f"s_cbranch_scc1 L_fd_{L}")
            self.o(f"s_mov_b32 m0, s{base + 1}")
            self.o(f"v_add_u32_e32 {T1}, s{base}, {T0}")
            self.o("s_nop 0")
            self.o(f"global_load_lds_dwordx4 {T1}, s[98:99]")
        self.o(f"L_fd_{L}:")
        self.o(f"s_mov_b32 {NEXTWIN}, s96")
        self.o("s_bitcmp1_b32 s97, 0")
        self.o(f"s_cbranch_scc0 L_fa_{L}")
        self.o("s_waitcnt vmcnt(0)")
        self.o("s_barrier")
        self.o(f"L_fa_{L}:")

    def window_switch(self, k1, L, y):
        """Windowed rows: if op k1 of the group (0..16) is the first of the next window, the next fetch event."""
        self.c("rows of the next window, if it starts with the next op")
        self.o(f"s_add_u32 {S0}, {POSBASE}, {k1}")
        self.o(f"s_cmp_eq_u32 {S0}, {NEXTWIN}")
        self.o(f"s_cbranch_scc0 L_nw_{L}")
        self.fetch_event(L, 64 + 16 * y)                    # (the first two position entries of this word are done with)
        # (the event's descriptors went through the registers that hold the recompute mask of the ops at odd positions:
        # window starts are multiples of four, so that is the op being processed)
        k = k1 - 1
        self.o(f"v_cmp_ne_u32_sdwa {MRC[k & 1]}, {D((k >> 2) & 1)['r8']}, 0 src0_sel:BYTE_{k & 3} src1_sel:DWORD")
        self.o(f"L_nw_{L}:")
        self.o(f"s_cmp_lg_u64 {M_ST}, 0")                   # (what the branch to the stage-end code tests)

    def reserved(self, cur, res):
        if self.mode == "max":          # max(rf + rb, W)
            self.o(f"v_add_f64 {res}, {RFM[cur]}, {RBM[cur]}")
            self.o(f"v_max_f64 {res}, {res}, {W_}")
        elif self.mode == "min":        # max(max(rf, rb), max(W, 0))
            self.o(f"v_max_f64 {res}, {RFM[cur]}, {RBM[cur]}")
            self.o(f"v_max_f64 {T01}, {W_}, 0")
            self.o(f"v_max_f64 {res}, {res}, {T01}")
        else:
            self.o(f"v_mov_b64 {res}, 0")

    def slot(self, k):
        j, b = k >> 2, k & 3
        y, x, x1 = j & 1, k & 1, (k + 1) & 1
        d, p, e = D(y), P(y, b), E(x)
        cur, nxt = k & 1, (k + 1) & 1          # reserved maxima: read `cur`, write `nxt`
        L = f"{k}_%="
        self.c(f"================ op {k} of the group")
        if b == 0:
            self.c("position entries of the next word")
            self.o(f"s_load_dwordx16 {PBUF((j + 1) & 1)}, {PPTR}, {64 * (j + 1)}")
        if b == 2:
            self.o("s_waitcnt lgkmcnt(0)")
            if k == 2 and not self.win:
                self.c("pacing: the two wavefronts of a SIMD that entered this group last get the issue priority, the two that are ahead yield")
                self.o(f"v_readfirstlane_b32 {S0}, {PACE}")
                self.o(f"s_bitcmp1_b32 {S0}, 1")
                self.o("s_cbranch_scc0 L_pp0_%=")
                self.o("s_setprio 3")
                self.o("s_branch L_ppd_%=")
                self.o("L_pp0_%=:")
                self.o("s_setprio 0")
                self.o("L_ppd_%=:")
        if k == 11:
            self.next_group_words()
        if b == 3:
            if j < 3:
                self.prep((j + 1) & 1, WORD[j + 1], WORD[j + 2] if j + 2 < 4 else NEXT[0])
            else:
                self.prep(0, NEXT[0], NEXT[1])
        sel = f"src0_sel:BYTE_{b} src1_sel:DWORD"
        # "recomputed" of the NEXT op (this op's was compared a step ago); (this op, next op) is a recompute pair if
        # both are recomputed and the next op does not start a stage: two scalar instructions instead of a third compare
        k1 = k + 1
        d1 = D((k1 >> 2) & 1)
        self.o(f"v_cmp_ne_u32_sdwa {MRC[k1 & 1]}, {d1['r8']}, 0 src0_sel:BYTE_{k1 & 3} src1_sel:DWORD")
        self.o(f"v_cmp_gt_u32_sdwa {M_ST}, {d['nw']}, 15 {sel}")
        self.o(f"s_and_b64 {M_P}, {MRC[0]}, {MRC[1]}")
        self.o(f"s_andn2_b64 {M_P}, {M_P}, {M_ST}")
        self.o(f"s_cmp_lg_u64 {M_ST}, 0")
        self.o(f"s_cbranch_scc0 L_ns_{L}")
        self.c("lanes whose next op opens a stage: that stage's table offsets; its first op pays no resharding")
        self.o(f"s_mov_b64 exec, {M_ST}")
        if self.win:
            self.stage_fetch(ZVRK)
            self.o("s_waitcnt lgkmcnt(0)")
        else:
            self.c("(asked for where the stage before began, before that op's table reads, of which all but the last two are in)")
            self.o("s_waitcnt lgkmcnt(2)")
            self.o(f"v_mov_b64 {ZVRK}, {NZVRK}")
        if self.rsh:
            self.o(f"v_mov_b32 {R(x1)}, 0")
        if not self.win:
            self.c("the offsets of the stage after the one that begins now, for when that one ends")
            self.stage_fetch(NZVRK)
        self.o(f"s_mov_b64 exec, {ALL}")
        self.o(f"L_ns_{L}:")
        if self.win and b == 3:
            self.window_switch(k + 1, L, y)
        self.issue(k + 1)
        if not self.rsh:
            self.o("s_waitcnt lgkmcnt(3)")
        self.c(f"op {k}: sums")
        zf, zb = ZV(x)
        self.o(f"v_add_f64 {FWD}, {FWD}, {e['fwd']}")
        self.o(f"v_add_f64 {BWD}, {BWD}, {e['bwd']}")
        self.o(f"v_add_f64 {W_}, {W_}, {e['w']}")
        self.o(f"v_add_f64 {A_}, {A_}, {e['act']}")
        if self.rsh:
            self.o(f"v_add_f64 {RSF}, {RSF}, {zf}")
            self.o(f"v_add_f64 {RSB}, {RSB}, {zb}")
        self.o(f"v_max_f64 {RFM[nxt]}, {RFM[cur]}, {e['rf']}")
        self.o(f"v_max_f64 {RBM[nxt]}, {RBM[cur]}, {e['rb']}")
        self.o(f"s_mov_b64 exec, {MRC[k & 1]}")
        self.o(f"v_add_f64 {RCS}, {RCS}, {e['fwd']}")
        self.o(f"s_cbranch_scc0 L_ne_{L}")
        self.c("lanes whose stage ends with this op: park the stage's values, start the next stage from zero")
        self.o(f"s_mov_b64 exec, {M_ST}")
        self.o(f"v_add_f64 {FB}, {FWD}, {BWD}")
        prevfl = P(y, b - 1)["fl"] if b else PREVFL
        self.c("the last segment closes into the peak if the op before this one is an ordinary one")
        self.o(f"s_bitcmp1_b32 {prevfl}, 1")
        self.o(f"s_cselect_b64 exec, {M_ST}, 0")
        self.o(f"v_max_f64 {PEAK}, {PEAK}, {RUN}")
        self.o(f"s_mov_b64 exec, {M_ST}")
        self.reserved(cur, RES[y])
        self.o(f"s_add_u32 {S0}, {POSBASE}, {k}")
        self.o(f"s_andn2_b32 {S1}, {p['fl']}, 0xff")
        self.o(f"s_lshl_b32 {S1}, {S1}, 8")
        self.o(f"s_or_b32 {S0}, {S0}, {S1}")
        self.o(f"v_mov_b32 {META[y]}, {S0}")                 # position of the stage's last op | its row << 16 | the next op's row << 24
        self.o(f"v_cmp_gt_u32_e32 vcc, {WSLIMIT}, {WSOFF}")
        self.o("s_and_b64 exec, exec, vcc")
        self.o(f"s_cselect_b32 {S0}, 5, 0")                     # (no lane with room: the stores may not be issued at all)
        self.o(f"s_add_u32 {VMN}, {VMN}, {S0}")
        self.o(f"global_store_dwordx4 {WSOFF}, v[32:35], %[recbase]")
        self.o(f"global_store_dwordx4 {WSOFF}, v[36:39], %[recbase] offset:16")
        self.o(f"global_store_dwordx4 {WSOFF}, v[40:43], %[recbase] offset:32")
        self.o(f"global_store_dwordx4 {WSOFF}, v[44:47], %[recbase] offset:48")
        self.o(f"global_store_dwordx4 {WSOFF}, {RESQ[y]}, %[recbase] offset:64")
        self.o(f"s_mov_b64 exec, {M_ST}")
        self.o(f"v_add_u32_e32 {WSOFF}, %[wsstride], {WSOFF}")
        self.o(f"v_mov_b64 {RUN}, 0")
        self.o(f"v_mov_b64 {PEAK}, 0")
        if True:
            for r in (FWD, BWD, RFM[nxt], RBM[nxt]):
                self.o(f"v_mov_b64 {r}, 0")
            self.o("s_nop 1")
            for r in (RCS, W_, A_, SAVED) + ((RSF, RSB) if self.rsh else ()):
                self.o(f"v_mov_b64 {r}, 0")
        self.c("that was the plan's last op (for every lane: the mark planted behind it): the padding positions need no walk")
        self.o(f"s_add_u32 {S0}, {POSBASE}, {k + 1}")
        self.o(f"s_cmp_eq_u32 {S0}, %[n_ops]")
        self.o("s_cbranch_scc1 L_exit_%=")
        self.o(f"L_ne_{L}:")
        self.c("recompute pair (this op, next op): saved activations, running segment, peak")
        self.o(f"s_bitcmp1_b32 {p['fl']}, 0")
        self.o(f"s_cselect_b64 {M_KP}, {M_P}, 0")
        self.o(f"s_mov_b64 exec, {M_P}")
        self.o(f"v_add_f64 {RUN}, {RUN}, {e['act']}")
        self.o(f"s_mov_b64 exec, {M_KP}")
        self.o(f"v_add_f64 {SAVED}, {SAVED}, {e['act']}")
        self.o(f"s_andn2_b64 exec, {ALL}, {M_KP}")
        self.o(f"v_max_f64 {PEAK}, {PEAK}, {RUN}")
        self.o(f"v_mov_b64 {RUN}, 0")
        self.o(f"s_mov_b64 exec, {ALL}")
        if b == 3:
            self.o(f"s_mov_b32 {PREVFL}, {p['fl']}")

    def apply_masks(self, regs, tag):
        """Code bytes of positions past the last op read as zero, and the byte right after the last op gets a stage-start
        bit, which is what ends the plan's last stage (LEFT = N - (first position of the group); five code bits used)."""
        self.o(f"s_cmp_ge_i32 {LEFT}, 16")
        self.o(f"s_cbranch_scc1 L_full_{tag}_%=")
        for j in range(4):
            self.o(f"s_sub_i32 {S0}, {LEFT}, {4 * j}")
            self.o(f"s_min_i32 {S1}, {S0}, 4")
            self.o(f"s_max_i32 {S1}, {S1}, 0")
            self.o(f"s_lshl_b32 {S1}, {S1}, 3")
            self.o(f"s_bfm_b64 {S23}, {S1}, 0")
            self.o(f"s_and_b32 {MASK}, {S2}, {K1F}")
            self.o(f"s_lshl_b64 {S23}, 16, {S1}")
            self.o(f"s_cmp_ge_i32 {S0}, 0")
            self.o(f"s_cselect_b32 {PLANT}, {S2}, 0")
            self.o(f"v_and_b32 {regs[j]}, {MASK}, {regs[j]}")
            self.o(f"v_or_b32 {regs[j]}, {PLANT}, {regs[j]}")
        self.o(f"s_branch L_masked_{tag}_%=")
        self.o(f"L_full_{tag}_%=:")
        for j in range(4):
            self.o(f"v_and_b32 {regs[j]}, {K1F}, {regs[j]}")
        self.o(f"L_masked_{tag}_%=:")

    def next_group_words(self):
        self.c("the next group's code words have arrived (zeros after the last group): padding and end-of-plan mark")
        if self.win:
            # (not if a window was entered since the words were asked for: they were waited for there, and the window
            # loads now in flight need not be)
            self.o(f"s_cmp_eq_u32 {ARRIVED}, 1")
            self.o("s_cbranch_scc1 L_arr_%=")
        # (vector-memory instructions complete in the order they were issued: only what was issued before the load and
        # the load itself have to be waited for, not the record stores of the last few ops)
        for n in (15, 10, 5):
            self.o(f"s_cmp_ge_u32 {VMN}, {n}")
            self.o(f"s_cbranch_scc1 L_vm{n}_%=")
        self.o("s_waitcnt vmcnt(0)")
        self.o("s_branch L_vmd_%=")
        for n in (15, 10, 5):
            self.o(f"L_vm{n}_%=:")
            self.o(f"s_waitcnt vmcnt({n})")
            if n != 5:
                self.o("s_branch L_vmd_%=")
        self.o("L_vmd_%=:")
        if self.win:
            self.o("L_arr_%=:")
        self.o(f"s_sub_i32 {LEFT}, %[n_ops], {POSBASE}")
        self.o(f"s_sub_i32 {LEFT}, {LEFT}, 16")
        self.apply_masks(NEXT, "nx")

    def build(self):
        o, c = self.o, self.c
        c("---- set-up")
        if self.win:
            c("issue priority of this wavefront (the deeper its plans, the higher; with rows resident the pacing sets it)")
            for lvl in (3, 2, 1):
                o(f"s_cmp_eq_u32 %[prio], {lvl}")
                o(f"s_cbranch_scc0 L_np{lvl}_%=")
                o(f"s_setprio {lvl}")
                o(f"L_np{lvl}_%=:")
        o(f"s_mov_b64 {ALL}, exec")
        o(f"s_add_u32 {NGRP}, %[n_ops], 15")
        o(f"s_lshr_b32 {NGRP}, {NGRP}, 4")
        o(f"v_mov_b64 {GLOGS}, %[glogs]")
        o(f"v_mov_b32 {LUT2}, %[lut2]")
        o(f"s_mov_b64 {CPTR}, %[codes]")
        o(f"s_mov_b64 {PPTR}, %[pos]")
        o(f"s_mov_b32 {K07}, 0x07070707")
        o(f"s_mov_b32 {K08}, 0x08080808")
        o(f"s_mov_b32 {K1F}, 0x1f1f1f1f")
        o(f"s_mov_b32 {GRP}, 0")
        o(f"s_mov_b32 {POSBASE}, 0")
        o(f"s_mov_b32 {PREVFL}, 0")
        if self.win:
            o(f"s_mov_b64 {DMAPTR}, %[dma]")
            o(f"s_mov_b32 {ARRIVED}, 0")
            o(f"s_mov_b32 {EVT}, 0")
            c("window 0 (waited for), then window 1")
            self.fetch_event("s0_%=", 80)
            self.fetch_event("s1_%=", 80)
        o(f"global_load_dwordx4 v[102:105], %[codeoff], {CPTR}")
        o(f"s_load_dwordx16 {PBUF(0)}, {PPTR}, 0")
        for r in (FWD, BWD, RUN, PEAK, RFM[0], RBM[0], RCS, RSF, RSB, W_, A_, SAVED):
            o(f"v_mov_b64 {r}, 0")
        o(f"v_mov_b32 {WSOFF}, %[recoff]")
        o(f"s_lshl_b32 {WSLIMIT}, %[wsstride], 4")
        o(f"v_mov_b32 {R(0)}, 0")
        self.stage_fetch(ZVRK)
        if not self.win:
            self.stage_fetch(NZVRK)
        o("s_waitcnt vmcnt(0) lgkmcnt(0)")
        o(f"s_mov_b32 {LEFT}, %[n_ops]")
        self.apply_masks(WORD, "w0")
        self.prep(0, WORD[0], WORD[1])
        o(f"v_cmp_ne_u32_sdwa {MRC[0]}, {D(0)['r8']}, 0 src0_sel:BYTE_0 src1_sel:DWORD")
        self.issue(0)
        c("---- one 16-op group per iteration")
        o("L_group_%=:")
        o(f"s_add_u32 {S0}, {GRP}, 1")
        o(f"s_cmp_lt_u32 {S0}, {NGRP}")
        o("s_cbranch_scc0 L_last_%=")
        o(f"s_add_u32 {CPTR_LO}, {CPTR_LO}, %[gstride_lo]")
        o(f"s_addc_u32 {CPTR_HI}, {CPTR_HI}, %[gstride_hi]")
        o(f"global_load_dwordx4 v[106:109], %[codeoff], {CPTR}")
        o("s_branch L_loaded_%=")
        o("L_last_%=:")
        for r in NEXT:
            o(f"v_mov_b32 {r}, 0")
        o("L_loaded_%=:")
        o(f"s_mov_b32 {VMN}, 0")
        if self.win:
            o(f"s_mov_b32 {ARRIVED}, 0")
        else:
            c("pacing: count this wavefront into this group's arrival counter of its SIMD (the count before it: its rank among the four)")
            o(f"s_and_b32 {S0}, {GRP}, 7")
            o(f"s_lshl_b32 {S0}, {S0}, 2")
            o(f"s_add_u32 {S0}, {S0}, %[pace]")
            o(f"v_mov_b32 {T1}, {S0}")
            o(f"v_mov_b32 {T0}, 1")
            o("s_mov_b64 exec, 1")
            o(f"ds_add_rtn_u32 {PACE}, {T1}, {T0}")
            o(f"s_mov_b64 exec, {ALL}")
        for k in range(16):
            self.slot(k)
        c("---- next group")
        for j in range(4):
            o(f"v_mov_b32 {WORD[j]}, {NEXT[j]}")
        o(f"s_add_u32 {PPTR_LO}, {PPTR_LO}, 256")
        o(f"s_addc_u32 {PPTR_HI}, {PPTR_HI}, 0")
        o(f"s_add_u32 {POSBASE}, {POSBASE}, 16")
        o(f"s_add_u32 {GRP}, {GRP}, 1")
        o(f"s_cmp_lt_u32 {GRP}, {NGRP}")
        o("s_cbranch_scc1 L_group_%=")
        o("L_exit_%=:")
        o(f"s_mov_b64 exec, {ALL}")
        o("s_waitcnt vmcnt(0) lgkmcnt(0)")
        o("s_setprio 0")
        o(f"v_mov_b32 %[wsoff], {WSOFF}")
        return self.lines


def c_string(lines):
    out = []
    for ln in lines:
        assert '"' not in ln and "\\" not in ln
        out.append('    "' + ln + '\\n"')
    return " \\\n".join(out)


def render():
    """The text of ace_score_loop_asm.inc."""
    parts = ["// Generated by gen_score_loop_asm.py -- do not edit.  gfx950 assembly of the plain scoring kernel's op loop",
             "// (deferred stage tails), one text per (resharding, reserved-memory rule); see the generator for the design.",
             "#pragma once", ""]
    for win in (0, 1):
        for rsh in (1, 0):
            for mode in ("max", "min", "none"):
                g = Gen(bool(rsh), mode, bool(win))
                parts.append(f"#define ACE_LOOP_ASM{'_WIN' if win else ''}_RSH{rsh}_{mode.upper()} \\")
                parts.append(c_string(g.build()))
                parts.append("")
    clob = ", ".join(f'"v{i}"' for i in range(28, 128)) + ", " + ", ".join(f'"s{i}"' for i in range(24, 100) if i not in (32, 33))   # (s32 / s33 are the ABI's stack registers)
    parts.append(f"#define ACE_LOOP_ASM_CLOBBERS {clob}, \"vcc\", \"scc\", \"m0\", \"memory\"")
    parts.append("")
    return "\n".join(parts)


def main():
    path = os.path.join(HERE, "ace_score_loop_asm.inc")
    with open(path, "w") as f:
        f.write(render())
    print("wrote", path)


if __name__ == "__main__":
    main()
