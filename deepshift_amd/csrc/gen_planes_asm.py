#!/usr/bin/env python3
"""Generates ds_planes_asm.inc: the hand-scheduled main loop of ds::shift_planes_kernel.

    python deepshift_amd/csrc/gen_planes_asm.py      # rewrites ds_planes_asm.inc next to this file

The loop is emitted as one inline-asm string per shift-field width BITS (1..4) because it uses
VGPR-relative addressing (s_set_gpr_idx_*), which needs a fixed register map:

    per reduction index k and pixel row r:  plane[r][s] = x >> s  for every shift amount s < 2^BITS
                                            (2^BITS vector shifts, shared by all 32 output channels)
    per (k, channel j):                     M0 <- the code's 16-bit pre-decoded form (scalar), mask <- sign
                                            acc[r][j] = (plane[r][M0] ^ mask) + acc[r][j]   (v_xad_u32)

so a shift-add term costs 1 + 2^BITS/32 vector instructions instead of 2.  Every width also comes in
a "zero top" form (DS_PLANES_ASM_B<n>Z) in which the plane of the highest field value is held at 0 and
never computed, for ternary weights re-packed so that this value stands for a zero weight, and in a
"top unused" form (DS_PLANES_ASM_B<n>U) for layers whose codes never carry that value: the plane does
not exist (one shift fewer per pixel row and reduction index) and in the 64-channel form of 4-bit
fields its three registers hold a third slot of the activation prefetch ring.

Register map (R = 3 pixels per lane, J = 32 channels, NUM = 32 // (BITS + 1) codes per word, D = depth
of the activation prefetch ring in reduction slots, a divisor of NUM):
    v[8 + R*(i % D) + r]      prefetched activation of reduction slot i, row r (loaded D slots ahead)
    v[8 + R*D + P*r + s]      plane[r][s], P = 2^BITS
    v[66 + 32*r + j]          acc[r][j]                                   (asm operands %0..%5)
162 registers for 4-bit fields, which with the few the surrounding C++ needs stays within the 168 that
let three waves share a SIMD.
    s[36:67]                  16-bit codes of the 32 channels for the two reduction slots being accumulated
    s[68:99]                  the next two slots' codes (in flight meanwhile)
    s4..s6                    walk over the reduction index: element offset, fw, fh of the next k to load
    s7..s15                   temporaries, loop counter, word pointer

Every loop also comes in a "wide" form (suffix W) for layers whose channel count is a multiple of 64:
J = 64 channels per lane, so the planes are shared by twice as many terms (1 + 2^BITS/64 vector
instructions per term) and ROWS_WIDE = 2 pixel rows: a code then costs two scalar and two vector
instructions, a pattern that the two waves of a SIMD interleave without gaps (with three rows the
vector pipe idled 13 % of the time in a compute-only replica of the loop).  It keeps 128 accumulators
in v[64 + 64*r + j], runs at two waves per SIMD, reads one code row per reduction slot -- word j holds
the codes of channels j (low half) and j + 32 (high half) -- alternates between the two SGPR sets
instead of copying, moves its code pointer and checks its priority turn once per K group.
A third family (DS_PAIRS_ASM_B<n>, fields of 1 or 2 bits) serves int8 activations: a lane register
holds TWO pixels, hi * 65536 + lo, the planes are built with packed 16-bit shifts, the sign of a code
selects a negated plane instead of an xor mask (plane index = field, 2^BITS + field for a negative
code, 2^(BITS+1) for a zero weight or a code past K: a plane held at 0), and one 32-bit v_add_u32
accumulates both pixels: (64 + 3 * 2^BITS + 1) / 128 vector instructions per term.  Each half holds 255
terms of an int8 activation, so the caller runs at most that many reduction slots per call.
    v[8 + 6*(i % D) + 2r + h]     prefetched activation of slot i, row r, pixel half h
    v[8 + 6*D + (2P+1)*r + idx]   planes of row r
    v[64 + 64*r + j]              acc[r][j], pixel 2r in the low half, pixel 2r + 1 in the high half
Its operands: %6..%11 per-pixel byte offsets, %12 descriptor, %13 word pointer, %14 groups,
%15..%22 the walk.

For 3- and 4-bit fields the int8 family has no room for negated planes; DS_PAIRX_ASM_B<n> keeps the
xor-mask form of the int32 loops on the two-pixel planes instead: acc = (plane[M0] ^ mask) + acc with
mask 0 or -1.  ~p = -p - 1 as a 32-bit number, so a negative term subtracts one from the LOW half only:
the caller adds the count of negative codes back to the pixels that live in low halves.  The highest
field value is reserved for "no contribution" (zero weights, reduction indices past K): its plane is
held at 0.  One activation slot is prefetched (D = 1: 6 ring + 48 plane registers for 4-bit fields).

Operands: %6..%8 per-row byte offsets (VGPR), %9 buffer descriptor, %10 word pointer, %11 number of
K groups, %12..%14 initial walk state (offset, fw, fh), %15 FW, %16 FH, %17 offset step when fw wraps,
%18 offset step when fh wraps, %19 largest valid offset (the walk runs D slots ahead and is clamped).
"""
import os

R = 3                                    # pixel rows per lane (the int8 forms: rows of two pixels)
ROWS_WIDE = 2                            # ... of the 64-channel int32 form
DEPTH = {1: 4, 2: 5, 3: 4, 4: 3}        # prefetch ring depth, 32-channel form
DEPTH_WIDE = {1: 4, 2: 5, 3: 4, 4: 3}   # 64-channel form
DEPTH_NARROW = {1: 4, 2: 5, 3: 4, 4: 3} # 32-channel form with two pixel rows
DEPTH_WIDE_U = {1: 4, 2: 5, 3: 4, 4: 3}  # 64-channel form without the top plane: its registers buy a third slot
DEPTH_PAIRED = {1: 4, 2: 2, 3: 1, 4: 1}  # int8 forms: six activation registers per slot
DEPTH_PAIRED_U = {1: 4, 2: 5}            # index forms without the planes of the top field value


class Form:
    """Register and operand layout of the 32-channel (wide=False) or 64-channel loop."""

    def __init__(self, bits, wide, paired=False, narrow=False):
        self.paired = paired
        self.J = 64 if wide else 32
        self.acc = 64 if wide or narrow else 66
        self.depth = (DEPTH_WIDE if wide else DEPTH_NARROW if narrow else DEPTH)[bits]
        self.waves = 2 if wide else 4 if narrow else 3
        self.R = ROWS_WIDE if (wide and not paired) or narrow else R
        nacc = 2 * self.R                       # accumulator operands, 16 or 32 registers each
        nx = 2 * R if paired else self.R        # activation offsets: one per pixel held by a lane
        if paired:
            self.depth = DEPTH_PAIRED[bits]
        self.op_xoff, self.op_rsrc, self.op_wptr, self.op_groups, self.op_walk = (
            nacc, nacc + nx, nacc + nx + 1, nacc + nx + 2, nacc + nx + 3)


XP = 8
W = 36
WS = 68
KOFF, FWC, FHC = 4, 5, 6
CNT, T0, T1, IDX, MASK, KB = 7, 8, 9, 10, 11, 12
WP = 14
PRIO = 13
TIME = 34


def load_words(dst=WS, offset=0):
    return ["s_load_dwordx16 s[%d:%d], s[%d:%d], 0x%x" % (dst, dst + 15, WP, WP + 1, offset),
            "s_load_dwordx16 s[%d:%d], s[%d:%d], 0x%x" % (dst + 16, dst + 31, WP, WP + 1, offset + 0x40)]


def walk_and_load(slot, f):
    """Issue the R loads of the walk's current k into ring slot `slot`, then step the walk to k + 1."""
    OP_XOFF, OP_RSRC, OP_WALK = f.op_xoff, f.op_rsrc, f.op_walk
    fw_end, fh_end, row_step, plane_step, koff_max = (OP_WALK + 3, OP_WALK + 4, OP_WALK + 5, OP_WALK + 6,
                                                      OP_WALK + 7)
    if f.paired:
        # int8 activations: element offsets are byte offsets; two pixels per row
        L = ["s_min_u32 s%d, s%d, %%%d" % (KB, KOFF, koff_max)]
        L += ["buffer_load_sbyte v%d, %%%d, %%%d, s%d offen" % (XP + 2 * R * slot + q, OP_XOFF + q, OP_RSRC, KB)
              for q in range(2 * R)]
    else:
        # int32 activations: the walk keeps byte offsets (the caller passes its steps times four)
        L = ["s_min_u32 s%d, s%d, %%%d" % (KB, KOFF, koff_max)]
        L += ["buffer_load_dword v%d, %%%d, %%%d, s%d offen" % (XP + f.R * slot + r, OP_XOFF + r, OP_RSRC, KB)
              for r in range(f.R)]
        # fw += 1, wrapping into fh, wrapping into the next input channel; row_step already contains
        # the ordinary step of one element, s_cmov / s_cselect leave the wrap flag in SCC for the add
        return L + ["s_add_u32 s%d, s%d, 1" % (FWC, FWC),
                    "s_cmp_eq_u32 s%d, %%%d" % (FWC, fw_end),
                    "s_cmov_b32 s%d, 0" % FWC,
                    "s_cselect_b32 s%d, %%%d, 4" % (T0, row_step),
                    "s_addc_u32 s%d, s%d, 0" % (FHC, FHC),
                    "s_add_u32 s%d, s%d, s%d" % (KOFF, KOFF, T0),
                    "s_cmp_eq_u32 s%d, %%%d" % (FHC, fh_end),
                    "s_cmov_b32 s%d, 0" % FHC,
                    "s_cselect_b32 s%d, %%%d, 0" % (T0, plane_step),
                    "s_add_u32 s%d, s%d, s%d" % (KOFF, KOFF, T0)]
    L += ["s_add_u32 s%d, s%d, 1" % (FWC, FWC),
          "s_add_u32 s%d, s%d, 1" % (KOFF, KOFF),
          "s_cmp_eq_u32 s%d, %%%d" % (FWC, fw_end),
          "s_cselect_b32 s%d, 0, s%d" % (FWC, FWC),
          "s_cselect_b32 s%d, %%%d, 0" % (T0, row_step),
          "s_cselect_b32 s%d, 1, 0" % T1,
          "s_add_u32 s%d, s%d, s%d" % (KOFF, KOFF, T0),
          "s_add_u32 s%d, s%d, s%d" % (FHC, FHC, T1),
          "s_cmp_eq_u32 s%d, %%%d" % (FHC, fh_end),
          "s_cselect_b32 s%d, 0, s%d" % (FHC, FHC),
          "s_cselect_b32 s%d, %%%d, 0" % (T0, plane_step),
          "s_add_u32 s%d, s%d, s%d" % (KOFF, KOFF, T0)]
    return L


def take_turn(tag, waves):
    """The waves that share a SIMD take turns at the issue priorities, by the clock: with equal
    priorities the arbiter favours the oldest wave, which then finishes early and leaves the others
    with a SIMD they cannot fill (a wave cannot overlap its own scalar and vector work).  A turn is
    41 us (bit 12 of the 100 MHz counter up) and is checked with every code row, because the wave that
    should take over is the one that is running slowly.  Three waves rotate through priorities 2, 1,
    0; two waves swap 2 and 0."""
    hi, mid, end = "%d" % (20 + tag), "%d" % (40 + tag), "%d" % (60 + tag)
    if waves == 4:
        return []   # four waves of one workgroup meet at its barrier anyway: no turns
    if waves == 2:
        # (the prologue of the 64-channel form reduced PRIO to its low bit: T1 holds a constant there)
        return ["s_bfe_u32 s%d, s%d, 0x1000c" % (T0, TIME),
                "s_cmp_eq_u32 s%d, s%d" % (T0, PRIO), "s_cbranch_scc1 %sf" % hi,
                "s_setprio 0", "s_branch %sf" % end,
                hi + ":", "s_setprio 2",
                end + ":"]
    return ["s_bfe_u32 s%d, s%d, 0xe000c" % (T0, TIME),          # 14 bits of turn counter
            "s_mul_i32 s%d, s%d, 0x5556" % (T1, T0),
            "s_lshr_b32 s%d, s%d, 16" % (T1, T1),                # turn counter / 3
            "s_mul_i32 s%d, s%d, 3" % (T1, T1),
            "s_sub_u32 s%d, s%d, s%d" % (T0, T0, T1),            # turn = counter mod 3
            "s_sub_i32 s%d, s%d, s%d" % (T0, PRIO, T0),          # wave slot relative to the turn
            "s_cmp_lt_i32 s%d, 0" % T0,
            "s_cselect_b32 s%d, 3, 0" % T1,
            "s_add_u32 s%d, s%d, s%d" % (T0, T0, T1),
            "s_cmp_eq_u32 s%d, 0" % T0, "s_cbranch_scc1 %sf" % hi,
            "s_cmp_eq_u32 s%d, 1" % T0, "s_cbranch_scc1 %sf" % mid,
            "s_setprio 0", "s_branch %sf" % end,
            hi + ":", "s_setprio 2", "s_branch %sf" % end,
            mid + ":", "s_setprio 1",
            end + ":"]


def body(bits, zero_top=False, wide=False, unused_top=False, narrow=False):
    """zero_top: the plane of the highest field value is held at 0 (it stands for a zero weight).
    unused_top: no code carries the highest field value, so its plane does not exist: PS planes per
    row instead of P, and in the 64-channel form of 4-bit fields room for a third prefetch slot."""
    assert not (zero_top and unused_top) and not (wide and narrow)
    f = Form(bits, wide, narrow=narrow)
    if unused_top and wide:
        f.depth = DEPTH_WIDE_U[bits]
    R = f.R
    cb = bits + 1
    num = 32 // cb
    P = 1 << bits
    PS = P - 1 if unused_top else P             # planes per row = register stride between rows
    D, ACC = f.depth, f.acc
    assert num % D == 0 and num % 2 == 0
    PL = XP + R * D
    assert PL + PS * R <= ACC and ACC + R * f.J <= (128 if narrow else 256)
    L = []
    # ---- prologue: mutable copies of the inputs, the first activation loads and code row
    L += ["s_getreg_b32 s%d, hwreg(HW_REG_HW_ID, 0, 4)" % PRIO,  # the wave's slot on its SIMD
          "s_mov_b32 s%d, %%%d" % (CNT, f.op_groups),
          "s_mov_b64 s[%d:%d], %%%d" % (WP, WP + 1, f.op_wptr),
          "s_mov_b32 s%d, %%%d" % (KOFF, f.op_walk), "s_mov_b32 s%d, %%%d" % (FWC, f.op_walk + 1),
          "s_mov_b32 s%d, %%%d" % (FHC, f.op_walk + 2)]
    if wide:
        # the loop adds a group's 128 * num bytes before its first use of the pointer
        L += ["s_sub_u32 s%d, s%d, %d" % (WP, WP, 128 * num), "s_subb_u32 s%d, s%d, 0" % (WP + 1, WP + 1)]
        L += load_words(W, 128 * num)
    else:
        L += load_words(WS)
    L += ["s_memrealtime s[%d:%d]" % (TIME, TIME + 1)]
    for i in range(D):
        L += walk_and_load(i, f)
    if zero_top:
        # the highest field value contributes nothing: its plane is 0, once and for all
        L += ["v_mov_b32 v%d, 0" % (PL + PS * r + P - 1) for r in range(R)]
    L += ["s_mov_b32 s%d, 0" % IDX, "s_set_gpr_idx_on s%d, 0x1" % IDX]  # src0 of vector ops is M0-relative
    if wide:
        # The bit-field descriptors of the two sign bits (width 1, offset 8 / 24) live in scalar registers:
        # as literals they would make each s_bfe_i32 eight bytes long, 4 of the 28 bytes of code per weight
        # code, and the loop draws close to what the instruction cache delivers.
        L += ["s_and_b32 s%d, s%d, 1" % (PRIO, PRIO),
              "s_mov_b32 s%d, 0x10008" % IDX, "s_mov_b32 s%d, 0x10018" % T1]
    # ---- one K group per iteration
    L += ["1:"]
    for i in range(num):
        if wide:
            # one code row per reduction slot; the two SGPR sets alternate (NUM is even, so the set
            # of slot 0 is the same in every group), the other set receives the next slot's row (one
            # row past the end reads the spare row that follows the codes in the weight blob)
            cur, nxt = (W, WS) if i % 2 == 0 else (WS, W)
            L += ["s_waitcnt lgkmcnt(0)"]
            if i == 0:
                # the word pointer moves once per group (no load is in flight here); the rows of the
                # group are at fixed offsets from it
                L += ["s_add_u32 s%d, s%d, %d" % (WP, WP, 128 * num), "s_addc_u32 s%d, s%d, 0" % (WP + 1, WP + 1)]
                L += take_turn(0, f.waves)  # once per K group: a group is a few us, a turn 41
            L += load_words(nxt, 128 * (i + 1))
            if i == num - 1:
                L += ["s_memrealtime s[%d:%d]" % (TIME, TIME + 1)]  # read at the next turn check
        elif i % 2 == 0:
            # one code row per two reduction slots: this row's codes leave the staging registers,
            # which then receive the next row's
            cur = W
            L += ["s_add_u32 s%d, s%d, 128" % (WP, WP), "s_addc_u32 s%d, s%d, 0" % (WP + 1, WP + 1),
                  "s_waitcnt lgkmcnt(0)"]
            L += take_turn(i // 2, f.waves)
            L += ["s_mov_b64 s[%d:%d], s[%d:%d]" % (W + 2 * q, W + 2 * q + 1, WS + 2 * q, WS + 2 * q + 1)
                  for q in range(16)]
            L += load_words(WS)
            L += ["s_memrealtime s[%d:%d]" % (TIME, TIME + 1)]  # read when the next row arrives
        slot = i % D
        L += ["s_waitcnt vmcnt(%d)" % (R * (D - 1))]
        # plane 0 = the activation itself (a shift by 0 keeps src0 a constant: not M0-relative)
        for r in range(R):
            L += ["v_ashrrev_i32 v%d, 0, v%d" % (PL + PS * r, XP + R * slot + r)]
        L += walk_and_load(slot, f)  # the ring slot is free again: load reduction slot i + D into it
        for s in range(1, P):
            for r in range(R):
                if (zero_top or unused_top) and s == P - 1:
                    continue  # held at 0 since the prologue, or absent
                else:
                    L += ["v_ashrrev_i32 v%d, %d, v%d" % (PL + PS * r + s, s, PL + PS * r)]
        # the 16-bit code is a ready M0 value: plane index in 7:0, "src0 relative" in 15:12.  32-channel
        # form: low / high half = even / odd slot of the row; 64-channel form: channel j / j + 32.
        halves = (0, 1) if wide else (i % 2,)
        for half in halves:
            for j in range(32):
                if half == 0:
                    L += ["s_mov_b32 m0, s%d" % (cur + j)]
                else:
                    L += ["s_lshr_b32 m0, s%d, 16" % (cur + j)]
                if wide:
                    L += ["s_bfe_i32 s%d, s%d, s%d" % (MASK, cur + j, T1 if half else IDX)]
                else:
                    L += ["s_bfe_i32 s%d, s%d, 0x%x" % (MASK, cur + j, (1 << 16) | (16 * half + 8))]
                ch = j + 32 * half if wide else j
                for r in range(R):
                    a = ACC + f.J * r + ch
                    L += ["v_xad_u32 v%d, v%d, s%d, v%d" % (a, PL + PS * r, MASK, a)]
    L += ["s_sub_u32 s%d, s%d, 1" % (CNT, CNT), "s_cmp_lg_u32 s%d, 0" % CNT, "s_cbranch_scc1 1b"]
    # ---- leave relative addressing, drain the loads that ran ahead of the last slot
    L += ["s_set_gpr_idx_off", "s_setprio %d" % (3 if wide else 0), "s_waitcnt vmcnt(0) lgkmcnt(0)"]
    return L


def clobbers(bits, wide=False, unused_top=False, narrow=False):
    f = Form(bits, wide, narrow=narrow)
    if unused_top and wide:
        f.depth = DEPTH_WIDE_U[bits]
    P = (1 << bits) - (1 if unused_top else 0)
    v = ['"v%d"' % n for n in range(XP, XP + f.R * f.depth + P * f.R)]
    s = ['"s%d"' % n for n in list(range(4, 16)) + list(range(W, WS + 32)) + [TIME, TIME + 1]]
    return ", ".join(v + s + ['"scc"', '"memory"'])


def body_paired(bits, unused_top=False):
    """The int8 form: 3 rows x 2 pixels x 64 channels per lane (see the module docstring).
    unused_top: no code carries the highest field value; P counts the shifts that exist, the plane
    indices close up (field, P + field, 2P) and the registers saved deepen the prefetch ring."""
    f = Form(bits, True, paired=True)
    if unused_top:
        f.depth = DEPTH_PAIRED_U[bits]
    num = 32 // (bits + 1)
    P = (1 << bits) - (1 if unused_top else 0)
    S = 2 * P + 1                               # planes per row: shifts, negated shifts, zero
    D, ACC = f.depth, f.acc
    assert num % D == 0 and num % 2 == 0
    PL = XP + 2 * R * D
    assert PL + S * R <= ACC and ACC + R * f.J <= 256
    L = []
    L += ["s_getreg_b32 s%d, hwreg(HW_REG_HW_ID, 0, 4)" % PRIO,
          "s_mov_b32 s%d, %%%d" % (CNT, f.op_groups),
          "s_mov_b64 s[%d:%d], %%%d" % (WP, WP + 1, f.op_wptr),
          "s_mov_b32 s%d, %%%d" % (KOFF, f.op_walk), "s_mov_b32 s%d, %%%d" % (FWC, f.op_walk + 1),
          "s_mov_b32 s%d, %%%d" % (FHC, f.op_walk + 2),
          "s_mov_b32 s%d, 0x05040100" % MASK,   # v_perm_b32 selector: low halves of (src0, src1)
          "s_and_b32 s%d, s%d, 1" % (PRIO, PRIO)]
    L += load_words(W)
    L += ["s_memrealtime s[%d:%d]" % (TIME, TIME + 1)]
    for i in range(D):
        L += walk_and_load(i, f)
    for r in range(R):
        L += ["v_mov_b32 v%d, 0" % (PL + S * r + 2 * P)]
    L += ["s_mov_b32 s%d, 0" % IDX]
    L += ["1:"]
    for i in range(num):
        cur, nxt = (W, WS) if i % 2 == 0 else (WS, W)
        L += ["s_add_u32 s%d, s%d, 128" % (WP, WP), "s_addc_u32 s%d, s%d, 0" % (WP + 1, WP + 1),
              "s_waitcnt lgkmcnt(0)"]
        if i % 2 == 0:
            L += take_turn(i // 2, f.waves)
        L += load_words(nxt)
        if i % 2 == 1:
            L += ["s_memrealtime s[%d:%d]" % (TIME, TIME + 1)]
        slot = i % D
        L += ["s_waitcnt vmcnt(%d)" % (2 * R * (D - 1))]
        # The planes, with relative addressing off (these instructions name two vector registers).
        # A plane holds hi * 65536 + lo as ONE 32-bit number (lo signed), so that the full-rate 32-bit
        # add accumulates both pixels: borrows of a negative lo run into the high half and come out
        # again when the sum is split.  Per row: pk = the two activations as 16-bit fields (into the
        # register of pixel b), c = 65536 where pixel a is negative (into its own register: a >> f has
        # the sign of a), then p[f] = (pk >> f per half) - c and the negated planes 0 - p[f].
        L += ["s_set_gpr_idx_off"]
        for r in range(R):
            lo, hi = XP + 2 * R * slot + 2 * r, XP + 2 * R * slot + 2 * r + 1
            L += ["v_perm_b32 v%d, v%d, v%d, s%d" % (hi, hi, lo, MASK),
                  "v_and_b32 v%d, 0x10000, v%d" % (lo, lo),
                  "v_sub_u32 v%d, v%d, v%d" % (PL + S * r, hi, lo)]
        for s in range(1, P):
            for r in range(R):
                lo, hi = XP + 2 * R * slot + 2 * r, XP + 2 * R * slot + 2 * r + 1
                L += ["v_pk_ashrrev_i16 v%d, %d, v%d op_sel_hi:[0,1]" % (PL + S * r + s, s, hi)]
        for s in range(1, P):
            for r in range(R):
                lo = XP + 2 * R * slot + 2 * r
                L += ["v_sub_u32 v%d, v%d, v%d" % (PL + S * r + s, PL + S * r + s, lo)]
        for s in range(P):
            for r in range(R):
                L += ["v_sub_u32 v%d, 0, v%d" % (PL + S * r + P + s, PL + S * r + s)]
        L += walk_and_load(slot, f)  # the ring slot is free again
        L += ["s_set_gpr_idx_on s%d, 0x1" % IDX]
        # the 16-bit code is the M0 value itself: plane index in 7:0, "src0 relative" in 15:12
        for half in (0, 1):
            for j in range(32):
                if half == 0:
                    L += ["s_mov_b32 m0, s%d" % (cur + j)]
                else:
                    L += ["s_lshr_b32 m0, s%d, 16" % (cur + j)]
                for r in range(R):
                    a = ACC + f.J * r + j + 32 * half
                    L += ["v_add_u32 v%d, v%d, v%d" % (a, PL + S * r, a)]
    L += ["s_sub_u32 s%d, s%d, 1" % (CNT, CNT), "s_cmp_lg_u32 s%d, 0" % CNT, "s_cbranch_scc1 1b"]
    L += ["s_set_gpr_idx_off", "s_setprio 0", "s_waitcnt vmcnt(0) lgkmcnt(0)"]
    return L


def body_pairx(bits):
    """The int8 form for 3- and 4-bit fields: two pixels per register, xor-mask signs."""
    f = Form(bits, True, paired=True)
    num = 32 // (bits + 1)
    P = 1 << bits
    S = P                                       # planes per row; plane P - 1 stays 0
    D, ACC = 1, f.acc
    PL = XP + 2 * R * D
    assert PL + S * R <= ACC and ACC + R * f.J <= 256 and num % 2 == 0
    SEL = IDX                                   # the relative-addressing switch takes a constant here
    L = []
    L += ["s_getreg_b32 s%d, hwreg(HW_REG_HW_ID, 0, 4)" % PRIO,
          "s_mov_b32 s%d, %%%d" % (CNT, f.op_groups),
          "s_mov_b64 s[%d:%d], %%%d" % (WP, WP + 1, f.op_wptr),
          "s_mov_b32 s%d, %%%d" % (KOFF, f.op_walk), "s_mov_b32 s%d, %%%d" % (FWC, f.op_walk + 1),
          "s_mov_b32 s%d, %%%d" % (FHC, f.op_walk + 2),
          "s_mov_b32 s%d, 0x05040100" % SEL,    # v_perm_b32 selector: low halves of (src0, src1)
          "s_and_b32 s%d, s%d, 1" % (PRIO, PRIO)]
    L += load_words(W)
    L += ["s_memrealtime s[%d:%d]" % (TIME, TIME + 1)]
    L += walk_and_load(0, f)
    for r in range(R):
        L += ["v_mov_b32 v%d, 0" % (PL + S * r + P - 1)]
    L += ["1:"]
    for i in range(num):
        cur, nxt = (W, WS) if i % 2 == 0 else (WS, W)
        L += ["s_add_u32 s%d, s%d, 128" % (WP, WP), "s_addc_u32 s%d, s%d, 0" % (WP + 1, WP + 1),
              "s_waitcnt lgkmcnt(0)"]
        if i % 2 == 0:
            L += take_turn(i // 2, f.waves)
        L += load_words(nxt)
        if i % 2 == 1:
            L += ["s_memrealtime s[%d:%d]" % (TIME, TIME + 1)]
        L += ["s_waitcnt vmcnt(0)", "s_set_gpr_idx_off"]
        for r in range(R):
            lo, hi = XP + 2 * r, XP + 2 * r + 1
            L += ["v_perm_b32 v%d, v%d, v%d, s%d" % (hi, hi, lo, SEL),      # both pixels as 16-bit fields
                  "v_and_b32 v%d, 0x10000, v%d" % (lo, lo),                 # 65536 where pixel a < 0
                  "v_sub_u32 v%d, v%d, v%d" % (PL + S * r, hi, lo)]         # plane 0 = hi * 65536 + lo
        for s in range(1, P - 1):
            for r in range(R):
                L += ["v_pk_ashrrev_i16 v%d, %d, v%d op_sel_hi:[0,1]" % (PL + S * r + s, s, XP + 2 * r + 1)]
        for s in range(1, P - 1):
            for r in range(R):
                L += ["v_sub_u32 v%d, v%d, v%d" % (PL + S * r + s, PL + S * r + s, XP + 2 * r)]
        L += walk_and_load(0, f)                # the ring is free again: the next slot's activations
        L += ["s_set_gpr_idx_on s%d, 0x1" % PRIO]
        for half in (0, 1):
            for j in range(32):
                if half == 0:
                    L += ["s_mov_b32 m0, s%d" % (cur + j)]
                else:
                    L += ["s_lshr_b32 m0, s%d, 16" % (cur + j)]
                L += ["s_bfe_i32 s%d, s%d, 0x%x" % (MASK, cur + j, (1 << 16) | (16 * half + 8))]
                for r in range(R):
                    a = ACC + f.J * r + j + 32 * half
                    L += ["v_xad_u32 v%d, v%d, s%d, v%d" % (a, PL + S * r, MASK, a)]
    L += ["s_sub_u32 s%d, s%d, 1" % (CNT, CNT), "s_cmp_lg_u32 s%d, 0" % CNT, "s_cbranch_scc1 1b"]
    L += ["s_set_gpr_idx_off", "s_setprio 0", "s_waitcnt vmcnt(0) lgkmcnt(0)"]
    return L


def clobbers_pairx(bits):
    P = 1 << bits
    v = ['"v%d"' % n for n in range(XP, XP + 2 * R + P * R)]
    s = ['"s%d"' % n for n in list(range(4, 16)) + list(range(W, WS + 32)) + [TIME, TIME + 1]]
    return ", ".join(v + s + ['"scc"', '"memory"'])


def clobbers_paired(bits, unused_top=False):
    f = Form(bits, True, paired=True)
    if unused_top:
        f.depth = DEPTH_PAIRED_U[bits]
    P = (1 << bits) - (1 if unused_top else 0)
    v = ['"v%d"' % n for n in range(XP, XP + 2 * R * f.depth + (2 * P + 1) * R)]
    s = ['"s%d"' % n for n in list(range(4, 16)) + list(range(W, WS + 32)) + [TIME, TIME + 1]]
    return ", ".join(v + s + ['"scc"', '"memory"'])


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    out = ["// Generated by gen_planes_asm.py -- do not edit by hand.", ""]
    for wide, wtag in ((False, ""), (True, "W")):
        for bits in (1, 2, 3, 4):
            for zero_top, tag in ((False, ""), (True, "Z"), (False, "U")):
                lines = body(bits, zero_top, wide, unused_top=tag == "U")
                out.append("#define DS_PLANES_ASM_B%d%s%s \\" % (bits, tag, wtag))
                out.append(" \\\n".join('    "%s\\n"' % line for line in lines))
                out.append("")
            out.append("#define DS_PLANES_CLOBBERS_B%d%s %s" % (bits, wtag, clobbers(bits, wide)))
            out.append("#define DS_PLANES_CLOBBERS_B%dU%s %s" % (bits, wtag, clobbers(bits, wide, True)))
            out.append("")
    for bits in (1, 2, 3, 4):
        for zero_top, tag in ((False, ""), (True, "Z"), (False, "U")):
            lines = body(bits, zero_top, False, unused_top=tag == "U", narrow=True)
            out.append("#define DS_PLANES_ASM_B%d%sN \\" % (bits, tag))
            out.append(" \\\n".join('    "%s\\n"' % line for line in lines))
            out.append("")
        out.append("#define DS_PLANES_CLOBBERS_B%dN %s" % (bits, clobbers(bits, narrow=True)))
        out.append("#define DS_PLANES_CLOBBERS_B%dUN %s" % (bits, clobbers(bits, unused_top=True, narrow=True)))
        out.append("")
    for bits in (1, 2):
        out.append("#define DS_PAIRS_ASM_B%d \\" % bits)
        out.append(" \\\n".join('    "%s\\n"' % line for line in body_paired(bits)))
        out.append("")
        out.append("#define DS_PAIRS_CLOBBERS_B%d %s" % (bits, clobbers_paired(bits)))
        out.append("")
        out.append("#define DS_PAIRS_ASM_B%dU \\" % bits)
        out.append(" \\\n".join('    "%s\\n"' % line for line in body_paired(bits, True)))
        out.append("")
        out.append("#define DS_PAIRS_CLOBBERS_B%dU %s" % (bits, clobbers_paired(bits, True)))
        out.append("")
    for bits in (3, 4):
        out.append("#define DS_PAIRX_ASM_B%d \\" % bits)
        out.append(" \\\n".join('    "%s\\n"' % line for line in body_pairx(bits)))
        out.append("")
        out.append("#define DS_PAIRX_CLOBBERS_B%d %s" % (bits, clobbers_pairx(bits)))
        out.append("")
    with open(os.path.join(here, "ds_planes_asm.inc"), "w") as f:
        f.write("\n".join(out))


if __name__ == "__main__":
    main()
