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
a "zero top" form (DS_PLANES_ASM_B<n>Z) for ternary weights: the highest field value stands for a
zero weight and its plane is 0 instead of x >> (2^BITS - 1).

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
Operands: %6..%8 per-row byte offsets (VGPR), %9 buffer descriptor, %10 word pointer, %11 number of
K groups, %12..%14 initial walk state (offset, fw, fh), %15 FW, %16 FH, %17 offset step when fw wraps,
%18 offset step when fh wraps, %19 largest valid offset (the walk runs D slots ahead and is clamped).
"""
import os

R, J = 3, 32
ACC = 66
DEPTH = {1: 4, 2: 5, 3: 4, 4: 3}
OP_XOFF, OP_RSRC, OP_WPTR, OP_GROUPS, OP_WALK = 6, 9, 10, 11, 12
XP = 8
W = 36
WS = 68
KOFF, FWC, FHC = 4, 5, 6
CNT, T0, T1, IDX, MASK, KB = 7, 8, 9, 10, 11, 12
WP = 14
PRIO = 13
TIME = 34


def load_words():
    return ["s_load_dwordx16 s[%d:%d], s[%d:%d], 0x0" % (WS, WS + 15, WP, WP + 1),
            "s_load_dwordx16 s[%d:%d], s[%d:%d], 0x40" % (WS + 16, WS + 31, WP, WP + 1)]


def walk_and_load(slot):
    """Issue the R loads of the walk's current k into ring slot `slot`, then step the walk to k + 1."""
    fw_end, fh_end, row_step, plane_step, koff_max = (OP_WALK + 3, OP_WALK + 4, OP_WALK + 5, OP_WALK + 6,
                                                      OP_WALK + 7)
    L = ["s_min_u32 s%d, s%d, %%%d" % (T0, KOFF, koff_max),
         "s_lshl_b32 s%d, s%d, 2" % (KB, T0)]
    L += ["buffer_load_dword v%d, %%%d, %%%d, s%d offen" % (XP + R * slot + r, OP_XOFF + r, OP_RSRC, KB)
          for r in range(R)]
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


def take_turn(tag):
    """The waves that share a SIMD take turns at the issue priorities 2, 1, 0, by the clock: with equal
    priorities the arbiter favours the oldest wave, which then finishes early and leaves the others
    with a SIMD they cannot fill (a wave cannot overlap its own scalar and vector work).  The turn is
    41 us (bit 12 of the 100 MHz counter) and is checked with every code row, because the wave that
    should take over is the one that is running slowly."""
    hi, mid, end = "%d" % (20 + tag), "%d" % (40 + tag), "%d" % (60 + tag)
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


def body(bits, zero_top=False):
    cb = bits + 1
    num = 32 // cb
    P = 1 << bits
    D = DEPTH[bits]
    assert num % D == 0 and num % 2 == 0
    PL = XP + R * D
    assert PL + P * R <= ACC
    L = []
    # ---- prologue: mutable copies of the inputs, the first activation loads and code row
    L += ["s_getreg_b32 s%d, hwreg(HW_REG_HW_ID, 0, 4)" % PRIO,  # the wave's slot on its SIMD
          "s_mov_b32 s%d, %%%d" % (CNT, OP_GROUPS),
          "s_mov_b64 s[%d:%d], %%%d" % (WP, WP + 1, OP_WPTR),
          "s_mov_b32 s%d, %%%d" % (KOFF, OP_WALK), "s_mov_b32 s%d, %%%d" % (FWC, OP_WALK + 1),
          "s_mov_b32 s%d, %%%d" % (FHC, OP_WALK + 2)]
    L += load_words()
    L += ["s_memrealtime s[%d:%d]" % (TIME, TIME + 1)]
    for i in range(D):
        L += walk_and_load(i)
    L += ["s_mov_b32 s%d, 0" % IDX, "s_set_gpr_idx_on s%d, 0x1" % IDX]  # src0 of vector ops is M0-relative
    # ---- one K group per iteration, two reduction slots (one row of 16-bit codes) at a time
    L += ["1:"]
    for i in range(num):
        if i % 2 == 0:
            # this row's codes leave the staging registers, which then receive the next row's (one
            # row past the end reads the spare row that follows the codes in the weight blob)
            L += ["s_add_u32 s%d, s%d, 128" % (WP, WP), "s_addc_u32 s%d, s%d, 0" % (WP + 1, WP + 1),
                  "s_waitcnt lgkmcnt(0)"]
            L += take_turn(i // 2)
            L += ["s_mov_b64 s[%d:%d], s[%d:%d]" % (W + 2 * q, W + 2 * q + 1, WS + 2 * q, WS + 2 * q + 1)
                  for q in range(16)]
            L += load_words()
            L += ["s_memrealtime s[%d:%d]" % (TIME, TIME + 1)]  # read when the next row arrives
        slot = i % D
        L += ["s_waitcnt vmcnt(%d)" % (R * (D - 1))]
        # plane 0 = the activation itself (a shift by 0 keeps src0 a constant: not M0-relative)
        for r in range(R):
            L += ["v_ashrrev_i32 v%d, 0, v%d" % (PL + P * r, XP + R * slot + r)]
        L += walk_and_load(slot)  # the ring slot is free again: load reduction slot i + D into it
        for s in range(1, P):
            for r in range(R):
                if zero_top and s == P - 1:
                    # the highest field value encodes a zero weight: its plane is 0
                    L += ["v_mov_b32 v%d, 0" % (PL + P * r + s)]
                else:
                    L += ["v_ashrrev_i32 v%d, %d, v%d" % (PL + P * r + s, s, PL + P * r)]
        for j in range(J):
            # the 16-bit code is a ready M0 value: plane index in 7:0, "src0 relative" in 15:12
            if i % 2 == 0:
                L += ["s_mov_b32 m0, s%d" % (W + j)]
            else:
                L += ["s_lshr_b32 m0, s%d, 16" % (W + j)]
            L += ["s_bfe_i32 s%d, s%d, 0x%x" % (MASK, W + j, (1 << 16) | (16 * (i % 2) + 8))]
            for r in range(R):
                a = ACC + 32 * r + j
                L += ["v_xad_u32 v%d, v%d, s%d, v%d" % (a, PL + P * r, MASK, a)]
    L += ["s_sub_u32 s%d, s%d, 1" % (CNT, CNT), "s_cmp_lg_u32 s%d, 0" % CNT, "s_cbranch_scc1 1b"]
    # ---- leave relative addressing, drain the loads that ran ahead of the last slot
    L += ["s_set_gpr_idx_off", "s_setprio 0", "s_waitcnt vmcnt(0) lgkmcnt(0)"]
    return L


def clobbers(bits):
    num = 32 // (bits + 1)
    P = 1 << bits
    v = ['"v%d"' % n for n in range(XP, XP + R * DEPTH[bits] + P * R)]
    s = ['"s%d"' % n for n in list(range(4, 16)) + list(range(W, WS + 32)) + [TIME, TIME + 1]]
    return ", ".join(v + s + ['"scc"', '"memory"'])


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    out = ["// Generated by gen_planes_asm.py -- do not edit by hand.", ""]
    for bits in (1, 2, 3, 4):
        for zero_top, tag in ((False, ""), (True, "Z")):
            lines = body(bits, zero_top)
            out.append("#define DS_PLANES_ASM_B%d%s \\" % (bits, tag))
            out.append(" \\\n".join('    "%s\\n"' % line for line in lines))
            out.append("")
        out.append("#define DS_PLANES_CLOBBERS_B%d %s" % (bits, clobbers(bits)))
        out.append("")
    with open(os.path.join(here, "ds_planes_asm.inc"), "w") as f:
        f.write("\n".join(out))


if __name__ == "__main__":
    main()
