#!/usr/bin/env python3
"""Generates ds_planes_asm.inc: the hand-scheduled main loop of ds::shift_planes_kernel.

    python deepshift_amd/csrc/gen_planes_asm.py      # rewrites ds_planes_asm.inc next to this file

The loop is emitted as one inline-asm string per shift-field width BITS (1..4) because it uses
VGPR-relative addressing (s_set_gpr_idx_*), which needs a fixed register map:

    per reduction index k and pixel row r:  plane[r][s] = x >> s  for every shift amount s < 2^BITS
                                            (2^BITS vector shifts, shared by all 32 output channels)
    per (k, channel j):                     M0 <- the code's 16-bit pre-decoded form (scalar), mask <- sign
                                            acc[r][j] = (plane[r][M0] ^ mask) + acc[r][j]   (v_xad_u32)

so a shift-add term costs 1 + 2^BITS/32 vector instructions instead of 2.

Register map (R = 4 pixels per lane, J = 32 channels, NUM = 32 // (BITS + 1) codes per word):
    v[8 + 4*i + r]            prefetched activation of reduction slot i, row r (loaded one K group ahead)
    v[8 + 4*NUM + P*r + s]    plane[r][s], P = 2^BITS
    v[96 + 32*r + j]          acc[r][j]                                   (asm operands %0..%7)
    s[36:67]                  16-bit codes of the 32 channels for the two reduction slots being accumulated
    s[68:99]                  the next two slots' codes (in flight meanwhile)
    s4..s6                    walk over the reduction index: element offset, fw, fh of the next k to load
    s7..s15                   temporaries, loop counter, word pointer
Operands: %8..%11 per-row byte offsets (VGPR), %12 buffer descriptor, %13 word pointer, %14 number of
K groups, %15..%17 initial walk state (offset, fw, fh), %18 FW, %19 FH, %20 offset step when fw wraps,
%21 offset step when fh wraps, %22 largest valid offset (the walk runs one group ahead and is clamped).
"""
import os

R, J = 4, 32
ACC = 96
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


def walk_and_load(i):
    """Issue the R loads of the walk's current k into slot i, then step the walk to k + 1."""
    L = ["s_min_u32 s%d, s%d, %%22" % (T0, KOFF),
         "s_lshl_b32 s%d, s%d, 2" % (KB, T0)]
    L += ["buffer_load_dword v%d, %%%d, %%12, s%d offen" % (XP + 4 * i + r, 8 + r, KB) for r in range(R)]
    L += ["s_add_u32 s%d, s%d, 1" % (FWC, FWC),
          "s_add_u32 s%d, s%d, 1" % (KOFF, KOFF),
          "s_cmp_eq_u32 s%d, %%18" % FWC,
          "s_cselect_b32 s%d, 0, s%d" % (FWC, FWC),
          "s_cselect_b32 s%d, %%20, 0" % T0,
          "s_cselect_b32 s%d, 1, 0" % T1,
          "s_add_u32 s%d, s%d, s%d" % (KOFF, KOFF, T0),
          "s_add_u32 s%d, s%d, s%d" % (FHC, FHC, T1),
          "s_cmp_eq_u32 s%d, %%19" % FHC,
          "s_cselect_b32 s%d, 0, s%d" % (FHC, FHC),
          "s_cselect_b32 s%d, %%21, 0" % T0,
          "s_add_u32 s%d, s%d, s%d" % (KOFF, KOFF, T0)]
    return L


def body(bits):
    cb = bits + 1
    num = 32 // cb
    P = 1 << bits
    PL = XP + 4 * num
    assert PL + P * R <= ACC
    L = []
    # ---- prologue: mutable copies of the inputs, the first group's activation loads and words
    L += ["s_getreg_b32 s%d, hwreg(HW_REG_HW_ID, 0, 1)" % PRIO,  # parity of the wave slot on its SIMD
          "s_mov_b32 s%d, %%14" % CNT,
          "s_mov_b64 s[%d:%d], %%13" % (WP, WP + 1),
          "s_mov_b32 s%d, %%15" % KOFF, "s_mov_b32 s%d, %%16" % FWC, "s_mov_b32 s%d, %%17" % FHC]
    L += load_words()
    L += ["s_memrealtime s[%d:%d]" % (TIME, TIME + 1)]
    for i in range(num):
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
            # The two waves that share a SIMD take turns at the higher issue priority, by the clock:
            # bit 12 of the 100 MHz counter (41 us each) against the parity of the wave's slot.  With
            # equal priorities the arbiter favours the older wave, which then finishes early and
            # leaves the other alone on the SIMD.  The turn is checked every row, because the wave
            # that should take over is the one that is running slowly.
            L += ["s_bfe_u32 s%d, s%d, 0x1000c" % (T0, TIME), "s_cmp_eq_u32 s%d, s%d" % (T0, PRIO),
                  "s_cbranch_scc0 %df" % (3 + i), "s_setprio 2", "s_branch %df" % (4 + i),
                  "%d:" % (3 + i), "s_setprio 0", "%d:" % (4 + i)]
            L += ["s_mov_b64 s[%d:%d], s[%d:%d]" % (W + 2 * q, W + 2 * q + 1, WS + 2 * q, WS + 2 * q + 1)
                  for q in range(16)]
            L += load_words()
            L += ["s_memrealtime s[%d:%d]" % (TIME, TIME + 1)]  # read when the next row arrives
        L += ["s_waitcnt vmcnt(%d)" % (4 * (num - 1))]
        # plane 0 = the activation itself (a shift by 0 keeps src0 a constant: not M0-relative)
        for r in range(R):
            L += ["v_ashrrev_i32 v%d, 0, v%d" % (PL + P * r, XP + 4 * i + r)]
        L += walk_and_load(i)  # the same slot of the next group
        for s in range(1, P):
            for r in range(R):
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
    # ---- leave relative addressing, drain the loads issued for the group after the last one
    L += ["s_set_gpr_idx_off", "s_setprio 0", "s_waitcnt vmcnt(0) lgkmcnt(0)"]
    return L


def clobbers(bits):
    num = 32 // (bits + 1)
    P = 1 << bits
    v = ['"v%d"' % n for n in range(XP, XP + 4 * num + P * R)]
    s = ['"s%d"' % n for n in list(range(4, 16)) + list(range(W, WS + 32)) + [TIME, TIME + 1]]
    return ", ".join(v + s + ['"scc"', '"memory"'])


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    out = ["// Generated by gen_planes_asm.py -- do not edit by hand.", ""]
    for bits in (1, 2, 3, 4):
        lines = body(bits)
        out.append("#define DS_PLANES_ASM_B%d \\" % bits)
        out.append(" \\\n".join('    "%s\\n"' % line for line in lines))
        out.append("")
        out.append("#define DS_PLANES_CLOBBERS_B%d %s" % (bits, clobbers(bits)))
        out.append("")
    with open(os.path.join(here, "ds_planes_asm.inc"), "w") as f:
        f.write("\n".join(out))


if __name__ == "__main__":
    main()
