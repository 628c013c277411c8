#!/usr/bin/env python3
"""Generates ds_planes_asm.inc: the hand-scheduled main loop of ds::shift_planes_kernel.

    python deepshift_amd/csrc/gen_planes_asm.py      # rewrites ds_planes_asm.inc next to this file

The loop is emitted as one inline-asm string per shift-field width BITS (1..4) because it uses
VGPR-relative addressing (s_set_gpr_idx_*), which needs a fixed register map:

    per reduction index k and pixel row r:  plane[r][s] = x >> s  for every shift amount s < 2^BITS
                                            (2^BITS vector shifts, shared by all 32 output channels)
    per (k, channel j):                     M0 <- shift field of the code (scalar), mask <- sign
                                            acc[r][j] = (plane[r][M0] ^ mask) + acc[r][j]   (v_xad_u32)

so a shift-add term costs 1 + 2^BITS/32 vector instructions instead of 2.

Register map (R = 4 pixels per lane, J = 32 channels, NUM = 32 // (BITS + 1) codes per word):
    v[8 + 4*i + r]                       prefetched activation of reduction slot i, row r
    v[8 + 4*NUM + P*r + s]               plane[r][s], P = 2^BITS
    v[96 + 32*r + j]                     acc[r][j]                       (asm operands %0..%7)
    s[4:35] packed words of the 32 channels, s[36:67] the next group's words (loading),
    s[68:83] next group's k-table entries, s84..s93 temps
Operands: %8..%11 per-row byte offsets (VGPR), %12 buffer descriptor, %13 word pointer, %14 k-table
pointer, %15 number of K groups, %16 / %17 plane and row pitch of the activations (elements).
"""
import os

R, J = 4, 32
ACC = 96
XP = 8
W = 4           # s[4:35]   words of the group being accumulated
WS = 36         # s[36:67]  words of the next group (in flight while this one is accumulated)
KT = 68         # s[68:83]
CNT, T0, WP, KP, T1, IDX, MASK, KOFF = 84, 85, 86, 88, 90, 91, 92, 93


def sload(dst, n, ptr, off):
    return "s_load_dword%s s[%d:%d], s[%d:%d], 0x%x" % ("x%d" % n if n > 1 else "", dst, dst + n - 1,
                                                         ptr, ptr + 1, off) if n > 1 else \
        "s_load_dword s%d, s[%d:%d], 0x%x" % (dst, ptr, ptr + 1, off)


def load_ktab(num):
    """Scalar loads of `num` consecutive k-table entries into s[KT..]."""
    out, done = [], 0
    for n in (16, 8, 4, 2, 1):
        while num - done >= n:
            out.append(sload(KT + done, n, KP, done * 4))
            done += n
    return out


def koff(i):
    """KOFF <- 4 * (ic * plane + fh * row + fw) for k-table entry i (ic << 10 | fh << 5 | fw)."""
    v = KT + i
    return [
        "s_lshr_b32 s%d, s%d, 10" % (T0, v),
        "s_mul_i32 s%d, s%d, %%16" % (T0, T0),
        "s_bfe_u32 s%d, s%d, 0x50005" % (T1, v),
        "s_mul_i32 s%d, s%d, %%17" % (T1, T1),
        "s_add_u32 s%d, s%d, s%d" % (T0, T0, T1),
        "s_and_b32 s%d, s%d, 31" % (T1, v),
        "s_add_u32 s%d, s%d, s%d" % (T0, T0, T1),
        "s_lshl_b32 s%d, s%d, 2" % (KOFF, T0),
    ]


def issue_loads(i):
    return ["buffer_load_dword v%d, %%%d, %%12, s%d offen" % (XP + 4 * i + r, 8 + r, KOFF) for r in range(R)]


def body(bits):
    cb = bits + 1
    num = 32 // cb
    P = 1 << bits
    PL = XP + 4 * num
    assert PL + P * R <= ACC
    L = []
    # ---- prologue: copies of the mutable inputs, first group's activation loads
    L += ["s_mov_b32 s%d, %%15" % CNT,
          "s_mov_b64 s[%d:%d], %%13" % (WP, WP + 1),
          "s_mov_b64 s[%d:%d], %%14" % (KP, KP + 1)]
    L += load_ktab(num)
    L += ["s_waitcnt lgkmcnt(0)"]
    for i in range(num):
        L += koff(i) + issue_loads(i)
    L += ["s_add_u32 s%d, s%d, %d" % (KP, KP, num * 4), "s_addc_u32 s%d, s%d, 0" % (KP + 1, KP + 1)]
    L += ["s_mov_b32 s%d, 0" % IDX, "s_set_gpr_idx_on s%d, 0x1" % IDX]  # src0 of vector ops is M0-relative
    # first group's words and second group's k-table entries: in flight into the staging registers
    L += [sload(WS, 16, WP, 0), sload(WS + 16, 16, WP, 64)] + load_ktab(num)
    # ---- one K group per iteration
    L += ["1:"]
    L += ["s_add_u32 s%d, s%d, 128" % (WP, WP), "s_addc_u32 s%d, s%d, 0" % (WP + 1, WP + 1),
          "s_add_u32 s%d, s%d, %d" % (KP, KP, num * 4), "s_addc_u32 s%d, s%d, 0" % (KP + 1, KP + 1),
          "s_waitcnt lgkmcnt(0)"]
    # this group's words move out of the staging registers, which then receive the next group's
    # (one group past the end reads the padding that follows the words in the weight blob)
    L += ["s_mov_b64 s[%d:%d], s[%d:%d]" % (W + 2 * q, W + 2 * q + 1, WS + 2 * q, WS + 2 * q + 1)
          for q in range(16)]
    L += ["s_mov_b64 s[%d:%d], s[%d:%d]" % (KT2 + 2 * q, KT2 + 2 * q + 1, KT + 2 * q, KT + 2 * q + 1)
          for q in range((num + 1) // 2)]
    L += [sload(WS, 16, WP, 0), sload(WS + 16, 16, WP, 64)] + load_ktab(num)
    for i in range(num):
        L += koff(i)
        L += ["s_waitcnt vmcnt(%d)" % (4 * (num - 1))]
        # plane 0 = the activation itself (a shift by 0 keeps src0 a constant: not M0-relative)
        for r in range(R):
            L += ["v_ashrrev_i32 v%d, 0, v%d" % (PL + P * r, XP + 4 * i + r)]
        L += issue_loads(i)  # same slot of the next group
        for s in range(1, P):
            for r in range(R):
                L += ["v_ashrrev_i32 v%d, %d, v%d" % (PL + P * r + s, s, PL + P * r)]
        for j in range(J):
            L += ["s_bfe_u32 s%d, s%d, 0x%x" % (IDX, W + j, (bits << 16) | (i * cb)),
                  "s_set_gpr_idx_idx s%d" % IDX,
                  "s_bfe_i32 s%d, s%d, 0x%x" % (MASK, W + j, (1 << 16) | (i * cb + bits))]
            for r in range(R):
                a = ACC + 32 * r + j
                L += ["v_xad_u32 v%d, v%d, s%d, v%d" % (a, PL + P * r, MASK, a)]
    L += ["s_sub_u32 s%d, s%d, 1" % (CNT, CNT), "s_cmp_lg_u32 s%d, 0" % CNT, "s_cbranch_scc1 1b"]
    # ---- drain the loads issued for the group after the last one, leave relative addressing
    L += ["s_set_gpr_idx_off", "s_waitcnt vmcnt(0)"]
    return L


def clobbers(bits):
    num = 32 // (bits + 1)
    P = 1 << bits
    v = ['"v%d"' % n for n in range(XP, XP + 4 * num + P * R)]
    s = ['"s%d"' % n for n in range(W, KOFF + 1)]
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
