#!/usr/bin/env python3
"""Writes gemm_loop_gfx950.inc: the main loop of the persistent W4A4 GEMM kernel (gemm_w4a4.hip,
gemm_w4a4_persistent_kernel) as one hand-scheduled gfx950 instruction sequence.

Why generated text and not C++: one wave per SIMD computes a 128 x 128 tile (4 x 4 MFMA tiles of 32 x 32, all 256
accumulator registers), so that a decoded fragment serves four MFMAs and the loop needs four decode instructions per
MFMA.  A SIMD issues one MFMA (8 cycles of issue for 32 of execution) or one other vector instruction (4 cycles) at a
time, so a loop with more than six vector instructions per MFMA is bound by instruction issue, and a single wave has
nobody to hide a stall behind: every instruction has a fixed place here, decode instructions four to an MFMA, LDS
reads a sub-step ahead of their first use, loads two K steps ahead.

Work of a wave per K step (128 K elements), operands as in the C++ kernel next to it:
  * A tile: 128 rows shared by the four waves, B tile: 128 rows of the wave's own; both packed e2m1, 64 bytes per row
    and step, 16-byte pieces stored at position piece ^ (row / 4 % 4); block scales in the blocked order they have
    in memory (1 KB per 128 rows and step).
  * sub-step s = 0..7 covers 16 K elements per lane half: dword s % 4 of the lane's 16-byte piece 2 * (s / 4) + lane / 32.
  * 16 MFMAs per sub-step, D[4 g + f] += B_g x A_f; between them the operands of the next sub-step are decoded
    (v_cvt_scalef32_pk_f16_fp4, then v_pk_mul_f16 by the block scale) into the other operand buffer.

Register plan (VGPRs are fixed, accumulators and inputs are asm operands):
  v0-63    operand buffers O[2][8 fragments][4]      v64-127  packed pieces R[2 halves][8][4]
  v128-143 block scales as f16 pairs S[2][8]         v144-151 raw scale bytes (A, B)
  v152     conversion temporary                       v160-168 addresses (see PROLOGUE)
  s56-87   step counters, global bases, LDS destinations.
"""
import sys

STAGE = 46080          # bytes per LDS stage: A 8192 | B 4 x 8192 | A scales 1024 | B scales 4 x 1024
A_SCALES = 40960
B_SCALES = 41984

# asm operands: %0..%15 accumulators, then the inputs in this order
INPUTS = ["N", "VOFF", "SOFF", "ARD", "SARD", "SH", "SA", "SB", "RB16", "SAS", "SBS", "W"]
OP = {name: "%%%d" % (16 + i) for i, name in enumerate(INPUTS)}


def O(b, frag, q=None):
    base = 32 * b + 4 * frag
    return "v[%d:%d]" % (base, base + 3) if q is None else "v%d" % (base + q)


def R(h, frag, j=None):
    base = 64 + 32 * h + 4 * frag
    return "v[%d:%d]" % (base, base + 3) if j is None else "v%d" % (base + j)


def S(h, frag):
    return "v%d" % (128 + 8 * h + frag)


def SR(x, i=None):
    base = 144 + 4 * x
    return "v[%d:%d]" % (base, base + 3) if i is None else "v%d" % (base + i)


T = "v152"
A_RD = ["v160", "v161"]
B_RD = ["v162", "v163"]
SA_RD, SB_RD, SH, VOFF, SOFF = "v164", "v165", "v166", "v167", "v168"
S_N, S_MORE = "s56", "s57"
S_A = ["s[58:59]", "s[60:61]"]
S_B = ["s[%d:%d]" % (62 + 2 * i, 63 + 2 * i) for i in range(8)]
S_AS, S_BS = "s[78:79]", "s[80:81]"
S_ADST, S_BDST, S_BSDST = "s82", "s83", "s84"
S_T0, S_T1, S_T2 = "s85", "s86", "s87"


def mfma(s, g, f):
    b = s & 1
    acc = "%%%d" % (4 * g + f)
    return "v_mfma_f32_32x32x16_f16 %s, %s, %s, %s" % (acc, O(b, 4 + g), O(b, f), acc)


def decode(s_next, frag):
    """Eight instructions: the 8 elements of fragment `frag` for sub-step s_next, scaled, into the operand buffer."""
    h, j, b = (s_next >> 2) & 1, s_next & 3, s_next & 1
    out = []
    for q in range(4):
        sel = " op_sel:[%d,%d,0]" % (q & 1, q >> 1) if q else ""
        out.append("v_cvt_scalef32_pk_f16_fp4 %s, %s, 1.0%s" % (T, R(h, frag, j), sel))
        if j < 2:   # block scale of the piece's first 16 elements: low half of the pair, for both lanes of the packed op
            out.append("v_pk_mul_f16 %s, %s, %s op_sel_hi:[0,1]" % (O(b, frag, q), S(h, frag), T))
        else:
            out.append("v_pk_mul_f16 %s, %s, %s op_sel:[1,0] op_sel_hi:[1,1]" % (O(b, frag, q), S(h, frag), T))
    return out


DECODE_ORDER = [0, 4, 1, 2, 3, 5, 6, 7]   # the order in which the next sub-step's MFMAs first need them


def decode_all(s_next):
    out = []
    for frag in DECODE_ORDER:
        out += decode(s_next, frag)
    return out


def lds_reads(stage, half):
    q = stage * STAGE
    out = []
    for f in range(4):
        out.append("ds_read_b128 %s, %s offset:%d" % (R(half, f), A_RD[half], q + 2048 * f))
    for g in range(4):
        out.append("ds_read_b128 %s, %s offset:%d" % (R(half, 4 + g), B_RD[half], q + 2048 * g))
    out.append("ds_read_b128 %s, %s offset:%d" % (SR(0), SA_RD, q + 512 * half))
    out.append("ds_read_b128 %s, %s offset:%d" % (SR(1), SB_RD, q + 512 * half))
    return out


def scale_conversion(half):
    """Per fragment: the lane's two scale bytes (which pair depends on the lane half) -> two f16 in one register."""
    out = []
    for frag in range(8):
        out.append(["v_lshrrev_b32 %s, %s, %s" % (T, SH, SR(frag >> 2, frag & 3)),
                    "v_cvt_scalef32_pk_f16_fp8 %s, %s, 1.0" % (S(half, frag), T)])
    return out


def loads(stage):
    """Twelve loads of 1 KB each, global memory straight into LDS stage `stage`; each entry is one load."""
    q = stage * STAGE
    out = []
    for i in range(2):
        out.append(["s_add_u32 m0, %s, %d" % (S_ADST, q + 1024 * i), "s_nop 0",
                    "global_load_lds_dwordx4 %s, %s" % (VOFF, S_A[i])])
    for i in range(8):
        out.append(["s_add_u32 m0, %s, %d" % (S_BDST, q + 1024 * i), "s_nop 0",
                    "global_load_lds_dwordx4 %s, %s" % (VOFF, S_B[i])])
    out.append(["s_mov_b32 m0, %d" % (q + A_SCALES), "s_nop 0", "global_load_lds_dwordx4 %s, %s" % (SOFF, S_AS)])
    out.append(["s_add_u32 m0, %s, %d" % (S_BSDST, q), "s_nop 0", "global_load_lds_dwordx4 %s, %s" % (SOFF, S_BS)])
    return out


def advance():
    """Point the load offsets at the next K step, unless the segment has no further step (then the same step is
    loaded again, into a stage nobody reads any more)."""
    return ["s_cmp_lg_u32 %s, 0" % S_MORE,
            "s_cselect_b32 %s, 64, 0" % S_T0,
            "s_cselect_b32 %s, 0x400, 0" % S_T1,
            "s_cselect_b32 %s, 1, 0" % S_T2,
            "s_sub_u32 %s, %s, %s" % (S_MORE, S_MORE, S_T2),
            "v_add_u32 %s, %s, %s" % (VOFF, S_T0, VOFF),
            "v_add_u32 %s, %s, %s" % (SOFF, S_T1, SOFF)]


def k_step(p):
    """One K step out of LDS stage p."""
    out = []
    for s in range(8):
        fill = decode_all((s + 1) & 7)
        extra = {m: [] for m in range(16)}
        if s == 1:      # the pieces and scales of this step's second half
            for m, ins in enumerate(lds_reads(p, 1)):
                extra[m].append(ins)
        elif s == 2:
            extra[0].append("s_waitcnt lgkmcnt(0)")
            for m, pair in enumerate(scale_conversion(1)):
                extra[1 + m] += pair
        elif s == 3:    # every wave has read stage p for the last time and has its loads of the next step in LDS
            extra[15] += ["s_waitcnt vmcnt(0)", "s_barrier"]
        elif s == 4:    # refill stage p with the step after next
            for m, ld in enumerate(loads(p)):
                extra[m] += ld
            extra[12] += advance()
        elif s == 5:    # the first half of the next step, out of the other stage
            for m, ins in enumerate(lds_reads(p ^ 1, 0)):
                extra[m].append(ins)
        elif s == 6:
            extra[0].append("s_waitcnt lgkmcnt(0)")
            for m, pair in enumerate(scale_conversion(0)):
                extra[1 + m] += pair
        for m in range(16):
            out.append(mfma(s, m >> 2, m & 3))
            out += fill[4 * m:4 * m + 4]
            out += extra[m]
    return out


def prologue():
    out = ["s_mov_b32 %s, %s" % (S_N, OP["N"]),
           "s_sub_u32 %s, %s, 1" % (S_MORE, OP["N"]),
           "v_mov_b32 %s, %s" % (VOFF, OP["VOFF"]),
           "v_mov_b32 %s, %s" % (SOFF, OP["SOFF"]),
           "v_mov_b32 %s, %s" % (A_RD[0], OP["ARD"]),
           "v_mov_b32 %s, %s" % (SA_RD, OP["SARD"]),
           "v_mov_b32 %s, %s" % (SH, OP["SH"]),
           "s_lshl_b32 %s, %s, 13" % (S_T0, OP["W"]),              # 8192 w
           "s_lshl_b32 %s, %s, 10" % (S_T1, OP["W"]),              # 1024 w
           "v_xor_b32 %s, 32, %s" % (A_RD[1], A_RD[0]),
           "s_add_u32 %s, %s, 8192" % (S_BDST, S_T0),              # LDS: the wave's B rows
           "v_add_u32 %s, %s, %s" % (B_RD[0], S_BDST, A_RD[0]),
           "v_xor_b32 %s, 32, %s" % (B_RD[1], B_RD[0]),
           "s_add_u32 %s, %s, %d" % (S_BSDST, S_T1, B_SCALES),    # LDS: the wave's B scales
           "s_add_u32 %s, %s, 1024" % (S_T2, S_T1),
           "v_add_u32 %s, %s, %s" % (SB_RD, S_T2, SA_RD),
           "s_lshl_b32 %s, %s, 11" % (S_ADST, OP["W"]),            # LDS: the wave's share (32 rows) of the A tile
           "s_mov_b64 %s, %s" % (S_A[0], OP["SA"]),
           "s_add_u32 s60, s58, %s" % OP["RB16"], "s_addc_u32 s61, s59, 0",
           "s_mov_b64 %s, %s" % (S_B[0], OP["SB"])]
    for i in range(1, 8):
        out += ["s_add_u32 s%d, s%d, %s" % (62 + 2 * i, 60 + 2 * i, OP["RB16"]), "s_addc_u32 s%d, s%d, 0" % (63 + 2 * i, 61 + 2 * i)]
    out += ["s_mov_b64 %s, %s" % (S_AS, OP["SAS"]), "s_mov_b64 %s, %s" % (S_BS, OP["SBS"]), "s_nop 4"]
    for stage in (0, 1):
        for ld in loads(stage):
            out += ld
        out += advance()
    out += ["s_waitcnt vmcnt(0)", "s_barrier"]
    out += lds_reads(0, 0)
    out.append("s_waitcnt lgkmcnt(0)")
    for pair in scale_conversion(0):
        out += pair
    out += decode_all(0)
    out.append("s_nop 1")
    return out


def program():
    out = prologue()
    out.append("1:")
    out += k_step(0)
    out += ["s_sub_u32 %s, %s, 1" % (S_N, S_N), "s_cmp_eq_u32 %s, 0" % S_N, "s_cbranch_scc1 2f"]
    out += k_step(1)
    out += ["s_sub_u32 %s, %s, 1" % (S_N, S_N), "s_cmp_lg_u32 %s, 0" % S_N, "s_cbranch_scc1 1b"]
    out.append("2:")
    out += ["s_nop 7", "s_nop 7", "s_nop 7"]   # the last MFMAs have written their accumulators before anything reads them
    return out


def main(path):
    lines = program()
    with open(path, "w") as f:
        f.write("// Generated by gemm_loop_gen.py - do not edit.  %d instructions; operands: %%0-%%15 accumulators, then %s.\n"
                % (sum(1 for l in lines if not l.endswith(":")), ", ".join(INPUTS)))
        for l in lines:
            f.write('"%s\\n"\n' % l)


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "gemm_loop_gfx950.inc")
