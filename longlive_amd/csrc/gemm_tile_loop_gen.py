#!/usr/bin/env python3
"""Writes gemm_tile_loop_<FA><FB>_gfx950.inc: the main loop of the one-workgroup-per-tile W4A4 GEMM kernel
(gemm_w4a4.hip, gemm_w4a4_asm_kernel<FA, FB>) as one hand-scheduled gfx950 instruction sequence.

A workgroup is 2 x 2 waves, two workgroups share a compute unit (two waves per SIMD).  A wave computes
(32 FA) x (32 FB) outputs: FA fragments of the A tile (activations, rows) and FB of the B tile (weights, columns),
FA * FB accumulators of 16 registers, kept in the AGPRs; everything else fits 128 VGPRs, so that two waves fit a SIMD.
A SIMD issues one vector instruction at a time (an MFMA holds the port 8 of its 32 cycles, anything else 4), and the
compiler's schedule of the same loop leaves the matrix pipe idle almost half of the time (register copies ahead of
MFMAs, waits for all LDS reads at once): here every instruction has a fixed place - (FA + FB) * 8 / (FA * FB) decode
instructions behind every MFMA, LDS reads a sub-step ahead of their first use, loads two K steps ahead, one barrier
per K step.

Work of a wave per K step (128 K elements), LDS stage layout (bytes):
  A tile   64 FA rows x 64, at 0             wave (wm, wn) reads rows 32 FA wm + 32 f, f < FA
  B tile   64 FB rows x 64, behind it        ... rows 32 FB wn + 32 g, g < FB
  scales   in the blocked order they have in memory: 1 KB per 128 rows and step (two halves of 512 bytes)
  16-byte pieces of a row are stored at position piece ^ (row / 4 % 4).
Sub-step s = 0..7 covers 16 K elements per lane half: dword s % 4 of the lane's 16-byte piece 2 (s / 4) + lane / 32.
The packed dwords are read from LDS two sub-steps at a time (ds_read_b64) into one of two small buffers.

Register plan (VGPRs fixed, accumulators and inputs are asm operands; NF = FA + FB fragments, A first):
  v0 ..            operand buffers O[2][NF][4]
  then             packed dwords R[2][NF][2], block scales as f16 pairs S[2][NF], raw scale bytes SR[2][4],
                   a temporary, nine address registers
  s56-s87          step counters, global bases, LDS destinations.
"""
import sys


class Plan:
    def __init__(self, fa, fb, waves=4):
        self.fa, self.fb, self.nf = fa, fb, fa + fb
        nf = self.nf
        self.a_bytes = 64 * fa * 64                      # A tile of a stage
        self.b_bytes = 64 * fb * 64
        self.a_groups = max(1, (64 * fa) // 128)         # 128-row groups of scales
        self.b_groups = max(1, (64 * fb) // 128)
        self.a_scales = self.a_bytes + self.b_bytes
        self.b_scales = self.a_scales + 1024 * self.a_groups
        self.stage = self.b_scales + 1024 * self.b_groups
        self.o0 = 0
        self.r0 = self.o0 + 2 * nf * 4
        self.s0 = self.r0 + 2 * nf * 2
        self.sr0 = self.s0 + 2 * nf
        self.t = self.sr0 + 8
        self.addr0 = self.t + 1
        self.n_vgprs = self.addr0 + 9
        # loads of a wave per K step: its quarter of the A tile and of the B tile (16 rows = 1 KB per load) and one
        # 1 KB scale block
        self.a_loads = (64 * fa) // 16 // waves
        self.b_loads = (64 * fb) // 16 // waves

    # ---- registers
    def O(self, b, frag, q=None):
        base = self.o0 + 4 * (self.nf * b + frag)
        return "v[%d:%d]" % (base, base + 3) if q is None else "v%d" % (base + q)

    def R(self, buf, frag, j=None):
        base = self.r0 + 2 * (self.nf * buf + frag)
        return "v[%d:%d]" % (base, base + 1) if j is None else "v%d" % (base + j)

    def S(self, h, frag):
        return "v%d" % (self.s0 + self.nf * h + frag)

    def SR(self, x, i=None):
        base = self.sr0 + 4 * x
        return "v[%d:%d]" % (base, base + 3) if i is None else "v%d" % (base + i)

    @property
    def T(self):
        return "v%d" % self.t

    def addr(self, i):
        return "v%d" % (self.addr0 + i)


# asm operands: %0 .. %(FA*FB-1) accumulators, then the inputs in this order
INPUTS = ["N", "VOFF", "SOFF", "ARD", "BRD", "SARD", "SBRD", "SH", "SA", "SB", "SS", "RB16", "ADST", "BDST", "SDST", "IDLE"]
# ARD / BRD: the lane's address of its first 16-byte piece (pieces 0, 1: first half of a K step) in fragment 0 of the
# wave's A / B rows, stage 0; the pieces of the second half lie at that address xor 32 (positions are swizzled).
# IDLE: not zero for a wave whose outputs all lie outside the matrix: it loads its share of the tiles and keeps the
# barriers, nothing else.
S_N, S_LEFT = "s56", "s57"   # K steps to compute, K steps not loaded yet
S_ADST, S_BDST, S_SDST = "s82", "s83", "s84"
S_SC = "s[80:81]"


def gen(fa, fb):
    P = Plan(fa, fb)
    nacc = fa * fb
    OP = {name: "%%%d" % (nacc + i) for i, name in enumerate(INPUTS)}
    SA_RD, SB_RD, SH, VOFF, SOFF = (P.addr(i) for i in (4, 5, 6, 7, 8))
    A_RD, B_RD = [P.addr(0), P.addr(1)], [P.addr(2), P.addr(3)]
    S_A = ["s[%d:%d]" % (58 + 2 * i, 59 + 2 * i) for i in range(P.a_loads)]
    S_B = ["s[%d:%d]" % (58 + 2 * (P.a_loads + i), 59 + 2 * (P.a_loads + i)) for i in range(P.b_loads)]
    assert 58 + 2 * (P.a_loads + P.b_loads) <= 80

    def mfma(s, g, f):
        b = s & 1
        acc = "%%%d" % (fa * g + f)
        return "v_mfma_f32_32x32x16_f16 %s, %s, %s, %s" % (acc, P.O(b, fa + g), P.O(b, f), acc)

    def decode(s_next, frag):
        """Eight instructions: the 8 elements of fragment `frag` for sub-step s_next, scaled, into the operand buffer."""
        h, j, b, buf = (s_next >> 2) & 1, s_next & 3, s_next & 1, (s_next >> 1) & 1
        out = []
        for q in range(4):
            sel = " op_sel:[%d,%d,0]" % (q & 1, q >> 1) if q else ""
            out.append("v_cvt_scalef32_pk_f16_fp4 %s, %s, 1.0%s" % (P.T, P.R(buf, frag, j & 1), sel))
            if j < 2:   # block scale of the piece's first 16 elements: low half of the pair
                out.append("v_pk_mul_f16 %s, %s, %s op_sel_hi:[0,1]" % (P.O(b, frag, q), P.S(h, frag), P.T))
            else:
                out.append("v_pk_mul_f16 %s, %s, %s op_sel:[1,0] op_sel_hi:[1,1]" % (P.O(b, frag, q), P.S(h, frag), P.T))
        return out

    # the order in which the next sub-step's MFMAs first need the fragments: A0, B0, A1 .. then B1 ..
    order = [0, fa] + list(range(1, fa)) + list(range(fa + 1, fa + fb))

    def decode_all(s_next):
        out = []
        for frag in order:
            out += decode(s_next, frag)
        return out

    def quarter_reads(stage, quarter):
        """The packed dwords of sub-steps 2 quarter, 2 quarter + 1 of the step in `stage`, into buffer quarter % 2."""
        base, h = stage * P.stage + 8 * (quarter & 1), quarter >> 1
        out = []
        for f in range(fa):
            out.append("ds_read_b64 %s, %s offset:%d" % (P.R(quarter & 1, f), A_RD[h], base + 2048 * f))
        for g in range(fb):
            out.append("ds_read_b64 %s, %s offset:%d" % (P.R(quarter & 1, fa + g), B_RD[h], base + 2048 * g))
        return out

    def scale_reads(stage, half):
        q = stage * P.stage + 512 * half

        def read(x, n, addr):   # one dword (four scale bytes) per fragment: 16 or 8 bytes of the lane's scale row
            if n == 4:
                return "ds_read_b128 %s, %s offset:%d" % (P.SR(x), addr, q)
            base = P.sr0 + 4 * x
            return "ds_read_b64 v[%d:%d], %s offset:%d" % (base, base + 1, addr, q)
        return [read(0, fa, SA_RD), read(1, fb, SB_RD)]

    def scale_conversion(half):
        """Per fragment: the lane's two scale bytes (which pair depends on the lane half) -> two f16 in one register.
        A wave with four fragments of an operand owns a whole 128-row group of scales (16 bytes per row and half
        step); with two fragments it owns half of one, and the kernel points SARD / SBRD at its 8 bytes."""
        out = []
        for f in range(fa):
            out.append(["v_lshrrev_b32 %s, %s, %s" % (P.T, SH, P.SR(0, f)),
                        "v_cvt_scalef32_pk_f16_fp8 %s, %s, 1.0" % (P.S(half, f), P.T)])
        for g in range(fb):
            out.append(["v_lshrrev_b32 %s, %s, %s" % (P.T, SH, P.SR(1, g)),
                        "v_cvt_scalef32_pk_f16_fp8 %s, %s, 1.0" % (P.S(half, fa + g), P.T)])
        return out

    def loads(stage):
        """The wave's loads of one K step, 1 KB each, global memory straight into LDS stage `stage`."""
        q = stage * P.stage
        out = []
        for i in range(P.a_loads):
            out.append(["s_add_u32 m0, %s, %d" % (S_ADST, q + 1024 * i), "s_nop 0",
                        "global_load_lds_dwordx4 %s, %s" % (VOFF, S_A[i])])
        for i in range(P.b_loads):
            out.append(["s_add_u32 m0, %s, %d" % (S_BDST, q + 1024 * i), "s_nop 0",
                        "global_load_lds_dwordx4 %s, %s" % (VOFF, S_B[i])])
        out.append(["s_add_u32 m0, %s, %d" % (S_SDST, q), "s_nop 0", "global_load_lds_dwordx4 %s, %s" % (SOFF, S_SC)])
        return out

    def advance():
        """A K step has been requested: point the load offsets at the next one."""
        return ["s_sub_u32 %s, %s, 1" % (S_LEFT, S_LEFT),
                "v_add_u32 %s, 64, %s" % (VOFF, VOFF),
                "v_add_u32 %s, 0x400, %s" % (SOFF, SOFF)]

    labels = iter(range(10, 100))

    def if_steps_left(with_loads, without):
        """Two versions of a stretch of the schedule: the last two K steps have nothing left to load."""
        skip, end = next(labels), next(labels)
        out = ["s_cmp_eq_u32 %s, 0" % S_LEFT, "s_cbranch_scc1 %df" % skip] + with_loads
        if without:
            return out + ["s_branch %df" % end, "%d:" % skip] + without + ["%d:" % end]
        return out + ["%d:" % skip]

    n_mfma = fa * fb

    def sub_step(p, s, with_loads=True):
        fill = decode_all((s + 1) & 7)
        per = len(fill) // n_mfma
        assert per * n_mfma == len(fill)
        extra = {m: [] for m in range(n_mfma)}
        head = []

        def spread(items, first=0):
            for i, ins in enumerate(items):
                extra[(first + i) % n_mfma] += ins if isinstance(ins, list) else [ins]

        if s == 0:      # dwords of sub-steps 2, 3
            spread(quarter_reads(p, 1))
        elif s == 1:    # the decode below reads them
            head.append("s_waitcnt lgkmcnt(0)")
        elif s == 2:    # dwords of sub-steps 4, 5 and the scales of the second half
            spread(quarter_reads(p, 2) + scale_reads(p, 1))
        elif s == 3:
            head.append("s_waitcnt lgkmcnt(0)")
            for pair in scale_conversion(1):
                head += pair
        elif s == 4:    # dwords of sub-steps 6, 7: the last reads of stage p
            spread(quarter_reads(p, 3))
        elif s == 5:    # every wave has read stage p for the last time and has its loads of the next step in LDS
            head.append("s_waitcnt lgkmcnt(0)")
            extra[n_mfma - 1] += ["s_waitcnt vmcnt(0)", "s_barrier"]
        elif s == 6:    # refill stage p with the step after next; first dwords and scales of the next step
            if with_loads:
                spread(loads(p))
                extra[n_mfma - 1] += advance()
            spread(quarter_reads(p ^ 1, 0) + scale_reads(p ^ 1, 0), first=len(loads(p)) % n_mfma)
        elif s == 7:
            head.append("s_waitcnt lgkmcnt(0)")
            for pair in scale_conversion(0):
                head += pair
        # The scale conversions of a half precede every decode that uses them: they sit ahead of the first MFMA.
        out = head
        for m in range(n_mfma):
            out.append(mfma(s, m // fa, m % fa))
            out += fill[per * m:per * (m + 1)]
            out += extra[m]
        return out

    def k_step(p):
        """One K step out of LDS stage p."""
        out = []
        for s in range(8):
            out += sub_step(p, s) if s != 6 else if_steps_left(sub_step(p, 6), sub_step(p, 6, with_loads=False))
        return out

    def idle_step(p):
        """The same K step for a wave without outputs: the barrier, its loads."""
        refill = [i for ld in loads(p) for i in ld] + advance()
        return ["s_waitcnt vmcnt(0)", "s_barrier"] + if_steps_left(refill, [])

    def prologue():
        out = ["s_mov_b32 %s, %s" % (S_N, OP["N"]),
               "s_mov_b32 %s, %s" % (S_LEFT, OP["N"]),
               "v_mov_b32 %s, %s" % (VOFF, OP["VOFF"]),
               "v_mov_b32 %s, %s" % (SOFF, OP["SOFF"]),
               "v_mov_b32 %s, %s" % (A_RD[0], OP["ARD"]),
               "v_mov_b32 %s, %s" % (B_RD[0], OP["BRD"]),
               "v_mov_b32 %s, %s" % (SA_RD, OP["SARD"]),
               "v_mov_b32 %s, %s" % (SB_RD, OP["SBRD"]),
               "v_mov_b32 %s, %s" % (SH, OP["SH"]),
               "s_mov_b32 %s, %s" % (S_ADST, OP["ADST"]),
               "s_mov_b32 %s, %s" % (S_BDST, OP["BDST"]),
               "s_mov_b32 %s, %s" % (S_SDST, OP["SDST"]),
               "s_mov_b64 %s, %s" % (S_A[0], OP["SA"])]
        regs = [58 + 2 * i for i in range(P.a_loads + P.b_loads)]
        for i in range(1, P.a_loads):
            out += ["s_add_u32 s%d, s%d, %s" % (regs[i], regs[i - 1], OP["RB16"]),
                    "s_addc_u32 s%d, s%d, 0" % (regs[i] + 1, regs[i - 1] + 1)]
        out.append("s_mov_b64 %s, %s" % (S_B[0], OP["SB"]))
        for i in range(P.a_loads + 1, P.a_loads + P.b_loads):
            out += ["s_add_u32 s%d, s%d, %s" % (regs[i], regs[i - 1], OP["RB16"]),
                    "s_addc_u32 s%d, s%d, 0" % (regs[i] + 1, regs[i - 1] + 1)]
        out += ["v_xor_b32 %s, 32, %s" % (A_RD[1], A_RD[0]), "v_xor_b32 %s, 32, %s" % (B_RD[1], B_RD[0]),
                "s_mov_b64 %s, %s" % (S_SC, OP["SS"]), "s_nop 4"]
        for stage in (0, 1):
            step = [i for ld in loads(stage) for i in ld] + advance()
            out += step if stage == 0 else if_steps_left(step, [])
        out += ["s_waitcnt vmcnt(0)", "s_barrier", "s_cmp_lg_u32 %s, 0" % OP["IDLE"], "s_cbranch_scc1 3f"]
        out += quarter_reads(0, 0) + scale_reads(0, 0)
        out.append("s_waitcnt lgkmcnt(0)")
        for pair in scale_conversion(0):
            out += pair
        out += decode_all(0)
        out.append("s_nop 1")
        return out

    out = prologue()
    out.append("1:")
    out += k_step(0)
    out += ["s_sub_u32 %s, %s, 1" % (S_N, S_N), "s_cmp_eq_u32 %s, 0" % S_N, "s_cbranch_scc1 2f"]
    out += k_step(1)
    out += ["s_sub_u32 %s, %s, 1" % (S_N, S_N), "s_cmp_lg_u32 %s, 0" % S_N, "s_cbranch_scc1 1b"]
    out.append("2:")
    # The last MFMAs have written their accumulators, and every wave has left the stages (the epilogue reuses LDS
    # behind a barrier of its own), before anything else happens.
    out += ["s_nop 7", "s_nop 7", "s_nop 7", "s_waitcnt vmcnt(0) lgkmcnt(0)", "s_branch 4f"]
    out.append("3:")
    out += idle_step(0)
    out += ["s_sub_u32 %s, %s, 1" % (S_N, S_N), "s_cmp_eq_u32 %s, 0" % S_N, "s_cbranch_scc1 2b"]
    out += idle_step(1)
    out += ["s_sub_u32 %s, %s, 1" % (S_N, S_N), "s_cmp_lg_u32 %s, 0" % S_N, "s_cbranch_scc1 3b", "s_branch 2b"]
    out.append("4:")
    return P, out


# ---------------------------------------------------------------------------------------------------------------------
# Eight waves per workgroup, the K range of every step split between two groups of four (gemm_w4a4_asm8_kernel).
#
# One workgroup per compute unit computes a (64 FA) x (64 FB) tile; waves 0-3 and 4-7 hold the same 2 x 2 arrangement of
# wave tiles, the first group multiplies the first 64 K elements of every K step, the second group the other 64, and
# the kernel adds the two partial tiles through LDS behind the loop.  A wave therefore walks four sub-steps per K
# step (dwords 0-3 of ONE 16-byte piece per lane and fragment; which piece, and which half of the scales, is in the
# addresses the kernel passes).  The stages form a ring of NSTAGE: their offset is kept in registers, not in the
# instructions, so the loop is not unrolled.  The barrier of step t sits behind sub-step 1, when the wave has issued
# its last read of stage t and has waited for its loads of step t + 1; behind it the wave requests step t + NSTAGE
# into the stage it just left and reads the first dwords and the scales of step t + 1.
SPLIT_INPUTS = ["N", "VOFF", "SOFF", "ARD", "BRD", "SARD", "SBRD", "SH", "SA", "SB", "SS", "RB16", "ADST", "BDST", "SDST", "IDLE",
                "HASSC"]
# HASSC: not zero for the waves that load a block of scales (one more load per K step than the others).


def gen_split(fa, fb, nstage=3):
    P = Plan(fa, fb, waves=8)
    nacc, n_mfma = fa * fb, fa * fb
    OP = {name: "%%%d" % (nacc + i) for i, name in enumerate(SPLIT_INPUTS)}
    A_RD, B_RD, SA_RD, SB_RD, SH, VOFF, SOFF = (P.addr(i) for i in range(7))
    S_A = ["s[%d:%d]" % (58 + 2 * i, 59 + 2 * i) for i in range(P.a_loads)]
    S_B = ["s[%d:%d]" % (58 + 2 * (P.a_loads + i), 59 + 2 * (P.a_loads + i)) for i in range(P.b_loads)]
    assert 58 + 2 * (P.a_loads + P.b_loads) <= 76
    S_RS, S_WS, S_DELTA, S_TMP, S_HASSC = "s76", "s77", "s78", "s79", "s85"
    ring = nstage * P.stage
    labels = iter(range(10, 100))

    def mfma(j, g, f):
        acc = "%%%d" % (fa * g + f)
        return "v_mfma_f32_32x32x16_f16 %s, %s, %s, %s" % (acc, P.O(j & 1, fa + g), P.O(j & 1, f), acc)

    def decode(j, frag):
        """Eight instructions: dword j of the lane's piece of fragment `frag`, scaled, into operand buffer j % 2."""
        out = []
        for q in range(4):
            sel = " op_sel:[%d,%d,0]" % (q & 1, q >> 1) if q else ""
            out.append("v_cvt_scalef32_pk_f16_fp4 %s, %s, 1.0%s" % (P.T, P.R(j >> 1, frag, j & 1), sel))
            if j < 2:   # the piece's first 16 elements: low half of the pair of block scales
                out.append("v_pk_mul_f16 %s, %s, %s op_sel_hi:[0,1]" % (P.O(j & 1, frag, q), P.S(0, frag), P.T))
            else:
                out.append("v_pk_mul_f16 %s, %s, %s op_sel:[1,0] op_sel_hi:[1,1]" % (P.O(j & 1, frag, q), P.S(0, frag), P.T))
        return out

    order = [0, fa] + list(range(1, fa)) + list(range(fa + 1, fa + fb))

    def decode_all(j):
        return [i for frag in order for i in decode(j, frag)]

    def quarter_reads(quarter):
        """Dwords 2 quarter, 2 quarter + 1 of the lane's pieces in the stage the address registers point at."""
        out = ["ds_read_b64 %s, %s offset:%d" % (P.R(quarter, f), A_RD, 8 * quarter + 2048 * f) for f in range(fa)]
        out += ["ds_read_b64 %s, %s offset:%d" % (P.R(quarter, fa + g), B_RD, 8 * quarter + 2048 * g) for g in range(fb)]
        return out

    def scale_reads():
        def read(x, n, addr):
            base = P.sr0 + 4 * x
            return ("ds_read_b128 %s, %s" % (P.SR(x), addr)) if n == 4 else ("ds_read_b64 v[%d:%d], %s" % (base, base + 1, addr))
        return [read(0, fa, SA_RD), read(1, fb, SB_RD)]

    def scale_conversion():
        out = []
        for f in range(fa):
            out += ["v_lshrrev_b32 %s, %s, %s" % (P.T, SH, P.SR(0, f)), "v_cvt_scalef32_pk_f16_fp8 %s, %s, 1.0" % (P.S(0, f), P.T)]
        for g in range(fb):
            out += ["v_lshrrev_b32 %s, %s, %s" % (P.T, SH, P.SR(1, g)), "v_cvt_scalef32_pk_f16_fp8 %s, %s, 1.0" % (P.S(0, fa + g), P.T)]
        return out

    def request():
        """The wave's loads of one K step into the stage at S_WS, then the offsets of the next step."""
        out = []
        for i in range(P.a_loads):
            out += ["s_add_u32 m0, %s, %s" % (S_ADST, S_WS)] + (["s_add_u32 m0, m0, %d" % (1024 * i)] if i else []) + \
                   ["s_nop 0", "global_load_lds_dwordx4 %s, %s" % (VOFF, S_A[i])]
        for i in range(P.b_loads):
            out += ["s_add_u32 m0, %s, %s" % (S_BDST, S_WS)] + (["s_add_u32 m0, m0, %d" % (1024 * i)] if i else []) + \
                   ["s_nop 0", "global_load_lds_dwordx4 %s, %s" % (VOFF, S_B[i])]
        skip = next(labels)
        out += ["s_cmp_eq_u32 %s, 0" % S_HASSC, "s_cbranch_scc1 %df" % skip,
                "s_add_u32 m0, %s, %s" % (S_SDST, S_WS), "s_nop 0", "global_load_lds_dwordx4 %s, %s" % (SOFF, S_SC), "%d:" % skip]
        out += ["s_sub_u32 %s, %s, 1" % (S_LEFT, S_LEFT), "v_add_u32 %s, 64, %s" % (VOFF, VOFF), "v_add_u32 %s, 0x400, %s" % (SOFF, SOFF)]
        return out

    def request_if_left():
        skip = next(labels)
        return ["s_cmp_eq_u32 %s, 0" % S_LEFT, "s_cbranch_scc1 %df" % skip] + request() + ["%d:" % skip]

    def rotate(with_addresses):
        """The stage just read becomes the one to refill; the address registers move on to the next stage."""
        out = ["s_mov_b32 %s, %s" % (S_WS, S_RS),
               "s_add_u32 %s, %s, %d" % (S_TMP, S_RS, P.stage),
               "s_cmp_eq_u32 %s, %d" % (S_TMP, ring),
               "s_cselect_b32 %s, 0, %s" % (S_TMP, S_TMP),
               "s_sub_u32 %s, %s, %s" % (S_DELTA, S_TMP, S_RS),
               "s_mov_b32 %s, %s" % (S_RS, S_TMP)]
        if with_addresses:
            out += ["v_add_u32 %s, %s, %s" % (r, S_DELTA, r) for r in (A_RD, B_RD, SA_RD, SB_RD)]
        return out

    def wait_and_barrier():
        """The wave's loads of step t + 1 have landed (those of step t + 2, if it exists, may still be under way)."""
        l0, l4, lb = next(labels), next(labels), next(labels)
        per_wave = P.a_loads + P.b_loads
        return ["s_cmp_le_u32 %s, 2" % S_N, "s_cbranch_scc1 %df" % l0,
                "s_cmp_lg_u32 %s, 0" % S_HASSC, "s_cbranch_scc1 %df" % l4,
                "s_waitcnt vmcnt(%d)" % per_wave, "s_branch %df" % lb,
                "%d:" % l4, "s_waitcnt vmcnt(%d)" % (per_wave + 1), "s_branch %df" % lb,
                "%d:" % l0, "s_waitcnt vmcnt(0)",
                "%d:" % lb, "s_barrier"]

    def k_step():
        out = []
        for j in range(4):
            fill = decode_all((j + 1) & 3)
            per = len(fill) // n_mfma
            assert per * n_mfma == len(fill)
            extra = {m: [] for m in range(n_mfma)}
            head = []
            if j == 0:      # dwords 2, 3: the last reads of this stage
                for i, ins in enumerate(quarter_reads(1)):
                    extra[i % n_mfma].append(ins)
            elif j == 1:
                head.append("s_waitcnt lgkmcnt(0)")
                extra[0] += rotate(True)
                extra[n_mfma - 1] += wait_and_barrier()
            elif j == 2:    # refill the stage just left; first dwords and scales of the next step
                extra[0] += request_if_left()
                for i, ins in enumerate(quarter_reads(0) + scale_reads()):
                    extra[1 + i % (n_mfma - 1)].append(ins)
            else:
                head.append("s_waitcnt lgkmcnt(0)")
                head += scale_conversion()
            out += head
            for m in range(n_mfma):
                out.append(mfma(j, m // fa, m % fa))
                out += fill[per * m:per * (m + 1)]
                out += extra[m]
        return out

    def prologue():
        out = ["s_mov_b32 %s, %s" % (S_N, OP["N"]),
               "s_mov_b32 %s, %s" % (S_LEFT, OP["N"]),
               "s_mov_b32 %s, %s" % (S_HASSC, OP["HASSC"]),
               "s_mov_b32 %s, 0" % S_RS,
               "s_mov_b32 %s, 0" % S_WS,
               "v_mov_b32 %s, %s" % (VOFF, OP["VOFF"]),
               "v_mov_b32 %s, %s" % (SOFF, OP["SOFF"]),
               "v_mov_b32 %s, %s" % (A_RD, OP["ARD"]),
               "v_mov_b32 %s, %s" % (B_RD, OP["BRD"]),
               "v_mov_b32 %s, %s" % (SA_RD, OP["SARD"]),
               "v_mov_b32 %s, %s" % (SB_RD, OP["SBRD"]),
               "v_mov_b32 %s, %s" % (SH, OP["SH"]),
               "s_mov_b32 %s, %s" % (S_ADST, OP["ADST"]),
               "s_mov_b32 %s, %s" % (S_BDST, OP["BDST"]),
               "s_mov_b32 %s, %s" % (S_SDST, OP["SDST"]),
               "s_mov_b64 %s, %s" % (S_A[0], OP["SA"])]
        regs = [58 + 2 * i for i in range(P.a_loads + P.b_loads)]
        for i in range(1, P.a_loads):
            out += ["s_add_u32 s%d, s%d, %s" % (regs[i], regs[i - 1], OP["RB16"]), "s_addc_u32 s%d, s%d, 0" % (regs[i] + 1, regs[i - 1] + 1)]
        out.append("s_mov_b64 %s, %s" % (S_B[0], OP["SB"]))
        for i in range(P.a_loads + 1, P.a_loads + P.b_loads):
            out += ["s_add_u32 s%d, s%d, %s" % (regs[i], regs[i - 1], OP["RB16"]), "s_addc_u32 s%d, s%d, 0" % (regs[i] + 1, regs[i - 1] + 1)]
        out += ["s_mov_b64 %s, %s" % (S_SC, OP["SS"]), "s_nop 4"]
        out += request()
        for stage in range(1, nstage):
            out.append("s_mov_b32 %s, %d" % (S_WS, stage * P.stage))
            out += request_if_left()
        out += ["s_waitcnt vmcnt(0)", "s_barrier", "s_cmp_lg_u32 %s, 0" % OP["IDLE"], "s_cbranch_scc1 3f"]
        out += quarter_reads(0) + scale_reads()
        out.append("s_waitcnt lgkmcnt(0)")
        out += scale_conversion()
        out += decode_all(0)
        out.append("s_nop 1")
        return out

    out = prologue()
    out.append("1:")
    out += k_step()
    out += ["s_sub_u32 %s, %s, 1" % (S_N, S_N), "s_cmp_lg_u32 %s, 0" % S_N, "s_cbranch_scc1 1b"]
    out.append("2:")
    out += ["s_nop 7", "s_nop 7", "s_nop 7", "s_waitcnt vmcnt(0) lgkmcnt(0)", "s_branch 4f"]
    out.append("3:")    # a wave without outputs: the barrier, the rotation, its loads
    out += wait_and_barrier() + rotate(False) + request_if_left()
    out += ["s_sub_u32 %s, %s, 1" % (S_N, S_N), "s_cmp_lg_u32 %s, 0" % S_N, "s_cbranch_scc1 3b", "s_branch 2b"]
    out.append("4:")
    return P, out


def main(fa, fb, path, waves=4):
    P, lines = gen(fa, fb) if waves == 4 else gen_split(fa, fb)
    inputs = INPUTS if waves == 4 else SPLIT_INPUTS
    with open(path, "w") as f:
        f.write("// Generated by gemm_tile_loop_gen.py %d %d%s - do not edit.  %d instructions, VGPRs v0-v%d, LDS stage %d bytes;\n"
                "// operands: %%0-%%%d accumulators, then %s.\n"
                % (fa, fb, "" if waves == 4 else " --waves 8", sum(1 for l in lines if not l.endswith(":")), P.n_vgprs - 1, P.stage,
                   fa * fb - 1, ", ".join(inputs)))
        for l in lines:
            f.write('"%s\\n"\n' % l)


if __name__ == "__main__":
    # usage: gemm_tile_loop_gen.py FA FB out.inc [--waves 8]
    args = sys.argv[1:]
    waves = 4
    if "--waves" in args:
        i = args.index("--waves")
        waves = int(args[i + 1])
        del args[i:i + 2]
    main(int(args[0]), int(args[1]), args[2], waves)
