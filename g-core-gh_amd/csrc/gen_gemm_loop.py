#!/usr/bin/env python3
"""Generates gemm_big_loop.inc: the hand-scheduled main loop of the 256 x 256 block-scaled
FP8 GEMM (fp32 scales) as one inline-asm string for gfx950.

Why generated assembly: the loop must keep eight MFMA results in flight while the VALU folds
the previous block into the fp32 accumulators and the LDS streams the next weight fragment.
With 128 accumulator registers per lane the compiler serialises MFMA -> fold -> MFMA instead;
fixing the register plan by hand removes that.

Register plan (per lane, all physical):
  v[128:255] acc[nb][mb][r] = v[128 + 16*nb + 4*mb + r]      (outputs of the asm statement)
  v[96:127]  p[buf][mb][r]  = v[96 + 16*buf + 4*mb + r]       MFMA results of block nb (buf = nb & 1)
  v[64:95]   af[mb]         = v[64 + 8*mb : 71 + 8*mb]        activation fragments of this K step
  v[48:63]   wf[buf]        = v[48 + 8*buf : 55 + 8*buf]      weight fragment of block nb
  v[44:47]   sc[mb]         = As[m, kb] * Bs[n/128, kb]
  v[40:43]   raw As of the next step
  v38, v39   LDS address of the lane's activation scales: buffer half 0, half in use
  v[30:37]   LDS read addresses: stage 0 (a0, a1, b0, b1) and stage 1
  s[40:55]   bases, counters, M0 base, buffer toggles
  s[56:59], s[60:63]  weight scales of this / the next group of four steps
One K step = 128 bytes of K = one scale block: 8 DMA instructions for the next stage, 10 + 14
LDS fragment reads, 32 MFMA 16x16x128 (zero C), 128 FMA folds.

Scales: a gather of one activation scale per lane per step costs the texture path about as much as
the operand copies themselves (16 distinct cache lines per instruction), so the scales move in groups
of four K steps: waves 0..3 copy 16 bytes per activation row (256 rows) straight into a small LDS
buffer with one global_load_lds_dwordx4 each, the four weight scales come with one s_load_dwordx4,
and each step reads its four activation scales from LDS.  Hence K must be a multiple of 512 here.
"""
import os

A_BYTES = 256 * 128
STAGE = 2 * A_BYTES          # 256 activation rows + 256 weight rows, 128 bytes each
NB, MB = 8, 4

ACC, P, AF, WF, SC, SAN = 128, 96, 64, 48, 44, 40
RD = {0: (30, 31, 32, 33), 1: (34, 35, 36, 37)}     # a0, a1, b0, b1 per stage
SCL_LDS = 2 * STAGE          # activation-scale buffer: 2 halves x 256 rows x 16 bytes, after the operand stages

lines = []


def emit(s):
    lines.append(s)


def vr(base, n):
    return f"v[{base}:{base + n - 1}]"


def dma(stage):
    """Issue the 8 global->LDS copies of one stage and advance the operand bases by one K step."""
    for i in range(4):
        emit(f"s_add_u32 m0, s48, {stage * STAGE + i * 8192}")
        emit("s_nop 0")
        emit(f"global_load_lds_dwordx4 %[aoff{i}], s[40:41]")
    for i in range(4):
        emit(f"s_add_u32 m0, s48, {stage * STAGE + A_BYTES + i * 8192}")
        emit("s_nop 0")
        emit(f"global_load_lds_dwordx4 %[boff{i}], s[42:43]")
    emit("s_add_u32 s40, s40, 128")
    emit("s_addc_u32 s41, s41, 0")
    emit("s_add_u32 s42, s42, 128")
    emit("s_addc_u32 s43, s43, 0")


def scale_group_copy_body(tag):
    """Copy the activation scales of the next group of four K steps into LDS (waves 0..3, one row per lane,
    16 bytes each) and load the four weight scales of that group into s[60:63]."""
    emit("s_cmp_eq_u32 s53, 0")
    emit(f"s_cbranch_scc1 Lnosc{tag}%=")
    emit("s_add_u32 m0, s48, s54")
    emit(f"s_add_u32 m0, m0, {SCL_LDS}")
    emit("s_nop 0")
    emit("global_load_lds_dwordx4 %[soff], s[44:45]")
    emit(f"Lnosc{tag}%=:")
    emit("s_load_dwordx4 s[60:63], s[46:47], 0x0")
    emit("s_add_u32 s44, s44, 16")
    emit("s_addc_u32 s45, s45, 0")
    emit("s_add_u32 s46, s46, 16")
    emit("s_addc_u32 s47, s47, 0")


def read_scales(col):
    """Activation scales of the lane's four block rows for one K step (column col of the group buffer v39)."""
    for mb in range(MB):
        emit(f"ds_read_b32 v{SAN + mb}, v39 offset:{mb * 256 + col * 4}")


def compute(stage):
    a0, a1, b0, b1 = RD[stage]
    for mb in range(MB):
        emit(f"ds_read_b128 {vr(AF + 8 * mb, 4)}, v{a0} offset:{mb * 2048}")
        emit(f"ds_read_b128 {vr(AF + 8 * mb + 4, 4)}, v{a1} offset:{mb * 2048}")
    emit(f"ds_read_b128 {vr(WF, 4)}, v{b0}")
    emit(f"ds_read_b128 {vr(WF + 4, 4)}, v{b1}")
    emit("s_waitcnt lgkmcnt(0)")
    for nb in range(NB):
        cur, nxt = nb & 1, (nb & 1) ^ 1
        if nb + 1 < NB:
            emit(f"ds_read_b128 {vr(WF + 8 * nxt, 4)}, v{b0} offset:{(nb + 1) * 2048}")
            emit(f"ds_read_b128 {vr(WF + 8 * nxt + 4, 4)}, v{b1} offset:{(nb + 1) * 2048}")
        for mb in range(MB):
            emit(f"v_mfma_f32_16x16x128_f8f6f4 {vr(P + 16 * cur + 4 * mb, 4)}, {vr(WF + 8 * cur, 8)}, {vr(AF + 8 * mb, 8)}, 0")
            if nb > 0:
                for r in range(4):
                    emit(f"v_fmac_f32 v{ACC + 16 * (nb - 1) + 4 * mb + r}, v{P + 16 * nxt + 4 * mb + r}, v{SC + mb}")
        if nb + 1 < NB:
            emit("s_waitcnt lgkmcnt(0)")
    # fold of the last block: the 12 folds of mb 0..2 separate the last MFMA from the read of its result
    last = (NB - 1) & 1
    for mb in range(MB):
        for r in range(4):
            emit(f"v_fmac_f32 v{ACC + 16 * (NB - 1) + 4 * mb + r}, v{P + 16 * last + 4 * mb + r}, v{SC + mb}")


def step(stage, c):
    """K step c (0..3) of a trip.  s50 = 1 on the last trip."""
    for mb in range(MB):
        emit(f"v_mul_f32 v{SC + mb}, s{56 + c}, v{SAN + mb}")
    if c == 0:
        # next group of scales: into the other half of the scale buffer
        emit("s_cmp_eq_u32 s50, 1")
        emit("s_cbranch_scc1 Lnogrp%=")
        emit("s_xor_b32 s54, s54, 4096")
        scale_group_copy_body("b")
        emit("Lnogrp%=:")
    if c == 3:
        emit("s_cmp_eq_u32 s50, 1")
        emit("s_cbranch_scc1 Lnodma%=")
        dma(stage ^ 1)
        emit("Lnodma%=:")
        # the next step belongs to the next group
        emit("s_xor_b32 s55, s55, 4096")
        emit("v_add_u32 v39, s55, v38")
        read_scales(0)
    else:
        dma(stage ^ 1)
        read_scales(c + 1)
    compute(stage)
    emit("s_waitcnt vmcnt(0) lgkmcnt(0)")
    emit("s_barrier")


def main():
    # ---- prologue
    emit("s_mov_b64 s[40:41], %[abase]")
    emit("s_mov_b64 s[42:43], %[bbase]")
    emit("s_mov_b64 s[44:45], %[sbase]")
    emit("s_mov_b64 s[46:47], %[bsptr]")
    emit("s_mov_b32 s48, %[m0base]")
    emit("s_mov_b32 s49, %[trips]")
    emit("s_mov_b32 s53, %[copies]")
    emit("s_mov_b32 s54, 0")
    emit("s_mov_b32 s55, 0")
    for i, name in enumerate(("ard0", "ard1", "brd0", "brd1")):
        emit(f"v_mov_b32 v{RD[0][i]}, %[{name}]")
        emit(f"v_add_u32 v{RD[1][i]}, {STAGE}, %[{name}]")
    emit("v_mov_b32 v38, %[srd]")
    emit("v_mov_b32 v39, %[srd]")
    for r in range(128):
        emit(f"v_mov_b32 v{ACC + r}, 0")
    scale_group_copy_body("a")
    dma(0)
    emit("s_waitcnt vmcnt(0) lgkmcnt(0)")
    emit("s_barrier")
    read_scales(0)
    emit("s_waitcnt lgkmcnt(0)")
    # ---- main loop: one trip = four K steps = one group of scales
    emit("Lloop%=:")
    emit("s_mov_b64 s[56:57], s[60:61]")
    emit("s_mov_b64 s[58:59], s[62:63]")
    emit("s_sub_u32 s49, s49, 1")
    emit("s_cmp_eq_u32 s49, 0")
    emit("s_cselect_b32 s50, 1, 0")
    for c in range(4):
        step(c & 1, c)
    emit("s_cmp_lg_u32 s50, 1")
    emit("s_cbranch_scc1 Lloop%=")

    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "gemm_big_loop.inc"), "w") as f:
        f.write("// Generated by gen_gemm_loop.py -- do not edit.\n")
        for ln in lines:
            f.write('"' + ln + '\\n"\n')


if __name__ == "__main__":
    main()
