#!/usr/bin/env python3
"""Generates gemm_big_loop.inc: the hand-scheduled main loop of the 256 x 256 block-scaled
FP8 GEMM (fp32 scales) as one inline-asm string for gfx950.

Why generated assembly: the loop must keep eight MFMA results in flight while the VALU folds
the previous block into the fp32 accumulators and the LDS streams the weight fragments two
blocks ahead.  With 128 accumulator registers per lane the compiler serialises
MFMA -> fold -> MFMA instead; fixing the register plan by hand removes that.

Register plan (per lane, all physical):
  v[128:255] acc[nb][mb][r] = v[128 + 16*nb + 4*mb + r]      (outputs of the asm statement)
  v[96:127]  p[buf][mb][r]  = v[96 + 16*buf + 4*mb + r]       MFMA results of block nb (buf = nb & 1)
  v[64:95]   af[mb]         = v[64 + 8*mb : 71 + 8*mb]        activation fragments of this K step
  v[48:63], v[36:43]  wf[nb % 3]                              weight fragment of block nb (three buffers)
  v[44:47]   sc[mb]         = As[m, kb] * Bs[n/128, kb]       (raw As of the next step from the end of a step on)
  v34, v35   LDS address of the lane's activation scales: buffer half 0, half in use
  v[30:33]   LDS fragment read addresses a0, a1, b0, b1 (stage and block go into the offset field)
  s[40:55]   bases, counters, M0 base, buffer toggles
  s[56:59], s[60:63]  weight scales of this / the next group of four steps
LDS: activation stages at 0 and 32 KB, weight stages at 64 and 96 KB, scale groups at 128 KB.
One K step = 128 bytes of K = one scale block: 8 DMA instructions for the next stage, 8 + 16
LDS fragment reads, 32 MFMA 16x16x128 (zero C), 128 FMA folds.  Fragment reads are waited for
one at a time (counted lgkmcnt), so the first MFMA of a step starts after 4 of the 14 reads.

Scales: a gather of one activation scale per lane per step costs the texture path about as much as
the operand copies themselves (16 distinct cache lines per instruction), so the scales move in groups
of four K steps: waves 0..3 copy 16 bytes per activation row (256 rows) straight into a small LDS
buffer with one global_load_lds_dwordx4 each, the four weight scales come with one s_load_dwordx4,
and each step reads its four activation scales from LDS.  Hence K must be a multiple of 512 here.
The scalar load shares lgkmcnt with the LDS reads and returns out of order, so it is only issued
where no counted wait follows before the next full wait.
"""
import os

MB = 4                                     # 16-row blocks per wave (64 activation rows)


def configure(tm, tn, waves_m, waves_n, ksub, hw=False, nstage=2, brow=False, early=False, wide=False, idle=False, pingpong=False, nn=False,
              bf16=False):
    """Tile tm x tn, waves_m x waves_n waves of 64 x (tn / waves_n); a stage holds ksub K blocks of 128; nstage
    stages in LDS (2: the copies of the next stage overlap this one; 4 with ksub 1: three K steps are in flight,
    for problems of about one tile per CU whose time is the chain of K steps)."""
    global A_BYTES, B_BYTES, SCL_LDS, SCL_HALF, NB, WAVES, KSUB, SPLIT, HW, NSTAGE, BROW, EARLY, WIDE, lines
    global ACC, P, AF, SC, SC2, SAN, WFB, RA0, RA1, RB0, RB1, SRD0, SRD, WS1, WS2, WSCUR, HALFSPLIT, ROT, WITH_IDLE, IDLE, PINGPONG, GRP, SPREAD, NN, BF, RBN
    global WIDE_GROUP, WIDE_PART, BF16
    # bf16: the operands are bf16 values (a K step of 128 bytes is 64 of them) and every matrix instruction of the
    # hardware-scaled loop becomes two v_mfma_f32_16x16x32_bf16 on the halves of the same fragment registers, accumulating
    # in place: a lane's first four registers hold values 16 lq .. 16 lq + 7 of its row and the other four 16 lq + 8 .. + 15,
    # for both operands alike, so the two instructions together sum over all 64 values.  Nothing else changes (copies,
    # fragment reads, waits, hand-backs; the scale operands are simply not used): the unscaled bf16 NT GEMM.
    BF16 = bf16
    assert not bf16 or (hw and not brow and not nn and not wide)
    # idle: a second copy of the loop for waves none of whose activation rows exist (s93 = 1): an expert's short tile
    # of at most 64 rows leaves the second wave row of the 128 x 256 tile without work
    WITH_IDLE, IDLE = idle, False
    # pingpong: a SIMD holds one wave of the first half of the workgroup's waves and one of the second half, and its
    # arbiter prefers the older one: measured on the 256 x 256 loop, waves 0..3 spent 38 % of the loop waiting at the
    # barriers for waves 4..7 (12 %), which then ran alone and could not keep the matrix pipe busy.  With pingpong the
    # two halves run their own copy of the loop in which the wave priority (s_setprio) alternates from block to block,
    # opposite in the two copies: one wave issues its block's matrix instructions while the other folds and reads.
    # Measured: the two halves then wait alike (13 % and 9 %) and the 256 x 256 and 256 x 288 loops gain 1 - 2 %; the
    # flat 128 x 256 loop of the grouped kernel gains nothing and keeps one body.
    PINGPONG, GRP = pingpong, 0
    HW = hw
    # nn: the weights are stored with the contraction index as their row index ([K, N] row-major: the data gradient of a
    # linear layer on the stored weight, C = A W).  A stage then holds 128 contraction rows of tn bytes each, copied as
    # stored (a copy instruction moves 4 rows of 256 bytes), and the matrix instruction's weight operand -- 32
    # consecutive contraction bytes of one column per lane -- is gathered by ds_read_b64_tr_b8, which hands lane
    # (i, p) of every 16 the bytes i of the eight 8-byte rows 2 j + p that the 16 lanes address: with lane pairs on
    # the two halves of 16 bytes of one contraction row, eight rows per instruction, a lane receives column i + 8 p
    # of 8 consecutive contraction rows, and four instructions fill the 32 bytes of a K step.  Every block of 16
    # columns has its own address register (the 16-byte chunks of a row are XOR-swizzled by the row, so a block is not
    # an offset away from the next).  All of a stage's weight rows are read until the end of a step: the early
    # hand-back returns the activation rows only, every weight copy waits for the end of the step.  The weight scale
    # of a K step is one byte of a row of the [K / 128, N / 128] table: four strided loads per group, put together
    # with scalar instructions.  Hardware-scaled loops only.
    NN = nn
    assert not nn or (hw and early and not wide and not brow and ksub == 1 and tn == 256)
    BF = 4 if nn else 2                                    # LDS instructions per weight fragment
    # A wave column of 64 weight rows is one copy of eight waves: its first half (the 32 rows the first two blocks read)
    # is then what waves 0 .. 3 copy and its second half what waves 4 .. 7 copy, so the early hand-back splits the
    # weight copies by wave (s87 = 1 for the first half of the waves) instead of by copy index.
    HALFSPLIT = early and tn // waves_n == 64 and waves_m * waves_n == 8 and not nn
    # one copy behind each matrix instruction instead of runs of copies (see dma_chunks); the flat tile, whose weight
    # copies are split by wave behind one branch, keeps its runs
    SPREAD = early and not HALFSPLIT and SPREAD_ON
    # wide: a wave owns 64 x 144 columns (nine 16-column blocks), e.g. the 256 x 288 tile that cuts 18432 weight rows
    # into exactly 64 tile columns, or 64 x 112 columns (seven blocks): the 256 x 224 tile that cuts 7168 weight rows
    # into 32.  144 columns always straddle two weight-scale blocks and 112 mostly do, at a 16-column boundary known
    # only at run time (s74 = first block that takes the second scale row; past the last block if there is none): the
    # folds read one set of scale products, which is switched to the second row's products when the loop reaches that
    # block.  The accumulators take up to 144 registers, so the plan below moves everything down; fragment read
    # addresses and the scale buffer base are used straight from the asm operands, and the weight copies share one
    # per-lane offset (the tile's weight rows are never clamped: N is a multiple of the tile width) with one scalar
    # base per copy.
    WIDE = wide
    if wide:
        assert tm == 256 and tn in WIDE_PLANS and waves_m == 4 and waves_n == 2 and ksub == 1 and nstage == 2 and not brow
        WIDE_GROUP, WIDE_PART = WIDE_PLANS[tn]
        ACC, P, AF, WFB = 112, 80, 48, (32, 40)
        SAN, SC, SC2, SRD = 24, 28, 20, "v19"
        WS1, WS2, WSCUR = "v20", "v21", "v22"            # hardware-scaled variant: weight-scale bytes of row 1, row 2, in use
        RA0, RA1, RB0, RB1, SRD0 = "%[ard0]", "%[ard1]", "%[brd0]", "%[brd1]", "%[srd]"
    else:
        ACC, P, AF, WFB = 128, 96, 64, (48, 56)
        SAN, SC, SC2, SRD = 40, 44, None, "v35"
        WS1 = WS2 = WSCUR = "v36"
        RA0, RA1, RB0, RB1, SRD0 = "v30", "v31", "v32", "v33", "v34"
    # early: a stage is handed back in two parts.  Half way through a K step every wave holds the step's activation
    # fragments in registers and has read the first half of its weight blocks, so after a barrier there the
    # activation rows and the first half of each wave column's weight rows are requested for the step after the
    # next; the other weight rows follow at the end of the step as before.  Every request then has about one and a
    # half steps to land instead of one (the loop spends its waiting time at the end-of-step wait for the copies).
    EARLY = early
    assert not early or (nstage in (2, 3) and ksub == 1)
    # Three stages (with the early hand-back): the stage a step uses no longer follows from its place in the trip of four,
    # so the stage offsets live in registers.  s89 / s90 = LDS offset of the stage in use (activations / weights), s91 / s92
    # = of the stage just finished (what the end-of-step copies overwrite); the fragment read addresses v30 .. v33 are the
    # lane's stage-0 addresses (asm operands) plus the offsets in use.  Requests then have two to two and a half steps to
    # land: for tiles whose time is the latency of their weight stream (few activation rows per expert).
    ROT = early and nstage == 3
    assert not ROT or not wide
    NSTAGE = nstage
    BROW = brow                 # weight scales per row and K step (e8m0, hardware-scaled loop only) instead of per 128 rows
    assert not brow or (hw and tm == 128 and tn == 128)
    assert nstage == 2 or (nstage in (3, 4) and ksub == 1)
    assert tm == 64 * waves_m
    WAVES = waves_m * waves_n
    KSUB = ksub
    A_BYTES, B_BYTES = tm * 128, tn * 128
    SCL_LDS = nstage * ksub * (A_BYTES + B_BYTES)          # activation-scale buffer: 2 halves x tm rows x 16 bytes
    SCL_HALF = tm * 16        # (the e8m0 variant uses 4 of every 16 bytes: one wave writes 64 rows x 4 bytes per KB)
    NB = tn // waves_n // 16
    RBN = [f"v{96 + b}" for b in range(NB)]               # nn: fragment read address of block b (the fp32 loops' result registers are free)
    # a wave whose columns are not a multiple of 128 wide can straddle two weight-scale blocks: two scale rows
    # are loaded and each pair of 16-column blocks takes the one the set-up code selected for it
    SPLIT = (tn // waves_n) % 128 != 0 and (tn // waves_n) > 64 and not wide
    assert (tm // 8) % WAVES == 0 and ((tn // 8) % WAVES == 0 or wide)
    assert not early or wide or ((tn // 8 // WAVES) % 2 == 0 and (tn // waves_n // 16) % 2 == 0)
    assert not HALFSPLIT or WAVES == 8
    lines = []


def a_lds(stage, sub):
    """LDS offset of the activation rows of K block sub of a stage (all activation blocks come first)."""
    return (stage * KSUB + sub) * A_BYTES


def b_lds(stage, sub):
    """Same for the weight rows, relative to the first weight block (at NSTAGE * KSUB * A_BYTES)."""
    return (stage * KSUB + sub) * B_BYTES


SCP = (44, 224, 228)        # scale products per pair of 16-column blocks when a wave straddles two weight-scale blocks
SRDB0, SRDB = 37, 38        # row-scaled weights: LDS address of the lane's weight-scale dwords (half 0, half in use)
WSN, WSC = 96, 100          # ... the dwords of this group / of the next one, one per 16-row block
WB_EXTRA = ("s[42:43]", "s[78:79]", "s[80:81]", "s[82:83]", "s[84:85]")     # wide: weight base per copy
# wide, 288 columns: the 36 groups of 8 weight rows are dealt to the waves so that the early hand-back can request the
# first 64 rows of both wave columns (groups 0..7 and 18..25: the rows blocks 0..3 read) half way through a step and the
# other 80 rows of each at its end.  Copy i of wave w moves group WIDE_GROUP[i] + w; the fifth copy exists for waves 0..3
# only and moves groups 16, 17 (waves 0, 1) and 34, 35 (waves 2, 3): its group (less w) comes from the set-up code, in
# s88 as an LDS offset, and its base in the copy's own register pair.  All group numbers have the parity of w, so one
# per-lane source offset (row 8 w + lane / 8, swizzled chunk) serves all.
# 224 columns: 28 groups, wave columns of 14.  Mid-step: groups 0..7 and 14..21 (blocks 0..3 of both wave columns); at
# the end of the step the third copy moves groups 8..13 (waves 0..5) and 22, 23 (waves 6, 7) -- the set-up code's group --
# and the fourth, of waves 0..3 only, groups 24..27.
WIDE_PLANS = {288: ((0, 18, 8, 26, None), ("mid", "mid", "end", "end", "end")),
              224: ((0, 14, None, 24), ("mid", "mid", "end", "end"))}
WIDE_GROUP, WIDE_PART = WIDE_PLANS[288]

_uid = 0


IDLE = False        # emitting the loop body of a wave whose rows of the tile are all missing (see generate)
GRP = 0             # which half of the waves the body being emitted is for (see configure: pingpong)


def emit(s):
    if IDLE:
        # such a wave keeps its share of the copies, the barriers and the counters, and drops the arithmetic: fragment
        # and scale reads, matrix instructions, folds, scale products, and the waits that only order those
        if s.startswith(("ds_read", "v_mfma", "v_fmac", "v_mul_f32", "v_mov_b32", "v_add_u32", "s_load_dword", "s_waitcnt lgkmcnt", "s_setprio")):
            return
        s = s.replace("%=", "i%=")
    elif GRP == 1:
        s = s.replace("%=", "b%=")
    lines.append(s)


def vr(base, n):
    return f"v[{base}:{base + n - 1}]"


def dma(stage, part="all"):
    """Issue the global->LDS copies of one stage; the operand bases advance by one K block after each.
    part "mid": the activation rows and the weight copies with an even index (the first half of each wave
    column's rows), then the activation base advances; part "end": the odd weight copies, then the weight base."""
    bbase = NSTAGE * KSUB * A_BYTES
    for sub in range(KSUB):
        if part in ("all", "mid"):
            for i in range(A_BYTES // 1024 // WAVES):
                if ROT:
                    emit(f"s_add_u32 m0, s48, {i * WAVES * 1024}")
                    emit("s_add_u32 m0, m0, s89")
                else:
                    emit(f"s_add_u32 m0, s48, {a_lds(stage, sub) + i * WAVES * 1024}")
                emit(f"s_mov_b64 exec, %[amask{i}]")          # lanes whose activation row exists (see the prologue)
                emit(f"global_load_lds_dwordx4 %[aoff{i}], s[40:41]")
                emit("s_mov_b64 exec, s[98:99]")
        ncopies = -(-B_BYTES // 1024 // WAVES)
        if HALFSPLIT and part != "all":
            global _uid
            _uid += 1
            emit(f"s_cmp_eq_u32 s87, {0 if part == 'mid' else 1}")          # mid: the first four waves copy, end: the others
            emit(f"s_cbranch_scc1 Lnoh{_uid}%=")
        for i in range(ncopies):
            if WIDE:
                if part != "all" and WIDE_PART[i] != part:
                    continue
            elif NN:
                if part == "mid":
                    continue
            elif not HALFSPLIT and ((part == "mid" and i % 2) or (part == "end" and i % 2 == 0)):
                continue
            partial = WIDE and (i + 1) * WAVES * 1024 > B_BYTES       # only the first waves have rows left for this copy
            if partial:
                _uid += 1
                emit("s_cmp_eq_u32 s86, 0")
                emit(f"s_cbranch_scc1 Lnobx{_uid}%=")
            if WIDE and WIDE_GROUP[i] is None:
                emit(f"s_add_u32 m0, s48, {bbase + b_lds(stage, sub)}")
                emit("s_add_u32 m0, m0, s88")
            elif WIDE:
                emit(f"s_add_u32 m0, s48, {bbase + b_lds(stage, sub) + WIDE_GROUP[i] * 1024}")
            elif ROT:
                emit(f"s_add_u32 m0, s48, {bbase + i * WAVES * 1024}")
                emit(f"s_add_u32 m0, m0, {'s90' if part == 'mid' else 's92'}")
            else:
                emit(f"s_add_u32 m0, s48, {bbase + b_lds(stage, sub) + i * WAVES * 1024}")
            emit("s_nop 0")
            if WIDE:
                emit(f"global_load_lds_dwordx4 %[boff0], {WB_EXTRA[i]}")
            else:
                emit(f"global_load_lds_dwordx4 %[boff{i}], s[42:43]" + (" nt" if ROT else ""))     # the flat tile's weights are read once: streamed past the L2's resident lines
            if partial:
                emit(f"Lnobx{_uid}%=:")
        if HALFSPLIT and part != "all":
            emit(f"Lnoh{_uid}%=:")
        if part in ("all", "mid"):
            emit("s_add_u32 s40, s40, 128")
            emit("s_addc_u32 s41, s41, 0")
        if part in ("all", "end"):
            for i in range(ncopies if WIDE else 1):
                lo = int(WB_EXTRA[i][2:4])
                emit(f"s_add_u32 s{lo}, s{lo}, {'s66' if NN else 128}")      # nn: 128 rows of the stored weight further on
                emit(f"s_addc_u32 s{lo + 1}, s{lo + 1}, 0")


def dma_chunks(stage, part):
    """The copies of dma(stage, part) as a list of pieces, one copy instruction each (with its m0 / exec set-up and the
    label that closes a copy only some waves have); the advance of the operand bases rides on the last piece.  The
    loop issues one piece behind each matrix instruction instead of all copies in one run: the eight waves reach the
    copies together (they follow a barrier), a run of six from each queues 48 KB of requests in front of the CU's one
    address unit, and a wave stuck at its third copy issues no matrix instruction either."""
    global lines
    saved, lines = lines, []
    dma(stage, part)
    body, lines = lines, saved
    out, cur, i = [], [], 0
    while i < len(body):
        cur.append(body[i])
        if body[i].startswith("global_load_lds"):
            while i + 1 < len(body) and (body[i + 1].startswith("Lnobx") or body[i + 1].startswith("s_mov_b64 exec, s[98:99]")):
                cur.append(body[i + 1])
                i += 1
            out.append(cur)
            cur = []
        i += 1
    if cur:
        assert out
        out[-1] += cur
    return out


def emit_piece(piece, tag, cond):
    """One piece of dma_chunks behind a matrix instruction; cond: skipped on the last trip (s50 = 1), when the step it
    would fill lies past the end of K."""
    if cond:
        emit("s_cmp_eq_u32 s50, 1")
        emit(f"s_cbranch_scc1 Lnop{tag}%=")
    lines.extend(piece)
    if cond:
        emit(f"Lnop{tag}%=:")


def copies_per_part():
    """Requests of one wave in the mid-step part and in the end-of-step part of a stage (early hand-back)."""
    a, b = A_BYTES // 1024 // WAVES, B_BYTES // 1024 // WAVES
    if NN:
        return a, b
    if WIDE:
        # waves 0 .. 3 issue one more request in the end part than the others; counting without it makes their waits
        # one request stricter
        return a + WIDE_PART.count("mid"), B_BYTES // 1024 // WAVES - WIDE_PART.count("mid")
    if HALFSPLIT:
        # a wave issues its weight copies in one of the two parts; either way the two parts together are a + b
        # requests, and counting none for the end part only makes the last trip's waits stricter
        return a + b, 0
    return a + (b + 1) // 2, b // 2


def younger_requests(c, at_end, last_trip):
    """Requests of one wave that are younger than the ones a wait in step c depends on.  The mid-step wait needs the
    end-of-step part issued NSTAGE steps earlier (the second weight half of this step), the end-of-step wait the
    mid-step part issued NSTAGE - 1 steps earlier (activations and first weight half of the next step).  Parts are
    issued in the order mid(j), end(j), mid(j + 1) ...; on the last trip a part of step j exists only if the step it
    fills, j + NSTAGE, is still inside the trip (steps of earlier trips, j < 0, always do)."""
    mid, end = copies_per_part()
    # nn: every block of a step reads all of the stage's weight rows, so the whole stage -- the activation rows asked for
    # mid-step and the weight rows asked for at the end of the same step -- must have landed when the step begins: the
    # end-of-step wait covers both, the mid-step wait has nothing to wait for (wait_copies leaves it out)
    need = (("end", c - NSTAGE + 1) if NN else ("mid", c - NSTAGE + 1)) if at_end else ("end", c - NSTAGE)
    upto = ("mid", c) if at_end else ("end", c - 1)
    parts = []
    for j in range(need[1], c + 1):
        parts += [("mid", j), ("end", j)]
    n = 0
    for kind, j in parts[parts.index(need) + 1:parts.index(upto) + 1]:
        if not last_trip or j < 0 or j + NSTAGE <= 3:
            n += mid if kind == "mid" else end
    return n


def wait_copies(c, at_end, extra=""):
    """Early hand-back: wait until the requests this point depends on have landed.  Requests return in order, so it
    is enough to bound how many younger ones may still be out (c = step within the trip, s50 = 1 on the last trip,
    on which nothing is requested for steps past the end)."""
    if NN and not at_end:
        emit(f"s_waitcnt{extra}")
        return
    steady, last = younger_requests(c, at_end, False), younger_requests(c, at_end, True)
    tag = f"{'e' if at_end else 'm'}{c}"
    if last != steady:
        emit("s_cmp_eq_u32 s50, 1")
        emit(f"s_cbranch_scc1 Lwl{tag}%=")
    emit(f"s_waitcnt vmcnt({steady}){extra}")
    if last != steady:
        emit(f"s_branch Lwj{tag}%=")
        emit(f"Lwl{tag}%=:")
        emit(f"s_waitcnt vmcnt({last}){extra}")
        emit(f"Lwj{tag}%=:")


def scale_group_copy(tag):
    """Copy the activation scales of the next group of four K steps into LDS (waves 0..3, one row per
    lane, 16 bytes each)."""
    emit("s_cmp_eq_u32 s53, 0")
    emit(f"s_cbranch_scc1 Lnosc{tag}%=")
    emit("s_add_u32 m0, s48, s54")
    if BROW:
        emit("s_add_u32 m0, m0, s51")                     # activation rows or weight rows: the set-up code says where
    else:
        emit(f"s_add_u32 m0, m0, {SCL_LDS}")
    emit("s_nop 0")
    emit("global_load_lds_dword %[soff], s[44:45]" if HW else "global_load_lds_dwordx4 %[soff], s[44:45]")
    emit(f"Lnosc{tag}%=:")
    emit(f"s_add_u32 s44, s44, {4 if HW else 16}")
    emit("s_addc_u32 s45, s45, 0")


def weight_scale_load():
    """The four weight scales of the next group into s[60:63] (and those of the second scale row into s[68:71])."""
    if BROW:
        return                                            # they travel with the activation scales, see scale_group_copy
    if NN:
        # one byte per K step, a table row (s64 bytes) apart: the aligned dword around each, taken apart at the top of the loop
        for i in range(4):
            emit(f"s_load_dword s{60 + i}, s[46:47], 0x0")
            emit("s_add_u32 s46, s46, s64")
            emit("s_addc_u32 s47, s47, 0")
        return
    if HW:
        emit("s_load_dword s60, s[46:47], 0x0")          # four e8m0 bytes = four K steps
        emit("s_add_u32 s46, s46, 4")
        emit("s_addc_u32 s47, s47, 0")
        if WIDE:
            emit("s_load_dword s68, s[72:73], 0x0")
            emit("s_add_u32 s72, s72, 4")
            emit("s_addc_u32 s73, s73, 0")
        return
    emit("s_load_dwordx4 s[60:63], s[46:47], 0x0")
    emit("s_add_u32 s46, s46, 16")
    emit("s_addc_u32 s47, s47, 0")
    if SPLIT or WIDE:
        emit("s_load_dwordx4 s[68:71], s[72:73], 0x0")
        emit("s_add_u32 s72, s72, 16")
        emit("s_addc_u32 s73, s73, 0")


def read_frag(dst, addr0, addr1, off):
    emit(f"ds_read_b128 {vr(dst, 4)}, {addr0} offset:{off}")
    emit(f"ds_read_b128 {vr(dst + 4, 4)}, {addr1} offset:{off}")


def read_bfrag(dst, nb, stage_off):
    """The weight fragment of block nb (16 columns x 128 bytes of K) into v[dst : dst + 7]."""
    if NN:
        for t in range(4):
            emit(f"ds_read_b64_tr_b8 {vr(dst + 2 * t, 2)}, {RBN[nb]} offset:{stage_off + 2048 * t}")
    else:
        read_frag(dst, RB0, RB1, stage_off + nb * 2048)


def read_scales(col):
    """Raw activation scales of the lane's four block rows for one K step (column col of the group half at v35).
    e8m0 variant: the four bytes of the next group, once per trip, into the spare set v[44:47]."""
    if HW:
        if col == 0:
            for mb in range(MB):
                emit(f"ds_read_b32 v{SC + mb}, {SRD} offset:{mb * 64}")
            if BROW:
                for nb in range(NB):
                    emit(f"ds_read_b32 v{WSC + nb}, v{SRDB} offset:{nb * 64}")
        return
    for mb in range(MB):
        emit(f"ds_read_b32 v{SAN + mb}, {SRD} offset:{mb * 256 + col * 4}")


def par(c, nb):
    """Which of the two weight-fragment / result buffers block nb of step c uses.  They alternate from block to block,
    across step boundaries too: with an odd number of blocks the first block of the next step (whose fragment is read
    while the last block of this step still computes) must not land in that block's buffer.  Four steps per trip
    make the pattern repeat from trip to trip."""
    return (c * NB + nb) & 1


def mfma(nb, mb, c=0):
    if HW:
        # scales applied by the matrix core: byte c of the weight-scale register (uniform) and of the lane's
        # activation-scale register; accumulation in place
        acc = vr(ACC + 16 * nb + 4 * mb, 4)
        if BF16:
            for half in (0, 4):
                emit(f"v_mfma_f32_16x16x32_bf16 {acc}, {vr(WFB[par(c, nb)] + half, 4)}, {vr(AF + 8 * mb + half, 4)}, {acc}")
            return
        wscale = f"v{WSN + nb}" if BROW else WSCUR
        emit(f"v_mfma_scale_f32_16x16x128_f8f6f4 {acc}, {vr(WFB[par(c, nb)], 8)}, {vr(AF + 8 * mb, 8)}, {acc}, {wscale}, v{SAN + mb} "
             f"op_sel:[{c & 1},{c & 1},0] op_sel_hi:[{c >> 1},{c >> 1},0]")
        return
    emit(f"v_mfma_f32_16x16x128_f8f6f4 {vr(P + 16 * par(c, nb) + 4 * mb, 4)}, {vr(WFB[par(c, nb)], 8)}, {vr(AF + 8 * mb, 8)}, 0")


def fold(nb, mb, c=0):
    if HW:
        return
    sc = SCP[nb >> 1] if SPLIT else SC
    for r in range(4):
        emit(f"v_fmac_f32 v{ACC + 16 * nb + 4 * mb + r}, v{P + 16 * par(c, nb) + 4 * mb + r}, v{sc + mb}")


def step(c):
    """K step c (0..3) of a trip; s50 = 1 on the last trip.

    On entry the fragments wf0 and af0..3 of this step are already on their way (10 LDS reads issued in the
    previous step's last block).  After the last K block of a stage comes the stage flip (wait for the copies
    of the next stage, barrier, issue the copies that overwrite the stage just finished); it and the first
    fragment reads of the next step happen inside the last block, so the matrix pipe keeps working across it."""
    stage, sub = (c // KSUB) % NSTAGE, c % KSUB
    flip = sub == KSUB - 1
    nstage, nsub = ((stage + 1) % NSTAGE, 0) if flip else (stage, sub + 1)
    aoff, boff = a_lds(stage, sub), b_lds(stage, sub)
    naoff, nboff = a_lds(nstage, nsub), b_lds(nstage, nsub)
    if ROT:
        aoff = boff = naoff = nboff = 0                  # the read addresses carry the stage
    if HW:
        pass
    elif SPLIT:
        # pairs 1 and 2 take the second scale row when their flag (s74, s75) is set
        emit("s_cmp_eq_u32 s74, 1")
        emit(f"s_cselect_b32 s76, s{64 + c}, s{56 + c}")
        emit("s_cmp_eq_u32 s75, 1")
        emit(f"s_cselect_b32 s77, s{64 + c}, s{56 + c}")
        for mb in range(MB):
            emit(f"v_mul_f32 v{SCP[0] + mb}, s{56 + c}, v{SAN + mb}")
            emit(f"v_mul_f32 v{SCP[1] + mb}, s76, v{SAN + mb}")
            emit(f"v_mul_f32 v{SCP[2] + mb}, s77, v{SAN + mb}")
    else:
        for mb in range(MB):
            emit(f"v_mul_f32 v{SC + mb}, s{56 + c}, v{SAN + mb}")
            if WIDE:
                emit(f"v_mul_f32 v{SC2 + mb}, s{64 + c}, v{SAN + mb}")
    if HW and WIDE:
        emit(f"v_mov_b32 {WSCUR}, {WS1}")
    if c == 0:
        # next group of scales: into the other half of the scale buffer
        emit("s_cmp_eq_u32 s50, 1")
        emit("s_cbranch_scc1 Lnogrp%=")
        emit(f"s_xor_b32 s54, s54, {SCL_HALF}")
        scale_group_copy("b")
        weight_scale_load()
        emit("Lnogrp%=:")
    if c == 3:
        # the next step belongs to the next group
        emit(f"s_xor_b32 s55, s55, {SCL_HALF}")
        emit(f"v_add_u32 {SRD}, s55, {SRD0}")
        if BROW:
            emit(f"v_add_u32 v{SRDB}, s55, v{SRDB0}")
    pieces = []                  # copies waiting for their slot behind a matrix instruction: (piece, tag, skipped on the last trip)
    read_bfrag(WFB[par(c, 1)], 1, boff)
    # LDS queue now: wf0, af0..3, wf1 = 12 reads (16 with four instructions per weight fragment)
    if PINGPONG:
        emit(f"s_setprio {(c * NB + GRP + 1) & 1}")
    for mb in range(MB):
        emit(f"s_waitcnt lgkmcnt({(3 - mb) * 2 + BF})")
        mfma(0, mb, c)
    read_scales((c + 1) & 3)
    for nb in range(1, NB):
        if PINGPONG:
            emit(f"s_setprio {(c * NB + nb + GRP + 1) & 1}")
        if HW and WIDE:
            # from the first block in the second weight-scale block on, the matrix instructions take that row's bytes
            emit(f"s_cmp_eq_u32 s74, {nb}")
            emit(f"s_cbranch_scc0 Lsw{c}_{nb}%=")
            emit(f"v_mov_b32 {WSCUR}, {WS2}")
            emit(f"Lsw{c}_{nb}%=:")
        # Early hand-back: the barrier sits in front of the first read of the second weight half (block NB / 2, read
        # one block ahead), so that half is known to have landed before anyone reads it, and behind every wave's
        # last read of the first half, so those rows and the activation rows can be requested again right after it.
        handback = EARLY and nb == (3 if WIDE else NB // 2 - 1)      # wide: blocks 0..3 are the first part whatever NB
        if handback:
            assert nb + 1 < NB and not pieces
            wait_copies(c, False, " lgkmcnt(0)")
            emit("s_barrier")
        if nb + 1 < NB:
            read_bfrag(WFB[par(c, nb + 1)], nb + 1, boff)
        if nb == 1:
            pending = 4 if (not HW or c == 3) else 0                # scale reads issued after block 0
            if BROW and c == 3:
                pending += NB
            emit(f"s_waitcnt lgkmcnt({pending + (BF if NB > 2 else 0)})")        # those and wf2 may still be outstanding
        elif nb + 1 < NB:
            emit(f"s_waitcnt lgkmcnt({BF})")
        if nb + 1 == NB:
            if flip:
                # every wave has read all of this stage and its share of the next stage has landed
                assert not pieces                # the waits count every copy of the mid-step part as issued
                if EARLY:
                    wait_copies(c, True, " lgkmcnt(0)")
                elif NSTAGE == 2:
                    emit("s_waitcnt vmcnt(0) lgkmcnt(0)")
                else:
                    # four stages: the copies of the two steps after the next one may stay in flight (the group's
                    # scale copy, one more request of some waves, is then counted with them: it makes the wait a
                    # request stricter and has itself landed by the flip of step 2, before step 3 reads the group).
                    # On the last trip nothing new is requested, so fewer are left behind each step.
                    per = (A_BYTES + B_BYTES) // 1024 // WAVES
                    steady, last = 2 * per, max(0, (2 - c) * per)
                    if last != steady:
                        emit("s_cmp_eq_u32 s50, 1")
                        emit(f"s_cbranch_scc1 Lwl{c}%=")
                    emit(f"s_waitcnt vmcnt({steady}) lgkmcnt(0)")
                    if last != steady:
                        emit(f"s_branch Lwj{c}%=")
                        emit(f"Lwl{c}%=:")
                        emit(f"s_waitcnt vmcnt({last}) lgkmcnt(0)")
                        emit(f"Lwj{c}%=:")
                emit("s_barrier")
                if ROT:
                    # the next stage becomes the one in use
                    emit("s_mov_b32 s91, s89")
                    emit("s_mov_b32 s92, s90")
                    emit(f"s_add_u32 s89, s89, {A_BYTES}")
                    emit(f"s_cmp_eq_u32 s89, {NSTAGE * A_BYTES}")
                    emit("s_cselect_b32 s89, 0, s89")
                    emit(f"s_add_u32 s90, s90, {B_BYTES}")
                    emit(f"s_cmp_eq_u32 s90, {NSTAGE * B_BYTES}")
                    emit("s_cselect_b32 s90, 0, s90")
                    emit(f"v_add_u32 {RA0}, s89, %[ard0]")
                    emit(f"v_add_u32 {RA1}, s89, %[ard1]")
                    if NN:
                        for b in range(NB):
                            emit(f"v_add_u32 {RBN[b]}, s90, %[brdn{b}]")
                    else:
                        emit(f"v_add_u32 {RB0}, s90, %[brd0]")
                        emit(f"v_add_u32 {RB1}, s90, %[brd1]")
            else:
                emit("s_waitcnt lgkmcnt(0)")
            read_bfrag(WFB[par(c + 1, 0)], 0, nboff)
        for mb in range(MB):
            mfma(nb, mb, c)
            fold(nb - 1, mb, c)
            if handback and mb == 0:
                # the activation rows and the first weight half of the step after the next, into the rows just freed
                cond = c + NSTAGE >= 4 if ROT else c + 1 + KSUB >= 4
                if SPREAD:
                    pieces += [(pc, f"m{c}_{i}", cond) for i, pc in enumerate(dma_chunks(stage, "mid"))]
                else:
                    if cond:
                        emit("s_cmp_eq_u32 s50, 1")
                        emit(f"s_cbranch_scc1 Lnodmam{c}%=")
                    dma(stage, "mid")
                    if cond:
                        emit(f"Lnodmam{c}%=:")
            if nb + 1 == NB:
                read_frag(AF + 8 * mb, RA0, RA1, naoff + mb * 2048)
                if mb == 0 and flip:
                    # copies for the K blocks after the next stage overwrite the stage just finished
                    cond = NSTAGE == 4 or (c + NSTAGE >= 4 if ROT else c + 1 + KSUB >= 4)
                    if SPREAD:
                        assert not pieces
                        pieces += [(pc, f"e{c}_{i}", cond) for i, pc in enumerate(dma_chunks(stage, "end"))]
                        assert len(pieces) <= MB
                    else:
                        if cond:
                            emit("s_cmp_eq_u32 s50, 1")
                            emit(f"s_cbranch_scc1 Lnodma{c}%=")
                        dma(stage, "end" if EARLY else "all")
                        if cond:
                            emit(f"Lnodma{c}%=:")
            if pieces:
                emit_piece(*pieces.pop(0))
        if WIDE and not HW:
            # the folds of block nb follow (in the next block's shadow): if it is the first block in the second
            # weight-scale block, they and all later ones use that row's products
            emit(f"s_cmp_eq_u32 s74, {nb}")
            emit(f"s_cbranch_scc0 Lsw{c}_{nb}%=")
            for mb in range(MB):
                emit(f"v_mov_b32 v{SC + mb}, v{SC2 + mb}")
            emit(f"Lsw{c}_{nb}%=:")
    assert not pieces
    # fold of the last block: the 12 folds of mb 0..2 separate the last MFMA from the read of its result
    for mb in range(MB):
        fold(NB - 1, mb, c)


def loop_body():
    emit("Lloop%=:")
    if HW:
        # scales of this group: the lane's activation-scale bytes and the weight-scale bytes (uniform)
        for mb in range(MB):
            emit(f"v_mov_b32 v{SAN + mb}, v{SC + mb}")
        if BROW:
            for nb in range(NB):
                emit(f"v_mov_b32 v{WSN + nb}, v{WSC + nb}")
        elif NN:
            # byte (address & 3) of each of the four dwords -> the four scale bytes of this group in one register
            for i in range(4):
                emit(f"s_bfe_u32 s{60 + i}, s{60 + i}, s65")
            emit("s_lshl_b32 s61, s61, 8")
            emit("s_lshl_b32 s62, s62, 16")
            emit("s_lshl_b32 s63, s63, 24")
            emit("s_or_b32 s60, s60, s61")
            emit("s_or_b32 s62, s62, s63")
            emit("s_or_b32 s60, s60, s62")
            emit(f"v_mov_b32 {WS1}, s60")
        else:
            emit(f"v_mov_b32 {WS1}, s60")
            if WIDE:
                emit(f"v_mov_b32 {WS2}, s68")
    emit("s_mov_b64 s[56:57], s[60:61]")
    emit("s_mov_b64 s[58:59], s[62:63]")
    if SPLIT or WIDE:
        emit("s_mov_b64 s[64:65], s[68:69]")
        emit("s_mov_b64 s[66:67], s[70:71]")
    emit("s_sub_u32 s49, s49, 1")
    emit("s_cmp_eq_u32 s49, 0")
    emit("s_cselect_b32 s50, 1, 0")
    for c in range(4):
        step(c)
    emit("s_cmp_lg_u32 s50, 1")
    emit("s_cbranch_scc1 Lloop%=")


def generate():
    # ---- prologue
    # Activation rows past the end of the matrix (or of an expert's rows) are not copied: their lanes are switched off
    # for the copy instruction (%[amaskI] = lanes of copy I whose row exists).  Pointing them at a valid row instead
    # makes a workgroup ask for cache lines it is already waiting for, and the in-order L1 then holds back the
    # weight requests queued behind them: a tile with 64 of 128 rows valid ran a third slower than a full one.
    # What the LDS rows of missing activation rows hold only reaches accumulator rows that are never stored.
    emit("s_mov_b64 s[98:99], exec")
    emit("s_mov_b64 s[40:41], %[abase]")
    emit("s_mov_b64 s[42:43], %[bbase]")
    emit("s_mov_b64 s[44:45], %[sbase]")
    emit("s_mov_b64 s[46:47], %[bsptr]")
    if SPLIT:
        emit("s_mov_b64 s[72:73], %[bsptr2]")
        emit("s_mov_b32 s74, %[sel1]")
        emit("s_mov_b32 s75, %[sel2]")
    if WIDE:
        emit("s_mov_b64 s[72:73], %[bsptr2]")
        emit("s_mov_b32 s74, %[splitnb]")
        emit("s_mov_b32 s86, %[bextra]")
        # weight base of copy i: WIDE_GROUP[i] groups of 8 rows further on (%[bstride] = bytes per group); the fifth
        # copy's group comes from the set-up code (%[g4])
        for i in range(1, len(WIDE_GROUP)):
            lo = int(WB_EXTRA[i][2:4])
            if WIDE_GROUP[i] is None:
                emit("s_mul_i32 s87, %[bstride], %[g4]")
                emit("s_lshl_b32 s88, %[g4], 10")
            else:
                emit(f"s_mul_i32 s87, %[bstride], {WIDE_GROUP[i]}")
            emit(f"s_add_u32 s{lo}, s42, s87")
            emit(f"s_addc_u32 s{lo + 1}, s43, 0")
    if HALFSPLIT:
        emit("s_bfe_u32 s87, %[flags], 0x10003")           # bit 3 of the wave flags: first half of the waves
    emit("s_mov_b32 s48, %[m0base]")
    emit("s_mov_b32 s49, %[trips]")
    emit("s_and_b32 s53, %[flags], 1")                    # wave flags (one operand): bit 0 = this wave copies scales,
    emit("s_mov_b32 s54, 0")
    emit("s_mov_b32 s55, 0")
    for reg, name in ((RA0, "ard0"), (RA1, "ard1"), (RB0, "brd0"), (RB1, "brd1"), (SRD0, "srd"), (SRD, "srd")):
        if NN and name.startswith("brd"):
            continue
        if not reg.startswith("%"):
            emit(f"v_mov_b32 {reg}, %[{name}]")
    if NN:
        for b in range(NB):
            emit(f"v_mov_b32 {RBN[b]}, %[brdn{b}]")
        emit("s_mov_b32 s64, %[bsstride]")                 # bytes between two rows of the weight-scale table
        emit("s_mov_b32 s65, %[bsbfe]")                    # s_bfe_u32 operand: 8 bits from bit 8 * (table address & 3)
        emit("s_mov_b32 s66, %[bstep]")                    # bytes between two K steps of the stored weight
    if BROW:
        emit("s_mov_b32 s51, %[sdst]")
        emit(f"v_mov_b32 v{SRDB0}, %[srdb]")
        emit(f"v_mov_b32 v{SRDB}, %[srdb]")
    for r in range(16 * NB):
        emit(f"v_mov_b32 v{ACC + r}, 0")
    scale_group_copy("a")
    weight_scale_load()
    if EARLY:
        # both stages are requested in the order of the steady state (mid part, end part), then stage 0 and the
        # scale group (older) are waited for: what may stay out is exactly what the first waits of the loop allow
        for st in range(NSTAGE):
            if ROT:
                emit(f"s_mov_b32 s89, {st * A_BYTES}")
                emit(f"s_mov_b32 s90, {st * B_BYTES}")
                emit(f"s_mov_b32 s92, {st * B_BYTES}")
            dma(st, "mid")
            dma(st, "end")
        if ROT:
            emit("s_mov_b32 s89, 0")
            emit("s_mov_b32 s90, 0")
        emit(f"s_waitcnt vmcnt({(NSTAGE - 1) * sum(copies_per_part())}) lgkmcnt(0)")
        emit("s_barrier")
    else:
        dma(0)
    if EARLY:
        pass
    elif NSTAGE == 2:
        emit("s_waitcnt vmcnt(0) lgkmcnt(0)")
        emit("s_barrier")
        dma(1)                               # K >= 512: there are at least four steps, which two stages hold at most
    else:
        per = (A_BYTES + B_BYTES) // 1024 // WAVES
        for st in range(1, NSTAGE):          # K >= 512: the four stages hold exactly the first four steps
            dma(st)
        emit(f"s_waitcnt vmcnt({(NSTAGE - 1) * per}) lgkmcnt(0)")
        emit("s_barrier")
    for mb in range(MB):
        emit(f"ds_read_b32 v{(SC if HW else SAN) + mb}, {SRD} offset:{mb * (64 if HW else 256)}")
    if BROW:
        for nb in range(NB):
            emit(f"ds_read_b32 v{WSC + nb}, v{SRDB} offset:{nb * 64}")
    emit("s_waitcnt lgkmcnt(0)")
    read_bfrag(WFB[0], 0, 0)
    for mb in range(MB):
        read_frag(AF + 8 * mb, RA0, RA1, mb * 2048)
    # ---- main loop: one trip = four K steps = one group of scales
    global IDLE
    global GRP
    if WITH_IDLE:
        emit("s_bitcmp1_b32 %[flags], 1")                  # bit 1 = none of its activation rows exist,
        emit("s_cbranch_scc1 Lloopi%=")
    if PINGPONG:
        emit("s_bitcmp1_b32 %[flags], 2")                  # bit 2 = second half of the waves (bit 3: first half, flat tile)
        emit("s_cbranch_scc1 Lloopb%=")
    loop_body()
    if PINGPONG:
        emit("s_branch Ldone%=")
        GRP = 1
        loop_body()
        GRP = 0
    if WITH_IDLE:
        emit("s_branch Ldone%=")
        IDLE = True
        loop_body()
        IDLE = False
    if WITH_IDLE or PINGPONG:
        emit("Ldone%=:")
    if PINGPONG:
        emit("s_setprio 0")
    emit("s_waitcnt vmcnt(0) lgkmcnt(0)")
    if HW:
        emit("s_nop 15")                         # the last MFMAs have written the accumulators before they are read
        emit("s_nop 15")



PP = os.environ.get("LP_GEN_PINGPONG", "1") == "1"
SPREAD_ON = os.environ.get("LP_GEN_SPREAD", "1") == "1"


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    for name, cfg in (("gemm_big_loop.inc", (256, 256, 4, 2, 1, False, 2, False, True, False, True, PP)), ("gemm_big192_loop.inc", (256, 192, 4, 2, 1)),
                      ("gemm_mid_loop.inc", (128, 128, 2, 2, 1, False, 2, False, True)), ("gemm_mid2_loop.inc", (128, 128, 2, 2, 2)),
                      ("gemm_big_hw_loop.inc", (256, 256, 4, 2, 1, True, 2, False, True, False, True, PP)),
                      ("gemm_mid_hw_loop.inc", (128, 128, 2, 2, 1, True, 2, False, True)),
                      ("gemm_wide_loop.inc", (256, 288, 4, 2, 1, False, 2, False, True, True, True, PP)),
                      ("gemm_wide_hw_loop.inc", (256, 288, 4, 2, 1, True, 2, False, True, True, True, PP)),
                      ("gemm_wide224_loop.inc", (256, 224, 4, 2, 1, False, 2, False, True, True, True, PP)),
                      ("gemm_wide224_hw_loop.inc", (256, 224, 4, 2, 1, True, 2, False, True, True, True, PP)),
                      ("gemm_flat_loop.inc", (128, 256, 2, 4, 1, False, 3, False, True, False, True)),
                      ("gemm_flat_hw_loop.inc", (128, 256, 2, 4, 1, True, 3, False, True, False, True)),
                      ("gemm_mid4_loop.inc", (128, 128, 2, 2, 1, False, 4)), ("gemm_mid4_hw_loop.inc", (128, 128, 2, 2, 1, True, 4)),
                      ("gemm_mid_hwrow_loop.inc", (128, 128, 2, 2, 1, True, 2, True, True)),
                      ("gemm_big_hw_nn_loop.inc", (256, 256, 4, 2, 1, True, 2, False, True, False, True, PP, True)),
                      ("gemm_flat_hw_nn_loop.inc", (128, 256, 2, 4, 1, True, 3, False, True, False, True, False, True)),
                      ("gemm_big_bf16_loop.inc", (256, 256, 4, 2, 1, True, 2, False, True, False, True, PP, False, True))):
        configure(*cfg)
        generate()
        write(here, name)
    probe_bodies(here)


def probe_bodies(here):
    """Bodies of the matrix-pipe probe (probe/probe.hip: probe_mfma): eight matrix instructions into eight result buffers
    v[32:63], each followed by k FMAs that fold a buffer finished four instructions ago into v[64:127] -- the arithmetic
    of the fp32-scaled loops with no operand movement at all."""
    global lines
    for k in (0, 2, 4, 6, 8):
        lines = []
        for j in range(8):
            lines.append(f"v_mfma_f32_16x16x128_f8f6f4 v[{32 + 4 * j}:{35 + 4 * j}], v[0:7], v[8:15], 0")
            src = (j + 4) % 8
            for f in range(k):
                lines.append(f"v_fmac_f32 v{64 + (j * 8 + f) % 64}, v{32 + 4 * src + f % 4}, v20")
        write(os.path.join(here, "probe"), f"probe_mfma_body{k}.inc")
    # the hardware-scaled form, accumulating in place as the e8m0 loops do (unit scale bytes in v21)
    lines = [f"v_mfma_scale_f32_16x16x128_f8f6f4 v[{32 + 4 * j}:{35 + 4 * j}], v[0:7], v[8:15], v[{32 + 4 * j}:{35 + 4 * j}], v21, v21 "
             "op_sel:[0,0,0] op_sel_hi:[0,0,0]" for j in range(8)]
    write(os.path.join(here, "probe"), "probe_mfma_body_scaled.inc")
    lines = [f"v_mfma_f32_16x16x128_f8f6f4 v[{32 + 4 * j}:{35 + 4 * j}], v[0:7], v[8:15], v[{32 + 4 * j}:{35 + 4 * j}]" for j in range(8)]
    write(os.path.join(here, "probe"), "probe_mfma_body_inplace.inc")


def write(here, name):
    text = "// Generated by gen_gemm_loop.py -- do not edit.\n" + "".join('"' + ln + '\\n"\n' for ln in lines)
    path = os.path.join(here, name)
    # only files whose content differs are rewritten (their time stamps drive the rebuild), so running the
    # generator on every build also undoes a hand edit to any of its outputs
    if not os.path.exists(path) or open(path).read() != text:
        with open(path, "w") as f:
            f.write(text)
        print("regenerated", name)


if __name__ == "__main__":
    main()
