#!/usr/bin/env python3
"""Generator of the K loop of the 256 x 256 tile on FOUR waves (gemm_quad_hw_loop.inc): e8m0 scales applied by the
matrix cores, one wave per SIMD, a wave owns 128 x 128 of the tile.

Why a second loop family: with eight waves of 64 x 128 a K step reads 192 KB of fragments from LDS for 64 KB staged;
with four waves of 128 x 128 it reads 128 KB, and the 256 accumulators of a wave live in a[0:255] (the matrix
instruction writes them in place; nothing else touches them until the loop ends), which leaves the 256 vector
registers to fragments.  One wave per SIMD has nobody to cover for it, so every fragment is in registers long before
its matrix instruction: the activation fragments of a whole K step (8 blocks of 16 rows, 64 registers) are double
buffered and read one step ahead, the weight fragments (8 registers each) run through a ring of four, read two blocks
of eight matrix instructions ahead.

LDS: two stages of 256 activation rows + 256 weight rows x 128 bytes (rows in the order lds_row() of gemm_fp8_big.hip,
16-byte chunks XOR-swizzled), then two halves of scale bytes (per half: 4 x 256 bytes of activation-scale dwords, one
per row = four K steps, and 4 x 256 bytes holding each wave's weight-scale dword in every lane's slot).

Hand-back of stage memory, two barriers per K step s (blocks are counted in matrix-instruction order, 0 .. 7):
  X(s), in front of block 2: every wave has read weight blocks 0 .. 3 of step s (the last of those reads was issued in
        block 1).  Needs landed: weight rows of blocks 4 .. 7 of step s and the activation rows of step s + 1.
        Requests: weight rows of blocks 0 .. 3 of step s + 2.
  Y(s), in front of block 6: every wave has read weight blocks 4 .. 7 of step s and all activation rows of step s + 1.
        Needs landed: weight rows of blocks 0 .. 3 of step s + 1.  Requests: activation rows of step s + 3 and weight
        rows of blocks 4 .. 7 of step s + 2.
Every request has a step and a half to land.  A wave's requests return in order, so each wait names how many younger
requests may still be out; the counts are not written by hand but found by running the instruction list of whole K
loops (1, 2, 3 and 5 trips) through a model of the two counters and taking, per wait site, the strictest value seen
(separately for the last trip, on which requests past the end of K are left out).

Registers named by the loop (everything else comes in as asm operands):
  a[0:255]        accumulators: block (nb, mb) at a[32 nb + 4 mb : +3]
  v72             scale read address of the group in use (%[srd] + half), v73 the same for the weight scale
  v76             weight-scale dword in use, v77 next group's
  v78 .. v85      activation-scale dwords in use (one per 16-row block), v86 .. v93 next group's
  v94 .. v125     ring of four weight fragments
  v126 .. v189    activation fragments of even steps, v190 .. v253 of odd steps
  s[40:41] activation source of the next request, s[42:43] / s[56:57] weight source (blocks 0..3 / 4..7), s[44:45]
  activation scales, s[46:47] weight scales, s48 LDS base of the wave's copies, s49 trips left, s50 = 1 on the last
  trip, s54 / s55 scale half written / read.
At the end the accumulators of the wave's first 64 rows are moved to v[128:255] (block nb at v[128 + 16 nb : +15]) for
the C++ epilogue; gemm_quad_tail_loop.inc moves the other 64 rows the same way.
"""
import os

A_BYTES = B_BYTES = 256 * 128
B_LDS = 2 * A_BYTES
S_LDS = 2 * (A_BYTES + B_BYTES)
S_HALF = 2048
RING, AF = 94, (126, 190)
SAN, SC, WS, WSN, SRD, WSRD = 78, 86, 76, 77, 72, 73
B1_COPIES, B2_COPIES = (0, 1, 4, 5), (2, 3, 6, 7)
# Weight fragments are read D blocks ahead of their matrix instructions, and behind every BURST-th matrix instruction come
# BURST memory operations.  Measured on the 2048 x 8192 problem (one tile per CU, ns per K step): D = 2 1235, D = 3 1234;
# BURST = 1 1249, 2 1273, 4 1314, 8 1384 -- the matrix pipe does not queue instructions deep enough to cover a run of
# memory operations, and the LDS latency is covered at D = 2 already.
D, BURST = 2, 1


def vr(base, n):
    return f"v[{base}:{base + n - 1}]"


class Prog:
    """Instruction list with symbolic waits.  Items: ("i", text) plain instruction; ("lds", text, tag) LDS read;
    ("vm", text, tag, cond) copy request, cond = steps ahead it fills (left out when that step is past the end of K);
    ("wl", site, tag) wait until the LDS reads tagged tag have returned; ("wv", site, tags, lds0) wait until the
    requests tagged tags have landed (and, with lds0, every LDS read)."""

    def __init__(self):
        self.items = []

    def i(self, text):
        self.items.append(("i", text))

    def lds(self, text, tag):
        self.items.append(("lds", text, tag))

    def vm(self, lines, tag, ahead):
        self.items.append(("vm", lines, tag, ahead))

    def wl(self, site, tag):
        self.items.append(("wl", site, tag))

    def wv(self, site, tags, lds0=True):
        self.items.append(("wv", site, tags, lds0))


def copy(p, kind, i, stage, tag, ahead):
    """One 1 KB request of this wave: activation copy i (kind "a") or weight copy i into stage `stage`."""
    if kind == "a":
        p.vm([f"s_add_u32 m0, s48, {stage * A_BYTES + i * 4096}", "s_nop 0", f"global_load_lds_dwordx4 %[aoff{i}], s[40:41]"], tag, ahead)
    else:
        base = "s[42:43]" if i in B1_COPIES else "s[56:57]"
        p.vm([f"s_add_u32 m0, s48, {B_LDS + stage * B_BYTES + i * 4096}", "s_nop 0", f"global_load_lds_dwordx4 %[boff{i}], {base}"], tag, ahead)


def advance(p, lo):
    p.i(f"s_add_u32 s{lo}, s{lo}, 128")
    p.i(f"s_addc_u32 s{lo + 1}, s{lo + 1}, 0")


def scale_copies(p, group_tag, ahead):
    """The wave's two scale requests of a group of four K steps into the half s54 points at."""
    p.vm(["s_add_u32 m0, s52, s54", "s_nop 0", "global_load_lds_dword %[soff], s[44:45]"], group_tag, ahead)
    p.vm(["s_add_u32 m0, s52, s54", "s_add_u32 m0, m0, 1024", "global_load_lds_dword %[zero], s[46:47]"], group_tag, ahead)
    p.i("s_add_u32 s44, s44, 4")
    p.i("s_addc_u32 s45, s45, 0")
    p.i("s_add_u32 s46, s46, 4")
    p.i("s_addc_u32 s47, s47, 0")


def read_b(p, slot, stage, nb, tag):
    for h, addr in enumerate(("%[brd0]", "%[brd1]")):
        p.lds(f"ds_read_b128 {vr(RING + 8 * slot + 4 * h, 4)}, {addr} offset:{stage * B_BYTES + nb * 2048}", tag)


def read_a(p, buf, stage, mb, tag):
    for h, addr in enumerate(("%[ard0]", "%[ard1]")):
        p.lds(f"ds_read_b128 {vr(AF[buf] + 8 * mb + 4 * h, 4)}, {addr} offset:{stage * A_BYTES + mb * 2048}", tag)


def read_scales(p, tag):
    for mb in range(8):
        p.lds(f"ds_read_b32 v{SC + mb}, v{SRD} offset:{mb * 64}", tag)
    p.lds(f"ds_read_b32 v{WSN}, v{WSRD}", tag)


def mfma(p, nb, mb, c):
    acc = f"a[{32 * nb + 4 * mb}:{32 * nb + 4 * mb + 3}]"
    p.i(f"v_mfma_scale_f32_16x16x128_f8f6f4 {acc}, {vr(RING + 8 * (nb & 3), 8)}, {vr(AF[c & 1] + 8 * mb, 8)}, {acc}, v{WS}, v{SAN + mb} "
        f"op_sel:[{c & 1},{c & 1},0] op_sel_hi:[{c >> 1},{c >> 1},0]")


def prologue():
    p = Prog()
    p.i("s_mov_b64 s[40:41], %[abase]")
    p.i("s_mov_b64 s[42:43], %[bbase]")
    p.i("s_mov_b64 s[56:57], %[bbase]")
    p.i("s_mov_b64 s[44:45], %[sbase]")
    p.i("s_mov_b64 s[46:47], %[bsptr]")
    p.i("s_mov_b32 s48, %[m0base]")
    p.i("s_mov_b32 s52, %[s0base]")
    p.i("s_mov_b32 s49, %[trips]")
    p.i("s_mov_b32 s54, 0")
    p.i("s_mov_b32 s55, 0")
    p.i(f"v_mov_b32 v{SRD}, %[srd]")
    p.i(f"v_mov_b32 v{WSRD}, %[wsrd]")
    for r in range(256):
        p.i(f"v_accvgpr_write_b32 a{r}, 0")
    scale_copies(p, ("S", 0), None)
    for st in (0, 1):
        for i in range(8):
            copy(p, "a", i, st, ("A", st), None)
        advance(p, 40)
        for i in B1_COPIES:
            copy(p, "b", i, st, ("B1", st), None)
        advance(p, 42)
        if st == 0:
            for i in B2_COPIES:
                copy(p, "b", i, 0, ("B2", 0), None)
            advance(p, 56)
    p.wv("p0", [("S", 0), ("A", 0), ("B1", 0)])
    p.i("s_barrier")
    read_scales(p, ("s", 0))
    for mb in range(8):
        read_a(p, 0, 0, mb, ("a", 0, mb))
    for nb in range(D):
        read_b(p, nb, 0, nb, ("b", 0, nb))
    p.wl("p1", "all")
    p.i("s_barrier")
    # "Y(-1)": the activation rows of step 0 are in registers everywhere
    for i in range(8):
        copy(p, "a", i, 0, ("A", 2), None)
    advance(p, 40)
    for i in B2_COPIES:
        copy(p, "b", i, 1, ("B2", 1), None)
    advance(p, 56)
    return p


def trip():
    """Four K steps; step numbers in tags are relative to the first step of the trip."""
    p = Prog()
    for mb in range(8):
        p.i(f"v_mov_b32 v{SAN + mb}, v{SC + mb}")
    p.i(f"v_mov_b32 v{WS}, v{WSN}")
    p.i("s_sub_u32 s49, s49, 1")
    p.i("s_cmp_eq_u32 s49, 0")
    p.i("s_cselect_b32 s50, 1, 0")
    pieces, lq = [], []
    for c in range(4):
        st, ot = c & 1, 1 - (c & 1)
        for nb in range(8):
            if nb == 4 - D:
                assert not pieces
                need = [("B2", c), ("A", c + 1)]
                p.wv(f"x{c}", need)
                p.i("s_barrier")
                q = Prog()
                for i in B1_COPIES:
                    copy(q, "b", i, st, ("B1", c + 2), 2)
                pieces += q.items
                pieces.append(("adv", 42))
                if c == 0:
                    pieces.append(("scales",))
            if nb == 8 - D:
                assert not pieces and not lq
                p.wv(f"y{c}", [("B1", c + 1)] + ([("S", 1)] if c == 2 else []))
                p.i("s_barrier")
                q = Prog()
                for i in range(8):
                    copy(q, "a", i, ot, ("A", c + 3), 3)
                pieces += q.items
                pieces.append(("adv", 40))
                q = Prog()
                for i in B2_COPIES:
                    copy(q, "b", i, st, ("B2", c + 2), 2)
                pieces += q.items
                pieces.append(("adv", 56))
            # Behind every matrix instruction at most one memory operation (the wave is alone on its SIMD: while it waits
            # to hand an operation to a full queue it issues no matrix instruction either).  LDS reads go first -- the
            # weight fragment D blocks on, then the next step's activation fragments (from X on), then the next
            # group's scales (first blocks of the trip's last step) -- and copy requests take the free slots.
            q = Prog()
            if nb + D < 8:
                read_b(q, (nb + D) & 3, st, nb + D, ("b", c, nb + D))
            else:
                read_b(q, (nb + D) & 3, ot, nb + D - 8, ("b", c + 1, nb + D - 8))
            lq[0:0] = [[x] for x in q.items]
            if nb == 4 - D:
                q = Prog()
                for mb in range(8):
                    read_a(q, ot, ot, mb, ("a", c + 1, mb))
                lq += [[x] for x in q.items]
            if c == 3 and nb == 0:
                q = Prog()
                q.i(f"s_xor_b32 s55, s55, {S_HALF}")
                q.i(f"v_add_u32 v{SRD}, s55, %[srd]")
                q.i(f"v_add_u32 v{WSRD}, s55, %[wsrd]")
                setup = q.items
                q = Prog()
                read_scales(q, ("s", 1))
                lq += [setup + q.items[:1]] + [[x] for x in q.items[1:]]
            p.wl(f"b{c}_{nb}", ("b", c, nb))
            for mb in range(8):
                mfma(p, nb, mb, c)
                if (mb + 1) % BURST:
                    continue
                for _ in range(BURST):
                    if lq:
                        p.items += lq.pop(0)
                    elif pieces:
                        it = pieces.pop(0)
                        if it[0] == "scales":
                            p.i("s_cmp_eq_u32 s50, 1")
                            p.i("s_cbranch_scc1 Lnosc%=")
                            p.i(f"s_xor_b32 s54, s54, {S_HALF}")
                            scale_copies(p, ("S", 1), 4)
                            p.i("Lnosc%=:")
                        else:
                            assert it[0] == "vm"
                            p.items.append(it)
                    while pieces and pieces[0][0] == "adv":          # the base advance rides behind its last copy
                        advance(p, pieces.pop(0)[1])
    assert not lq and not pieces
    p.i("s_cmp_lg_u32 s50, 1")
    p.i("s_cbranch_scc1 Lloop%=")
    return p


def run(pro, body, trips):
    """Model of the two counters over a whole K loop -> {(site, last trip?): fewest younger operations seen}."""
    lds, vm, out = [], [], {}
    total = 4 * trips

    def absolute(tag, t):
        return (tag[0], tag[1] + (t if tag[0] in ("S", "s") else 4 * t)) + tuple(tag[2:])

    def exists(tag):
        return tag[1] < (trips if tag[0] == "S" else total)

    for t, prog in [(-1, pro)] + [(t, body) for t in range(trips)]:
        last = t == trips - 1
        tt = max(t, 0)
        skipping = False
        for it in prog.items:
            if it[0] == "i":
                # the scale requests of the next group are jumped over on the last trip
                if it[1].startswith("s_cbranch_scc1 Lnosc"):
                    skipping = last
                elif it[1].startswith("Lnosc"):
                    skipping = False
                continue
            if skipping:
                continue
            if it[0] == "lds":
                lds.append(absolute(it[2], tt))
            elif it[0] == "vm":
                tag = absolute(it[2], tt)
                if it[3] is None or exists(tag):
                    vm.append(tag)
            elif it[0] == "wl":
                if it[2] == "all":
                    n = 0
                else:
                    tag = absolute(it[2], tt)
                    idx = [i for i, x in enumerate(lds) if x == tag]
                    n = len(lds) - 1 - max(idx) if idx else len(lds)          # returned already: nothing to wait for
                key = (it[1], last)
                out[key] = min(out.get(key, 99), n)
                del lds[:len(lds) - n]
            elif it[0] == "wv":
                tags = [absolute(x, tt) for x in it[2]]
                idx = [i for i, x in enumerate(vm) if x in tags]
                for x in tags:
                    assert not exists(x) or x in vm or x in landed_tags, (it, x)        # never waits for a request not made
                n = len(vm) - 1 - max(idx) if idx else len(vm)
                key = (it[1], last)
                out[key] = min(out.get(key, 99), n)
                landed_tags.update(vm[:len(vm) - n])
                del vm[:len(vm) - n]
                if it[3]:
                    lds.clear()
    return out


landed_tags = set()


def render(prog, counts, lines, suffix=""):
    for it in prog.items:
        if it[0] == "i":
            lines.append(it[1])
        elif it[0] == "lds":
            lines.append(it[1])
        elif it[0] == "vm":
            if it[3] is not None and it[3] > 0 and it[2][0] != "S":
                # left out on the last trip when the step it fills lies past the end of K
                cstep = it[2][1]                    # step (relative to the trip) that the request fills
                if cstep >= 4:
                    tag = f"{it[2][0]}{cstep}_{len(lines)}"
                    lines.append("s_cmp_eq_u32 s50, 1")
                    lines.append(f"s_cbranch_scc1 Lnoc{tag}%=")
                    lines.extend(it[1])
                    lines.append(f"Lnoc{tag}%=:")
                    continue
            lines.extend(it[1])
        elif it[0] == "wl":
            n = min(counts.get((it[1], False), 99), counts.get((it[1], True), 99))
            lines.append(f"s_waitcnt lgkmcnt({min(n, 15)})")
        elif it[0] == "wv":
            steady, last = counts.get((it[1], False)), counts.get((it[1], True))
            extra = " lgkmcnt(0)" if it[3] else ""
            if steady is None or last is None or steady == last:
                n = steady if last is None else last if steady is None else steady
                lines.append(f"s_waitcnt vmcnt({min(n, 63)}){extra}")
            else:
                lines.append("s_cmp_eq_u32 s50, 1")
                lines.append(f"s_cbranch_scc1 Lwl{it[1]}%=")
                lines.append(f"s_waitcnt vmcnt({min(steady, 63)}){extra}")
                lines.append(f"s_branch Lwj{it[1]}%=")
                lines.append(f"Lwl{it[1]}%=:")
                lines.append(f"s_waitcnt vmcnt({min(last, 63)}){extra}")
                lines.append(f"Lwj{it[1]}%=:")


def wait_counts():
    """Strictest count per wait site over whole loops of 1, 2, 3 and 5 trips."""
    pro, body = prologue(), trip()
    counts = {}
    for trips in (1, 2, 3, 5):
        landed_tags.clear()
        for key, n in run(pro, body, trips).items():
            counts[key] = min(counts.get(key, 99), n)
    return pro, body, counts


def generate():
    pro, body, counts = wait_counts()
    lines = []
    render(pro, counts, lines)
    lines.append("Lloop%=:")
    render(body, counts, lines)
    lines.append("s_waitcnt vmcnt(0) lgkmcnt(0)")
    for _ in range(3):
        lines.append("s_nop 15")                  # the last matrix instructions have written the accumulators
    tail = []
    for half, dst in ((0, lines), (1, tail)):
        for nb in range(8):
            for mb in range(4):
                for r in range(4):
                    dst.append(f"v_accvgpr_read_b32 v{128 + 16 * nb + 4 * mb + r}, a{32 * nb + 4 * (4 * half + mb) + r}")
    return lines, tail


def write(path, lines):
    text = "// generated by gen_gemm_quad_loop.py -- do not edit\n" + "".join(f'"{l}\\n"\n' for l in lines)
    if os.path.exists(path) and open(path).read() == text:
        return
    with open(path, "w") as f:
        f.write(text)
    print("regenerated", os.path.basename(path))


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    lines, tail = generate()
    write(os.path.join(here, "gemm_quad_hw_loop.inc"), lines)
    write(os.path.join(here, "gemm_quad_tail_loop.inc"), tail)


if __name__ == "__main__":
    main()
