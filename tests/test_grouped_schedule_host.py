"""The device-side tile schedule of the grouped GEMM with two tile heights (gemm_asm_grouped_mixed in
csrc/gemm_fp8_big.hip), restated on the host: from the rows per expert every workgroup derives its class, its
expert, its row tile and its column tile.  Over the grid the host launches, every tile of every expert must come up
exactly once, nothing else may come up, the grid bound must cover the schedule, and the tiles an XCD runs together
must belong to one expert or to neighbours.  A mistake here shows on the GPU as missing or doubly written output
rows, so it is checked where a mistake costs nothing.  Also the wide tile's weight-copy plan (256 x 288 loop)."""
import pytest

CHUNK, GROUP_M = 32, 8


def padded_grid(tiles_m, tiles_n):
    chunks = (tiles_m * tiles_n + CHUNK - 1) // CHUNK
    return (chunks + 7) // 8 * 8 * CHUNK


def classes(rows):
    rem = rows & 255
    return (rows >> 8) + (1 if rem > 128 else 0), (1 if 0 < rem <= 128 else 0)


def schedule(m_splits, N, small_first):
    """-> list of (class, expert, local row tile, column tile) per workgroup that gets a tile; grid size."""
    E, M_total, tiles_n = len(m_splits), sum(m_splits), N >> 8
    nb = [classes(r)[0] for r in m_splits]
    ns = [classes(r)[1] for r in m_splits]
    tot_big, tot_small = sum(nb), sum(ns)
    slots = lambda tiles: ((tiles + CHUNK - 1) // CHUNK + 7) // 8 * CHUNK
    slots_big, slots_small = slots(tot_big * tiles_n), slots(tot_small * tiles_n)
    grid = padded_grid(M_total // 256 + E, tiles_n) + 2 * 8 * CHUNK                     # what the host launches
    assert grid >= 8 * (slots_big + slots_small), "host grid bound below the device schedule"
    out = []
    for b in range(grid):
        xcd, sidx = b & 7, b >> 3
        if sidx >= slots_big + slots_small:
            continue
        if small_first > 0:
            if xcd < small_first:
                big = sidx >= slots_small
                idx = sidx - slots_small if big else sidx
            else:
                big = sidx < slots_big
                idx = sidx if big else sidx - slots_big
        else:
            ps = max(1, (slots_small + slots_big // 2) // slots_big if slots_big > 0 else 1)
            period = 1 + ps
            rounds = min(slots_big, slots_small // ps)
            if sidx < rounds * period:
                r, q = sidx % period, sidx // period
                big = r == 0
                idx = q if big else q * ps + (r - 1)
            else:
                w, left_big = sidx - rounds * period, slots_big - rounds
                big = w < left_big
                idx = rounds + w if big else rounds * ps + (w - left_big)
        lin = ((idx // CHUNK) * 8 + xcd) * CHUNK + idx % CHUNK
        cnts = nb if big else ns
        if lin >= (tot_big if big else tot_small) * tiles_n:
            continue
        gmt = lin // tiles_n
        incl, e = 0, None
        for i, c in enumerate(cnts):                       # the expert whose running count covers gmt
            if incl <= gmt < incl + c:
                e, first = i, incl
            incl += c
        assert e is not None
        in_e = lin - first * tiles_n
        per_group = GROUP_M * tiles_n
        grp, in_grp = divmod(in_e, per_group)
        gm = min(cnts[e] - grp * GROUP_M, GROUP_M)
        gn = CHUNK // gm
        nblk, in_blk = divmod(in_grp, gm * gn)
        local, tn = grp * GROUP_M + in_blk % gm, nblk * gn + in_blk // gm
        out.append(("big" if big else "small", e, local, tn, xcd, idx))
    return out, grid


CASES = {
    "zipf": None,                                           # the benchmark's rows per expert
    "ragged": [300, 0, 129, 128, 1, 255, 256, 257, 2048 + 130, 64, 0, 7146],
    "all_small": [5, 128, 77, 1],
    "all_big": [256, 512, 129, 3000],
    "one_heavy": [0, 0, 9000, 0],
    "empty": [0, 0, 0],
}


@pytest.mark.parametrize("name", list(CASES))
@pytest.mark.parametrize("small_first", [0, 4, 8])
@pytest.mark.parametrize("N", [4096, 7168, 256])
def test_every_tile_exactly_once(name, small_first, N):
    if CASES[name] is None:
        from tests._inputs import zipf_m_splits
        m_splits = zipf_m_splits().tolist()
    else:
        m_splits = CASES[name]
    got, grid = schedule(m_splits, N, small_first)
    want = set()
    for e, r in enumerate(m_splits):
        b, s = classes(r)
        for tn in range(N >> 8):
            want |= {("big", e, m, tn) for m in range(b)} | {("small", e, 0, tn) for _ in range(s)}
    tiles = [g[:4] for g in got]
    assert len(tiles) == len(set(tiles)), "a tile is handed out twice"
    assert set(tiles) == want
    # rows covered: big tiles take 256 rows each from the expert's start, the small tile what is left after them
    for e, r in enumerate(m_splits):
        b, s = classes(r)
        covered = min(r, b * 256) + (r - (r >> 8) * 256 if s else 0)
        assert covered == r, (e, r, b, s)


@pytest.mark.parametrize("workgroups", [8, 256, 304, 1 << 20])
@pytest.mark.parametrize("all_slots", [0, 8 * 32, 8 * 32 * 47, 8 * 32 * 300])
def test_slot_walk_of_the_persistent_launch(workgroups, all_slots):
    """With fewer workgroups than slots, workgroup b takes slots b, b + G, b + 2 G ... (G = workgroups rounded down to a
    multiple of 8, what the host launches), looked up 256 at a time, one slot per thread: every slot comes up exactly once,
    and always on the XCD (slot mod 8) of the workgroup that takes it, which keeps the per-XCD order of the schedule."""
    K_TABLE = 256
    G = workgroups // 8 * 8 if all_slots > workgroups else max(all_slots, 8)
    seen = []
    for b in range(min(G, all_slots)):
        first = b
        while first < all_slots:                            # one look-up batch
            for t in range(K_TABLE):
                slot = first + t * G
                if slot < all_slots:
                    assert slot % 8 == b % 8
                    seen.append(slot)
            first += K_TABLE * G
    assert sorted(seen) == list(range(all_slots))


def test_an_xcd_runs_neighbouring_tiles_together():
    """32 consecutive positions of an XCD's sequence within a class are 32 consecutive tile numbers: at most two
    experts unless experts have fewer than 16 tiles, and for an expert with at least 8 row tiles a block of 8 x 4."""
    from tests._inputs import zipf_m_splits
    got, _ = schedule(zipf_m_splits().tolist(), 4096, 4)
    by = {}
    for cls, e, m, tn, xcd, idx in got:
        by.setdefault((cls, xcd, idx // CHUNK), []).append((e, m, tn))
    for (cls, xcd, chunk), tiles in by.items():
        experts = {t[0] for t in tiles}
        assert len(experts) <= 3, (cls, xcd, chunk, experts)           # 16 column tiles per row tile: 32 numbers span <= 3 experts
        if len(experts) == 1 and cls == "big":
            ms, ns = {t[1] for t in tiles}, {t[2] for t in tiles}
            assert len(ms) * len(ns) >= len(tiles)                     # a rectangle of row x column tiles, not a line of 32


def test_wide_tile_weight_copy_plan():
    """256 x 288 loop: copy i of wave w moves the group of 8 weight rows WIDE_GROUP[i] + w (the fifth copy: waves 0..3,
    groups 16, 17, 34, 35).  The 36 groups must each be moved once; the mid-step part must be exactly the first 64
    rows of both wave columns; every group of a wave must have the wave's parity (one swizzled source offset serves all)."""
    group = (0, 18, 8, 26)
    moved, mid = [], []
    for w in range(8):
        mine = [g + w for g in group] + ([(16 if w < 2 else 32) + w] if w < 4 else [])
        assert all(g % 2 == w % 2 for g in mine)
        moved += mine
        mid += mine[:2]
    assert sorted(moved) == list(range(36))
    rows_mid = sorted(r for g in mid for r in range(8 * g, 8 * g + 8))
    assert rows_mid == list(range(0, 64)) + list(range(144, 208))


def test_weight_gradient_padding_and_launch_split():
    """Host side of the grouped weight gradient: blocks of 128 rows per expert under each padding rule (the rule the
    column-wise quantiser applies on the device), and the deal of the problems to kernels: every problem with K blocks in
    exactly one table, each table's K block counts multiples of what the launch promises, the running offsets those of
    the operands' layout, problems without rows listed apart."""
    pytest.importorskip("torch")
    from gcore_lowp import _abi as A
    from gcore_lowp.grouped_gemm_fp8 import choose_colwise_pad, padded_blocks, rowscale_launches
    rows = [0, 1, 128, 129, 256, 257, 512, 513, 1024, 1025, 7163]
    assert [padded_blocks(r, 128) for r in rows] == [0, 1, 1, 2, 2, 3, 4, 5, 8, 9, 56]
    assert [padded_blocks(r, 256) for r in rows] == [0, 2, 2, 2, 2, 4, 4, 6, 8, 10, 56]
    assert [padded_blocks(r, 512) for r in rows] == [0, 4, 4, 4, 4, 4, 4, 8, 8, 12, 56]
    assert [padded_blocks(r, A.PAD_MIXED) for r in rows] == [0, 1, 1, 2, 2, 4, 4, 8, 8, 12, 56]
    assert choose_colwise_pad(rows) == A.PAD_MIXED
    k_blocks = [4, 1, 0, 8, 3, 12, 0, 5, 2, 1, 2]
    launches, empty = rowscale_launches(k_blocks)
    assert empty == [2, 6]
    seen = {}
    for table, multiple in launches:
        assert table and multiple in (1, 2, 4)
        for e, kb, before, zero in table:
            assert e not in seen and kb == k_blocks[e] and kb % multiple == 0 and zero == 0
            assert before == sum(k_blocks[:e])
            seen[e] = multiple
        if multiple == 2:
            assert all(kb == 2 for _, kb, _, _ in table)
    assert sorted(seen) == [e for e, kb in enumerate(k_blocks) if kb]
    assert {e for e, m in seen.items() if m == 4} == {0, 3, 5}
    # the problems of one K block and the odd ones never share a table: the kernel without a K loop takes a table whose
    # largest problem has one block
    ones = [t for t, m in launches if m == 1 and all(kb == 1 for _, kb, _, _ in t)]
    assert len(ones) == 1 and {e for e, _, _, _ in ones[0]} == {1, 9}
    # a mixed padding never leaves a problem to the compiler-scheduled kernel
    launches, _ = rowscale_launches([padded_blocks(r, A.PAD_MIXED) for r in range(0, 3000, 37)])
    assert all(m in (2, 4) or all(kb == 1 for _, kb, _, _ in t) for t, m in launches)
