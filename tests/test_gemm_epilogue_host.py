"""Index arithmetic of the GEMM's staged bf16 epilogue (StagedEpilogue in csrc/gemm_fp8_big.hip), restated on the
host: what a wave writes into its staging region per accumulator block and what it reads back per pass must cover
every element of the 64-row wave tile exactly once, at aligned offsets inside the region, for the four wave-tile
widths in use.  A mistake here would show on the GPU as wrong results at best and as an out-of-range access at
worst, so it is checked where a mistake costs nothing."""
import pytest


def layout(cols):
    pitch = cols * 2 + 16
    chunks = cols // 8
    return {"pitch": pitch, "wave_bytes": 64 * pitch, "chunks": chunks, "passes": chunks}


@pytest.mark.parametrize(("cols", "waves", "lds_bytes"), [(128, 8, 2 * (256 + 256) * 128 + 2 * 256 * 16),      # 256 x 256 tile
                                                          (96, 8, 2 * (256 + 192) * 128 + 2 * 256 * 16),       # 256 x 192 tile
                                                          (144, 8, 8 * 64 * (144 * 2 + 16)),                   # 256 x 288 tile: LDS sized for it
                                                          (64, 4, 2 * (128 + 128) * 128 + 2 * 128 * 16)])      # 128 x 128 tile
def test_staged_epilogue_mapping(cols, waves, lds_bytes):
    L = layout(cols)
    assert waves * L["wave_bytes"] <= lds_bytes
    region = [None] * (L["wave_bytes"] // 2)                 # one slot per bf16
    for mb in range(4):
        for nb in range(cols // 16):
            for l16 in range(16):
                for lq in range(4):
                    off = (mb * 16 + l16) * L["pitch"] + (nb * 16 + 4 * lq) * 2
                    assert off % 8 == 0 and off + 8 <= L["wave_bytes"]
                    for r in range(4):
                        assert region[off // 2 + r] is None          # nobody else writes this slot
                        region[off // 2 + r] = (mb * 16 + l16, nb * 16 + 4 * lq + r)
    seen = set()
    for p in range(L["passes"]):
        for lane in range(64):
            row, chunk = (p * 64 + lane) // L["chunks"], (p * 64 + lane) % L["chunks"]
            off = row * L["pitch"] + chunk * 16
            assert off % 16 == 0 and off + 16 <= L["wave_bytes"] and 0 <= row < 64
            for j in range(8):
                assert region[off // 2 + j] == (row, chunk * 8 + j)
                assert (row, chunk * 8 + j) not in seen
                seen.add((row, chunk * 8 + j))
    assert len(seen) == 64 * cols


def test_staged_epilogue_bank_spread():
    """The 8-byte writes of one instruction (16 rows x 4 lanes) touch each LDS bank at most twice."""
    for cols in (144, 128, 96, 64):
        L = layout(cols)
        for nb in range(cols // 16):
            hits = {}
            for l16 in range(16):
                for lq in range(4):
                    off = l16 * L["pitch"] + (nb * 16 + 4 * lq) * 2
                    for b in ((off // 4) % 64, (off // 4 + 1) % 64):
                        hits[b] = hits.get(b, 0) + 1
            assert max(hits.values()) <= 2, (cols, nb, max(hits.values()))


@pytest.mark.parametrize(("cols", "waves", "lds_bytes"), [(128, 8, 8 * 64 * (128 * 2 + 16)), (64, 4, 2 * (128 + 128) * 128 + 2 * 128 * 16)])
def test_staged_fp8_epilogue_mapping(cols, waves, lds_bytes):
    """The e4m3 form (StagedEpilogueFp8: one byte per element, 4 bytes written per lane and block, 16-byte chunks of 16
    columns read back): every byte of the 64-row wave tile exactly once, aligned, inside the region."""
    pitch, chunks = cols + 16, cols // 16
    wave_bytes = 64 * pitch
    assert waves * wave_bytes <= lds_bytes
    region = [None] * wave_bytes
    for mb in range(4):
        for nb in range(cols // 16):
            for l16 in range(16):
                for lq in range(4):
                    off = (mb * 16 + l16) * pitch + nb * 16 + 4 * lq
                    assert off % 4 == 0 and off + 4 <= wave_bytes
                    for r in range(4):
                        assert region[off + r] is None
                        region[off + r] = (mb * 16 + l16, nb * 16 + 4 * lq + r)
    seen = set()
    for p in range(chunks):
        for lane in range(64):
            row, chunk = (p * 64 + lane) // chunks, (p * 64 + lane) % chunks
            off = row * pitch + chunk * 16
            assert off % 16 == 0 and off + 16 <= wave_bytes and 0 <= row < 64
            for j in range(16):
                assert region[off + j] == (row, chunk * 16 + j)
                seen.add((row, chunk * 16 + j))
    assert len(seen) == 64 * cols
