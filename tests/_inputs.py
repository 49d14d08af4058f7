"""Seeded synthetic inputs shared by CPU and GPU tests (shapes follow the benchmark configs)."""
import torch

E4M3_MAX = 448.0


def weight_like(rows, cols, seed, dtype=torch.bfloat16, outliers=True):
    """N(0, 0.02) with 0.1 % of entries set to +-1.0."""
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(rows, cols, generator=g) * 0.02
    if outliers:
        m = torch.rand(rows, cols, generator=g) < 1e-3
        sgn = torch.where(torch.rand(rows, cols, generator=g) < 0.5, -1.0, 1.0)
        w = torch.where(m, sgn, w)
    return w.to(dtype)


def act_like(rows, cols, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(rows, cols, generator=g).to(dtype)


def fp4_expert(rows, cols, seed, lo=117, hi=127):
    """Packed e2m1 bytes uniform in 0..255 and e8m0 scale bytes uniform in lo..hi."""
    g = torch.Generator().manual_seed(seed)
    packed = torch.randint(0, 256, (rows, cols // 2), generator=g, dtype=torch.int32).to(torch.uint8).view(torch.int8)
    sb = torch.randint(lo, hi + 1, (rows, cols // 32), generator=g, dtype=torch.int32).to(torch.uint8)
    return packed, sb.view(torch.float8_e8m0fnu)


def edge_tiles():
    """128 x (128*k) bf16-grid tensor whose tiles hit the scale-exponent boundaries, a wide
    exponent range, every e4m3 rounding midpoint, a zero tile and a single-element tile
    (cases of tests/test_gfused/test_fp_qat_128x128.py:89-185,271-275 in the reference)."""
    tiles = []
    for i, amax in enumerate((223.0, 224.0, 225.0, 446.0, 448.0, 450.0, 892.0, 896.0, 900.0)):
        t = torch.linspace(-amax / 4, amax / 4, 128).to(torch.bfloat16).float().repeat(128, 1)
        t[i, i] = -amax if i % 2 else amax
        tiles.append(t)
    pattern = torch.linspace(-0.75, 0.75, 128)
    for i, e in enumerate((-60, -30, -15, 0, 15, 30, 60)):
        amax = 448.0 * 2.0 ** e
        t = (pattern * amax).repeat(128, 1)
        t[i, 127 - i] = -amax if i % 2 else amax
        tiles.append(t)
    mids = []
    for k in range(8):
        m = 1.0625 + k * 0.125
        mids += [m - 0.0078125, m, m + 0.0078125]
    vals = torch.tensor([-448.0, -0.001953125, -0.0, 0.0, 0.001953125] + [-v for v in reversed(mids)] + mids + [448.0])
    rep = (128 * 128 + vals.numel() - 1) // vals.numel()
    tiles.append(vals.repeat(rep)[:128 * 128].reshape(128, 128))
    tiles.append(torch.zeros(128, 128))
    one = torch.zeros(128, 128)
    one[77, 5] = -3.0e-3
    tiles.append(one)
    stripe = torch.full((128, 128), 0.125)
    stripe[17 + 29 * 3, 3 * 32 + 31] = -1792.0
    tiles.append(stripe)
    return torch.cat(tiles, dim=1).to(torch.bfloat16)


def zipf_m_splits(experts=256, tokens=8192, topk=8, seed=4321, exponent=1.1):
    """Rows per expert of the grouped-GEMM benchmark problem: expert popularity ~ rank^-exponent, every token picks
    `topk` distinct experts (seeded, without replacement), rows are then sorted by expert.  Returns an int64 tensor
    [experts] summing to tokens * topk."""
    g = torch.Generator().manual_seed(seed)
    pop = torch.arange(1, experts + 1, dtype=torch.float64) ** -exponent
    choice = torch.multinomial(pop.expand(tokens, experts), topk, replacement=False, generator=g)
    return torch.bincount(choice.flatten(), minlength=experts)



def zipf_m_splits_with_idle_expert(experts=256, tokens=8192, topk=8, seed=4321, exponent=1.1):
    """The grouped-GEMM benchmark problem as it is timed and tested: the Zipf law over experts - 1 experts and one
    expert in the middle of the list that no token chose (per-expert rows then range from 0 upwards, and the kernels'
    empty-expert path is part of the measured launch).  Same total: tokens * topk rows."""
    m = zipf_m_splits(experts - 1, tokens, topk, seed, exponent)
    mid = experts // 2
    return torch.cat([m[:mid], torch.zeros(1, dtype=m.dtype), m[mid:]])
