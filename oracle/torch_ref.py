"""Eager-PyTorch CPU oracle for the low-precision weight / GEMM path.

TEST INFRASTRUCTURE ONLY.  This module restates, op for op, the arithmetic the
reference performs with eager torch ops, so that it (a) serves as the checker
in parity tests and (b) stands in for "the reference's PyTorch CPU path" in the
benchmark's cpu-baseline leg.  The product package never imports it.

Each function names the reference lines it follows.  What pins each one
independently of its own formula is listed in oracle/lowp_oracle.c's header;
the tests additionally require this module and the scalar C oracle -- two
independent restatements -- to agree byte for byte.
"""
from __future__ import annotations

import torch

E4M3_MAX = 448.0
_E4M3 = torch.float8_e4m3fn
_E8M0 = torch.float8_e8m0fnu

# e2m1 code point -> value; index 8 differs between the two reference tables.
_MAG = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)
LUT_NEG_ZERO = torch.tensor(_MAG + tuple(-m for m in _MAG), dtype=torch.float32)  # eager_quant_kernels.py:56-58
LUT_POS_ZERO = LUT_NEG_ZERO.clone()                                                # convert_deepseek_v4_fp4_to_bf16.py:15-18
LUT_POS_ZERO[8] = 0.0


def _tiles(v: torch.Tensor, bm: int, bn: int) -> torch.Tensor:
    """[..., M, N] -> [..., M/bm, bm, N/bn, bn] view."""
    *lead, m, n = v.shape
    return v.reshape(*lead, m // bm, bm, n // bn, bn)


def _tile_amax(t: torch.Tensor) -> torch.Tensor:
    return t.abs().amax(dim=(-3, -1))


def _bcast(s: torch.Tensor) -> torch.Tensor:
    return s.unsqueeze(-1).unsqueeze(-3)


def _to_e4m3_clamped(t: torch.Tensor) -> torch.Tensor:
    return t.clamp(min=-E4M3_MAX, max=E4M3_MAX).to(_E4M3)


# --------------------------------------------------------------------- a1

def quant_fp8_e4m3_scale_e8m0(value: torch.Tensor, block_size=(128, 128)):
    """gpatch_v4/kernel/quantize/eager_quant_kernels.py:132-181."""
    m, n = value.shape[-2:]
    bm, bn = block_size
    assert m % bm == 0 and n % bn == 0, f"value shape ({m}, {n}) not divisible by block ({bm}, {bn})"
    assert not torch.isnan(value).any(), "quant_fp8_e4m3_scale_e8m0: input contains NaN"
    t = _tiles(value.float(), bm, bn)
    amax = _tile_amax(t)
    r = amax.clamp(min=torch.finfo(torch.float32).tiny) / E4M3_MAX
    s = torch.pow(2.0, torch.ceil(torch.log2(r)))
    s = torch.where(amax > 0, s, torch.ones_like(s))
    q = _to_e4m3_clamped(t / _bcast(s)).reshape(value.shape).contiguous()
    return q, s.to(_E8M0)


def quant_fp4_e2m1_scale_e8m0_packed(value: torch.Tensor, block_size=(1, 32)):
    """gpatch_v4/kernel/quantize/eager_quant_kernels.py:63-129: packed e2m1 codes (int8, low nibble = even
    column) + e8m0 block scales; ties between two code points go to the smaller magnitude (bucketize)."""
    m, n = value.shape[-2:]
    bm, bn = block_size
    assert m % bm == 0 and n % bn == 0, f"value shape ({m}, {n}) not divisible by block ({bm}, {bn})"
    assert n % 2 == 0, f"FP4 packing requires N (={n}) to be even (two nibbles per byte)"
    assert not torch.isnan(value).any(), "quant_fp4_e2m1_scale_e8m0_packed: input contains NaN"
    lead = value.shape[:-2]
    t = _tiles(value.float(), bm, bn)
    amax = _tile_amax(t)
    r = amax.clamp(min=torch.finfo(torch.float32).tiny) / 6.0
    s = torch.pow(2.0, torch.ceil(torch.log2(r)))
    s = torch.where(amax > 0, s, torch.ones_like(s))
    y = t / _bcast(s)
    pos = torch.tensor(_MAG, dtype=torch.float32)
    mid = (pos[1:] + pos[:-1]) / 2.0
    idx = torch.bucketize(y.abs().contiguous(), mid)
    code = (idx + torch.signbit(y).to(torch.int64) * 8).to(torch.uint8).reshape(*lead, m, n)
    pair = code.reshape(*lead, m, n // 2, 2)
    packed = (pair[..., 0] | (pair[..., 1] << 4)).view(torch.int8).contiguous()
    return packed, s.to(_E8M0)


def sgl_expert_to_official(weight: torch.Tensor, scale: torch.Tensor):
    """tools/dsv4_quant_and_dequant/kernels.py:136-140: FP8 expert (fp32 128x128 scales) -> packed FP4 + e8m0 1x32."""
    full = dequant_fp4_e2m1_fp8_scale_e8m0_packed(weight, scale).float()
    return quant_fp4_e2m1_scale_e8m0_packed(full, (1, 32))


# --------------------------------------------------------------------- fused QAT kernels (bit-defined scales)

def _log2_ceil_bits(x: torch.Tensor) -> torch.Tensor:
    """gpatch_v4/kernel/quantize/fused_quant_kernels.py:32-38 / qat.py:98-103: ceil(log2 x) from the fp32 bits,
    literally (exponent field - 127, + 1 when any mantissa bit is set)."""
    b = x.contiguous().view(torch.int32)
    return ((b >> 23) & 0xFF) - 127 + ((b & 0x7FFFFF) != 0).to(torch.int32)


def _pow2_bits(e: torch.Tensor) -> torch.Tensor:
    """fused_quant_kernels.py:41-44: 2^e built as fp32 bits, literally."""
    return ((e + 127) << 23).to(torch.int32).view(torch.float32)


def fp_qat_128x128(weight: torch.Tensor) -> torch.Tensor:
    """fused_quant_kernels.py:277-403: bf16 [M, N] -> e4m3 quantise / dequantise with one power-of-two scale per
    128 x 128 tile, s = 2^ceil(log2(max(amax, 1e-30) / 448)) (1 for a zero tile), back to bf16."""
    assert weight.dtype == torch.bfloat16 and weight.ndim == 2
    t = _tiles(weight.float(), 128, 128)
    amax = _tile_amax(t)
    s = _pow2_bits(_log2_ceil_bits(amax.clamp(min=1.0e-30) / E4M3_MAX))
    s = torch.where(amax > 0, s, torch.ones_like(s))
    q = (t / _bcast(s)).clamp(-E4M3_MAX, E4M3_MAX).to(_E4M3)
    return (q.float() * _bcast(s)).to(torch.bfloat16).reshape(weight.shape)


def fp4_qat_then_to_fp8(weight: torch.Tensor):
    """fused_quant_kernels.py:102-274: fp32 [M, N] -> e2m1 with a 1 x 32 scale max(2^ceil(log2(amax/6)), 2^-126)
    (1 for a zero group), value half way between two code points to the smaller magnitude, -0.0 kept; then
    rebased to e4m3 with one e8m0 scale max(largest group scale / 64, 2^-126) per 128 x 128 tile."""
    assert weight.dtype == torch.float32 and weight.ndim == 2
    m, n = weight.shape
    g = weight.reshape(m, n // 32, 32)
    amax = g.abs().amax(dim=-1)
    sg = torch.maximum(_pow2_bits(_log2_ceil_bits(amax / 6.0)), torch.tensor(2.0 ** -126))
    sg = torch.where(amax > 0, sg, torch.ones_like(sg))
    y = (g / sg.unsqueeze(-1)).clamp(-6.0, 6.0)
    pos = torch.tensor(_MAG, dtype=torch.float32)
    idx = torch.bucketize(y.abs().contiguous(), (pos[1:] + pos[:-1]) / 2.0)
    q4 = torch.where(torch.signbit(y), -pos[idx], pos[idx])                  # -0.0 survives
    st = sg.reshape(m // 128, 128, n // 128, 4)
    outer = (st.amax(dim=(1, 3)) / 64.0).clamp(min=2.0 ** -126)              # [M/128, N/128]
    off = sg.reshape(m // 128, 128, n // 128, 4) / outer[:, None, :, None]
    q8 = (q4.reshape(m // 128, 128, n // 128, 4, 32) * off.unsqueeze(-1)).reshape(m, n).to(_E4M3)
    return q8, outer.to(_E8M0)


def act_quant(x: torch.Tensor, block_size: int = 128, scale_fmt=None):
    """gpatch_v4/kernel/quantize/qat.py:116-223 (inplace=False): 1 x block_size groups along the last dim,
    s = max(amax, 1e-4) * fl32(1/448), rounded up to a power of two when scale_fmt is set;
    y = e4m3(clamp(x / s)); returns (y, s fp32 [..., N / block_size])."""
    n = x.size(-1)
    assert n % block_size == 0
    g = x.float().reshape(-1, n // block_size, block_size)
    amax = g.abs().amax(dim=-1).clamp(min=1e-4)
    s = amax * torch.tensor(1 / 448.0, dtype=torch.float32)
    if scale_fmt is not None:
        s = _pow2_bits(_log2_ceil_bits(s))
    y = (g / s.unsqueeze(-1)).clamp(-E4M3_MAX, E4M3_MAX).to(_E4M3).reshape(x.shape)
    return y, s.reshape(*x.shape[:-1], n // block_size)


def act_quant_inplace(x: torch.Tensor, block_size: int = 128, scale_fmt=None) -> torch.Tensor:
    """gpatch_v4/kernel/quantize/qat.py:116-223 with inplace=True: the kernel's output type is then the input type
    (:131), so the quotient is cast to bf16, not to e4m3 (:163-175): bf16(fp32(bf16(clamp(x / s))) * s)."""
    assert x.dtype == torch.bfloat16
    n = x.size(-1)
    g = x.float().reshape(-1, n // block_size, block_size)
    s = g.abs().amax(dim=-1).clamp(min=1e-4) * torch.tensor(1 / 448.0, dtype=torch.float32)
    if scale_fmt is not None:
        s = _pow2_bits(_log2_ceil_bits(s))
    s = s.unsqueeze(-1)
    y = (g / s).clamp(-E4M3_MAX, E4M3_MAX).to(torch.bfloat16)
    return (y.float() * s).to(torch.bfloat16).reshape(x.shape)


def fp8_simulate(x: torch.Tensor, block_size: int) -> torch.Tensor:
    """qat.py:286-301: act_quant(x, block_size, "ue8m0") then tile_kernels' per_token_cast_back, which is
    fp32(y) * s cast to the output type (bf16)."""
    assert x.dtype == torch.bfloat16
    y, s = act_quant(x, block_size, "ue8m0")
    n = x.size(-1)
    out = y.float().reshape(-1, n // block_size, block_size) * s.reshape(-1, n // block_size, 1)
    return out.to(torch.bfloat16).reshape(x.shape)


def fp4_simulate(x: torch.Tensor, block_size: int = 32) -> torch.Tensor:
    """qat.py:226-279, 350-366: bf16 -> e2m1 quantise / dequantise per 1 x 32 group with
    s = 2^ceil(log2(max(amax, 6 * 2^-126) * fl32(1/6))) taken from the bits of the product; a quotient half way
    between two code points goes to the smaller magnitude (fused_quant_kernels.py:65-99); -0.0 is kept."""
    assert x.dtype == torch.bfloat16 and block_size == 32
    n = x.size(-1)
    g = x.float().reshape(-1, n // 32, 32)
    amax = g.abs().amax(dim=-1).clamp(min=6.0 * 2.0 ** -126)
    s = _pow2_bits(_log2_ceil_bits(amax * torch.tensor(1.0 / 6.0, dtype=torch.float32))).unsqueeze(-1)
    y = (g / s).clamp(-6.0, 6.0)
    pos = torch.tensor(_MAG, dtype=torch.float32)
    idx = torch.bucketize(y.abs().contiguous(), (pos[1:] + pos[:-1]) / 2.0)
    q4 = torch.where(torch.signbit(y), -pos[idx], pos[idx])
    return (q4 * s).to(torch.bfloat16).reshape(x.shape)


# --------------------------------------------------------------------- a2

def quantize_fp8_blockwise(weight: torch.Tensor, block_size, *, device=None, scale_dtype=torch.bfloat16):
    """tools/convert_fp8/qwen3_5/qwen3_mtp_fp8_postprocess.py:102-151 (multiply form)."""
    if weight.ndim != 2:
        raise ValueError(f"Expected a 2D weight, got shape={tuple(weight.shape)}")
    bm, bn = block_size
    rows, cols = weight.shape
    if rows % bm or cols % bn:
        raise ValueError(f"Matrix dimensions ({rows}, {cols}) must be divisible by block sizes ({bm}, {bn})")
    t = _tiles(weight.to(dtype=torch.float32), bm, bn)
    amax = t.abs().amax(dim=(1, 3))
    one = torch.ones_like(amax)
    f = E4M3_MAX / torch.where(amax > 0, amax, one)
    f = torch.where(amax > 0, f, one)
    q = _to_e4m3_clamped(t * f[:, None, :, None]).reshape(rows, cols)
    return q, (1.0 / f).to(scale_dtype)


def per_block_cast_to_fp8(x: torch.Tensor):
    """SGLang / DeepGEMM per_block_cast_to_fp8 as published (the dense quantiser the weight-update path imports,
    gpatch_v4/generation_backend/sglang_model_specific/sglang_weight_update_dsv4.py:205-223,309-310; the library
    is not in the reference tree, so this restatement is not pinned by any fixture): 128 x 128 blocks, ragged edge
    zero-padded, amax clamped at 1e-4, x * (448 / amax) -> e4m3fn, scale amax / 448 in fp32."""
    assert x.dim() == 2
    m, n = x.shape
    mp, np_ = -(-m // 128) * 128, -(-n // 128) * 128
    pad = torch.zeros(mp, np_, dtype=x.dtype)
    pad[:m, :n] = x
    v = pad.view(-1, 128, np_ // 128, 128)
    amax = v.abs().float().amax(dim=(1, 3), keepdim=True).clamp(1e-4)
    q = (v * (448.0 / amax)).to(_E4M3)
    return q.view(mp, np_)[:m, :n].contiguous(), (amax / 448.0).view(v.size(0), v.size(2))


# ---------------------------------------------------------------- a3 / a4

def quant_block_fp32_scale(x: torch.Tensor, block_size, *, amax_floor=1e-12, zero_scale_to_one=False):
    """Divide form with an fp32 scale = amax/448.

    amax_floor=1e-12: tests/test_gfused/test_te_gemm_fp8.py:82-101,
    tests/test_gfused/test_deepseek_tilekernels_quant.py:22-58.
    amax_floor=None, zero_scale_to_one=True:
    tests/test_gpatch_v4/test_deep_gemm_grouped_gemm_fp8.py:29-72.
    Works for 1 x 128 activation groups and 128 x 128 weight tiles alike.
    """
    bm, bn = block_size
    t = _tiles(x.float(), bm, bn)
    amax = _tile_amax(t)
    if amax_floor is not None:
        amax = amax.clamp(min=amax_floor)
    s = amax / E4M3_MAX
    if zero_scale_to_one:
        s = torch.where(s == 0, torch.ones_like(s), s)
    q = _to_e4m3_clamped(t / _bcast(s)).reshape(x.shape).contiguous()
    return q, s.to(torch.float32)


def quant_block_pow2_scale(x: torch.Tensor, block_size, *, amax_floor=1e-12):
    """round_sf=True branch of tests/test_gfused/test_deepseek_tilekernels_quant.py:22-58."""
    bm, bn = block_size
    t = _tiles(x.float(), bm, bn)
    amax = _tile_amax(t).clamp(min=amax_floor)
    s = torch.pow(2.0, torch.ceil(torch.log2(amax / E4M3_MAX)))
    q = _to_e4m3_clamped(t / _bcast(s)).reshape(x.shape).contiguous()
    return q, s


# ---------------------------------------------------------------- a5 / a6

def unpack_fp4(packed: torch.Tensor, lut: torch.Tensor) -> torch.Tensor:
    """Low nibble -> even column, high nibble -> odd column
    (eager_quant_kernels.py:190-197)."""
    b = packed.contiguous().view(torch.uint8)
    lo = (b & 0xF).long()
    hi = ((b >> 4) & 0xF).long()
    return torch.stack((lut[lo], lut[hi]), dim=-1).reshape(*packed.shape[:-1], 2 * packed.shape[-1])


def dequant_fp4_e2m1_fp8_scale_e8m0_packed(quantized: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """eager_quant_kernels.py:200-233: block = shape ratio, fp32 product, result in
    scales.dtype when that is a float of >= 2 bytes, else bf16."""
    fp4x2 = getattr(torch, "float4_e2m1fn_x2", None)
    if quantized.dtype == torch.int8 or (fp4x2 is not None and quantized.dtype == fp4x2):
        qf = unpack_fp4(quantized, LUT_NEG_ZERO)
    else:
        qf = quantized.to(torch.float32)
    rows, cols = qf.shape[-2:]
    sr, sc = scales.shape[-2:]
    if rows % sr or cols % sc:
        raise ValueError(f"Weight shape ({rows}, {cols}) not divisible by scale grid ({sr}, {sc}).")
    out_dtype = scales.dtype if scales.dtype.is_floating_point and scales.element_size() >= 2 else torch.bfloat16
    t = qf.reshape(-1, sr, rows // sr, sc, cols // sc)
    s = scales.to(torch.float32).reshape(-1, sr, sc)[:, :, None, :, None]
    return (t * s).to(out_dtype).reshape(qf.shape)


def cast_e4m3fn_to_bf16(x: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """tools/convert_deepseek_v4_fp4_to_bf16.py:51-63."""
    assert x.dtype == _E4M3 and x.ndim == 2
    o, i = x.shape
    assert o % 128 == 0 and i % 128 == 0
    assert tuple(scale.shape) == (o // 128, i // 128)
    s = scale.float().repeat_interleave(128, 0).repeat_interleave(128, 1)
    return (x.float() * s).bfloat16()


# --------------------------------------------------------------------- a7

def cast_e2m1fn_to_bf16(x: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """tools/convert_deepseek_v4_fp4_to_bf16.py:24-46."""
    assert x.dtype == torch.int8 and x.ndim == 2
    o, half = x.shape
    i = half * 2
    assert i % 32 == 0
    assert scale.size(0) == o and scale.size(1) == i // 32
    v = unpack_fp4(x, LUT_POS_ZERO)
    return (v * scale.float().repeat_interleave(32, dim=-1)).bfloat16()


# --------------------------------------------------------------------- a8

def cast_e2m1fn_to_e4m3fn(x: torch.Tensor, scale: torch.Tensor):
    """tools/dsv4_quant_and_dequant/kernels.py:91-126."""
    assert x.dtype == torch.int8 and x.ndim == 2
    o, half = x.shape
    i = half * 2
    assert i % 128 == 0 and o % 128 == 0
    assert scale.size(0) == o and scale.size(1) == i // 32
    v = unpack_fp4(x, LUT_POS_ZERO)                                    # [o, i]
    bo, bi = o // 128, i // 128
    vt = v.view(bo, 128, bi, 128).transpose(1, 2)                      # [bo, bi, 128, 128]
    st = scale.float().view(bo, 128, bi, 4).transpose(1, 2).flatten(2)  # [bo, bi, 512]
    outer = st.amax(dim=-1, keepdim=True) / 64.0
    off = (st / outer).unflatten(-1, (128, 4)).repeat_interleave(32, dim=-1)
    y = (vt * off).transpose(1, 2).reshape(o, i)
    return y.to(_E4M3), outer.squeeze(-1).to(_E8M0)


def official_expert_to_sgl(weight: torch.Tensor, scale: torch.Tensor):
    """tools/dsv4_quant_and_dequant/kernels.py:129-133."""
    q, s = cast_e2m1fn_to_e4m3fn(weight, scale)
    return q, s.float().contiguous()


# --------------------------------------------------------------------- a9

def fp4_to_fp8_amax(x: torch.Tensor, scale: torch.Tensor, *, amax_floor=1e-12, zero_scale_to_one=False):
    """FP4 -> bf16 -> e4m3fn with a 128 x 128 fp32 scale = amax/448: the two-step
    composition cast_e2m1fn_to_bf16 followed by the divide-form block quantiser."""
    w = cast_e2m1fn_to_bf16(x, scale)
    return quant_block_fp32_scale(w, (128, 128), amax_floor=amax_floor, zero_scale_to_one=zero_scale_to_one)


# -------------------------------------------------------------- a10 - a12

def dequant_act_f32(q: torch.Tensor, s: torch.Tensor) -> torch.Tensor:
    m, k = q.shape
    return (q.float().reshape(m, k // 128, 128) * s.float().unsqueeze(-1)).reshape(m, k)


def dequant_weight_f32(q: torch.Tensor, s: torch.Tensor) -> torch.Tensor:
    *lead, n, k = q.shape
    t = q.float().reshape(*lead, n // 128, 128, k // 128, 128)
    return (t * s.float().unsqueeze(-1).unsqueeze(-3)).reshape(q.shape)


def gemm_fp8_block_scaling_ref(Aq, As, Bq, Bs) -> torch.Tensor:
    """fp32 dequant then fp32 matmul: the numeric reference of gfused/mygemm_fp8.py:44-97
    (tests/test_gfused/test_my_gemm_fp8.py:176-186 does the same in bf16)."""
    return dequant_act_f32(Aq, As) @ dequant_weight_f32(Bq, Bs).T


def grouped_gemm_fp8_ref(xq, xs, wq, ws, m_splits) -> torch.Tensor:
    """tests/test_gpatch_v4/test_deep_gemm_grouped_gemm_fp8.py:75-89 with rows given
    as consecutive per-expert counts."""
    x = dequant_act_f32(xq, xs)
    w = dequant_weight_f32(wq, ws)
    out = torch.zeros(x.shape[0], w.shape[1], dtype=torch.float32)
    r = 0
    for e, cnt in enumerate(m_splits):
        if cnt:
            out[r:r + cnt] = x[r:r + cnt] @ w[e].T
        r += cnt
    return out


def quant_colwise_t(x: torch.Tensor, m_splits):
    """Column-wise operands of the grouped linear's weight-gradient GEMM
    (gpatch_v4/models/deepseek_v4/fp8.py:292-294,325-341; Float8BlockScaling with power-of-two scales): per expert,
    blocks of 128 rows x 1 column restarting at the expert's first row, scale 2^ceil(log2(amax / 448)) (1 for a
    zero block, as quant_fp8_e4m3_scale_e8m0), output transposed and zero-padded to whole blocks.
    Returns per expert (codes e4m3fn [C, P_e], scales e8m0 [C, P_e / 128])."""
    out, r = [], 0
    for m in m_splits:
        p = (m + 127) // 128 * 128
        xe = torch.zeros(p, x.shape[1], dtype=torch.float32)
        xe[:m] = x[r:r + m].float()
        r += m
        if p == 0:
            out.append((torch.zeros(x.shape[1], 0, dtype=_E4M3), torch.zeros(x.shape[1], 0, dtype=_E8M0)))
            continue
        q, s = quant_fp8_e4m3_scale_e8m0(xe.t().contiguous(), (1, 128))
        out.append((q, s))
    return out


def gemm_rowscale_ref(aq, a_s, bq, b_s) -> torch.Tensor:
    """fp32 reference of the GEMM with a scale per row and 128 of K on both operands."""
    a = dequant_act_f32(aq, a_s.float())
    b = dequant_act_f32(bq, b_s.float())
    return a.double() @ b.double().T

