"""Grouped (MoE) block-scaled FP8 GEMM, MI355X drop-ins.

* m_grouped_gemm_fp8_fp8_bf16_nt_contiguous -- the DeepGEMM-style call the
  reference makes at tests/test_gpatch_v4/test_deep_gemm_grouped_gemm_fp8.py:106-109.
* MyTeGroupedLinearFp8 -- gpatch_v4/models/deepseek_v4/fp8.py:180-394, forward and backward:
  activations are quantised per 1 x 128, weights per 128 x 128 (or taken
  pre-quantised), one grouped GEMM; no per-expert row padding copies.
"""
from __future__ import annotations

import torch

from . import _abi as A
from . import ops

__all__ = ["grouped_gemm_fp8", "grouped_gemm_fp8_nn", "m_grouped_gemm_fp8_fp8_bf16_nt_contiguous", "MyTeGroupedLinearFp8",
           "quant_fp8_colwise_t", "gemm_fp8_rowscale"]



def _quant_pow2(value: torch.Tensor, block_size):
    """quant_fp8_e4m3_scale_e8m0's codes and scales without its NaN assertion, which reads a counter back from the device
    and so stalls the stream once per call: inside the grouped linear (three quantisations per step and layer) a NaN
    simply propagates into the product, as it does in the reference, whose layer quantises inside TransformerEngine
    (fp8.py:180-343) without such a check."""
    q, s, _ = ops.quant_fp8_block(value, block_size, scale_mode=A.SCALE_POW2, scale_dtype=ops.E8M0, count_nan=False)
    return q, s

def _scale_arg(s, dev):
    s = s.to(dev)
    if s.dtype == ops.E8M0:
        return s.contiguous(), A.E8M0
    return s.to(torch.float32).contiguous(), A.F32


def _check_offsets(m_offsets: torch.Tensor, E: int, dev, what: str) -> torch.Tensor:
    """The kernels read m_offsets as E + 1 int32 values in device memory: give them exactly that."""
    assert isinstance(m_offsets, torch.Tensor) and m_offsets.dim() == 1 and m_offsets.numel() == E + 1, \
        f"{what}: m_offsets must hold E + 1 = {E + 1} values"
    assert not m_offsets.dtype.is_floating_point, f"{what}: m_offsets must be an integer tensor"
    return m_offsets.to(device=dev, dtype=torch.int32).contiguous()


def grouped_gemm_fp8(xq, xs, wq, ws, m_offsets: torch.Tensor, out: torch.Tensor | None = None,
                     out_dtype=torch.bfloat16, total_rows: int | None = None, validate: bool = False) -> torch.Tensor:
    """xq [M,K] e4m3fn, xs [M,K/128], wq [E,N,K] e4m3fn, ws [E,N/128,K/128],
    m_offsets integer [E+1] (rows of expert e: m_offsets[e]..m_offsets[e+1]-1, non-decreasing from 0, last <= M).
    Rows at or beyond m_offsets[E] belong to no expert: a freshly allocated `out` has them zeroed, a caller's `out`
    keeps them.  A table that breaks the contract (does not start at 0, decreases) leaves the rows that fall outside
    every expert's range of a freshly allocated `out` undefined.  total_rows: m_offsets[E] when the caller knows it on
    the host (saves reading it back); validate: check the offsets, and total_rows against them, on the host (one device
    read-back)."""
    M, K = xq.shape
    E, N, K2 = wq.shape
    assert K == K2 and K % 128 == 0 and N % 128 == 0
    assert tuple(xs.shape) == (M, K // 128) and tuple(ws.shape) == (E, N // 128, K // 128)
    dev = xq.device
    assert dev.type == "cuda", "grouped_gemm_fp8 takes GPU tensors"
    sa, ca = _scale_arg(xs, dev)
    sb, cb = _scale_arg(ws, dev)
    if ca != cb:
        sa, sb, ca = sa.to(torch.float32), sb.to(torch.float32), A.F32
    offs = _check_offsets(m_offsets, E, dev, "grouped_gemm_fp8")
    if validate:
        o = offs.cpu()
        if int(o[0]) != 0 or bool((o[1:] < o[:-1]).any()) or int(o[-1]) > M:
            raise ValueError(f"grouped_gemm_fp8: m_offsets must start at 0, never decrease and end at or below M = {M}")
        if total_rows is not None and E > 0 and int(o[-1]) != total_rows:
            raise ValueError(f"grouped_gemm_fp8: total_rows = {total_rows} but m_offsets ends at {int(o[-1])}")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=dev)
        if total_rows is None:
            total_rows = int(offs[-1].item()) if E > 0 else 0
        if total_rows < M:
            out[total_rows:].zero_()
    assert out.is_contiguous() and tuple(out.shape) == (M, N) and out.dtype in (torch.bfloat16, torch.float32)
    with torch.cuda.device(dev):
        A.check(A.lib().lp_gemm_fp8_grouped(
            xq.contiguous().data_ptr(), sa.data_ptr(), wq.contiguous().data_ptr(), sb.data_ptr(), ca,
            offs.data_ptr(), E, M, N, K, out.data_ptr(),
            A.BF16 if out.dtype == torch.bfloat16 else A.F32, A.stream_ptr()))
    return out


def grouped_gemm_fp8_nn(xq, xs, wq, ws, m_offsets: torch.Tensor, out: torch.Tensor | None = None,
                        out_dtype=torch.bfloat16, total_rows: int | None = None) -> torch.Tensor:
    """out_e = x_e W_e on weights stored [E, K, N] (K = the contraction): the data gradient of the grouped linear on the
    layer's own [out, in] weights, general_grouped_gemm(..., layout="NN") at gpatch_v4/models/deepseek_v4/fp8.py:301-313.
    xq [M, K] e4m3fn with xs [M, K/128], wq [E, K, N] e4m3fn with ws [E, K/128, N/128], all scales e8m0.
    The kernel turns the weight operand while it reads it out of LDS; shapes it does not take (N or K not a multiple of
    512, more than 512 experts) go through a transposed copy of the weights and grouped_gemm_fp8."""
    M, K = xq.shape
    E, K2, N = wq.shape
    assert K == K2 and K % 128 == 0 and N % 128 == 0
    assert tuple(xs.shape) == (M, K // 128) and tuple(ws.shape) == (E, K // 128, N // 128)
    assert xs.dtype == ops.E8M0 and ws.dtype == ops.E8M0, "grouped_gemm_fp8_nn: power-of-two (e8m0) scales"
    dev = xq.device
    assert dev.type == "cuda", "grouped_gemm_fp8_nn takes GPU tensors"
    offs = _check_offsets(m_offsets, E, dev, "grouped_gemm_fp8_nn")
    fresh = out is None
    if fresh:
        out = torch.empty((M, N), dtype=out_dtype, device=dev)
        if total_rows is None:
            total_rows = int(offs[-1].item()) if E > 0 else 0
        if total_rows < M:
            out[total_rows:].zero_()
    assert out.is_contiguous() and tuple(out.shape) == (M, N) and out.dtype in (torch.bfloat16, torch.float32)
    wqc, wsc, xsc = wq.contiguous(), ws.contiguous(), xs.contiguous()
    with torch.cuda.device(dev):
        rc = A.lib().lp_gemm_fp8_grouped_nn(
            xq.contiguous().data_ptr(), xsc.data_ptr(), wqc.data_ptr(), wsc.data_ptr(), A.E8M0, offs.data_ptr(), E, M, N, K,
            out.data_ptr(), A.BF16 if out.dtype == torch.bfloat16 else A.F32, A.stream_ptr())
    if rc == -2:            # LP_ERR_UNSUPPORTED: a shape the transposing-read kernel does not take
        wt = wqc.view(torch.uint8).transpose(1, 2).contiguous().view(ops.E4M3)
        wst = wsc.view(torch.uint8).transpose(1, 2).contiguous().view(ops.E8M0)
        return grouped_gemm_fp8(xq, xs, wt, wst, offs, out=out)
    A.check(rc)
    return out


def offsets_from_m_indices(m_indices: torch.Tensor, E: int) -> torch.Tensor:
    """Row ranges [E + 1] from a DeepGEMM-style contiguous layout: m_indices[r] = expert of row r, non-decreasing
    over the real rows, -1 on the padding rows that close an expert's (aligned) segment.  A padding row is attached to
    the expert whose segment it closes (leading ones to expert 0), so every real row keeps its own expert's range;
    no value is read back to the host."""
    idx = m_indices.to(torch.int64)
    owner = torch.cummax(idx, 0).values.clamp(min=0) if idx.numel() else idx
    counts = torch.bincount(owner, minlength=E)[:E]
    offs = torch.zeros(E + 1, dtype=torch.int32, device=m_indices.device)
    offs[1:] = torch.cumsum(counts, 0).to(torch.int32)
    return offs


def m_grouped_gemm_fp8_fp8_bf16_nt_contiguous(lhs, rhs, out: torch.Tensor, m_indices: torch.Tensor) -> None:
    """lhs = (x_fp8 [M,K], x_scale [M,K/128]); rhs = (w_fp8 [E,N,K], w_scale [E,N/128,K/128]);
    m_indices int32 [M], non-decreasing expert id per row, -1 = padding row; writes `out` [M,N] bf16 in place.
    DeepGEMM skips padding rows; here they are computed with the weights of the expert whose segment they close, so
    their rows of `out` hold unspecified (finite-input dependent) values instead of staying untouched -- every real
    row is the same either way."""
    xq, xs = lhs
    wq, ws = rhs
    assert m_indices.dim() == 1 and m_indices.numel() == xq.shape[0], (tuple(m_indices.shape), xq.shape[0])
    grouped_gemm_fp8(xq, xs, wq, ws, offsets_from_m_indices(m_indices.to(xq.device), wq.shape[0]), out=out)


def padded_blocks(rows: int, pad_rows: int) -> int:
    """128-row blocks an expert of `rows` rows takes in the column-wise operands (lp_quant_fp8_colwise_t's rule)."""
    rows = int(rows)
    if pad_rows == A.PAD_MIXED:
        return (rows + 127) // 128 if rows <= 256 else (rows + 511) // 512 * 4
    return (rows + pad_rows - 1) // pad_rows * (pad_rows // 128)


def choose_colwise_pad(m_splits) -> int:
    """How the experts' rows are padded in the column-wise operands: A.PAD_MIXED -- experts of at most 256 rows to 128 or
    256 (the row-scaled GEMM has a kernel without a K loop for problems of one and two K blocks: a weight gradient of a
    short expert is a write of N x K values more than a GEMM), the others to multiples of 512 (its hand-scheduled loop
    needs K in multiples of 512).  256 experts of [4096, 7168] with 0 .. 7163 rows: 6.7 ms with every expert padded to
    512, 9.7 ms with every expert padded to 128 (the experts above 256 rows then run on the compiler-scheduled kernel)."""
    return A.PAD_MIXED


def quant_fp8_colwise_t(x: torch.Tensor, m_offsets: torch.Tensor, m_splits, pad_rows: int | None = None):
    """Column-wise quantisation of expert-grouped rows with transposed output (the operands of the weight-gradient
    GEMM): x [M, C] bf16/fp32 on the GPU -> (codes uint8 [C * P], e8m0 scales [C * P / 128], blocks per expert),
    expert e's [C, P_e] / [C, P_e / 128] matrices stored one after the other, P_e = M_e rounded up to pad_rows (128, 256,
    512, or A.PAD_MIXED: 128 up to 256 rows and 512 beyond).  pad_rows None: choose_colwise_pad(m_splits)."""
    assert x.is_cuda and x.dim() == 2 and x.dtype in (torch.bfloat16, torch.float32)
    rows, cols = x.shape
    assert all(int(m) >= 0 for m in m_splits) and sum(int(m) for m in m_splits) <= rows, "m_splits must fit the rows of x"
    m_offsets = _check_offsets(m_offsets, len(m_splits), x.device, "quant_fp8_colwise_t")
    if pad_rows is None:
        pad_rows = choose_colwise_pad(m_splits)
    nblk = [padded_blocks(m, pad_rows) for m in m_splits]
    total = sum(nblk)
    q = torch.empty(cols * total * 128, dtype=torch.uint8, device=x.device)
    s = torch.empty(cols * total, dtype=ops.E8M0, device=x.device)
    x = x.contiguous()
    with torch.cuda.device(x.device):
        A.check(A.lib().lp_quant_fp8_colwise_t(x.data_ptr(), A.BF16 if x.dtype == torch.bfloat16 else A.F32, rows, cols,
                                               m_offsets.data_ptr(), len(nblk), total, pad_rows, q.data_ptr(), s.data_ptr(),
                                               A.E8M0, A.stream_ptr()))
    return q, s, nblk


def gemm_fp8_rowscale(aq, a_s, bq, b_s, M, N, K, out: torch.Tensor) -> torch.Tensor:
    """out[M, N] = sum over K blocks of (aq . bq^T) * a_s[m, kb] * b_s[n, kb]: e8m0 scales per row and 128 of K on
    both operands; aq / bq are flat uint8 views of [M, K] / [N, K]."""
    assert out.is_contiguous() and tuple(out.shape) == (M, N) and out.dtype in (torch.bfloat16, torch.float32)
    with torch.cuda.device(out.device):
        A.check(A.lib().lp_gemm_fp8_rowscale(aq.data_ptr(), a_s.data_ptr(), bq.data_ptr(), b_s.data_ptr(), A.E8M0, M, N, K,
                                             out.data_ptr(), A.BF16 if out.dtype == torch.bfloat16 else A.F32, A.stream_ptr()))
    return out


def rowscale_launches(k_blocks):
    """How the row-scaled problems of a grouped weight gradient are dealt to kernels: -> (launches, empty) with launches a
    list of (table, multiple) -- table rows {problem, K blocks, K blocks of the problems before it, 0} as
    lp_gemm_fp8_rowscale_grouped reads them, multiple = what every K block count of the table is a multiple of -- and
    empty the problems without K blocks (their outputs are zeros).  Problems whose K is a multiple of 512 share the
    hand-scheduled loop, those of one K block and those of two the kernel without a K loop, whatever is left the
    compiler-scheduled kernel."""
    before, fast, one, two, rest, empty = 0, [], [], [], [], []
    for e, kb in enumerate(k_blocks):
        kb = int(kb)
        assert kb >= 0
        if kb == 0:
            empty.append(e)
        else:
            (fast if kb % 4 == 0 else one if kb == 1 else two if kb == 2 else rest).append((e, kb, before, 0))
        before += kb
    return [(g, m) for g, m in ((fast, 4), (one, 1), (two, 2), (rest, 1)) if g], empty


def gemm_fp8_rowscale_grouped(aq, a_s, bq, b_s, k_blocks, M, N, out: torch.Tensor) -> torch.Tensor:
    """out[e] [M, N] = the row-scaled product of problem e, whose operands ([M, K_e] / [N, K_e] codes and their e8m0
    scales, K_e = 128 * k_blocks[e]) lie one after the other in aq / a_s / bq / b_s.  The problems whose K is a multiple
    of 512 go to the hand-scheduled loop in one launch, those of one and of two K blocks to the kernel without a K loop
    (a launch each), the others to the compiler-scheduled kernel; problems with no K blocks are zero-filled.  (The
    reference issues one grouped GEMM call: fp8.py:325-341.)"""
    E = len(k_blocks)
    assert out.is_contiguous() and tuple(out.shape) == (E, M, N) and out.dtype in (torch.bfloat16, torch.float32)
    launches, empty = rowscale_launches(k_blocks)
    if empty:
        out[torch.tensor(empty, device=out.device)] = 0
    odt = A.BF16 if out.dtype == torch.bfloat16 else A.F32
    with torch.cuda.device(out.device):
        for groups, multiple in launches:
            table = torch.tensor(groups, dtype=torch.int32).to(out.device)
            A.check(A.lib().lp_gemm_fp8_rowscale_grouped(aq.data_ptr(), a_s.data_ptr(), bq.data_ptr(), b_s.data_ptr(), A.E8M0,
                                                         table.data_ptr(), len(groups), max(g[1] for g in groups), multiple,
                                                         M, N, out.data_ptr(), odt, A.stream_ptr()))
            table.record_stream(torch.cuda.current_stream())
    return out


def _offsets(m_splits, dev):
    offs = torch.zeros(len(m_splits) + 1, dtype=torch.int32)
    offs[1:] = torch.cumsum(torch.tensor(m_splits, dtype=torch.int64), 0).to(torch.int32)
    return offs.to(dev)


class _GroupedGemmFp8(torch.autograd.Function):
    """gpatch_v4/models/deepseek_v4/fp8.py:180-343 without TransformerEngine, Float8BlockScaling with power-of-two
    scales: forward y_e = x_e W_e^T on 1 x 128 activations and 128 x 128 weights; backward
      dgrad  dx_e = dY_e W_e      (layout NN): dY quantised 1 x 128 along N, on the stored weight codes and scales: the
                                  kernel turns the weight operand while it reads it out of LDS (a 128 x 128 block
                                  scaling is its own transpose, its table is read by column); no transposed copy;
      wgrad  dW_e = dY_e^T X_e    (layout NT over column-wise operands): dY and X quantised per (column, 128 rows of
                                  the expert), transposed, the experts' row-scaled GEMMs in one launch per kind of
                                  expert (rowscale_launches: at most four) straight into dW.
    The reference pads every expert to a multiple of 16 rows for TE (fp8.py:29-58); here a ragged expert needs no
    padding in the forward and dgrad (tiles are masked), and the column-wise operands are zero-padded to whole blocks
    of 128 rows (choose_colwise_pad), which does not change any block's amax or sum."""

    @staticmethod
    def forward(ctx, inp, weight, wq, ws, m_splits, out_dtype):
        E, n_out, k_in = wq.shape
        x = inp.reshape(-1, k_in)
        xq, xs = _quant_pow2(x, (1, 128))
        offs = _offsets(m_splits, x.device)
        out = grouped_gemm_fp8(xq, xs, wq, ws, offs, out_dtype=out_dtype, total_rows=sum(m_splits))
        ctx.need_wgrad = weight is not None and weight.requires_grad
        ctx.need_dgrad = inp.requires_grad
        saved = [wq.view(torch.uint8), ws.view(torch.uint8), offs]
        if ctx.need_wgrad:
            ctx.pad_rows = choose_colwise_pad(m_splits)
            xtq, xts, _ = quant_fp8_colwise_t(x.detach(), offs, m_splits, ctx.pad_rows)
            saved += [xtq, xts.view(torch.uint8)]
        ctx.save_for_backward(*saved)
        ctx.m_splits, ctx.inp_shape, ctx.dims, ctx.out_dtype = m_splits, inp.shape, (E, n_out, k_in), out_dtype
        return out.view(*inp.shape[:-1], n_out)

    @staticmethod
    def backward(ctx, grad_output):
        E, n_out, k_in = ctx.dims
        wq, ws, offs = ctx.saved_tensors[:3]
        dy = grad_output.contiguous().view(-1, n_out)
        dgrad = wgrad = None
        if ctx.need_dgrad:
            dyq, dys = _quant_pow2(dy, (1, 128))
            dgrad = grouped_gemm_fp8_nn(dyq, dys, wq.view(ops.E4M3), ws.view(ops.E8M0), offs, out_dtype=ctx.out_dtype,
                                        total_rows=sum(ctx.m_splits)).view(ctx.inp_shape)
        if ctx.need_wgrad:
            xtq, xts = ctx.saved_tensors[3:5]
            dtq, dts, nblk = quant_fp8_colwise_t(dy, offs, ctx.m_splits, ctx.pad_rows)       # padded like X^T in the forward
            wgrad = torch.empty((E, n_out, k_in), dtype=ctx.out_dtype, device=dy.device)
            gemm_fp8_rowscale_grouped(dtq, dts.view(torch.uint8), xtq, xts, nblk, n_out, k_in, wgrad)
        return dgrad, wgrad, None, None, None, None


class MyTeGroupedLinearFp8(torch.nn.Module):
    """fp8.py:346-394 without TransformerEngine: weight is passed in ([E,N,K] bf16/fp32, or pre-quantised: a
    (data, scale) pair or a tensor / object with `_data` and `_scale`, 128 x 128 power-of-two scales), rows of `inp`
    are concatenated in expert order.  Differentiable in `inp` and in a tensor `weight` (fp8.py:285-343)."""

    def __init__(self, num_gemms: int, recipe=None):
        super().__init__()
        self.num_gemms = num_gemms
        self.recipe = recipe

    def forward(self, inp: torch.Tensor, weight, m_splits: list) -> torch.Tensor:
        assert len(m_splits) == self.num_gemms, (len(m_splits), self.num_gemms)
        m_splits = [int(x) for x in m_splits]
        assert all(m >= 0 for m in m_splits), "m_splits must not be negative"
        if hasattr(weight, "_data") and hasattr(weight, "_scale"):
            wq, ws = weight._data, weight._scale
        elif isinstance(weight, (tuple, list)):
            wq, ws = weight
        else:
            wq, ws = None, None
        shape = weight.shape if wq is None else wq.shape
        assert len(shape) == 3 and shape[0] == self.num_gemms, (tuple(shape), m_splits)
        n_out, k_in = shape[1], shape[2]
        assert inp.size(-1) == k_in, (inp.size(-1), k_in)
        assert sum(m_splits) == inp.numel() // k_in, (sum(m_splits), inp.numel() // k_in)
        if wq is None:
            # Float8BlockScaling recipe: power-of-two scales for activations and weights
            wq, ws = _quant_pow2(weight.detach(), (128, 128))
        if wq.dtype == torch.uint8:
            wq = wq.view(ops.E4M3)
        if ws.dtype != ops.E8M0:
            raise TypeError(f"pre-quantised weight scales must be float8_e8m0fnu (power of two), got {ws.dtype}")
        # fp8.py:139-161: codes shaped like the logical weight, one scale per 128 x 128 block
        assert wq.dtype == ops.E4M3, wq.dtype
        assert n_out % 128 == 0 and k_in % 128 == 0, (n_out, k_in)
        assert tuple(ws.shape) == (self.num_gemms, n_out // 128, k_in // 128), (tuple(ws.shape), tuple(shape))
        wt = weight if isinstance(weight, torch.Tensor) else None
        out_dtype = inp.dtype if inp.dtype in (torch.bfloat16, torch.float32) else torch.bfloat16
        return _GroupedGemmFp8.apply(inp, wt, wq.detach(), ws.detach(), m_splits, out_dtype)
