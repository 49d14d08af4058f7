"""The C-ABI library loads without a GPU, exports every symbol include/lowp.h declares,
and rejects bad arguments on the host before anything is launched."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from gcore_lowp import _abi
    if not os.path.exists(_abi.LIB_PATH):
        pytest.fail(f"{_abi.LIB_PATH} missing: run `python g-core-gh_amd/build.py`")
    return _abi


def _declared(header="lowp.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lp_[a-z0-9_]+)\s*\(", text)))


def _declarations_with_comments(header="lowp.h"):
    """(name, text of the comment block right in front of the declaration) for every entry point of a header."""
    text = open(os.path.join(ROOT, "include", header)).read()
    out = []
    for m in re.finditer(r"/\*((?:(?!\*/).)*)\*/\s*(?:const\s+char\s*\*|int64_t|int)\s*(lp_[a-z0-9_]+)\s*\(", text, flags=re.S):
        out.append((m.group(2), m.group(1)))
    return out


def test_every_declared_symbol_is_exported_and_bound(lib):
    names = _declared()
    assert len(names) >= 12
    L = lib.lib()
    for n in names:
        assert hasattr(L, n), f"{n} declared in include/lowp.h but not exported"
        assert n in lib.PROTOTYPES, f"{n} has no ctypes prototype"
    assert sorted(lib.PROTOTYPES) == names
    assert L.lp_version() >= 100


def test_drop_in_header_lists_only_reference_interfaces(lib):
    """include/lowp.h is the drop-in ABI: every entry point's comment cites the reference interface it stands in for
    (a file:line in the reference tree), or is one of the plumbing calls of the library itself (version, error text,
    workspace / scratch sizes), or says that it has no counterpart and whom it is for (the entry point that allocates
    nothing).  Measurement aids and self tests live in include/lowp_probe.h and in a library of their own."""
    plumbing = {"lp_version", "lp_last_error", "lp_gemm_workspace_bytes", "lp_gemm_static_scratch_bytes"}
    cite = re.compile(r"[A-Za-z0-9_/]+\.py:\d+")
    decls = _declarations_with_comments()
    names = {n for n, _ in decls}
    assert names | plumbing >= set(_declared()), sorted(set(_declared()) - names - plumbing)
    for name, comment in decls:
        if name in plumbing:
            continue
        assert "probe" not in name and "selftest" not in name and "debug" not in name, name
        assert cite.search(comment) or "no counterpart in the reference" in comment, f"{name}: no reference citation"
    probe = _declared("lowp_probe.h")
    assert not set(probe) & set(_declared()), "an entry point is declared in both headers"


def test_probe_header_matches_probe_library(lib):
    from gcore_lowp import _probe_abi as P
    if not os.path.exists(P.LIB_PATH):
        pytest.fail(f"{P.LIB_PATH} missing: run `python g-core-gh_amd/build.py`")
    names = _declared("lowp_probe.h")
    L = P.lib()
    for n in names:
        assert hasattr(L, n), f"{n} declared in include/lowp_probe.h but not exported"
    assert sorted(P.PROTOTYPES) == names
    # the product library exports none of them, and does not depend on the probe library
    prod = lib.lib()
    for n in names:
        assert not hasattr(prod, n), f"{n} is exported by the product library"
    one = ctypes.c_void_p(16)
    assert L.lp_probe_mfma(3, 10, None, 16, None) == -1 and b"FMAs" in L.lp_probe_last_error()
    assert L.lp_probe_stream(one, 15, one, 16, 8, None) == -1
    assert L.lp_selftest(9, one, None) == -1
    assert L.lp_debug_cast(0, None, None, 0, None) == 0


def test_host_side_validation(lib):
    L = lib.lib()
    one = ctypes.c_void_p(16)       # never dereferenced: validation fails first
    # shape not divisible by the block
    rc = L.lp_quant_fp8_block(one, lib.BF16, 100, 128, 128, 128, lib.SCALE_DIV, 0.0, 0, one, one, lib.F32, None, None)
    assert rc == -1 and "not divisible" in lib.last_error()
    rc = L.lp_quant_fp8_block(one, 7, 128, 128, 128, 128, lib.SCALE_DIV, 0.0, 0, one, one, lib.F32, None, None)
    assert rc == -1 and "x_dtype" in lib.last_error()
    rc = L.lp_quant_fp8_block(None, lib.BF16, 128, 128, 128, 128, lib.SCALE_DIV, 0.0, 0, one, one, lib.F32, None, None)
    assert rc == -1 and "null" in lib.last_error()
    rc = L.lp_dequant_fp8_block(one, one, lib.F32, 128, 100, 128, 128, one, lib.BF16, None)
    assert rc == -1 and "not divisible" in lib.last_error()
    rc = L.lp_fp4_to_fp8_rebase(one, one, 128, 64, one, one, lib.E8M0, None)
    assert rc == -1 and "multiple of 128" in lib.last_error()
    rc = L.lp_gemm_fp8_block(one, one, one, one, lib.F32, 64, 128, 100, one, lib.BF16, None, 0, None)
    assert rc == -1 and "multiple of 128" in lib.last_error()
    rc = L.lp_gemm_fp8_grouped(one, one, one, one, lib.F32, None, 4, 64, 128, 128, one, lib.BF16, None)
    assert rc == -1 and "m_offsets" in lib.last_error()
    # the entry points added around the path: QAT conversions, FP4 quantiser, backward of the grouped linear
    rc = L.lp_quant_fp8_block(one, lib.BF16, 128, 128, 128, 128, 6, 0.0, 0, one, one, lib.F32, None, None)
    assert rc == -1 and "scale_mode" in lib.last_error()
    rc = L.lp_quant_fp4_block(one, lib.BF16, 128, 100, 1, 32, one, one, None, None)
    assert rc == -1
    rc = L.lp_qdq_fp8_tile128(one, 128, 100, one, None)
    assert rc == -1 and "128 x 128" in lib.last_error()
    rc = L.lp_fp4_qat_to_fp8(one, 100, 128, one, one, None)
    assert rc == -1 and "128 x 128" in lib.last_error()
    rc = L.lp_fp4_qdq_row32(one, 100, one, None, None)
    assert rc == -1 and "multiple of 32" in lib.last_error()
    rc = L.lp_act_qdq_group(one, 1024, 48, 1, 0, one, None, None)
    assert rc == -1 and "power of two" in lib.last_error()
    rc = L.lp_act_qdq_group(one, 1000, 64, 1, 0, one, None, None)
    assert rc == -1 and "multiple of the group size" in lib.last_error()
    rc = L.lp_act_qdq_group(one, 1024, 64, 0, 0, one, None, None)
    assert rc == -1 and "power-of-two scales" in lib.last_error()
    rc = L.lp_quant_fp8_colwise_t(one, lib.BF16, 256, 100, one, 2, 2, 128, one, one, lib.E8M0, None)
    assert rc == -1 and "multiple of 128" in lib.last_error()
    rc = L.lp_quant_fp8_colwise_t(one, lib.BF16, 256, 128, one, 2, 2, 100, one, one, lib.E8M0, None)
    assert rc == -1 and "pad_rows" in lib.last_error()
    rc = L.lp_gemm_fp8_rowscale(one, one, one, one, lib.E8M0, 64, 100, 128, one, lib.BF16, None)
    assert rc == -1 and "multiple of 128" in lib.last_error()
    # empty problems succeed without touching the device
    assert L.lp_fp4_qdq_row32(None, 0, None, None, None) == 0
    assert L.lp_act_qdq_group(None, 0, 128, 1, 0, None, None, None) == 0
    assert L.lp_quant_fp8_colwise_t(None, lib.BF16, 0, 128, None, 0, 0, 128, None, None, lib.E8M0, None) == 0
    assert L.lp_gemm_fp8_rowscale(None, None, None, None, lib.E8M0, 0, 128, 128, None, lib.BF16, None) == 0
    assert L.lp_gemm_fp8_rowscale_grouped(None, None, None, None, lib.E8M0, None, 0, 0, 1, 128, 128, None, lib.BF16, None) == 0
    rc = L.lp_gemm_fp8_rowscale_grouped(one, one, one, one, lib.E8M0, one, 2, 4, 4, 100, 128, one, lib.BF16, None)
    assert rc == -1 and "multiple of 128" in lib.last_error()
    assert L.lp_quant_fp8_block(None, lib.BF16, 0, 128, 128, 128, lib.SCALE_DIV, 0.0, 0, None, None, lib.F32, None, None) == 0
    assert L.lp_gemm_fp8_block(None, None, None, None, lib.F32, 0, 128, 128, None, lib.BF16, None, 0, None) == 0
    assert L.lp_gemm_fp8_block_static(None, None, None, None, lib.F32, 0, 128, 128, None, lib.BF16, None) == 0


def test_static_scratch_holds_the_largest_split_and_bad_shapes_are_refused(lib):
    """The entry point that brings its own K-split scratch: the K split is taken for at most 32 tiles of 128 x 128 in at
    most 16 K ranges, i.e. 32 MiB of fp32 partial sums, which is the built-in buffer's size, so no shape the dispatcher
    would split is turned away (the size check in the entry point stays as a guard against a dispatcher that changes);
    arguments the GEMM refuses are refused here as well, before anything is launched or looked up on the device."""
    import ctypes
    import random
    L = lib.lib()
    cap = L.lp_gemm_static_scratch_bytes()
    assert cap == 32 << 20
    assert L.lp_gemm_workspace_bytes(2048, 256, 8192) >= 16 * 2048 * 256 * 4 == cap        # the largest: 32 tiles x 16 ranges
    rng = random.Random(5)
    split_seen = 0
    for _ in range(4000):
        M, N, K = rng.randint(1, 8192), 128 * rng.randint(1, 64), 128 * rng.randint(1, 160)
        need = L.lp_gemm_workspace_bytes(M, N, K)
        # besides the partial sums the workspace holds fp32 copies of e8m0 scales (a tuning aid, not part of the static entry's need)
        r256 = lambda x: (x + 255) // 256 * 256
        scale_copies = r256(M * (K // 128) * 4) + r256((N // 128) * (K // 128) * 4) if M > 64 and K % 512 == 0 else 0
        partial = need - scale_copies
        assert partial >= 0 and partial % (M * N * 4) == 0 and partial <= cap, (M, N, K, need)
        tiles = (M + 127) // 128 * (N // 128)
        assert partial == 0 or (tiles <= 32 and 2 <= partial // (M * N * 4) <= 16), (M, N, K, need)
        split_seen += partial > 0
    assert split_seen > 20
    buf = ctypes.create_string_buffer(64)
    one = ctypes.cast(ctypes.addressof(buf) + (-ctypes.addressof(buf)) % 16, ctypes.c_void_p)
    rc = L.lp_gemm_fp8_block_static(one, one, one, one, lib.F32, 64, 100, 128, one, lib.BF16, None)
    assert rc == -1 and "multiple of 128" in lib.last_error()


def test_wrappers_keep_reference_exceptions(lib):
    """Shape / dtype errors are raised as the reference raises them, before any GPU work."""
    import torch
    import gcore_lowp as G

    with pytest.raises(AssertionError):
        G.quant_fp8_e4m3_scale_e8m0(torch.zeros(100, 128), (128, 128))
    with pytest.raises(ValueError):
        G.quantize_fp8_blockwise(torch.zeros(2, 128, 128), (128, 128))
    with pytest.raises(ValueError):
        G.quantize_fp8_blockwise(torch.zeros(100, 128), (128, 128))
    with pytest.raises(AssertionError):
        G.cast_e2m1fn_to_bf16(torch.zeros(4, 16, dtype=torch.uint8), torch.zeros(4, 1))
    with pytest.raises(AssertionError):
        G.cast_e4m3fn_to_bf16(torch.zeros(128, 128).to(torch.float8_e4m3fn), torch.zeros(2, 1))
    with pytest.raises(AssertionError):
        G.cast_e2m1fn_to_e4m3fn(torch.zeros(128, 32, dtype=torch.int8), torch.zeros(128, 2))
    with pytest.raises(AssertionError):
        G.gemm_fp8_block_scaling_impl(torch.zeros(4, 128).to(torch.float8_e4m3fn), torch.zeros(4, 2),
                                      torch.zeros(128, 128).to(torch.float8_e4m3fn), torch.zeros(1, 1))


@pytest.mark.skipif(__import__("torch").cuda.is_available(), reason="GPU present")
def test_no_cpu_fallback_without_gpu(lib):
    import torch
    import gcore_lowp as G

    with pytest.raises(lib.LowpError, match="no GPU"):
        G.quant_2d(torch.zeros(128, 128, dtype=torch.bfloat16))
