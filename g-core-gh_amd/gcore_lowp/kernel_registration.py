"""Registration of this package's functions with the reference's device-dispatched kernel registry
(gpatch_v4/kernel/registry.py:73-113: `register_kernel(name, fn, devices=...)`, one package
`gpatch_v4/kernel/<kernel_device_name>/__init__.py` per kernel device, imported once by `get_kernel`;
`kernel_device_name` comes from the `DeviceProtocol` subclass, gpatch_v4/core/device/protocol.py:38-46).

The reference's registry carries no quantiser or GEMM today (its quantisers are imported by module path), so nothing
here is needed for the import swaps; it exists so that a maintainer who adds a kernel device for this hardware can put

    from gpatch_v4.kernel.registry import register_kernel
    from gcore_lowp.kernel_registration import register_lowp_kernels
    register_lowp_kernels(register_kernel, devices="<kernel_device_name>")

into that device's package and dispatch with `get_kernel("quant_fp8_e4m3_scale_e8m0")(...)` like any other kernel.
Names are the reference's function names."""
from __future__ import annotations

from collections.abc import Callable, Sequence


def lowp_kernels() -> dict[str, Callable]:
    """name -> function, every entry callable with the reference function's arguments."""
    import importlib
    (convert_deepseek_v4_fp4_to_bf16, dsv4_kernels, eager_quant_kernels, fp8_blockwise, fused_quant_kernels, grouped_gemm_fp8,
     mygemm_fp8, qat) = (importlib.import_module(f"{__package__}.{m}") for m in (
         "convert_deepseek_v4_fp4_to_bf16", "dsv4_kernels", "eager_quant_kernels", "fp8_blockwise", "fused_quant_kernels",
         "grouped_gemm_fp8", "mygemm_fp8", "qat"))     # by module name: the package exports a function called grouped_gemm_fp8
    table = {
        "quant_fp8_e4m3_scale_e8m0": eager_quant_kernels.quant_fp8_e4m3_scale_e8m0,
        "quant_fp4_e2m1_scale_e8m0_packed": eager_quant_kernels.quant_fp4_e2m1_scale_e8m0_packed,
        "dequant_fp4_e2m1_fp8_scale_e8m0_packed": eager_quant_kernels.dequant_fp4_e2m1_fp8_scale_e8m0_packed,
        "quantize_fp8_blockwise": fp8_blockwise.quantize_fp8_blockwise,
        "cast_e2m1fn_to_bf16": convert_deepseek_v4_fp4_to_bf16.cast_e2m1fn_to_bf16,
        "cast_e4m3fn_to_bf16": convert_deepseek_v4_fp4_to_bf16.cast_e4m3fn_to_bf16,
        "cast_e2m1fn_to_e4m3fn": dsv4_kernels.cast_e2m1fn_to_e4m3fn,
        "official_expert_to_sgl": dsv4_kernels.official_expert_to_sgl,
        "fp4_qat_then_to_fp8": fused_quant_kernels.fp4_qat_then_to_fp8,
        "fp_qat_128x128": fused_quant_kernels.fp_qat_128x128,
        "act_quant": qat.act_quant,
        "fp4_simulate_qat": qat.fp4_simulate_qat,
        "fp8_simulate_qat": qat.fp8_simulate_qat,
        "fp8_simulate_qat_128x128": qat.fp8_simulate_qat_128x128,
        "gemm_fp8_block_scaling_impl": mygemm_fp8.gemm_fp8_block_scaling_impl,
        "gemm_impl": mygemm_fp8.gemm_impl,
        "m_grouped_gemm_fp8_fp8_bf16_nt_contiguous": grouped_gemm_fp8.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous,
    }
    return table


def register_lowp_kernels(register_kernel: Callable, devices: str | Sequence[str], only: Sequence[str] | None = None) -> list[str]:
    """Call `register_kernel(name, fn, devices=devices)` for every function of lowp_kernels() (or those named in `only`);
    returns the names registered.  Errors of the registry (a name already registered for a device: ValueError) pass
    through unchanged, before anything else of that name is registered."""
    table = lowp_kernels()
    if only is not None:
        unknown = [n for n in only if n not in table]
        if unknown:
            raise KeyError(f"not a kernel of this package: {unknown}")
    names = [n for n in table if only is None or n in only]
    for n in names:
        register_kernel(n, table[n], devices=devices)
    return names
