"""gcore_lowp: MI355X-native block-FP8 / FP4 quantise, dequantise, convert and GEMM path.

Python call signatures follow the reference functions they replace; the work is
done by hand-written gfx950 HIP kernels behind a C ABI (include/lowp.h).
"""
from . import _abi  # noqa: F401
from .eager_quant_kernels import (  # noqa: F401
    dequant_fp4_e2m1_fp8_scale_e8m0_packed, quant_fp4_e2m1_scale_e8m0_packed, quant_fp8_e4m3_scale_e8m0)
from .fp8_blockwise import quant_1d, quant_2d, quant_act, quant_weight, quantize_fp8_blockwise  # noqa: F401
from .convert_deepseek_v4_fp4_to_bf16 import cast_e2m1fn_to_bf16, cast_e4m3fn_to_bf16  # noqa: F401
from .dsv4_kernels import (  # noqa: F401
    cast_e2m1fn_to_e4m3fn, dequant_fp8_block, fp4_to_fp8_blockwise, official_dense_to_sgl,
    official_expert_to_sgl, official_wo_a_to_sgl, sgl_dense_to_official, sgl_wo_a_to_official,
)
from .mygemm_fp8 import gemm_fp8_block_scaling_impl, gemm_impl  # noqa: F401
from .grouped_gemm_fp8 import (  # noqa: F401
    MyTeGroupedLinearFp8, gemm_fp8_rowscale, gemm_fp8_rowscale_grouped, grouped_gemm_fp8, grouped_gemm_fp8_nn,
    m_grouped_gemm_fp8_fp8_bf16_nt_contiguous,
    quant_fp8_colwise_t,
)
from .fp8_tensor import Fp8TensorAg, Fp8TensorTrain  # noqa: F401
