"""Entry points of the MXFP4 hot path, named as in ``alto/kernels/fp4/mxfp4/__init__.py:5-26``."""
from .attention import LPScaledDotProductAttention, attention_mxfp4_forward, quantize_qkv, triton_attention_mxfp4
from .config import TrainingOpConfig
from .grouped_gemm import (ALIGN_SIZE_M, MXFP4GroupedGEMM, _quantize_then_mxfp_scaled_grouped_mm,
                           create_indices_from_offsets_nosync, mxfp4_grouped_gemm, mxfp4_grouped_gemm_backward_inputs,
                           mxfp4_grouped_gemm_backward_weights, mxfp4_grouped_gemm_forward)
from .hadamard import HadamardFactory, HadamardTransform
from .linear import (MXFP4LinearFunction, _to_mxfp4_then_scaled_mm, blockwise_mxfp4_gemm, clear_weight_cache, enable_weight_cache,
                     transpose_codes, use_packed_scales, weight_cache_stats)
from .ops import register_torch_ops
from .qdq import _make_qdq_fn_for, quantize_dequantize
from .quantization import BLOCK_SIZE_DEFAULT, convert_from_mxfp4, convert_to_mxfp4, hadamard_left, quantize_rowcol
from ._runtime import enable_device_philox_state, set_rand_bits_source, use_hardware_stochastic_rounding
from .tensor import MXFP4TrainingWeightWrapperTensor, TrainingWeightWrapperBaseTensor, swap_params

__all__ = (
    "_quantize_then_mxfp_scaled_grouped_mm",
    "_to_mxfp4_then_scaled_mm",
    "ALIGN_SIZE_M",
    "BLOCK_SIZE_DEFAULT",
    "convert_from_mxfp4",
    "convert_to_mxfp4",
    "blockwise_mxfp4_gemm",
    "MXFP4LinearFunction",
    "mxfp4_grouped_gemm",
    "MXFP4GroupedGEMM",
    "mxfp4_grouped_gemm_forward",
    "mxfp4_grouped_gemm_backward_inputs",
    "mxfp4_grouped_gemm_backward_weights",
    "create_indices_from_offsets_nosync",
    "HadamardFactory",
    "HadamardTransform",
    "TrainingOpConfig",
    "quantize_rowcol",
    "hadamard_left",
    "transpose_codes",
    "set_rand_bits_source",
    "enable_device_philox_state",
    "use_hardware_stochastic_rounding",
    "MXFP4TrainingWeightWrapperTensor",
    "TrainingWeightWrapperBaseTensor",
    "swap_params",
    "enable_weight_cache",
    "use_packed_scales",
    "clear_weight_cache",
    "weight_cache_stats",
    "quantize_dequantize",
    "_make_qdq_fn_for",
    "triton_attention_mxfp4",
    "attention_mxfp4_forward",
    "quantize_qkv",
    "LPScaledDotProductAttention",
    "register_torch_ops",
)
