"""MI355X-native FP8 contraction path of modded-nanogpt: `nanogpt::mm`, the FP8 MLP forward with
fused ReLU^2, and the fused softcapped cross-entropy, as hand-written HIP kernels for gfx950
behind the reference's torch.library operator names.

Importing this package registers the operators (torch.ops.nanogpt.*).  The compute library
(lib/libngpt_fp8.so, built by `python -m modded_nanogpt_amd.build`) is loaded on first use and
its absence is an error: there is no fallback implementation.
"""
from . import _lib, ops                                   # noqa: F401  (registers torch.ops.nanogpt.*)
from .fused import (FusedLinearReLUSquareFunction, FusedSoftcappedCrossEntropy, ReLUSqrdMLP,  # noqa: F401
                    linear_relu_square, quantize_transpose_mlp_down_weights, reduce_mlp_activation_scales,
                    transpose_add, transpose_copy)
from .ops import gemm_fp8_tn, mlp_input_quant, quant_fp8, quant_fp8_2d, quant_up_weights     # noqa: F401

__all__ = [
    "FusedLinearReLUSquareFunction", "FusedSoftcappedCrossEntropy", "ReLUSqrdMLP",
    "linear_relu_square", "transpose_copy", "transpose_add", "quantize_transpose_mlp_down_weights",
    "reduce_mlp_activation_scales", "gemm_fp8_tn", "quant_fp8", "quant_fp8_2d", "mlp_input_quant", "quant_up_weights",
]
