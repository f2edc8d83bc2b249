"""Mirror of paddle.nn.quant's weight-only entry points
(python/paddle/nn/quant/__init__.py:28-42 in the reference)."""
from .moe import moe_ffn, moe_quantize_experts  # noqa: F401
from .quantized_linear import (  # noqa: F401
    apply_per_channel_scale,
    llm_int8_linear,
    weight_dequantize,
    weight_only_linear,
    weight_only_linear_fused,
    weight_quantize,
)

__all__ = ["weight_only_linear", "weight_quantize", "weight_dequantize", "apply_per_channel_scale",
           "llm_int8_linear", "weight_only_linear_fused", "moe_ffn", "moe_quantize_experts"]
