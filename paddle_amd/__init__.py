"""MI355X (gfx950) native weight-only quantized linear for Paddle's
weight_quantize / weight_dequantize / weight_only_linear path.

The compute lives in paddle_amd/lib/libwol_gfx950.so (hand-written HIP, C ABI
in include/wol_c_api.h).  paddle_amd.nn.quant mirrors paddle.nn.quant on
torch tensors, which serve only as device memory and stream handles.
"""
from . import _lib  # noqa: F401
from .nn import quant  # noqa: F401

__all__ = ["quant"]
