"""ctypes binding of libwol_gfx950.so (the C ABI of include/wol_c_api.h).

The library is the only compute path: if it is missing, import fails loudly
instead of falling back to anything else.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libwol_gfx950.so")

DTYPE_F16, DTYPE_BF16 = 0, 1
ROUND_RNE, ROUND_TRUNC = 0, 1
LAYOUT_CANONICAL, LAYOUT_PADDLE_HIP, LAYOUT_GFX950 = 0, 1, 2

# every symbol include/wol_c_api.h and include/wol_diag.h declare
SYMBOLS = (
    "wol_status_str",
    "wol_layout_version",
    "wol_quantize_workspace",
    "wol_quantize",
    "wol_quantize_static",
    "wol_quantize_llm_int8",
    "wol_dequantize",
    "wol_linear_workspace",
    "wol_linear",
    "wol_linear_f32",
    "wol_linear_workspace_for",
    "wol_linear_on",
    "wol_linear_fused_workspace",
    "wol_linear_fused",
    "wol_linear_grad_workspace",
    "wol_linear_grad",
    "wol_linear_grad_f32",
    "wol_moe_ffn_workspace",
    "wol_moe_ffn",
    "wol_repack",
    "wol_repack_host",
    "wol_code_offset",
    "wol_apply_per_channel_scale",
    "wol_read_floor",
    "wol_mfma_ceiling",
    "wol_mfma_probe",
    "wol_prefill_phases",
    "wol_decode_phases",
    "wol_linear_plan",
    "wol_linear_grad_plan",
    "wol_llm_int8_linear_workspace",
    "wol_llm_int8_linear",
    "wol_llm_int8_linear_stage_offsets",
)


class WolError(RuntimeError):
    """A non-zero wol_status that is not an argument error."""


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libwol_gfx950.so is not built (%s); run paddle_amd/csrc/build.sh or "
            "__graft_entry__.build()" % LIB_PATH
        )
    lib = ctypes.CDLL(LIB_PATH)
    vp, i64, ci, sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t
    lib.wol_status_str.argtypes = [ci]
    lib.wol_status_str.restype = ctypes.c_char_p
    lib.wol_layout_version.argtypes = []
    lib.wol_layout_version.restype = ci
    lib.wol_quantize_workspace.argtypes = [i64, i64, ci, ci]
    lib.wol_quantize_workspace.restype = sz
    lib.wol_quantize.argtypes = [vp, ci, i64, i64, ci, ci, ci, ci, vp, vp, vp, sz, vp]
    lib.wol_quantize.restype = ci
    lib.wol_quantize_static.argtypes = [vp, ci, i64, i64, ci, ci, ci, ci, vp, vp, vp]
    lib.wol_quantize_static.restype = ci
    lib.wol_quantize_llm_int8.argtypes = [vp, ci, i64, i64, ci, ci, vp, vp, vp, sz, vp]
    lib.wol_quantize_llm_int8.restype = ci
    lib.wol_dequantize.argtypes = [vp, ci, vp, ci, i64, i64, ci, ci, vp, vp]
    lib.wol_dequantize.restype = ci
    lib.wol_linear_workspace.argtypes = [i64, i64, i64, ci, ci]
    lib.wol_linear_workspace.restype = sz
    lib.wol_linear.argtypes = [vp, vp, vp, vp, ci, i64, i64, i64, ci, ci, vp, vp, sz, vp]
    lib.wol_linear.restype = ci
    lib.wol_linear_f32.argtypes = [vp, vp, vp, vp, ci, i64, i64, i64, ci, ci, vp, vp, sz, vp]
    lib.wol_linear_f32.restype = ci
    lib.wol_linear_workspace_for.argtypes = [i64, i64, i64, ci, ci, ci]
    lib.wol_linear_workspace_for.restype = sz
    lib.wol_linear_on.argtypes = [vp, vp, vp, vp, ci, i64, i64, i64, ci, ci, vp, ci, ci, vp, sz, vp]
    lib.wol_linear_on.restype = ci
    lib.wol_linear_fused_workspace.argtypes = [i64, i64, i64, ci, ci, ci, ci]
    lib.wol_linear_fused_workspace.restype = sz
    lib.wol_linear_fused.argtypes = [vp, vp, vp, vp, vp, ci, i64, i64, i64, ci, ci, ci, vp, vp, sz, vp]
    lib.wol_linear_fused.restype = ci
    lib.wol_linear_grad_workspace.argtypes = [i64, i64, i64, ci, ci]
    lib.wol_linear_grad_workspace.restype = sz
    lib.wol_linear_grad.argtypes = [vp, vp, vp, ci, i64, i64, i64, ci, ci, vp, vp, sz, vp]
    lib.wol_linear_grad.restype = ci
    lib.wol_linear_grad_f32.argtypes = [vp, vp, vp, ci, i64, i64, i64, ci, ci, vp, vp, sz, vp]
    lib.wol_linear_grad_f32.restype = ci
    lib.wol_moe_ffn_workspace.argtypes = [i64, i64, i64, ci]
    lib.wol_moe_ffn_workspace.restype = sz
    lib.wol_moe_ffn.argtypes = [vp, vp, vp, vp, vp, vp, vp, ci, i64, i64, i64, ci, ci, vp, vp, sz, vp]
    lib.wol_moe_ffn.restype = ci
    lib.wol_repack.argtypes = [vp, ci, vp, ci, i64, i64, ci, vp]
    lib.wol_repack.restype = ci
    lib.wol_repack_host.argtypes = [vp, ci, vp, ci, i64, i64, ci]
    lib.wol_repack_host.restype = ci
    lib.wol_code_offset.argtypes = [ci, i64, i64, ci, i64, i64, ctypes.POINTER(ci)]
    lib.wol_code_offset.restype = i64
    lib.wol_apply_per_channel_scale.argtypes = [vp, vp, ci, i64, i64, vp, vp]
    lib.wol_apply_per_channel_scale.restype = ci
    lib.wol_read_floor.argtypes = [vp, i64, i64, ci, vp, vp]
    lib.wol_read_floor.restype = ci
    lib.wol_mfma_ceiling.argtypes = [vp, ci, ci, vp, vp]
    lib.wol_mfma_ceiling.restype = ci
    lib.wol_mfma_probe.argtypes = [ci, vp, sz, ci, ci, vp, vp]
    lib.wol_mfma_probe.restype = ci
    lib.wol_prefill_phases.argtypes = [vp, vp, vp, i64, i64, i64, vp, vp, sz, vp]
    lib.wol_prefill_phases.restype = ci
    lib.wol_decode_phases.argtypes = [vp, vp, vp, i64, i64, ci, vp, vp, sz, vp]
    lib.wol_decode_phases.restype = ci
    lib.wol_linear_plan.argtypes = [i64, i64, i64, ci, ci, sz, ctypes.c_char_p, sz]
    lib.wol_linear_plan.restype = ci
    lib.wol_linear_grad_plan.argtypes = [i64, i64, i64, ctypes.c_char_p, sz]
    lib.wol_linear_grad_plan.restype = ci
    lib.wol_llm_int8_linear_workspace.argtypes = [i64, i64, i64]
    lib.wol_llm_int8_linear_workspace.restype = sz
    lib.wol_llm_int8_linear.argtypes = [vp, vp, vp, vp, ctypes.c_float, ci, i64, i64, i64, vp, vp, sz, vp]
    lib.wol_llm_int8_linear.restype = ci
    lib.wol_llm_int8_linear_stage_offsets.argtypes = [i64, i64, i64, ctypes.POINTER(i64)]
    lib.wol_llm_int8_linear_stage_offsets.restype = ci
    return lib


lib = _load()

# statuses that are argument errors (the reference raises InvalidArgument,
# which Paddle surfaces as ValueError)
_ARG_ERRORS = {1, 2, 3, 4, 5, 6, 7, 8, 9}

ACT_NONE, ACT_GELU, ACT_SWIGLU = 0, 1, 2

# wol_kernel
KERNEL_AUTO, KERNEL_STREAM, KERNEL_GEMM, KERNEL_BATCH, KERNEL_BATCH_SPLIT = 0, 1, 2, 3, 4


def check(status):
    if status == 0:
        return
    msg = lib.wol_status_str(status).decode()
    if status in _ARG_ERRORS:
        raise ValueError("(InvalidArgument) %s [wol_status %d]" % (msg, status))
    raise WolError("%s [wol_status %d]" % (msg, status))
