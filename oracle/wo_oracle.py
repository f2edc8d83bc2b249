"""ctypes front end of the CPU oracle (oracle/wo_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and
by the cpu_baseline leg of bench.py, always as the checker or the timed CPU
baseline, never by the shipped package.

Arrays are numpy: weights / activations / scales travel as uint16 bit patterns
of float16 or bfloat16, codes as int8.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libwo_oracle.so")

F16, BF16 = 0, 1
CAST_RNE, CAST_TRUNC = 0, 1

_u16p = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")
_i8p = np.ctypeslib.ndpointer(np.int8, flags="C_CONTIGUOUS")
_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_i64 = ctypes.c_int64
_int = ctypes.c_int


def build(force=False):
    """Compile the oracle (and oracle/_ref when the reference tree exists)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B"] if force else ["make", "-C", _HERE])


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.wo_from_f32.argtypes = [ctypes.c_float, _int, _int]
        L.wo_from_f32.restype = ctypes.c_uint16
        L.wo_to_f32.argtypes = [ctypes.c_uint16, _int]
        L.wo_to_f32.restype = ctypes.c_float
        L.wo_cast_array_from_f32.argtypes = [_f32p, _i64, _int, _int, _u16p]
        L.wo_cast_array_to_f32.argtypes = [_u16p, _i64, _int, _f32p]
        L.wo_per_channel_scale.argtypes = [_u16p, _i64, _i64, _int, ctypes.c_float, _int, _u16p]
        L.wo_group_wise_scale.argtypes = [_u16p, _i64, _i64, _int, ctypes.c_float, _i64, _int, _u16p]
        L.wo_quant_codes.argtypes = [_u16p, _u16p, _i64, _i64, _int, _int, _i64, _int, _i8p]
        L.wo_weight_quantize.argtypes = [_u16p, _i64, _i64, _int, _int, _i64, _int, _int, _i8p, _u16p]
        L.wo_weight_quantize.restype = _int
        L.wo_weight_quantize_llm_int8.argtypes = [_u16p, _i64, _i64, _int, _i64, _i8p, _f32p]
        L.wo_weight_quantize_llm_int8.restype = _int
        L.wo_transpose_bytes.argtypes = [_i8p, _i64, _i64, _i8p]
        L.wo_apply_per_channel_scale.argtypes = [_u16p, _u16p, _i64, _i64, _int, _u16p]
        L.wo_apply_per_channel_scale.restype = None
        L.wo_llm_int8_linear.argtypes = [_u16p, _i8p, ctypes.c_void_p, _f32p, ctypes.c_float, _i64, _i64, _i64,
                                         _int, _u16p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                         ctypes.c_void_p]
        L.wo_llm_int8_linear.restype = None
        L.wo_div127_fma_mismatches.argtypes = [ctypes.c_uint32, ctypes.c_uint32, _i64]
        L.wo_div127_fma_mismatches.restype = _i64
        L.wo_dequantize.argtypes = [_i8p, _u16p, _i64, _i64, _int, _int, _i64, _int, _int,
                                    ctypes.c_void_p, ctypes.c_void_p]
        L.wo_linear.argtypes = [_u16p, _i8p, ctypes.c_void_p, _u16p, _i64, _i64, _i64, _int, _int,
                                _i64, _int, _int, _f32p, ctypes.c_void_p]
        L.wo_activation.argtypes = [_f32p, _i64, _i64, _int, _int, _f32p, ctypes.c_void_p]
        L.wo_activation.restype = None
        L.wo_linear_grad.argtypes = [_u16p, _i8p, _u16p, _i64, _i64, _i64, _int, _int, _i64, _int, _int, _f32p,
                                     ctypes.c_void_p]
        L.wo_linear_grad.restype = None
        L.wo_linear_grad_rounded_weight.argtypes = [_u16p, _i8p, _u16p, _i64, _i64, _i64, _int, _int, _i64, _int, _int, _f32p,
                                     ctypes.c_void_p]
        L.wo_linear_grad_rounded_weight.restype = None
        _lib = L
    return _lib


def from_f32(a, dtype, cast_mode=CAST_RNE):
    a = np.ascontiguousarray(a, dtype=np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().wo_cast_array_from_f32(a.reshape(-1), a.size, dtype, cast_mode, out.reshape(-1))
    return out


def to_f32(a, dtype):
    a = np.ascontiguousarray(a, dtype=np.uint16)
    out = np.empty(a.shape, np.float32)
    lib().wo_cast_array_to_f32(a.reshape(-1), a.size, dtype, out.reshape(-1))
    return out


def weight_quantize(w_bits, dtype, bits, group_size=-1, cast_mode=CAST_RNE, nibble_bias=0):
    """w_bits: [K,N] uint16.  Returns (codes, scale): canonical codes [K,N] int8
    or [K,N/2] packed nibbles, scale [N] or [ceil(K/g),N] uint16."""
    w_bits = np.ascontiguousarray(w_bits, dtype=np.uint16)
    K, N = w_bits.shape
    codes = np.empty((K, N if bits == 8 else N // 2), np.int8)
    if group_size == -1:
        scale = np.empty((N,), np.uint16)
    else:
        scale = np.empty(((K + group_size - 1) // group_size, N), np.uint16)
    rc = lib().wo_weight_quantize(w_bits, K, N, dtype, bits, group_size, cast_mode, nibble_bias,
                                  codes, scale)
    if rc != 0:
        raise ValueError("oracle: shape/group_size outside the weight_quantize contract")
    return codes, scale


def weight_quantize_llm_int8(w_bits, dtype, group_size=-1):
    """algo="llm.int8": canonical int8 codes [K,N] and fp32 scales [N] or [ceil(K/g),N]."""
    w_bits = np.ascontiguousarray(w_bits, dtype=np.uint16)
    K, N = w_bits.shape
    codes = np.empty((K, N), np.int8)
    shape = (N,) if group_size == -1 else ((K + group_size - 1) // group_size, N)
    scale = np.empty(shape, np.float32)
    if lib().wo_weight_quantize_llm_int8(w_bits, K, N, dtype, group_size, codes, scale) != 0:
        raise ValueError("oracle: shape/group_size outside the weight_quantize contract")
    return codes, scale


def apply_per_channel_scale(x_bits, scale_bits, dtype):
    """x_bits [rows, cols] uint16, scale_bits [cols] uint16 -> T-bits [rows, cols]."""
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    scale_bits = np.ascontiguousarray(scale_bits, dtype=np.uint16)
    rows, cols = x_bits.shape
    assert scale_bits.shape == (cols,)
    out = np.empty((rows, cols), np.uint16)
    lib().wo_apply_per_channel_scale(x_bits, scale_bits, rows, cols, dtype, out)
    return out


def llm_int8_linear(x_bits, w_nk, bias_bits, wscale, threshold, dtype):
    """x_bits [M,K] uint16, w_nk [N,K] int8, wscale [N] float32.  Returns a dict:
    out (T bits [M,N]), qx (int8 [M,K]), acc (int32 [M,N]), ranges (float32 [M]),
    outlier (bool [K])."""
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    w_nk = np.ascontiguousarray(w_nk, dtype=np.int8)
    wscale = np.ascontiguousarray(wscale, dtype=np.float32)
    M, K = x_bits.shape
    N = w_nk.shape[0]
    assert w_nk.shape == (N, K) and wscale.shape == (N,)
    out = np.empty((M, N), np.uint16)
    qx = np.empty((M, K), np.int8)
    acc = np.empty((M, N), np.int32)
    ranges = np.empty(M, np.float32)
    outlier = np.empty(K, np.uint8)
    bias_ptr = None
    if bias_bits is not None:
        bias_bits = np.ascontiguousarray(bias_bits, dtype=np.uint16)
        bias_ptr = bias_bits.ctypes.data
    lib().wo_llm_int8_linear(x_bits, w_nk, bias_ptr, wscale, float(threshold), M, K, N, dtype, out,
                             qx.ctypes.data, acc.ctypes.data, ranges.ctypes.data, outlier.ctypes.data)
    return {"out": out, "qx": qx, "acc": acc, "ranges": ranges, "outlier": outlier.astype(bool)}


def div127_fma_mismatches(first, stride, count):
    """Inputs (float bit patterns first, first + stride, ...) on which the FMA-corrected
    reciprocal multiply of the HIP epilogue differs from the IEEE division by 127."""
    return int(lib().wo_div127_fma_mismatches(first, stride, count))


def transpose_bytes(a):
    a = np.ascontiguousarray(a, dtype=np.int8)
    out = np.empty((a.shape[1], a.shape[0]), np.int8)
    lib().wo_transpose_bytes(a, a.shape[0], a.shape[1], out)
    return out


def dequantize(codes, scale, dtype, bits, group_size=-1, nibble_bias=0, cast_mode=CAST_RNE):
    """Returns (fp32 [K,N], T-bits [K,N])."""
    codes = np.ascontiguousarray(codes, dtype=np.int8)
    scale = np.ascontiguousarray(scale, dtype=np.uint16)
    K = codes.shape[0]
    N = codes.shape[1] if bits == 8 else codes.shape[1] * 2
    out32 = np.empty((K, N), np.float32)
    outT = np.empty((K, N), np.uint16)
    lib().wo_dequantize(codes, scale, K, N, dtype, bits, group_size, nibble_bias, cast_mode,
                        out32.ctypes.data, outT.ctypes.data)
    return out32, outT


def linear(x_bits, codes, scale, bias_bits, dtype, bits, group_size=-1, nibble_bias=0, acc64=False):
    """x_bits [M,K] uint16.  Returns (out32 [M,N] fp32, outT [M,N] uint16)."""
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    codes = np.ascontiguousarray(codes, dtype=np.int8)
    scale = np.ascontiguousarray(scale, dtype=np.uint16)
    M, K = x_bits.shape
    N = codes.shape[1] if bits == 8 else codes.shape[1] * 2
    assert codes.shape[0] == K
    out32 = np.empty((M, N), np.float32)
    outT = np.empty((M, N), np.uint16)
    bias_ptr = None
    if bias_bits is not None:
        bias_bits = np.ascontiguousarray(bias_bits, dtype=np.uint16)
        bias_ptr = bias_bits.ctypes.data
    lib().wo_linear(x_bits, codes, bias_ptr, scale, M, K, N, dtype, bits, group_size, nibble_bias,
                    1 if acc64 else 0, out32, outT.ctypes.data)
    return out32, outT


ACT_NONE, ACT_GELU, ACT_SWIGLU = 0, 1, 2


def activation(in32, act, dtype):
    """The fused epilogue on fp32 sums [M,N]: returns (fp32, T-bits), [M,N] for
    none/gelu, [M,N/2] for swiglu."""
    in32 = np.ascontiguousarray(in32, dtype=np.float32)
    M, N = in32.shape
    No = N // 2 if act == ACT_SWIGLU else N
    out32 = np.empty((M, No), np.float32)
    outT = np.empty((M, No), np.uint16)
    lib().wo_activation(in32, M, N, act, dtype, out32, outT.ctypes.data)
    return out32, outT


def linear_fused(x_bits, pre_scale_bits, codes, scale, bias_bits, dtype, bits, group_size=-1, act=ACT_NONE):
    """apply_per_channel_scale (when pre_scale_bits is given), weight_only_linear
    and the activation, as the fused entry point composes them."""
    if pre_scale_bits is not None:
        x_bits = apply_per_channel_scale(x_bits, pre_scale_bits, dtype)
    o32, _ = linear(x_bits, codes, scale, bias_bits, dtype, bits, group_size)
    return activation(o32, act, dtype)


def linear_grad(out_grad_bits, codes, scale, dtype, bits, group_size=-1, acc64=False):
    """x_grad [M,K] = out_grad [M,N] . dequant(W)[K,N]^T with the fp32 dequantised
    weight.  Returns (fp32, T-bits)."""
    g = np.ascontiguousarray(out_grad_bits, dtype=np.uint16)
    codes = np.ascontiguousarray(codes, dtype=np.int8)
    scale = np.ascontiguousarray(scale, dtype=np.uint16)
    M, N = g.shape
    K = codes.shape[0]
    out32 = np.empty((M, K), np.float32)
    outT = np.empty((M, K), np.uint16)
    lib().wo_linear_grad(g, codes, scale, M, K, N, dtype, bits, group_size, 0, 1 if acc64 else 0, out32,
                         outT.ctypes.data)
    return out32, outT


def linear_grad_rounded_weight(out_grad_bits, codes, scale, dtype, bits, group_size=-1, acc64=False):
    """The reference's composition of the same gradient: the dequantised weight
    rounded to T (weight_dequantize), then the product with fp32 sums.  Returns
    (fp32, T-bits)."""
    g = np.ascontiguousarray(out_grad_bits, dtype=np.uint16)
    codes = np.ascontiguousarray(codes, dtype=np.int8)
    scale = np.ascontiguousarray(scale, dtype=np.uint16)
    M, N = g.shape
    K = codes.shape[0]
    out32 = np.empty((M, K), np.float32)
    outT = np.empty((M, K), np.uint16)
    lib().wo_linear_grad_rounded_weight(g, codes, scale, M, K, N, dtype, bits, group_size, 0, 1 if acc64 else 0,
                                        out32, outT.ctypes.data)
    return out32, outT


def ref_casts(flavour):
    """Load oracle/_ref/libref_casts_<flavour>.so (plain | f16c | hipflavour), or None."""
    path = os.path.join(_HERE, "_ref", "libref_casts_%s.so" % flavour)
    if not os.path.exists(path):
        return None
    L = ctypes.CDLL(path)
    L.ref_f32_to_bf16_array.argtypes = [_f32p, _i64, _u16p]
    if flavour != "hipflavour":
        L.ref_f32_to_f16_array.argtypes = [_f32p, _i64, _u16p]
        L.ref_f16_to_f32_array.argtypes = [_u16p, _i64, _f32p]
    return L
