"""weight_quantize / weight_dequantize / weight_only_linear /
apply_per_channel_scale with the signatures, defaults, checks and error
behaviour of paddle.nn.quant (python/paddle/nn/quant/quantized_linear.py:64-282
and :351-388 in the reference), computed by the gfx950 library through its C
ABI.

Tensors are torch tensors on the GPU; torch only provides the memory and the
stream.  The shape checks restate the reference's InferMeta functions and raise
ValueError where Paddle raises InvalidArgument; the group-size checks are
asserts, as in the reference's Python.
"""
import torch

from ... import _lib

_ALGOS = ("weight_only_int8", "weight_only_int4", "llm.int8")


def _get_arch_info():
    """The reference probes the CUDA SM version here (quantized_linear.py:45-61)
    and only validates it in CUDA builds; on AMD any value is accepted and it
    selects nothing, so report the gfx950 generation number."""
    return 95


def _dtype_id(t, what):
    if t.dtype == torch.float16:
        return _lib.DTYPE_F16
    if t.dtype == torch.bfloat16:
        return _lib.DTYPE_BF16
    raise ValueError(
        "(InvalidArgument) %s must be float16 or bfloat16, but got %s" % (what, t.dtype)
    )


def _stream_ptr(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def _require_gpu(t, what):
    if not t.is_cuda:
        raise RuntimeError(
            "%s must live on the GPU: this build has no CPU kernels (the compute is "
            "libwol_gfx950.so)" % what
        )


def _check_group_size(group_size, op):
    assert (
        group_size == -1 or group_size == 64 or group_size == 128
    ), f"Currently {op} only support group size of -1, 64 or 128. but got {group_size} "


def _algo_bits(algo):
    if algo == "weight_only_int8":
        return 8
    if algo == "weight_only_int4":
        return 4
    if algo == "llm.int8":
        return 8
    raise ValueError(
        "(InvalidArgument) The algo must be in ['weight_only_int8', 'weight_only_int4', "
        "'llm.int8'], but got[%s]" % algo
    )


def weight_quantize_infer_meta(x_shape, algo, group_size):
    """WeightQuantizeInferMeta (paddle/phi/infermeta/unary.cc:5946-6011):
    returns (out_shape, scale_shape)."""
    if len(x_shape) != 2:
        raise ValueError(
            "(InvalidArgument) The x tensor of quant op must be 2D, but got[%d]" % len(x_shape)
        )
    K, N = int(x_shape[0]), int(x_shape[1])
    if K % 64 != 0:
        raise ValueError(
            "(InvalidArgument) The first dimension of input must be divisible by 64, but got[%d]" % K
        )
    if N % 16 != 0:
        raise ValueError(
            "(InvalidArgument) The second dimension of input must be divisible by 16, but got[%d]" % N
        )
    if group_size not in (-1, 64, 128):
        raise ValueError("(InvalidArgument) Currently, group_size only support -1, 64 or 128.")
    scale_shape = [N] if group_size == -1 else [(K + group_size - 1) // group_size, N]
    if algo in ("weight_only_int8", "llm.int8"):
        out_shape = [N, K]
    elif algo == "weight_only_int4":
        out_shape = [N // 2, K]
    else:
        raise ValueError(
            "(InvalidArgument) The algo must be in ['weight_only_int8', 'weight_only_int4', "
            "'llm.int8'], but got[%s]" % algo
        )
    return out_shape, scale_shape


def weight_dequantize_infer_meta(x_shape, scale_shape, algo, group_size):
    """WeightDequantizeInferMeta (paddle/phi/infermeta/binary.cc:4499-4570):
    returns the output shape [K, N]."""
    if len(x_shape) != 2:
        raise ValueError(
            "(InvalidArgument) The x tensor of dequantize op must be 2D, but got[%d]" % len(x_shape)
        )
    if group_size not in (-1, 64, 128):
        raise ValueError("(InvalidArgument) group_size must be -1, 64 or 128.")
    if algo == "weight_only_int8":
        channels = int(x_shape[0])
    elif algo == "weight_only_int4":
        channels = int(x_shape[0]) * 2
    else:
        raise ValueError(
            "(InvalidArgument) Currently, we only support weight_only_int8 and weight_only_int4 algo."
        )
    K = int(x_shape[1])
    if group_size == -1:
        if len(scale_shape) != 1:
            raise ValueError(
                "(InvalidArgument) The scale tensor of dequantize op must be 1D in per-channel "
                "mode, but got[%d]" % len(scale_shape)
            )
        if int(scale_shape[0]) != channels:
            raise ValueError(
                "(InvalidArgument) The scale tensor's shape must be equal to the x tensor's "
                "shape, but got [%d] not equal to [%d]" % (scale_shape[0], x_shape[0])
            )
    else:
        if len(scale_shape) != 2:
            raise ValueError(
                "(InvalidArgument) The scale tensor of dequantize op must be 2D in group-wise "
                "mode, but got[%d]" % len(scale_shape)
            )
        want = (K + group_size - 1) // group_size
        if int(scale_shape[0]) != want:
            raise ValueError(
                "(InvalidArgument) The input(weight_scale) dim[0] must be equal to "
                "(Input(weight).dim[1] + (group_size -1)) / group_size But receive %d and %d"
                % (scale_shape[0], want)
            )
        if int(scale_shape[1]) != channels:
            raise ValueError(
                "(InvalidArgument) The scale tensor's shape must be equal to the real channel "
                "size, but got [%d] not equal to [%d]" % (scale_shape[0], channels)
            )
    return [K, channels]


def weight_only_linear_infer_meta(x_shape, w_shape, bias_shape, scale_shape, weight_dtype, group_size):
    """WeightOnlyLinearInferMeta (paddle/phi/infermeta/multiary.cc:5495-5575):
    returns (out_shape, n)."""
    if group_size not in (-1, 64, 128):
        raise ValueError("(InvalidArgument) group_size must be -1, 64 or 128.")
    if weight_dtype not in ("int8", "int4"):
        raise ValueError("(InvalidArgument) quant_method must be 'int8' or 'int4'.")
    if len(w_shape) != 2:
        raise ValueError("(InvalidArgument) The input(weight) must be a 2D Tensor.")
    if int(w_shape[0]) % 16 != 0:
        raise ValueError(
            "(InvalidArgument) The first dimension of input must be divisible by 16, but got[%d]"
            % w_shape[0]
        )
    if int(w_shape[1]) % 16 != 0:
        raise ValueError(
            "(InvalidArgument) The second dimension of input must be divisible by 16, but got[%d]"
            % w_shape[1]
        )
    if int(x_shape[-1]) != int(w_shape[1]):
        raise ValueError(
            "(InvalidArgument) Input(X) dim[-1] and Input(Weight) dim[1] should be equal."
            "But received Input(X) dim[-1](%s) != Input(Weight) dim[1](%s)" % (x_shape[-1], w_shape[1])
        )
    if bias_shape is not None and len(bias_shape) != 1:
        raise ValueError(
            "(InvalidArgument) The size of Input(Bias)'s dimension should equal to 1UL."
        )
    if group_size == -1:
        if len(scale_shape) != 1:
            raise ValueError(
                "(InvalidArgument) The input(weight_scale) must be a 1D Tensor.in per-channel mode."
            )
        n = int(scale_shape[0])
    else:
        if len(scale_shape) != 2:
            raise ValueError(
                "(InvalidArgument) The input(weight_scale) must be a 2D Tensor in groupwise mode."
            )
        want = (int(w_shape[1]) + group_size - 1) // group_size
        if int(scale_shape[0]) != want:
            raise ValueError(
                "(InvalidArgument) The input(weight_scale) dim[0] must be equal to Input(weight) "
                "dim[1] / group_size But receive %d and %d" % (scale_shape[0], want)
            )
        n = int(scale_shape[1])
    return list(x_shape[:-1]) + [n], n


def weight_quantize(x, algo="weight_only_int8", arch=None, group_size=-1):
    """Quantise a [K, N] float16/bfloat16 weight.

    Returns (out, scale): out is int8 with the reference's shape, [N, K] for
    int8 and [N/2, K] for int4, holding the codes in the gfx950 streaming
    layout; scale is [N] or [ceil(K/group_size), N] in x's dtype.  Codes and
    scales equal the reference's CPU kernel bit for bit (before its own layout
    step).  arch is accepted and ignored, as in a ROCm build of the reference.

    algo="llm.int8" (the input of llm_int8_linear, not of weight_only_linear)
    keeps the scale in float32 and returns the codes as the reference does for
    that algo: plain int8 [N, K], the transpose of the code matrix.
    """
    if arch is None:
        arch = _get_arch_info()
    assert (
        group_size == -1 or group_size == 64 or group_size == 128
    ), f"Currently group_size only support -1/64/128. but got {group_size} "
    out_shape, scale_shape = weight_quantize_infer_meta(tuple(x.shape), algo, group_size)
    bits = _algo_bits(algo)
    dt = _dtype_id(x, "x")
    _require_gpu(x, "x")
    x = x.contiguous()
    K, N = x.shape
    out = torch.empty(out_shape, dtype=torch.int8, device=x.device)
    ws_bytes = _lib.lib.wol_quantize_workspace(K, N, bits, group_size)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=x.device)
    if algo == "llm.int8":
        scale = torch.empty(scale_shape, dtype=torch.float32, device=x.device)
        with torch.cuda.device(x.device):
            _lib.check(
                _lib.lib.wol_quantize_llm_int8(
                    x.data_ptr(), dt, K, N, group_size, _lib.LAYOUT_PADDLE_HIP, out.data_ptr(),
                    scale.data_ptr(), ws.data_ptr(), ws_bytes, _stream_ptr(x),
                )
            )
        return out, scale
    scale = torch.empty(scale_shape, dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(
            _lib.lib.wol_quantize(
                x.data_ptr(), dt, K, N, bits, group_size, _lib.ROUND_RNE, _lib.LAYOUT_GFX950,
                out.data_ptr(), scale.data_ptr(), ws.data_ptr(), ws_bytes, _stream_ptr(x),
            )
        )
    return out, scale


def weight_dequantize(x, scale, algo="weight_only_int8", out_dtype="float16", group_size=-1):
    """Dequantise a weight made by weight_quantize back to [K, N] out_dtype."""
    assert (
        group_size == -1 or group_size == 64 or group_size == 128
    ), f"Currently group_size only support -1/64/128. but got {group_size} "
    names = {"float16": torch.float16, "bfloat16": torch.bfloat16,
             torch.float16: torch.float16, torch.bfloat16: torch.bfloat16}
    if out_dtype not in names:
        raise TypeError(
            "The data type of 'out_dtype' in weight_dequantize must be ['float16', 'bfloat16'], "
            "but received %s." % (out_dtype,)
        )
    tdtype = names[out_dtype]
    out_shape = weight_dequantize_infer_meta(tuple(x.shape), tuple(scale.shape), algo, group_size)
    bits = _algo_bits(algo)
    _require_gpu(x, "x")
    if x.dtype != torch.int8:
        raise ValueError("(InvalidArgument) x must be int8, but got %s" % x.dtype)
    if scale.dtype != tdtype:
        raise ValueError(
            "(InvalidArgument) scale dtype %s does not match out_dtype %s" % (scale.dtype, tdtype)
        )
    x = x.contiguous()
    scale = scale.contiguous()
    K, N = out_shape
    out = torch.empty(out_shape, dtype=tdtype, device=x.device)
    dt = _lib.DTYPE_F16 if tdtype == torch.float16 else _lib.DTYPE_BF16
    with torch.cuda.device(x.device):
        _lib.check(
            _lib.lib.wol_dequantize(
                x.data_ptr(), _lib.LAYOUT_GFX950, scale.data_ptr(), dt, K, N, bits, group_size,
                out.data_ptr(), _stream_ptr(x),
            )
        )
    return out


def _linear_call(fn, x, weight, bias, weight_scale, weight_dtype, group_size, out_dtype):
    out_shape, N = weight_only_linear_infer_meta(
        tuple(x.shape), tuple(weight.shape), None if bias is None else tuple(bias.shape),
        tuple(weight_scale.shape), weight_dtype, group_size,
    )
    dt = _dtype_id(x, "x")
    _require_gpu(x, "x")
    if weight.dtype != torch.int8:
        raise ValueError("(InvalidArgument) weight must be int8, but got %s" % weight.dtype)
    if weight_scale.dtype != x.dtype or (bias is not None and bias.dtype != x.dtype):
        raise ValueError("(InvalidArgument) weight_scale and bias must have x's dtype")
    bits = 8 if weight_dtype == "int8" else 4
    K = int(weight.shape[1])
    if int(weight.shape[0]) * 8 // bits != N:
        raise ValueError(
            "(InvalidArgument) weight rows (%d) do not match the %d output channels of "
            "weight_scale" % (weight.shape[0], N)
        )
    if bias is not None and int(bias.shape[0]) != N:
        raise ValueError("(InvalidArgument) bias must have %d elements" % N)
    x = x.contiguous()
    weight = weight.contiguous()
    weight_scale = weight_scale.contiguous()
    bias = None if bias is None else bias.contiguous()
    M = x.numel() // K
    out = torch.empty(out_shape, dtype=out_dtype or x.dtype, device=x.device)
    ws_bytes = _lib.lib.wol_linear_workspace(M, K, N, bits, group_size)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
    with torch.cuda.device(x.device):
        _lib.check(
            fn(
                x.data_ptr(), weight.data_ptr(), None if bias is None else bias.data_ptr(),
                weight_scale.data_ptr(), dt, M, K, N, bits, group_size, out.data_ptr(),
                None if ws is None else ws.data_ptr(), ws_bytes, _stream_ptr(x),
            )
        )
    return out


def weight_only_linear_grad(x, weight, bias, weight_scale, out_grad, weight_dtype="int8", arch=None,
                            group_size=-1):
    """x_grad of weight_only_linear, the op's only gradient
    (paddle/phi/kernels/gpu/weight_only_linear_grad_kernel.cu:27-72,
    backward.yaml:3651-3661): x_grad[M,K] = out_grad[M,N] . dequant(W)[K,N]^T.
    The reference dequantises the weight to T and calls a library GEMM, for
    per-channel scales and arch 80/86 only; here wol_linear_grad contracts over
    n straight from the packed codes, for every group size, without rounding
    code * scale to T.  x is only used for its shape (no_need_buffer in the
    reference's backward.yaml); bias gets no gradient and is ignored."""
    if weight_dtype not in ("int8", "int4"):
        raise ValueError("(InvalidArgument) weight_dtype must be 'int8' or 'int4', but got %r" % (weight_dtype,))
    _check_group_size(group_size, "weight_only_linear_grad")
    _require_gpu(out_grad, "out_grad")
    _require_gpu(weight, "weight")
    dt = _dtype_id(out_grad, "out_grad")
    bits = 8 if weight_dtype == "int8" else 4
    N = out_grad.shape[-1]
    K = x.shape[-1]
    if weight_scale.dtype != out_grad.dtype:
        raise ValueError("(InvalidArgument) weight_scale and out_grad must have the same dtype")
    g2 = out_grad.reshape(-1, N).contiguous()
    M = g2.shape[0]
    out = torch.empty((M, K), dtype=out_grad.dtype, device=out_grad.device)
    if M:
        with torch.cuda.device(out_grad.device):
            ws_bytes = _lib.lib.wol_linear_grad_workspace(M, K, N, bits, group_size)
            ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=out_grad.device)
            _lib.check(
                _lib.lib.wol_linear_grad(
                    g2.data_ptr(), weight.data_ptr(), weight_scale.data_ptr(), dt, M, K, N, bits,
                    group_size, out.data_ptr(), ws.data_ptr(), ws_bytes, _stream_ptr(out_grad),
                )
            )
    return out.reshape(tuple(x.shape))


class _WeightOnlyLinearFn(torch.autograd.Function):
    """weight_only_linear with the reference's backward (x_grad only: the
    quantised weight, its scale and the bias get no gradient, backward.yaml:3651-3661)."""

    @staticmethod
    def forward(ctx, x, weight, bias, weight_scale, weight_dtype, group_size):
        ctx.save_for_backward(weight, weight_scale)
        ctx.meta = (weight_dtype, group_size, x.shape)
        return _linear_call(_lib.lib.wol_linear, x, weight, bias, weight_scale, weight_dtype,
                            group_size, None)

    @staticmethod
    def backward(ctx, out_grad):
        weight, weight_scale = ctx.saved_tensors
        weight_dtype, group_size, x_shape = ctx.meta
        x_like = torch.empty(x_shape, dtype=out_grad.dtype, device="meta")
        gx = weight_only_linear_grad(x_like, weight, None, weight_scale, out_grad.contiguous(),
                                     weight_dtype, None, group_size)
        return gx, None, None, None, None, None


def weight_only_linear(x, weight, bias=None, weight_scale=None, weight_dtype="int8", arch=None,
                       group_size=-1):
    """out = x . dequant(weight) + bias, in x's dtype (fp32 accumulation, one
    final rounding).  weight / weight_scale are the outputs of weight_quantize;
    leading dimensions of x are flattened into M."""
    if arch is None:
        arch = _get_arch_info()
    assert (
        group_size == -1 or group_size == 64 or group_size == 128
    ), f"Currently weight_quantize only support group size of -1, 64 or 128. but got {group_size} "
    if weight_scale is None:
        raise ValueError("(InvalidArgument) weight_scale is required")
    if x.requires_grad and torch.is_grad_enabled():
        return _WeightOnlyLinearFn.apply(x, weight, bias, weight_scale, weight_dtype, group_size)
    return _linear_call(_lib.lib.wol_linear, x, weight, bias, weight_scale, weight_dtype,
                        group_size, None)


_ACTS = {None: 0, "none": 0, "None": 0, "gelu": 1, "swiglu": 2}


def weight_only_linear_fused(x, weight, bias=None, weight_scale=None, weight_dtype="int8", group_size=-1,
                             pre_scale=None, act="none"):
    """weight_only_linear with its neighbours folded in: apply_per_channel_scale
    in front (pre_scale: [K] in x's dtype, each product rounded to x's dtype as
    that op rounds it) and an activation behind, applied to the fp32 sums before
    the one rounding: act "none", "gelu" (the tanh form of the reference's GEMV
    epilogue, act_method in paddle/phi/kernels/funcs/weight_only_gemv.h:33) or
    "swiglu" (silu of the first half of the output columns times the second
    half: the result has N/2 columns).  No counterpart in the reference's Python
    API, which composes these from separate ops."""
    assert (
        group_size == -1 or group_size == 64 or group_size == 128
    ), f"Currently weight_quantize only support group size of -1, 64 or 128. but got {group_size} "
    if act not in _ACTS:
        raise ValueError("(InvalidArgument) act must be 'none', 'gelu' or 'swiglu', but got %r" % (act,))
    if weight_scale is None:
        raise ValueError("(InvalidArgument) weight_scale is required")
    out_shape, N = weight_only_linear_infer_meta(
        tuple(x.shape), tuple(weight.shape), None if bias is None else tuple(bias.shape),
        tuple(weight_scale.shape), weight_dtype, group_size,
    )
    dt = _dtype_id(x, "x")
    _require_gpu(x, "x")
    if weight.dtype != torch.int8:
        raise ValueError("(InvalidArgument) weight must be int8, but got %s" % weight.dtype)
    if weight_scale.dtype != x.dtype or (bias is not None and bias.dtype != x.dtype):
        raise ValueError("(InvalidArgument) weight_scale and bias must have x's dtype")
    bits = 8 if weight_dtype == "int8" else 4
    K = int(weight.shape[1])
    if pre_scale is not None and (pre_scale.dtype != x.dtype or tuple(pre_scale.shape) != (K,)):
        raise ValueError("(InvalidArgument) pre_scale must be [%d] in x's dtype" % K)
    a = _ACTS[act]
    if a == 2:
        if N % 32 != 0:
            raise ValueError("(InvalidArgument) swiglu needs an even number of 16-column strips")
        out_shape = tuple(out_shape[:-1]) + (N // 2,)
    x = x.contiguous()
    weight = weight.contiguous()
    weight_scale = weight_scale.contiguous()
    bias = None if bias is None else bias.contiguous()
    pre_scale = None if pre_scale is None else pre_scale.contiguous()
    M = x.numel() // K
    out = torch.empty(out_shape, dtype=x.dtype, device=x.device)
    if M == 0:
        return out
    ws_bytes = _lib.lib.wol_linear_fused_workspace(M, K, N, bits, group_size, 0 if pre_scale is None else 1, a)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
    with torch.cuda.device(x.device):
        _lib.check(
            _lib.lib.wol_linear_fused(
                x.data_ptr(), None if pre_scale is None else pre_scale.data_ptr(), weight.data_ptr(),
                None if bias is None else bias.data_ptr(), weight_scale.data_ptr(), dt, M, K, N, bits,
                group_size, a, out.data_ptr(), None if ws is None else ws.data_ptr(), ws_bytes, _stream_ptr(x),
            )
        )
    return out


def weight_only_linear_fp32(x, weight, bias=None, weight_scale=None, weight_dtype="int8",
                            group_size=-1):
    """weight_only_linear without the final cast: returns the fp32 accumulators
    (plus bias).  Not part of the reference API; it exists so the arithmetic
    can be checked apart from the output rounding."""
    return _linear_call(_lib.lib.wol_linear_f32, x, weight, bias, weight_scale, weight_dtype,
                        group_size, torch.float32)


def apply_per_channel_scale_infer_meta(x_shape, scales_shape):
    """ApplyPerChannelScaleInferMeta (paddle/phi/infermeta/binary.cc:3452-3481):
    x is 2-D, scales 1-D with x's second dimension; out has x's shape."""
    if len(x_shape) != 2:
        raise ValueError(
            "(InvalidArgument) The rank of Input(x) must be 2, but received %d." % len(x_shape)
        )
    if len(scales_shape) != 1:
        raise ValueError(
            "(InvalidArgument) The rank of Input(scales) must be 1, but received %d."
            % len(scales_shape)
        )
    if x_shape[1] != scales_shape[0]:
        raise ValueError(
            "(InvalidArgument) The second dim of Input(x) must be equal to the first dim of scales,"
            "but received %d and %d." % (x_shape[1], scales_shape[0])
        )
    return tuple(x_shape)


def apply_per_channel_scale(x, scales):
    """Apply pre-quant per channel scale on activations: out = x * scales, in
    x's dtype (python/paddle/nn/quant/quantized_linear.py:351-388)."""
    out_shape = apply_per_channel_scale_infer_meta(tuple(x.shape), tuple(scales.shape))
    dt = _dtype_id(x, "x")
    if scales.dtype != x.dtype:
        raise ValueError(
            "(InvalidArgument) scales dtype %s does not match x dtype %s" % (scales.dtype, x.dtype)
        )
    _require_gpu(x, "x")
    _require_gpu(scales, "scales")
    x = x.contiguous()
    scales = scales.contiguous()
    out = torch.empty(out_shape, dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(
            _lib.lib.wol_apply_per_channel_scale(
                x.data_ptr(), scales.data_ptr(), dt, out_shape[0], out_shape[1], out.data_ptr(),
                _stream_ptr(x),
            )
        )
    return out


def llm_int8_linear_infer_meta(x_shape, w_shape, bias_shape, scale_shape):
    """LLMInt8LinearInferMeta (paddle/phi/infermeta/multiary.cc:3792-3837):
    returns the output shape."""
    if len(w_shape) != 2:
        raise ValueError("(InvalidArgument) The input(weight) must be a 2D Tensor.")
    if x_shape[-1] != w_shape[1]:
        raise ValueError(
            "(InvalidArgument) Input(X) dim[-1] and Input(Weight) dim[1] should be equal."
            "But received Input(X) dim[-1](%s) != Input(Weight) dim[1](%s)" % (x_shape[-1], w_shape[1])
        )
    if w_shape[0] % 16 != 0:
        raise ValueError(
            "(InvalidArgument) The first dimension of input must be divisible by 16, but got[%d]" % w_shape[0]
        )
    if w_shape[1] % 16 != 0:
        raise ValueError(
            "(InvalidArgument) The second dimension of input must be divisible by 16, but got[%d]" % w_shape[1]
        )
    if scale_shape[0] != w_shape[0]:
        raise ValueError(
            "(InvalidArgument) Input(weight_scale) dim[0] and Input(Weight) dim[0] should be equal."
            "But received Input(weight_scale) dim[0](%s) != Input(Weight) dim[0](%s)" % (scale_shape[0], w_shape[0])
        )
    return tuple(x_shape[:-1]) + (w_shape[0],)


def llm_int8_linear(x, weight, bias=None, weight_scale=None, threshold=6.0):
    """paddle.nn.quant.llm_int8_linear (python/paddle/nn/quant/quantized_linear.py:285-349
    in the reference): x [..., K] float16/bfloat16, weight [N, K] int8 and
    weight_scale [N] float32 as weight_quantize(algo="llm.int8") returns them,
    bias [N] in x's dtype or None.  Columns of x holding an element above
    threshold are multiplied in x's dtype with the dequantised weight, the
    rest as int8 x int8 with a per-row dynamic scale.  The weight must have K
    divisible by 64 (what weight_quantize accepts), not only by 16."""
    out_shape = llm_int8_linear_infer_meta(
        tuple(x.shape), tuple(weight.shape), None if bias is None else tuple(bias.shape),
        tuple(weight_scale.shape),
    )
    dt = _dtype_id(x, "x")
    _require_gpu(x, "x")
    if weight.dtype != torch.int8:
        raise ValueError("(InvalidArgument) weight must be int8, but got %s" % weight.dtype)
    if weight_scale.dtype != torch.float32:
        raise ValueError("(InvalidArgument) weight_scale must be float32, but got %s" % weight_scale.dtype)
    if bias is not None and bias.dtype != x.dtype:
        raise ValueError("(InvalidArgument) bias must have x's dtype")
    N, K = int(weight.shape[0]), int(weight.shape[1])
    if bias is not None and int(bias.shape[0]) != N:
        raise ValueError("(InvalidArgument) bias must have %d elements" % N)
    x = x.contiguous()
    weight = weight.contiguous()
    weight_scale = weight_scale.contiguous()
    bias = None if bias is None else bias.contiguous()
    M = x.numel() // K
    out = torch.empty(out_shape, dtype=x.dtype, device=x.device)
    if M == 0:
        return out
    ws_bytes = _lib.lib.wol_llm_int8_linear_workspace(M, K, N)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(
            _lib.lib.wol_llm_int8_linear(
                x.data_ptr(), weight.data_ptr(), None if bias is None else bias.data_ptr(),
                weight_scale.data_ptr(), float(threshold), dt, M, K, N, out.data_ptr(), ws.data_ptr(),
                ws_bytes, _stream_ptr(x),
            )
        )
    return out
