"""Expert FFN of a mixture-of-experts layer on weight-only quantised experts:
the mirror of paddle.incubate.nn.functional.moe_ffn
(python/paddle/incubate/nn/functional/fused_moe.py:248-330 in the reference)
for quant_method "weight_only_int8" / "weight_only_int4"."""
import torch

from ... import _lib
from .quantized_linear import _dtype_id, _require_gpu, _stream_ptr, weight_quantize


def moe_quantize_experts(w, algo="weight_only_int8"):
    """w: [E, K, N] float16/bfloat16, one [K, N] weight per expert.  Returns
    (codes [E, N or N/2, K] int8 in the gfx950 layout, scales [E, N]) -- the
    per-expert outputs of weight_quantize stacked, which is what moe_ffn takes."""
    outs = [weight_quantize(w[e].contiguous(), algo=algo) for e in range(w.shape[0])]
    return torch.stack([o[0] for o in outs]), torch.stack([o[1] for o in outs])


def moe_ffn(permute_input, token_nums_per_expert, ffn1_weight, ffn2_weight, ffn1_bias=None, ffn1_scale=None,
            ffn2_scale=None, quant_method="weight_only_int8"):
    """permute_input [rows, hidden] (tokens in expert order), token_nums_per_expert
    [E] int64 as moe_dispatch returns it (the running total of rows up to and
    including each expert), ffn1_weight / ffn2_weight and their scales from
    moe_quantize_experts, ffn1_bias [E, 1, inter] or [E, inter] or None.
    Returns [rows, hidden]: swiglu(x . W1 + b1) . W2 per expert."""
    if quant_method not in ("weight_only_int8", "weight_only_int4"):
        raise ValueError("(InvalidArgument) quant_method must be weight_only_int8 or weight_only_int4 here, "
                         "but got %r" % (quant_method,))
    bits = 8 if quant_method == "weight_only_int8" else 4
    if ffn1_scale is None or ffn2_scale is None:
        raise ValueError("(InvalidArgument) ffn1_scale and ffn2_scale are required for %s" % quant_method)
    dt = _dtype_id(permute_input, "permute_input")
    _require_gpu(permute_input, "permute_input")
    if permute_input.dim() != 2:
        raise ValueError("(InvalidArgument) permute_input must be [rows, hidden]")
    if token_nums_per_expert.dtype != torch.int64:
        raise ValueError("(InvalidArgument) token_nums_per_expert must be int64")
    rows, hidden = int(permute_input.shape[0]), int(permute_input.shape[1])
    E = int(ffn1_weight.shape[0])
    inter = int(ffn1_scale.shape[-1])
    if tuple(ffn1_weight.shape) != (E, inter * bits // 8, hidden) or tuple(ffn2_weight.shape) != (E, hidden * bits // 8, inter // 2):
        raise ValueError("(InvalidArgument) expert weights must be [E, inter(/2), hidden] and [E, hidden(/2), inter/2] "
                         "as moe_quantize_experts returns them")
    if int(token_nums_per_expert.numel()) != E or tuple(ffn2_scale.shape) != (E, hidden):
        raise ValueError("(InvalidArgument) token_nums_per_expert / ffn2_scale do not match the %d experts" % E)
    for t in (ffn1_scale, ffn2_scale) + (() if ffn1_bias is None else (ffn1_bias,)):
        if t.dtype != permute_input.dtype:
            raise ValueError("(InvalidArgument) scales and bias must have permute_input's dtype")
    x = permute_input.contiguous()
    out = torch.empty_like(x)
    if rows == 0:
        return out
    b1 = None if ffn1_bias is None else ffn1_bias.reshape(E, inter).contiguous()
    ws_bytes = _lib.lib.wol_moe_ffn_workspace(rows, hidden, inter, E)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=x.device)
    w1, w2 = ffn1_weight.contiguous(), ffn2_weight.contiguous()
    s1, s2 = ffn1_scale.contiguous(), ffn2_scale.contiguous()
    cnt = token_nums_per_expert.contiguous()
    with torch.cuda.device(x.device):
        _lib.check(
            _lib.lib.wol_moe_ffn(
                x.data_ptr(), cnt.data_ptr(), w1.data_ptr(), None if b1 is None else b1.data_ptr(), s1.data_ptr(),
                w2.data_ptr(), s2.data_ptr(), dt, rows, hidden, inter, E, bits, out.data_ptr(), ws.data_ptr(),
                ws_bytes, _stream_ptr(x),
            )
        )
    return out
