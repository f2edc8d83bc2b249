"""Layouts of quantised weights at rest.

weight_quantize of this package returns codes in the gfx950 streaming layout,
which only this library reads.  A checkpoint that should outlive the library
version, or come from / go to a stock ROCm build of the reference, holds the
codes in the layout that build produces instead: the plain transpose [N, K]
for int8 and [N/2, K] nibble pairs (+8) for int4
(paddle/phi/kernels/cpu/weight_quantize_kernel.cc:113-125 under
PADDLE_WITH_HIP).  Both have the shape WeightQuantizeInferMeta gives, so only
a tag tells them apart: files written here carry the layout name and, for the
gfx950 layout, its version in their safetensors metadata; a file without the
tag is taken to come from the reference.

The conversion is wol_repack, a permutation on the device.
"""
import json

import torch

from ... import _lib

LAYOUTS = {"canonical": _lib.LAYOUT_CANONICAL, "paddle_hip": _lib.LAYOUT_PADDLE_HIP,
           "gfx950": _lib.LAYOUT_GFX950}
_META_KEY = "wol_weight_only"


def _bits(weight_dtype):
    if weight_dtype == "int8":
        return 8
    if weight_dtype == "int4":
        return 4
    raise ValueError("(InvalidArgument) weight_dtype must be 'int8' or 'int4', but got %r" % (weight_dtype,))


def convert_weight_layout(weight, weight_dtype, src, dst):
    """Re-lays a quantised weight ([N, K] int8, or [N/2, K] for int4) from
    layout `src` to layout `dst` ("gfx950", "paddle_hip" or "canonical"; the
    canonical layout is the reference's code matrix [K, N] / [K, N/2] before
    any layout step, and is returned with that shape)."""
    if src not in LAYOUTS or dst not in LAYOUTS:
        raise ValueError("(InvalidArgument) unknown layout %r -> %r; expected one of %s"
                         % (src, dst, sorted(LAYOUTS)))
    bits = _bits(weight_dtype)
    if weight.dtype != torch.int8 or weight.dim() != 2:
        raise ValueError("(InvalidArgument) a quantised weight is a 2-D int8 tensor")
    if not weight.is_cuda:
        raise RuntimeError("the weight must live on the GPU: the conversion is a device kernel")
    if src == "canonical":
        K, N = weight.shape[0], weight.shape[1] * (8 // bits)
    else:
        K, N = weight.shape[1], weight.shape[0] * (8 // bits)
    out_shape = (K, N * bits // 8) if dst == "canonical" else (N * bits // 8, K)
    weight = weight.contiguous()
    out = torch.empty(out_shape, dtype=torch.int8, device=weight.device)
    with torch.cuda.device(weight.device):
        _lib.check(_lib.lib.wol_repack(weight.data_ptr(), LAYOUTS[src], out.data_ptr(), LAYOUTS[dst],
                                       K, N, bits, torch.cuda.current_stream(weight.device).cuda_stream))
    return out


def save_quantized(path, tensors, quantized, layout="paddle_hip"):
    """Writes `tensors` (name -> tensor) as one safetensors file.  `quantized`
    maps the names of quantised weights (held in the gfx950 layout, as
    weight_quantize returns them) to their weight_dtype; they are stored in
    `layout`.  Everything else is stored as it is."""
    from safetensors.torch import save_file

    if layout not in ("paddle_hip", "gfx950"):
        raise ValueError("(InvalidArgument) checkpoints hold 'paddle_hip' or 'gfx950' weights, not %r" % (layout,))
    out = {}
    for name, t in tensors.items():
        if name in quantized and layout != "gfx950":
            t = convert_weight_layout(t, quantized[name], "gfx950", layout)
        out[name] = t.detach().cpu().contiguous()
    for name in quantized:
        if name not in tensors:
            raise KeyError(name)
        _bits(quantized[name])
    meta = {"layout": layout, "quantized": dict(quantized)}
    if layout == "gfx950":
        meta["layout_version"] = int(_lib.lib.wol_layout_version())
    save_file(out, path, metadata={_META_KEY: json.dumps(meta)})


def load_quantized(path, device, quantized=None):
    """Reads a file written by save_quantized, or by the reference (no tag: pass
    `quantized`, name -> weight_dtype, and the weights are taken to be in the
    layout of its ROCm build).  Returns (tensors on `device` with the quantised
    weights in the gfx950 layout, the name -> weight_dtype map)."""
    from safetensors import safe_open

    tensors = {}
    with safe_open(path, framework="pt", device="cpu") as f:
        raw = (f.metadata() or {}).get(_META_KEY)
        for name in f.keys():
            tensors[name] = f.get_tensor(name)
    if raw is None:
        meta = {"layout": "paddle_hip", "quantized": dict(quantized or {})}
    else:
        meta = json.loads(raw)
        if quantized is not None and dict(quantized) != meta["quantized"]:
            raise ValueError("(InvalidArgument) the file names other quantised weights than the caller: %r"
                             % (meta["quantized"],))
    layout = meta["layout"]
    if layout == "gfx950" and int(meta.get("layout_version", -1)) != int(_lib.lib.wol_layout_version()):
        raise ValueError(
            "(InvalidArgument) the file holds gfx950 layout version %s, this library reads version %d; "
            "store checkpoints in the 'paddle_hip' layout to carry them across versions"
            % (meta.get("layout_version"), _lib.lib.wol_layout_version()))
    out = {}
    for name, t in tensors.items():
        t = t.to(device)
        if name in meta["quantized"] and layout != "gfx950":
            t = convert_weight_layout(t, meta["quantized"][name], layout, "gfx950")
        out[name] = t
    return out, meta["quantized"]
