"""Thin wrappers that call the C ABI (through paddle_amd._lib) on torch device
memory, for the GPU parity tests."""
import numpy as np
import torch

import helpers as H
from paddle_amd import _lib

DEV = "cuda:0"


def quantize(w_bits, dt, bits, g, layout=_lib.LAYOUT_GFX950, round_mode=_lib.ROUND_RNE):
    """Returns (codes as flat uint8 numpy, scale bits numpy) from wol_quantize."""
    w = H.bits_to_torch(w_bits, dt, DEV)
    K, N = w.shape
    codes = torch.full((K * N * bits // 8,), 0x55, dtype=torch.uint8, device=DEV)
    sshape = (N,) if g == -1 else ((K + g - 1) // g, N)
    scale = torch.zeros(sshape, dtype=w.dtype, device=DEV)
    wsb = _lib.lib.wol_quantize_workspace(K, N, bits, g)
    ws = torch.full((max(wsb, 16),), 0xAB, dtype=torch.uint8, device=DEV)  # dirty on purpose
    _lib.check(_lib.lib.wol_quantize(w.data_ptr(), dt, K, N, bits, g, round_mode, layout, codes.data_ptr(),
                                     scale.data_ptr(), ws.data_ptr(), wsb, None))
    torch.cuda.synchronize()
    return codes.cpu().numpy(), H.torch_to_bits(scale)


def dequantize(codes_u8, layout, scale_bits, dt, K, N, bits, g):
    c = torch.from_numpy(np.ascontiguousarray(codes_u8)).to(DEV)
    s = H.bits_to_torch(scale_bits, dt, DEV)
    out = torch.zeros((K, N), dtype=s.dtype, device=DEV)
    _lib.check(_lib.lib.wol_dequantize(c.data_ptr(), layout, s.data_ptr(), dt, K, N, bits, g, out.data_ptr(), None))
    torch.cuda.synchronize()
    return H.torch_to_bits(out)


def repack(codes_u8, layout_in, layout_out, K, N, bits):
    c = torch.from_numpy(np.ascontiguousarray(codes_u8)).to(DEV)
    o = torch.full_like(c, 0x33)
    _lib.check(_lib.lib.wol_repack(c.data_ptr(), layout_in, o.data_ptr(), layout_out, K, N, bits, None))
    torch.cuda.synchronize()
    return o.cpu().numpy()


def quantize_llm_int8(w_bits, dt, g, layout=1):
    """algo="llm.int8" through the C ABI: (codes uint8 in `layout`, fp32 scale)."""
    w = H.bits_to_torch(w_bits, dt, DEV)
    K, N = w.shape
    codes = torch.zeros(K * N, dtype=torch.uint8, device=DEV)
    scale = torch.zeros((N,) if g == -1 else ((K + g - 1) // g, N), dtype=torch.float32, device=DEV)
    wsb = _lib.lib.wol_quantize_workspace(K, N, 8, g)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device=DEV)
    _lib.check(_lib.lib.wol_quantize_llm_int8(w.data_ptr(), dt, K, N, g, layout, codes.data_ptr(), scale.data_ptr(),
                                              ws.data_ptr(), wsb, None))
    torch.cuda.synchronize()
    return codes.cpu().numpy(), scale.cpu().numpy()


def linear(x_bits, codes_u8, bias_bits, scale_bits, dt, N, bits, g, f32=False, no_workspace=False,
           kernel=None, ws_bytes=None):
    """codes_u8 in gfx950 layout.  Returns fp32 numpy [M,N] (f32=True) or T bits.
    kernel pins a wol_kernel (streaming 1, GEMM 2, batched 3, batched with K
    runs 4) through wol_linear_on;
    ws_bytes overrides the size of the scratch buffer handed in."""
    x = H.bits_to_torch(x_bits, dt, DEV)
    c = torch.from_numpy(np.ascontiguousarray(codes_u8)).to(DEV)
    s = H.bits_to_torch(scale_bits, dt, DEV)
    b = None if bias_bits is None else H.bits_to_torch(bias_bits, dt, DEV)
    out = linear_dev(x, c, b, s, dt, N, bits, g, f32=f32, no_workspace=no_workspace, kernel=kernel, ws_bytes=ws_bytes)
    return out.cpu().numpy() if f32 else H.torch_to_bits(out)


def linear_dev(x, c, b, s, dt, N, bits, g, f32=False, no_workspace=False, kernel=None, ws_bytes=None):
    """The same on tensors that already live on the device; returns the output tensor."""
    M, K = x.shape
    out = torch.full((M, N), float("nan"), dtype=torch.float32 if f32 else x.dtype, device=DEV)
    if kernel is None:
        wsb = _lib.lib.wol_linear_workspace(M, K, N, bits, g)
    else:
        wsb = _lib.lib.wol_linear_workspace_for(M, K, N, bits, g, kernel)
    if no_workspace:
        wsb = 0
    if ws_bytes is not None:
        wsb = ws_bytes
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device=DEV) if wsb else None
    args = (x.data_ptr(), c.data_ptr(), None if b is None else b.data_ptr(), s.data_ptr(), dt, M, K, N, bits, g,
            out.data_ptr())
    tail = (None if ws is None else ws.data_ptr(), wsb, None)
    if kernel is None:
        fn = _lib.lib.wol_linear_f32 if f32 else _lib.lib.wol_linear
        _lib.check(fn(*args, *tail))
    else:
        _lib.check(_lib.lib.wol_linear_on(*args, 1 if f32 else 0, kernel, *tail))
    torch.cuda.synchronize()
    return out


def linear_plan(M, K, N, bits, g, ws_bytes):
    """What wol_linear would launch for the problem, given ws_bytes of scratch."""
    import ctypes

    buf = ctypes.create_string_buffer(512)
    _lib.check(_lib.lib.wol_linear_plan(M, K, N, bits, g, ws_bytes, buf, 512))
    return buf.value.decode()


def llm_int8_linear(x_bits, w_nk, bias_bits, wscale, threshold, dt, stages=False):
    """wol_llm_int8_linear through the C ABI.  w_nk [N,K] int8, wscale [N] float32.
    Returns the output's T bits, and with stages=True also a dict of the
    intermediate results left in the workspace."""
    import ctypes

    x = H.bits_to_torch(x_bits, dt, DEV)
    M, K = x.shape
    w = torch.from_numpy(np.ascontiguousarray(w_nk, dtype=np.int8)).to(DEV)
    N = w.shape[0]
    s = torch.from_numpy(np.ascontiguousarray(wscale, dtype=np.float32)).to(DEV)
    b = None if bias_bits is None else H.bits_to_torch(bias_bits, dt, DEV)
    out = torch.full((M, N), float("nan"), dtype=x.dtype, device=DEV)
    wsb = _lib.lib.wol_llm_int8_linear_workspace(M, K, N)
    ws = torch.full((wsb,), 0xA5, dtype=torch.uint8, device=DEV)  # dirty on purpose
    _lib.check(_lib.lib.wol_llm_int8_linear(x.data_ptr(), w.data_ptr(), None if b is None else b.data_ptr(),
                                            s.data_ptr(), float(threshold), dt, M, K, N, out.data_ptr(),
                                            ws.data_ptr(), wsb, None))
    torch.cuda.synchronize()
    if not stages:
        return H.torch_to_bits(out)
    offs = (ctypes.c_int64 * 7)()
    _lib.check(_lib.lib.wol_llm_int8_linear_stage_offsets(M, K, N, offs))
    raw = ws.cpu().numpy()
    count = int(raw[offs[2]:offs[2] + 4].view(np.int32)[0])
    mask_words = raw[offs[1]:offs[1] + K // 32 * 4].view(np.uint32)
    st = {
        "ranges": raw[offs[0]:offs[0] + 4 * M].view(np.float32).copy(),
        "outlier": ((mask_words[:, None] >> np.arange(32, dtype=np.uint32)[None, :]) & 1).astype(bool).reshape(-1),
        "count": count,
        "list": raw[offs[3]:offs[3] + 4 * count].view(np.int32).copy(),
        "qx": raw[offs[4]:offs[4] + M * K].view(np.int8).reshape(M, K).copy(),
        "acc": None if offs[5] < 0 else
        raw[offs[5]:offs[5] + 4 * M * N * offs[6]].view(np.int32).reshape(offs[6], M, N).sum(axis=0, dtype=np.int32),
        "runs": int(offs[6]),
    }
    return H.torch_to_bits(out), st
