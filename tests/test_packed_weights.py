"""Quantised weights at rest: conversion between the gfx950 layout and the
layout a ROCm build of the reference stores
(paddle/phi/kernels/cpu/weight_quantize_kernel.cc:113-125), and the tagged
safetensors files built on it."""
import json

import numpy as np
import pytest
import torch

import helpers as H
from paddle_amd.nn.quant import packed_weights as PW


def test_argument_checks_without_gpu(tmp_path):
    w = torch.zeros(16, 64, dtype=torch.int8)
    with pytest.raises(ValueError, match="unknown layout"):
        PW.convert_weight_layout(w, "int8", "gfx950", "cutlass")
    with pytest.raises(ValueError, match="weight_dtype"):
        PW.convert_weight_layout(w, "int2", "gfx950", "paddle_hip")
    with pytest.raises(ValueError, match="2-D int8"):
        PW.convert_weight_layout(w.float(), "int8", "gfx950", "paddle_hip")
    with pytest.raises(RuntimeError, match="GPU"):
        PW.convert_weight_layout(w, "int8", "gfx950", "paddle_hip")
    with pytest.raises(ValueError, match="'paddle_hip' or 'gfx950'"):
        PW.save_quantized(str(tmp_path / "a.safetensors"), {"w": w}, {"w": "int8"}, layout="canonical")
    with pytest.raises(KeyError):
        PW.save_quantized(str(tmp_path / "a.safetensors"), {"w": w}, {"v": "int8"}, layout="gfx950")


def test_gfx950_files_carry_the_layout_version(tmp_path):
    # no conversion needed for the gfx950 layout, so this runs without a GPU
    from safetensors import safe_open
    from safetensors.torch import save_file
    from paddle_amd import _lib

    w = torch.arange(16 * 64, dtype=torch.int32).to(torch.int8).reshape(16, 64)
    s = torch.ones(16, dtype=torch.float16)
    p = str(tmp_path / "g.safetensors")
    PW.save_quantized(p, {"l.w": w, "l.s": s}, {"l.w": "int8"}, layout="gfx950")
    with safe_open(p, framework="pt") as f:
        meta = json.loads(f.metadata()["wol_weight_only"])
    assert meta == {"layout": "gfx950", "quantized": {"l.w": "int8"}, "layout_version": _lib.lib.wol_layout_version()}
    got, q = PW.load_quantized(p, "cpu")
    assert q == {"l.w": "int8"} and torch.equal(got["l.w"], w) and torch.equal(got["l.s"], s)
    with pytest.raises(ValueError, match="names other quantised weights"):
        PW.load_quantized(p, "cpu", quantized={"l.s": "int8"})
    # another layout version is refused, not misread
    meta["layout_version"] += 1
    save_file({"l.w": w, "l.s": s}, p, metadata={"wol_weight_only": json.dumps(meta)})
    with pytest.raises(ValueError, match="layout version"):
        PW.load_quantized(p, "cpu")


@pytest.mark.gpu
@pytest.mark.parametrize("bits", [8, 4])
def test_conversions_match_the_layout_definitions(device, oracle, bits):
    dt = H.F16
    K, N = 320, 96  # int4: ends in a half tile
    wb = H.make_weight(K, N, dt, seed=3)
    codes, _ = oracle.weight_quantize(wb, dt, bits, 64)
    q = H.q_from_canonical(codes, bits)
    wd = "int8" if bits == 8 else "int4"
    rows = N * bits // 8
    gfx = torch.from_numpy(H.gfx950_from_q(q, bits).view(np.int8).reshape(rows, K)).to(device)
    hip = PW.convert_weight_layout(gfx, wd, "gfx950", "paddle_hip")
    assert tuple(hip.shape) == (rows, K)
    assert np.array_equal(hip.cpu().numpy(), H.paddle_hip_from_q(q, bits))
    can = PW.convert_weight_layout(hip, wd, "paddle_hip", "canonical")
    assert tuple(can.shape) == (K, rows)
    assert np.array_equal(can.cpu().numpy(), H.canonical_from_q(q, bits))
    back = PW.convert_weight_layout(can, wd, "canonical", "gfx950")
    assert torch.equal(back, gfx)


@pytest.mark.gpu
@pytest.mark.parametrize("algo,g", [("weight_only_int8", -1), ("weight_only_int4", 128)])
def test_checkpoint_round_trip_and_reference_files(device, oracle, tmp_path, algo, g):
    from safetensors.torch import save_file
    from paddle_amd.nn import quant as Q

    dt = H.BF16
    K, N, M = 256, 64, 3
    wb = H.make_weight(K, N, dt, seed=8)
    w = H.bits_to_torch(wb, dt, device)
    qw, qs = Q.weight_quantize(w, algo=algo, group_size=g)
    wd = "int8" if algo == "weight_only_int8" else "int4"
    bits = 8 if wd == "int8" else 4
    x = H.bits_to_torch(H.make_act(M, K, dt, seed=9), dt, device)
    want = Q.weight_only_linear(x, qw, None, qs, wd, None, g)
    p = str(tmp_path / "c.safetensors")
    PW.save_quantized(p, {"fc.weight": qw, "fc.scale": qs}, {"fc.weight": wd})
    got, qmap = PW.load_quantized(p, device)
    assert qmap == {"fc.weight": wd}
    assert torch.equal(got["fc.weight"], qw) and torch.equal(got["fc.scale"], qs)
    assert torch.equal(Q.weight_only_linear(x, got["fc.weight"], None, got["fc.scale"], wd, None, g), want)
    # a file as a ROCm build of the reference would write it: its layout, no tag
    codes, scale = oracle.weight_quantize(wb, dt, bits, g)
    hip = H.paddle_hip_from_q(H.q_from_canonical(codes, bits), bits)
    p2 = str(tmp_path / "ref.safetensors")
    save_file({"fc.weight": torch.from_numpy(hip.copy()), "fc.scale": H.bits_to_torch(scale, dt)}, p2)
    got2, _ = PW.load_quantized(p2, device, quantized={"fc.weight": wd})
    assert torch.equal(got2["fc.weight"], qw) and torch.equal(got2["fc.scale"], qs)
