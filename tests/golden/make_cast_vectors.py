"""Writes tests/golden/cast_vectors.npz: float32 inputs and the bit patterns
the reference's own float16.h / bfloat16.h produce for them, in each build
flavour.  Runs only where the reference tree is mounted: it loads oracle/_ref
(the reference headers compiled by oracle/Makefile), never the oracle itself.

    python tests/golden/make_cast_vectors.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import wo_oracle as O  # noqa: E402  (only for locating / loading oracle/_ref)


def inputs():
    rng = np.random.default_rng(20240607)
    parts = [
        rng.standard_normal(4096).astype(np.float32),
        (rng.standard_normal(2048) * 1e-4).astype(np.float32),
        (rng.standard_normal(2048) * 1e-7).astype(np.float32),  # fp16 subnormal range
        (rng.standard_normal(1024) * 3e4).astype(np.float32),   # near the fp16 maximum
        rng.integers(0, 2**32, 4096, dtype=np.uint64).astype(np.uint32).view(np.float32),
    ]
    # halfway cases between neighbouring fp16 / bf16 values, and their neighbours
    h = rng.integers(0x0001, 0x7BFF, 1024).astype(np.uint16)
    lo = h.view(np.float16).astype(np.float32)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float32)
    mid = ((lo.astype(np.float64) + hi.astype(np.float64)) / 2).astype(np.float32)
    parts += [mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(np.inf)), -mid]
    b = rng.integers(0x0001, 0x7F7F, 1024).astype(np.uint32)
    blo = (b << 16).view(np.float32)
    bmid = ((b << 16) | 0x8000).astype(np.uint32).view(np.float32)
    parts += [bmid, np.nextafter(bmid, np.float32(0)), np.nextafter(bmid, np.float32(np.inf)), -bmid, blo]
    special = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 65504.0, 65519.99, 65520.0, 65536.0, 1e38,
                        2.0**-14, 2.0**-24, 2.0**-25, 2.0**-26, 1.0 + 0.75 * 2.0**-10, 1.0 + 0.75 * 2.0**-7,
                        5.9604645e-08, 6.0975552e-05, 3.4028235e38, 1e-45], dtype=np.float32)
    parts.append(special)
    return np.concatenate(parts).astype(np.float32)


def main():
    x = inputs()
    n = x.size
    out = {"x": x}
    plain, f16c, hipf = O.ref_casts("plain"), O.ref_casts("f16c"), O.ref_casts("hipflavour")
    if plain is None or f16c is None or hipf is None:
        raise SystemExit("oracle/_ref is not built (needs the reference tree): make -C oracle")
    for name, lib, fn in (("f16_trunc", plain, "ref_f32_to_f16_array"), ("f16_rne", f16c, "ref_f32_to_f16_array"),
                          ("bf16_rne", plain, "ref_f32_to_bf16_array"), ("bf16_trunc", hipf, "ref_f32_to_bf16_array")):
        o = np.empty(n, np.uint16)
        getattr(lib, fn)(x, n, o)
        out[name] = o
    h = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    w = np.empty(65536, np.float32)
    plain.ref_f16_to_f32_array(h, 65536, w)
    out["f16_to_f32_bits"] = w.view(np.uint32)
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "cast_vectors.npz"), **out)
    print("wrote cast_vectors.npz:", n, "inputs")


if __name__ == "__main__":
    main()
