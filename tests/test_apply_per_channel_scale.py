"""apply_per_channel_scale: the oracle against library half-precision multiplies
and exactness cases (CPU), and the HIP kernel against the oracle, bit for bit,
through the C ABI (GPU).  The reference's own test
(test/quantization/test_apply_per_channel_scale.py:52-110) compares with
paddle.multiply on rows x cols = 32 x 128 ... 64 x 4096 inputs drawn from
U(0, 1); those shapes are among the cases here."""
import numpy as np
import pytest

import helpers as H

REF_TEST_SHAPES = [(32, 128), (16, 128), (64, 4096), (1, 4096)]  # the reference's test matrix
SHAPES = REF_TEST_SHAPES + [(1, 8), (3, 40), (7, 1000), (5, 13), (9, 2051), (2048, 4096), (17, 11008)]


def _inputs(rows, cols, dt, seed, dist="uniform"):
    rng = np.random.default_rng(seed)
    if dist == "uniform":
        x = rng.random((rows, cols), dtype=np.float32)
        s = rng.random(cols, dtype=np.float32)
    else:  # wide dynamic range, both signs, results that round, overflow and underflow
        x = rng.standard_normal((rows, cols), dtype=np.float32) * np.exp2(rng.integers(-14, 14, (rows, cols))).astype(np.float32)
        s = rng.standard_normal(cols, dtype=np.float32) * np.exp2(rng.integers(-8, 8, cols)).astype(np.float32)
    return H.f32_to_bits(x, dt), H.f32_to_bits(s, dt)


def _library_multiply(xb, sb, dt):
    """x * s in T by a library: numpy's float16 multiply, torch's bfloat16 multiply."""
    import torch

    if dt == H.F16:
        return (xb.view(np.float16) * sb.view(np.float16)[None, :]).view(np.uint16)
    x = H.bits_to_torch(xb, dt)
    s = H.bits_to_torch(sb, dt)
    return H.torch_to_bits(x * s[None, :])


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("dist", ["uniform", "wide"])
def test_oracle_matches_library_half_multiplies(oracle, dt, dist):
    for i, (rows, cols) in enumerate([(32, 128), (5, 13), (64, 4096)]):
        xb, sb = _inputs(rows, cols, dt, 100 + i, dist)
        with np.errstate(over="ignore"):
            want = _library_multiply(xb, sb, dt)
        got = oracle.apply_per_channel_scale(xb, sb, dt)
        finite = np.isfinite(H.bits_to_f32(want, dt))
        assert np.array_equal(got[finite], want[finite])
        assert np.array_equal(np.isnan(H.bits_to_f32(got, dt)), np.isnan(H.bits_to_f32(want, dt)))
        inf = np.isinf(H.bits_to_f32(want, dt))
        assert np.array_equal(got[inf], want[inf])


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
def test_oracle_exact_cases(oracle, dt):
    xb, _ = _inputs(6, 24, dt, 7, "wide")
    one = H.f32_to_bits(np.ones(24, np.float32), dt)
    assert np.array_equal(oracle.apply_per_channel_scale(xb, one, dt), xb)  # x * 1 = x
    # a power-of-two scale only moves the exponent: exact while the result stays normal
    x = (np.arange(1, 6 * 24 + 1, dtype=np.float32) / 8.0).reshape(6, 24)
    xb = H.f32_to_bits(x, dt)
    p = H.f32_to_bits(np.full(24, 0.25, np.float32), dt)
    assert np.array_equal(H.bits_to_f32(oracle.apply_per_channel_scale(xb, p, dt), dt), H.bits_to_f32(xb, dt) * 0.25)
    # a tie rounds to even: 1.5 * (1 + e) = 1.5 + 1.5 e lies exactly between 1.5 + e (odd
    # mantissa) and 1.5 + 2 e (even), e = the spacing of T at 1; 2.5 * (1 + e) = 2.5 + 2.5 e
    # lies between 2.5 + 2 e (mantissa 2^(m-2) + 1, odd) and 2.5 + 4 e: a quarter, not a tie
    m = 10 if dt == H.F16 else 7
    e = 2.0 ** -m
    xb1 = H.f32_to_bits(np.array([[1.5, -1.5]], np.float32), dt)
    sb1 = H.f32_to_bits(np.array([1 + e, 1 + e], np.float32), dt)
    got = H.bits_to_f32(oracle.apply_per_channel_scale(xb1, sb1, dt), dt)
    assert got[0, 0] == np.float32(1.5 + 2 * e) and got[0, 1] == np.float32(-1.5 - 2 * e)
    # 1.25 * (1 + e) = 1.25 + 1.25 e: below the midpoint, rounds down to 1.25 + e
    xb2 = H.f32_to_bits(np.array([[1.25]], np.float32), dt)
    got = H.bits_to_f32(oracle.apply_per_channel_scale(xb2, sb1[:1], dt), dt)
    assert got[0, 0] == np.float32(1.25 + e)


def test_python_api_argument_checks_without_gpu():
    import torch
    from paddle_amd.nn import quant as Q
    from paddle_amd.nn.quant.quantized_linear import apply_per_channel_scale_infer_meta as meta

    assert meta((32, 128), (128,)) == (32, 128)
    with pytest.raises(ValueError, match="rank of Input\\(x\\) must be 2"):
        meta((2, 32, 128), (128,))
    with pytest.raises(ValueError, match="rank of Input\\(scales\\) must be 1"):
        meta((32, 128), (1, 128))
    with pytest.raises(ValueError, match="second dim"):
        meta((32, 128), (64,))
    with pytest.raises(ValueError):  # float32 activations are outside the op's dtypes
        Q.apply_per_channel_scale(torch.zeros(4, 8), torch.zeros(8))
    with pytest.raises(RuntimeError, match="GPU"):  # no CPU kernel behind this build
        Q.apply_per_channel_scale(torch.zeros(4, 8, dtype=torch.float16), torch.zeros(8, dtype=torch.float16))


def test_c_abi_argument_errors():
    from paddle_amd import _lib

    f = _lib.lib.wol_apply_per_channel_scale
    assert f(None, None, 3, 4, 8, None, None) == 2  # dtype
    assert f(None, None, 0, -1, 8, None, None) == 5  # rows
    assert f(None, None, 0, 4, 0, None, None) == 5  # cols
    assert f(None, None, 0, 4, (1 << 24) + 1, None, None) == 5
    assert f(None, None, 0, 0, 8, None, None) == 0  # nothing to do
    assert f(None, None, 1, 4, 8, None, None) == 1  # null pointers


# --------------------------------------------------------------------------- GPU


def _gpu_call(xb, sb, dt, in_place=False, offset=0):
    import torch
    from paddle_amd import _lib

    rows, cols = xb.shape
    dev = "cuda:0"
    # offset (in elements) shifts the buffers off 16-byte alignment
    xbuf = torch.zeros(rows * cols + 8, dtype=torch.int16, device=dev)
    sbuf = torch.zeros(cols + 8, dtype=torch.int16, device=dev)
    obuf = torch.full((rows * cols + 16,), 0x5555, dtype=torch.int16, device=dev)
    xbuf[offset:offset + rows * cols] = torch.from_numpy(xb.view(np.int16).reshape(-1)).to(dev)
    sbuf[offset:offset + cols] = torch.from_numpy(sb.view(np.int16)).to(dev)
    x_ptr = xbuf.data_ptr() + 2 * offset
    o_ptr = x_ptr if in_place else obuf.data_ptr() + 2 * offset
    _lib.check(_lib.lib.wol_apply_per_channel_scale(x_ptr, sbuf.data_ptr() + 2 * offset, dt, rows, cols, o_ptr, None))
    torch.cuda.synchronize()
    src = xbuf if in_place else obuf
    out = src[offset:offset + rows * cols].cpu().numpy().view(np.uint16).reshape(rows, cols)
    if not in_place:  # nothing written outside the output
        rest = torch.cat([obuf[:offset], obuf[offset + rows * cols:]]).cpu().numpy()
        assert np.all(rest == 0x5555)
    return out


def _same_bits_or_both_nan(got, want, dt):
    g32, w32 = H.bits_to_f32(got, dt), H.bits_to_f32(want, dt)
    nan = np.isnan(w32)
    assert np.array_equal(np.isnan(g32), nan)
    assert np.array_equal(got[~nan], want[~nan])


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [H.F16, H.BF16])
def test_gpu_bit_exact_against_oracle(device, oracle, dt):
    for i, (rows, cols) in enumerate(SHAPES):
        for dist in ("uniform", "wide"):
            print("case", dt, rows, cols, dist, flush=True)
            xb, sb = _inputs(rows, cols, dt, 500 + i, dist)
            want = oracle.apply_per_channel_scale(xb, sb, dt)
            _same_bits_or_both_nan(_gpu_call(xb, sb, dt), want, dt)


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [H.F16, H.BF16])
def test_gpu_in_place_and_unaligned(device, oracle, dt):
    xb, sb = _inputs(11, 264, dt, 9, "wide")
    want = oracle.apply_per_channel_scale(xb, sb, dt)
    _same_bits_or_both_nan(_gpu_call(xb, sb, dt, in_place=True), want, dt)
    for off in (1, 3, 4):  # pointers off 16-byte alignment take the element-wise kernel
        print("offset", off, flush=True)
        _same_bits_or_both_nan(_gpu_call(xb, sb, dt, offset=off), want, dt)


@pytest.mark.gpu
def test_gpu_special_values(device, oracle):
    for dt in (H.F16, H.BF16):
        vals = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 65504.0, 6e-8, 1e-40, 3.0e38], np.float32)
        xb = H.f32_to_bits(np.tile(vals, (len(vals), 1)).T.copy(), dt)  # [11, 11]: every pair
        sb = H.f32_to_bits(vals, dt)
        want = oracle.apply_per_channel_scale(xb, sb, dt)
        _same_bits_or_both_nan(_gpu_call(xb, sb, dt), want, dt)


@pytest.mark.gpu
def test_python_api_feeds_weight_only_linear(device, oracle):
    """The op sits in front of weight_only_linear (AWQ-style smoothing)."""
    import torch
    from paddle_amd.nn import quant as Q

    dt = H.BF16
    K, N, M = 256, 64, 5
    xb, sb = _inputs(M, K, dt, 77)
    wb = H.make_weight(K, N, dt, seed=78)
    x = H.bits_to_torch(xb, dt, device)
    s = H.bits_to_torch(sb, dt, device)
    w = H.bits_to_torch(wb, dt, device)
    qw, qs = Q.weight_quantize(w, algo="weight_only_int4", group_size=64)
    xs = Q.apply_per_channel_scale(x, s)
    assert xs.dtype == x.dtype and tuple(xs.shape) == (M, K)
    want_xs = oracle.apply_per_channel_scale(xb, sb, dt)
    assert np.array_equal(H.torch_to_bits(xs), want_xs)
    out = Q.weight_only_linear(xs, qw, None, qs, "int4", None, 64)
    codes, scale = oracle.weight_quantize(wb, dt, 4, 64)
    o32, _ = oracle.linear(want_xs, codes, scale, None, dt, 4, 64)
    assert H.rel_l2(H.bits_to_f32(H.torch_to_bits(out), dt), o32) < 4e-3  # one bf16 rounding of the output
