"""Pins the CPU oracle (oracle/wo_oracle.c) without a GPU.

What pins what:
  casts          the committed vectors made from the reference's own
                 float16.h / bfloat16.h (tests/golden/cast_vectors.npz), the
                 same headers loaded directly when oracle/_ref is present, and
                 the known answers recorded from a run of those headers
  scales, codes  an independent numpy statement of max|w|/bound -> cast ->
                 divide -> round half away -> clip (helpers.np_quantize),
                 invariants of the closed form, and the known answers of the
                 reference for an all-zero column
  dequant/linear exact arithmetic in float64
"""
import os

import numpy as np
import pytest

import helpers as H

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "cast_vectors.npz")

SHAPES = [(64, 16), (64, 256), (128, 288), (192, 48), (320, 64)]
GROUPS = [-1, 64, 128]


# ------------------------------------------------------------------ casts
def test_casts_match_reference_header_vectors(oracle):
    g = np.load(GOLD)
    x = g["x"]
    for name, dt, mode in (("f16_rne", H.F16, oracle.CAST_RNE), ("f16_trunc", H.F16, oracle.CAST_TRUNC),
                           ("bf16_rne", H.BF16, oracle.CAST_RNE), ("bf16_trunc", H.BF16, oracle.CAST_TRUNC)):
        got = oracle.from_f32(x, dt, mode)
        assert np.array_equal(got, g[name]), name
    h = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    assert np.array_equal(oracle.to_f32(h, H.F16).view(np.uint32), g["f16_to_f32_bits"])


def test_casts_match_reference_headers_directly(oracle):
    plain, f16c, hipf = oracle.ref_casts("plain"), oracle.ref_casts("f16c"), oracle.ref_casts("hipflavour")
    if plain is None or f16c is None or hipf is None:
        pytest.skip("oracle/_ref not built here (needs the reference tree)")
    rng = np.random.default_rng(7)
    x = rng.integers(0, 2**32, 1 << 20, dtype=np.uint64).astype(np.uint32).view(np.float32)
    out = np.empty(x.size, np.uint16)
    for lib, fn, dt, mode in ((plain, "ref_f32_to_f16_array", H.F16, oracle.CAST_TRUNC),
                              (f16c, "ref_f32_to_f16_array", H.F16, oracle.CAST_RNE),
                              (plain, "ref_f32_to_bf16_array", H.BF16, oracle.CAST_RNE),
                              (hipf, "ref_f32_to_bf16_array", H.BF16, oracle.CAST_TRUNC)):
        getattr(lib, fn)(x, x.size, out)
        assert np.array_equal(out, oracle.from_f32(x, dt, mode)), fn


def test_cast_known_answers_from_reference_run(oracle):
    # float16(1 + 0.75 * 2^-10): 0x3c00 from a host build without F16C (truncation),
    # 0x3c01 with F16C; bfloat16(1 + 0.75 * 2^-7): 0x3f81 either way.
    v = np.array([1.0 + 0.75 * 2.0**-10], np.float32)
    assert oracle.from_f32(v, H.F16, oracle.CAST_TRUNC)[0] == 0x3C00
    assert oracle.from_f32(v, H.F16, oracle.CAST_RNE)[0] == 0x3C01
    b = np.array([1.0 + 0.75 * 2.0**-7], np.float32)
    assert oracle.from_f32(b, H.BF16, oracle.CAST_RNE)[0] == 0x3F81
    assert oracle.from_f32(b, H.BF16, oracle.CAST_TRUNC)[0] == 0x3F80


def test_rne_casts_against_numpy_and_torch(oracle):
    rng = np.random.default_rng(11)
    x = np.concatenate([rng.standard_normal(50000), rng.standard_normal(50000) * 1e-6,
                        rng.standard_normal(20000) * 7e4]).astype(np.float32)
    assert np.array_equal(oracle.from_f32(x, H.F16), H.f32_to_bits(x, H.F16))
    assert np.array_equal(oracle.from_f32(x, H.BF16), H.f32_to_bits(x, H.BF16))
    hb = rng.integers(0, 65536, 50000).astype(np.uint16)
    assert np.array_equal(oracle.to_f32(hb, H.BF16).view(np.uint32), H.bits_to_f32(hb, H.BF16).view(np.uint32))
    finite = (hb & 0x7C00) != 0x7C00
    assert np.array_equal(oracle.to_f32(hb, H.F16)[finite], H.bits_to_f32(hb, H.F16)[finite])


# ------------------------------------------------------- scales and codes
@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("g", GROUPS)
def test_quantize_matches_numpy_statement(oracle, dt, bits, g):
    for K, N in SHAPES:
        for wb in (H.make_weight(K, N, dt, seed=K * 7 + N), H.adversarial_weight(K, N, dt)):
            codes, scale = oracle.weight_quantize(wb, dt, bits, g)
            q, sb = H.np_quantize(wb, dt, bits, g)
            assert np.array_equal(scale, sb), (K, N)
            assert np.array_equal(H.q_from_canonical(codes, bits), q), (K, N)
            assert np.array_equal(codes, H.canonical_from_q(q, bits))


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("g", GROUPS)
def test_llm_int8_flavour_matches_numpy_statement(oracle, dt, g):
    # algo="llm.int8": fp32 scales (no cast), codes divided by them.  Beyond the
    # numpy statement: scale * 127 returns the column maximum to one fp32 ulp,
    # every non-degenerate group reaches |code| = 127, and the codes differ from
    # the T-scale flavour's only where the scale rounding moved a quotient
    # across a rounding boundary (never by more than one step).
    for K, N in SHAPES:
        wb = H.make_weight(K, N, dt, seed=K * 3 + N)
        codes, scale = oracle.weight_quantize_llm_int8(wb, dt, g)
        q, s = H.np_quantize_llm_int8(wb, dt, g)
        assert scale.dtype == np.float32 and np.array_equal(scale.view(np.uint32), s.view(np.uint32))
        assert np.array_equal(codes.astype(np.int32), q)
        w = H.bits_to_f32(wb, dt)
        gs = K if g == -1 else g
        amax = np.stack([np.abs(w[i:i + gs]).max(axis=0) for i in range(0, K, gs)])
        assert np.allclose(scale.reshape(amax.shape) * np.float32(127.0), amax, rtol=2e-7, atol=0)
        top = np.stack([np.abs(codes[i:i + gs].astype(np.int32)).max(axis=0) for i in range(0, K, gs)])
        assert (top[amax > 0] == 127).all()
        tcodes, _ = oracle.weight_quantize(wb, dt, 8, g)
        assert np.abs(codes.astype(np.int32) - tcodes.astype(np.int32)).max() <= 1
    adv = H.adversarial_weight(128, 64, dt)
    codes, scale = oracle.weight_quantize_llm_int8(adv, dt, g)
    q, s = H.np_quantize_llm_int8(adv, dt, g)
    assert np.array_equal(codes.astype(np.int32), q)
    assert np.array_equal(scale.view(np.uint32), s.view(np.uint32))


def test_zero_column_known_answers(oracle):
    # Recorded from the reference header: an all-zero column gives scale bits
    # 0x0000, int8 code 127 and int4 nibble 0x9 (-7), for fp16 and bf16.
    for dt in (H.F16, H.BF16):
        w = H.make_weight(64, 16, dt, seed=3)
        w[:, 4] = 0
        c8, s8 = oracle.weight_quantize(w, dt, 8, -1)
        assert s8[4] == 0 and np.all(c8[:, 4] == 127)
        c4, s4 = oracle.weight_quantize(w, dt, 4, -1)
        assert s4[4] == 0 and np.all((c4.view(np.uint8)[:, 2] & 0xF) == 0x9)
        # group-wise: same codes, and a column that is zero in one group only
        w2 = H.make_weight(128, 16, dt, seed=4)
        w2[:64, 5] = 0
        c, s = oracle.weight_quantize(w2, dt, 8, 64)
        assert s[0, 5] == 0 and np.all(c[:64, 5] == 127) and s[1, 5] != 0


def test_per_channel_first_element_rules(oracle):
    # The per-channel maximum starts from the signed first element
    # (impl/weight_quantize_kernel_impl.h:49): a column of zeros that starts
    # with -0 keeps the sign in its scale; group-wise starts from +0.
    for dt in (H.F16, H.BF16):
        w = H.make_weight(64, 16, dt, seed=5)
        w[:, 3] = 0
        w[0, 3] = 0x8000
        _, s = oracle.weight_quantize(w, dt, 8, -1)
        assert s[3] == 0x8000
        _, sg = oracle.weight_quantize(w, dt, 8, 64)
        assert sg[0, 3] == 0x0000


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("g", GROUPS)
def test_quantize_invariants(oracle, dt, bits, g):
    K, N = 256, 64
    wb = H.make_weight(K, N, dt, seed=99)
    codes, scale = oracle.weight_quantize(wb, dt, bits, g)
    q = H.q_from_canonical(codes, bits)
    bound = 127 if bits == 8 else 7
    assert np.abs(q).max() <= bound
    w = H.bits_to_f32(wb, dt).astype(np.float64)
    s = H.bits_to_f32(scale, dt).astype(np.float64)
    s_full = np.broadcast_to(s, (K, N)) if g == -1 else np.repeat(s, g, axis=0)[:K]
    assert (s_full >= 0).all()
    # every group of a Gaussian weight has a normal scale, hence reaches the bound
    gg = K if g == -1 else g
    for k0 in range(0, K, gg):
        assert (np.abs(q[k0:k0 + gg]).max(axis=0) == bound).all()
    # unclipped codes are the nearest integers: |w/s - q| <= 1/2 (plus one fp32 ulp of the quotient)
    r = w / s_full
    unclipped = np.abs(r) < bound
    assert (np.abs(r - q)[unclipped] <= 0.5 + 1e-5).all()
    # scale * bound is the abs-max up to the cast's rounding
    amax = np.abs(w).reshape(-1, gg, N).max(axis=1) if g != -1 else np.abs(w).max(axis=0)
    rel = 2.0**-8 if dt == H.BF16 else 2.0**-11
    assert np.allclose(s * bound, amax, rtol=rel * 1.01, atol=0)


def test_half_away_rounding_and_clip_after_round(oracle):
    # scale 1.0 exactly (abs-max 127): ties go away from zero; 126.5 rounds to 127
    dt = H.F16
    col = np.zeros(64, np.float32)
    col[:8] = [127.0, 0.5, -0.5, 1.5, -2.5, 126.5, -126.5, 0.49]
    w = np.zeros((64, 16), np.float32)
    w[:, 0] = col
    codes, scale = oracle.weight_quantize(H.f32_to_bits(w, dt), dt, 8, -1)
    assert H.bits_to_f32(scale, dt)[0] == 1.0
    assert list(codes[:8, 0]) == [127, 1, -1, 2, -3, 127, -127, 0]
    # int4: abs-max 7 -> scale 1.0; 6.5 -> 7, -7.0 stays, ties away
    col4 = np.zeros(64, np.float32)
    col4[:6] = [7.0, 6.5, -6.5, 0.5, -0.5, 2.5]
    w[:, 0] = col4
    c4, s4 = oracle.weight_quantize(H.f32_to_bits(w, dt), dt, 4, -1)
    q4 = H.q_from_canonical(c4, 4)
    assert list(q4[:6, 0]) == [7, 7, -7, 1, -1, 3]


def test_scale_rounded_down_clips_the_maximum(oracle):
    # bf16 truncation flavour rounds the scale down, so max|w| / scale exceeds
    # the bound and is clipped after rounding: codes stay in range.
    dt = H.BF16
    wb = H.make_weight(128, 32, dt, seed=21)
    codes, _ = oracle.weight_quantize(wb, dt, 8, -1, cast_mode=oracle.CAST_TRUNC)
    assert np.abs(codes.astype(np.int32)).max() == 127
    c4, _ = oracle.weight_quantize(wb, dt, 4, -1, cast_mode=oracle.CAST_TRUNC)
    assert np.abs(H.q_from_canonical(c4, 4)).max() == 7


def test_fp16_subnormal_scale_fixture(oracle):
    # 0.001 * U[0,1) weights (the reference's pass test) give int8 scales below
    # the fp16 normal range: the codes must follow the coarsely rounded scale.
    rng = np.random.default_rng(5)
    w = (rng.random((64, 32), dtype=np.float32) * np.float32(0.001))
    wb = H.f32_to_bits(w, H.F16)
    codes, scale = oracle.weight_quantize(wb, H.F16, 8, -1)
    assert ((scale & 0x7C00) == 0).all()  # all subnormal
    q, sb = H.np_quantize(wb, H.F16, 8, -1)
    assert np.array_equal(scale, sb) and np.array_equal(codes.astype(np.int32), q)


def test_int4_nibble_order_and_hip_flavour(oracle):
    dt = H.F16
    wb = H.make_weight(64, 32, dt, seed=8)
    codes, _ = oracle.weight_quantize(wb, dt, 4, -1)
    q = H.q_from_canonical(codes, 4)
    b = codes.view(np.uint8)
    assert np.array_equal(b & 0xF, q[:, 0::2] & 0xF)  # even column in the low nibble
    assert np.array_equal(b >> 4, q[:, 1::2] & 0xF)
    hip, _ = oracle.weight_quantize(wb, dt, 4, -1, nibble_bias=8)
    assert np.array_equal(hip.view(np.uint8) & 0xF, q[:, 0::2] + 8)
    assert np.array_equal(oracle.transpose_bytes(hip), np.ascontiguousarray(hip.T))
    assert np.array_equal(oracle.transpose_bytes(hip), H.paddle_hip_from_q(q, 4))


def test_ragged_last_group(oracle):
    # K = 192 with group 128: the second group has 64 rows (the reference's j+k<m guard)
    dt = H.BF16
    wb = H.make_weight(192, 16, dt, seed=12)
    codes, scale = oracle.weight_quantize(wb, dt, 8, 128)
    assert scale.shape == (2, 16)
    q, sb = H.np_quantize(wb, dt, 8, 128)
    assert np.array_equal(scale, sb) and np.array_equal(codes.astype(np.int32), q)


def test_contract_rejections(oracle):
    dt = H.F16
    with pytest.raises(ValueError):
        oracle.weight_quantize(np.zeros((32, 16), np.uint16), dt, 8, -1)
    with pytest.raises(ValueError):
        oracle.weight_quantize(np.zeros((64, 8), np.uint16), dt, 8, -1)
    with pytest.raises(ValueError):
        oracle.weight_quantize(np.zeros((64, 16), np.uint16), dt, 8, 32)


# ------------------------------------------------------ dequant and linear
@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("g", GROUPS)
def test_dequantize_is_exact_product(oracle, dt, bits, g):
    K, N = 192, 48
    wb = H.make_weight(K, N, dt, seed=31)
    codes, scale = oracle.weight_quantize(wb, dt, bits, g)
    d32, dT = oracle.dequantize(codes, scale, dt, bits, g)
    q = H.q_from_canonical(codes, bits).astype(np.float64)
    s = H.bits_to_f32(scale, dt).astype(np.float64)
    s_full = np.broadcast_to(s, (K, N)) if g == -1 else np.repeat(s, g, axis=0)[:K]
    assert np.array_equal(d32.astype(np.float64), q * s_full)  # <= 8 x 11 bits: exact in fp32
    assert np.array_equal(dT, H.f32_to_bits(d32, dt))
    # quantise -> dequantise stays within half a step of the input
    w = H.bits_to_f32(wb, dt).astype(np.float64)
    assert (np.abs(d32 - w) <= s_full * 0.5 * (1 + 2.0**-7) + 1e-12).all()


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("g", GROUPS)
def test_linear_against_float64_matmul(oracle, dt, bits, g):
    M, K, N = 5, 256, 64
    wb = H.make_weight(K, N, dt, seed=41)
    xb = H.make_act(M, K, dt, seed=42)
    bb = H.make_bias(N, dt, seed=43)
    codes, scale = oracle.weight_quantize(wb, dt, bits, g)
    d32, _ = oracle.dequantize(codes, scale, dt, bits, g)
    ref = H.bits_to_f32(xb, dt).astype(np.float64) @ d32.astype(np.float64) + H.bits_to_f32(bb, dt).astype(np.float64)
    o32, oT = oracle.linear(xb, codes, scale, bb, dt, bits, g)
    assert H.rel_l2(o32, ref) < 2e-6  # fp32 accumulation over K
    o64, _ = oracle.linear(xb, codes, scale, bb, dt, bits, g, acc64=True)
    assert np.array_equal(o64, ref.astype(np.float32))
    assert np.array_equal(oT, H.f32_to_bits(o32, dt))
    # no bias; one-hot x returns a dequantised row; zero x returns the bias
    o_nb, _ = oracle.linear(xb, codes, scale, None, dt, bits, g)
    assert H.rel_l2(o_nb, ref - H.bits_to_f32(bb, dt)) < 2e-6
    onehot = np.zeros((1, K), np.float32)
    onehot[0, 77] = 1.0
    o1, _ = oracle.linear(H.f32_to_bits(onehot, dt), codes, scale, None, dt, bits, g)
    assert np.array_equal(o1[0], d32[77])
    oz, _ = oracle.linear(H.f32_to_bits(np.zeros((2, K), np.float32), dt), codes, scale, bb, dt, bits, g)
    assert np.array_equal(oz[0], H.bits_to_f32(bb, dt))
