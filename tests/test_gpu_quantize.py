"""GPU parity of weight_quantize / weight_dequantize / repack against the CPU
oracle, through the C ABI.  Codes and scales must be bit-exact."""
import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu

SHAPES = [(64, 16), (64, 256), (128, 288), (192, 48), (320, 1040), (512, 1024)]


@pytest.fixture(scope="module")
def G(device):
    import gpu_calls

    return gpu_calls


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("g", [-1, 64, 128])
def test_quantize_bit_exact_all_layouts(G, oracle, dt, bits, g):
    for K, N in SHAPES:
        for adv in (False, True):
            print("case", dt, bits, g, K, N, adv, flush=True)
            wb = H.adversarial_weight(K, N, dt) if adv else H.make_weight(K, N, dt, seed=K + N)
            oc, osc = oracle.weight_quantize(wb, dt, bits, g)
            q = H.q_from_canonical(oc, bits)
            gc, gs = G.quantize(wb, dt, bits, g, layout=0)
            assert np.array_equal(gs, osc)
            assert np.array_equal(gc.view(np.int8).reshape(oc.shape), oc)
            gp, gs2 = G.quantize(wb, dt, bits, g, layout=2)
            assert np.array_equal(gs2, osc)
            assert np.array_equal(gp, H.gfx950_from_q(q, bits))
            gh, _ = G.quantize(wb, dt, bits, g, layout=1)
            assert np.array_equal(gh, H.paddle_hip_from_q(q, bits).view(np.uint8).reshape(-1))


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("g", [-1, 64, 128])
def test_quantize_llm_int8_flavour_bit_exact(G, oracle, dt, g):
    # algo="llm.int8": fp32 scales, codes as the plain [N,K] transpose (what the
    # reference returns for it) and in the other two layouts
    for K, N in SHAPES:
        for adv in (False, True):
            wb = H.adversarial_weight(K, N, dt) if adv else H.make_weight(K, N, dt, seed=K + N)
            oc, osc = oracle.weight_quantize_llm_int8(wb, dt, g)
            gh, gs = G.quantize_llm_int8(wb, dt, g, layout=1)
            assert np.array_equal(gs.view(np.uint32), osc.view(np.uint32))
            assert np.array_equal(gh.view(np.int8).reshape(N, K), oc.T)
            gc, _ = G.quantize_llm_int8(wb, dt, g, layout=0)
            assert np.array_equal(gc.view(np.int8).reshape(K, N), oc)
            gp, _ = G.quantize_llm_int8(wb, dt, g, layout=2)
            assert np.array_equal(gp, H.gfx950_from_q(oc.astype(np.int32), 8))


def test_python_api_llm_int8(device, oracle):
    import torch
    from paddle_amd.nn import quant as Q

    wb = H.make_weight(256, 64, H.F16, seed=5)
    w = H.bits_to_torch(wb, H.F16, torch.device("cuda:0"))
    out, scale = Q.weight_quantize(w, algo="llm.int8")
    oc, osc = oracle.weight_quantize_llm_int8(wb, H.F16, -1)
    assert out.dtype == torch.int8 and tuple(out.shape) == (64, 256) and scale.dtype == torch.float32
    assert np.array_equal(out.cpu().numpy(), oc.T)
    assert np.array_equal(scale.cpu().numpy().view(np.uint32), osc.view(np.uint32))
    with pytest.raises(ValueError):  # weight_dequantize refuses llm.int8 (binary.cc:4521-4525)
        Q.weight_dequantize(out, scale.half(), algo="llm.int8")


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("bits", [8, 4])
def test_quantize_truncating_scale_flavour(G, oracle, dt, bits):
    K, N = 256, 128
    for g in (-1, 128):
        for wb in (H.make_weight(K, N, dt, seed=3), H.adversarial_weight(K, N, dt)):
            oc, osc = oracle.weight_quantize(wb, dt, bits, g, cast_mode=oracle.CAST_TRUNC)
            gc, gs = G.quantize(wb, dt, bits, g, layout=0, round_mode=1)
            assert np.array_equal(gs, osc)
            assert np.array_equal(gc.view(np.int8).reshape(oc.shape), oc)


@pytest.mark.parametrize("bits", [8, 4])
def test_quantize_nan_and_inf_inputs(G, oracle, bits):
    # NaN never wins a maximum (unless it is the first element of a per-channel
    # column); infinities give an infinite scale and zero / NaN quotients.
    dt = H.BF16
    K, N = 128, 32
    wb = H.make_weight(K, N, dt, seed=17)
    wb[5, 2] = 0x7FC0   # NaN inside a column
    wb[0, 3] = 0x7FC0   # NaN as first element
    wb[70, 4] = 0x7F80  # +inf
    wb[9, 5] = 0xFF80   # -inf
    for g in (-1, 64):
        oc, osc = oracle.weight_quantize(wb, dt, bits, g)
        gc, gs = G.quantize(wb, dt, bits, g, layout=0)
        assert np.array_equal(gs, osc)
        assert np.array_equal(gc.view(np.int8).reshape(oc.shape), oc)


def _near_tie_weight(dt, bits, K, N, seed):
    """Columns whose quotients w / scale sit on and right next to the rounding
    boundaries k + 0.5 (every k up to the bound, both signs, and the neighbours
    one unit in the last place of T either side), under scales that span the
    exponent range of T: where a quantiser that multiplies by a reciprocal
    instead of dividing would go wrong first."""
    rng = np.random.default_rng(seed)
    bound = 127 if bits == 8 else 7
    lo_e, hi_e = (-12, 14) if dt == H.F16 else (-110, 110)
    wb = np.zeros((K, N), np.uint16)
    for c in range(N):
        amax = np.float32(rng.uniform(1.0, 2.0) * 2.0 ** int(rng.integers(lo_e, hi_e)))
        a_bits = H.f32_to_bits(np.array([amax], np.float32), dt)[0]
        a_val = H.bits_to_f32(np.array([a_bits], np.uint16), dt)[0]
        s_val = H.bits_to_f32(H.f32_to_bits(np.array([a_val / np.float32(bound)], np.float32), dt), dt)[0]
        ks = rng.integers(0, bound, K).astype(np.float32) + np.float32(0.5)
        sign = np.where(rng.integers(0, 2, K) == 0, np.float32(1), np.float32(-1))
        col = H.f32_to_bits((ks * s_val * sign).astype(np.float32), dt).astype(np.int32)
        col += rng.integers(-1, 2, K)  # the value itself or a neighbour in T
        col = col.astype(np.uint16)
        col[int(rng.integers(K))] = a_bits  # the column maximum that fixes the scale
        if c % 7 == 0:  # the maximum in every 64-row group, so group-wise scales match too
            col[::64] = a_bits
        wb[:, c] = col
    return wb


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("bits", [8, 4])
def test_quantize_near_rounding_boundaries(G, oracle, dt, bits):
    K, N = 512, 128
    for seed, g in ((1, -1), (2, 64), (3, 128), (4, -1)):
        print("case", dt, bits, g, seed, flush=True)
        wb = _near_tie_weight(dt, bits, K, N, seed)
        oc, osc = oracle.weight_quantize(wb, dt, bits, g)
        gc, gs = G.quantize(wb, dt, bits, g, layout=0)
        assert np.array_equal(gs, osc)
        got = gc.view(np.int8).reshape(oc.shape)
        assert np.array_equal(got, oc), np.argwhere(got != oc)[:5]
    # the construction does what it says: hundreds of quotients are exact ties
    # (the rest lie within a few units in the last place of T of one)
    w32 = H.bits_to_f32(wb, dt)
    s32 = H.bits_to_f32(osc, dt)
    frac = np.abs(np.abs(w32 / s32[None, :]) % 1.0 - 0.5)
    assert (frac == 0).sum() > 300, (frac == 0).sum()


@pytest.mark.parametrize("bits", [8, 4])
def test_repack_round_trips(G, bits):
    rng = np.random.default_rng(bits)
    bound = 127 if bits == 8 else 7
    for K, N in [(64, 16), (192, 48), (320, 1040)]:
        q = rng.integers(-bound, bound + 1, (K, N)).astype(np.int32)
        forms = {0: H.canonical_from_q(q, bits).view(np.uint8).reshape(-1),
                 1: H.paddle_hip_from_q(q, bits).view(np.uint8).reshape(-1),
                 2: H.gfx950_from_q(q, bits)}
        for a in (0, 1, 2):
            for b in (0, 1, 2):
                got = G.repack(forms[a], a, b, K, N, bits)
                assert np.array_equal(got, forms[b]), (K, N, a, b)


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("g", [-1, 64, 128])
def test_dequantize_bit_exact(G, oracle, dt, bits, g):
    for K, N in SHAPES:
        wb = H.make_weight(K, N, dt, seed=K + 3 * N)
        oc, osc = oracle.weight_quantize(wb, dt, bits, g)
        _, oT = oracle.dequantize(oc, osc, dt, bits, g)
        q = H.q_from_canonical(oc, bits)
        for layout, codes in ((0, oc.view(np.uint8).reshape(-1)), (1, H.paddle_hip_from_q(q, bits).view(np.uint8).reshape(-1)),
                              (2, H.gfx950_from_q(q, bits))):
            got = G.dequantize(codes, layout, osc, dt, K, N, bits, g)
            assert np.array_equal(got, oT), (K, N, layout)


def test_quantize_dequantize_round_trip_full_size(G):
    # the reference's own round-trip check (test_weight_only_linear.py:675-706)
    # at its size, 4096 x 12288: |dequant(quant(w)) - w| <= scale / 2 everywhere
    import torch

    from paddle_amd.nn import quant as Q

    for dt, tdt in ((H.F16, torch.float16), (H.BF16, torch.bfloat16)):
        gen = torch.Generator(device="cuda").manual_seed(5)
        w = (torch.randn(4096, 12288, device="cuda", generator=gen) * 0.02).to(tdt)
        for algo, bound, g in (("weight_only_int8", 127, -1), ("weight_only_int4", 7, 128)):
            codes, scale = Q.weight_quantize(w, algo=algo, group_size=g)
            back = Q.weight_dequantize(codes, scale, algo=algo, out_dtype=DT_NAME[dt], group_size=g)
            s_full = scale.float() if g == -1 else scale.float().repeat_interleave(g, dim=0)
            err = (back.float() - w.float()).abs()
            # half a quantisation step plus the rounding of the product to T
            rel = 2.0**-8 if dt == H.BF16 else 2.0**-11
            assert bool((err <= s_full * 0.5 * (1 + 2**-7) + back.float().abs() * rel).all())
            amax = w.float().abs().amax(dim=0) if g == -1 else w.float().abs().view(-1, g, 12288).amax(dim=1)
            assert torch.allclose(scale.float() * bound, amax, rtol=rel * 1.01, atol=0)


DT_NAME = {H.F16: "float16", H.BF16: "bfloat16"}
