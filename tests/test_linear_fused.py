"""weight_only_linear with apply_per_channel_scale folded in front and an
activation (gelu, swiglu) behind: wol_linear_fused against the oracle's
composition of the three (apply_per_channel_scale -> linear -> activation on
the fp32 sums), through the C ABI; and the pins of the oracle's activation
formulas (no GPU)."""
import numpy as np
import pytest

import helpers as H

TOL = 1e-3


# ---- the oracle's formulas, pinned without a GPU ---------------------------
def test_oracle_gelu_against_numpy_float64(oracle):
    # the tanh form of the reference's GEMV epilogue
    # (paddle/phi/kernels/funcs/weight_only_gemv.cu:147-157), evaluated by numpy
    # in float64 and rounded once to float32; known values and both tails
    rng = np.random.default_rng(3)
    v = np.concatenate([rng.standard_normal(4000) * 3, [0.0, -0.0, 1.0, -1.0, 40.0, -40.0, 1e-8, 88.0, -88.0]])
    v = v.astype(np.float32).reshape(1, -1)
    o32, oT = oracle.activation(v, oracle.ACT_GELU, H.F16)
    x = v.astype(np.float64)
    want = (x * 0.5 * (1.0 + np.tanh(0.7978845608028654 * (x + 0.044715 * x ** 3)))).astype(np.float32)
    # 1 + tanh cancels in the far negative tail, where libm's and numpy's tanh
    # may differ in the last place: identical bits elsewhere, absolute there
    assert np.allclose(o32, want, rtol=1e-6, atol=1e-9)
    assert np.array_equal(o32[np.abs(v) < 4], want[np.abs(v) < 4])
    assert np.array_equal(oT, H.f32_to_bits(o32, H.F16))
    # known answers: gelu(0) = 0, gelu(x) -> x for large x, -> -0 for very negative x, gelu(1) = 0.8411919906...
    i = 4000
    assert o32[0, i] == 0.0 and o32[0, i + 4] == 40.0 and o32[0, i + 5] == 0.0
    assert abs(float(o32[0, i + 2]) - 0.8411919906082768) < 1e-7
    # act 0 is the identity
    n32, _ = oracle.activation(v, oracle.ACT_NONE, H.BF16)
    assert np.array_equal(n32, v)


def test_oracle_swiglu_against_numpy_float64(oracle):
    # silu(first half) * second half (paddle/phi/kernels/gpu/swiglu_kernel.cu:32-52)
    rng = np.random.default_rng(4)
    v = (rng.standard_normal((7, 64)) * 4).astype(np.float32)
    v[0, :4] = [0.0, 30.0, -30.0, 1.0]
    v[0, 32:36] = [5.0, 2.0, 2.0, 3.0]
    o32, oT = oracle.activation(v, oracle.ACT_SWIGLU, H.BF16)
    g, u = v[:, :32].astype(np.float64), v[:, 32:].astype(np.float64)
    want = (g / (1.0 + np.exp(-g)) * u).astype(np.float32)
    assert o32.shape == (7, 32) and np.array_equal(o32, want)
    assert np.array_equal(oT, H.f32_to_bits(want, H.BF16))
    assert o32[0, 0] == 0.0 and abs(o32[0, 1] - 60.0) < 1e-5 and abs(o32[0, 2]) < 1e-10
    assert abs(float(o32[0, 3]) - 3 * 0.7310585786300049) < 1e-6


# ---- the fused entry point ----------------------------------------------------
def _fused_dev(x, ps, c, b, s, dt, N, bits, g, act):
    """wol_linear_fused on device tensors; returns the output tensor."""
    import torch
    from paddle_amd import _lib

    dev = "cuda:0"
    M, K = x.shape
    No = N // 2 if act == 2 else N
    out = torch.full((M, No), float("nan"), dtype=x.dtype, device=dev)
    wsb = _lib.lib.wol_linear_fused_workspace(M, K, N, bits, g, 0 if ps is None else 1, act)
    ws = torch.full((max(wsb, 16),), 0x5A, dtype=torch.uint8, device=dev)
    _lib.check(_lib.lib.wol_linear_fused(x.data_ptr(), None if ps is None else ps.data_ptr(), c.data_ptr(),
                                         None if b is None else b.data_ptr(), s.data_ptr(), dt, M, K, N, bits, g, act,
                                         out.data_ptr(), ws.data_ptr() if wsb else None, wsb, None))
    torch.cuda.synchronize()
    return out


def _fused(x_bits, pre_bits, packed, bias_bits, scale_bits, dt, N, bits, g, act):
    import torch

    dev = "cuda:0"
    x = H.bits_to_torch(x_bits, dt, dev)
    c = torch.from_numpy(np.ascontiguousarray(packed)).to(dev)
    s = H.bits_to_torch(scale_bits, dt, dev)
    b = None if bias_bits is None else H.bits_to_torch(bias_bits, dt, dev)
    ps = None if pre_bits is None else H.bits_to_torch(pre_bits, dt, dev)
    return H.torch_to_bits(_fused_dev(x, ps, c, b, s, dt, N, bits, g, act))


# rows x (K, N): one row (streaming kernel), a small batch on a K and N the
# batched decode kernel takes, and row counts / shapes that go to the streaming
# kernel with several rows and to the GEMM
SHAPES = [(1, 512, 256), (1, 4096, 1024), (8, 2048, 12288), (5, 4096, 10272), (3, 512, 256), (40, 1024, 512),
          (100, 512, 1024)]


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("g", [-1, 64, 128])
def test_fused_against_oracle(device, oracle, dt, bits, g):
    import torch
    from paddle_amd.nn import quant as Q

    rng = np.random.default_rng(11)
    for M, K, N in SHAPES:
        xb = H.make_act(M, K, dt, seed=M)
        bb = H.make_bias(N, dt, seed=5)
        pre = H.f32_to_bits((0.5 + rng.random(K, dtype=np.float32)).astype(np.float32), dt)
        big = K * N > 1e7  # the large shapes take a subset that still has every activation, pre-scale and bias
        if big:
            # weight made and quantised on the device (its quantiser has its own
            # bit-exact tests); the oracle quantises and multiplies column slices
            gen = torch.Generator(device="cuda").manual_seed(K + N)
            w = (torch.randn(K, N, device="cuda", generator=gen) * 0.02).to(H.torch_dtype(dt))
            codes, scale = Q.weight_quantize(w, algo="weight_only_int8" if bits == 8 else "weight_only_int4",
                                             group_size=g)
            x_d, b_d, p_d = (H.bits_to_torch(v, dt, "cuda:0") for v in (xb, bb, pre))
            slices = {}
            for c0 in (0, (N // 4) // 32 * 32, N // 2 - 32):
                for pair in (False, True):  # swiglu needs a gate slice and the up slice that goes with it
                    cols = np.r_[c0:c0 + 32, N // 2 + c0:N // 2 + c0 + 32] if pair else np.r_[c0:c0 + 64]
                    oc, osc = oracle.weight_quantize(H.torch_to_bits(w[:, cols].contiguous()), dt, bits, g)
                    assert np.array_equal(osc, H.torch_to_bits(scale[..., cols].contiguous()))
                    slices[(c0, pair)] = (cols, oc, osc)
        else:
            wb = H.make_weight(K, N, dt, seed=K + N)
            oc, osc = oracle.weight_quantize(wb, dt, bits, g)
            packed = H.gfx950_from_q(H.q_from_canonical(oc, bits), bits)
        for act in (0, 1, 2):
            for use_pre in (False, True):
                for bias in (None, bb):
                    if act == 0 and not use_pre:
                        continue  # plain wol_linear, covered elsewhere
                    if big and (act, use_pre, bias is not None) not in ((0, True, True), (1, True, False),
                                                                        (1, False, True), (2, True, False),
                                                                        (2, False, True)):
                        continue
                    print("case", dt, bits, g, M, K, N, act, use_pre, bias is not None, flush=True)
                    if not big:
                        _, wantT = oracle.linear_fused(xb, pre if use_pre else None, oc, osc, bias, dt, bits, g, act)
                        got = _fused(xb, pre if use_pre else None, packed, bias, osc, dt, N, bits, g, act)
                        err = H.rel_l2(H.bits_to_f32(got, dt), H.bits_to_f32(wantT, dt))
                        assert err <= TOL, (err, dt, bits, g, M, K, N, act, use_pre)
                        continue
                    got = _fused_dev(x_d, p_d if use_pre else None, codes, None if bias is None else b_d, scale, dt, N,
                                     bits, g, act)
                    assert bool(torch.isfinite(got.float()).all())
                    for (c0, pair), (cols, soc, sosc) in slices.items():
                        if pair != (act == 2):
                            continue
                        _, wantT = oracle.linear_fused(xb, pre if use_pre else None, soc, sosc,
                                                       None if bias is None else bias[cols], dt, bits, g, act)
                        part = got[:, c0:c0 + (32 if act == 2 else 64)].contiguous()
                        err = H.rel_l2(H.bits_to_f32(H.torch_to_bits(part), dt), H.bits_to_f32(wantT, dt))
                        assert err <= TOL, (err, dt, bits, g, M, K, N, act, use_pre, c0)


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("g", [-1, 64, 128])
def test_swiglu_in_the_gemm_epilogue(device, oracle, dt, bits, g):
    # above 64 rows the GEMM pairs gate and up columns in one wavefront and
    # writes [M, N/2] itself: no fp32 sums, no extra pass (group-wise scales: the
    # tiles whose sums are kept in units of the group scale; their scales are
    # gathered from the gate and the up columns like the codes).
    # 128-row and 256-row tiles, rows off the tile height, a gate half that ends
    # inside a column tile (N/2 = 1168), with and without bias
    from paddle_amd import _lib

    shapes = [(100, 512, 1024), (200, 512, 512), (300, 1024, 2336), (1000, 256, 768)]
    if g == -1:
        shapes.append((513, 256, 768))
    for M, K, N in shapes:
        assert _lib.lib.wol_linear_fused_workspace(M, K, N, bits, g, 0, 2) == _lib.lib.wol_linear_workspace(M, K, N, bits, g)
        wb = H.make_weight(K, N, dt, seed=K + N + M)
        xb = H.make_act(M, K, dt, seed=M)
        bb = H.make_bias(N, dt, seed=6)
        oc, osc = oracle.weight_quantize(wb, dt, bits, g)
        packed = H.gfx950_from_q(H.q_from_canonical(oc, bits), bits)
        for bias in (None, bb):
            _, wantT = oracle.linear_fused(xb, None, oc, osc, bias, dt, bits, g, 2)
            got = _fused(xb, None, packed, bias, osc, dt, N, bits, g, 2)
            assert got.shape == (M, N // 2)
            err = H.rel_l2(H.bits_to_f32(got, dt), H.bits_to_f32(wantT, dt))
            assert err <= TOL, (err, dt, bits, g, M, K, N, bias is not None)


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("g", [-1, 128])
def test_swiglu_in_the_streaming_kernel(device, oracle, dt, bits, g):
    # up to 16 rows the streaming kernel gives half of a workgroup's wavefronts
    # the gate strip and the other half the up strip and writes [M, N/2] itself.
    # Shapes: every operand height (1, 2, 4, 8, 16 rows), K whose units go one,
    # two or four to a wavefront at once, K that a wavefront walks (8192, and
    # 11008 / 1088 with their partial last unit and int4 half tile), one pair
    # of strips and many; K = 512 ... 1088 keep the batched kernel out at
    # several rows
    import ctypes

    from paddle_amd import _lib

    rng = np.random.default_rng(3)
    for M, K, N in ((1, 512, 32), (1, 4096, 1024), (1, 8192, 256), (1, 11008, 64), (2, 1024, 96), (3, 512, 256),
                    (4, 1088, 64), (5, 1024, 160), (8, 512, 64), (9, 1024, 96), (16, 1088, 128)):
        lws = _lib.lib.wol_linear_workspace(M, K, N, bits, g)
        plan = ctypes.create_string_buffer(256)
        _lib.check(_lib.lib.wol_linear_plan(M, K, N, bits, g, lws, plan, 256))
        if b"stream_kernel" in plan.value:  # (16 rows of int8 at K = 1088 go to the batched kernel and the pass)
            assert _lib.lib.wol_linear_fused_workspace(M, K, N, bits, g, 0, 2) == lws
        wb = H.make_weight(K, N, dt, seed=K + N + M)
        xb = H.make_act(M, K, dt, seed=M)
        bb = H.make_bias(N, dt, seed=6)
        pre = H.f32_to_bits((0.5 + rng.random(K, dtype=np.float32)).astype(np.float32), dt)
        oc, osc = oracle.weight_quantize(wb, dt, bits, g)
        packed = H.gfx950_from_q(H.q_from_canonical(oc, bits), bits)
        for bias, use_pre in ((None, False), (bb, False), (bb, M == 1)):
            print("case", dt, bits, g, M, K, N, bias is not None, use_pre, flush=True)
            _, wantT = oracle.linear_fused(xb, pre if use_pre else None, oc, osc, bias, dt, bits, g, 2)
            got = _fused(xb, pre if use_pre else None, packed, bias, osc, dt, N, bits, g, 2)
            assert got.shape == (M, N // 2)
            err = H.rel_l2(H.bits_to_f32(got, dt), H.bits_to_f32(wantT, dt))
            assert err <= TOL, (err, dt, bits, g, M, K, N, bias is not None, use_pre)


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("g", [-1, 64, 128])
def test_swiglu_in_the_batched_kernel(device, oracle, dt, bits, g):
    # 2 to 16 rows at K = 2048, 4096 (and 8192 for int4) on weights wide enough
    # for the batched kernel (2.5 strips per CU and more): a workgroup owns a
    # range of strip pairs (gate strip, up strip) and combines them at the end
    # of every run of three pairs.  Workgroups with one or two pairs, with three
    # or four (a second run of one pair), with a remainder.  The weights are made
    # and quantised on the device; the oracle checks column slices
    import ctypes

    import torch
    from paddle_amd import _lib
    from paddle_amd.nn import quant as Q

    shapes = [(9, 2048, 28704), (12, 4096, 10272), (7, 4096, 28704), (16, 4096, 28704)]
    if bits == 4 and g != 64:
        shapes += [(9, 8192, 12320), (2, 8192, 12320)]
    for M, K, N in shapes:
        lws = _lib.lib.wol_linear_workspace(M, K, N, bits, g)
        plan = ctypes.create_string_buffer(256)
        _lib.check(_lib.lib.wol_linear_plan(M, K, N, bits, g, lws, plan, 256))
        assert b"batch_kernel" in plan.value and b"reduce" not in plan.value, plan.value
        assert _lib.lib.wol_linear_fused_workspace(M, K, N, bits, g, 0, 2) == lws
        xb = H.make_act(M, K, dt, seed=M)
        bb = H.make_bias(N, dt, seed=6)
        gen = torch.Generator(device="cuda").manual_seed(K + N)
        w = (torch.randn(K, N, device="cuda", generator=gen) * 0.02).to(H.torch_dtype(dt))
        codes, scale = Q.weight_quantize(w, algo="weight_only_int8" if bits == 8 else "weight_only_int4", group_size=g)
        x_d, b_d = (H.bits_to_torch(v, dt, "cuda:0") for v in (xb, bb))
        for bias in (None, bb):
            print("case", dt, bits, g, M, K, N, bias is not None, flush=True)
            got = _fused_dev(x_d, None, codes, None if bias is None else b_d, scale, dt, N, bits, g, 2)
            assert got.shape == (M, N // 2) and bool(torch.isfinite(got.float()).all())
            # the first workgroup's pairs (the fourth is a run of its own where it has four), pairs in the
            # middle and at the end of the range
            # (slices of 64 columns: with a few rows a slice of 16 is a hundred values, and one value of T that rounds
            # the other way is 1e-3 of such a slice by itself)
            for c0 in (0, 64, (N // 4) // 16 * 16, N // 2 - 64):
                cols = np.r_[c0:c0 + 64, N // 2 + c0:N // 2 + c0 + 64]
                oc, osc = oracle.weight_quantize(H.torch_to_bits(w[:, cols].contiguous()), dt, bits, g)
                assert np.array_equal(osc, H.torch_to_bits(scale[..., cols].contiguous()))
                _, wantT = oracle.linear_fused(xb, None, oc, osc, None if bias is None else bias[cols], dt, bits, g, 2)
                part = got[:, c0:c0 + 64].contiguous()
                err = H.rel_l2(H.bits_to_f32(H.torch_to_bits(part), dt), H.bits_to_f32(wantT, dt))
                assert err <= TOL, (err, dt, bits, g, M, K, N, c0, bias is not None)


@pytest.mark.gpu
@pytest.mark.parametrize("dt,bits,g,M,K,N", [(H.BF16, 8, -1, 48, 4096, 12288), (H.F16, 4, 128, 17, 8192, 22016),
                                             (H.BF16, 4, 64, 40, 4096, 22016), (H.F16, 8, 64, 64, 8192, 28672)])
def test_swiglu_where_the_small_m_gemm_adds_its_runs(device, oracle, dt, bits, g, M, K, N):
    # 17 to 64 rows on a large weight: the GEMM cuts K into runs and the kernel
    # that adds them forms the swiglu, so the fused call needs the linear's own
    # scratch and nothing more.  Device-made weight, oracle on column slices.
    import ctypes

    import torch
    from paddle_amd import _lib
    from paddle_amd.nn import quant as Q

    lws = _lib.lib.wol_linear_workspace(M, K, N, bits, g)
    plan = ctypes.create_string_buffer(256)
    _lib.check(_lib.lib.wol_linear_plan(M, K, N, bits, g, lws, plan, 256))
    assert b"gemm_dma_kernel" in plan.value and b"reduce_partials" in plan.value, plan.value
    assert _lib.lib.wol_linear_fused_workspace(M, K, N, bits, g, 0, 2) == lws > 0
    xb = H.make_act(M, K, dt, seed=M)
    bb = H.make_bias(N, dt, seed=6)
    gen = torch.Generator(device="cuda").manual_seed(K + N)
    w = (torch.randn(K, N, device="cuda", generator=gen) * 0.02).to(H.torch_dtype(dt))
    codes, scale = Q.weight_quantize(w, algo="weight_only_int8" if bits == 8 else "weight_only_int4", group_size=g)
    x_d, b_d = (H.bits_to_torch(v, dt, "cuda:0") for v in (xb, bb))
    for bias in (None, bb):
        got = _fused_dev(x_d, None, codes, None if bias is None else b_d, scale, dt, N, bits, g, 2)
        assert got.shape == (M, N // 2) and bool(torch.isfinite(got.float()).all())
        for c0 in (0, 256 - 16, (N // 4) // 16 * 16, N // 2 - 32):
            cols = np.r_[c0:c0 + 32, N // 2 + c0:N // 2 + c0 + 32]
            oc, osc = oracle.weight_quantize(H.torch_to_bits(w[:, cols].contiguous()), dt, bits, g)
            assert np.array_equal(osc, H.torch_to_bits(scale[..., cols].contiguous()))
            _, wantT = oracle.linear_fused(xb, None, oc, osc, None if bias is None else bias[cols], dt, bits, g, 2)
            part = got[:, c0:c0 + 32].contiguous()
            err = H.rel_l2(H.bits_to_f32(H.torch_to_bits(part), dt), H.bits_to_f32(wantT, dt))
            assert err <= TOL, (err, dt, bits, g, M, K, N, c0, bias is not None)
    # without the scratch the call is refused, not run on another plan
    out = torch.empty((M, N // 2), dtype=x_d.dtype, device="cuda")
    rc = _lib.lib.wol_linear_fused(x_d.data_ptr(), None, codes.data_ptr(), None, scale.data_ptr(), dt, M, K, N, bits, g, 2,
                                   out.data_ptr(), None, 0, None)
    assert rc == 8  # WOL_ERR_WORKSPACE


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [H.F16, H.BF16])
def test_fused_pre_scale_equals_the_two_ops(device, oracle, dt):
    # folding apply_per_channel_scale into the linear must not change a bit:
    # the same products, rounded the same way, enter the same kernel
    import gpu_calls as G
    import torch
    from paddle_amd import _lib

    rng = np.random.default_rng(12)
    for M, K, N, bits, g in ((1, 4096, 512, 4, 128), (8, 4096, 8192, 4, -1), (16, 2048, 8192, 8, 64), (6, 512, 256, 8, -1),
                             (200, 1024, 512, 8, -1)):
        wb = H.make_weight(K, N, dt, seed=K + N)
        xb = H.make_act(M, K, dt, seed=M)
        pre = H.f32_to_bits((0.25 + 2 * rng.random(K, dtype=np.float32)).astype(np.float32), dt)
        oc, osc = oracle.weight_quantize(wb, dt, bits, g)
        packed = H.gfx950_from_q(H.q_from_canonical(oc, bits), bits)
        fused = _fused(xb, pre, packed, None, osc, dt, N, bits, g, 0)
        x = H.bits_to_torch(xb, dt, "cuda:0")
        ps = H.bits_to_torch(pre, dt, "cuda:0")
        xs = torch.empty_like(x)
        _lib.check(_lib.lib.wol_apply_per_channel_scale(x.data_ptr(), ps.data_ptr(), dt, M, K, xs.data_ptr(), None))
        torch.cuda.synchronize()
        assert np.array_equal(H.torch_to_bits(xs), oracle.apply_per_channel_scale(xb, pre, dt))
        two = G.linear(H.torch_to_bits(xs), packed, None, osc, dt, N, bits, g)
        assert np.array_equal(fused, two), (M, K, N, bits, g)


@pytest.mark.gpu
@pytest.mark.parametrize("act,use_pre", [(1, False), (2, False), (2, True)])
def test_fused_on_the_batched_kernel_with_k_runs(device, oracle, act, use_pre):
    # 24 rows on a 25 MB int8 weight: wol_linear takes the batched kernel with K
    # runs, so bias, gelu and swiglu are applied by the kernel that adds the
    # runs; with activation scales the call takes another kernel (here the
    # GEMM, whose group-wise form leaves the swiglu to a pass over fp32 sums)
    # and the pre-scale is a pass in front
    from paddle_amd import _lib
    import ctypes

    dt, bits, g, M, K, N = H.BF16, 8, 64, 24, 2048, 12288
    buf = ctypes.create_string_buffer(512)
    assert _lib.lib.wol_linear_plan(M, K, N, bits, g, 1 << 30, buf, 512) == 0 and b"K runs" in buf.value
    if not use_pre:  # nothing but the linear's own scratch: no extra pass
        assert _lib.lib.wol_linear_fused_workspace(M, K, N, bits, g, 0, act) == _lib.lib.wol_linear_workspace(M, K, N, bits, g)
    rng = np.random.default_rng(13)
    wb = H.make_weight(K, N, dt, seed=3)
    xb = H.make_act(M, K, dt, seed=4)
    bb = H.make_bias(N, dt, seed=5)
    pre = H.f32_to_bits((0.5 + rng.random(K, dtype=np.float32)).astype(np.float32), dt) if use_pre else None
    oc, osc = oracle.weight_quantize(wb, dt, bits, g)
    packed = H.gfx950_from_q(H.q_from_canonical(oc, bits), bits)
    _, wantT = oracle.linear_fused(xb, pre, oc, osc, bb, dt, bits, g, act)
    got = _fused(xb, pre, packed, bb, osc, dt, N, bits, g, act)
    err = H.rel_l2(H.bits_to_f32(got, dt), H.bits_to_f32(wantT, dt))
    assert err <= TOL, (err, act, use_pre)


@pytest.mark.gpu
def test_fused_python_wrapper_and_errors(device):
    import torch
    from paddle_amd.nn import quant as Q

    w = (torch.randn(512, 256, device="cuda") * 0.02).half()
    codes, scale = Q.weight_quantize(w, algo="weight_only_int4", group_size=64)
    x = torch.randn(2, 3, 512, device="cuda").half()
    ps = (torch.rand(512, device="cuda") + 0.5).half()
    out = Q.weight_only_linear_fused(x, codes, None, scale, "int4", 64, pre_scale=ps, act="swiglu")
    assert list(out.shape) == [2, 3, 128] and out.dtype == torch.float16
    lin = Q.weight_only_linear(Q.apply_per_channel_scale(x.reshape(-1, 512), ps), codes, None, scale, "int4", None, 64)
    ref = torch.nn.functional.silu(lin[:, :128].float()) * lin[:, 128:].float()
    assert torch.allclose(out.reshape(-1, 128).float(), ref, rtol=2e-2, atol=2e-3)
    gel = Q.weight_only_linear_fused(x, codes, None, scale, "int4", 64, act="gelu")
    lin2 = Q.weight_only_linear(x, codes, None, scale, "int4", None, 64)
    assert torch.allclose(gel.float(), torch.nn.functional.gelu(lin2.float(), approximate="tanh"), rtol=2e-2, atol=2e-3)
    with pytest.raises(ValueError):
        Q.weight_only_linear_fused(x, codes, None, scale, "int4", 64, act="relu")
    with pytest.raises(ValueError):
        Q.weight_only_linear_fused(x, codes, None, scale, "int4", 64, pre_scale=ps[:100])
    assert list(Q.weight_only_linear_fused(x[:0], codes, None, scale, "int4", 64, act="swiglu").shape) == [0, 3, 128]
