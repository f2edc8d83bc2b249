"""GPU parity of weight_only_linear against the CPU oracle, through the C ABI.

Bar: relative L2 error <= 1e-3 between the kernel's fp32 accumulators and the
oracle's fp32 dequantise-then-matmul, and between the kernel's T output and
the oracle's result cast to T with the same rounding.  (A T output is never
compared with the unrounded oracle: one bf16 rounding alone is 1.7e-3.)
"""
import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu

TOL = 1e-3


@pytest.fixture(scope="module")
def G(device):
    import gpu_calls

    return gpu_calls


def check(G, oracle, dt, bits, g, M, K, N, bias=True, seed=0, outliers=0.0, tol32=2e-5, xdist="normal", **kw):
    wb = H.make_weight(K, N, dt, seed=seed + K + N, outlier_cols=outliers)
    xb = H.make_act(M, K, dt, seed=seed + M, dist=xdist)
    bb = H.make_bias(N, dt, seed=seed + 1) if bias else None
    oc, osc = oracle.weight_quantize(wb, dt, bits, g)
    packed = H.gfx950_from_q(H.q_from_canonical(oc, bits), bits)
    r32, rT = oracle.linear(xb, oc, osc, bb, dt, bits, g)
    got32 = G.linear(xb, packed, bb, osc, dt, N, bits, g, f32=True, **kw)
    gotT = G.linear(xb, packed, bb, osc, dt, N, bits, g, f32=False, **kw)
    e32 = H.rel_l2(got32, r32)
    eT = H.rel_l2(H.bits_to_f32(gotT, dt), H.bits_to_f32(rT, dt))
    assert np.isfinite(got32).all()
    assert e32 <= tol32, (e32, dt, bits, g, M, K, N)   # far inside the 1e-3 bar
    assert eT <= TOL, (eT, dt, bits, g, M, K, N)
    # the T output is the RNE cast of the fp32 accumulators
    assert np.array_equal(gotT, H.f32_to_bits(got32, dt))
    return e32, eT


def check_sampled(G, oracle, dt, bits, g, M, K, N, bias=True, seed=0, tol32=2e-5, ncols=96, **kw):
    """check() for weights that would keep the scalar oracle busy for seconds:
    the weight is made and quantised on the device (the quantiser is pinned bit
    for bit by its own tests); the oracle quantises three column slices of the
    same weight -- first, middle, last, which must reproduce the device's
    scales -- and multiplies them; the whole output must be the rounded fp32
    sums, and finite."""
    import torch
    from paddle_amd.nn import quant as Q

    tdt = H.torch_dtype(dt)
    gen = torch.Generator(device="cuda").manual_seed(seed + K + N)
    w = (torch.randn(K, N, device="cuda", generator=gen) * 0.02).to(tdt)
    codes, scale = Q.weight_quantize(w, algo="weight_only_int8" if bits == 8 else "weight_only_int4", group_size=g)
    xb = H.make_act(M, K, dt, seed=seed + M)
    bb = H.make_bias(N, dt, seed=seed + 1) if bias else None
    x = H.bits_to_torch(xb, dt, "cuda:0")
    b = None if bb is None else H.bits_to_torch(bb, dt, "cuda:0")
    got32 = G.linear_dev(x, codes, b, scale, dt, N, bits, g, f32=True, **kw)
    gotT = G.linear_dev(x, codes, b, scale, dt, N, bits, g, f32=False, **kw)
    assert bool(torch.isfinite(got32).all())
    assert torch.equal(gotT, got32.to(tdt))  # the T output is the RNE cast of the fp32 accumulators
    for c0 in (0, (N // 2) // 32 * 32, N - ncols):
        cols = slice(c0, c0 + ncols)
        oc, osc = oracle.weight_quantize(H.torch_to_bits(w[:, cols].contiguous()), dt, bits, g)
        assert np.array_equal(osc, H.torch_to_bits(scale[..., cols].contiguous()))
        r32, rT = oracle.linear(xb, oc, osc, None if bb is None else bb[cols], dt, bits, g)
        e32 = H.rel_l2(got32[:, cols].cpu().numpy(), r32)
        eT = H.rel_l2(H.bits_to_f32(H.torch_to_bits(gotT[:, cols].contiguous()), dt), H.bits_to_f32(rT, dt))
        assert e32 <= tol32, (e32, dt, bits, g, M, K, N, c0)
        assert eT <= TOL, (eT, dt, bits, g, M, K, N, c0)


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("g", [-1, 64, 128])
def test_linear_small_shapes_all_m(G, oracle, dt, bits, g):
    # every M class of the streaming kernel (1, 2, 4, 8, 16 rows per operand,
    # 2-4 tiles) and the GEMM kernel, ragged M, K with and without a half tile
    for K, N in [(64, 256), (128, 288), (192, 64), (512, 1024), (1088, 96)]:
        if bits == 4 and N % 32:
            continue
        for M in (1, 2, 3, 4, 7, 8, 15, 16, 17, 33, 48, 64, 65, 100, 300):
            print("case", dt, bits, g, K, N, M, flush=True)
            check(G, oracle, dt, bits, g, M, K, N, bias=(M % 2 == 1), seed=M)


KERNEL_STREAM, KERNEL_GEMM, KERNEL_BATCH = 1, 2, 3


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("g", [-1, 64, 128])
def test_linear_batch_kernel_pinned(G, oracle, dt, bits, g):
    # the batched decode kernel on every K it is built for (every wavefront
    # owns 1, 2 or 4 tiles of a strip); fewer strips than CUs, one, two and
    # many strips per workgroup (more than the weight ring holds, more than one
    # run of seven strips shares the LDS); N that is 16 mod 32
    shapes = [(2048, 1024), (4096, 4128), (8192, 272), (2048, 12368), (2048, 48), (2048, 36880), (4096, 32800)]
    for K, N in shapes:
        if K == 8192 and (bits == 8 or g == 64):
            with pytest.raises(ValueError):  # not built: the A fragments alone take 64 registers
                check(G, oracle, dt, bits, g, 4, K, N, seed=1, kernel=KERNEL_BATCH)
            continue
        for M in ((1, 2, 3, 5, 8, 13, 16) if K * N < 5e6 else ((2, 16) if K * N < 5e7 else (7,))):
            print("case", dt, bits, g, K, N, M, flush=True)
            (check if K * N < 5e6 else check_sampled)(G, oracle, dt, bits, g, M, K, N, bias=(M % 2 == 1), seed=M,
                                                      kernel=KERNEL_BATCH)
    # refused: more than 16 rows, any other K
    with pytest.raises(ValueError):
        check(G, oracle, dt, bits, g, 17, 2048, 256, seed=1, kernel=KERNEL_BATCH)
    with pytest.raises(ValueError):
        check(G, oracle, dt, bits, g, 4, 1024, 256, seed=1, kernel=KERNEL_BATCH)


KERNEL_BATCH_SPLIT = 4


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("g", [-1, 64, 128])
def test_linear_batch_split_kernel_pinned(G, oracle, dt, bits, g):
    # the batched decode kernel with K cut into runs across workgroups: K that
    # fills its runs exactly (2048, 4096), K whose last run is mostly past the
    # end (one tile more than a run; 11008), K long enough for the 256-k runs
    # (14336); fewer strips than strip sets, more strips per set than one LDS
    # run holds; N that is 16 mod 32; 1 to 16 rows and the two-operand form up
    # to 32
    tk = 64 if bits == 8 else 128
    shapes = [(2048, 1024), (2048 + tk, 4128), (4096, 272), (11008, 528), (14336, 272), (2048, 48), (2048, 36880)]
    for K, N in shapes:
        for M in ((1, 2, 5, 16, 17, 24, 32) if K * N < 5e6 else ((3, 16, 31) if K * N < 5e7 else (20,))):
            print("case", dt, bits, g, K, N, M, flush=True)
            (check if K * N < 5e6 else check_sampled)(G, oracle, dt, bits, g, M, K, N, bias=(M % 2 == 1), seed=M,
                                                      kernel=KERNEL_BATCH_SPLIT)
    # refused: more than 32 rows, fewer than 16 weight tiles, a K that ends in
    # half a tile (int4), scratch that is too small
    with pytest.raises(ValueError):
        check(G, oracle, dt, bits, g, 33, 2048, 256, seed=1, kernel=KERNEL_BATCH_SPLIT)
    with pytest.raises(ValueError):
        check(G, oracle, dt, bits, g, 4, 15 * tk, 256, seed=1, kernel=KERNEL_BATCH_SPLIT)
    if bits == 4:
        with pytest.raises(ValueError):
            check(G, oracle, dt, bits, g, 4, 2048 + 64, 256, seed=1, kernel=KERNEL_BATCH_SPLIT)
    with pytest.raises(ValueError):
        check(G, oracle, dt, bits, g, 4, 4096, 256, seed=1, kernel=KERNEL_BATCH_SPLIT, ws_bytes=4 * 256 * 4)


def test_linear_takes_the_split_batch_kernel_where_it_is_measured_faster(G, oracle):
    # the dispatcher's choice (named by wol_linear_plan), with and without the
    # scratch that kernel needs, and the same call checked against the oracle
    big = 1 << 30
    assert "K runs" in G.linear_plan(12, 13824, 5120, 4, 128, big)       # ragged last round of strips
    assert "K runs" in G.linear_plan(16, 14336, 4096, 4, -1, big)        # int4, long K
    assert "K runs" in G.linear_plan(24, 4096, 11008, 8, 64, big)        # two 16-row operands, int8
    assert "K runs" not in G.linear_plan(12, 13824, 5120, 4, 128, 0)     # no scratch: one of the others
    assert "K runs" not in G.linear_plan(4, 13824, 5120, 4, 128, big)    # few rows: the streaming kernel
    assert "K runs" not in G.linear_plan(12, 4096, 11008, 4, 128, big)   # the one-launch batched kernel
    check(G, oracle, H.BF16, 4, 128, 12, 6144, 384 * 16, seed=2)
    check(G, oracle, H.F16, 8, 64, 24, 4096, 5120, seed=3)


@pytest.mark.parametrize("kernel", [KERNEL_STREAM, KERNEL_BATCH, KERNEL_BATCH_SPLIT, KERNEL_GEMM])
@pytest.mark.parametrize("dt", [H.F16, H.BF16])
def test_linear_int4_offset_cancellation_with_biased_activations(G, oracle, dt, kernel):
    # activations that are all positive (what follows a gelu or a relu) make the
    # term that cancels the dequantiser's offset as large as it gets; the sums
    # must still be far inside the bar.  Ragged N (16 mod 32) on every kernel.
    for M, K, N in ((4, 4096, 1040), (16, 2048, 48)):
        check(G, oracle, dt, 4, 128, M, K, N, seed=5, xdist="uniform", tol32=1e-4, kernel=kernel)


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("g", [-1, 64, 128])
def test_linear_gemm_kernel_small_m(G, oracle, dt, bits, g):
    # the MFMA GEMM pinned on the row counts that the cost model would hand to
    # the streaming kernel at these sizes: one row block of 32 or 64 rows, K
    # split across workgroups (512 / 64 = 8 k tiles for int8, 1024 / 128 = 8 for
    # int4), ragged N (not a multiple of the 256-column tile), with and without bias
    for K, N in [(512, 1024), (1024, 288), (1024, 1056)]:
        if bits == 4 and N % 32:
            continue
        for M in (1, 9, 16, 31, 32, 33, 64):
            print("case", dt, bits, g, K, N, M, flush=True)
            check(G, oracle, dt, bits, g, M, K, N, bias=(M % 2 == 1), seed=M, kernel=KERNEL_GEMM)


def test_linear_gemm_split_k_scratch_sizes(G, oracle):
    # the scratch buffer is optional: with none, or one that holds fewer runs
    # than planned, the same problem still comes out right (K is split less)
    dt, bits, g, M, K, N = H.BF16, 8, 64, 24, 2048, 512
    from paddle_amd import _lib
    full = _lib.lib.wol_linear_workspace_for(M, K, N, bits, g, KERNEL_GEMM)
    assert full >= 2 * M * N * 4 and full % (M * N * 4) == 0
    for wsb in (0, M * N * 4, 2 * M * N * 4, full - 4, full):
        check(G, oracle, dt, bits, g, M, K, N, seed=3, kernel=KERNEL_GEMM, ws_bytes=wsb)
    # above 64 rows K is split only when the output tiles leave most CUs idle
    for dt, bits, g, M, K, N in ((H.BF16, 8, -1, 100, 2048, 512), (H.F16, 4, 128, 130, 4096, 256)):
        full = _lib.lib.wol_linear_workspace(M, K, N, bits, g)
        assert full >= 2 * M * N * 4 and full % (M * N * 4) == 0
        for wsb in (0, 2 * M * N * 4, full):
            check(G, oracle, dt, bits, g, M, K, N, seed=4, ws_bytes=wsb)


@pytest.mark.parametrize("bits", [8, 4])
def test_linear_stream_kernel_pinned_large_m(G, oracle, bits):
    # the streaming kernel up to its limit of 64 rows, and the refusal beyond
    for M in (17, 48, 64):
        check(G, oracle, H.F16, bits, 128, M, 512, 256, seed=M, kernel=KERNEL_STREAM)
    with pytest.raises(ValueError):
        check(G, oracle, H.F16, bits, 128, 65, 512, 256, seed=1, kernel=KERNEL_STREAM)


def test_both_kernels_agree_on_full_size_decode_shape(G, oracle):
    # LLaMA-7B FFN shape at M = 16 (where the two kernels' costs cross): the
    # two fp32 results differ only by summation order
    dt, bits, g, M, K, N = H.BF16, 4, 128, 16, 4096, 11008
    wb = H.make_weight(K, N, dt, seed=77)
    xb = H.make_act(M, K, dt, seed=78)
    oc, osc = oracle.weight_quantize(wb, dt, bits, g)
    packed = H.gfx950_from_q(H.q_from_canonical(oc, bits), bits)
    a = G.linear(xb, packed, None, osc, dt, N, bits, g, f32=True, kernel=KERNEL_STREAM)
    b = G.linear(xb, packed, None, osc, dt, N, bits, g, f32=True, kernel=KERNEL_GEMM)
    assert H.rel_l2(a, b) <= 5e-6  # each carries ~1.5e-6 of offset-cancellation rounding
    r32, _ = oracle.linear(xb, oc, osc, None, dt, bits, g)
    assert H.rel_l2(b, r32) <= 2e-5


def test_linear_random_shapes_all_kernels(G, oracle):
    # seeded sweep over the whole contract: any M, K a multiple of 64 (so both
    # the k-tile-aligned and the ragged GEMM paths, and int4 strips that end in
    # a half tile), N a multiple of 16 (32 for int4), every kernel that accepts
    # the shape, with and without bias
    rng = np.random.default_rng(20240607)
    for case in range(36):
        dt = [H.F16, H.BF16][int(rng.integers(2))]
        bits = [8, 4][int(rng.integers(2))]
        g = [-1, 64, 128][int(rng.integers(3))]
        M = int(rng.choice([1, 2, 5, 8, 9, 13, 16, 20, 31, 33, 50, 64, 65, 96, 129, 200, 257]))
        K = 64 * int(rng.integers(1, 33))
        N = (32 if bits == 4 else 16) * int(rng.integers(1, 41))
        kernels = [None, KERNEL_GEMM] + ([KERNEL_STREAM] if M <= 64 else [])
        if M <= 16 and K == 2048:
            kernels.append(KERNEL_BATCH)
        kernel = kernels[int(rng.integers(len(kernels)))]
        print("case", case, dt, bits, g, M, K, N, kernel, flush=True)
        kw = {} if kernel is None else {"kernel": kernel}
        check(G, oracle, dt, bits, g, M, K, N, bias=bool(rng.integers(2)), seed=case, **kw)


def test_linear_random_shapes_batch_split_kernel(G, oracle):
    # the same for the batched kernel with K runs: any K of 16 or more whole
    # weight tiles (so last runs that are full, nearly empty and anything in
    # between), 1 to 32 rows
    rng = np.random.default_rng(20250311)
    for case in range(24):
        dt = [H.F16, H.BF16][int(rng.integers(2))]
        bits = [8, 4][int(rng.integers(2))]
        g = [-1, 64, 128][int(rng.integers(3))]
        M = int(rng.integers(1, 33))
        K = (64 if bits == 8 else 128) * int(rng.integers(16, 90))
        N = (32 if bits == 4 else 16) * int(rng.integers(1, 30))
        print("case", case, dt, bits, g, M, K, N, flush=True)
        check(G, oracle, dt, bits, g, M, K, N, bias=bool(rng.integers(2)), seed=case, kernel=KERNEL_BATCH_SPLIT)


@pytest.mark.parametrize("bits,g", [(8, -1), (4, 64)])
def test_cpu_quantised_weight_through_repack_host(G, oracle, bits, g):
    # The flow of a weight that never saw the GPU quantiser: quantised on the CPU
    # (the oracle stands for the reference's CPU kernel), stored in the layout a
    # ROCm build of that kernel emits (cpu/weight_quantize_kernel.cc:113-125),
    # re-laid once on the host with wol_repack_host, then used by the GPU linear
    # at one row, a few rows and a GEMM-sized batch.  Fed to the kernels without
    # the re-layout the same bytes give numbers that are simply wrong.
    from paddle_amd import _lib

    dt, K, N = H.BF16, 512, 256
    wb = H.make_weight(K, N, dt, seed=21)
    oc, osc = oracle.weight_quantize(wb, dt, bits, g)
    hip = np.ascontiguousarray(H.paddle_hip_from_q(H.q_from_canonical(oc, bits), bits)).view(np.uint8).reshape(-1)
    packed = np.full(hip.size, 0xEE, np.uint8)
    assert _lib.lib.wol_repack_host(hip.ctypes.data, 1, packed.ctypes.data, 2, K, N, bits) == 0
    for M in (1, 5, 96):
        xb = H.make_act(M, K, dt, seed=M)
        _, wantT = oracle.linear(xb, oc, osc, None, dt, bits, g)
        got = G.linear(xb, packed, None, osc, dt, N, bits, g)
        assert H.rel_l2(H.bits_to_f32(got, dt), H.bits_to_f32(wantT, dt)) <= 1e-3, (bits, g, M)
        wrong = G.linear(xb, hip, None, osc, dt, N, bits, g)
        assert H.rel_l2(H.bits_to_f32(wrong, dt), H.bits_to_f32(wantT, dt)) > 0.1


# The reference's own test matrix (test/quantization/test_weight_only_linear.py:
# 62-614): dtype x weight dtype x bias x token x group size x (K, N), x ~ U[0,1),
# compared there with a dense fp16/bf16 Linear at atol 1e-2 .. 0.13; here against
# the oracle at the 1e-3 bar.
REFERENCE_CASES = [
    # dtype, wdtype, bias, batch, token, K, N, group
    (H.F16, 8, True, 1, 32, 64, 256, -1), (H.F16, 8, False, 1, 32, 64, 256, -1), (H.BF16, 8, True, 1, 32, 64, 256, -1),
    (H.F16, 4, True, 1, 32, 64, 256, -1), (H.F16, 4, False, 1, 32, 64, 256, -1), (H.BF16, 4, True, 1, 32, 64, 256, -1),
    (H.F16, 8, True, 1, 1, 64, 256, -1), (H.F16, 8, False, 1, 1, 64, 256, -1), (H.BF16, 8, True, 1, 1, 64, 256, -1),
    (H.BF16, 8, False, 1, 1, 64, 256, -1), (H.F16, 4, True, 1, 1, 64, 256, -1), (H.F16, 4, False, 1, 1, 64, 256, -1),
    (H.BF16, 4, False, 1, 1, 64, 256, -1), (H.BF16, 4, False, 1, 1, 64, 256, 64), (H.BF16, 4, False, 1, 1, 64, 256, 128),
    (H.F16, 4, False, 1, 1, 64, 256, 64), (H.F16, 4, False, 1, 1, 64, 256, 128), (H.BF16, 4, False, 1, 2, 64, 256, 128),
    (H.BF16, 8, False, 1, 1, 64, 256, 64), (H.BF16, 8, False, 1, 1, 64, 256, 128),
    (H.F16, 8, True, 1, 32, 128, 288, -1), (H.F16, 8, False, 1, 32, 128, 288, -1), (H.BF16, 8, True, 1, 32, 128, 288, -1),
    (H.BF16, 4, True, 1, 32, 128, 288, -1), (H.F16, 4, True, 1, 300, 128, 288, -1), (H.BF16, 8, True, 1, 300, 128, 288, 128),
    (H.F16, 4, False, 2, 300, 128, 288, 64),
]


@pytest.mark.parametrize("case", REFERENCE_CASES)
def test_reference_test_matrix(G, oracle, case):
    import torch

    from paddle_amd.nn import quant as Q

    dt, bits, bias, batch, token, K, N, g = case
    rng = np.random.default_rng(123)
    tdt = H.torch_dtype(dt)
    w = torch.from_numpy(((rng.random((K, N), dtype=np.float32) - 0.5) / np.sqrt(K)).astype(np.float32)).to(tdt).cuda()
    x = torch.from_numpy(rng.random((batch, token, K), dtype=np.float32)).to(tdt).cuda()
    b = torch.from_numpy(rng.random((N,), dtype=np.float32) - 0.5).to(tdt).cuda() if bias else None
    algo = "weight_only_int8" if bits == 8 else "weight_only_int4"
    codes, scale = Q.weight_quantize(w, algo=algo, group_size=g)
    assert list(codes.shape) == [N * bits // 8, K] and codes.dtype == torch.int8
    out = Q.weight_only_linear(x, codes, bias=b, weight_scale=scale, weight_dtype="int8" if bits == 8 else "int4", group_size=g)
    assert list(out.shape) == [batch, token, N] and out.dtype == tdt
    # oracle on the same bits
    wb, xb = H.torch_to_bits(w), H.torch_to_bits(x).reshape(-1, K)
    oc, osc = oracle.weight_quantize(wb, dt, bits, g)
    assert np.array_equal(H.torch_to_bits(scale), osc)
    assert np.array_equal(codes.cpu().numpy().view(np.uint8).reshape(-1), H.gfx950_from_q(H.q_from_canonical(oc, bits), bits))
    _, rT = oracle.linear(xb, oc, osc, None if b is None else H.torch_to_bits(b), dt, bits, g)
    assert H.rel_l2(H.bits_to_f32(H.torch_to_bits(out).reshape(-1, N), dt), H.bits_to_f32(rT, dt)) <= TOL
    # and the reference's own criterion: close to the dense layer it replaces
    dense = (x.float().reshape(-1, K) @ w.float()) + (0 if b is None else b.float())
    atol = 1e-2 if (dt == H.F16 and bits == 8) else 0.13
    assert torch.allclose(out.float().reshape(-1, N), dense, rtol=1e-5, atol=atol)
    # dequantise returns [K, N] in the requested dtype, bit-exact with the oracle
    back = Q.weight_dequantize(codes, scale, algo=algo, out_dtype=H.DT_NAMES[dt], group_size=g)
    _, oT = oracle.dequantize(oc, osc, dt, bits, g)
    assert np.array_equal(H.torch_to_bits(back), oT)


def test_baseline_config_1_int8_per_channel(G, oracle):
    # x [1,4096] bf16, W [4096,4096] int8 per-channel, bias zeros
    e32, eT = check(G, oracle, H.BF16, 8, -1, 1, 4096, 4096, bias=False, seed=1234)
    print("config 1 rel-L2: fp32 %.2e, bf16 %.2e" % (e32, eT))


@pytest.mark.parametrize("M", [1, 4, 16])
@pytest.mark.parametrize("KN", [(4096, 11008), (11008, 4096)])
def test_baseline_config_2_llama_ffn_int4(G, oracle, M, KN):
    check(G, oracle, H.BF16, 4, -1, M, KN[0], KN[1], bias=True, seed=1234)


def test_headline_decode_shape_int4_group128(G, oracle):
    check(G, oracle, H.BF16, 4, 128, 1, 4096, 11008, bias=False, seed=1234)


@pytest.mark.parametrize("M", [1, 8, 32, 64])
def test_baseline_config_3_groupwise_outliers(G, oracle, M):
    # [8192, 28672] is checked through properties below; the oracle-sized slice
    # keeps the outlier columns, group 128 and fp16
    check(G, oracle, H.F16, 4, 128, M, 8192, 2048, bias=False, seed=1234, outliers=0.01)


@pytest.mark.parametrize("M", [512, 2048])
def test_baseline_config_4_prefill_slice(G, oracle, M):
    # int8 per-channel prefill; N sliced to what the oracle finishes in seconds
    # (at 2048 rows the oracle multiplies three slices of 32 columns)
    if M <= 512:
        check(G, oracle, H.BF16, 8, -1, M, 4096, 768, bias=False, seed=1234)
    else:
        check_sampled(G, oracle, H.BF16, 8, -1, M, 4096, 768, bias=False, seed=1234, ncols=32)


@pytest.mark.parametrize("shape", [(8, 4096, 12288), (8, 4096, 4096), (8, 11008, 4096), (1024, 4096, 512)])
def test_baseline_config_5_int8_group64(G, oracle, shape):
    M, K, N = shape
    check(G, oracle, H.BF16, 8, 64, M, K, N if M < 64 else N, bias=False, seed=1234)


def test_baseline_config_5_as_a_sequence(device, oracle):
    # Configuration 5 the way it runs: the four linears of consecutive decoder
    # layers (int8, group 64, bf16, full K and N, every layer its own weights)
    # as a decode step at 8 rows, then one prefill chunk of 1024 rows, then the
    # decode step again, all enqueued back to back on one stream.  Every output
    # is checked against the oracle on its first columns (the quantiser and the
    # linear are column-wise, so a column slice of the oracle is exact), and the
    # two decode steps must agree bit for bit: nothing carries over between calls.
    import torch
    from paddle_amd.nn import quant as Q

    dt, g, cols = H.BF16, 64, 128
    shapes = [(4096, 12288), (4096, 4096), (4096, 22016), (11008, 4096)]
    gen = torch.Generator(device="cuda").manual_seed(55)
    layers = []
    for layer in range(2):
        for K, N in shapes:
            w = (torch.randn(K, N, device="cuda", generator=gen) * 0.02).to(torch.bfloat16)
            codes, scale = Q.weight_quantize(w, algo="weight_only_int8", group_size=g)
            layers.append((K, N, H.torch_to_bits(w[:, :cols].contiguous()), codes, scale))
            del w
    xs = {(M, K): (torch.randn(M, K, device="cuda", generator=gen)).to(torch.bfloat16)
          for M in (8, 1024) for K in (4096, 11008)}

    def step(M):
        return [Q.weight_only_linear(xs[(M, K)], codes, None, scale, "int8", None, g) for K, N, _, codes, scale in layers]

    d1 = step(8)
    pf = step(1024)
    d2 = step(8)
    torch.cuda.synchronize()
    for i, (K, N, wb, codes, scale) in enumerate(layers):
        oc, osc = oracle.weight_quantize(wb, dt, 8, g)
        assert np.array_equal(H.torch_to_bits(scale[:, :cols].contiguous()), osc)
        for M, outs in ((8, d1), (1024, pf)):
            rows = 64 if M > 64 else M  # the oracle is scalar code
            xb = H.torch_to_bits(xs[(M, K)][:rows].contiguous())
            _, wantT = oracle.linear(xb, oc, osc, None, dt, 8, g)
            got = H.bits_to_f32(H.torch_to_bits(outs[i][:rows, :cols].contiguous()), dt)
            err = H.rel_l2(got, H.bits_to_f32(wantT, dt))
            assert err <= TOL, (err, i, M, K, N)
        assert torch.equal(d1[i], d2[i]), (i, K, N)


# ---- full-size properties (no oracle needed: size-independent identities) ----
def _full_size_properties(dt, bits, g, M, K, N, outliers=0.0):
    import torch

    from paddle_amd.nn import quant as Q
    from paddle_amd.nn.quant import quantized_linear as QL

    tdt = H.torch_dtype(dt)
    gen = torch.Generator(device="cuda").manual_seed(1234)
    w = torch.randn(K, N, device="cuda", generator=gen) * 0.02
    if outliers:
        cols = torch.randperm(N, device="cuda", generator=gen)[: int(np.ceil(outliers * N))]
        w[:, cols] *= 20.0
    w = w.to(tdt)
    algo = "weight_only_int8" if bits == 8 else "weight_only_int4"
    wd = "int8" if bits == 8 else "int4"
    codes, scale = Q.weight_quantize(w, algo=algo, group_size=g)
    wdq = Q.weight_dequantize(codes, scale, algo=algo, out_dtype=H.DT_NAMES[dt], group_size=g)
    x = torch.randn(M, K, device="cuda", generator=gen).to(tdt)
    out32 = QL.weight_only_linear_fp32(x, codes, None, scale, wd, g)
    # (1) against torch's fp32 matmul of the fp32 dequantised weight, built here
    #     from the canonical codes (wol_repack, a bijection the small tests pin)
    #     times the scales, without any rounding to T -- the same quantity the
    #     oracle forms, so the path's own 1e-3 bar applies to both dtypes.
    from paddle_amd.nn.quant.packed_weights import convert_weight_layout

    canon = convert_weight_layout(codes, wd, "gfx950", "canonical")
    if bits == 8:
        q = canon.float()
    else:
        b = canon.view(torch.uint8).to(torch.int16)
        lo, hi = b & 15, b >> 4
        q = torch.stack([lo, hi], dim=2).reshape(K, N)
        q = (q - 16 * (q > 7)).float()
    sc = scale.float()
    w32 = q * (sc if g == -1 else sc.repeat_interleave(g, dim=0)[:K])
    del q, canon
    # the T-rounded dequantised weight of the library is the rounding of that one
    assert torch.equal(w32.to(tdt), wdq)
    hi_prec = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    ref = x.float() @ w32
    torch.backends.cuda.matmul.allow_tf32 = hi_prec
    del w32
    err = float((out32 - ref).norm() / ref.norm())
    assert err <= 1e-3, err
    # (2) one-hot activations read back dequantised rows exactly (before their cast)
    ks = [0, 1, 63, 64, 127, 128, K // 2 + 5, K - 1][: max(1, min(8, M))]
    onehot = torch.zeros(len(ks), K, device="cuda", dtype=tdt)
    for i, k in enumerate(ks):
        onehot[i, k] = 1.0
    rows = QL.weight_only_linear_fp32(onehot, codes, None, scale, wd, g)
    assert torch.equal(rows.to(tdt), wdq[ks])
    # (3) linearity in x: f(2x) == 2 f(x) exactly (powers of two commute with every rounding)
    out2 = QL.weight_only_linear_fp32((x.float() * 2).to(tdt), codes, None, scale, wd, g)
    assert torch.equal(out2, out32 * 2)
    # (4) the bias is added after accumulation
    bias = (torch.randn(N, device="cuda", generator=gen) * 0.01).to(tdt)
    outb = QL.weight_only_linear_fp32(x, codes, bias, scale, wd, g)
    assert torch.allclose(outb, out32 + bias.float(), rtol=0, atol=1e-6 * float(out32.abs().max()))
    # (5) the T output is the rounded accumulator
    outT = Q.weight_only_linear(x, codes, None, scale, wd, None, g)
    assert torch.equal(outT, out32.to(tdt))


def test_calls_replay_correctly_from_a_hip_graph(device):
    # Every entry point is stream-ordered and allocation-free, so a captured
    # sequence must replay to the eager results: quantise (per-channel, with its
    # scratch), decode, the small-M GEMM with its K runs and reduction, the
    # prefill GEMM, llm_int8_linear.  Replayed three times with eager work in between.
    import torch
    from paddle_amd import _lib
    from paddle_amd.nn import quant as Q

    dev = torch.device("cuda:0")
    K, N = 2048, 1024
    gen = torch.Generator(device="cuda").manual_seed(3)
    w = (torch.randn(K, N, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
    xs = {M: torch.randn(M, K, device=dev, generator=gen).to(torch.bfloat16) for M in (1, 40, 300)}

    def work():
        codes, scale = Q.weight_quantize(w, algo="weight_only_int8", group_size=-1)
        c4, s4 = Q.weight_quantize(w, algo="weight_only_int4", group_size=128)
        outs = [Q.weight_only_linear(x, codes, None, scale, "int8", None, -1) for x in xs.values()]
        outs += [Q.weight_only_linear(x, c4, None, s4, "int4", None, 128) for x in xs.values()]
        # llm_int8_linear: one row (single-workgroup activation stages, K runs), 40 rows (K runs, with
        # threshold 3 more outlier columns than the epilogue takes: the outlier kernel), 300 rows (fused)
        lw, ls = Q.weight_quantize(w, algo="llm.int8")
        outs += [Q.llm_int8_linear(x, lw, None, ls, 3.0) for x in xs.values()]
        # the quantiser that brings its own scratch (the eager pass below is its warm-up call)
        cst = torch.empty(K * N, dtype=torch.uint8, device=dev)
        sst = torch.empty(N, dtype=torch.bfloat16, device=dev)
        _lib.check(_lib.lib.wol_quantize_static(w.data_ptr(), _lib.DTYPE_BF16, K, N, 8, -1, _lib.ROUND_RNE,
                                                _lib.LAYOUT_GFX950, cst.data_ptr(), sst.data_ptr(),
                                                torch.cuda.current_stream().cuda_stream))
        return [codes, scale, c4, s4, lw, ls, cst, sst] + outs

    eager = [t.clone() for t in work()]
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        captured = work()
    for rep in range(3):
        for t in captured:
            t.zero_()
        _ = work()  # eager work between the replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for a, b in zip(eager, captured):
            assert torch.equal(a, b), rep


def test_fused_grad_moe_and_batched_decode_replay_from_a_hip_graph(device):
    # the same for the batched decode kernel (in one launch, and with K runs and
    # the kernel that adds them), the fused linear (pre-scale folded
    # into the loads, gelu, swiglu through its pass), weight_only_linear_grad
    # (its prepare launches and the GEMM) and the MoE expert FFN (table built on
    # the device): replayed three times with eager work in between
    import torch
    from paddle_amd.nn import quant as Q
    from paddle_amd.nn.quant import quantized_linear as QL

    dev = torch.device("cuda:0")
    K, N = 2048, 12288
    gen = torch.Generator(device="cuda").manual_seed(4)
    w = (torch.randn(K, N, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
    codes, scale = Q.weight_quantize(w, algo="weight_only_int8", group_size=64)
    c4, s4 = Q.weight_quantize(w, algo="weight_only_int4", group_size=-1)
    xs = {M: torch.randn(M, K, device=dev, generator=gen).to(torch.bfloat16) for M in (1, 8, 200)}
    x24 = torch.randn(24, K, device=dev, generator=gen).to(torch.bfloat16)
    pre = (0.5 + torch.rand(K, device=dev, generator=gen)).to(torch.bfloat16)
    gos = {M: torch.randn(M, N, device=dev, generator=gen).to(torch.bfloat16) for M in (8, 300)}
    E, hidden, inter = 4, 256, 512
    w1 = (torch.randn(E, hidden, inter, device=dev, generator=gen) * 0.05).to(torch.bfloat16)
    w2 = (torch.randn(E, inter // 2, hidden, device=dev, generator=gen) * 0.05).to(torch.bfloat16)
    q1, s1 = Q.moe_quantize_experts(w1)
    q2, s2 = Q.moe_quantize_experts(w2)
    tokens = torch.randn(300, hidden, device=dev, generator=gen).to(torch.bfloat16)
    cum = torch.tensor([40, 40, 171, 300], dtype=torch.int64, device=dev)

    def work():
        outs = [Q.weight_only_linear(xs[8], codes, None, scale, "int8", None, 64)]  # batched decode kernel
        outs.append(Q.weight_only_linear(x24, codes, None, scale, "int8", None, 64))  # the same with K runs + reduce
        for M, x in xs.items():
            outs.append(Q.weight_only_linear_fused(x, codes, None, scale, "int8", 64, pre_scale=pre, act="gelu"))
            outs.append(Q.weight_only_linear_fused(x, c4, None, s4, "int4", -1, pre_scale=None, act="swiglu"))
        for M, go in gos.items():
            x_like = torch.empty((M, K), dtype=go.dtype, device="meta")
            outs.append(QL.weight_only_linear_grad(x_like, codes, None, scale, go, "int8", None, 64))
            outs.append(QL.weight_only_linear_grad(x_like, c4, None, s4, go, "int4", None, -1))
        outs.append(Q.moe_ffn(tokens, cum, q1, q2, None, s1, s2, "weight_only_int8"))
        return outs

    eager = [t.clone() for t in work()]
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        captured = work()
    for rep in range(3):
        for t in captured:
            t.zero_()
        _ = work()  # eager work between the replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(eager, captured)):
            assert torch.equal(a, b), (rep, i)


def test_weight_larger_than_2_gib(device):
    # byte offsets beyond 2^31: a 8192 x 327680 int8 weight (2.7 GB of codes).
    # One-hot activations must read back the dequantised rows, also at the far
    # end of the tensor, on the streaming kernel (M = 4) and the GEMM (M = 80).
    import torch
    from paddle_amd.nn import quant as Q
    from paddle_amd.nn.quant import quantized_linear as QL

    K, N = 8192, 327680
    gen = torch.Generator(device="cuda").manual_seed(7)
    w = torch.empty(K, N, device="cuda", dtype=torch.bfloat16)
    for k0 in range(0, K, 1024):  # in slabs: randn has no bf16 generator path for 2.7 G elements at once
        w[k0:k0 + 1024] = (torch.randn(1024, N, device="cuda", generator=gen) * 0.02).to(torch.bfloat16)
    codes, scale = Q.weight_quantize(w, algo="weight_only_int8", group_size=128)
    assert codes.numel() > 2 ** 31
    wdq = Q.weight_dequantize(codes, scale, algo="weight_only_int8", out_dtype="bfloat16", group_size=128)
    del w
    for M in (4, 80):
        ks = [0, 1, K // 2 + 3, K - 1][: min(4, M)]
        onehot = torch.zeros(M, K, device="cuda", dtype=torch.bfloat16)
        for i, k in enumerate(ks):
            onehot[i, k] = 1.0
        rows = QL.weight_only_linear_fp32(onehot, codes, None, scale, "int8", 128)
        if M == 4:
            assert torch.equal(rows[: len(ks)].to(torch.bfloat16), wdq[ks])
        else:
            # the GEMM keeps its sums in units of the current group's scale and
            # rescales them from group to group (a rounding of 2^-24 each time),
            # so a row comes back to within a few fp32 ulps of code * scale: half
            # a bf16 ulp (2^-8 relative at most) from the rounded value, and a little
            want = wdq[ks].float()
            assert bool(((rows[: len(ks)] - want).abs() <= want.abs() * (2.0 ** -8 + 1e-5)).all())
            assert bool((rows[: len(ks)] != 0).eq(want != 0).all())
        assert not rows[len(ks):].any()


@pytest.mark.parametrize("M", [1, 8, 32, 64])
def test_config_3_full_size_properties(device, M):
    _full_size_properties(H.F16, 4, 128, M, 8192, 28672, outliers=0.01)


@pytest.mark.parametrize("M", [512, 2048, 8192])
def test_config_4_full_size_properties(device, M):
    _full_size_properties(H.BF16, 8, -1, M, 4096, 12288)


@pytest.mark.parametrize("dt", [H.BF16, H.F16])
def test_int4_prefill_full_size_properties(device, dt):
    # int4 per-channel at prefill size: 256 x 256 tiles on the columns of whole
    # rounds (bf16: offset dequantiser with row sums by dot products; fp16: the
    # exact dequantiser), 128 x 256 tiles on the rest
    from paddle_amd import _lib
    import ctypes

    buf = ctypes.create_string_buffer(256)
    assert _lib.lib.wol_linear_plan(2048, 4096, 12288, 4, -1, 0, buf, 256) == 0 and b"256x256" in buf.value
    _full_size_properties(dt, 4, -1, 2048, 4096, 12288)


@pytest.mark.parametrize("shape", [(8, 4096, 22016), (1024, 4096, 22016), (1024, 11008, 4096), (1024, 4096, 12288)])
def test_config_5_full_size_properties(device, shape):
    _full_size_properties(H.BF16, 8, 64, *shape)


@pytest.mark.parametrize("bits,g", [(4, 128), (8, -1), (4, 64)])
def test_strip_numbering_around_whole_rounds_of_workgroups(device, oracle, bits, g):
    # The streaming kernel hands its strips to workgroups in an order that
    # follows the CUs (257 to 1024 workgroups) or the XCDs (otherwise): strip
    # counts on both sides of every switch and of whole rounds of 256, at row
    # counts that take every all-at-once split.  Device-made weights, the oracle
    # on the strips where a wrong numbering would show (first, last, around the
    # multiples of 256 and of 32) and on a few others.
    import torch
    import gpu_calls as G
    from paddle_amd.nn import quant as Q

    dt, K = H.BF16, 2048
    rng = np.random.default_rng(bits * 100 + (g if g > 0 else 0))
    for strips in (255, 256, 257, 300, 511, 512, 513, 688, 1023, 1024, 1025, 1100):
        N = strips * 16
        gen = torch.Generator(device="cuda").manual_seed(strips)
        w = (torch.randn(K, N, device="cuda", generator=gen) * 0.02).to(H.torch_dtype(dt))
        codes, scale = Q.weight_quantize(w, algo="weight_only_int8" if bits == 8 else "weight_only_int4", group_size=g)
        picks = sorted(set([0, 1, 2, 3, 31, 32, 33, 255, 256, 257, 258, 511, 512, 513, 767, 768, 769, strips - 34, strips - 33,
                            strips - 2, strips - 1] + [int(v) for v in rng.integers(0, strips, 8)]))
        picks = [s_ for s_ in picks if 0 <= s_ < strips]
        cols = np.concatenate([np.arange(s_ * 16, s_ * 16 + 16) for s_ in picks])
        oc, osc = oracle.weight_quantize(H.torch_to_bits(w[:, cols].contiguous()), dt, bits, g)
        assert np.array_equal(osc, H.torch_to_bits(scale[..., cols].contiguous()))
        for M in (1, 2, 5):
            xb = H.make_act(M, K, dt, seed=strips + M)
            bb = H.make_bias(N, dt, seed=strips)
            out = G.linear_dev(H.bits_to_torch(xb, dt, "cuda:0"), codes, H.bits_to_torch(bb, dt, "cuda:0"), scale, dt, N,
                               bits, g, kernel=KERNEL_STREAM)
            got = H.torch_to_bits(out)
            # every strip is written: none keeps the NaN the output was filled with (a strip computed
            # in another's place fails the slices below)
            assert np.isfinite(H.bits_to_f32(got, dt)).all()
            _, wantT = oracle.linear(xb, oc, osc, bb[cols], dt, bits, g)
            err = H.rel_l2(H.bits_to_f32(got[:, cols], dt), H.bits_to_f32(wantT, dt))
            assert err <= 1e-3, (err, strips, M, bits, g)


def test_empty_batch_and_leading_dims(device):
    import torch

    from paddle_amd.nn import quant as Q

    w = (torch.randn(128, 64, device="cuda") * 0.02).half()
    codes, scale = Q.weight_quantize(w)
    out = Q.weight_only_linear(torch.zeros(0, 128, device="cuda", dtype=torch.float16), codes, weight_scale=scale)
    assert list(out.shape) == [0, 64]
    x = torch.randn(2, 3, 5, 128, device="cuda").half()
    out = Q.weight_only_linear(x, codes, weight_scale=scale)
    flat = Q.weight_only_linear(x.reshape(-1, 128), codes, weight_scale=scale)
    assert list(out.shape) == [2, 3, 5, 64] and torch.equal(out.reshape(-1, 64), flat)


def test_mfma_probe_variants_run(device):
    # the measurement aid behind bench.py's inner-loop ladder: every variant
    # launches, finishes and leaves finite sums (two workgroups, three k tiles)
    import torch
    from paddle_amd import _lib

    need = 64 * 8 * 49152 + 65536
    ops = (torch.randn(need // 2, device=device) * 0.5).to(torch.bfloat16)
    out = torch.full((2 * 512,), float("nan"), device=device)
    for v in range(9):
        out.fill_(float("nan"))
        _lib.check(_lib.lib.wol_mfma_probe(v, ops.data_ptr(), need, 2, 3, out.data_ptr(), None))
        torch.cuda.synchronize()
        assert bool(torch.isfinite(out).all()), v


def test_decode_phases_counts_and_output(device):
    # the clock-stamped instantiation of the headline decode kernel: its output
    # is the product's bit for bit and every wavefront's phases add up
    import torch
    from paddle_amd import _lib
    from paddle_amd.nn import quant as Q

    K, N = 4096, 1024
    gen = torch.Generator(device="cuda").manual_seed(6)
    w = (torch.randn(K, N, device="cuda", generator=gen) * 0.02).to(torch.bfloat16)
    x = torch.randn(1, K, device="cuda", generator=gen).to(torch.bfloat16)
    for g in (64, 128):
        codes, scale = Q.weight_quantize(w, algo="weight_only_int4", group_size=g)
        want = Q.weight_only_linear(x, codes, None, scale, "int4", None, g)
        out = torch.full((1, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        ph = torch.zeros(N // 16 * 64, dtype=torch.int64, device="cuda")
        _lib.check(_lib.lib.wol_decode_phases(x.data_ptr(), codes.data_ptr(), scale.data_ptr(), K, N, g, out.data_ptr(),
                                              ph.data_ptr(), ph.numel() * 8, None))
        torch.cuda.synchronize()
        assert torch.equal(out, want)
        c = ph.cpu().numpy().reshape(-1, 8)
        assert (c[:, 1] >= c[:, 0]).all() and (c[:, 2:8] > 0).all() and (c[:, 2:8].sum(axis=1) < 10 ** 8).all()
        # the device's 100 MHz clock and the shader cycles tell the same story: 0.5 to 3 GHz
        life_us = (c[:, 1] - c[:, 0]) * 0.01
        long_ = life_us > 1.0
        if long_.any():
            ghz = c[long_, 2:8].sum(axis=1) / life_us[long_] / 1e3
            assert 0.5 < ghz.mean() < 3.0


def test_prefill_phases_counts_and_output(device):
    # the cycle-stamped instantiation of the prefill GEMM: its output is the
    # product's bit for bit, and every wavefront's counts add up (the phases
    # between entry and end sum to the total, the k-tile count is K / 64)
    import torch
    from paddle_amd import _lib
    from paddle_amd.nn import quant as Q

    import ctypes

    M, K, N = 2048, 256, 8192  # 256 tiles of 256 x 256: what wol_linear launches for this shape, in one piece
    plan = ctypes.create_string_buffer(256)
    _lib.check(_lib.lib.wol_linear_plan(M, K, N, 8, -1, 0, plan, 256))
    assert plan.value.endswith(b"256x256 tiles on columns [0,8192)"), plan.value
    gen = torch.Generator(device="cuda").manual_seed(5)
    w = (torch.randn(K, N, device="cuda", generator=gen) * 0.02).to(torch.bfloat16)
    x = torch.randn(M, K, device="cuda", generator=gen).to(torch.bfloat16)
    codes, scale = Q.weight_quantize(w, algo="weight_only_int8")
    want = Q.weight_only_linear(x, codes, None, scale, "int8")
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    wgs = (M // 256) * (N // 256)
    ph = torch.zeros(wgs * 64, dtype=torch.int64, device="cuda")
    _lib.check(_lib.lib.wol_prefill_phases(x.data_ptr(), codes.data_ptr(), scale.data_ptr(), M, K, N, out.data_ptr(),
                                           ph.data_ptr(), ph.numel() * 8, None))
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    c = ph.cpu().numpy().reshape(wgs * 8, 8)
    assert (c[:, 7] == K // 64).all()
    assert (c[:, :7] > 0).all() and (c[:, 6] < 10 ** 9).all()
    assert (c[:, 0:6].sum(axis=1) == c[:, 6]).all()


def test_read_floor_reads_every_byte_once(device):
    # the measurement aid behind bench.py's read_floor: each wavefront XORs the
    # dwords of its eighth of a strip
    import torch
    from paddle_amd import _lib

    K, N, bits = 2048, 96, 8
    rng = np.random.default_rng(5)
    codes = rng.integers(0, 256, K * N, dtype=np.uint8)
    d = torch.from_numpy(codes).to(device)
    out = torch.zeros(N // 16 * 8, dtype=torch.int32, device=device)
    _lib.check(_lib.lib.wol_read_floor(d.data_ptr(), K, N, bits, out.data_ptr(), None))
    torch.cuda.synchronize()
    got = out.cpu().numpy().view(np.uint32)
    # lane 0 of a wavefront holds the XOR over the lane-0 pieces only: 4 dwords of every 64 x 4
    per_wave = codes.view(np.uint32).reshape(N // 16 * 8, -1, 64, 4)[:, :, 0, :]
    want = np.bitwise_xor.reduce(per_wave.reshape(per_wave.shape[0], -1), axis=1)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("bits", [8, 4])
def test_stream_kernel_every_k_tail(G, oracle, bits):
    # every K from 64 to 2560 in steps of 64 at the row counts whose units span
    # several weight tiles (1, 2 and 4 rows): whole units, a partial unit, the
    # int4 half tile and their combinations, with one wavefront and with many
    # (N = 64 gives 4 strips, so K decides the wavefront count)
    N = 64
    for K in range(64, 2561, 64):
        for M, g in ((1, -1), (2, 64), (4, 128 if K % 128 == 0 else 64)):
            print("case", bits, K, M, g, flush=True)
            check(G, oracle, H.BF16 if (K // 64) % 2 else H.F16, bits, g, M, K, N, bias=(K // 64) % 3 == 0,
                  seed=K + M, kernel=KERNEL_STREAM)


@pytest.mark.parametrize("dt,bits,g,M,K,N", [(H.BF16, 8, 64, 700, 2048, 22016), (H.F16, 4, 128, 300, 4096, 22016)])
def test_gemm_partial_last_round_split(G, oracle, dt, bits, g, M, K, N):
    # above 64 rows the tiles of a partial last round are launched with K cut
    # into runs: their columns go through fp32 partial sums and a reduce over
    # that column range only.  Checked against the same call without scratch
    # (one launch, no split) and, on a few rows, against the oracle.
    from paddle_amd import _lib

    need = _lib.lib.wol_linear_workspace(M, K, N, bits, g)
    assert 0 < need < 2 * 4 * M * N  # a split of some of the columns only
    wb = H.make_weight(K, N, dt, seed=31)
    xb = H.make_act(M, K, dt, seed=32)
    bb = H.make_bias(N, dt, seed=33)
    oc, osc = oracle.weight_quantize(wb, dt, bits, g)
    packed = H.gfx950_from_q(H.q_from_canonical(oc, bits), bits)
    split32 = G.linear(xb, packed, bb, osc, dt, N, bits, g, f32=True)
    plain32 = G.linear(xb, packed, bb, osc, dt, N, bits, g, f32=True, no_workspace=True)
    assert np.isfinite(split32).all()
    assert H.rel_l2(split32, plain32) < 2e-6  # the same products, summed in another order
    # the columns outside the split are bit-identical
    same = (split32 == plain32).all(axis=0)
    assert same.sum() >= N // 2
    splitT = G.linear(xb, packed, bb, osc, dt, N, bits, g)
    assert np.array_equal(splitT, H.f32_to_bits(split32, dt))
    rows = np.r_[0:3, M - 3:M]
    r32, _ = oracle.linear(xb[rows], oc, osc, bb, dt, bits, g)
    assert H.rel_l2(split32[rows], r32) < 2e-5


@pytest.mark.parametrize("dt,bits,g,M,K,N,spread", [
    (H.BF16, 8, 64, 700, 2048, 22016, (-12, 4)),    # 256 x 256 tiles + a 256 x 128 remainder with K in runs
    (H.F16, 8, 128, 300, 2112, 4096, (-8, 3)),      # groups of two k tiles, an odd number of tiles, K in runs of whole groups
    (H.BF16, 8, 128, 300, 2048, 8192, (-100, 20)),  # scales of a column further apart than fp32 sums can span
    (H.BF16, 4, 64, 300, 4096, 4096, (-12, 4)),     # int4: 128 x 256 tiles, two groups per k tile
    (H.F16, 4, 128, 130, 2048, 4096, (-8, 3)),      # int4: 256 x 128 tiles
])
def test_group_wise_gemm_keeps_its_sums_in_units_of_the_group_scale(G, oracle, dt, bits, g, M, K, N, spread):
    # above 64 rows the GEMM has one set of accumulators for group-wise scales: the
    # sums are multiplied by (previous unit / new unit) where a group starts and by
    # the last unit at the end.  Weights whose groups differ by many powers of two
    # inside a column, with all-zero groups (scale 0) at the start, in the middle
    # and at the end of K: every column must still match the oracle's fp32 sums,
    # column by column (a whole-matrix norm would hide the small columns).
    rng = np.random.default_rng(K + N + M)
    ng = (K + g - 1) // g
    lo, hi = spread
    e = rng.integers(lo, hi + 1, size=(ng, N)).astype(np.float32)
    if lo < -64:  # mostly ordinary groups, a few absurdly small or large ones
        e = np.where(rng.random((ng, N)) < 0.8, rng.integers(-4, 3, size=(ng, N)), e).astype(np.float32)
    mag = np.exp2(e)
    mag[rng.random((ng, N)) < 0.1] = 0.0
    mag[0, : N // 3] = 0.0       # columns that start with a zero group
    mag[-1, N // 4 : N // 2] = 0.0  # ... and end with one
    mag[:, 5] = 0.0              # an all-zero column
    w = rng.standard_normal((K, N), dtype=np.float32) * 0.02 * np.repeat(mag, g, axis=0)[:K]
    wb = H.f32_to_bits(w, dt)
    xb = H.make_act(M, K, dt, seed=M)
    oc, osc = oracle.weight_quantize(wb, dt, bits, g)
    packed = H.gfx950_from_q(H.q_from_canonical(oc, bits), bits)
    got = G.linear(xb, packed, None, osc, dt, N, bits, g, f32=True)
    assert np.isfinite(got).all()
    rows = np.r_[0:4, M // 2:M // 2 + 2, M - 3:M]
    want, _ = oracle.linear(xb[rows], oc, osc, None, dt, bits, g)
    err = np.linalg.norm(got[rows] - want, axis=0)
    ref = np.linalg.norm(want, axis=0)
    assert (got[:, 5] == 0).all() and (err[ref == 0] == 0).all()
    worst = (err[ref > 0] / ref[ref > 0]).max()
    assert worst < 2e-5, worst
    # the same through T outputs and with K in runs where the plan has them (the scratch decides)
    gotT = G.linear(xb, packed, None, osc, dt, N, bits, g)
    assert np.array_equal(gotT, H.f32_to_bits(got, dt))
    plain = G.linear(xb, packed, None, osc, dt, N, bits, g, f32=True, no_workspace=True)
    errp = np.linalg.norm(plain[rows] - want, axis=0)
    assert (errp[ref > 0] / ref[ref > 0]).max() < 2e-5


def test_call_log_names_the_kernel(device):
    # WOL_LOG=1: one line per call on stderr with the problem and the kernel taken
    # (read once per process, hence a child process)
    import os
    import subprocess
    import sys

    code = (
        "import torch\n"
        "from paddle_amd.nn import quant as Q\n"
        "w = (torch.randn(2048, 12288, device='cuda') * 0.02).to(torch.bfloat16)\n"
        "c, s = Q.weight_quantize(w, algo='weight_only_int8')\n"
        "for M in (1, 12, 300):\n"
        "    Q.weight_only_linear(torch.randn(M, 2048, device='cuda').to(torch.bfloat16), c, None, s, 'int8')\n"
        "torch.cuda.synchronize()\n"
    )
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", code], env=dict(os.environ, WOL_LOG="1", PYTHONPATH=root),
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [ln for ln in r.stderr.splitlines() if ln.startswith("[wol] linear ")]
    assert len(lines) == 3
    assert "M=1 K=2048 N=12288 int8" in lines[0] and lines[0].endswith("-> stream kernel")
    assert lines[1].endswith("-> batch kernel") and lines[2].endswith("-> gemm kernel")


def test_roctx_ranges_do_not_disturb_the_calls(device):
    # WOL_ROCTX=1: every compute call pushes and pops a roctx range (the marker
    # library is loaded at the first call); results are what they are without
    # it.  Read once per process, hence a child process.
    import os
    import subprocess
    import sys

    code = (
        "import torch\n"
        "from paddle_amd.nn import quant as Q\n"
        "g = torch.Generator(device='cuda').manual_seed(1)\n"
        "w = (torch.randn(2048, 1024, device='cuda', generator=g) * 0.02).to(torch.bfloat16)\n"
        "c, s = Q.weight_quantize(w, algo='weight_only_int8')\n"
        "x = torch.randn(8, 2048, device='cuda', generator=g).to(torch.bfloat16)\n"
        "y = Q.weight_only_linear(x, c, None, s, 'int8')\n"
        "torch.cuda.synchronize()\n"
        "print(float(y.float().abs().sum()))\n"
    )
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    outs = []
    for flag in ("0", "1"):
        r = subprocess.run([sys.executable, "-c", code], env=dict(os.environ, WOL_ROCTX=flag, PYTHONPATH=root),
                           capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stderr[-2000:]
        outs.append(r.stdout.strip().splitlines()[-1])
    assert outs[0] == outs[1]

