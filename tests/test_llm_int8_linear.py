"""llm_int8_linear: the oracle against an independent numpy statement, the
reference test's own expectation and invariants (CPU), and the HIP path against
the oracle, bit for bit, through the C ABI (GPU).

The reference's test (test/quantization/test_llm_int8_linear.py:34-180) draws
x from U(0, 1) with threshold 6.0, so it never reaches the outlier branch; it
compares with a dense matmul at atol 1e-1.  Its expectation for outliers
(:84-111) multiplies the outlier columns of x with the matching weight rows in
T, which is what the oracle and the kernel do.  PARITY UNPINNED for that
branch against the reference's CUDA kernel, whose weight indexing there
belongs to another layout (impl/llm_int8_matmul_kernel_impl.h:351-362)."""
import numpy as np
import pytest

import helpers as H


def _weights(K, N, dt, seed):
    """[N,K] int8 codes and fp32 scales as weight_quantize(algo="llm.int8")
    returns them (numpy statement of the quantiser)."""
    wb = H.make_weight(K, N, dt, seed=seed)
    q, scale = H.np_quantize_llm_int8(wb, dt, -1)
    return wb, np.ascontiguousarray(q.T.astype(np.int8)), scale.astype(np.float32)


def _act(M, K, dt, seed, kind):
    rng = np.random.default_rng(seed)
    if kind == "uniform":  # the reference test's activations: no outliers at threshold 6
        x = rng.random((M, K), dtype=np.float32)
    elif kind == "normal":
        x = rng.standard_normal((M, K), dtype=np.float32)
    else:  # "spiky": a few columns carry large values in some rows, as LLM activations do
        x = rng.standard_normal((M, K), dtype=np.float32)
        cols = rng.choice(K, size=max(1, K // 100), replace=False)
        rows = rng.random((M, cols.size)) < 0.5
        x[:, cols] = np.where(rows, x[:, cols] * np.float32(12.0), x[:, cols])
    return H.f32_to_bits(x, dt)


def _adversarial_act(M, K, dt, seed):
    """Rows of zeros, negative zeros, one huge element, values on the threshold and on quantisation ties, tiny and
    subnormal rows: the corners of the activation quantiser."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((M, K), dtype=np.float32)
    x[0] = 0.0                                     # range 0: 0 * inf, codes 0
    x[1 % M] = -0.0
    x[2 % M, 5] = 6.0                              # exactly the threshold: not an outlier (compare is >)
    x[3 % M, 9] = 60000.0 if dt == H.F16 else 3.0e38
    x[4 % M] = np.float32(2.0 ** -20) * rng.standard_normal(K).astype(np.float32)   # tiny row
    x[5 % M] = np.float32(6.0e-8 if dt == H.F16 else 1.0e-39) * rng.integers(-3, 4, K).astype(np.float32)  # subnormal T
    x[6 % M] = np.float32(1.0)                     # every element the row maximum: codes 127
    x[6 % M, ::2] = np.float32(-0.5)               # x * 127 / range = -63.5: the only exact tie a power-of-two range has
    x[7 % M, :] = np.float32(-5.5)
    return H.f32_to_bits(x, dt)


def _round_half_away(a64):
    return np.sign(a64) * np.floor(np.abs(a64) + 0.5)


def np_llm_int8(xb, w_nk, bias_b, wscale, threshold, dt):
    """Independent numpy statement (no code shared with the C oracle)."""
    x = H.bits_to_f32(xb, dt)
    thr = H.bits_to_f32(H.f32_to_bits(np.array([threshold], np.float32), dt), dt)[0]
    ax = np.abs(x)
    big = ax > thr
    outlier = big.any(axis=0)
    ranges = np.where(big, np.float32(0), ax).max(axis=1).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        inv = (np.float32(1.0) / ranges).astype(np.float32)
        t = ((x * np.float32(127.0)).astype(np.float32) * inv[:, None]).astype(np.float32)
    t = _round_half_away(t.astype(np.float64))
    t = np.clip(t, -127, 127)
    t = np.where(np.isnan(t), 0.0, t)
    qx = np.where(outlier[None, :], 0, t).astype(np.int8)
    acc = qx.astype(np.int32) @ w_nk.T.astype(np.int32)
    sub = np.zeros(acc.shape, np.float32)
    for k in np.nonzero(outlier)[0]:  # ascending, fp32 running sum
        wd = H.bits_to_f32(H.f32_to_bits((w_nk[:, k].astype(np.float32) * wscale).astype(np.float32), dt), dt)
        sub = (sub + x[:, k:k + 1] * wd[None, :]).astype(np.float32)
    subT = H.bits_to_f32(H.f32_to_bits(sub, dt), dt)
    dq = (((acc.astype(np.float32) * ranges[:, None]).astype(np.float32) * wscale[None, :]).astype(np.float32)
          / np.float32(127.0)).astype(np.float32)
    dqT = H.bits_to_f32(H.f32_to_bits(dq, dt), dt)
    out = _cast_f64(subT.astype(np.float64) + dqT.astype(np.float64), dt)  # one rounding, as a T addition has
    if bias_b is not None:
        b = H.bits_to_f32(bias_b, dt)
        out = _cast_f64(H.bits_to_f32(out, dt).astype(np.float64) + b[None, :].astype(np.float64), dt)
    return {"out": out, "qx": qx, "acc": acc, "ranges": ranges, "outlier": outlier}


def _cast_f64(a64, dt):
    """float64 -> T with a single rounding."""
    import torch

    t = torch.from_numpy(np.ascontiguousarray(a64))
    return H.torch_to_bits(t.to(H.torch_dtype(dt)))


CASES = [  # M, K, N, kind, threshold, bias
    (32, 64, 128, "uniform", 6.0, True),     # the reference test's shape
    (2, 64, 32, "uniform", 6.0, True),       # the docstring example's shape
    (5, 128, 48, "normal", 2.0, True),       # many outlier columns
    (7, 256, 64, "spiky", 6.0, False),
    (33, 192, 80, "spiky", 6.0, True),
    (3, 64, 16, "normal", 0.0, True),        # every column an outlier: ranges 0
    (4, 64, 16, "normal", 100.0, False),     # none
]


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("case", CASES)
def test_oracle_matches_numpy_statement(oracle, dt, case):
    M, K, N, kind, thr, has_bias = case
    _, w_nk, ws = _weights(K, N, dt, seed=K + N)
    xb = _act(M, K, dt, seed=M, kind=kind)
    bb = H.make_bias(N, dt, seed=3, std=1.0) if has_bias else None
    o = oracle.llm_int8_linear(xb, w_nk, bb, ws, thr, dt)
    r = np_llm_int8(xb, w_nk, bb, ws, thr, dt)
    assert np.array_equal(o["outlier"], r["outlier"])
    assert np.array_equal(o["ranges"], r["ranges"])
    assert np.array_equal(o["qx"], r["qx"])
    assert np.array_equal(o["acc"], r["acc"])
    assert np.array_equal(o["out"], r["out"])
    if kind != "uniform" and thr < 100:
        assert r["outlier"].any()


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
def test_oracle_matches_numpy_statement_on_corner_cases(oracle, dt):
    M, K, N = 8, 128, 32
    _, w_nk, ws = _weights(K, N, dt, seed=21)
    xb = _adversarial_act(M, K, dt, seed=22)
    bb = H.make_bias(N, dt, seed=3, std=1.0)
    o = oracle.llm_int8_linear(xb, w_nk, bb, ws, 6.0, dt)
    r = np_llm_int8(xb, w_nk, bb, ws, 6.0, dt)
    for key in ("outlier", "ranges", "qx", "acc", "out"):
        assert np.array_equal(o[key], r[key]), key
    assert not o["qx"][0].any() and not o["qx"][1].any()
    assert not o["outlier"][5] and o["outlier"][9]
    assert set(np.unique(o["qx"][6][~o["outlier"]]).tolist()) <= {-64, 127}


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("M", [8, 40, 200])
def test_gpu_llm_int8_linear_corner_cases_bit_exact(device, oracle, dt, M):
    import gpu_calls as G

    K, N = 128, 48
    print("llm_int8 corner cases M", M, "dtype", dt, flush=True)
    _, w_nk, ws = _weights(K, N, dt, seed=21)
    xb = _adversarial_act(M, K, dt, seed=22)
    bb = H.make_bias(N, dt, seed=3, std=1.0)
    o = oracle.llm_int8_linear(xb, w_nk, bb, ws, 6.0, dt)
    got, st = G.llm_int8_linear(xb, w_nk, bb, ws, 6.0, dt, stages=True)
    assert np.array_equal(st["ranges"], o["ranges"])
    assert np.array_equal(st["outlier"], o["outlier"])
    assert np.array_equal(st["qx"], o["qx"])
    assert np.array_equal(got, o["out"])


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
def test_oracle_invariants_and_reference_expectation(oracle, dt):
    # the reference test's configuration: x in U(0,1), 32 tokens, 64 -> 128, bias
    M, K, N = 32, 64, 128
    wb, w_nk, ws = _weights(K, N, dt, seed=7)
    xb = _act(M, K, dt, seed=8, kind="uniform")
    bb = H.f32_to_bits(np.ones(N, np.float32), dt)
    o = oracle.llm_int8_linear(xb, w_nk, bb, ws, 6.0, dt)
    assert not o["outlier"].any()
    assert np.abs(o["qx"].astype(np.int32)).max(axis=1).tolist() == [127] * M  # every row reaches the bound
    x = H.bits_to_f32(xb, dt)
    assert np.array_equal(o["ranges"], np.abs(x).max(axis=1))
    dense = x.astype(np.float64) @ H.bits_to_f32(wb, dt).astype(np.float64) + 1.0
    np.testing.assert_allclose(H.bits_to_f32(o["out"], dt), dense, rtol=1e-5, atol=1e-1)  # the reference's tolerance
    # closed form without outliers: out = T(T(acc * range * scale / 127) + bias)
    acc = o["qx"].astype(np.int64) @ w_nk.T.astype(np.int64)
    assert np.array_equal(acc, o["acc"])
    # outlier columns: zero codes, and the output equals the T-arithmetic product when every column is one
    xs = _act(4, K, dt, seed=9, kind="normal")
    o2 = oracle.llm_int8_linear(xs, w_nk, None, ws, 0.0, dt)
    zero_cols = H.bits_to_f32(xs, dt) == 0
    assert o2["outlier"].all() or zero_cols.any()
    assert not o2["qx"].any() and not o2["acc"].any()
    wd = H.bits_to_f32(H.f32_to_bits(w_nk.astype(np.float32) * ws[:, None], dt), dt)
    want = H.bits_to_f32(xs, dt).astype(np.float64) @ wd.T.astype(np.float64)
    assert H.rel_l2(H.bits_to_f32(o2["out"], dt), want) < (2e-3 if dt == H.F16 else 1e-2)


def test_division_by_127_as_the_kernel_does_it(oracle):
    # q = v * RN(1/127); r = fma(-q, 127, v); q + r * RN(1/127): equal to v / 127.0f on all 2^32 floats (the full
    # sweep takes half a minute on eight cores and was run once); here every 1021st pattern, the values around
    # zero, the subnormal boundary, infinity and the int32 range the accumulators come from
    assert oracle.div127_fma_mismatches(0, 1021, (1 << 32) // 1021) == 0
    for first in (0x00000000, 0x80000000, 0x007FFF00, 0x7F7FFF00, 0xFF7FFF00, 0x4B000000, 0x4EFFFF00):
        assert oracle.div127_fma_mismatches(first, 1, 1 << 12) == 0


def test_infer_meta_checks():
    from paddle_amd.nn.quant import quantized_linear as QL

    assert QL.llm_int8_linear_infer_meta((1, 2, 64), (32, 64), (32,), (32,)) == (1, 2, 32)
    for bad in (((2, 64), (32, 48), None, (32,)), ((2, 64), (24, 64), None, (24,)), ((2, 72), (32, 72), None, (32,)),
                ((2, 64), (32, 64), None, (16,)), ((2, 64), (32, 64, 1), None, (32,))):
        with pytest.raises(ValueError, match="InvalidArgument"):
            QL.llm_int8_linear_infer_meta(*bad)


def test_c_abi_argument_errors():
    from paddle_amd import _lib

    L = _lib.lib
    assert L.wol_llm_int8_linear_workspace(4, 64, 16) > 0
    assert L.wol_llm_int8_linear_workspace(4, 48, 16) == 0  # K must be a multiple of 64
    assert L.wol_llm_int8_linear_workspace(4, 64, 8) == 0
    assert L.wol_llm_int8_linear(None, None, None, None, 6.0, 0, 4, 48, 16, None, None, 0, None) == 5
    assert L.wol_llm_int8_linear(None, None, None, None, 6.0, 2, 4, 64, 16, None, None, 0, None) == 2
    assert L.wol_llm_int8_linear(None, None, None, None, 6.0, 0, 0, 64, 16, None, None, 0, None) == 0  # empty batch
    assert L.wol_llm_int8_linear(None, None, None, None, 6.0, 0, 4, 64, 16, None, None, 0, None) == 1
    assert L.wol_llm_int8_linear(16, 16, None, 16, 6.0, 0, 4, 64, 16, 16, None, 0, None) == 8  # workspace missing
    assert L.wol_llm_int8_linear_workspace(4, 131072, 16) > 0
    assert L.wol_llm_int8_linear_workspace(4, 131072 + 64, 16) == 0  # int32 sums must not wrap
    assert L.wol_llm_int8_linear(16, 16, None, 16, 6.0, 0, 4, 131072 + 64, 16, 16, 16, 1 << 30, None) == 5
    assert L.wol_llm_int8_linear(16, 16, None, 16, 6.0, 0, 1 << 24, 64, 1 << 20, 16, 16, 1 << 30, None) == 5  # M * N above 2^40
    assert L.wol_llm_int8_linear(24, 16, None, 16, 6.0, 0, 4, 64, 16, 16, 16, 1 << 30, None) == 9  # x not 16-byte aligned


# ---------------------------------------------------------------------------
# GPU: the HIP path through the C ABI against the oracle, bit for bit
# ---------------------------------------------------------------------------
GPU_CASES = [  # M, K, N, kind, threshold, bias
    (32, 64, 128, "uniform", 6.0, True),      # the reference test's shape
    (2, 64, 32, "uniform", 6.0, True),
    (1, 256, 272, "spiky", 6.0, True),        # one row; N past one 256-column tile by 16
    (5, 128, 48, "normal", 2.0, True),        # many outlier columns
    (33, 192, 80, "spiky", 6.0, False),       # 64-row tile
    (100, 320, 400, "spiky", 6.0, True),      # 128-row tile, one run
    (130, 1024, 144, "spiky", 6.0, True),     # 256-row tile, fused epilogue, ragged in M and N
    (300, 512, 1040, "normal", 3.0, False),   # several row tiles, column tiles not a multiple of 8
    (257, 64, 2048, "spiky", 6.0, True),      # one k tile; column tiles spread over the XCD bands
    (3, 64, 16, "normal", 0.0, True),         # every column an outlier
    (16, 4096, 512, "spiky", 6.0, True),      # K cut into runs
    (1, 4096, 512, "spiky", 6.0, True),       # one row, K runs: the merge kernel multiplies the outlier columns itself
    (4, 2048, 256, "normal", 2.0, False),     # four rows, K runs, most columns outliers
    (128, 2048, 272, "spiky", 6.0, True),     # 128-row tile, two runs
    (700, 512, 8192, "spiky", 6.0, True),     # 256x256 tiles
]


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("case", GPU_CASES)
def test_gpu_llm_int8_linear_bit_exact(device, oracle, dt, case):
    import gpu_calls as G

    M, K, N, kind, thr, has_bias = case
    print("llm_int8 case", case, "dtype", dt, flush=True)
    _, w_nk, ws = _weights(K, N, dt, seed=K + N)
    xb = _act(M, K, dt, seed=M + 1, kind=kind)
    bb = H.make_bias(N, dt, seed=3, std=1.0) if has_bias else None
    o = oracle.llm_int8_linear(xb, w_nk, bb, ws, thr, dt)
    got, st = G.llm_int8_linear(xb, w_nk, bb, ws, thr, dt, stages=True)
    assert np.array_equal(st["outlier"], o["outlier"])
    assert st["count"] == int(o["outlier"].sum())
    assert np.array_equal(st["list"], np.nonzero(o["outlier"])[0])
    assert np.array_equal(st["ranges"], o["ranges"])
    assert np.array_equal(st["qx"], o["qx"])
    if st["acc"] is not None:
        assert np.array_equal(st["acc"], o["acc"])
    bad = np.nonzero(got != o["out"])
    assert bad[0].size == 0, "first mismatch at m=%d n=%d: %#x vs %#x (%d in all)" % (
        bad[0][0], bad[1][0], got[bad[0][0], bad[1][0]], o["out"][bad[0][0], bad[1][0]], bad[0].size)


@pytest.mark.gpu
@pytest.mark.parametrize("N", [12288, 8192])  # 128x256 tiles (three rounds of the CUs), 256x256 tiles (one round)
def test_gpu_llm_int8_linear_large_properties(device, oracle, N):
    """M = 2048, K = 4096, N = 12288 | 8192 (too large for the scalar oracle): rows
    checked against the oracle on a slice of the columns, and the whole result
    against a float64 statement of the no-outlier formula."""
    import gpu_calls as G

    dt, M, K = H.BF16, 2048, 4096
    rng = np.random.default_rng(5)
    w_nk = rng.integers(-127, 128, (N, K), dtype=np.int8)
    ws = (rng.random(N, dtype=np.float32) * np.float32(1e-3) + np.float32(1e-4)).astype(np.float32)
    xb = _act(M, K, dt, seed=6, kind="spiky")
    got, st = G.llm_int8_linear(xb, w_nk, None, ws, 6.0, dt, stages=True)
    assert st["count"] > 0
    cols = np.r_[0:32, 6000:6016, N - 16:N]
    rows = np.r_[0:8, 1000:1004, M - 4:M]
    o = oracle.llm_int8_linear(xb[rows], w_nk[cols], None, ws[cols], 6.0, dt)
    # the outlier columns depend on every row: the slice agrees only where the
    # slice's own outliers are the full problem's
    if np.array_equal(o["outlier"], st["outlier"]):
        assert np.array_equal(got[np.ix_(rows, cols)], o["out"])
    assert np.array_equal(st["qx"][rows][:, ~st["outlier"]], o["qx"][:, ~st["outlier"]])
    # whole result: float64 evaluation of sub + acc * range * scale / 127
    x = H.bits_to_f32(xb, dt).astype(np.float64)
    acc = st["qx"].astype(np.float32) @ w_nk.T.astype(np.float32)  # exact: |sums| < 2^24 is not guaranteed, so check loosely
    kk = st["list"]
    wd = H.bits_to_f32(H.f32_to_bits(w_nk[:, kk].astype(np.float32) * ws[:, None], dt), dt).astype(np.float64)
    want = x[:, kk] @ wd.T + acc.astype(np.float64) * st["ranges"][:, None].astype(np.float64) * ws[None, :] / 127.0
    assert H.rel_l2(H.bits_to_f32(got, dt), want) < 4e-3  # bf16 output rounding (2^-9 relative, twice)


@pytest.mark.gpu
def test_gpu_python_api_llm_int8_linear(device, oracle):
    import torch

    from paddle_amd.nn import quant as Q

    dt = H.F16
    wb = H.make_weight(64, 128, dt, seed=11)
    w = H.bits_to_torch(wb, dt, device)
    weight, scale = Q.weight_quantize(w, algo="llm.int8")
    assert weight.shape == (128, 64) and scale.dtype == torch.float32
    xb = _act(32, 64, dt, seed=12, kind="uniform").reshape(1, 32, 64)
    x = H.bits_to_torch(xb, dt, device)
    bias = torch.ones(128, dtype=torch.float16, device=device)
    out = Q.llm_int8_linear(x, weight, bias=bias, weight_scale=scale, threshold=6.0)
    assert out.shape == (1, 32, 128) and out.dtype == torch.float16
    dense = torch.matmul(x.float(), w.float()) + 1.0
    np.testing.assert_allclose(out.float().cpu().numpy(), dense.cpu().numpy(), rtol=1e-5, atol=1e-1)
    o = oracle.llm_int8_linear(xb.reshape(32, 64), weight.cpu().numpy(), H.torch_to_bits(bias), scale.cpu().numpy(),
                               6.0, dt)
    assert np.array_equal(H.torch_to_bits(out).reshape(32, 128), o["out"])
    assert Q.llm_int8_linear(x[:, :0], weight, None, scale).shape == (1, 0, 128)
    with pytest.raises(ValueError, match="InvalidArgument"):
        Q.llm_int8_linear(x[..., :48], weight, None, scale)
