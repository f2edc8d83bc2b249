"""x_grad of weight_only_linear (paddle/phi/kernels/gpu/weight_only_linear_grad_kernel.cu:27-72):
the oracle's wo_linear_grad pinned against a float64 product (no GPU), and
wol_linear_grad through the C ABI against the oracle."""
import numpy as np
import pytest

import helpers as H

TOL = 1e-3


# ---- the oracle, pinned without a GPU ---------------------------------------
@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("bits,g", [(8, -1), (4, -1), (8, 64), (4, 128)])
def test_oracle_linear_grad_against_float64_matmul(oracle, dt, bits, g):
    # the definition: out_grad [M,N] times the transpose of the fp32
    # dequantised weight [K,N], evaluated by numpy in float64.  A transposed
    # operand, a scale taken from the wrong group or a dropped rounding step
    # shows here: M, K and N all differ, and K spans several groups.
    M, K, N = 5, 256, 48
    wb = H.make_weight(K, N, dt, seed=3)
    oc, osc = oracle.weight_quantize(wb, dt, bits, g)
    w32, _ = oracle.dequantize(oc, osc, dt, bits, g)
    gb = H.make_act(M, N, dt, seed=4)
    want = H.bits_to_f32(gb, dt).astype(np.float64) @ w32.astype(np.float64).T
    o64, _ = oracle.linear_grad(gb, oc, osc, dt, bits, g, acc64=True)
    assert o64.shape == (M, K)
    assert np.array_equal(o64, want.astype(np.float32))
    o32, oT = oracle.linear_grad(gb, oc, osc, dt, bits, g, acc64=False)
    assert H.rel_l2(o32, want) < 2e-6
    assert np.array_equal(oT, H.f32_to_bits(o32, dt))


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
def test_oracle_reference_composition_of_the_gradient(oracle, dt):
    # the reference dequantises to T and multiplies that tensor: pinned against
    # numpy in float64 on the oracle's T-rounded dequantised weight (itself
    # bit-exact against the reference's formula elsewhere)
    M, K, N, bits, g = 4, 192, 80, 8, 64
    wb = H.make_weight(K, N, dt, seed=5)
    oc, osc = oracle.weight_quantize(wb, dt, bits, g)
    _, wT = oracle.dequantize(oc, osc, dt, bits, g)
    gb = H.make_act(M, N, dt, seed=6)
    want = H.bits_to_f32(gb, dt).astype(np.float64) @ H.bits_to_f32(wT, dt).astype(np.float64).T
    o64, _ = oracle.linear_grad_rounded_weight(gb, oc, osc, dt, bits, g, acc64=True)
    assert np.array_equal(o64, want.astype(np.float32))
    # it differs from the fp32-weight contract by one rounding of every weight to T
    exact, _ = oracle.linear_grad(gb, oc, osc, dt, bits, g, acc64=True)
    d = H.rel_l2(o64, exact)
    assert (5e-4 < d < 4e-3) if dt == H.BF16 else (5e-5 < d < 5e-4), d


def test_oracle_linear_grad_is_the_adjoint_of_linear(oracle):
    # <linear(x), g> == <x, linear_grad(g)> for any x and g: fixes the pairing of
    # the two functions' index conventions independently of the dequantiser
    dt, bits, g = H.F16, 8, 64
    M, K, N = 3, 128, 32
    wb = H.make_weight(K, N, dt, seed=8)
    oc, osc = oracle.weight_quantize(wb, dt, bits, g)
    xb = H.make_act(M, K, dt, seed=9)
    gb = H.make_act(M, N, dt, seed=10)
    y32, _ = oracle.linear(xb, oc, osc, None, dt, bits, g, acc64=True)
    gx32, _ = oracle.linear_grad(gb, oc, osc, dt, bits, g, acc64=True)
    lhs = np.sum(y32.astype(np.float64) * H.bits_to_f32(gb, dt).astype(np.float64))
    rhs = np.sum(H.bits_to_f32(xb, dt).astype(np.float64) * gx32.astype(np.float64))
    assert abs(lhs - rhs) <= 1e-5 * max(abs(lhs), abs(rhs))


# ---- the kernel ---------------------------------------------------------------
def _grad(g_bits, packed, scale_bits, dt, K, bits, group, f32=False):
    import torch
    from paddle_amd import _lib

    dev = "cuda:0"
    go = H.bits_to_torch(g_bits, dt, dev)
    M, N = go.shape
    c = torch.from_numpy(np.ascontiguousarray(packed)).to(dev)
    s = H.bits_to_torch(scale_bits, dt, dev)
    out = torch.full((M, K), float("nan"), dtype=torch.float32 if f32 else go.dtype, device=dev)
    wsb = _lib.lib.wol_linear_grad_workspace(M, K, N, bits, group)
    assert wsb > 0
    ws = torch.full((wsb,), 0x5A, dtype=torch.uint8, device=dev)
    fn = _lib.lib.wol_linear_grad_f32 if f32 else _lib.lib.wol_linear_grad
    _lib.check(fn(go.data_ptr(), c.data_ptr(), s.data_ptr(), dt, M, K, N, bits, group, out.data_ptr(),
                  ws.data_ptr(), wsb, None))
    torch.cuda.synchronize()
    return out.cpu().numpy() if f32 else H.torch_to_bits(out)


def _case(oracle, dt, bits, g, M, K, N, seed=0, gstd=1.0):
    """Returns (rel-L2 of the fp32 sums against the oracle's fp32 result,
    rel-L2 of the T output against the oracle's T output)."""
    wb = H.make_weight(K, N, dt, seed=K + N + seed)
    oc, osc = oracle.weight_quantize(wb, dt, bits, g)
    packed = H.gfx950_from_q(H.q_from_canonical(oc, bits), bits)
    gb = H.make_act(M, N, dt, seed=M + seed)
    if gstd != 1.0:
        gb = H.f32_to_bits(H.bits_to_f32(gb, dt) * np.float32(gstd), dt)
    want32, wantT = oracle.linear_grad(gb, oc, osc, dt, bits, g)
    got32 = _grad(gb, packed, osc, dt, K, bits, g, f32=True)
    got = _grad(gb, packed, osc, dt, K, bits, g)
    assert np.isfinite(got32).all()
    # the T output is the round-to-nearest-even cast of the fp32 sums
    assert np.array_equal(got, H.f32_to_bits(got32, dt))
    return H.rel_l2(got32, want32), H.rel_l2(H.bits_to_f32(got, dt), H.bits_to_f32(wantT, dt))


# every tile shape of the kernel (by the number of output tiles), N that is and
# is not a multiple of the 64-column chunk, M off the tile height, K off the
# tile width and, for int4, a K that ends in a half tile; the last two have few
# tiles and a long N, which the kernel cuts into four and two runs
SHAPES = [(24, 512, 256), (1, 64, 16), (130, 192, 48), (300, 1088, 144), (1000, 2048, 512), (2100, 4096, 320),
          (100, 256, 2048), (500, 512, 1040)]


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("g", [-1, 64, 128])
def test_linear_grad_against_oracle(device, oracle, dt, bits, g):
    for M, K, N in SHAPES:
        if bits == 4 and N % 32:
            N += 16
        print("case", dt, bits, g, M, K, N, flush=True)
        err32, errT = _case(oracle, dt, bits, g, M, K, N)
        # The fp32 sums carry the one rounding of code * scale to 11 bits
        # (about 1.5e-4) and are held to 3e-4; _case has already checked that
        # the T output is exactly their round-to-nearest-even cast.  Together
        # that is the whole statement about the T output.  Comparing it with
        # the oracle's T output on top is only meaningful where the output is
        # large enough for the rel-L2 of two bfloat16 roundings of nearby sums
        # (neighbouring values now and then, 2^-8 apart) to average out.
        assert err32 <= 3e-4, (err32, dt, bits, g, M, K, N)
        if dt == H.F16 or M * K >= 4096:
            assert errT <= TOL, (errT, dt, bits, g, M, K, N)


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("bits", [8, 4])
def test_linear_grad_distance_to_the_reference_composition(device, oracle, dt, bits):
    # The reference rounds code * scale to T before its GEMM; this kernel rounds
    # it to 11 bits (fp16 operands for both dtypes).  Its fp32 sums are therefore
    # not the reference's bits: recorded here is how far they are from the
    # reference's composition (one T rounding of the weights: about 2e-3 for
    # bfloat16, 2e-4 for float16) and that they are nearer to the exact product
    # than that composition is for bfloat16.
    M, K, N, g = 96, 512, 384, -1
    wb = H.make_weight(K, N, dt, seed=21)
    oc, osc = oracle.weight_quantize(wb, dt, bits, g)
    packed = H.gfx950_from_q(H.q_from_canonical(oc, bits), bits)
    gb = H.make_act(M, N, dt, seed=22)
    exact, _ = oracle.linear_grad(gb, oc, osc, dt, bits, g)
    ref, _ = oracle.linear_grad_rounded_weight(gb, oc, osc, dt, bits, g)
    got32 = _grad(gb, packed, osc, dt, K, bits, g, f32=True)
    to_ref, to_exact, ref_to_exact = H.rel_l2(got32, ref), H.rel_l2(got32, exact), H.rel_l2(ref, exact)
    print("distance to the reference composition %.2e, to the exact product %.2e (the composition's own %.2e)"
          % (to_ref, to_exact, ref_to_exact))
    assert to_ref <= (4e-3 if dt == H.BF16 else 6e-4), to_ref
    assert to_exact <= 3e-4
    if dt == H.BF16:
        assert to_exact < ref_to_exact


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [H.F16, H.BF16])
def test_linear_grad_keeps_its_accuracy_at_any_magnitude(device, oracle, dt):
    # out_grad as small as a loss-scaled gradient gets, and large: the powers of
    # two taken out per row and per column keep the fp16 operands in range
    for gstd in (1e-6, 3e-3, 200.0):
        err32, errT = _case(oracle, dt, 4, 128, 64, 512, 256, seed=5, gstd=gstd)
        assert err32 <= 3e-4, (err32, gstd)
        # float16 results of the smallest case are subnormal (about 3e-7): the
        # output grid itself is then coarser than the bar
        if not (dt == H.F16 and gstd < 1e-4):
            assert errT <= TOL, (errT, gstd)


@pytest.mark.gpu
def test_linear_grad_zero_rows_and_linearity(device, oracle):
    # a zero row of out_grad gives a zero row of x_grad (its normaliser must not
    # divide by zero), and the map is linear in out_grad: grad(2 g) = 2 grad(g) bit for bit
    dt, bits, g = H.BF16, 8, -1
    M, K, N = 70, 256, 128
    wb = H.make_weight(K, N, dt, seed=2)
    oc, osc = oracle.weight_quantize(wb, dt, bits, g)
    packed = H.gfx950_from_q(H.q_from_canonical(oc, bits), bits)
    g32 = H.bits_to_f32(H.make_act(M, N, dt, seed=6), dt)
    g32[3, :] = 0.0
    g32[69, :] = 0.0
    gb = H.f32_to_bits(g32, dt)
    got = H.bits_to_f32(_grad(gb, packed, osc, dt, K, bits, g), dt)
    assert np.all(got[3] == 0.0) and np.all(got[69] == 0.0)
    twice = H.bits_to_f32(_grad(H.f32_to_bits(g32 * 2, dt), packed, osc, dt, K, bits, g), dt)
    assert np.array_equal(twice, got * 2)


@pytest.mark.gpu
@pytest.mark.parametrize("dt,bits,g", [(H.F16, 8, -1), (H.BF16, 4, 128), (H.F16, 4, 64), (H.BF16, 8, 64)])
def test_x_grad_through_autograd(device, oracle, dt, bits, g):
    # the Python mirror's backward reaches wol_linear_grad; x_grad only
    # (backward.yaml:3651-3661)
    import torch
    from paddle_amd.nn import quant as Q

    M, K, N = 24, 512, 256
    wb = H.make_weight(K, N, dt, seed=11)
    oc, osc = oracle.weight_quantize(wb, dt, bits, g)
    tdt = H.torch_dtype(dt)
    codes, scale = Q.weight_quantize(H.bits_to_torch(wb, dt, device),
                                     algo="weight_only_int8" if bits == 8 else "weight_only_int4", group_size=g)
    xb = H.make_act(M, K, dt, seed=12)
    gob = H.make_act(M, N, dt, seed=13)
    x = H.bits_to_torch(xb, dt, device).reshape(2, 12, K).requires_grad_(True)
    go = H.bits_to_torch(gob, dt, device).reshape(2, 12, N)
    out = Q.weight_only_linear(x, codes, None, scale, "int8" if bits == 8 else "int4", None, g)
    out.backward(go)
    assert x.grad is not None and x.grad.shape == x.shape and x.grad.dtype == tdt
    _, wantT = oracle.linear_grad(gob, oc, osc, dt, bits, g)
    err = H.rel_l2(x.grad.float().cpu().numpy().reshape(M, K), H.bits_to_f32(wantT, dt))
    assert err <= TOL, err
    with torch.no_grad():
        out2 = Q.weight_only_linear(x, codes, None, scale, "int8" if bits == 8 else "int4", None, g)
    assert torch.equal(out.detach(), out2)


def test_linear_grad_argument_checks():
    # no GPU needed: the checks come before any device call
    from paddle_amd import _lib

    L = _lib.lib
    assert L.wol_linear_grad_workspace(0, 64, 16, 8, -1) == 0
    assert L.wol_linear_grad_workspace(4, 64, 16, 8, 32) == 0  # group size
    assert L.wol_linear_grad_workspace(4, 64, 16, 8, -1) > 0
    assert L.wol_linear_grad(None, None, None, 0, 4, 64, 16, 3, -1, None, None, 0, None) == 3
    assert L.wol_linear_grad(None, None, None, 0, 4, 65, 16, 8, -1, None, None, 0, None) == 5
    assert L.wol_linear_grad(None, None, None, 0, 0, 64, 16, 8, -1, None, None, 0, None) == 0  # nothing to do
    assert L.wol_linear_grad(None, None, None, 0, 4, 64, 16, 8, -1, None, None, 0, None) == 1


@pytest.mark.gpu
@pytest.mark.parametrize("case", [(2048, 4096, 4096, 8, -1, H.BF16), (8192, 4096, 4096, 4, 64, H.BF16),
                                  (512, 8192, 8192, 4, 128, H.F16), (1000, 11008, 4096, 8, 64, H.F16)])
def test_linear_grad_full_size_is_the_adjoint_of_the_linear(device, case):
    # at the benchmark's sizes, where the oracle would take minutes: for any x and
    # g, <linear(x), g> = <x, linear_grad(g)> (both sides through the fp32
    # outputs of the two kernels, summed in float64).  A wrong tile, a dropped
    # chunk of N or a mis-indexed scale group breaks the identity; the fp16
    # rounding of code * scale in the grad kernel leaves about 1e-4.
    import torch
    from paddle_amd import _lib
    from paddle_amd.nn import quant as Q

    M, K, N, bits, g, dt = case
    tdt = H.torch_dtype(dt)
    gen = torch.Generator(device="cuda").manual_seed(M + K)
    w = (torch.randn(K, N, device="cuda", generator=gen) * 0.02).to(tdt)
    codes, scale = Q.weight_quantize(w, algo="weight_only_int8" if bits == 8 else "weight_only_int4", group_size=g)
    del w
    x = torch.randn(M, K, device="cuda", generator=gen).to(tdt)
    go = torch.randn(M, N, device="cuda", generator=gen).to(tdt)
    L = _lib.lib
    y32 = torch.empty(M, N, device="cuda", dtype=torch.float32)
    wsb = L.wol_linear_workspace(M, K, N, bits, g)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda")
    _lib.check(L.wol_linear_f32(x.data_ptr(), codes.data_ptr(), None, scale.data_ptr(), dt, M, K, N, bits, g,
                                y32.data_ptr(), ws.data_ptr() if wsb else None, wsb, None))
    gx32 = torch.empty(M, K, device="cuda", dtype=torch.float32)
    gsb = L.wol_linear_grad_workspace(M, K, N, bits, g)
    gws = torch.empty(gsb, dtype=torch.uint8, device="cuda")
    _lib.check(L.wol_linear_grad_f32(go.data_ptr(), codes.data_ptr(), scale.data_ptr(), dt, M, K, N, bits, g,
                                     gx32.data_ptr(), gws.data_ptr(), gsb, None))
    torch.cuda.synchronize()
    # row by row (every row of the batch has its own normaliser in the grad
    # kernel), measured against the size of the terms: the inner products
    # themselves are sums of random signs and may come out near zero
    lhs = (y32.double() * go.double()).sum(dim=1)
    rhs = (x.double() * gx32.double()).sum(dim=1)
    size = y32.double().norm(dim=1) * go.double().norm(dim=1)
    rel = ((lhs - rhs).abs() / size).max().item()
    print("adjoint mismatch", case, rel, flush=True)
    # the grad kernel's 1.7e-4 per element averages down by sqrt(N) in the inner
    # product (measured 3e-6 .. 1e-5); one missing chunk of 64 columns would read 2e-3
    assert rel <= 1e-4, rel
    # and the T output is the cast of the fp32 one
    gxT = torch.empty(M, K, device="cuda", dtype=tdt)
    _lib.check(L.wol_linear_grad(go.data_ptr(), codes.data_ptr(), scale.data_ptr(), dt, M, K, N, bits, g,
                                 gxT.data_ptr(), gws.data_ptr(), gsb, None))
    torch.cuda.synchronize()
    assert torch.equal(gxT, gx32.to(tdt))
