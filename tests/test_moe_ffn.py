"""moe_ffn on weight-only quantised experts (wol_moe_ffn: two grouped GEMM
launches over a device-side row-tile table, swiglu between) against the oracle:
per expert, the oracle's linear (rounded to T, as the reference's fc1 output
is), swiglu in float on those T values, the oracle's linear again
(paddle/phi/kernels/fusion/cutlass/moe_ffn.cu:74-183)."""
import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu


def _oracle_moe(oracle, xb, cum, w1b, b1b, w2b, dt, bits):
    rows, hidden = xb.shape
    out = np.zeros((rows, hidden), np.uint16)
    prev = 0
    for e, end in enumerate(cum):
        end = int(end)
        if end > prev:
            c1, s1 = oracle.weight_quantize(w1b[e], dt, bits, -1)
            c2, s2 = oracle.weight_quantize(w2b[e], dt, bits, -1)
            _, fc1 = oracle.linear(xb[prev:end], c1, s1, None if b1b is None else b1b[e], dt, bits, -1)
            _, act = oracle.activation(H.bits_to_f32(fc1, dt), oracle.ACT_SWIGLU, dt)
            _, o = oracle.linear(act, c2, s2, None, dt, bits, -1)
            out[prev:end] = o
        prev = end
    return out


# rows per expert: none, a few, exactly one tile, a tile and a bit, many, none at
# the end (128-row tiles); few rows per expert, with whole and partial tiles
# and one expert far above the average (64-row tiles; 32-row tiles for int4);
# an average of 38 rows (64-row tiles for both bit widths); many rows
ROWS_PER_EXPERT = [[0, 5, 128, 131, 300, 0], [0, 5, 33, 64, 1, 17], [40, 64, 0, 70, 3, 50], [2, 1, 150, 0, 3, 4],
                   [600, 256, 0, 1000, 700, 520]]  # 512 and more on average: 256-row tiles for int8


@pytest.mark.parametrize("dt", [H.F16, H.BF16])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("per,inter", [(p, 512) for p in ROWS_PER_EXPERT] + [(p, 4096) for p in ROWS_PER_EXPERT[1:4]])
def test_moe_ffn_against_oracle(device, oracle, dt, bits, per, inter):
    # inter = 4096 with few rows per expert: the second GEMM (K = 2048) runs with
    # its K cut into runs across workgroups and the kernel that adds them
    import torch
    from paddle_amd.nn import quant as Q

    hidden, E = 256, 6
    cum = np.cumsum(per).astype(np.int64)
    rows = int(cum[-1]) + 3  # three rows that belong to no expert
    rng = np.random.default_rng(5)
    xb = H.make_act(rows, hidden, dt, seed=1)
    w1b = np.stack([H.make_weight(hidden, inter, dt, seed=10 + e) for e in range(E)])
    w2b = np.stack([H.make_weight(inter // 2, hidden, dt, seed=20 + e, std=0.05) for e in range(E)])
    b1b = np.stack([H.make_bias(inter, dt, seed=30 + e) for e in range(E)])
    algo = "weight_only_int8" if bits == 8 else "weight_only_int4"
    w1, s1 = Q.moe_quantize_experts(H.bits_to_torch(w1b, dt, device), algo)
    w2, s2 = Q.moe_quantize_experts(H.bits_to_torch(w2b, dt, device), algo)
    x = H.bits_to_torch(xb, dt, device)
    cnt = torch.from_numpy(cum).to(device)
    for bias in (None, b1b):
        b1 = None if bias is None else H.bits_to_torch(bias, dt, device).reshape(E, 1, inter)
        out = Q.moe_ffn(x, cnt, w1, w2, b1, s1, s2, algo)
        torch.cuda.synchronize()
        got = H.torch_to_bits(out)[: int(cum[-1])]
        want = _oracle_moe(oracle, xb, cum, w1b, bias, w2b, dt, bits)[: int(cum[-1])]
        err = H.rel_l2(H.bits_to_f32(got, dt), H.bits_to_f32(want, dt))
        assert err <= 1e-3, (err, dt, bits, bias is not None)
        # every expert on its own, so that a small expert cannot hide behind a large one
        prev = 0
        for e, end in enumerate(cum):
            if end > prev:
                ee = H.rel_l2(H.bits_to_f32(got[prev:end], dt), H.bits_to_f32(want[prev:end], dt))
                assert ee <= 2e-3, (e, ee)
            prev = int(end)


def test_moe_ffn_clamps_running_totals_it_cannot_trust(device):
    # token_nums_per_expert comes from the device and is read there only.  Totals
    # that run backwards or past the input's rows are clamped by the table
    # builder to [previous total, rows]: the call computes what it would with
    # the clamped totals and touches no row outside the input.
    import torch
    from paddle_amd.nn import quant as Q

    hidden, inter, E = 256, 512, 5
    gen = torch.Generator(device="cuda").manual_seed(3)
    w1 = (torch.randn(E, hidden, inter, device="cuda", generator=gen) * 0.02).to(torch.bfloat16)
    w2 = (torch.randn(E, inter // 2, hidden, device="cuda", generator=gen) * 0.02).to(torch.bfloat16)
    q1, s1 = Q.moe_quantize_experts(w1)
    q2, s2 = Q.moe_quantize_experts(w2)
    rows = 200
    x = torch.randn(rows, hidden, device="cuda", generator=gen).to(torch.bfloat16)
    bad = torch.tensor([70, 30, 150, 10 ** 9, -5], dtype=torch.int64, device="cuda")   # backwards, huge, negative
    good = torch.tensor([70, 70, 150, 200, 200], dtype=torch.int64, device="cuda")     # what the clamp makes of it
    want = Q.moe_ffn(x, good, q1, q2, None, s1, s2, "weight_only_int8")
    got = Q.moe_ffn(x, bad, q1, q2, None, s1, s2, "weight_only_int8")
    torch.cuda.synchronize()
    assert torch.equal(got, want)


def test_moe_ffn_equals_per_expert_calls(device):
    # the grouped launches against a loop of ordinary calls on each expert's rows
    import torch
    from paddle_amd.nn import quant as Q

    hidden, inter, E = 512, 1024, 4
    gen = torch.Generator(device="cuda").manual_seed(9)
    w1 = (torch.randn(E, hidden, inter, device="cuda", generator=gen) * 0.02).to(torch.bfloat16)
    w2 = (torch.randn(E, inter // 2, hidden, device="cuda", generator=gen) * 0.02).to(torch.bfloat16)
    q1, s1 = Q.moe_quantize_experts(w1)
    q2, s2 = Q.moe_quantize_experts(w2)
    per = [40, 0, 260, 17]
    cum = torch.tensor(np.cumsum(per), dtype=torch.int64, device="cuda")
    x = torch.randn(sum(per), hidden, device="cuda", generator=gen).to(torch.bfloat16)
    out = Q.moe_ffn(x, cum, q1, q2, None, s1, s2, "weight_only_int8")
    prev = 0
    for e, n in enumerate(per):
        if n:
            fc1 = Q.weight_only_linear(x[prev:prev + n], q1[e], None, s1[e], "int8")
            act = (torch.nn.functional.silu(fc1[:, : inter // 2].float()) * fc1[:, inter // 2:].float()).to(torch.bfloat16)
            ref = Q.weight_only_linear(act, q2[e], None, s2[e], "int8")
            err = float((out[prev:prev + n].float() - ref.float()).norm() / ref.float().norm())
            assert err <= 2e-3, (e, err)
        prev += n
    with pytest.raises(ValueError):
        Q.moe_ffn(x, cum, q1, q2, None, s1, s2, "None")
    with pytest.raises(ValueError):
        Q.moe_ffn(x, cum.int(), q1, q2, None, s1, s2, "weight_only_int8")
