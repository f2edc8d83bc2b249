"""fused_weight_only_linear_pass on torch.fx graphs: which matmuls it rewrites
(the constraints of the reference's patterns,
paddle/fluid/pir/transforms/gpu/fused_weight_only_linear_pass.cc:69-106,
:213-236), what it puts in their place, and -- on the GPU -- that the rewritten
graph computes what weight_quantize + weight_only_linear compute.  The
reference's own test (test/ir/pir/fused_pass/test_fused_weight_only_linear_pass.py)
counts the ops after the pass and compares outputs with the unfused program at
1e-2 / 1e-3; the structure checks below are the op counts."""
import numpy as np
import pytest
import torch
import torch.fx

import helpers as H
from paddle_amd.nn.quant import quantized_linear as QL
from paddle_amd.nn.quant.fused_weight_only_linear_pass import fused_weight_only_linear_pass


def _fake_quantize(w, algo="weight_only_int8", arch=None, group_size=-1):
    K, N = w.shape
    rows = N if algo == "weight_only_int8" else N // 2
    sshape = (N,) if group_size == -1 else (K // group_size, N)
    return torch.zeros(rows, K, dtype=torch.int8), torch.ones(sshape, dtype=w.dtype)


class Net(torch.nn.Module):
    """Two projections the pass takes (bias on either side), one without bias,
    and matmuls it must leave alone."""

    def __init__(self, dtype=torch.float16, K=128, N=64):
        super().__init__()
        g = torch.Generator().manual_seed(3)
        mk = lambda *s: torch.nn.Parameter((torch.randn(*s, generator=g) * 0.05).to(dtype), requires_grad=False)
        self.w1, self.b1 = mk(K, N), mk(N)
        self.w2, self.b2 = mk(N, K), mk(K)
        self.w3 = mk(K, 32)
        self.w_odd = mk(K, 24)  # 24 % 16 != 0
        self.w_k = mk(96, 16)  # 96 % 64 != 0
        self.w_f32 = torch.nn.Parameter(torch.randn(K, 16, generator=g), requires_grad=False)

    def forward(self, x):
        h = torch.matmul(x, self.w1) + self.b1  # matmul, then bias
        h = self.b2 + (h @ self.w2)  # bias, then matmul
        a = torch.matmul(h, self.w3)  # no bias
        b = torch.matmul(h, self.w_odd)  # N not a multiple of 16
        c = torch.matmul(h[..., :96], self.w_k)  # K not a multiple of 64
        d = torch.matmul(h.float(), self.w_f32)  # float32 weight
        e = torch.matmul(h, h.transpose(-1, -2))  # second operand is not persistable
        return a, b, c, d, e


def _targets(gm):
    return [n.target for n in gm.graph.nodes if n.op == "call_function"]


def test_rewrites_the_three_patterns_and_nothing_else():
    gm = torch.fx.symbolic_trace(Net())
    n = fused_weight_only_linear_pass(gm, "weight_only_int8", quantize=_fake_quantize)
    assert n == 3
    calls = [nd for nd in gm.graph.nodes if nd.op == "call_function" and nd.target is QL.weight_only_linear]
    assert len(calls) == 3
    by_weight = {c.args[1].target: c for c in calls}
    assert set(by_weight) == {"w1_quanted_weight", "w2_quanted_weight", "w3_quanted_weight"}
    c1, c2, c3 = by_weight["w1_quanted_weight"], by_weight["w2_quanted_weight"], by_weight["w3_quanted_weight"]
    assert c1.args[2].target == "b1" and c2.args[2].target == "b2" and c3.args[2] is None
    assert c1.args[3].target == "w1_weight_scale"
    assert c1.args[4:] == ("int8", None, -1)
    # both adds are gone, the four other matmuls stay
    t = _targets(gm)
    assert t.count(torch.matmul) == 4 and not any(x in t for x in (torch.add,))
    import operator
    assert operator.add not in t and operator.matmul not in t
    # the half-precision copies of the rewritten weights are dropped, the others kept
    names = dict(gm.named_parameters())
    assert "w1" not in names and "w2" not in names and "w3" not in names
    assert {"w_odd", "w_k", "w_f32", "b1", "b2"} <= set(names)
    assert gm.w1_quanted_weight.dtype == torch.int8 and tuple(gm.w1_quanted_weight.shape) == (64, 128)


def test_int4_and_group_size_options_reach_the_calls():
    gm = torch.fx.symbolic_trace(Net(torch.bfloat16))
    seen = []

    def q(w, algo="weight_only_int8", arch=None, group_size=-1):
        seen.append((tuple(w.shape), algo, group_size))
        return _fake_quantize(w, algo, arch, group_size)

    assert fused_weight_only_linear_pass(gm, "weight_only_int4", group_size=64, quantize=q) == 3
    assert sorted(seen) == [((64, 128), "weight_only_int4", 64), ((128, 32), "weight_only_int4", 64),
                            ((128, 64), "weight_only_int4", 64)]
    for nd in gm.graph.nodes:
        if nd.op == "call_function" and nd.target is QL.weight_only_linear:
            assert nd.args[4:] == ("int4", None, 64)
    assert tuple(gm.w1_quanted_weight.shape) == (32, 128) and tuple(gm.w1_weight_scale.shape) == (2, 64)


def test_option_errors():
    gm = torch.fx.symbolic_trace(Net())
    with pytest.raises(ValueError, match="only support weight_only_int8 or weight_only_int4, but get llm.int8"):
        fused_weight_only_linear_pass(gm, "llm.int8", quantize=_fake_quantize)
    with pytest.raises(AssertionError, match="group size"):
        fused_weight_only_linear_pass(gm, "weight_only_int8", group_size=32, quantize=_fake_quantize)


def test_shared_weight_is_quantised_once_and_multi_use_matmul_keeps_its_add():
    class Shared(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.w = torch.nn.Parameter(torch.zeros(64, 16, dtype=torch.float16), requires_grad=False)
            self.b = torch.nn.Parameter(torch.zeros(16, dtype=torch.float16), requires_grad=False)

        def forward(self, x, y):
            m = torch.matmul(x, self.w)
            return m + self.b, m * 2, torch.matmul(y, self.w)

    calls = []

    def q(w, algo="weight_only_int8", arch=None, group_size=-1):
        calls.append(1)
        return _fake_quantize(w, algo, arch, group_size)

    gm = torch.fx.symbolic_trace(Shared())
    assert fused_weight_only_linear_pass(gm, quantize=q) == 2
    assert len(calls) == 1
    import operator
    t = _targets(gm)
    assert operator.add in t  # the matmul has a second user: only the matmul is replaced
    for nd in gm.graph.nodes:
        if nd.op == "call_function" and nd.target is QL.weight_only_linear:
            assert nd.args[2] is None


def test_shape_metadata_vetoes_a_mismatched_activation():
    from torch.fx.passes.shape_prop import ShapeProp

    class One(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.w = torch.nn.Parameter(torch.zeros(64, 16, dtype=torch.float16), requires_grad=False)

        def forward(self, x):
            return torch.matmul(x, self.w)

    gm = torch.fx.symbolic_trace(One())
    ShapeProp(gm).propagate(torch.zeros(64, dtype=torch.float16))  # rank-1 activation
    assert fused_weight_only_linear_pass(gm, quantize=_fake_quantize) == 0
    gm = torch.fx.symbolic_trace(One())
    ShapeProp(gm).propagate(torch.zeros(2, 3, 64, dtype=torch.float16))
    assert fused_weight_only_linear_pass(gm, quantize=_fake_quantize) == 1


@pytest.mark.gpu
@pytest.mark.parametrize("algo,group_size", [("weight_only_int8", -1), ("weight_only_int4", -1),
                                             ("weight_only_int4", 64), ("weight_only_int8", 128)])
def test_rewritten_graph_matches_quantize_plus_linear(device, oracle, algo, group_size):
    dt = H.BF16
    net = Net(torch.bfloat16, K=256, N=128).to(device)
    x = H.bits_to_torch(H.make_act(2 * 5, 256, dt, seed=12), dt, device).reshape(2, 5, 256)
    want = net(x)
    gm = torch.fx.symbolic_trace(net)
    w1b, w2b, w3b = (H.torch_to_bits(p) for p in (net.w1, net.w2, net.w3))
    assert fused_weight_only_linear_pass(gm, algo, group_size=group_size) == 3
    got = gm(x)
    bits = 8 if algo == "weight_only_int8" else 4
    # the weights the graph now holds are weight_quantize's, bit for bit
    from paddle_amd.nn import quant as Q
    for name, wb in (("w1", w1b), ("w2", w2b), ("w3", w3b)):
        qw, qs = Q.weight_quantize(H.bits_to_torch(wb, dt, device), algo=algo, group_size=group_size)
        assert torch.equal(getattr(gm, name + "_quanted_weight"), qw)
        assert torch.equal(getattr(gm, name + "_weight_scale"), qs)
        _, oscale = oracle.weight_quantize(wb, dt, bits, group_size)
        assert np.array_equal(H.torch_to_bits(qs), oscale)
    # and the outputs follow the unfused graph to quantisation accuracy (the
    # reference's test uses 1e-2 / 1e-3 on its own data)
    tol = 0.03 if bits == 8 else 0.25
    a_got, a_want = got[0].float(), want[0].float()
    assert a_got.shape == a_want.shape == (2, 5, 32)
    assert (a_got - a_want).norm() / a_want.norm() < tol
    # untouched branches are bit-identical given identical inputs only; they read h, which
    # changed, so compare loosely
    assert (got[3] - want[3]).norm() / want[3].norm() < tol
