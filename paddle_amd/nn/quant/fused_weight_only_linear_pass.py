"""Graph-level caller of the weight-only path: rewrites `matmul(x, w) [+ bias]`
with a persistable 2-D half-precision `w` into `weight_quantize` (once, at
rewrite time, on the device) + `weight_only_linear`.

This is the host-side counterpart of the reference's
`fused_weight_only_linear_pass`
(paddle/fluid/pir/transforms/gpu/fused_weight_only_linear_pass.cc:39-323) for
graphs held as `torch.fx.GraphModule`: the same three patterns (bias on either
side of the add with benefit 2, no bias with benefit 1), the same constraints
(:79-106, :213-236) and the same `weight_only_algo` option and error (:294-303).
Differences, all deliberate:
  * it always applies on gfx950 (the reference gates on CUTLASS and SM 80/86/89/90,
    :30-37, :312-318);
  * int4 is quantised on the device like int8 (the reference copies the weight
    to the host, quantises there and copies back, :111-136);
  * `group_size` may be 64 or 128 as well as -1 (the reference hard-codes -1).
"""
import operator

import torch
import torch.fx

from . import quantized_linear as _ql

_MATMULS = (torch.matmul, operator.matmul)
_ADDS = (torch.add, operator.add)


def _attr(gm, target):
    obj = gm
    for part in target.split("."):
        obj = getattr(obj, part)
    return obj


def _persistable(gm, node):
    """A get_attr node that names a parameter or buffer of the module
    (pir::ValueIsPersistable in the reference, :72-74)."""
    if not isinstance(node, torch.fx.Node) or node.op != "get_attr":
        return None
    try:
        t = _attr(gm, node.target)
    except AttributeError:
        return None
    return t if isinstance(t, torch.Tensor) else None


def _is_matmul(node):
    if node.op == "call_function" and node.target in _MATMULS:
        return len(node.args) == 2 and not node.kwargs
    if node.op == "call_method" and node.target == "matmul":
        return len(node.args) == 2 and not node.kwargs
    return False


def _is_add(node):
    if node.op == "call_function" and node.target in _ADDS:
        return len(node.args) == 2 and not node.kwargs  # torch.add(..., alpha=) is another op
    if node.op == "call_method" and node.target == "add":
        return len(node.args) == 2 and not node.kwargs
    return False


def _shape_of(node):
    meta = node.meta.get("tensor_meta") if isinstance(node, torch.fx.Node) else None
    return tuple(meta.shape) if meta is not None else None


def _weight_ok(w):
    """The constraints of both patterns on w (:84-104, :222-232)."""
    if w.dim() != 2 or w.dtype not in (torch.float16, torch.bfloat16):
        return False
    return w.shape[0] % 64 == 0 and w.shape[1] % 16 == 0


def _x_ok(x_node, w):
    """x has rank >= 2 and its last dimension is w's first (:91-102); checked
    when the graph carries shapes (torch.fx.passes.shape_prop), otherwise left
    to weight_only_linear's own check at run time."""
    shape = _shape_of(x_node)
    if shape is None:
        return True
    return len(shape) >= 2 and shape[-1] == w.shape[0]


def fused_weight_only_linear_pass(gm, weight_only_algo="weight_only_int8", group_size=-1,
                                  quantize=None):
    """Rewrites `gm` in place and returns the number of matmuls replaced.

    weight_only_algo: "weight_only_int8" or "weight_only_int4" (the pass option
    of the same name).  quantize: the weight_quantize to call, for callers that
    bring their own (defaults to this package's, which needs the weights on the
    GPU)."""
    if weight_only_algo not in ("weight_only_int8", "weight_only_int4"):
        raise ValueError(
            "(InvalidArgument) fused_weight_only_linear_pass only support weight_only_int8 or "
            "weight_only_int4, but get %s." % weight_only_algo
        )
    _ql._check_group_size(group_size, "fused_weight_only_linear_pass")
    quantize = quantize or _ql.weight_quantize
    weight_dtype = "int8" if weight_only_algo == "weight_only_int8" else "int4"
    graph = gm.graph
    quantized = {}  # weight attribute -> (codes node target, scale node target)
    replaced = 0

    def quantized_attrs(w_node, w):
        if w_node.target not in quantized:
            codes, scale = quantize(w.detach(), algo=weight_only_algo, group_size=group_size)
            base = w_node.target.replace(".", "_")
            names = (base + "_quanted_weight", base + "_weight_scale")
            gm.register_buffer(names[0], codes)
            gm.register_buffer(names[1], scale)
            quantized[w_node.target] = names
        return quantized[w_node.target]

    for mm in list(graph.nodes):
        if not _is_matmul(mm):
            continue
        x_node, w_node = mm.args
        w = _persistable(gm, w_node)
        if w is None or not _weight_ok(w) or not _x_ok(x_node, w):
            continue
        # with-bias patterns first (benefit 2): the matmul's only user is an add
        # whose other operand is a 1-D tensor (a parameter, or known from the
        # graph's shape metadata)
        target, bias_node = mm, None
        users = list(mm.users)
        if len(users) == 1 and _is_add(users[0]):
            add = users[0]
            other = add.args[1] if add.args[0] is mm else add.args[0]
            b = _persistable(gm, other)
            rank = b.dim() if b is not None else (len(_shape_of(other)) if _shape_of(other) is not None else None)
            if isinstance(other, torch.fx.Node) and other is not mm and rank == 1:
                target, bias_node = add, other
        with graph.inserting_before(target):
            names = quantized_attrs(w_node, w)
            codes_node = graph.get_attr(names[0])
            scale_node = graph.get_attr(names[1])
            new = graph.call_function(
                _ql.weight_only_linear,
                (x_node, codes_node, bias_node, scale_node, weight_dtype, None, group_size),
            )
        target.replace_all_uses_with(new)
        if target is not mm:
            graph.erase_node(target)
        graph.erase_node(mm)
        replaced += 1

    if replaced:
        graph.eliminate_dead_code()  # the get_attr nodes of weights that are no longer read
        live = {n.target for n in graph.nodes if n.op == "get_attr"}
        for name in quantized:
            if name in live:
                continue
            owner_path, _, leaf = name.rpartition(".")
            owner = _attr(gm, owner_path) if owner_path else gm
            for table in (owner._parameters, owner._buffers):
                table.pop(leaf, None)  # the fp16/bf16 copy is what the pass exists to drop
        graph.lint()
        gm.recompile()
    return replaced
