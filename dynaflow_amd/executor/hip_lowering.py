"""Rewrite a traced sub-graph onto the hand-written HIP operators.

This pass takes the slot that TorchInductor has in the reference
(dynaflow/executor/inductor.py:111-141 compiles a deep copy of the sub-graph):
it deep-copies the sub-``GraphModule`` and replaces

* ``linear(x, w)`` (no bias, bf16 or fp32)            -> ``dynaflow_hip.linear``
* ``mul(silu(g), u)`` / ``mul(u, silu(g))``           -> ``dynaflow_hip.silu_mul``
* ``rms_norm(x, (H,), w, eps)`` (bf16, last dim)      -> ``dynaflow_hip.rms_norm``
* ``apply_rope(t, cos, sin)`` (bf16, one graph node)  -> ``dynaflow_hip.rope``
* ``attend_and_append(qkv, k_cache, v_cache, ...)``   -> ``dynaflow_hip.decode_attention``
* ``causal_gqa_attention(q, k, v)`` (bf16, d 128, S%64) -> ``dynaflow_hip.causal_attention``

* ``add(r, linear(x, w))`` (bf16, same shapes, the linear used once) -> ``dynaflow_hip.linear_add``
  (the residual addition as the GEMM's epilogue; same roundings, same bits)

* two or more bf16 ``linear`` nodes of the same activation (q / k / v projections) -> ONE
  ``dynaflow_hip.linear_multi`` against the stacked weights, results as column ranges of one buffer
* two ``rope`` nodes with the same tables (q and k) -> ``dynaflow_hip.rope_pair`` (one launch when the inputs
  are neighbouring column ranges of one buffer)
* the ``linear`` / ``linear_add`` whose result is what the sub-graph returns -> ``*_to_output``
  (writes into rows offered by the engine, so the nano-batch outputs need no concatenation)

With ``fuse_silu_epilogue`` a third rewrite follows: a ``silu_mul`` whose gate and up
inputs are two bf16 ``linear`` nodes of the same activation becomes one
``dynaflow_hip.gate_up_silu(x, w_gate, w_up)`` - the SiLU*mul as the GEMM's epilogue.

Everything else stays as traced and keeps running on PyTorch's own ROCm
kernels.  The pass only decides by what tracing recorded (``example_value``
dtypes and static trailing dimensions); token counts stay symbolic.

``silu_mul`` is emitted with ``round_silu=True`` for bf16: two separate bf16
aten kernels round ``silu(g)`` to bf16 before the product, and so does this.
"""
from __future__ import annotations

import copy
import operator
from typing import Any

import torch
import torch.fx as fx

_LINEAR_NAMES = {"linear"}
_SILU_NAMES = {"silu"}
_MUL_TARGETS = {operator.mul, torch.mul}


def _target_name(node: fx.Node) -> str | None:
    if node.op != "call_function":
        return None
    name = getattr(node.target, "__name__", None)
    if isinstance(node.target, torch._ops.OpOverload):   # "name.overload" -> "name"
        name = node.target.overloadpacket.__name__
    return name


def _example(node: Any) -> Any:
    if isinstance(node, fx.Node):
        return node.meta.get("example_value", None)
    return None


def _static_int(value: Any) -> int | None:
    return value if isinstance(value, int) and not isinstance(value, torch.SymInt) else None


def _traced_int(value: Any) -> int | None:
    """A dimension as a number: a plain int, or the value a symbolic dimension had while tracing.

    ``view(-1, seq_len, ...)`` of a token-shaped tensor leaves dynamo with an unsimplified
    expression such as ``s // (s // seq_len)`` for the constant ``seq_len``.  The operator that is
    put in checks the real size again at run time and raises if it cannot handle it.
    """
    if isinstance(value, torch.SymInt):
        hint = getattr(value.node, "hint", None)
        return int(hint) if hint is not None else None
    return value if isinstance(value, int) else None


def _linear_supported(x: Any, w: Any) -> bool:
    ex, ew = _example(x), _example(w)
    if not isinstance(ex, torch.Tensor) or not isinstance(ew, torch.Tensor):
        return False
    if ex.dtype != ew.dtype or ew.dim() != 2 or ex.dim() < 2:
        return False
    n, k = _static_int(ew.shape[0]), _static_int(ew.shape[1])
    if n is None or k is None:
        return False
    if ex.dtype == torch.bfloat16:
        return k % 64 == 0 and n % 8 == 0
    if ex.dtype == torch.float32:
        return k % 4 == 0
    return False


def _silu_mul_supported(g: Any) -> bool:
    eg = _example(g)
    if not isinstance(eg, torch.Tensor) or eg.dim() < 1:
        return False
    d = _static_int(eg.shape[-1])
    if d is None:
        return False
    if eg.dtype == torch.bfloat16:
        return d % 8 == 0
    if eg.dtype == torch.float32:
        return d % 4 == 0
    return False


def lower_to_hip(gm: fx.GraphModule, fuse_silu_epilogue: bool = False,
                 stack_projections: bool = True) -> tuple[fx.GraphModule, dict[str, int]]:
    """Return a lowered deep copy of ``gm`` and a count of each rewrite."""
    # registering the operators is a side effect of importing them
    from dynaflow_amd import ops

    lowered = copy.deepcopy(gm)
    graph = lowered.graph
    stats = {"linear": 0, "silu_mul": 0}
    if any(_target_name(n) == "rms_norm" and n.target is not ops.rms_norm for n in graph.nodes):
        stats["rms_norm"] = 0
        for node in list(graph.nodes):
            if _target_name(node) != "rms_norm" or node.target is ops.rms_norm:
                continue
            args = list(node.args) + [None] * (4 - len(node.args))
            x, shape = args[0], args[1]
            weight = args[2] if args[2] is not None else node.kwargs.get("weight")
            eps = args[3] if args[3] is not None else node.kwargs.get("eps")
            ex, ew = _example(x), _example(weight)
            if not isinstance(ex, torch.Tensor) or not isinstance(ew, torch.Tensor) or eps is None:
                continue
            h = _static_int(ex.shape[-1])
            if ex.dtype != torch.bfloat16 or ew.dtype != torch.bfloat16 or h is None or h % 8 or h > 16384:
                continue
            if len(tuple(shape)) != 1:
                continue
            with graph.inserting_before(node):
                new = graph.call_function(ops.rms_norm, (x, weight, float(eps)))
            new.meta = dict(node.meta)
            node.replace_all_uses_with(new)
            graph.erase_node(node)
            stats["rms_norm"] += 1
    if fuse_silu_epilogue:
        stats["gate_up_silu"] = 0

    for node in list(graph.nodes):
        name = _target_name(node)
        if name in _LINEAR_NAMES and node.target is not ops.linear:
            bias = node.args[2] if len(node.args) > 2 else node.kwargs.get("bias", None)
            if bias is not None or len(node.args) < 2:
                continue
            x, w = node.args[0], node.args[1]
            if not _linear_supported(x, w):
                continue
            with graph.inserting_before(node):
                new = graph.call_function(ops.linear, (x, w))
            new.meta = dict(node.meta)
            node.replace_all_uses_with(new)
            graph.erase_node(node)
            stats["linear"] += 1

    for node in list(graph.nodes):
        if node.op != "call_function" or node.target not in _MUL_TARGETS or len(node.args) != 2:
            continue
        lhs, rhs = node.args
        for silu, other in ((lhs, rhs), (rhs, lhs)):
            if not isinstance(silu, fx.Node) or not isinstance(other, fx.Node):
                continue
            if _target_name(silu) not in _SILU_NAMES or len(silu.users) != 1:
                continue
            if silu.kwargs.get("inplace", False):
                continue
            gate = silu.args[0]
            eg, eo = _example(gate), _example(other)
            if not _silu_mul_supported(gate) or not isinstance(eo, torch.Tensor):
                continue
            if eg.dtype != eo.dtype or eg.dim() != eo.dim():
                continue
            with graph.inserting_before(node):
                new = graph.call_function(ops.silu_mul, (gate, other, eg.dtype == torch.bfloat16))
            new.meta = dict(node.meta)
            node.replace_all_uses_with(new)
            graph.erase_node(node)
            graph.erase_node(silu)
            stats["silu_mul"] += 1
            break

    for node in list(graph.nodes):
        if _target_name(node) != "apply_rope" or len(node.args) != 3:
            continue
        et = _example(node.args[0])
        if not isinstance(et, torch.Tensor) or et.dtype != torch.bfloat16 or et.dim() != 4:
            continue
        d = _static_int(et.shape[-1])
        if d is None or d % 16:
            continue
        with graph.inserting_before(node):
            new = graph.call_function(ops.rope, tuple(node.args))
        new.meta = dict(node.meta)
        node.replace_all_uses_with(new)
        graph.erase_node(node)
        stats["rope"] = stats.get("rope", 0) + 1

    for node in list(graph.nodes):
        if _target_name(node) != "causal_gqa_attention" or len(node.args) != 3:
            continue
        et = _example(node.args[0])
        if not isinstance(et, torch.Tensor) or et.dtype != torch.bfloat16 or et.dim() != 4:
            continue
        seq, d = _traced_int(et.shape[1]), _static_int(et.shape[3])
        if seq is None or seq % 64 or d != 128:
            continue
        with graph.inserting_before(node):
            new = graph.call_function(ops.causal_attention, tuple(node.args))
        new.meta = dict(node.meta)
        node.replace_all_uses_with(new)
        graph.erase_node(node)
        stats["causal_attention"] = stats.get("causal_attention", 0) + 1

    for node in list(graph.nodes):
        if _target_name(node) != "attend_and_append" or len(node.args) != 9:
            continue
        et = _example(node.args[0])
        if not isinstance(et, torch.Tensor) or et.dtype != torch.bfloat16:
            continue
        with graph.inserting_before(node):
            new = graph.call_function(ops.decode_attention, tuple(node.args))
        new.meta = dict(node.meta)
        node.replace_all_uses_with(new)
        graph.erase_node(node)
        stats["decode_attention"] = stats.get("decode_attention", 0) + 1

    _ADD_TARGETS = {operator.add, torch.add}
    for node in list(graph.nodes):
        if node.op != "call_function" or node.target not in _ADD_TARGETS or len(node.args) != 2 or node.kwargs:
            continue
        for lin, other in ((node.args[1], node.args[0]), (node.args[0], node.args[1])):
            if not isinstance(lin, fx.Node) or not isinstance(other, fx.Node):
                continue
            if lin.op != "call_function" or lin.target is not ops.linear or len(lin.users) != 1:
                continue
            el, eo = _example(lin), _example(other)
            if not isinstance(el, torch.Tensor) or not isinstance(eo, torch.Tensor):
                continue
            if el.dtype != torch.bfloat16 or eo.dtype != torch.bfloat16 or el.dim() != eo.dim():
                continue
            # no broadcasting: every dimension equal as traced (a token dimension may be written as two
            # different symbolic expressions of the same number; the operator checks the real shapes)
            if any(_traced_int(a) != _traced_int(b) or _traced_int(a) is None for a, b in zip(el.shape, eo.shape)):
                continue
            with graph.inserting_before(node):
                new = graph.call_function(ops.linear_add, (lin.args[0], lin.args[1], other))
            new.meta = dict(node.meta)
            node.replace_all_uses_with(new)
            graph.erase_node(node)
            graph.erase_node(lin)
            stats["linear_add"] = stats.get("linear_add", 0) + 1
            break

    if fuse_silu_epilogue:
        for node in list(graph.nodes):
            if node.op != "call_function" or node.target is not ops.silu_mul:
                continue
            gate, up = node.args[0], node.args[1]
            if not (isinstance(gate, fx.Node) and isinstance(up, fx.Node)):
                continue
            if gate.target is not ops.linear or up.target is not ops.linear:
                continue
            if gate.args[0] is not up.args[0] or len(gate.users) != 1 or len(up.users) != 1:
                continue
            eg = _example(gate)
            if not isinstance(eg, torch.Tensor) or eg.dtype != torch.bfloat16:
                continue
            with graph.inserting_before(node):
                new = graph.call_function(ops.gate_up_silu, (gate.args[0], gate.args[1], up.args[1]))
            new.meta = dict(node.meta)
            node.replace_all_uses_with(new)
            graph.erase_node(node)
            graph.erase_node(gate)
            graph.erase_node(up)
            stats["gate_up_silu"] += 1
            stats["linear"] -= 2
            stats["silu_mul"] -= 1

    # Several bf16 projections of one activation (q / k / v; gate / up when they are not fused with the product)
    # become one GEMM against the stacked weights: narrow products (1024 columns) fill the chip badly on their own.
    # (``stack_projections=False`` keeps them apart: the stacked weights are a second copy of the members.)
    groups: dict[fx.Node, list[fx.Node]] = {}
    for node in graph.nodes:
        if not stack_projections:
            break
        if node.op == "call_function" and node.target is ops.linear and isinstance(node.args[0], fx.Node):
            ex, ew = _example(node.args[0]), _example(node.args[1])
            if (isinstance(ex, torch.Tensor) and ex.dtype == torch.bfloat16 and isinstance(ew, torch.Tensor)
                    and isinstance(node.args[1], fx.Node) and node.args[1].op == "placeholder"
                    and _static_int(ew.shape[0]) is not None and _static_int(ew.shape[0]) % 8 == 0):
                groups.setdefault(node.args[0], []).append(node)
    for x, members in groups.items():
        if len(members) < 2:
            continue
        with graph.inserting_before(members[0]):
            multi = graph.call_function(ops.linear_multi, (x, [m.args[1] for m in members]))
            parts = [graph.call_function(operator.getitem, (multi, i)) for i in range(len(members))]
        for member, part in zip(members, parts):
            part.meta = dict(member.meta)
            member.replace_all_uses_with(part)
            graph.erase_node(member)
        stats["linear_multi"] = stats.get("linear_multi", 0) + 1
        stats["linear"] -= len(members)

    # Two rotations with the same tables (q and k of one attention block) -> one operator, which rotates both
    # in one launch when it finds k's heads right behind q's (the column ranges of a stacked q / k / v product).
    order = {n: i for i, n in enumerate(graph.nodes)}
    ropes = [n for n in graph.nodes if n.op == "call_function" and n.target is ops.rope]
    while len(ropes) >= 2:
        first, second = ropes[0], ropes[1]
        ropes = ropes[2:]
        if first.args[1] is not second.args[1] or first.args[2] is not second.args[2]:
            continue
        if any(order[user] < order[second] for user in first.users):
            continue                                   # the first result is needed before the second input exists
        with graph.inserting_before(second):
            pair = graph.call_function(ops.rope_pair, (first.args[0], second.args[0], first.args[1], first.args[2]))
            parts = [graph.call_function(operator.getitem, (pair, i)) for i in range(2)]
        for node, part in zip((first, second), parts):
            part.meta = dict(node.meta)
            node.replace_all_uses_with(part)
            graph.erase_node(node)
        stats["rope_pair"] = stats.get("rope_pair", 0) + 1

    # The projection whose result the sub-graph returns (and nothing else reads) may write straight into the
    # rows that the engine offers for the model output; without an offer it behaves like the plain operator.
    output = next(n for n in graph.nodes if n.op == "output")
    returned = output.args[0]
    if isinstance(returned, fx.Node) and returned.op == "call_function" and len(returned.users) == 1:
        packet = getattr(returned.target, "overloadpacket", returned.target)   # traced calls carry the overload
        into = {ops.linear: ops.linear_to_output, ops.linear_add: ops.linear_add_to_output,
                ops.linear_fp8: ops.linear_fp8_to_output}.get(packet)
        if into is not None and not returned.kwargs:
            returned.target = into
            stats["to_output"] = 1

    graph.lint()
    lowered.recompile()
    return lowered, stats
