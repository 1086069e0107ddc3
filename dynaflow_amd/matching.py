"""Pattern rules over the ordered FX node list, the partitioner and the tagger.

Semantics follow dynaflow/matching.py and must give *identical* partition ids:

* ``Op(pattern)``  one ``call_function`` node whose ``target.__name__`` fully
  matches the regular expression                      (dynaflow/matching.py:8-15)
* ``Mod(cls)``     the longest run of nodes traced from one instance of exactly
  ``cls`` (innermost ``nn_module_stack`` entry)         (dynaflow/matching.py:18-49)
* ``MatchingRule`` a sequence of conditions matched left to right starting at
  a position; ``getitem`` nodes are absorbed for free   (dynaflow/matching.py:52-90)
* ``split_graph``  numbering of nodes into partitions + ``split_module``
                                                         (dynaflow/matching.py:93-126)
* ``tag_graph``    union of tag sets onto top-level sub-modules
                                                         (dynaflow/matching.py:129-158)
"""
from __future__ import annotations

import re
from collections.abc import Callable, Sequence
from dataclasses import dataclass

import torch
import torch.fx
from torch.fx.passes.split_module import split_module


def _is_getitem(node: torch.fx.Node) -> bool:
    return node.op == "call_function" and getattr(node.target, "__name__", None) == "getitem"


@dataclass(frozen=True)
class Op:
    """Matches a single function-call node by the name of its target."""

    pattern: str

    def matches(self, node: torch.fx.Node) -> bool:
        if node.op != "call_function":
            return False
        target = node.target
        if not callable(target):
            return False
        return re.fullmatch(self.pattern, target.__name__) is not None


@dataclass(frozen=True)
class Mod:
    """Matches the run of nodes that one ``target_cls`` instance produced."""

    target_cls: type[torch.nn.Module]

    @classmethod
    def get_module_info(cls, node: torch.fx.Node) -> tuple[str, type[torch.nn.Module]] | None:
        """Innermost owning module of ``node`` as ``(qualified name, class)``.

        Dynamo records the stack of enclosing modules in
        ``node.meta["nn_module_stack"]``; entries are ordered here by qualified
        name and the last one is taken as innermost.
        """
        stack = node.meta.get("nn_module_stack")
        if stack is None:
            return None
        entries = sorted(stack.values(), key=lambda entry: entry[0])
        name, klass = entries[-1]
        return name, klass

    def matches(self, node_list: Sequence[torch.fx.Node]) -> int:
        """Length of the leading run of ``node_list`` owned by one instance."""
        owner: str | None = None
        count = 0
        for node in node_list:
            info = self.get_module_info(node)
            if info is None:
                break
            name, klass = info
            if klass is not self.target_cls:
                break
            if owner is None:
                owner = name
            elif name != owner:
                break
            count += 1
        return count


@dataclass(frozen=True)
class MatchingRule:
    """A condition sequence plus an optional veto hook.

    ``matches`` returns how many nodes starting at ``start_idx`` the rule
    covers (0 = no match).  ``hook(node_list, start_idx)`` may reject a match.
    """

    condition: Op | Mod | tuple[Op | Mod, ...]
    hook: Callable[[list[torch.fx.Node], int], bool] | None = None

    def _conditions(self) -> tuple[Op | Mod, ...]:
        if isinstance(self.condition, (Op, Mod)):
            return (self.condition,)
        return tuple(self.condition)

    def matches(self, node_list: list[torch.fx.Node], start_idx: int) -> int:
        conditions = self._conditions()
        pos = start_idx
        which = 0
        total = len(node_list)
        # Conditions are consumed in order.  A getitem node never consumes a
        # condition; it is swallowed wherever it appears while conditions are
        # still pending (also in front of the first one).  If the list ends
        # with conditions pending, the span matched so far is still returned.
        while pos < total and which < len(conditions):
            node = node_list[pos]
            if _is_getitem(node):
                pos += 1
                continue
            cond = conditions[which]
            if isinstance(cond, Op):
                if not cond.matches(node):
                    return 0
                pos += 1
            else:
                run = cond.matches(node_list[pos:])
                if run == 0:
                    return 0
                pos += run
            which += 1
        span = pos - start_idx
        if span > 0 and self.hook is not None and not self.hook(node_list, start_idx):
            return 0
        return span


def assign_partition_ids(
    nodes: list[torch.fx.Node], split_rules: Sequence[MatchingRule]
) -> dict[torch.fx.Node, int]:
    """Number every node of the ordered list with its partition id.

    The running id is bumped once *before* and once *after* each matched span,
    so a match always sits alone in its partition and unmatched stretches on
    either side get different ids.  Rules are tried in list order; the first
    one with a non-empty match wins.  Ids may therefore be sparse.
    """
    ids: dict[torch.fx.Node, int] = {}
    current = 0
    pos = 0
    while pos < len(nodes):
        span = 0
        for rule in split_rules:
            span = rule.matches(nodes, pos)
            if span > 0:
                break
        if span > 0:
            current += 1
            for node in nodes[pos : pos + span]:
                ids[node] = current
            current += 1
            pos += span
        else:
            ids[nodes[pos]] = current
            pos += 1
    return ids


def split_graph(graph: torch.fx.GraphModule, split_rules: list[MatchingRule]) -> torch.fx.GraphModule:
    """Cut a full graph into ``submod_<id>`` sub-modules around rule matches."""
    ids = assign_partition_ids(list(graph.graph.nodes), split_rules)
    return split_module(
        graph,
        None,
        lambda node: ids.get(node, 0),
        keep_original_order=True,
    )


def tag_graph(gm: torch.fx.GraphModule, tag_rules: dict[MatchingRule, set[str]]) -> None:
    """Give each top-level sub-graph a ``tag`` set from the rules it contains."""
    for name, module in gm.named_modules():
        if name == "" or "." in name or not hasattr(module, "graph"):
            continue
        tags: set[str] = set()
        nodes = list(module.graph.nodes)
        pos = 0
        while pos < len(nodes):
            step = 1
            for rule, rule_tags in tag_rules.items():
                span = rule.matches(nodes, pos)
                if span > 0:
                    tags.update(rule_tags)
                    step = span
                    break
            pos += step
        module.tag = tags  # type: ignore[assignment]
