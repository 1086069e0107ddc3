"""Graph matching, partition numbering and tagging on plain node records.

A node is a dict ``{"op": str, "name": str, "stack": [(qualname, cls), ...]}``
where ``name`` stands for ``target.__name__`` of a ``call_function`` node and
``stack`` for the values of ``meta["nn_module_stack"]`` (absent = no key).
Conditions are ``("op", regex)`` or ``("mod", cls)``; a rule is
``{"cond": [conditions...], "hook": callable or None}``.

Follows dynaflow/matching.py: Op.matches 12-15, Mod.get_module_info 22-31,
Mod.matches 33-49, MatchingRule.matches 57-90, split_graph numbering 99-117,
tag_graph 143-158.  The final ``split_module`` call (matching.py:119-124) is the
same torch function in both implementations and is not restated.
"""
import re


def op_matches(pattern, node):
    # matching.py:12-15
    if node["op"] != "call_function" or node.get("name") is None:
        return False
    return bool(re.fullmatch(pattern, node["name"]))


def module_info(node):
    # matching.py:22-31: entries sorted by qualified name, last one wins
    if "stack" not in node or node["stack"] is None:
        return None
    entries = sorted(node["stack"], key=lambda e: e[0])
    return entries[-1]


def mod_matches(cls, nodes):
    # matching.py:33-49
    last = None
    idx = 0
    while idx < len(nodes):
        info = module_info(nodes[idx])
        if info is None:
            return idx
        name, klass = info
        if klass is not cls:
            return idx
        if last is None:
            last = name
        elif last != name:
            return idx
        idx += 1
    return idx


def rule_matches(rule, nodes, start):
    # matching.py:57-90
    conds = rule["cond"]
    node_idx = start
    cond_idx = 0
    while node_idx < len(nodes) and cond_idx < len(conds):
        node = nodes[node_idx]
        if node["op"] == "call_function" and node.get("name") == "getitem":
            node_idx += 1
            continue
        kind, arg = conds[cond_idx]
        if kind == "op":
            if not op_matches(arg, node):
                return 0
            node_idx += 1
        else:
            run = mod_matches(arg, nodes[node_idx:])
            if run == 0:
                return 0
            node_idx += run
        cond_idx += 1
    hook = rule.get("hook")
    if node_idx - start > 0 and hook is not None and not hook(nodes, start):
        return 0
    return node_idx - start


def partition_ids(nodes, rules):
    # matching.py:99-117
    ids = []
    current = 0
    idx = 0
    while idx < len(nodes):
        matched = False
        for rule in rules:
            length = rule_matches(rule, nodes, idx)
            if length > 0:
                current += 1
                ids.extend([current] * length)
                idx += length
                current += 1
                matched = True
                break
        if not matched:
            ids.append(current)
            idx += 1
    return ids


def subgraph_tags(nodes, tag_rules):
    # matching.py:146-158; tag_rules is a list of (rule, set) in dict order
    tags = set()
    idx = 0
    while idx < len(nodes):
        matched = False
        for rule, rule_tags in tag_rules:
            length = rule_matches(rule, nodes, idx)
            if length > 0:
                tags |= set(rule_tags)
                idx += length
                matched = True
                break
        if not matched:
            idx += 1
    return tags
