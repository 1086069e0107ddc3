"""Pins oracle/schedule_trace.py with hand-derived traces and checks the real
engine + schedulers (on the recording device seam) against it."""
import asyncio

import pytest
import torch

from conftest import load_golden
from oracle import schedule_trace as ref

CASES = load_golden("schedule_traces.json")["cases"]


def norm_top(top):
    return [tuple(t) if isinstance(t, list) else t for t in top]


@pytest.mark.parametrize("case", CASES, ids=lambda c: c["name"])
def test_launch_order_golden(case):
    trace = ref.simulate(norm_top(case["top"]), case["n"], case["scheduler"], lambda m: case["streams"][m])
    assert ref.launches(trace) == [tuple(x) for x in case["launches"]]
    if "trace" in case:
        assert trace == [tuple(x) for x in case["trace"]]


@pytest.mark.parametrize("case", CASES, ids=lambda c: c["name"])
def test_trace_invariants(case):
    n = case["n"]
    trace = ref.simulate(norm_top(case["top"]), n, case["scheduler"], lambda m: case["streams"][m])
    modules = [t[1] for t in norm_top(case["top"]) if isinstance(t, tuple)]
    launched = ref.launches(trace)
    # every (module, nano-batch) exactly once; per nano-batch in graph order
    assert sorted((m, b) for m, b, _ in launched) == sorted((m, b) for m in modules for b in range(n))
    for b in range(n):
        assert [m for m, bb, _ in launched if bb == b] == modules
    assert sorted(e[1] for e in trace if e[0] == "sentinel") == list(range(n))
    # event chain: each launch is bracketed by wait / record of its own nano-batch on its stream
    for i, e in enumerate(trace):
        if e[0] == "launch":
            assert trace[i - 1] == ("wait", e[2], e[3]) and trace[i + 1] == ("record", e[2], e[3])


def test_early_return_is_a_deadlock():
    def lazy(n):
        op = yield ("pop", 0)
        yield ("exec", op)

    ref.SCHEDULERS["lazy"] = lazy
    try:
        with pytest.raises(ref.Deadlock):
            ref.simulate(["in", ("mod", "s0"), "fn", ("mod", "s1"), "out"], 1, "lazy", lambda m: "A")
    finally:
        del ref.SCHEDULERS["lazy"]
