"""Deterministic replay of the engine <-> scheduler protocol, without asyncio.

Restates, as a single-threaded simulation, what the two coroutines of a forward
do to the device: which (sub-graph, nano-batch) pairs are launched in which
order on which stream, and the per-nano-batch event chain around them.

  engine    dynaflow/runtime/engine.py:222-424 (preamble 248-266, publish loop
            272-293, serve one request 295-389, advance 391-421)
  round-robin scheduler   examples/ae/scheduler/hf/nanoflow.py:122-146
  staggered scheduler     examples/ae/scheduler/megatron/nanoflow.py:78-102

The graph is given as the ordered list of top-level node kinds: "in" for a
placeholder, "fn" for any inline node (getitem, call_function ...),
("mod", name) for a sub-graph call and "out" for the output node.  The engine
always runs until it blocks on the execute queue before the scheduler resumes
(queue puts on a non-full asyncio queue do not yield), which makes the
interleaving deterministic.
"""
from collections import deque

QUEUE_LIMIT = 10  # manager.py:215


class Deadlock(RuntimeError):
    pass


def _round_robin(n):
    # hf/nanoflow.py:127-146 (iterating over a copy of the live list)
    live = list(range(n))
    while live:
        ops = []
        for b in list(live):
            op = yield ("pop", b)
            if op is None:
                live.remove(b)
                continue
            ops.append(op)
        for op in ops:
            yield ("exec", op)


def _staggered(n):
    # megatron/nanoflow.py:82-102
    live = list(range(n))
    if n >= 2:
        op = yield ("pop", 0)
        if op is None:
            live.remove(0)
        else:
            yield ("exec", op)
    while live:
        for b in list(live):
            op = yield ("pop", b)
            if op is None:
                live.remove(b)
                continue
            yield ("exec", op)


SCHEDULERS = {"round_robin": _round_robin, "staggered": _staggered}


def simulate(top, n, scheduler, stream_of, caller_stream="caller"):
    """Return the device-visible trace of one forward.

    ``stream_of(module_name)`` names the stream the scheduler makes current for
    that sub-graph.  Trace entries:
      ("record", b, stream) / ("wait", b, stream)   event chain of nano-batch b
      ("launch", module, b, stream)
      ("sentinel", b)                               None put on b's op queue
      ("join", b, stream)                           final wait by the caller
    """
    trace = []
    pos = [0] * n
    queues = [deque() for _ in range(n)]
    outstanding = [deque() for _ in range(n)]

    def kind(b):
        return top[pos[b]] if pos[b] < len(top) else None

    def is_mod(k):
        return isinstance(k, tuple) and k[0] == "mod"

    def advance(b):
        # engine.py:393-421: inline nodes up to the next sub-graph call; at the
        # output node the result is taken and the sentinel is queued
        while pos[b] < len(top):
            k = kind(b)
            if is_mod(k):
                return
            pos[b] += 1
            if k == "out":
                queues[b].append(None)
                trace.append(("sentinel", b))
                return

    def publish():
        # engine.py:272-293
        for b in range(n):
            while pos[b] < len(top) and is_mod(kind(b)) and len(queues[b]) < QUEUE_LIMIT:
                op = (kind(b)[1], b)
                queues[b].append(op)
                outstanding[b].append(op)
                pos[b] += 1

    # engine.py:248-266: bind inputs of every nano-batch, record its first event
    for b in range(n):
        while pos[b] < len(top) and not is_mod(kind(b)) and kind(b) != "out":
            pos[b] += 1
        trace.append(("record", b, caller_stream))
    publish()

    sched = SCHEDULERS[scheduler](n)
    reply = None
    try:
        request = sched.send(None)
        while True:
            if request[0] == "pop":
                b = request[1]
                if not queues[b]:
                    raise Deadlock(f"scheduler popped nano-batch {b} with nothing ready")
                reply = queues[b].popleft()
            else:
                module, b = request[1]
                stream = stream_of(module)
                # engine.py:302-303, 372-389
                trace.append(("wait", b, stream))
                trace.append(("launch", module, b, stream))
                trace.append(("record", b, stream))
                if not outstanding[b] or outstanding[b][0] != (module, b):
                    raise AssertionError(f"{module} of nano-batch {b} executed out of order")
                outstanding[b].popleft()
                for other in range(n):
                    if not outstanding[other]:
                        advance(other)
                publish()
                reply = None
            request = sched.send(reply)
    except StopIteration:
        pass
    if any(pos[b] < len(top) for b in range(n)):
        raise Deadlock("scheduler returned before every nano-batch finished")
    # manager.py:236-237
    for b in range(n):
        trace.append(("join", b, caller_stream))
    return trace


def launches(trace):
    return [(e[1], e[2], e[3]) for e in trace if e[0] == "launch"]
