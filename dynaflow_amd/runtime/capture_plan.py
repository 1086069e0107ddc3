"""From which stream a multi-stream schedule can be captured into one hipGraph.

Stream capture starts on one stream (the origin); every other stream joins the capture when it first
waits for an event that a capturing stream recorded.  The HIP runtime books that as "the waiting
stream is a child of the recording stream" - again at every later wait, whichever streams are involved,
unless the waiting stream is the origin - and the end of the capture walks the children of the origin,
their children and so on.  A schedule in which a stream other than the origin waits for an event that it
recorded itself, or in which two such streams wait for each other's events, makes that walk endless: the
process dies with a segmentation fault inside the end-of-capture call.  That is what five captures of
this package did (the one-stream schedule, one stream per nano-batch, the six-segment decode schedule),
and no capture that worked had such a cycle.

Two things keep a schedule clear of it, neither of which changes what the graph computes:

* a wait for an event on the very stream that recorded it orders nothing that stream order does not
  order already, so the device seam never issues it (``HipEvent.wait``);
* the origin is exempt, so a schedule whose two streams wait for each other is captured FROM one of them
  (``choose_origin``) instead of from a third stream.

The functions below work on the (``"record"`` | ``"wait"``, event id, stream) log that both device seams
write, so the plan for a schedule can be made - and tested - without a GPU.
"""
from __future__ import annotations

from collections.abc import Hashable, Iterable

LogEntry = tuple


def wait_edges(log: Iterable[LogEntry]) -> list[tuple[Hashable, Hashable]]:
    """(recording stream, waiting stream) of every wait for an event that has been recorded, in log order."""
    recorded_on: dict[Hashable, Hashable] = {}
    edges = []
    for entry in log:
        kind = entry[0]
        if kind == "record":
            recorded_on[entry[1]] = entry[2]
        elif kind == "wait" and entry[1] in recorded_on:
            edges.append((recorded_on[entry[1]], entry[2]))
    return edges


def join_cycle(log: Iterable[LogEntry], caller: Hashable, origin: Hashable) -> list | None:
    """A cycle in the child-of relation that capturing ``log`` from ``origin`` would build, or None.

    ``log`` was written with ``caller`` as the current stream of the forward; under capture the origin takes
    that part.  Waits on the recording stream are left out (the seam does not issue them), and so are the
    waits of the origin (it is never made anybody's child).
    """
    children: dict[Hashable, set] = {}
    for src, dst in wait_edges(log):
        src = origin if src == caller else src
        dst = origin if dst == caller else dst
        if src == dst or dst == origin:
            continue
        children.setdefault(src, set()).add(dst)
    state: dict[Hashable, int] = {}

    def walk(node: Hashable, path: list) -> list | None:
        state[node] = 1
        for child in sorted(children.get(node, ()), key=repr):
            if state.get(child) == 1:
                loop = path + [node, child]
                return loop[loop.index(child):]          # the cycle itself, without the way that led to it
            if child not in state:
                found = walk(child, path + [node])
                if found:
                    return found
        state[node] = 2
        return None

    for node in sorted(children, key=repr):
        if node not in state:
            found = walk(node, [])
            if found:
                return found
    return None


def choose_origin(log: Iterable[LogEntry], caller: Hashable) -> Hashable | None:
    """The stream to start the capture on: ``caller`` if that is safe, else the first stream of the log
    (in order of appearance) from which the schedule has no cycle, else None."""
    log = list(log)
    candidates = [caller]
    for entry in log:
        if entry[0] in ("record", "wait") and entry[2] not in candidates:
            candidates.append(entry[2])
    for origin in candidates:
        if join_cycle(log, caller, origin) is None:
            return origin
    return None
