"""Small host helpers shared by schedulers and the engine."""
from __future__ import annotations

from collections.abc import Sequence


def pack_tokens(num_tokens: int, cudagraph_capture_sizes: Sequence[int]) -> tuple[int, bool]:
    """Round a token count up to the nearest graph-capture size.

    Returns ``(padded, True)`` where ``padded`` is the least capture size that
    is ``>= num_tokens``; when no capture size is large enough the count is
    returned unchanged with ``False`` (graphs cannot be used for it).
    Same contract as dynaflow/utils.py:1-5.
    """
    best = None
    for size in cudagraph_capture_sizes:
        if size >= num_tokens and (best is None or size < best):
            best = size
    if best is None:
        return num_tokens, False
    return best, True
