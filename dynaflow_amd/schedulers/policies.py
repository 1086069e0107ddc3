"""Split policies: how a batch of requests is cut into nano-batches.

Pure functions of integers, shared by the schedulers.

``balanced_two_way``  the NanoFlow rule of
    examples/ae/scheduler/hf/nanoflow.py:65-120 (the same code is repeated in
    the vllm / sglang / dbo / tokenweave schedulers): cut once, at the request
    boundary that best balances the token counts of the two sides.
``equal_n_way``       the rule of examples/ae/scheduler/megatron/nanoflow.py:
    42-76: ``n`` equal chunks, the last one taking the remainder, with fewer
    chunks when they would get too small.
"""
from __future__ import annotations

from collections.abc import Sequence
from itertools import accumulate

from dynaflow_amd.interface import InputInfo, SplitConfig
from dynaflow_amd.utils import pack_tokens


def _single(batch_size: int, total: int, padded: int, use_cudagraph: bool) -> SplitConfig:
    return SplitConfig(
        num_nano_batches=1,
        batch_sizes=[batch_size],
        batch_indices=[0, batch_size],
        num_tokens=[total],
        num_tokens_padded=[padded],
        split_indices=[0, total],
        is_dryrun=False,
        use_cudagraph=use_cudagraph,
    )


def balanced_two_way(
    input_info: InputInfo,
    use_cudagraph: bool,
    min_nano_split_tokens: int,
    capture_sizes: Sequence[int],
) -> SplitConfig:
    """One cut at the request boundary with the smallest token imbalance.

    Among equally good boundaries the first wins.  If either side would hold
    fewer than ``min_nano_split_tokens`` tokens the batch stays whole.  Under
    graphs each side is padded to a capture size; if any side does not fit,
    graphs are switched off for this forward.
    """
    prefix = [0] + list(accumulate(input_info.num_tokens))
    total = prefix[-1]
    cut = 0
    best = None
    for i, left in enumerate(prefix):
        imbalance = abs(left - (total - left))
        if best is None or imbalance < best:
            best, cut = imbalance, i
    left, right = prefix[cut], total - prefix[cut]

    if left < min_nano_split_tokens or right < min_nano_split_tokens:
        padded = total
        if use_cudagraph:
            padded, use_cudagraph = pack_tokens(total, capture_sizes)
        return _single(input_info.batch_size, total, padded, use_cudagraph)

    padded_sides = [left, right]
    if use_cudagraph:
        packed = [pack_tokens(n, capture_sizes) for n in padded_sides]
        if all(ok for _, ok in packed):
            padded_sides = [size for size, _ in packed]
        else:
            use_cudagraph = False
    return SplitConfig(
        num_nano_batches=2,
        batch_sizes=[cut, input_info.batch_size - cut],
        batch_indices=[0, cut, input_info.batch_size],
        num_tokens=[left, right],
        num_tokens_padded=padded_sides,
        split_indices=[0, left, total],
        is_dryrun=False,
        use_cudagraph=use_cudagraph,
    )


def equal_n_way(
    input_info: InputInfo,
    use_cudagraph: bool,
    num_nano_batches: int,
    min_nano_split_tokens: int,
) -> SplitConfig:
    """``n`` chunks of ``batch_size // n`` requests, remainder to the last.

    When a chunk would fall below ``min_nano_split_tokens`` the number of
    chunks drops to ``max(1, batch_size // min_nano_split_tokens)``.  Token
    offsets come from the requests' token counts; with one token per request
    (the case the reference rule is written for, where it uses the request
    count as the token count) offsets and request indices coincide.
    """
    batch_size = input_info.batch_size
    n = num_nano_batches
    chunk = batch_size // n
    if chunk < min_nano_split_tokens:
        n = max(1, batch_size // min_nano_split_tokens)
        chunk = batch_size // n if n > 1 else batch_size
    per_request = list(input_info.num_tokens)
    uniform = len(per_request) != batch_size or all(t == 1 for t in per_request)
    if n <= 1:
        total = batch_size if uniform else sum(per_request)
        return _single(batch_size, total, total, use_cudagraph)
    sizes = [chunk] * n
    sizes[-1] = batch_size - chunk * (n - 1)
    indices = [chunk * i for i in range(n)] + [batch_size]
    if uniform:
        tokens, offsets = list(sizes), list(indices)
    else:
        prefix = [0] + list(accumulate(per_request))
        offsets = [prefix[i] for i in indices]
        tokens = [offsets[i + 1] - offsets[i] for i in range(n)]
    return SplitConfig(
        num_nano_batches=n,
        batch_sizes=sizes,
        batch_indices=indices,
        num_tokens=tokens,
        num_tokens_padded=list(tokens),
        split_indices=offsets,
        is_dryrun=False,
        use_cudagraph=use_cudagraph,
    )
