"""Split policies restated on plain integers (returns dicts, not dataclasses).

Follows, line by line:
  pack_tokens        dynaflow/utils.py:1-5
  trivial_split      dynaflow/manager.py:139-149
  balanced_two_way   examples/ae/scheduler/hf/nanoflow.py:65-120
  equal_n_way        examples/ae/scheduler/megatron/nanoflow.py:42-76
"""
import itertools


def pack_tokens(num_tokens, capture_sizes):
    # utils.py:3-5
    if num_tokens <= max(capture_sizes):
        return min(size for size in capture_sizes if size >= num_tokens), True
    return num_tokens, False


def _record(n, batch_sizes, batch_indices, num_tokens, padded, split_indices, is_dryrun, use_cudagraph):
    return {
        "num_nano_batches": n,
        "batch_sizes": list(batch_sizes),
        "batch_indices": list(batch_indices),
        "num_tokens": list(num_tokens),
        "num_tokens_padded": list(padded),
        "split_indices": list(split_indices),
        "is_dryrun": is_dryrun,
        "use_cudagraph": use_cudagraph,
    }


def trivial_split(batch_size, num_tokens, is_dryrun, use_cudagraph):
    # manager.py:139-149
    total = sum(num_tokens)
    return _record(1, [batch_size], [0, batch_size], [total], [total], [0, total], is_dryrun, use_cudagraph)


def balanced_two_way(batch_size, num_tokens, use_cudagraph, min_nano_split_tokens, capture_sizes):
    # hf/nanoflow.py:71-76: prefix sums and the FIRST index minimising the imbalance
    prefix_sum = [0] + list(itertools.accumulate(num_tokens))
    mid = min(
        range(len(prefix_sum)),
        key=lambda i: abs(prefix_sum[i] - (prefix_sum[-1] - prefix_sum[i])),
    )
    left = prefix_sum[mid]
    right = prefix_sum[-1] - prefix_sum[mid]
    if left < min_nano_split_tokens or right < min_nano_split_tokens:
        # hf/nanoflow.py:78-96
        padded = prefix_sum[-1]
        if use_cudagraph:
            padded, use_cudagraph = pack_tokens(prefix_sum[-1], capture_sizes)
        return _record(1, [batch_size], [0, batch_size], [prefix_sum[-1]], [padded], [0, prefix_sum[-1]],
                       False, use_cudagraph)
    # hf/nanoflow.py:97-120
    padded = [left, right]
    if use_cudagraph:
        packed = [pack_tokens(n, capture_sizes) for n in padded]
        if all(ok for _, ok in packed):
            padded = [p for p, _ in packed]
        else:
            use_cudagraph = False
    return _record(2, [mid, batch_size - mid], [0, mid, batch_size], [left, right], padded,
                   [0, left, prefix_sum[-1]], False, use_cudagraph)


def equal_n_way(batch_size, use_cudagraph, num_nano_batches, min_nano_split_tokens):
    # megatron/nanoflow.py:46-76 (the request count doubles as the token count there)
    n = num_nano_batches
    chunk = batch_size // n
    if chunk < min_nano_split_tokens:
        n = max(1, batch_size // min_nano_split_tokens)
        chunk = batch_size // n if n > 1 else batch_size
    if n <= 1:
        return _record(1, [batch_size], [0, batch_size], [batch_size], [batch_size], [0, batch_size],
                       False, use_cudagraph)
    sizes = [chunk] * n
    sizes[-1] = batch_size - chunk * (n - 1)
    indices = [chunk * i for i in range(n)] + [batch_size]
    return _record(n, sizes, indices, sizes, sizes, indices, False, use_cudagraph)
