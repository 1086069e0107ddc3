"""Pins oracle/split_policy.py: hand-derived goldens, brute force, invariants;
then checks the product's policies against it bit for bit."""
import dataclasses
import itertools
import random

import pytest

from conftest import load_golden
from dynaflow_amd.interface import InputInfo
from dynaflow_amd.manager import trivial_split
from dynaflow_amd.schedulers import policies
from dynaflow_amd.utils import pack_tokens
from oracle import split_policy as ref

CASES = load_golden("split_cases.json")
FIELDS = ["num_nano_batches", "batch_sizes", "batch_indices", "num_tokens", "num_tokens_padded", "split_indices"]


def as_dict(cfg):
    return dataclasses.asdict(cfg)


@pytest.mark.parametrize("case", CASES["pack_tokens"], ids=lambda c: f"{c['n']}-{c['sizes']}")
def test_pack_tokens_golden(case):
    want = tuple(case["expect"])
    assert ref.pack_tokens(case["n"], case["sizes"]) == want
    assert pack_tokens(case["n"], case["sizes"]) == want


def test_pack_tokens_is_least_capture_size_not_below_n():
    rng = random.Random(0)
    for _ in range(2000):
        sizes = rng.sample(range(1, 64), rng.randint(1, 6))
        n = rng.randint(1, 80)
        padded, ok = ref.pack_tokens(n, sizes)
        fitting = [s for s in sizes if s >= n]
        assert ok == bool(fitting)
        assert padded == (min(fitting) if fitting else n)
        assert pack_tokens(n, sizes) == (padded, ok)


@pytest.mark.parametrize("case", CASES["balanced_two_way"], ids=lambda c: c["name"])
def test_balanced_two_way_golden(case):
    got = ref.balanced_two_way(case["batch_size"], case["num_tokens"], case["use_cudagraph"], case["min"], case["sizes"])
    for key, want in case["expect"].items():
        assert got[key] == want, key
    prod = policies.balanced_two_way(
        InputInfo(case["batch_size"], case["num_tokens"], sum(case["num_tokens"])),
        case["use_cudagraph"], case["min"], case["sizes"])
    for key, want in case["expect"].items():
        assert as_dict(prod)[key] == want, key


@pytest.mark.parametrize("case", CASES["equal_n_way"], ids=lambda c: c["name"])
def test_equal_n_way_golden(case):
    got = ref.equal_n_way(case["batch_size"], False, case["n"], case["min"])
    for key, want in case["expect"].items():
        assert got[key] == want, key
    prod = policies.equal_n_way(InputInfo(case["batch_size"], [case["batch_size"]], case["batch_size"]),
                                False, case["n"], case["min"])
    for key, want in case["expect"].items():
        assert as_dict(prod)[key] == want, key


def brute_force_cut(num_tokens):
    """Independent O(n^2) search: smallest |left - right|, earliest cut on ties."""
    best, best_cut = None, None
    for cut in range(len(num_tokens) + 1):
        left = sum(num_tokens[:cut])
        right = sum(num_tokens[cut:])
        if best is None or abs(left - right) < best:
            best, best_cut = abs(left - right), cut
    return best_cut


def check_invariants(cfg, batch_size, total):
    n = cfg["num_nano_batches"]
    assert len(cfg["batch_sizes"]) == len(cfg["num_tokens"]) == len(cfg["num_tokens_padded"]) == n
    assert len(cfg["batch_indices"]) == len(cfg["split_indices"]) == n + 1
    assert cfg["split_indices"][0] == 0 and cfg["split_indices"][-1] == total
    assert cfg["batch_indices"][0] == 0 and cfg["batch_indices"][-1] == batch_size
    assert sum(cfg["batch_sizes"]) == batch_size and sum(cfg["num_tokens"]) == total
    for b in range(n):
        assert cfg["split_indices"][b + 1] - cfg["split_indices"][b] == cfg["num_tokens"][b]
        assert cfg["batch_indices"][b + 1] - cfg["batch_indices"][b] == cfg["batch_sizes"][b]
        assert cfg["num_tokens_padded"][b] >= cfg["num_tokens"][b]
    if n > 1:
        assert all(a < b for a, b in zip(cfg["split_indices"], cfg["split_indices"][1:]))


def test_balanced_two_way_brute_force_and_product_parity():
    rng = random.Random(1)
    sizes = [16, 64, 256, 1024]
    for _ in range(3000):
        bs = rng.randint(1, 12)
        toks = [rng.randint(1, 300) for _ in range(bs)]
        use_graph = rng.random() < 0.5
        minimum = rng.choice([1, 16, 64, 200])
        got = ref.balanced_two_way(bs, toks, use_graph, minimum, sizes)
        check_invariants(got, bs, sum(toks))
        cut = brute_force_cut(toks)
        left, right = sum(toks[:cut]), sum(toks[cut:])
        if left < minimum or right < minimum:
            assert got["num_nano_batches"] == 1
        else:
            assert got["num_nano_batches"] == 2 and got["batch_indices"][1] == cut
            assert got["split_indices"][1] == left
        if got["use_cudagraph"]:
            assert use_graph and all(p in sizes for p in got["num_tokens_padded"])
        else:
            assert got["num_tokens_padded"] == got["num_tokens"]
        prod = as_dict(policies.balanced_two_way(InputInfo(bs, toks, sum(toks)), use_graph, minimum, sizes))
        for key in FIELDS + ["use_cudagraph", "is_dryrun"]:
            assert prod[key] == got[key], key


def test_equal_n_way_invariants_and_product_parity():
    for bs, n, minimum in itertools.product([1, 2, 7, 64, 100, 128, 255, 256, 4096, 8192], [1, 2, 3, 4, 8], [1, 64, 128]):
        got = ref.equal_n_way(bs, False, n, minimum)
        check_invariants(got, bs, bs)
        if got["num_nano_batches"] > 1:
            sizes = got["batch_sizes"]
            assert all(s == sizes[0] for s in sizes[:-1]) and sizes[-1] >= sizes[0]
        prod = as_dict(policies.equal_n_way(InputInfo(bs, [bs], bs), False, n, minimum))
        for key in FIELDS:
            assert prod[key] == got[key], (bs, n, minimum, key)
        # one token per request: the same answer from the per-request token list
        if bs <= 256:
            prod = as_dict(policies.equal_n_way(InputInfo(bs, [1] * bs, bs), False, n, minimum))
            for key in FIELDS:
                assert prod[key] == got[key]


def test_equal_n_way_multi_token_requests_use_prefix_sums():
    cfg = policies.equal_n_way(InputInfo(4, [5, 7, 2, 9], 23), False, 2, 1)
    assert cfg.batch_indices == [0, 2, 4] and cfg.split_indices == [0, 12, 23] and cfg.num_tokens == [12, 11]
    cfg.validate()


def test_trivial_split_matches_restatement():
    for dry, graph in itertools.product([False, True], repeat=2):
        got = as_dict(trivial_split(3, [5, 6, 7], dry, graph))
        want = ref.trivial_split(3, [5, 6, 7], dry, graph)
        for key, value in want.items():
            assert got[key] == value
        assert got["allow_fallback"] is True
