"""Which steps may run from a captured graph, decided on the host: no GPU needed."""

from __future__ import annotations

from types import SimpleNamespace

from cie_amd.engine.graphs import DecodeGraphs, MixedGraphs
from cie_amd.engine.runner import StepEntry


def graphs(limit=4, largest=8):
    runner = SimpleNamespace(config=SimpleNamespace(max_model_len=4096, token_budget=256))
    return MixedGraphs(runner, SimpleNamespace(largest=largest), limit)


def entry(name, count, start=0, want=None):
    return StepEntry(name, list(range(count)), start, (count - 1,) if want is None else want)


def test_decode_buckets_are_powers_of_two():
    assert [DecodeGraphs.bucket_of(n) for n in (1, 2, 3, 4, 5, 8, 9, 64)] == [1, 2, 4, 4, 8, 8, 16, 64]


def test_shape_is_the_decode_bucket_and_the_portion_lengths():
    g = graphs()
    step = [entry("a", 1, 40), entry("b", 1, 7), entry("c", 1, 90), entry("p", 16, 32), entry("q", 5, 0, want=())]
    assert g.shape_of(step) == (4, (16, 5))
    assert g.shape_of([entry("p", 16, 32)]) == (0, (16,))
    # other positions, other requests, other contexts: the same shape
    assert g.shape_of([entry("x", 1, 3), entry("y", 1, 9), entry("z", 1, 1), entry("w", 16, 640), entry("v", 5, 5)]) == (4, (16, 5))


def test_steps_that_no_graph_takes():
    g = graphs()
    assert g.shape_of([entry("a", 1), entry("b", 1)]) is None                       # decode only: the decode graphs' business
    assert g.shape_of([entry("p", 16, want=(3,))]) is None                           # logits inside a portion
    assert g.shape_of([entry("p", 16, want=(14, 15))]) is None
    assert g.shape_of([entry(str(i), 4) for i in range(5)]) is None                  # more than four portions
    assert g.shape_of([entry("p", 200)]) is None                                     # more rows than the host is slower for
    assert g.shape_of([entry(str(i), 1) for i in range(9)] + [entry("p", 8)]) is None  # more decode rows than the largest bucket
    assert g.shape_of([entry(str(i), 1) for i in range(5)] + [entry("p", 121)]) is None  # bucket 8 + 121 rows


def test_a_shape_is_wanted_from_its_second_coming_and_never_with_limit_zero():
    g = graphs()
    step = [entry("a", 1, 4), entry("p", 16, 32)]
    assert g.wants(step) is None
    assert g.wants(step) == (1, (16,))
    assert g.wants([entry("b", 1, 9), entry("q", 16, 0)]) == (1, (16,))
    assert g.wants([entry("b", 1, 9), entry("q", 17, 0)]) is None
    off = graphs(limit=0)
    assert off.wants(step) is None and off.wants(step) is None
