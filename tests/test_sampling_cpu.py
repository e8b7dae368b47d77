"""CPU: the uniform numbers behind temperature sampling."""

from cie_amd.sampling import Sampler, uniform_for


def test_uniform_numbers_are_reproducible_and_spread():
    values = [uniform_for(1, 2, i) for i in range(2000)]
    assert values == [uniform_for(1, 2, i) for i in range(2000)]
    assert all(0.0 <= v < 1.0 for v in values)
    assert abs(sum(values) / len(values) - 0.5) < 0.03
    assert len(set(values)) > 1990
    assert uniform_for(1, 2, 0) != uniform_for(1, 3, 0) != uniform_for(2, 2, 0)
    assert all(v * (1 << 24) == int(v * (1 << 24)) for v in values[:50]), "24 bits: exact in float32"


def test_request_seed_overrides_the_engine_stream():
    sampler = Sampler(seed=9)
    assert sampler.uniform(None, 4, 0) == uniform_for(9, 4, 0)
    assert sampler.uniform(123, 4, 7) == sampler.uniform(123, 99, 7) == uniform_for(123, 0, 7)
