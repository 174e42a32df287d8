"""The host twin of the selection kernel against the plain implementation (no GPU)."""
import numpy as np
import pytest

import plain_llama as P
from gpullama3_java_amd.sampling import SamplingParams, sample_host, select_sampler, uniform


def test_uniform_is_a_function_of_its_counters():
    u = [uniform(3, r, s) for r in range(20) for s in range(50)]
    assert all(0 <= x < 1 for x in u) and len(set(u)) > 990
    assert uniform(3, 4, 5) == uniform(3, 4, 5) != uniform(4, 4, 5)
    assert all(np.float32(x) == x for x in u)                   # exact in float32
    assert abs(np.mean(u) - 0.5) < 0.03


@pytest.mark.parametrize("temperature, top_p", [(0.0, 0.95), (0.8, 0.95), (1.0, 1.0), (1.3, 0.0), (0.5, 0.3), (1.0, 1e-6)])
def test_twin_agrees_with_the_plain_rule(temperature, top_p):
    rng = np.random.default_rng(0)
    for n in (2, 17, 300):
        for _ in range(40):
            logits = (rng.standard_normal(n) * rng.uniform(0.5, 4)).astype(np.float32)
            u = float(np.float32(rng.random()))
            assert sample_host(logits, temperature, top_p, u) == P.sample(logits, temperature, top_p, u)


def test_ties_and_edges():
    assert sample_host(np.array([1, 3, 3, 2], np.float32), 0, 1, 0.5) == 1
    flat = np.zeros(8, np.float32)
    assert [sample_host(flat, 1.0, 1.0, u) for u in (0.0, 0.13, 0.99)] == [0, 1, 7]
    # equal probabilities under top-p: lower indices are kept first
    assert [sample_host(flat, 1.0, 0.3, u) for u in (0.0, 0.4, 0.99)] == [0, 1, 2]


def test_validation_as_the_reference_options():
    with pytest.raises(ValueError):
        SamplingParams(-0.1, 0.5)
    with pytest.raises(ValueError):
        SamplingParams(0.5, 1.5)
    assert select_sampler(100, 0.7, 0.9, 42) == SamplingParams(0.7, 0.9, 42)
