"""Host side of sampling (no GPU): the uniform generator and the host sampler
against the plain implementation."""

import math

import torch

import plain_llama as P
from kllm_amd.sampling import sample_host, uniform


def test_uniform_is_a_pure_function_in_the_unit_interval():
    us = [uniform(7, i) for i in range(2000)]
    assert us == [uniform(7, i) for i in range(2000)]
    assert all(0.0 <= u < 1.0 for u in us)
    assert all(float(torch.tensor(u, dtype=torch.float32)) == u for u in us[:100])   # exact in float32
    assert abs(sum(us) / len(us) - 0.5) < 0.03
    assert len(set(us)) > 1990
    assert [uniform(8, i) for i in range(5)] != us[:5]
    hist = [0] * 10
    for u in us:
        hist[int(u * 10)] += 1
    assert min(hist) > 140 and max(hist) < 260


def test_host_sampler_matches_the_plain_one():
    g = torch.Generator().manual_seed(0)
    logits = torch.randn(40, 97, generator=g) * 3
    for t in (0.0, 0.3, 1.0, 2.5):
        us = [uniform(3, i) for i in range(40)]
        got = sample_host(logits.tolist(), [t] * 40, us)
        want = [P.sample_inverse_cdf(logits[i], t, us[i]) for i in range(40)]
        assert got == want
    ties = [[1.0, 4.0, 4.0, 0.0]]
    assert sample_host(ties, [0.0], [0.5]) == [1]            # first maximum


def test_frequencies_follow_softmax():
    row = [0.0, math.log(2.0), math.log(5.0), -30.0]
    n = 8000
    counts = [0] * 4
    for i in range(n):
        counts[sample_host([row], [1.0], [uniform(1, i)])[0]] += 1
    want = [1 / 8, 2 / 8, 5 / 8]
    chi2 = sum((counts[k] - n * want[k]) ** 2 / (n * want[k]) for k in range(3))
    assert chi2 < 13.8 and counts[3] == 0                    # p = 0.001 at 2 degrees of freedom
