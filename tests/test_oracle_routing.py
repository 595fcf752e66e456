"""Pins the oracle's router, mixture and scalar operators against the reference's own known-answer
tests (native/tests/test_routing.cpp, native/tests/test_operators.cpp) and an independent
probability-sort specification."""
import math

import numpy as np
import pytest


def std_mt19937(seed):
    """numpy's MT19937 core with the C++ std::mt19937(seed) initialisation, so random_raw() yields the
    same 32-bit stream the reference's test draws from."""
    key = np.empty(624, dtype=np.uint32)
    x = seed & 0xFFFFFFFF
    key[0] = x
    for i in range(1, 624):
        x = (1812433253 * (x ^ (x >> 30)) + i) & 0xFFFFFFFF
        key[i] = x
    bg = np.random.MT19937()
    bg.state = {"bit_generator": "MT19937", "state": {"key": key, "pos": 624}}
    return bg


def test_std_mt19937_known_answer():
    # The C++ standard fixes the 10000th output of a default-seeded mt19937.
    bg = std_mt19937(5489)
    assert int(bg.random_raw(10000)[-1]) == 4123659995


def test_router_vs_probability_ordering(cpu):
    # native/tests/test_routing.cpp:24-48, seed 0x726f7574, 1000 trials, both modes, both normalisations.
    bg = std_mt19937(0x726F7574)
    for _ in range(1000):
        count = 1 + int(bg.random_raw()) % 1024
        selected = 1 + int(bg.random_raw()) % min(64, count)
        logits = (bg.random_raw(count).astype(np.int64) % 2001 - 1000) / 100.0
        for mode in (0, 1):
            p = np.exp(logits) if mode == 0 else 1 / (1 + np.exp(-logits))
            if mode == 0:
                total = 0.0
                for v in p:  # the reference sums sequentially
                    total += v
                p = p / total
            order = np.argsort(-p, kind="stable")[:selected]
            for normalize in (False, True):
                ids, w = cpu.route_reference(logits, selected, mode, normalize)
                assert np.array_equal(ids, order.astype(np.uint32))
                denom = p[order].sum() if normalize else 1.0
                assert np.abs(w - p[order] / denom).max() < 1e-13


def test_router_goldens(cpu):
    # native/tests/test_routing.cpp:49-64
    from oracle.oracle import FormatError
    ties = [3, 3, 2, 1, 3]
    ids, _ = cpu.route_reference(ties, 3, 0, True)
    assert list(ids) == [0, 1, 4]
    mix = cpu.mixture_reference([1, 2, 3, 4], [0.25, 0.75], [5, 6], 0)
    assert list(mix) == [5, 6.5]
    for bad in (lambda: cpu.route_reference(ties, 0, 0, True), lambda: cpu.route_reference(ties, 6, 0, True),
                lambda: cpu.route_reference([], 1, 0, True), lambda: cpu.route_reference(ties, 1, 99, True),
                lambda: cpu.route_reference([math.nan], 1, 0, True),
                lambda: cpu.mixture_reference([1, 2, 3, 4], [0.25, 0.75], [], 0),
                lambda: cpu.mixture_reference([1, 2, 3, 4], [math.nan], [5, 6], 0)):
        with pytest.raises(FormatError):
            bad()
    assert list(cpu.route_reference([-1000], 1, 1, True)[1]) == [1]
    ids, w = cpu.route_reference([-1000], 1, 0, True)
    assert list(ids) == [0] and list(w) == [1]


def test_all_zero_logits_pick_lowest_ids(cpu):
    # native/tests/test_moe_mm_many_gpu.cpp:252-253
    ids, w = cpu.route_reference(np.zeros(512), 10, 0, True)
    assert list(ids) == list(range(10))
    assert np.allclose(w, 0.1, rtol=0, atol=1e-16)


def test_scalar_operators(cpu):
    # native/tests/test_operators.cpp:27-34: closed-form points.
    assert cpu.stable_sigmoid(0) == 0.5
    assert abs(cpu.stable_sigmoid(2) - 1 / (1 + math.exp(-2))) < 1e-16
    assert abs(cpu.stable_sigmoid(-2) - math.exp(-2) / (1 + math.exp(-2))) < 1e-16
    assert cpu.stable_sigmoid(-1000) == 0 and cpu.stable_sigmoid(1000) == 1
    assert cpu.stable_silu(0) == 0
    assert abs(cpu.stable_silu(3) - 3 / (1 + math.exp(-3))) < 1e-15
    assert abs(cpu.stable_softplus(0) - math.log(2)) < 1e-16
    assert cpu.stable_softplus(1000) == 1000 and cpu.stable_softplus(-1000) == 0
    for x in np.linspace(-30, 30, 61):
        assert abs(cpu.stable_sigmoid(x) + cpu.stable_sigmoid(-x) - 1) < 1e-15
        assert abs(cpu.stable_softplus(x) - cpu.stable_softplus(-x) - x) < 1e-12


def test_rms_and_residual_goldens(cpu):
    # native/tests/test_operators.cpp:35-59: the scalar gated-residual case worked by hand, and two RMS groups.
    a, b = 2 / math.sqrt(5.0), 6 / math.sqrt(10.0)
    projected = (0.25 * a - 0.5 * b) / 2
    hidden = projected / (1 + math.exp(-projected))
    expected = (a / (1 + math.exp(-0.3 * hidden)) + b / (1 + math.exp(0.7 * hidden))) / 2
    read, scales = cpu.gated_residual_reference([2, 3], [1, 2], [0.25, -0.5], [0.3, -0.7], [0.1, 0.2, -0.5, 0.7], 2, 1, 1, 1.0)
    assert abs(read[0] - expected) < 1e-15
    assert abs(scales[0] - 2 / (1 + math.exp(-(0.1 * a + 0.2 * b) / 2))) < 1e-15
    assert abs(scales[1] - 2 / (1 + math.exp(-(-0.5 * a + 0.7 * b) / 2))) < 1e-15
    written = cpu.residual_write_reference([2, 3], read, scales)
    assert abs(written[0] - (2 + read[0] * scales[0])) < 1e-15 and abs(written[1] - (3 + read[0] * scales[1])) < 1e-15
    normalized = cpu.group_rms_reference([3, 4, 0, 2], [1, 1, 1, 1], 2, 0.5)
    assert abs(normalized[0] - 3 / math.sqrt(13.0)) < 1e-15 and abs(normalized[3] - 2 / math.sqrt(2.5)) < 1e-15
    from oracle.oracle import FormatError
    for bad in (lambda: cpu.group_rms_reference([3, 4, 0, 2], [1, 1, 1, 1], 3, 1e-6), lambda: cpu.group_rms_reference([3, 4, 0, 2], [1, 1, 1, 1], 2, 0.0)):
        with pytest.raises(FormatError):
            bad()
    # against plain numpy on a wider case: three branches, rank 4
    rng = np.random.default_rng(5)
    branches, channels, rank = 3, 17, 4
    width = branches * channels
    streams, gains = rng.normal(size=width), 1 + 0.1 * rng.normal(size=width)
    down, up, inject = 0.1 * rng.normal(size=(rank, width)), 0.1 * rng.normal(size=(width, rank)), 0.1 * rng.normal(size=(branches, width))
    n = (streams.reshape(branches, channels) / np.sqrt((streams.reshape(branches, channels) ** 2).mean(axis=1, keepdims=True) + 1e-6)).reshape(-1) * gains
    assert np.allclose(cpu.group_rms_reference(streams, gains, channels, 1e-6), n, rtol=1e-14)
    z = down @ n / branches
    bottleneck = z / (1 + np.exp(-z))
    scores = 1 / (1 + np.exp(-(up @ bottleneck)))
    read, scales = cpu.gated_residual_reference(streams, gains, down, up, inject, branches, channels, rank, 1e-6)
    assert np.allclose(read, (n * scores).reshape(branches, channels).mean(axis=0), rtol=1e-13)
    assert np.allclose(scales, 2 / (1 + np.exp(-(inject @ n) / branches)), rtol=1e-13)


def test_oracle_equals_reference_routing(orc, ref):
    rng = np.random.default_rng(3)
    for _ in range(200):
        n = int(rng.integers(1, 600))
        k = int(rng.integers(1, min(64, n) + 1))
        logits = np.round(rng.normal(size=n) * 4, 1)  # coarse grid: plenty of exact ties
        for mode in (0, 1):
            for normalize in (False, True):
                a, b = orc.route_reference(logits, k, mode, normalize), ref.route_reference(logits, k, mode, normalize)
                assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
        experts = rng.normal(size=(k, 7))
        w = np.abs(rng.normal(size=k))
        shared = rng.normal(size=7)
        assert np.array_equal(orc.mixture_reference(experts, w, shared, 0.3), ref.mixture_reference(experts, w, shared, 0.3))
