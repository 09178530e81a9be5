"""The provider's own host sampling code (the functions the verify step calls
between the GPU passes) through the C ABI, on the CPU: bit-exact against the
vectors produced by the reference's C++ (tests/golden/sampling_golden.json),
against the reference's known answers, and against the oracle on fresh seeded
inputs.  No device is touched."""
import json
import os

import numpy as np
import pytest

import oracle_lib as ol
import qllm_provider as qp

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden",
                                     "sampling_golden.json")))
# the golden files record 0 = ok, 1 = std::invalid_argument, 2 = std::runtime_error
STATUS = {1: 4, 2: 10}


def fromhex(values):
    return [float.fromhex(v) for v in values]


def expect_failure(status, call):
    with pytest.raises(qp.ProviderError) as caught:
        call()
    assert caught.value.code == STATUS[status]
    assert str(caught.value).split(": ", 1)[1]      # the reference's text came along


def test_counter_uniform_matches_the_reference_vectors():
    for case in GOLDEN["counter_uniform"]:
        got = qp.counter_uniform(case["seed"], case["position"], case["stream"],
                                 case["index"])
        assert got == float.fromhex(case["value_hex"])
    assert qp.counter_uniform(1, 0, 100, 0) == 0.98957930235518243
    assert qp.counter_uniform(314159, 7, 300) == 0.8587919965661901


def test_make_sampling_distribution_matches_the_reference_vectors():
    for case in GOLDEN["make_sampling_distribution"]:
        call = lambda: qp.make_sampling_distribution(
            np.array(fromhex(case["logits_hex"]), dtype=np.float32),
            case["tokens"], case["temperature_ppm"], case["top_p_ppm"],
            case["min_p_ppm"])
        if case["status"]:
            expect_failure(case["status"], call)
            continue
        tokens, probabilities = call()
        assert tokens == case["out_tokens"]
        assert probabilities == fromhex(case["out_probabilities_hex"])


def test_nucleus_known_answer():
    # runtime/tests/cache_state_test.cpp:105-114
    tokens, probabilities = qp.make_sampling_distribution(
        [4.0, 3.0, 2.0, 1.0], [9, 5, 2, 1], 1000000, 800000, 0)
    assert tokens == [9, 5]
    assert abs(probabilities[0] - 0.7310585786300049) < 1e-12


def test_sample_distribution_matches_the_reference_vectors():
    for case in GOLDEN["sample_distribution"]:
        call = lambda: qp.sample_distribution(
            case["tokens"], fromhex(case["probabilities_hex"]),
            float.fromhex(case["uniform_hex"]))
        if case["status"]:
            expect_failure(case["status"], call)
        else:
            assert call() == case["token"]


def test_rejection_sample_matches_the_reference_vectors():
    for case in GOLDEN["rejection_sample"]:
        call = lambda: qp.rejection_sample(
            case["proposal"],
            (case["target_tokens"], fromhex(case["target_probabilities_hex"])),
            (case["draft_tokens"], fromhex(case["draft_probabilities_hex"])),
            float.fromhex(case["acceptance_uniform_hex"]),
            float.fromhex(case["correction_uniform_hex"]))
        if case["status"]:
            expect_failure(case["status"], call)
            continue
        accepted, token, p, q = call()
        assert accepted == case["accepted"] and token == case["token"]
        assert p == float.fromhex(case["target_probability_hex"])
        assert q == float.fromhex(case["draft_probability_hex"])


def test_error_behaviour():
    expect_failure(1, lambda: qp.sample_distribution([1, 1], [0.5, 0.5], 0.1))
    expect_failure(1, lambda: qp.sample_distribution([1, 2], [0.5, 0.4], 0.1))
    expect_failure(1, lambda: qp.sample_distribution([1], [1.0], 1.0))
    expect_failure(1, lambda: qp.sample_distribution([], [], 0.5))
    expect_failure(1, lambda: qp.rejection_sample(
        4, ([4], [1.0]), ([5], [1.0]), 0.5, 0.5))
    expect_failure(1, lambda: qp.make_sampling_distribution(
        [1.0, 2.0], [3, 4], 1000000, 1000000, 0))          # not descending
    expect_failure(1, lambda: qp.make_sampling_distribution(
        [1.0], [3], 0, 1000000, 0))                         # temperature 0


def test_host_code_equals_the_oracle_on_fresh_inputs():
    rng = np.random.default_rng(2024)
    for trial in range(200):
        n = int(rng.integers(1, 40))
        logits = np.sort(rng.normal(0, 3, n).astype(np.float32))[::-1].copy()
        tokens = rng.permutation(1000)[:n].astype(np.uint32)
        # equal logits must come with ascending ids
        for i in range(1, n):
            if logits[i] == logits[i - 1] and tokens[i] < tokens[i - 1]:
                tokens[i - 1], tokens[i] = tokens[i], tokens[i - 1]
        temperature = int(rng.integers(1, 2000001))
        top_p = int(rng.integers(1, 1000001))
        min_p = int(rng.integers(0, 500001))
        status, want_tokens, want_probabilities = ol.make_sampling_distribution(
            logits, tokens, temperature, top_p, min_p)
        assert status == 0
        got = qp.make_sampling_distribution(logits, tokens, temperature, top_p, min_p)
        assert got == (want_tokens, want_probabilities)

        m = int(rng.integers(1, 12))
        support = rng.permutation(16)[:m].astype(np.uint32)
        q = rng.dirichlet(np.ones(m))
        draft = (support.tolist(), (q / q.sum()).tolist())
        m2 = int(rng.integers(1, 12))
        support2 = rng.permutation(16)[:m2].astype(np.uint32)
        p = rng.dirichlet(np.ones(m2))
        target = (support2.tolist(), (p / p.sum()).tolist())
        proposal = int(support[rng.integers(0, m)])
        u1, u2 = float(rng.random()), float(rng.random())
        want = ol.rejection_sample(proposal, target, draft, u1, u2)
        if want[0] == 0:
            assert qp.rejection_sample(proposal, target, draft, u1, u2) == want[1:]
        else:
            expect_failure(want[0], lambda: qp.rejection_sample(
                proposal, target, draft, u1, u2))
