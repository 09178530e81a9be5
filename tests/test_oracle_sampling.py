"""Pins the oracle's sampling mathematics (qo_make_sampling_distribution,
qo_sample_distribution, qo_rejection_sample, qo_counter_uniform) against
vectors produced by the reference's own C++ (tests/golden/sampling_golden.json,
see make_sampling_golden.py), against the reference's known answers, and -
where oracle/_ref was built - against the reference library on fresh inputs."""
import json
import os

import numpy as np
import pytest

import oracle_lib as ol

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden",
                                     "sampling_golden.json")))


def fromhex(values):
    return [float.fromhex(v) for v in values]


def test_counter_uniform_golden():
    for case in GOLDEN["counter_uniform"]:
        got = ol.counter_uniform(case["seed"], case["position"], case["stream"],
                                 case["index"])
        assert got == float.fromhex(case["value_hex"])


def test_counter_uniform_known_answers():
    # values recorded from the reference source (integer splitmix64, exact)
    assert ol.counter_uniform(1, 0, 100, 0) == 0.98957930235518243
    assert ol.counter_uniform(1, 32768, 200, 3) == 0.1518630800940044
    assert ol.counter_uniform(314159, 7, 300, 0) == 0.8587919965661901


def test_make_sampling_distribution_golden():
    for case in GOLDEN["make_sampling_distribution"]:
        status, tokens, probs = ol.make_sampling_distribution(
            np.array(fromhex(case["logits_hex"]), dtype=np.float32),
            case["tokens"], case["temperature_ppm"], case["top_p_ppm"],
            case["min_p_ppm"])
        assert status == case["status"]
        assert tokens == case["out_tokens"]
        assert probs == fromhex(case["out_probabilities_hex"])  # bit-exact


def test_nucleus_known_answer():
    # runtime/tests/cache_state_test.cpp:105-114
    status, tokens, probs = ol.make_sampling_distribution(
        [4.0, 3.0, 2.0, 1.0], [9, 5, 2, 1], 1000000, 800000, 0)
    assert status == 0 and tokens == [9, 5]
    assert abs(probs[0] - 0.7310585786300049) < 1e-12


def test_sample_distribution_golden():
    for case in GOLDEN["sample_distribution"]:
        status, token = ol.sample_distribution(
            case["tokens"], fromhex(case["probabilities_hex"]),
            float.fromhex(case["uniform_hex"]))
        assert status == case["status"]
        if status == 0:
            assert token == case["token"]


def test_rejection_sample_golden():
    for case in GOLDEN["rejection_sample"]:
        status, accepted, token, p, q = ol.rejection_sample(
            case["proposal"],
            (case["target_tokens"], fromhex(case["target_probabilities_hex"])),
            (case["draft_tokens"], fromhex(case["draft_probabilities_hex"])),
            float.fromhex(case["acceptance_uniform_hex"]),
            float.fromhex(case["correction_uniform_hex"]))
        assert status == case["status"]
        if status == 0:
            assert accepted == case["accepted"] and token == case["token"]
            assert p == float.fromhex(case["target_probability_hex"])
            assert q == float.fromhex(case["draft_probability_hex"])


def test_rejection_sampling_output_law():
    """runtime/tests/cache_state_test.cpp:57-103: accepted mass is min(p,q), the
    rejected mass is redistributed over normalised max(p-q,0)."""
    target = ([3, 7, 11], [0.50, 0.30, 0.20])
    draft = ([3, 7, 13], [0.20, 0.70, 0.10])
    tokens = [3, 7, 11, 13]
    p = dict(zip(*target))
    q = dict(zip(*draft))
    expected = np.array([min(p.get(t, 0.0), q.get(t, 0.0)) for t in tokens])
    rejection = sum(q.get(t, 0.0) - min(p.get(t, 0.0), q.get(t, 0.0)) for t in tokens)
    residual = np.array([max(0.0, p.get(t, 0.0) - q.get(t, 0.0)) for t in tokens])
    assert abs(rejection - residual.sum()) < 1e-12
    expected = expected + rejection * residual / residual.sum()
    trials = 60000
    observed = np.zeros(4)
    for trial in range(trials):
        _, proposal = ol.sample_distribution(*draft, ol.counter_uniform(19, trial, 1))
        status, _, token, _, _ = ol.rejection_sample(
            proposal, target, draft, ol.counter_uniform(19, trial, 2),
            ol.counter_uniform(19, trial, 3))
        assert status == 0
        observed[tokens.index(token)] += 1
    assert np.abs(observed / trials - expected).max() < 0.008


def test_greedy_is_token_equality():
    """One-hot distributions reduce rejection sampling to draft == argmax."""
    for draft_token, target_token in [(5, 5), (5, 9)]:
        status, accepted, token, _, _ = ol.rejection_sample(
            draft_token, ([target_token], [1.0]), ([draft_token], [1.0]), 0.3, 0.7)
        assert status == 0
        assert accepted == (draft_token == target_token)
        assert token == target_token


def test_error_behaviour():
    assert ol.sample_distribution([1, 1], [0.5, 0.5], 0.1)[0] == 1   # duplicate
    assert ol.sample_distribution([1, 2], [0.5, 0.4], 0.1)[0] == 1   # not normalised
    assert ol.sample_distribution([1], [1.0], 1.0)[0] == 1           # uniform == 1
    # proposal without draft mass -> invalid_argument
    assert ol.rejection_sample(4, ([4], [1.0]), ([5], [1.0]), 0.5, 0.5)[0] == 1
    # identical one-hot distributions, forced rejection impossible (u < 1 = a)
    assert ol.rejection_sample(4, ([4], [1.0]), ([4], [1.0]), 0.999, 0.5)[1] is True


@pytest.mark.skipif(ol.ref() is None, reason="oracle/_ref was not built")
def test_against_reference_library_on_fresh_inputs():
    rng = np.random.default_rng(5)
    for _ in range(200):
        n = int(rng.integers(1, 40))
        logits = np.sort(rng.standard_normal(n).astype(np.float32) * 4)[::-1].copy()
        tokens = np.sort(rng.choice(1000, n, replace=False)).astype(np.uint32)
        args = (logits, tokens, int(rng.integers(1, 2000001)),
                int(rng.integers(1, 1000001)), int(rng.integers(0, 100001)))
        assert ol.make_sampling_distribution(*args) == \
            ol.make_sampling_distribution(*args, lib="ref")
    for _ in range(300):
        def dist(n):
            t = rng.choice(30, n, replace=False)
            p = rng.dirichlet(np.full(n, 0.3))
            p = p / p.sum()
            return [int(x) for x in t], [float(x) for x in p]
        target, draft = dist(int(rng.integers(1, 12))), dist(int(rng.integers(1, 12)))
        proposal = int(rng.choice(draft[0]))
        ua, uc = float(rng.random()), float(rng.random())
        assert ol.rejection_sample(proposal, target, draft, ua, uc) == \
            ol.rejection_sample(proposal, target, draft, ua, uc, lib="ref")
    for _ in range(100):
        a = [int(x) for x in rng.integers(0, 2**32, 3)]
        seed = int(rng.integers(0, 2**63))
        assert ol.counter_uniform(seed, *a) == ol.counter_uniform(seed, *a, lib="ref")


def test_acceptance_loop_uniform_streams():
    """Streams 100/200 (index = depth) and 300, positions position+depth
    (runtime/tools/dense_fp4_provider.cpp:11209-11234), replayed by hand."""
    rng = np.random.default_rng(11)
    vocabulary = 40
    for trial in range(50):
        n = 4
        drafts, draft_dists, targets = [], [], []
        for _ in range(n):
            q = rng.dirichlet(np.full(vocabulary, 0.3)); q = q / q.sum()
            drafts.append(int(rng.choice(vocabulary, p=q)))
            draft_dists.append((list(range(vocabulary)), [float(x) for x in q]))
        for _ in range(n + 1):
            p = rng.dirichlet(np.full(vocabulary, 0.3)); p = p / p.sum()
            targets.append((list(range(vocabulary)), [float(x) for x in p]))
        seed, position = 1000 + trial, 32768 + trial
        status, accepted, next_token = ol.accept_stochastic(
            targets, draft_dists, drafts, seed, position)
        assert status == 0
        expect_accepted, expect_next = n, None
        for depth in range(n):
            s, ok, token, _, _ = ol.rejection_sample(
                drafts[depth], targets[depth], draft_dists[depth],
                ol.counter_uniform(seed, position + depth, 100, depth),
                ol.counter_uniform(seed, position + depth, 200, depth))
            if not ok:
                expect_accepted, expect_next = depth, token
                break
        if expect_next is None:
            _, expect_next = ol.sample_distribution(
                *targets[n], ol.counter_uniform(seed, position + n, 300, 0))
        assert (accepted, next_token) == (expect_accepted, expect_next)
