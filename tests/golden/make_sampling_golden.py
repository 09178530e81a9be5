"""Writes tests/golden/sampling_golden.json from the reference's own host
sampling code.

The expected values come from oracle/_ref/libqllm_ref.so, which `make -C oracle`
compiles from the reference source file runtime/src/speculative_sampling.cpp
where it lies in the reference tree (plus a C shim that adds no arithmetic).
Run in a container that has the reference tree; the JSON is committed so the
vectors travel to machines that do not."""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import oracle_lib as ol  # noqa: E402


def main():
    if ol.ref() is None:
        raise SystemExit("oracle/_ref/libqllm_ref.so is missing: run `make -C oracle`")
    rng = np.random.default_rng(20241125)
    golden = {"counter_uniform": [], "make_sampling_distribution": [],
              "sample_distribution": [], "rejection_sample": []}
    for seed, position, stream, index in [
            (1, 0, 100, 0), (1, 32768, 200, 3), (314159, 7, 300, 0),
            (0, 0, 0, 0), (2**64 - 1, 2**32 - 1, 300, 4), (19, 12345, 1, 0),
            (42, 131072, 100, 2), (7, 262143, 200, 1)]:
        value = ol.counter_uniform(seed, position, stream, index, lib="ref")
        golden["counter_uniform"].append(
            {"seed": seed, "position": position, "stream": stream,
             "index": index, "value_hex": float(value).hex()})

    def distribution_case(logits, tokens, t, p, m):
        status, out_tokens, out_probs = ol.make_sampling_distribution(
            logits, tokens, t, p, m, lib="ref")
        return {"logits_hex": [float(x).hex() for x in np.asarray(logits, np.float32)],
                "tokens": [int(x) for x in tokens], "temperature_ppm": t,
                "top_p_ppm": p, "min_p_ppm": m, "status": status,
                "out_tokens": out_tokens,
                "out_probabilities_hex": [float(x).hex() for x in out_probs]}

    golden["make_sampling_distribution"].append(
        distribution_case([4.0, 3.0, 2.0, 1.0], [9, 5, 2, 1], 1000000, 800000, 0))
    golden["make_sampling_distribution"].append(
        distribution_case([4.0, 3.0, 2.0, 1.0], [9, 5, 2, 1], 700000, 950000, 0))
    golden["make_sampling_distribution"].append(
        distribution_case([1.0, 2.0], [0, 1], 1000000, 1000000, 0))  # unordered
    golden["make_sampling_distribution"].append(
        distribution_case([2.0, 2.0], [5, 3], 1000000, 1000000, 0))  # tie order
    golden["make_sampling_distribution"].append(
        distribution_case([2.0, 2.0, float("nan")], [3, 5, 9], 500000, 999999, 100000))
    golden["make_sampling_distribution"].append(
        distribution_case([0.0], [7], 0, 1000000, 0))  # invalid temperature
    for _ in range(24):
        n = int(rng.integers(1, 65))
        logits = np.sort(rng.standard_normal(n).astype(np.float32) * 3.0)[::-1].copy()
        if n > 4 and rng.random() < 0.3:
            logits[2] = logits[1]  # a tie, ids ascending below
        tokens = np.sort(rng.choice(200000, n, replace=False)).astype(np.uint32)
        golden["make_sampling_distribution"].append(distribution_case(
            logits, tokens, int(rng.integers(1, 2000001)),
            int(rng.integers(1, 1000001)), int(rng.integers(0, 200001))))

    def random_distribution(n, universe):
        tokens = rng.choice(universe, n, replace=False).astype(np.uint32)
        p = rng.dirichlet(np.full(n, 0.5))
        p = p / p.sum()
        return [int(t) for t in tokens], [float(x) for x in p]

    for _ in range(16):
        tokens, probs = random_distribution(int(rng.integers(1, 12)), 50)
        u = float(rng.random())
        status, token = ol.sample_distribution(tokens, probs, u, lib="ref")
        golden["sample_distribution"].append(
            {"tokens": tokens, "probabilities_hex": [x.hex() for x in probs],
             "uniform_hex": u.hex(), "status": status, "token": token})

    fixed_target = ([3, 7, 11], [0.50, 0.30, 0.20])
    fixed_draft = ([3, 7, 13], [0.20, 0.70, 0.10])
    cases = []
    for proposal in (3, 7, 13):
        for _ in range(8):
            cases.append((proposal, fixed_target, fixed_draft,
                          float(rng.random()), float(rng.random())))
    for _ in range(40):
        target = random_distribution(int(rng.integers(1, 10)), 24)
        draft = random_distribution(int(rng.integers(1, 10)), 24)
        proposal = int(rng.choice(draft[0])) if rng.random() < 0.9 else 25
        cases.append((proposal, target, draft, float(rng.random()),
                      float(rng.random())))
    for proposal, target, draft, ua, uc in cases:
        status, accepted, token, p, q = ol.rejection_sample(
            proposal, target, draft, ua, uc, lib="ref")
        golden["rejection_sample"].append(
            {"proposal": proposal, "target_tokens": target[0],
             "target_probabilities_hex": [float(x).hex() for x in target[1]],
             "draft_tokens": draft[0],
             "draft_probabilities_hex": [float(x).hex() for x in draft[1]],
             "acceptance_uniform_hex": ua.hex(), "correction_uniform_hex": uc.hex(),
             "status": status, "accepted": accepted, "token": token,
             "target_probability_hex": float(p).hex(),
             "draft_probability_hex": float(q).hex()})
    with open(os.path.join(HERE, "sampling_golden.json"), "w") as handle:
        json.dump(golden, handle, indent=1)
    print({k: len(v) for k, v in golden.items()})


if __name__ == "__main__":
    main()
