"""The reference's default activation contract through the provider: an
artifact that does not declare dense_activation_input_bf16 gets per-row Q8
activations into every projection and the integer statement of the linears
(prepare_dense_activation / project_quantized,
runtime/tools/dense_fp4_provider.cpp:5983-6003, 6229-6267), intermediate
activations in F32.  Held to the composed oracle in the same contract
(qo_quantize_q8_rows + qo_fp4_linear_block32_q8), to the proposer's oracle, and
driven through the artifact reader and the worker."""
import numpy as np
import pytest

import artifact_writer as aw
import oracle_lib as ol
import qllm_provider as qp
import step_oracle
import worker_client as wc
from test_gpu_artifact_provider import geometry_of

pytestmark = pytest.mark.gpu


def q8_model(seed, output_gated=True, head_dim=128):
    rng = np.random.default_rng(seed)
    model = step_oracle.TinyModel(
        rng, 256, 512, 2, 8, 2, head_dim, 1024, ol.SCALE_UE8M0_BLOCK32,
        output_gated=output_gated, qk_norm=output_gated, zero_centered=output_gated,
        rotary_dim=64 if output_gated else None)
    model.activation_q8 = True
    return rng, model


@pytest.mark.parametrize("output_gated,head_dim", [(True, 256), (False, 128)])
def test_target_pass_in_the_q8_contract_matches_the_composed_oracle(device, output_gated,
                                                                    head_dim):
    rng, model = q8_model(7, output_gated, head_dim)
    provider = step_oracle.build_provider(model, qp)
    page_tokens = 64
    layer_bytes = ol.q4h_layer_bytes(page_tokens, model.kv_heads, model.head_dim)
    pages = [np.zeros(layer_bytes * model.layers, dtype=np.uint8) for _ in range(4)]
    position = 0
    for _ in range(3):
        tokens = rng.integers(0, model.vocabulary, 5).astype(np.uint32)
        provider.run_target(tokens, position)
        logits, hidden = provider.logits(5), provider.hidden(5)
        observed = [provider.kv_page(i) for i in range(4)]
        report = {}
        want_logits, want_hidden = step_oracle.run_target(
            model, tokens, position, pages, page_tokens, observed, report)
        assert report["record_byte_diffs"] <= 0.03 * report["record_bytes"]
        # Both sides compute the same arithmetic; they part where a last-bit
        # difference in an F32 activation moves a Q8 code by one step, 1 / 127
        # of the row's maximum - twice the step of a bf16 rounding, hence twice
        # the bf16 contract's end-to-end bound.  Per projection the gate is the
        # reference's own 2e-4 (test_gpu_gemm.py).
        relative = np.linalg.norm(logits - want_logits) / np.linalg.norm(want_logits)
        assert relative < 4e-2, relative
        assert np.abs(hidden - want_hidden).max() < 0.05 * np.abs(want_hidden).max()
        assert np.array_equal(logits.argmax(1), want_logits.argmax(1))
        position += 5
    assert provider.telemetry("provider_dense_activation_input_bf16") == 0
    provider.close()


def test_the_two_contracts_differ_and_each_follows_its_own_oracle(device):
    """The same weights under both contracts: Q8 noise is larger than the
    tolerance between them, which is why an artifact's contract has to be
    honoured rather than approximated."""
    rng, model = q8_model(19, False)
    tokens = rng.integers(0, model.vocabulary, 5).astype(np.uint32)
    outputs = {}
    for q8 in (True, False):
        model.activation_q8 = q8
        provider = step_oracle.build_provider(model, qp)
        provider.run_target(tokens, 0)
        outputs[q8] = provider.logits(5).copy()
        pages = [np.zeros(ol.q4h_layer_bytes(64, model.kv_heads, model.head_dim) *
                          model.layers, dtype=np.uint8) for _ in range(4)]
        want, _ = step_oracle.run_target(model, tokens, 0, pages, 64,
                                         [provider.kv_page(i) for i in range(4)], {})
        assert np.linalg.norm(outputs[q8] - want) / np.linalg.norm(want) < 2e-2
        provider.close()
    between = np.linalg.norm(outputs[True] - outputs[False]) / np.linalg.norm(outputs[False])
    assert 1e-3 < between < 0.1, between


def test_proposer_and_decode_cycle_in_the_q8_contract(device):
    """Captured passes equal uncaptured ones bit for bit, and the first
    proposer pass follows its oracle (Q8 linears over its Q8 cache)."""
    rng, model = q8_model(29)
    streams = []
    for eager in ("1", "0"):
        import os
        os.environ["QLLM_PROVIDER_EAGER"] = eager
        try:
            provider = step_oracle.build_provider(model, qp, mtp=True, draft_vocabulary=256)
        finally:
            del os.environ["QLLM_PROVIDER_EAGER"]
        provider.run_target(np.array([3, 5, 7, 11, 13], dtype=np.uint32), 0)
        provider.begin_request(temperature_ppm=0)
        token, position = 17, 5
        provider.synchronize(token, position)
        stream = [provider.drafts()]
        for _ in range(5):
            emitted, token, advanced = provider.verify(token, position, 200)
            position += advanced
            stream.append((emitted, token, provider.drafts()))
        streams.append(stream)
        provider.close()
    assert streams[0] == streams[1]


def test_an_artifact_without_the_bf16_declaration_runs_q8(device, tmp_path):
    rng, model = q8_model(37)
    root = str(tmp_path / "artifact")
    aw.write_artifact(root, model, draft_vocabulary=128, max_context=4096)   # no bf16 kernel
    loaded = qp.Provider.from_artifact(root, geometry_of(model, 256), max_context=256,
                                       kv_page_tokens=64)
    staged = step_oracle.build_provider(model, qp, mtp=True, draft_vocabulary=128)
    assert loaded.telemetry("provider_dense_activation_input_bf16") == 0
    tokens = rng.integers(0, model.vocabulary, 5).astype(np.uint32)
    results = []
    for provider in (loaded, staged):
        provider.run_target(tokens, 0)
        results.append((provider.logits(5).copy(), provider.hidden(5).copy()))
    assert np.array_equal(results[0][0], results[1][0])
    assert np.array_equal(results[0][1], results[1][1])
    # the same model with the declaration takes bf16 input and gives other logits
    declared = str(tmp_path / "declared")
    aw.write_artifact(declared, model, draft_vocabulary=128, max_context=4096,
                      activation_input="bf16")
    other = qp.Provider.from_artifact(declared, geometry_of(model, 256), max_context=256,
                                      kv_page_tokens=64)
    assert other.telemetry("provider_dense_activation_input_bf16") == 1
    other.run_target(tokens, 0)
    assert not np.array_equal(other.logits(5), results[0][0])
    # the worker serves the Q8 artifact: long prompts go through the program in
    # row batches (the tall prompt path takes bf16 input)
    worker = wc.Worker(root, max_context=256, kv_page_tokens=64)
    try:
        prompt = rng.integers(0, model.vocabulary, 12).astype(np.uint32)
        assert worker.begin(1, 200, prompt) == {"type": "begun", "id": 1}
        got = [worker.next(1, 0) for _ in range(4)]
        assert all(reply["type"] == "token" for reply in got), got
        # the provider, driven the same way
        loaded.begin_request_with(
            reserved_context_tokens=200, sampling_temperature_ppm=0,
            sampling_top_p_ppm=1000000, sampling_top_k=0, sampling_min_p_ppm=0,
            sampling_presence_penalty_biased_ppm=2000000,
            sampling_first_output_position=len(prompt) - 1, sampling_seed=0,
            exact_decode_enabled=1)
        token = None
        for first in range(0, len(prompt), 5):
            rows = prompt[first:first + 5]
            token = loaded.execute_program(rows, first)
            successors = list(prompt[first + 1:first + len(rows) + 1])
            last = first + len(rows) == len(prompt)
            if last:
                successors.append(token)
            loaded.synchronize_batch(successors[:len(rows)], first, last)
        position, expected = len(prompt), []
        for _ in range(4):
            emitted, token, advanced = loaded.verify(token, position, 200)
            position += advanced
            expected.append(emitted)
        assert [reply["tokens"] for reply in got] == expected
        assert worker.ask("END", 1) == {"type": "ended", "id": 1}
        assert worker.ask("SHUTDOWN") == {"type": "shutdown"}
    finally:
        worker.close()
    for provider in (loaded, staged, other):
        provider.close()
