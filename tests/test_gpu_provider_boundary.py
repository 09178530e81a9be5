"""The provider behind the common VM's interface on the GPU: the program run
operation by operation through IOperationProvider::execute, and the whole
decode driven by the reference's own VM - its registry, its program executor
with sessions and exact-decode result validation, compiled from the reference's
sources with this provider linked in (oracle/_ref/libqllm_ref_vm.so) - against
the same provider driven directly."""
import numpy as np
import pytest

import artifact_writer as aw
import oracle_lib as ol
import qllm_provider as qp
import reference_vm
import step_oracle
from test_gpu_artifact_provider import geometry_of, tiny_model

pytestmark = pytest.mark.gpu
# (the library itself is loaded inside the test, after the device fixture)
needs_vm = pytest.mark.skipif(not reference_vm.built(),
                              reason="oracle/_ref/libqllm_ref_vm.so is not built")


def request(temperature_ppm=0, top_k=0, seed=5, penalty_ppm=0, exact=1, reserved=200):
    return dict(reserved_context_tokens=reserved, sampling_temperature_ppm=temperature_ppm,
                sampling_top_p_ppm=950000, sampling_top_k=top_k, sampling_min_p_ppm=0,
                sampling_presence_penalty_biased_ppm=2000000 + penalty_ppm,
                sampling_first_output_position=0, sampling_seed=seed,
                exact_decode_enabled=exact)


def test_program_executed_operation_by_operation(device, monkeypatch):
    """execute() on embedding, attention, FFN and head in program order gives
    the logits of the target pass launched as a whole (with the residual adds
    in the projections' epilogues on both sides, the kernels are the same)."""
    monkeypatch.setenv("QLLM_PROVIDER_K_SPLITS", "0")
    rng, model = tiny_model(71)
    stepwise = step_oracle.build_provider(model, qp, mtp=True, draft_vocabulary=128)
    whole = step_oracle.build_provider(model, qp, mtp=True, draft_vocabulary=128)
    stepwise.begin_request_with(**request(exact=0))
    position = 0
    for rows in (5, 1, 3):
        tokens = rng.integers(0, model.vocabulary, rows).astype(np.uint32)
        selected = stepwise.execute_program(tokens, position)
        whole.run_target(tokens, position)
        want = whole.logits(rows)
        # the head of a batch scores its last row only (row 0 of the logits)
        assert np.array_equal(stepwise.logits(1)[0], want[rows - 1])
        assert selected == ol.argmax(want[rows - 1])
        assert np.array_equal(stepwise.hidden(rows), whole.hidden(rows))
        for page in range(2):
            assert np.array_equal(stepwise.kv_page(page), whole.kv_page(page))
        position += rows
    # ports are checked: a batch that changes width between operations, a
    # token outside the vocabulary
    with pytest.raises(qp.ProviderError):
        stepwise.execute_program(np.array([model.vocabulary], dtype=np.uint32), position)
    stepwise.close()
    whole.close()


def test_head_sampling_and_presence_through_execute(device):
    """The head under a sampled request: top-k candidates, stream-0 uniform at
    the row's position, the emitted token marked and penalised afterwards
    (run_head with a request, dense_fp4_provider.cpp:8433-8517)."""
    rng, model = tiny_model(73)
    provider = step_oracle.build_provider(model, qp, mtp=True, draft_vocabulary=128)
    raw = step_oracle.build_provider(model, qp, mtp=True, draft_vocabulary=128)
    V, seed, penalty = model.vocabulary, 99, np.float32(1.25)
    provider.begin_request_with(**request(800000, 20, seed, 1250000, exact=0))
    emitted = np.zeros(V, dtype=np.uint8)
    position, token = 0, 3
    for step in range(6):
        selected = provider.execute_program(np.array([token], dtype=np.uint32), position)
        raw.run_target(np.array([token], dtype=np.uint32), position)
        logits = ol.presence_penalty(raw.logits(1)[0], emitted, penalty)
        values, indices = ol.topk(logits, 20)
        status, tokens, probabilities = ol.make_sampling_distribution(
            values, indices, 800000, 950000, 0)
        assert status == 0
        want = qp.sample_distribution(tokens, probabilities,
                                      qp.counter_uniform(seed, position, 0, 0))
        assert selected == want, step
        emitted[selected] = 1
        token, position = selected, position + 1
    provider.close()
    raw.close()


@needs_vm
@pytest.mark.parametrize("temperature_ppm,top_k,penalty_ppm", [(0, 0, 0), (900000, 20, 0),
                                                               (0, 0, 1500000)])
def test_reference_vm_drives_the_provider(device, tmp_path, temperature_ppm, top_k,
                                          penalty_ppm):
    """Prompt in execute() batches, synchronisation, then exact-decode steps,
    all through the reference's executor and session objects; the tokens must
    be those of the provider driven through its own C ABI, and every result has
    passed the executor's validation (emitted[0] == guaranteed token,
    positions_advanced == emitted.size(), tokens inside the vocabulary)."""
    rng, model = tiny_model(67)
    root = str(tmp_path / "artifact")
    aw.write_artifact(root, model, draft_vocabulary=128, max_context=4096)
    vm = reference_vm.Machine(root, 256, 64, vocabulary=model.vocabulary)
    service = vm.service()
    assert service == dict(kv_dtype="q4-f16-per-head", kv_page_tokens=64,
                           prefill_chunk_tokens=5, mtp_enabled=True, sampling_supported=True)
    direct = qp.Provider.from_artifact(root, geometry_of(model, 256), max_context=256,
                                       kv_page_tokens=64)
    parameters = request(temperature_ppm, top_k, 31, penalty_ppm)
    vm.begin_session(**parameters)
    direct.begin_request_with(**parameters)
    assert vm.exact_available()

    prompt = rng.integers(0, model.vocabulary, 13).astype(np.uint32)
    position = 0
    streams = {"vm": [], "direct": []}
    for name, machine in (("vm", vm), ("direct", direct)):
        position, following = 0, None
        while position < len(prompt):
            chunk = prompt[position:position + 5]
            execute = machine.execute if name == "vm" else machine.execute_program
            following = execute(chunk, position)
            # the proposer learns the successor of every row of the batch; the
            # last batch ends with the token the head selected and rolls the
            # first drafts out (the runner's feed, moe_vm_runner.cpp:682-745)
            last = position + len(chunk) == len(prompt)
            successors = [*prompt[position + 1:position + len(chunk)],
                          following if last else prompt[position + len(chunk)]]
            synchronize = machine.synchronize if name == "vm" else machine.synchronize_batch
            synchronize(np.array(successors, dtype=np.uint32), position, last)
            position += len(chunk)
        token = following
        for step in range(6):
            decode = machine.exact_decode if name == "vm" else machine.verify
            emitted, following, advanced = decode(token, position, 200)
            assert emitted[0] == token and advanced == len(emitted)
            streams[name].append((emitted, following))
            token, position = following, position + advanced
    assert streams["vm"] == streams["direct"]
    assert vm.telemetry("provider_exact_calls") == 6
    # a stream the provider cannot continue is turned down through the VM too
    with pytest.raises(reference_vm.VmError):
        vm.exact_decode(token + 1 if token + 1 < model.vocabulary else 0, position, 200)
    vm.close()
    direct.close()
