"""Request slots, the scripted lines of the reference's service tests and GPU
phase timing, through the worker process and through the reference's own VM:
two interleaved requests must give the tokens each gives alone
(dense_fp4_provider.cpp:6554-6588 - one page-table row, one set of presence
bytes and one proposer state per slot; runtime/tools/moe_vm_runner.cpp:1076-
1100 - STEP batches), a request beyond the capacity is turned down, and the
ready line passes the service's own reading of it (worker_client.ServiceView,
pinned by tests/test_worker_protocol_fixture.py)."""
import json
import os

import numpy as np
import pytest

import artifact_writer as aw
import reference_vm
import worker_client as wc
from test_gpu_artifact_provider import tiny_model

pytestmark = pytest.mark.gpu

CONTEXT = 1024
LAUNCH = dict(max_context=CONTEXT, requested_capacity=2, ram_cache_gib=1, vram_cache_gib=1,
              kv_page_tokens=64, placement_profile="latency", mtp_draft_depth=4)
SAMPLED = (800000, 950000, 40, 0, 500000, 7)

with open(os.path.join(os.path.dirname(__file__), "golden", "worker_protocol.json"),
          encoding="utf-8") as source:
    PROTOCOL = json.load(source)


@pytest.fixture(scope="module")
def artifact(tmp_path_factory):
    rng, model = tiny_model(91)
    root = str(tmp_path_factory.mktemp("slots") / "artifact")
    aw.write_artifact(root, model, draft_vocabulary=128, max_context=4096)
    return rng, model, root


@pytest.fixture(scope="module")
def worker(artifact):
    _, _, root = artifact
    process = wc.Worker(root, max_context=CONTEXT, kv_page_tokens=64, capacity=2,
                        mtp_draft_depth=4)
    yield process
    process.close()


def conversation(worker, request, prompt, steps, sampling=None, close=True):
    assert worker.begin(request, 200, prompt, sampling) == {"type": "begun", "id": request}
    stream = [worker.next(request, 0)["tokens"] for _ in range(steps)]
    if close:
        stream.append(worker.next(request, 1)["tokens"])
    return stream


def test_ready_line_passes_the_service_client(worker):
    view = wc.ServiceView(worker.ready, LAUNCH)
    assert view.protocol == 13 and view.capacity == 2 and view.mtp_draft_depth == 4
    assert view.placement_mode == "resident" and view.kv_dtype == "q4-f16-per-head"
    assert not view.gpu_phase_timing and view.sampling_supported
    # the client refuses the same line for a launch it does not answer
    with pytest.raises(wc.ContractError):
        wc.ServiceView(worker.ready, {**LAUNCH, "requested_capacity": 1})
    with pytest.raises(wc.ContractError):
        wc.ServiceView(worker.ready, {**LAUNCH, "kv_page_tokens": 256})


def test_scripted_lines_of_the_service_tests(worker):
    """The literal command lines the reference's service tests expect on the
    wire, sent as they are: a worker without session retention answers each
    with the runner's error line and keeps its requests."""
    lines = {item["line"].split("\t")[0]: item["line"] for item in PROTOCOL["command_lines"]
             if not item["line"].startswith("\t")}
    retention = {"type": "error",
                 "message": "callable provider does not support session retention"}
    assert worker.ask(lines["BEGIN"]) == retention          # BEGIN 7 1024 <empty> RESUME 9 ..
    assert worker.ask(lines["END"]) == {"type": "error", "message": "unknown active request"}
    assert worker.begin(7, 200, [1, 2, 3])["type"] == "begun"
    assert worker.ask(lines["END"]) == retention            # END 7 RETAIN 9 AT 300
    assert worker.ask("STATS")["active_requests"] == 1      # still there
    assert worker.ask(lines["DROP"]) == retention
    # the sampling group exactly as the service serialises it
    sampling = next(item["line"] for item in PROTOCOL["command_lines"]
                    if item["line"].startswith("\tSAMPLING"))
    assert worker.ask("BEGIN\t8\t200\t4,5,6" + sampling) == {"type": "begun", "id": 8}
    assert worker.ask("END", 8) == {"type": "ended", "id": 8}
    assert worker.ask("END", 7) == {"type": "ended", "id": 7}


@pytest.mark.parametrize("sampling", [None, SAMPLED])
def test_interleaved_requests_equal_the_same_requests_alone(artifact, worker, sampling):
    rng, model, _ = artifact
    first = rng.integers(0, model.vocabulary, 9).astype(np.uint32)     # tall prefill
    second = rng.integers(0, model.vocabulary, 3).astype(np.uint32)    # program steps
    alone = [conversation(worker, 1, first, 6, sampling),
             conversation(worker, 2, second, 6, sampling)]
    assert worker.begin(1, 200, first, sampling)["type"] == "begun"
    assert worker.begin(2, 200, second, sampling)["type"] == "begun"
    assert worker.ask("BEGIN", 3, 200, "1,2")["message"] == \
        "callable provider capacity is exhausted"
    together = [[], []]
    for step in range(6):
        if step % 2:
            # one STEP line for both requests: one batch reply, in the line's order
            reply = worker.ask("STEP", "2,0", "1,0")
            assert reply["type"] == "batch" and [i["id"] for i in reply["items"]] == [2, 1]
            together[1].append(reply["items"][0]["tokens"])
            together[0].append(reply["items"][1]["tokens"])
        else:
            together[0].append(worker.next(1, 0)["tokens"])
            together[1].append(worker.next(2, 0)["tokens"])
    assert worker.ask("STEP", "1,0", "1,0")["message"] == "STEP request mismatch"
    assert worker.ask("STEP", "1,0", "2,0", "1,0")["message"] == "invalid STEP"
    stats = worker.ask("STATS")
    assert stats["active_requests"] == 2 and stats["kv_reserved_pages"] >= 2
    reply = worker.ask("STEP", "1,1", "2,1")
    together[0].append(reply["items"][0]["tokens"])
    together[1].append(reply["items"][1]["tokens"])
    assert together == alone
    assert worker.ask("STATS")["active_requests"] == 0


def test_reference_vm_interleaves_two_sessions(artifact):
    """The reference's own executor with two sessions open on this provider:
    each sees the tokens it sees alone, and a third is turned down with the
    reference's backpressure status."""
    if not reference_vm.built():
        pytest.skip("oracle/_ref/libqllm_ref_vm.so is not built")
    rng, model, root = artifact
    machine = reference_vm.Machine(root, CONTEXT, 64, mtp_draft_depth=4,
                                   vocabulary=model.vocabulary, capacity=2)
    parameters = dict(reserved_context_tokens=200, sampling_temperature_ppm=0,
                      sampling_top_p_ppm=1000000, sampling_top_k=0, sampling_min_p_ppm=0,
                      sampling_presence_penalty_biased_ppm=2000000, sampling_seed=0,
                      exact_decode_enabled=1)
    prompts = [rng.integers(0, model.vocabulary, 4).astype(np.uint32),
               rng.integers(0, model.vocabulary, 5).astype(np.uint32)]

    def begin(session):
        prompt = prompts[session]
        machine.select(session)
        machine.begin_session(sampling_first_output_position=len(prompt) - 1, **parameters)
        token = machine.execute(prompt, 0)
        machine.synchronize(list(prompt[1:]) + [token], 0, True)
        return token, len(prompt)

    def step(session, token, position):
        machine.select(session)
        emitted, token, advanced = machine.exact_decode(token, position, 200)
        return emitted, token, position + advanced

    try:
        alone = []
        for session in range(2):
            token, position = begin(session)
            stream = []
            for _ in range(5):
                emitted, token, position = step(session, token, position)
                stream.append(emitted)
            alone.append(stream)
            machine.end_session()
        state = [begin(0), begin(1)]
        machine.select(2)
        with pytest.raises(reference_vm.VmError, match="no free request slot"):
            machine.begin_session(sampling_first_output_position=0, **parameters)
        together = [[], []]
        for _ in range(5):
            for session in (1, 0):
                emitted, token, position = step(session, *state[session])
                state[session] = (token, position)
                together[session].append(emitted)
        assert together == alone
        # a slot comes back when its session ends
        machine.select(0)
        machine.end_session()
        machine.select(2)
        machine.begin_session(sampling_first_output_position=0, **parameters)
    finally:
        machine.close()


def test_gpu_phase_timing_is_opt_in_and_changes_no_token(artifact, worker):
    rng, model, root = artifact
    prompt = rng.integers(0, model.vocabulary, 7).astype(np.uint32)
    plain = conversation(worker, 5, prompt, 4)
    assert not any(name.startswith("provider_gpu_") for name in worker.ask("STATS"))
    timed = wc.Worker(root, max_context=CONTEXT, kv_page_tokens=64, capacity=1,
                      mtp_draft_depth=4, profile_gpu_phases=True)
    try:
        assert timed.ready["gpu_phase_timing"] is True
        assert conversation(timed, 5, prompt, 4) == plain
        stats = timed.ask("STATS")
        for phase in ("embedding", "full_attention", "ffn", "head", "mtp"):
            assert stats[f"provider_gpu_{phase}_ns"] > 0, phase
        assert stats["provider_gpu_measured_batches"] > 0
        assert timed.ask("SHUTDOWN") == {"type": "shutdown"}
    finally:
        timed.close()
