"""The worker process against the provider driven directly: a scripted
conversation over the reference runner's line protocol
(runtime/tools/moe_vm_runner.cpp:655-1470) on a tiny artifact must emit the
token stream the same provider gives through its own interface, bit for bit -
long prompts (tall prefill), short prompts (program steps + proposer
synchronisation), greedy and sampled requests, plain steps, and the error
lines of a worker without session retention."""
import numpy as np
import pytest

import artifact_writer as aw
import qllm_provider as qp
import worker_client as wc
from test_gpu_artifact_provider import geometry_of, tiny_model

pytestmark = pytest.mark.gpu

CONTEXT = 200


def request_parameters(prompt_length, sampling=None, exact=True):
    temperature, top_p, top_k, min_p, presence, seed = sampling or (0, 1000000, 0, 0, 0, 0)
    return dict(reserved_context_tokens=CONTEXT, sampling_temperature_ppm=temperature,
                sampling_top_p_ppm=top_p, sampling_top_k=top_k, sampling_min_p_ppm=min_p,
                sampling_presence_penalty_biased_ppm=presence + 2000000,
                sampling_first_output_position=prompt_length - 1, sampling_seed=seed,
                exact_decode_enabled=int(exact))


def direct_stream(provider, prompt, steps, sampling=None):
    """What the worker does for BEGIN + `steps` decode steps, on the provider."""
    provider.begin_request_with(**request_parameters(len(prompt), sampling))
    chunk = 5                                  # draft depth 4 + the guaranteed token
    if len(prompt) > chunk:
        token = provider.prefill(prompt, 0)
    else:
        token = provider.execute_program(prompt, 0)
        provider.synchronize_batch(list(prompt[1:]) + [token], 0, True)
    position, stream = len(prompt), []
    for _ in range(steps):
        emitted, token, advanced = provider.verify(token, position, CONTEXT)
        position += advanced
        stream.append(emitted)
    return stream, token


@pytest.fixture(scope="module")
def served(tmp_path_factory):
    rng, model = tiny_model(83)
    root = str(tmp_path_factory.mktemp("worker") / "artifact")
    aw.write_artifact(root, model, draft_vocabulary=128, max_context=4096)
    worker = wc.Worker(root, max_context=256, kv_page_tokens=64)
    provider = qp.Provider.from_artifact(root, geometry_of(model, 256), max_context=256,
                                         kv_page_tokens=64)
    yield rng, model, worker, provider
    worker.close()
    provider.close()


def test_ready_line_describes_the_service(served):
    _, model, worker, _ = served
    ready = worker.ready
    assert ready["type"] == "ready" and ready["protocol"] == 13
    assert ready["capacity"] == 1 and ready["vocab_size"] == model.vocabulary
    assert ready["mtp_enabled"] and ready["mtp_runtime_ready"] and ready["mtp_draft_depth"] == 4
    assert ready["sampling_supported"] and ready["sampling_presence_penalty_supported"]
    assert not ready["session_retention"] and not ready["session_persistence"]
    assert ready["kv_page_tokens"] == 64 and ready["kv_dtype"] == "q4-f16-per-head"
    assert ready["placement_mode"] == "resident" and ready["prefill_chunk_tokens"] == 5
    assert worker.ask("PING") == {"type": "pong"}


@pytest.mark.parametrize("prompt_length", [12, 3, 1])
@pytest.mark.parametrize("sampling", [None, (800000, 950000, 40, 0, 0, 7),
                                      (700000, 1000000, 20, 50000, 600000, 11)])
def test_conversation_equals_the_provider(served, prompt_length, sampling):
    rng, model, worker, provider = served
    prompt = rng.integers(0, model.vocabulary, prompt_length).astype(np.uint32)
    expected, pending = direct_stream(provider, prompt, 5, sampling)
    calls = worker.ask("STATS")["exact_decode_calls"]
    assert worker.begin(1, CONTEXT, prompt, sampling) == {"type": "begun", "id": 1}
    got = [worker.next(1, 0) for _ in range(5)]
    assert all(reply["type"] == "token" and reply["id"] == 1 for reply in got), got
    assert [reply["tokens"] for reply in got] == expected
    stats = worker.ask("STATS")
    assert stats["exact_decode_calls"] == calls + 5      # every step was speculative
    assert stats["exact_decode_positions"] >= stats["exact_decode_calls"]
    # mode 1 emits the pending token and closes the request
    assert worker.next(1, 1) == {"type": "token", "id": 1, "tokens": [pending]}
    assert worker.ask("END", 1)["type"] == "error"


def test_plain_steps_and_batches(served):
    rng, model, worker, provider = served
    prompt = rng.integers(0, model.vocabulary, 4).astype(np.uint32)
    provider.begin_request_with(**request_parameters(len(prompt)))
    token = provider.execute_program(prompt, 0)
    provider.synchronize_batch(list(prompt[1:]) + [token], 0, True)
    expected = []
    for position in range(4, 8):
        expected.append(token)
        token = provider.execute_program([token], position)
        provider.synchronize_batch([token], position, True)   # the proposer follows
    assert worker.begin(7, CONTEXT, prompt)["type"] == "begun"
    got = [worker.ask("STEP", "7,2") for _ in range(4)]
    assert got == [{"type": "batch", "items": [{"id": 7, "tokens": [t]}]} for t in expected]
    stats = worker.ask("STATS")
    assert stats["type"] == "stats" and stats["active_requests"] == 1
    assert stats["kv_reserved_pages"] == 1 and stats["program_steps"] >= 8
    assert worker.ask("SHUTDOWN") == {
        "type": "error", "message": "SHUTDOWN requires no retained state"}
    assert worker.ask("END", 7) == {"type": "ended", "id": 7}


def test_error_lines_keep_the_worker_serving(served):
    _, model, worker, _ = served
    message = lambda *fields: worker.ask(*fields).get("message")
    assert message("HELLO") == "unknown worker command"
    assert message("BEGIN", 1, CONTEXT, str(model.vocabulary)) == "token is outside model vocabulary"
    assert message("BEGIN", 0, CONTEXT, "1,2") == "invalid BEGIN request identity or context"
    assert message("BEGIN", 1, 100000, "1,2") == "invalid BEGIN request identity or context"
    assert message("BEGIN", 1, 3, "1,2,3") == "prompt exhausts request context"
    assert message("BEGIN", 1, CONTEXT, "1,2", "RESUME", 5) == \
        "callable provider does not support session retention"
    assert message("BEGIN", 1, CONTEXT, "1,2", "SAMPLING", 1, 2) == "invalid BEGIN sampling marker"
    assert message("BEGIN", 1, CONTEXT, "1,2", "SAMPLING", 3000000, 1, 0, 0, 0, 0) == \
        "invalid BEGIN sampling values"
    assert message("BEGIN", 1, CONTEXT, "1,2", "EXTRA") == "unknown BEGIN request fields"
    assert message("NEXT", 9, 0) == "STEP request mismatch"
    assert message("END", 9) == "unknown active request"
    assert message("DROP", 9) == "callable provider does not support session retention"
    assert message("SAVE", 9, "a", "b") == "callable provider does not support session persistence"
    # a second request while one is active exceeds the capacity of one
    assert worker.begin(3, CONTEXT, [1, 2, 3])["type"] == "begun"
    assert message("BEGIN", 4, CONTEXT, "1,2") == "callable provider capacity is exhausted"
    assert message("BEGIN", 3, CONTEXT, "1,2") == "invalid BEGIN request identity or context"
    worker.send("CANCEL", 3)                    # no reply line
    assert worker.ask("PING") == {"type": "pong"}
    assert worker.ask("STATS")["active_requests"] == 0


def test_context_limit_ends_speculation(served):
    """Driven as the service drives it: decode steps while two positions are
    left, then the pending token with mode 1.  A verify step never runs past
    the request's context."""
    rng, model, worker, provider = served
    prompt = rng.integers(0, model.vocabulary, 6).astype(np.uint32)
    limit = 12
    assert worker.begin(5, limit, prompt)["type"] == "begun"
    emitted = []
    while len(prompt) + len(emitted) + 1 < limit:
        reply = worker.next(5, 0)
        assert reply["type"] == "token", reply
        emitted += reply["tokens"]
        assert len(prompt) + len(emitted) + 1 <= limit
    emitted += worker.next(5, 1)["tokens"]
    assert len(prompt) + len(emitted) == limit
    # the same stream without speculation: plain steps give the same tokens
    provider.begin_request_with(**request_parameters(len(prompt), exact=False))
    provider.execute_program(prompt[:5], 0)          # the program takes five rows
    token, plain = provider.execute_program(prompt[5:], 5), []
    for position in range(len(prompt), limit - 1):
        plain.append(token)
        token = provider.execute_program([token], position)
    assert emitted == plain + [token]


def test_exhausted_context_is_an_error_line(served):
    _, _, worker, _ = served
    assert worker.begin(6, 5, [1, 2, 3])["type"] == "begun"
    emitted = []
    for _ in range(4):
        reply = worker.next(6, 0)
        if reply["type"] == "error":        # at the latest when no position is left
            break
        emitted += reply["tokens"]
    assert reply["type"] == "error" and len(emitted) <= 2
    assert worker.next(6, 0) == {"type": "error", "message": "request context is exhausted"}
    assert worker.ask("END", 6) == {"type": "ended", "id": 6}


def test_zz_shutdown(served):
    _, _, worker, _ = served
    assert worker.ask("SHUTDOWN") == {"type": "shutdown"}
    assert worker.process.wait(timeout=30) == 0
