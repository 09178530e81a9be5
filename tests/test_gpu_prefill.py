"""Prompt prefill (tall-batch linears, attention and K/V store in row batches)
against the same prompt fed through the verify step's own row-batch pass."""
import numpy as np
import pytest

import oracle_lib as ol
import qllm_provider as qp
import step_oracle
from test_gpu_verify_step import CONFIGS

pytestmark = pytest.mark.gpu


def make(name, seed, mtp=False, **kwargs):
    rng = np.random.default_rng(seed)
    c = CONFIGS[name]
    model = step_oracle.TinyModel(
        rng, 256, 512, 2, 8, 2, c["head_dim"], 256, c["scheme"],
        output_gated=c["output_gated"], qk_norm=c["qk_norm"],
        zero_centered=c["zero_centered"], rotary_dim=c["rotary_dim"])
    build = lambda: step_oracle.build_provider(model, qp, mtp=mtp, draft_vocabulary=128,
                                               **kwargs)
    return rng, model, build


@pytest.mark.parametrize("count", [1, 23, 150])
@pytest.mark.parametrize("kv_encoding", [0, 1])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_prefill_equals_row_batches(device, name, kv_encoding, count):
    rng, model, build = make(name, 50 + count, kv_encoding=kv_encoding, max_context=512)
    tokens = rng.integers(0, model.vocabulary, count).astype(np.uint32)
    fast, slow = build(), build()
    predicted = fast.prefill(tokens, 3)
    for first in range(0, count, 5):
        slow.run_target(tokens[first:first + 5], 3 + first)
    last_rows = count - (count - 1) // 5 * 5
    want_logits = slow.logits(last_rows)[-1]
    want_hidden = slow.hidden(last_rows)[-1]
    got_logits, got_hidden = fast.logits(1)[0], fast.hidden(1)[0]
    # Same arithmetic up to the F32 summation order of the linears.  bf16
    # activation rounding and the Q4H encoding turn last-bit differences into
    # one-step flips, so the end-to-end comparison is statistical, with the
    # bound the verify step's own end-to-end test uses; the tall GEMM itself
    # is held to 1e-2 / 1e-3 against the oracle in its own test.
    scale = np.abs(want_hidden).max()
    assert np.abs(got_hidden - want_hidden).max() < 2e-2 * scale
    assert (np.linalg.norm(got_logits - want_logits) /
            np.linalg.norm(want_logits)) < 2e-2
    assert predicted == int(want_logits.argmax()) or (
        want_logits.max() - want_logits[predicted] < 1e-2 * np.abs(want_logits).max())
    # the caches hold the same records
    pages = (3 + count + 63) // 64
    differing = total = 0
    for page in range(pages):
        a, b = fast.kv_page(page), slow.kv_page(page)
        if kv_encoding == 0:
            differing += int((a != b).sum())
            total += a.size
        else:
            x, y = a.view(np.float16).astype(np.float32), b.view(np.float16).astype(np.float32)
            assert np.abs(x - y).max() <= 2e-2 * max(1.0, np.abs(y).max())
    if kv_encoding == 0:
        assert differing <= 0.03 * total
    fast.close()
    slow.close()


@pytest.mark.parametrize("count", [7, 131])
def test_prefill_feeds_the_proposer_and_decoding_continues(device, count):
    rng, model, build = make("reference", 90 + count, mtp=True, max_context=512)
    tokens = rng.integers(0, model.vocabulary, count).astype(np.uint32)
    fast, slow = build(), build()
    fast.begin_request(temperature_ppm=0)
    predicted = fast.prefill(tokens, 0)
    drafts = fast.drafts()
    assert len(drafts) == 4
    assert fast.telemetry("provider_mtp_rows") >= count
    # the prompt's pairs go through the proposer in one tall pass per chunk
    # (then the last pair and three rollout passes), not five rows at a time
    assert fast.telemetry("provider_mtp_passes") == (5 if count > 1 else 4)
    # the same stream token by token: target row, then the proposer's pair
    slow.begin_request(temperature_ppm=0)
    for index in range(count):
        slow.run_target(tokens[index:index + 1], index)
        successor = int(tokens[index + 1]) if index + 1 < count else int(
            slow.logits(1)[0].argmax())
        slow.synchronize(successor, index + 1)
    want_hidden, want_logits = slow.mtp_state()
    got_hidden, got_logits = fast.mtp_state()
    assert (np.linalg.norm(got_logits - want_logits) /
            np.linalg.norm(want_logits)) < 3e-2
    assert np.abs(got_hidden - want_hidden).max() < 5e-2 * np.abs(want_hidden).max()
    assert drafts[0] == slow.drafts()[0] or (
        want_logits.max() - want_logits[drafts[0]] < 1e-2 * np.abs(want_logits).max())
    # decoding goes on from the prompt
    token, position = predicted, count
    for _ in range(3):
        emitted, token, advanced = fast.verify(token, position, 400)
        assert emitted[0] == (predicted if position == count else emitted[0])
        position += advanced
        assert len(fast.drafts()) == 4
    fast.close()
    slow.close()


@pytest.mark.parametrize("kv_encoding", [0, 1])
def test_chunked_prefill_equals_one_pass(device, kv_encoding):
    """A prompt cut into chunks of 64 and 17 rows (the last one ragged) against
    the same prompt in one pass: the chunks see the earlier ones through the
    cache only, so logits and hidden state agree within the end-to-end bound
    and the proposer ends in the same state."""
    rng, model, _ = make("reference", 77)
    tokens = rng.integers(0, model.vocabulary, 150).astype(np.uint32)
    results = []
    for chunk_rows in (0, 64, 17):
        provider = step_oracle.build_provider(
            model, qp, mtp=True, draft_vocabulary=128, kv_encoding=kv_encoding,
            max_context=512, prefill_chunk_rows=chunk_rows)
        provider.begin_request(temperature_ppm=0)
        predicted = provider.prefill(tokens, 2)
        passes = provider.telemetry("provider_mtp_passes")
        chunks = 1 if chunk_rows == 0 else -(-150 // chunk_rows)
        assert passes == chunks + 4            # a tall pass per chunk, last pair, 3 rollouts
        results.append((predicted, provider.logits(1)[0], provider.hidden(1)[0],
                        provider.mtp_state(), provider.drafts()))
        provider.close()
    want = results[0]
    for got in results[1:]:
        assert (np.linalg.norm(got[1] - want[1]) / np.linalg.norm(want[1])) < 2e-2
        assert np.abs(got[2] - want[2]).max() < 2e-2 * np.abs(want[2]).max()
        assert got[0] == want[0] or (
            want[1].max() - want[1][got[0]] < 1e-2 * np.abs(want[1]).max())
        assert (np.linalg.norm(got[3][1] - want[3][1]) / np.linalg.norm(want[3][1])) < 3e-2
        assert len(got[4]) == 4


def test_long_prompt_in_one_pass_equals_chunks(device):
    """5000 prompt rows in one pass (834 row batches: 105 layers of the prompt
    attention's grid, the longest contexts first) against passes of 1024 rows:
    the same logits and hidden state within the end-to-end bound, the same
    cache records up to the quantiser's one-step flips."""
    rng, model, _ = make("reference", 123)
    count = 5000
    tokens = rng.integers(0, model.vocabulary, count).astype(np.uint32)
    results = []
    for chunk_rows in (0, 1024):
        provider = step_oracle.build_provider(
            model, qp, draft_vocabulary=128, max_context=5120, page_tokens=256,
            prefill_chunk_rows=chunk_rows)
        if chunk_rows == 0:
            provider.prefill(tokens[:10], 0)     # a short prompt first: the workspace grows
        predicted = provider.prefill(tokens, 0)
        pages = [provider.kv_page(page) for page in range((count + 255) // 256)]
        results.append((predicted, provider.logits(1)[0], provider.hidden(1)[0], pages))
        provider.close()
    (want_token, want_logits, want_hidden, want_pages), \
        (got_token, got_logits, got_hidden, got_pages) = results
    assert (np.linalg.norm(got_logits - want_logits) / np.linalg.norm(want_logits)) < 2e-2
    assert np.abs(got_hidden - want_hidden).max() < 2e-2 * np.abs(want_hidden).max()
    assert got_token == want_token or (
        want_logits.max() - want_logits[got_token] < 1e-2 * np.abs(want_logits).max())
    differing = sum(int((a != b).sum()) for a, b in zip(got_pages, want_pages))
    assert differing <= 0.03 * sum(a.size for a in want_pages)


def test_prefill_rejects_bad_prompts(device):
    rng, model, build = make("baseline", 3, max_context=128)
    provider = build()
    with pytest.raises(qp.ProviderError, match="prompt"):
        provider.prefill(np.arange(200, dtype=np.uint32) % 7, 0)       # beyond the context
    with pytest.raises(qp.ProviderError, match="vocabulary"):
        provider.prefill(np.array([1, 99999], dtype=np.uint32), 0)
    provider.close()
