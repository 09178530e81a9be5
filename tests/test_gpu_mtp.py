"""The proposer (one MTP layer with its own Q8 KV cache) inside the provider:
its passes against the composed CPU oracle on a small decoder, and the decode
cycle verify -> proposer advance -> draft rollout (execute_exact_decode with
run_mtp / extend_mtp_rollout, dense_fp4_provider.cpp:8681-8852, 11262-11288)."""
import numpy as np
import pytest

import gpu_util as gu
import oracle_lib as ol
import qllm_provider as qp
import step_oracle
from test_gpu_verify_step import CONFIGS

pytestmark = pytest.mark.gpu

DRAFT_VOCABULARY = 128     # the proposer scores the first 128 of 256 head rows


def make(name, seed, **kwargs):
    rng = np.random.default_rng(seed)
    c = CONFIGS[name]
    model = step_oracle.TinyModel(
        rng, 256, 512, 2, 8, 2, c["head_dim"], 256, c["scheme"],
        output_gated=c["output_gated"], qk_norm=c["qk_norm"],
        zero_centered=c["zero_centered"], rotary_dim=c["rotary_dim"])
    provider = step_oracle.build_provider(model, qp, mtp=True,
                                          draft_vocabulary=DRAFT_VOCABULARY, **kwargs)
    return rng, model, provider


def q8_records(provider, model, page_index, page_tokens):
    """The proposer's layer of one device page, re-laid as reference records."""
    offset = provider.telemetry("provider_mtp_kv_page_offset")
    return gu.q8_planes_to_records(provider.kv_page(page_index), offset, page_tokens,
                                   model.kv_heads, model.head_dim)


@pytest.mark.parametrize("name", list(CONFIGS))
def test_proposer_passes_match_the_composed_oracle(device, name):
    rng, model, provider = make(name, 21)
    page_tokens = 64
    V = model.vocabulary
    tokens = rng.integers(0, V, 5).astype(np.uint32)
    provider.run_target(tokens, 0)
    target_hidden = provider.hidden(5)
    guaranteed = int(provider.logits(5)[0].argmax())

    # synchronise at position 1: proposer row (token at 1, target hidden at 0),
    # then three single-row rollout passes on its own hidden state
    provider.begin_request(temperature_ppm=0)
    provider.synchronize(guaranteed, 1)
    drafts = provider.drafts()
    assert len(drafts) == 4 and all(t < DRAFT_VOCABULARY for t in drafts)
    assert provider.telemetry("provider_mtp_passes") == 4
    assert provider.telemetry("provider_mtp_rows") == 4
    got_hidden, got_logits = provider.mtp_state()

    layer_bytes = ol.q8_layer_bytes(page_tokens, model.kv_heads, model.head_dim)
    pages = [np.zeros(layer_bytes, dtype=np.uint8)]
    observed = [q8_records(provider, model, 0, page_tokens)]
    previous, token = target_hidden[:1], guaranteed
    for depth in range(4):
        report = {}
        logits, hidden = step_oracle.run_mtp(
            model, np.array([token], dtype=np.uint32), previous, depth, pages,
            page_tokens, DRAFT_VOCABULARY, observed, 0, report)
        # the GPU's draft must be the oracle's arg-max up to the tolerance
        assert logits[drafts[depth]] >= logits.max() - 2e-2 * np.abs(logits).max()
        # Q8 records: the first pass has identical inputs on both sides, so its
        # bytes agree except where a last-bit difference crossed a rounding
        # boundary; the rollout passes run on each side's own previous hidden
        # state (1e-2 apart after the bf16 rounding points), which moves codes
        # by a unit here and there - their dequantised values must still agree
        if depth == 0:
            assert report["record_byte_diffs"] <= 0.03 * report["record_bytes"]
        assert report["value_error"] < 0.05, (depth, report)
        previous, token = hidden[-1:], drafts[depth]
    relative = np.linalg.norm(got_logits - logits) / np.linalg.norm(logits)
    assert relative < 2e-2, relative
    assert np.abs(got_hidden - hidden[-1]).max() < 0.05 * np.abs(hidden).max()
    provider.close()


def test_multi_row_proposer_pass_after_accepted_drafts(device):
    """Drafts that the target accepts make the next proposer pass a micro-batch
    (accepted drafts + next token); its result against the oracle."""
    rng, model, provider = make("baseline", 23)
    page_tokens, V = 64, model.vocabulary
    provider.run_target(rng.integers(0, V, 5).astype(np.uint32), 0)
    position = 5
    guaranteed = int(rng.integers(0, V))
    provider.begin_request(temperature_ppm=0)
    provider.synchronize(guaranteed, position)
    # replace the proposer's drafts by the target's own arg-max chain
    drafts = rng.integers(0, V, 4).astype(np.uint32)
    for depth in range(3):
        provider.run_target(np.array([guaranteed, *drafts], dtype=np.uint32), position)
        drafts[depth] = provider.logits(5)[depth].argmax()
    provider.set_drafts(drafts)
    before = [q8_records(provider, model, 0, page_tokens)]
    passes = provider.telemetry("provider_mtp_passes")
    emitted, next_token, advanced = provider.verify(guaranteed, position, 256)
    assert advanced >= 4 and emitted == [guaranteed, *drafts[:advanced - 1].tolist()]
    target_hidden = provider.hidden(5)
    assert provider.telemetry("provider_mtp_passes") == passes + 4
    new_drafts = provider.drafts()
    assert len(new_drafts) == 4

    # the advance pass: rows = accepted drafts + next token, cached from `position`
    mtp_tokens = np.array([*drafts[:advanced - 1], next_token], dtype=np.uint32)
    observed = [q8_records(provider, model, 0, page_tokens)]
    pages = [before[0].copy()]
    report = {}
    logits, hidden = step_oracle.run_mtp(
        model, mtp_tokens, target_hidden[:advanced], position, pages, page_tokens,
        DRAFT_VOCABULARY, observed, 0, report)
    assert report["record_byte_diffs"] <= 0.03 * report["record_bytes"]
    assert report["value_error"] < 0.05
    assert logits[new_drafts[0]] >= logits.max() - 2e-2 * np.abs(logits).max()
    # the verify step that follows starts where the stream now stands
    emitted, after, advanced2 = provider.verify(next_token, position + advanced, 256)
    assert emitted[0] == next_token and 1 <= advanced2 <= 5
    provider.close()


@pytest.mark.parametrize("temperature,top_k", [(0, 0), (800000, 20)])
def test_decode_cycle_runs_on_its_own_drafts(device, temperature, top_k):
    """Several cycles without outside drafts; greedy acceptance is checked on the
    logits of each verify step, sampled decoding must be reproducible."""
    streams = []
    for attempt in range(2):
        rng, model, provider = make("reference", 31)
        V = model.vocabulary
        provider.run_target(rng.integers(0, V, 5).astype(np.uint32), 0)
        position, token = 5, 7
        provider.begin_request(temperature_ppm=temperature, top_p_ppm=950000,
                               top_k=top_k, seed=77)
        provider.synchronize(token, position)
        stream = []
        for step in range(6):
            drafts = provider.drafts()
            assert len(drafts) == 4
            emitted, next_token, advanced = provider.verify(token, position, 256)
            if temperature == 0:
                accepted, want_next = ol.accept_greedy(
                    provider.logits(5), np.array(drafts, dtype=np.uint32))
                assert advanced == accepted + 1 and next_token == want_next
            assert emitted == [token, *drafts[:advanced - 1]]
            stream += emitted
            token, position = next_token, position + advanced
        assert provider.telemetry("provider_exact_calls") == 6
        assert provider.telemetry("provider_mtp_passes") == 4 * 7
        streams.append(stream)
        provider.close()
    assert streams[0] == streams[1]


@pytest.mark.parametrize("temperature,top_k", [(0, 0), (800000, 20)])
def test_captured_proposer_passes_equal_the_eager_ones(device, monkeypatch,
                                                       temperature, top_k):
    """The proposer replayed from captured graphs (positions read on the device,
    greedy passes chained without the host) against the same passes launched
    one kernel at a time: tokens, drafts, hidden state and logits are equal."""
    runs = []
    for eager in ("1", "0"):
        monkeypatch.setenv("QLLM_PROVIDER_EAGER", eager)
        rng, model, provider = make("reference", 41, max_context=256)
        V = model.vocabulary
        provider.run_target(rng.integers(0, V, 5).astype(np.uint32), 0)
        position, token, limit = 5, 11, 40
        provider.begin_request(temperature_ppm=temperature, top_p_ppm=950000,
                               top_k=top_k, seed=5)
        provider.synchronize(token, position)
        record = []
        while provider.drafts():
            drafts = provider.drafts()
            emitted, token, advanced = provider.verify(token, position, limit)
            position += advanced
            hidden, logits = provider.mtp_state()
            record.append((drafts, emitted, token, hidden.copy(), logits.copy()))
        assert position >= limit - 2
        runs.append(record)
        provider.close()
    assert len(runs[0]) == len(runs[1]) >= 7
    for eager_step, graph_step in zip(*runs):
        assert eager_step[:3] == graph_step[:3]
        assert np.array_equal(eager_step[3], graph_step[3])
        assert np.array_equal(eager_step[4], graph_step[4])


@pytest.mark.parametrize("temperature,top_k", [(0, 0), (800000, 20)])
def test_decode_cycle_with_a_presence_penalty(device, temperature, top_k):
    """The proposer penalises its draft logits at the emitted tokens and at the
    drafts of the rollout so far (dense_fp4_provider.cpp:8822-8847, 11290-11296):
    the last draft is the arg-max of the penalised logits it left behind, the
    target's acceptance is the oracle's on the penalised target logits, and a
    repeated run gives the same stream."""
    streams = []
    for attempt in range(2):
        rng, model, provider = make("reference", 31)
        V = model.vocabulary
        provider.run_target(rng.integers(0, V, 5).astype(np.uint32), 0)
        position, token = 5, 7
        provider.begin_request_with(
            reserved_context_tokens=256, sampling_temperature_ppm=temperature,
            sampling_top_p_ppm=950000, sampling_top_k=top_k, sampling_min_p_ppm=0,
            sampling_presence_penalty_biased_ppm=4000000,      # penalty 2.0
            sampling_first_output_position=0, sampling_seed=77, exact_decode_enabled=1)
        provider.synchronize(token, position)
        stream, emitted_tokens = [], set()
        for step in range(6):
            drafts = provider.drafts()
            assert len(drafts) == 4
            if temperature == 0:
                _, draft_logits = provider.mtp_state()
                assert drafts[-1] == ol.argmax(draft_logits)
            emitted, next_token, advanced = provider.verify(token, position, 256)
            if temperature == 0:
                accepted, want_next = ol.accept_greedy(
                    provider.logits(5), np.array(drafts, dtype=np.uint32))
                assert advanced == accepted + 1 and next_token == want_next
            assert emitted == [token, *drafts[:advanced - 1]]
            stream += emitted
            token, position = next_token, position + advanced
        streams.append(stream)
        provider.close()
    assert streams[0] == streams[1]


def test_draft_logits_without_a_finite_maximum_are_reported(device):
    """A draft norm full of NaN makes every draft logit NaN: the device-side
    arg-max selects no token, the chained pass embeds zeros for it, every
    kernel runs to its end and the step reports the failure."""
    rng = np.random.default_rng(5)
    c = CONFIGS["baseline"]
    model = step_oracle.TinyModel(
        rng, 256, 512, 2, 8, 2, c["head_dim"], 256, c["scheme"],
        output_gated=c["output_gated"], qk_norm=c["qk_norm"],
        zero_centered=c["zero_centered"], rotary_dim=c["rotary_dim"])
    model.mtp["draft_norm"][:] = np.nan
    provider = step_oracle.build_provider(model, qp, mtp=True,
                                          draft_vocabulary=DRAFT_VOCABULARY)
    provider.run_target(rng.integers(0, 256, 5).astype(np.uint32), 0)
    provider.begin_request(temperature_ppm=0)
    with pytest.raises(qp.ProviderError) as error:      # uncaptured passes
        provider.synchronize(3, 5)
    assert "draft" in str(error.value)
    # the captured rollout at the end of a verify step chains its four passes on
    # the device: the token nobody selected (0xffffffff) is embedded as zeros
    provider.set_drafts(np.array([1, 2, 3, 4], dtype=np.uint32))
    with pytest.raises(qp.ProviderError) as error:
        provider.verify(3, 5, 256)
    assert "draft" in str(error.value)
    # the device is intact: the target still runs and gives finite logits
    provider.run_target(rng.integers(0, 256, 5).astype(np.uint32), 0)
    assert np.isfinite(provider.logits(5)).all()
    provider.close()


def test_target_logits_without_a_finite_maximum_leave_the_request_as_it_was(device):
    """A final norm full of NaN makes every target logit NaN: the rows' arg-max
    selects no token (0xffffffff).  The greedy verify step reports that before
    it touches the proposer or the request - the drafts it was given are still
    there and no proposer pass ran - and so does the head of a prompt."""
    rng = np.random.default_rng(6)
    c = CONFIGS["baseline"]
    model = step_oracle.TinyModel(
        rng, 256, 512, 2, 8, 2, c["head_dim"], 256, c["scheme"],
        output_gated=c["output_gated"], qk_norm=c["qk_norm"],
        zero_centered=c["zero_centered"], rotary_dim=c["rotary_dim"])
    model.final_norm[:] = np.nan
    provider = step_oracle.build_provider(model, qp, mtp=True,
                                          draft_vocabulary=DRAFT_VOCABULARY)
    provider.run_target(rng.integers(0, 256, 5).astype(np.uint32), 0)
    provider.begin_request(temperature_ppm=0)
    provider.synchronize(3, 5)        # the proposer has its own norms: drafts exist
    drafts = provider.drafts()
    assert len(drafts) == 4
    passes = provider.telemetry("provider_mtp_passes")
    for attempt in range(2):          # the same call fails the same way again
        with pytest.raises(qp.ProviderError) as error:
            provider.verify(3, 5, 256)
        assert "target logits have no finite maximum" in str(error.value)
        assert provider.drafts() == drafts
        assert provider.telemetry("provider_mtp_passes") == passes
        assert provider.telemetry("provider_exact_calls") == 0
    with pytest.raises(qp.ProviderError) as error:
        provider.prefill(rng.integers(0, 256, 7).astype(np.uint32), 0)
    assert "head logits have no finite maximum" in str(error.value)
    provider.close()


def test_rollout_stops_at_the_context_limit(device):
    rng, model, provider = make("baseline", 37, max_context=64)
    V = model.vocabulary
    provider.run_target(rng.integers(0, V, 5).astype(np.uint32), 0)
    provider.begin_request(temperature_ppm=0)
    provider.synchronize(3, 5)
    token, position, limit = 3, 5, 12
    while True:
        drafts = provider.drafts()
        if not drafts:
            break
        assert position + len(drafts) < limit          # the drafts fit the context
        emitted, token, advanced = provider.verify(token, position, limit)
        position += advanced
    assert position >= limit - 2
    with pytest.raises(qp.ProviderError):               # no drafts left
        provider.verify(token, position, limit)
    provider.close()
