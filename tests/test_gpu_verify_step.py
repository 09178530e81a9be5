"""The whole verify step through the provider: target pass parity against the
composed CPU oracle on a 2-layer decoder, and acceptance (greedy, stochastic
whole-vocabulary, stochastic top-k) bit-exact against the oracle evaluated on
the very logits the GPU produced."""
import numpy as np
import pytest

import oracle_lib as ol
import qllm_provider as qp
import step_oracle

pytestmark = pytest.mark.gpu

CONFIGS = {
    # benchmark model style: plain GQA, full rotary, binary16 scale per 16
    "baseline": dict(scheme=ol.SCALE_F16_BLOCK16, output_gated=False, qk_norm=False,
                     zero_centered=False, head_dim=128, rotary_dim=None),
    # reference-style: ABI 3 weights, output gate, q/k norm, partial rotary, d=256
    "reference": dict(scheme=ol.SCALE_UE8M0_BLOCK32, output_gated=True, qk_norm=True,
                      zero_centered=True, head_dim=256, rotary_dim=64),
}


def make(name, seed):
    rng = np.random.default_rng(seed)
    c = CONFIGS[name]
    model = step_oracle.TinyModel(
        rng, 256, 512, 2, 8, 2, c["head_dim"], 1024, c["scheme"],
        output_gated=c["output_gated"], qk_norm=c["qk_norm"],
        zero_centered=c["zero_centered"], rotary_dim=c["rotary_dim"])
    return rng, model, step_oracle.build_provider(model, qp)


@pytest.mark.parametrize("qkv_splits", ["0", "4"])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_target_pass_matches_composed_oracle(device, monkeypatch, name, qkv_splits):
    # qkv_splits 4: the q/k/v projection as four K-split partials that the
    # rope + store kernel adds up (off by default)
    monkeypatch.setenv("QLLM_PROVIDER_QKV_SPLITS", qkv_splits)
    rng, model, provider = make(name, 7)
    page_tokens = 64
    layer_bytes = ol.q4h_layer_bytes(page_tokens, model.kv_heads, model.head_dim)
    pages = [np.zeros(layer_bytes * model.layers, dtype=np.uint8) for _ in range(4)]
    position = 0
    for step in range(3):
        tokens = rng.integers(0, model.vocabulary, 5).astype(np.uint32)
        provider.run_target(tokens, position)
        logits, hidden = provider.logits(5), provider.hidden(5)
        observed = [provider.kv_page(i) for i in range(4)]
        report = {}
        want_logits, want_hidden = step_oracle.run_target(
            model, tokens, position, pages, page_tokens, observed, report)
        # Q4H records: identical except where a last-bit difference crossed a
        # rounding boundary (layer 1 sees activations that already differ in
        # the low bits); such flips stay rare
        assert report["record_byte_diffs"] <= 0.03 * report["record_bytes"]
        # bf16 activation rounding turns ~1e-3 differences into one-ulp flips,
        # so the end-to-end check is statistical; the per-operation tests hold
        # the 1e-2 / 1e-3 tolerance
        relative = (np.linalg.norm(logits - want_logits) /
                    np.linalg.norm(want_logits))
        assert relative < 2e-2, relative
        assert np.abs(hidden - want_hidden).max() < 0.05 * np.abs(want_hidden).max()
        assert np.array_equal(logits.argmax(1), want_logits.argmax(1))
        position += 5
    provider.close()


@pytest.mark.parametrize("name", list(CONFIGS))
def test_target_pass_with_exact_f16_cache(device, name):
    """The same pass over the exact-F16 KV cache (kv-cache-dtype fp16)."""
    rng = np.random.default_rng(11)
    c = CONFIGS[name]
    model = step_oracle.TinyModel(
        rng, 256, 512, 2, 8, 2, c["head_dim"], 1024, c["scheme"],
        output_gated=c["output_gated"], qk_norm=c["qk_norm"],
        zero_centered=c["zero_centered"], rotary_dim=c["rotary_dim"])
    provider = step_oracle.build_provider(model, qp, kv_encoding=1)
    page_tokens = 64
    page_bytes = model.layers * 2 * page_tokens * model.kv_heads * model.head_dim * 2
    pages = [np.zeros(page_bytes, dtype=np.uint8) for _ in range(4)]
    position = 0
    for step in range(3):
        tokens = rng.integers(0, model.vocabulary, 5).astype(np.uint32)
        provider.run_target(tokens, position)
        logits, hidden = provider.logits(5), provider.hidden(5)
        want_logits, want_hidden = step_oracle.run_target(
            model, tokens, position, pages, page_tokens, kv_encoding=1)
        relative = (np.linalg.norm(logits - want_logits) /
                    np.linalg.norm(want_logits))
        assert relative < 2e-2, relative
        assert np.abs(hidden - want_hidden).max() < 0.05 * np.abs(want_hidden).max()
        assert np.array_equal(logits.argmax(1), want_logits.argmax(1))
        position += 5
    provider.close()


@pytest.mark.parametrize("name", list(CONFIGS))
def test_acceptance_is_bit_exact_on_the_same_logits(device, name):
    rng, model, provider = make(name, 11)
    V = model.vocabulary
    position = 0
    # build some context first
    provider.run_target(rng.integers(0, V, 5).astype(np.uint32), position)
    position = 5
    guaranteed = int(rng.integers(0, V))

    # ---- greedy: make the first two drafts the true argmax chain -------------
    provider.begin_request(temperature_ppm=0)
    provider.synchronize(guaranteed, position)
    drafts = rng.integers(0, V, 4).astype(np.uint32)
    for depth in range(2):
        provider.run_target(np.array([guaranteed, *drafts], dtype=np.uint32), position)
        drafts[depth] = provider.logits(5)[depth].argmax()
    provider.set_drafts(drafts)
    emitted, next_token, advanced = provider.verify(guaranteed, position, 256)
    logits = provider.logits(5)
    accepted, want_next = ol.accept_greedy(logits, drafts)
    assert accepted >= 2
    assert advanced == accepted + 1 and next_token == want_next
    assert emitted == [guaranteed, *drafts[:accepted].tolist()]
    position += advanced

    # ---- stochastic, whole-vocabulary candidates (top_k = 0) ------------------
    def dirichlet_drafts():
        tokens, distributions = [], []
        for _ in range(4):
            q = rng.dirichlet(np.full(V, 0.1))
            q = q / q.sum()
            tokens.append(int(rng.choice(V, p=q)))
            distributions.append((np.arange(V, dtype=np.uint32), q))
        return tokens, distributions

    for trial in range(3):
        seed = 1234 + trial
        provider.begin_request(temperature_ppm=700000, top_p_ppm=950000, top_k=0,
                               min_p_ppm=0, seed=seed)
        provider.synchronize(next_token, position)
        tokens, distributions = dirichlet_drafts()
        provider.set_drafts(np.array(tokens, dtype=np.uint32), distributions)
        emitted, after, advanced = provider.verify(next_token, position, 256)
        logits = provider.logits(5)
        targets = []
        for row in range(5):
            order = np.lexsort((np.arange(V), -logits[row].astype(np.float64)))
            status, t, p = ol.make_sampling_distribution(
                logits[row][order], order.astype(np.uint32), 700000, 950000, 0)
            assert status == 0
            targets.append((t, p))
        status, accepted, want_next = ol.accept_stochastic(
            targets, distributions, tokens, seed, position)
        assert status == 0
        assert advanced == accepted + 1 and after == want_next
        assert emitted == [next_token, *tokens[:accepted]]
        next_token, position = after, position + advanced

    # ---- stochastic, GPU top-k candidates (the reference's bounded form) ------
    provider.begin_request(temperature_ppm=1000000, top_p_ppm=950000, top_k=20,
                           min_p_ppm=0, seed=99)
    provider.synchronize(next_token, position)
    tokens, distributions = dirichlet_drafts()
    provider.set_drafts(np.array(tokens, dtype=np.uint32), distributions)
    emitted, after, advanced = provider.verify(next_token, position, 256)
    logits = provider.logits(5)
    targets = []
    for row in range(5):
        values, indices = ol.topk(logits[row], 20)
        status, t, p = ol.make_sampling_distribution(values, indices, 1000000, 950000, 0)
        targets.append((t, p))
    status, accepted, want_next = ol.accept_stochastic(targets, distributions, tokens,
                                                       99, position)
    assert advanced == accepted + 1 and after == want_next
    assert provider.telemetry("provider_exact_calls") == 5
    provider.close()


def request_with(temperature_ppm, top_k, seed, penalty_ppm, **extra):
    return dict(reserved_context_tokens=256, sampling_temperature_ppm=temperature_ppm,
                sampling_top_p_ppm=950000, sampling_top_k=top_k, sampling_min_p_ppm=0,
                sampling_presence_penalty_biased_ppm=2000000 + penalty_ppm,
                sampling_first_output_position=0, sampling_seed=seed,
                exact_decode_enabled=1, **extra)


@pytest.mark.parametrize("temperature_ppm,top_k", [(0, 0), (900000, 20), (700000, 0)])
def test_presence_penalty_in_the_verify_step(device, temperature_ppm, top_k):
    """A request with a presence penalty of 1.5 (and one of -0.75): every row's
    logits are penalised at the tokens emitted so far and at the drafts of the
    rows before it, before arg-max / top-k (dense_fp4_provider.cpp:8331-8349,
    11182-11202, 11261-11270); tokens bit-exact against the oracle applying
    qo_presence_penalty to the logits the GPU produced."""
    for penalty_ppm in (1500000, -750000):
        rng, model, provider = make("baseline", 17)
        V = model.vocabulary
        penalty = np.float32(penalty_ppm / 1e6)
        provider.run_target(rng.integers(0, V, 5).astype(np.uint32), 0)
        position, token, seed = 5, int(rng.integers(0, V)), 4242
        provider.begin_request_with(**request_with(temperature_ppm, top_k, seed, penalty_ppm))
        provider.synchronize(token, position)
        emitted_so_far = np.zeros(V, dtype=np.uint8)
        for step in range(4):
            drafts = rng.integers(0, V, 4).astype(np.uint32)
            if step:
                drafts[0] = drafts[2]          # a draft that repeats inside the step
            rows = np.array([token, *drafts], dtype=np.uint32)
            provider.run_target(rows, position)
            raw = provider.logits(5)
            if temperature_ppm == 0:
                # make the first draft the penalised arg-max so that it is accepted
                drafts[0] = ol.argmax(ol.presence_penalty(raw[0], emitted_so_far, penalty))
                rows[1] = drafts[0]
                provider.run_target(rows, position)
                raw = provider.logits(5)
            if temperature_ppm == 0:
                provider.set_drafts(drafts)
                draft_distributions = [(np.array([t], np.uint32), np.array([1.0]))
                                       for t in drafts]
            else:
                draft_distributions = []
                for t in drafts:
                    q = rng.dirichlet(np.full(V, 0.1)); q /= q.sum()
                    q_tokens = np.arange(V, dtype=np.uint32)
                    if q[t] == 0.0:
                        q[t] = 1e-6; q /= q.sum()
                    draft_distributions.append((q_tokens, q))
                provider.set_drafts(drafts, draft_distributions)
            got_emitted, got_next, advanced = provider.verify(token, position, 256)
            # the oracle's statement on the raw logits
            present = emitted_so_far.copy()
            penalised = np.empty_like(raw)
            for row in range(5):
                penalised[row] = ol.presence_penalty(raw[row], present, penalty)
                if row < 4:
                    present[drafts[row]] = 1
            assert np.array_equal(provider.logits(5), penalised), (penalty_ppm, step)
            if temperature_ppm == 0:
                accepted, want_next = ol.accept_greedy(penalised, drafts)
                assert accepted >= 1
            else:
                targets = []
                for row in range(5):
                    if top_k:
                        values, indices = ol.topk(penalised[row], top_k)
                    else:
                        indices = np.lexsort((np.arange(V), -penalised[row].astype(np.float64))).astype(np.uint32)
                        values = penalised[row][indices]
                    status, t, p = ol.make_sampling_distribution(
                        values, indices, temperature_ppm, 950000, 0)
                    assert status == 0
                    targets.append((t, p))
                status, accepted, want_next = ol.accept_stochastic(
                    targets, draft_distributions, drafts.tolist(), seed, position)
                assert status == 0
            assert advanced == accepted + 1 and got_next == want_next, (penalty_ppm, step)
            assert got_emitted == [token, *drafts[:accepted].tolist()]
            emitted_so_far[drafts[:accepted]] = 1
            emitted_so_far[got_next] = 1
            token, position = got_next, position + advanced
        provider.close()


def test_request_profiles_the_provider_turns_down(device):
    rng, model, provider = make("baseline", 3)
    with pytest.raises(qp.ProviderError):      # sampled, penalty parameter above 4,000,000
        provider.begin_request_with(**request_with(700000, 20, 1, 2000001))
    bad = request_with(700000, 20, 1, 0)
    del bad["sampling_first_output_position"]
    with pytest.raises(qp.ProviderError):      # sampled without a first output position
        provider.begin_request_with(**bad)
    # a greedy request carries the parameter too, and it is checked when used
    provider.begin_request_with(**request_with(0, 0, 1, 2000001))
    provider.synchronize(5, 10)
    provider.set_drafts(np.array([1, 2, 3, 4], dtype=np.uint32))
    with pytest.raises(qp.ProviderError):
        provider.verify(5, 10, 256)
    provider.close()


def test_provider_rejects_invalid_streams(device):
    rng, model, provider = make("baseline", 3)
    provider.begin_request(temperature_ppm=0)
    provider.synchronize(5, 10)
    with pytest.raises(qp.ProviderError):          # no drafts set
        provider.verify(5, 10, 256)
    provider.set_drafts(np.array([1, 2, 3, 4], dtype=np.uint32))
    with pytest.raises(qp.ProviderError):          # wrong guaranteed token
        provider.verify(6, 10, 256)
    with pytest.raises(qp.ProviderError):          # wrong position
        provider.verify(5, 11, 256)
    with pytest.raises(qp.ProviderError):          # context limit reached
        provider.verify(5, 10, 11)
    emitted, next_token, advanced = provider.verify(5, 10, 256)
    assert emitted[0] == 5 and 1 <= advanced <= 5 and len(emitted) == advanced
    with pytest.raises(qp.ProviderError):          # drafts were consumed
        provider.verify(next_token, 10 + advanced, 256)
    with pytest.raises(qp.ProviderError):
        provider.prepare("moe.swiglu.routed.merge-shared.v1")   # not provided
    provider.close()


def test_graph_replay_reproduces_the_eager_pass(device):
    rng, model, provider = make("baseline", 5)
    tokens = rng.integers(0, model.vocabulary, 5).astype(np.uint32)
    provider.run_target(tokens, 0)
    eager = provider.logits(5)
    provider.capture_target(tokens, 0)
    for _ in range(3):
        provider.replay_target()
        provider.run_target(tokens, 0)          # eager work between the replays
        provider.synchronize_stream()
        provider.replay_target()
        assert np.array_equal(provider.logits(5), eager)
    provider.close()


def test_one_graph_follows_advancing_positions(device):
    """The graph captured at the first position is replayed with new tokens and
    positions in device memory; it must match eager launches step by step."""
    rng, model, graphed = make("baseline", 9)
    _, _, eager = make("baseline", 9)            # same seed -> same model
    position = 0
    for step in range(6):
        tokens = rng.integers(0, model.vocabulary, 5).astype(np.uint32)
        graphed.capture_target(tokens, position)    # run_target_graph
        eager.run_target(tokens, position)
        assert np.array_equal(graphed.logits(5), eager.logits(5)), step
        for page in range(2):
            assert np.array_equal(graphed.kv_page(page), eager.kv_page(page))
        position += int(rng.integers(1, 6))
    graphed.close()
    eager.close()
