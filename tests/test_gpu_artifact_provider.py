"""A provider created from an artifact directory (manifest, model program,
dense pack) against the same model handed over tensor by tensor: the
geometry derived from the program, the bound tensors and the decode cycle are
the same, bit for bit."""
import numpy as np
import pytest

import artifact_writer as aw
import oracle_lib as ol
import qllm_provider as qp
import step_oracle

pytestmark = pytest.mark.gpu


def tiny_model(seed, output_gated=True):
    rng = np.random.default_rng(seed)
    model = step_oracle.TinyModel(
        rng, 256, 512, 2, 8, 2, 128, 256, ol.SCALE_UE8M0_BLOCK32,
        output_gated=output_gated, qk_norm=output_gated, zero_centered=True,
        rotary_dim=64 if output_gated else None)
    return rng, model


def geometry_of(model, max_context, draft_depth=4, draft_vocabulary=128, kv_encoding=0):
    m = model
    return dict(hidden=m.hidden, intermediate=m.intermediate, layers=m.layers,
                query_heads=m.query_heads, kv_heads=m.kv_heads, head_dim=m.head_dim,
                rotary_dim=m.rotary_dim, vocabulary=m.vocabulary, rope_theta=m.rope_theta,
                norm_epsilon=m.eps, output_gated=int(m.output_gated), qk_norm=int(m.qk_norm),
                zero_centered_norm=int(m.zero_centered), scale_scheme=m.scheme,
                kv_encoding=kv_encoding, kv_page_tokens=64, max_context=max_context,
                draft_depth=draft_depth, mtp_layers=1, draft_vocabulary=draft_vocabulary)


@pytest.mark.parametrize("output_gated", [True, False])
@pytest.mark.parametrize("kv_cache_dtype,kv_encoding", [("artifact", 0), ("fp16", 1)])
def test_artifact_provider_equals_the_staged_one(device, tmp_path, output_gated,
                                                 kv_cache_dtype, kv_encoding):
    rng, model = tiny_model(61, output_gated)
    root = str(tmp_path / "artifact")
    aw.write_artifact(root, model, draft_vocabulary=128, max_context=4096)
    loaded = qp.Provider.from_artifact(
        root, geometry_of(model, 256, kv_encoding=kv_encoding), max_context=256,
        kv_page_tokens=64, kv_cache_dtype=kv_cache_dtype)
    staged = step_oracle.build_provider(model, qp, kv_encoding=kv_encoding, mtp=True,
                                        draft_vocabulary=128)
    assert loaded.telemetry("provider_weight_bytes") == staged.telemetry("provider_weight_bytes")
    tokens = rng.integers(0, model.vocabulary, 5).astype(np.uint32)
    streams = []
    for provider in (loaded, staged):
        provider.run_target(tokens, 0)
        logits, hidden = provider.logits(5).copy(), provider.hidden(5).copy()
        provider.begin_request(temperature_ppm=0)
        position, token = 5, 9
        provider.synchronize(token, position)
        stream = [provider.drafts()]
        for _ in range(4):
            emitted, token, advanced = provider.verify(token, position, 200)
            position += advanced
            stream.append((emitted, token, provider.drafts()))
        streams.append((logits, hidden, stream))
        provider.close()
    assert np.array_equal(streams[0][0], streams[1][0])
    assert np.array_equal(streams[0][1], streams[1][1])
    assert streams[0][2] == streams[1][2]


def test_draft_depth_and_context_come_from_the_artifact(device, tmp_path):
    rng, model = tiny_model(67)
    root = str(tmp_path / "artifact")
    aw.write_artifact(root, model, draft_vocabulary=128, max_context=512)
    # depth 2 applied to the program at load; context defaults to the artifact's
    provider = qp.Provider.from_artifact(root, geometry_of(model, 512, draft_depth=2),
                                         kv_page_tokens=64, mtp_draft_depth=2)
    provider.run_target(rng.integers(0, model.vocabulary, 3).astype(np.uint32), 0)
    provider.begin_request(temperature_ppm=0)
    provider.synchronize(4, 3)
    assert len(provider.drafts()) == 2
    emitted, token, advanced = provider.verify(4, 3, 500)
    assert 1 <= advanced <= 3 and emitted[0] == 4
    provider.close()
    with pytest.raises(qp.ProviderError, match="exceeds the artifact's maximum"):
        qp.Provider.from_artifact(root, geometry_of(model, 1024), max_context=1024)


def test_unsupported_artifacts_name_the_reason(device, tmp_path):
    rng, model = tiny_model(71)
    tensors = {}
    text = aw.dense_program(model, tensors, draft_vocabulary=128)
    # a recurrent layer in the layer program is outside this provider
    recurrent = text.replace(
        "layer\t1\tblock.full-attention.output-gated.v1",
        "layer\t1\tblock.recurrent-linear-attention.split-gated-delta.v1").replace(
        "kernel\tblock.full-attention.output-gated.v1\t1\n",
        "kernel\tblock.full-attention.output-gated.v1\t1\n"
        "kernel\tblock.recurrent-linear-attention.split-gated-delta.v1\t1\n")
    root = str(tmp_path / "recurrent")
    aw.write_artifact(root, model, program_text=recurrent)
    with pytest.raises(qp.ProviderError, match="full-attention layers only"):
        qp.Provider.from_artifact(root, geometry_of(model, 256), max_context=256)
    # a tensor the program names but the pack does not hold
    missing = text.replace("operation_tensor\t1\tinput_norm\tmodel.layers.0.input_layernorm.weight",
                           "operation_tensor\t1\tinput_norm\tmodel.layers.0.absent.weight")
    root = str(tmp_path / "missing")
    aw.write_artifact(root, model, program_text=missing)
    with pytest.raises(qp.ProviderError, match="absent from the dense index"):
        qp.Provider.from_artifact(root, geometry_of(model, 256), max_context=256)
