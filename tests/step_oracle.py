"""CPU statement of one target pass + acceptance for a small dense decoder,
composed from the oracle's per-op functions in the order of the reference's
run_target (runtime/tools/dense_fp4_provider.cpp:8529-8635), run_full_attention
(:6892), run_ffn (:8250-8293) and run_head (:8393-8432).  Test infrastructure."""
from __future__ import annotations

import numpy as np

import oracle_lib as ol
import synth


class TinyModel:
    """Random-init dense decoder held as host tensors (row-major FP4)."""

    def __init__(self, rng, hidden, intermediate, layers, query_heads, kv_heads,
                 head_dim, vocabulary, scheme, output_gated=False, qk_norm=False,
                 zero_centered=False, rotary_dim=None, rope_theta=1.0e6,
                 eps=1.0e-6, weight_scale=0.05):
        self.hidden, self.intermediate, self.layers = hidden, intermediate, layers
        self.query_heads, self.kv_heads, self.head_dim = query_heads, kv_heads, head_dim
        self.vocabulary, self.scheme = vocabulary, scheme
        self.output_gated, self.qk_norm, self.zero_centered = output_gated, qk_norm, zero_centered
        self.rotary_dim = rotary_dim or head_dim
        self.rope_theta, self.eps = rope_theta, eps
        q_rows = query_heads * head_dim * (2 if output_gated else 1)

        def matrix(rows, columns, gain=1.0):
            # weights ~ gain / sqrt(columns) in RMS, so every block's output is
            # comparable to the residual stream (a well-conditioned decoder)
            codes = rng.integers(0, 256, size=(rows, columns // 2), dtype=np.uint8)
            target = gain / (2.93 * np.sqrt(columns))
            if scheme == ol.SCALE_F16_BLOCK16:
                scales = (target * np.exp(0.5 * rng.standard_normal(
                    (rows, columns // 16)))).astype(np.float16).view(np.uint16)
            else:
                base = int(np.round(np.log2(target)))
                scales = (127 + base + rng.integers(
                    -1, 2, size=(rows, columns // 32))).astype(np.uint8)
            return codes, scales

        def norm(n):
            base = 0.0 if zero_centered else 1.0
            return (base + 0.1 * rng.standard_normal(n)).astype(np.float32)

        self.embedding = matrix(vocabulary, hidden, gain=np.sqrt(hidden))
        self.blocks = []
        for _ in range(layers):
            block = dict(
                input_norm=norm(hidden), post_attention_norm=norm(hidden),
                query=matrix(q_rows, hidden), key=matrix(kv_heads * head_dim, hidden),
                value=matrix(kv_heads * head_dim, hidden),
                output=matrix(hidden, query_heads * head_dim),
                gate=matrix(intermediate, hidden), up=matrix(intermediate, hidden),
                down=matrix(hidden, intermediate))
            if qk_norm:
                block["query_norm"] = (0.1 * rng.standard_normal(head_dim)).astype(np.float32)
                block["key_norm"] = (0.1 * rng.standard_normal(head_dim)).astype(np.float32)
            self.blocks.append(block)
        self.final_norm = norm(hidden)
        self.head = matrix(vocabulary, hidden)
        # the proposer: two input norms, fusion projection, one block, draft norm
        # (validate_exact, dense_fp4_provider.cpp:4730-4787)
        self.mtp = dict(
            embedding_norm=norm(hidden), hidden_norm=norm(hidden), draft_norm=norm(hidden),
            fusion=matrix(hidden, 2 * hidden),
            input_norm=norm(hidden), post_attention_norm=norm(hidden),
            query=matrix(q_rows, hidden), key=matrix(kv_heads * head_dim, hidden),
            value=matrix(kv_heads * head_dim, hidden),
            output=matrix(hidden, query_heads * head_dim),
            gate=matrix(intermediate, hidden), up=matrix(intermediate, hidden),
            down=matrix(hidden, intermediate))
        if qk_norm:
            self.mtp["query_norm"] = (0.1 * rng.standard_normal(head_dim)).astype(np.float32)
            self.mtp["key_norm"] = (0.1 * rng.standard_normal(head_dim)).astype(np.float32)

    # The artifact's activation contract (prepare_dense_activation,
    # dense_fp4_provider.cpp:5983-6003): False = bf16 activations into every
    # projection, True = per-row Q8 and the integer statement (block-32 UE8M0
    # weights only); intermediate activations then stay F32.
    activation_q8 = False

    def linear(self, m, x, rows):
        codes, scales = m
        padded = codes.shape[1] * 2
        if self.activation_q8:
            q8, act_scales = ol.quantize_q8_rows(x, padded)
            return ol.fp4_linear_block32_q8(codes, scales, rows, padded, q8, act_scales)
        return ol.fp4_linear_f64(codes, scales, self.scheme, rows, padded, x)

    def activations(self, x):
        """A projection's input as the contract has it: bf16-rounded, or F32
        (the Q8 quantisation is part of the projection)."""
        return np.asarray(x, dtype=np.float32) if self.activation_q8 else ol.bf16_round(x)


def _record_slices(model, layer, page_tokens, position, kv_head):
    """Byte ranges (K codes, K scale, V codes, V scale) of one Q4H record."""
    d, KV = model.head_dim, model.kv_heads
    records = page_tokens * KV
    base = layer * ol.q4h_layer_bytes(page_tokens, KV, d)
    record = kv_head * page_tokens + position % page_tokens
    key_codes = base + record * (d // 2)
    key_scale = base + records * (d // 2) + record * 2
    value_codes = base + records * (d // 2) + records * 2 + record * (d // 2)
    value_scale = base + 2 * records * (d // 2) + records * 2 + record * 2
    return [slice(key_codes, key_codes + d // 2), slice(key_scale, key_scale + 2),
            slice(value_codes, value_codes + d // 2),
            slice(value_scale, value_scale + 2)]


def _f16_store(page, layer, page_tokens, position, kv_head, kv_heads, d, key, value):
    """Exact-F16 page: per layer K [page_tokens][kv][d] then V, binary16."""
    halves = page.view(np.float16)
    page_values = page_tokens * kv_heads * d
    base = layer * 2 * page_values + ((position % page_tokens) * kv_heads + kv_head) * d
    halves[base: base + d] = key.astype(np.float16)
    halves[base + page_values: base + page_values + d] = value.astype(np.float16)


def run_target(model: TinyModel, tokens, first_position, kv_pages, page_tokens,
               observed_pages=None, report=None, kv_encoding=0):
    """Returns (logits [rows, V], hidden [rows, H]); writes K/V of the rows into
    kv_pages (list of uint8 arrays, all layers per page; Q4H records, or
    binary16 K/V planes when kv_encoding is 1).

    Q4H encoding is a discontinuous function of K/V: a last-bit difference in
    a projection can move a value across a rounding boundary and change a
    4-bit code.  When `observed_pages` (the pages of the implementation under
    test) is given, every record this pass writes is compared with the
    observed one - differing bytes are counted in report["record_byte_diffs"]
    - and the observed record is then adopted, so that the comparison of the
    downstream values is not dominated by such flips."""
    m = model
    rows = len(tokens)
    d, Q, KV = m.head_dim, m.query_heads, m.kv_heads
    stride = d * (2 if m.output_gated else 1)
    codes, scales = m.embedding
    hidden = ol.fp4_embedding(codes, scales, m.scheme, m.hidden, m.hidden, tokens)
    for layer, block in enumerate(m.blocks):
        x = ol.rms_norm_rows(hidden, block["input_norm"], m.eps, m.zero_centered,
                             not m.activation_q8)
        q = m.linear(block["query"], x, Q * stride).reshape(rows, Q, stride)
        k = m.linear(block["key"], x, KV * d).reshape(rows, KV, d)
        v = m.linear(block["value"], x, KV * d).reshape(rows, KV, d)
        for r in range(rows):
            position = first_position + r
            for h in range(Q):
                q[r, h, :d] = ol.head_norm_rope(
                    q[r, h, :d], block.get("query_norm"), m.rotary_dim, position,
                    m.eps, m.rope_theta)
            for h in range(KV):
                k[r, h] = ol.head_norm_rope(
                    k[r, h], block.get("key_norm"), m.rotary_dim, position,
                    m.eps, m.rope_theta)
                page = kv_pages[position // page_tokens]
                if kv_encoding == 1:
                    _f16_store(page, layer, page_tokens, position, h, KV, d,
                               k[r, h], v[r, h])
                    continue
                ol.q4h_store(page, layer, page_tokens, position, h, KV, d,
                             k[r, h], v[r, h])
                if observed_pages is not None:
                    observed = observed_pages[position // page_tokens]
                    for part in _record_slices(m, layer, page_tokens, position, h):
                        if report is not None:
                            report["record_bytes"] = report.get("record_bytes", 0) + (part.stop - part.start)
                            report["record_byte_diffs"] = report.get("record_byte_diffs", 0) + int((page[part] != observed[part]).sum())
                        page[part] = observed[part]
        shape = ol.AttentionShape(rows, Q, KV, d, first_position + 1, page_tokens,
                                  layer, int(m.output_gated))
        if kv_encoding == 1:
            attention = ol.attention_f16(shape, q, kv_pages, True)
        else:
            attention = ol.attention_q4h(shape, q, kv_pages, "f64")
        attention = m.activations(attention.reshape(rows, Q * d))
        hidden = hidden + m.linear(block["output"], attention, m.hidden)
        x = ol.rms_norm_rows(hidden, block["post_attention_norm"], m.eps,
                             m.zero_centered, not m.activation_q8)
        gate = m.linear(block["gate"], x, m.intermediate)
        up = m.linear(block["up"], x, m.intermediate)
        activation = ol.silu_product(gate, up, not m.activation_q8)
        hidden = hidden + m.linear(block["down"], activation, m.hidden)
    x = ol.rms_norm_rows(hidden, m.final_norm, m.eps, m.zero_centered,
                         not m.activation_q8)
    logits = m.linear(m.head, x, m.vocabulary)
    return logits, hidden


def run_mtp(model: TinyModel, tokens, previous_hidden, mtp_length, q8_pages,
            page_tokens, draft_vocabulary, observed_pages=None, page_offset=0,
            report=None):
    """One proposer pass (run_mtp, dense_fp4_provider.cpp:8681-8792).  Row r
    embeds tokens[r], takes previous_hidden[r], is cached at mtp_length + r and
    rotated at mtp_length + r + 1.  q8_pages: list of uint8 arrays holding the
    proposer's layer as reference records (oracle layout).  Returns (draft
    logits [draft_vocabulary] of the last row, final hidden [rows, H]).
    `observed_pages` (reference-record view of the implementation's pages) are
    adopted record by record after counting differing bytes, as in run_target."""
    m, w = model, model.mtp
    rows = len(tokens)
    d, Q, KV = m.head_dim, m.query_heads, m.kv_heads
    stride = d * (2 if m.output_gated else 1)
    codes, scales = m.embedding
    embedding = ol.fp4_embedding(codes, scales, m.scheme, m.hidden, m.hidden, tokens)
    rounded = not m.activation_q8
    fused = np.concatenate([
        ol.rms_norm_rows(embedding, w["embedding_norm"], m.eps, m.zero_centered, rounded),
        ol.rms_norm_rows(previous_hidden, w["hidden_norm"], m.eps, m.zero_centered,
                         rounded)],
        axis=1)
    hidden = m.linear(w["fusion"], fused, m.hidden)
    x = ol.rms_norm_rows(hidden, w["input_norm"], m.eps, m.zero_centered, rounded)
    q = m.linear(w["query"], x, Q * stride).reshape(rows, Q, stride)
    k = m.linear(w["key"], x, KV * d).reshape(rows, KV, d)
    v = m.linear(w["value"], x, KV * d).reshape(rows, KV, d)
    record_bytes = d + 2
    for r in range(rows):
        cache_position, rotary_position = mtp_length + r, mtp_length + r + 1
        for h in range(Q):
            q[r, h, :d] = ol.head_norm_rope(q[r, h, :d], w.get("query_norm"),
                                            m.rotary_dim, rotary_position, m.eps,
                                            m.rope_theta)
        for h in range(KV):
            k[r, h] = ol.head_norm_rope(k[r, h], w.get("key_norm"), m.rotary_dim,
                                        rotary_position, m.eps, m.rope_theta)
            page = q8_pages[cache_position // page_tokens]
            ol.q8_store(page, page_offset, page_tokens, cache_position, h, KV, d,
                        k[r, h], v[r, h])
            if observed_pages is not None:
                observed = observed_pages[cache_position // page_tokens]
                record = (cache_position % page_tokens) * KV + h
                for kind in range(2):
                    first = page_offset + (kind * page_tokens * KV + record) * record_bytes
                    part = slice(first, first + record_bytes)
                    if report is not None:
                        report["record_bytes"] = report.get("record_bytes", 0) + record_bytes
                        report["record_byte_diffs"] = report.get("record_byte_diffs", 0) + int((page[part] != observed[part]).sum())
                        # the same comparison on the dequantised values, relative
                        # to the record's largest magnitude
                        def decode(record):
                            scale = float(record[d:].view(np.float16)[0])
                            return record[:d].view(np.int8).astype(np.float64) * scale
                        mine, theirs = decode(page[part].copy()), decode(observed[part].copy())
                        report["value_error"] = max(
                            report.get("value_error", 0.0),
                            float(np.abs(mine - theirs).max() / max(np.abs(mine).max(), 1e-30)))
                    page[part] = observed[part]
    shape = ol.AttentionShape(rows, Q, KV, d, mtp_length + 1, page_tokens, 0,
                              int(m.output_gated))
    attention = ol.attention_q8(shape, q, q8_pages, page_offset)
    attention = m.activations(attention.reshape(rows, Q * d))
    hidden = hidden + m.linear(w["output"], attention, m.hidden)
    x = ol.rms_norm_rows(hidden, w["post_attention_norm"], m.eps, m.zero_centered,
                         rounded)
    activation = ol.silu_product(m.linear(w["gate"], x, m.intermediate),
                                 m.linear(w["up"], x, m.intermediate), rounded)
    hidden = hidden + m.linear(w["down"], activation, m.hidden)
    x = ol.rms_norm_rows(hidden[-1:], w["draft_norm"], m.eps, m.zero_centered, rounded)
    head_codes, head_scales = m.head
    logits = m.linear((head_codes[:draft_vocabulary], head_scales[:draft_vocabulary]), x,
                      draft_vocabulary)[0]
    return logits, hidden


def build_provider(model: TinyModel, qp, page_tokens=64, max_context=256,
                   kv_encoding=0, mtp=False, draft_vocabulary=0, prefill_chunk_rows=0):
    """Hands the host tensors to the provider operation by operation, the way
    the common VM calls prepare() in artifact order."""
    m = model
    provider = qp.Provider(
        hidden=m.hidden, intermediate=m.intermediate, layers=m.layers,
        query_heads=m.query_heads, kv_heads=m.kv_heads, head_dim=m.head_dim,
        rotary_dim=m.rotary_dim, vocabulary=m.vocabulary, rope_theta=m.rope_theta,
        norm_epsilon=m.eps, output_gated=int(m.output_gated), qk_norm=int(m.qk_norm),
        zero_centered_norm=int(m.zero_centered), scale_scheme=m.scheme,
        kv_encoding=kv_encoding, kv_page_tokens=page_tokens, max_context=max_context,
        draft_depth=4, mtp_layers=int(mtp), draft_vocabulary=draft_vocabulary,
        prefill_chunk_rows=prefill_chunk_rows, activation_q8=int(m.activation_q8))
    abi = 16 if m.scheme == ol.SCALE_F16_BLOCK16 else 3
    tag = "fp4-f16-block16" if m.scheme == ol.SCALE_F16_BLOCK16 else "fp4-block32"
    d, Q, KV, H, I, V = m.head_dim, m.query_heads, m.kv_heads, m.hidden, m.intermediate, m.vocabulary
    provider.stage_fp4("token_embedding", *m.embedding, V, H, abi)
    provider.prepare(f"embedding.lookup.{tag}.v1")
    for block in m.blocks:
        provider.stage_f32("input_norm", block["input_norm"])
        provider.stage_fp4("query_projection", *block["query"],
                           Q * d * (2 if m.output_gated else 1), H, abi)
        provider.stage_fp4("key_projection", *block["key"], KV * d, H, abi)
        provider.stage_fp4("value_projection", *block["value"], KV * d, H, abi)
        provider.stage_fp4("output_projection", *block["output"], H, Q * d, abi)
        if m.qk_norm:
            provider.stage_f32("query_norm", block["query_norm"])
            provider.stage_f32("key_norm", block["key_norm"])
        provider.prepare("block.full-attention.output-gated.v1" if m.output_gated
                         else "block.full-attention.standard-gqa.v1")
        provider.stage_f32("post_attention_norm", block["post_attention_norm"])
        provider.stage_fp4("gate_projection", *block["gate"], I, H, abi)
        provider.stage_fp4("up_projection", *block["up"], I, H, abi)
        provider.stage_fp4("down_projection", *block["down"], H, I, abi)
        provider.prepare(f"ffn.swiglu.dense.{tag}.v1")
    provider.stage_f32("hidden_norm", m.final_norm)
    provider.stage_fp4("output_head", *m.head, V, H, abi)
    provider.prepare(f"head.rmsnorm.token-select.{tag}.v1")
    if mtp:
        w = m.mtp
        for role in ("embedding_norm", "hidden_norm", "draft_norm"):
            provider.stage_f32(role, w[role])
        provider.stage_fp4("fusion_projection", *w["fusion"], H, 2 * H, abi)
        provider.stage_f32("layer.0.input_norm", w["input_norm"])
        provider.stage_fp4("layer.0.query_projection", *w["query"],
                           Q * d * (2 if m.output_gated else 1), H, abi)
        provider.stage_fp4("layer.0.key_projection", *w["key"], KV * d, H, abi)
        provider.stage_fp4("layer.0.value_projection", *w["value"], KV * d, H, abi)
        provider.stage_fp4("layer.0.output_projection", *w["output"], H, Q * d, abi)
        if m.qk_norm:
            provider.stage_f32("layer.0.query_norm", w["query_norm"])
            provider.stage_f32("layer.0.key_norm", w["key_norm"])
        provider.stage_f32("layer.0.post_attention_norm", w["post_attention_norm"])
        provider.stage_fp4("layer.0.gate_projection", *w["gate"], I, H, abi)
        provider.stage_fp4("layer.0.up_projection", *w["up"], I, H, abi)
        provider.stage_fp4("layer.0.down_projection", *w["down"], H, I, abi)
    provider.prepare_exact_decode(f"decode.mtp.dense-full-attention.{tag}.exact.v2")
    return provider
