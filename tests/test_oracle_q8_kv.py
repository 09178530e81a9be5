"""Pins the oracle's Q8 KV cache functions (the proposer's cache: int8 codes and
one binary16 scale per record) against the two fixtures the reference holds
for it, q8_kv_attention_check and q8_five_query_microbatch_check
(runtime/tools/dense_fp4_cuda_smoke.cpp:896-1177): record bytes must equal the
fixture's independent encoder exactly, and the attention must lie within the
fixture's 2e-3 of its bf16-rounded float statement (:4921-4926)."""
import numpy as np

import oracle_lib as ol


def _bf16(x):
    return ol.bf16_round(np.asarray(x, dtype=np.float32))


def _fixture_records(source, d):
    """Independent encoder of the fixture (:1061-1088): returns the record bytes
    [rows, d + 2] and the dequantised values."""
    source = np.asarray(source, dtype=np.float32).reshape(-1, d)
    records = np.zeros((source.shape[0], d + 2), dtype=np.uint8)
    decoded = np.zeros_like(source)
    for row, x in enumerate(source):
        maximum = np.float32(np.abs(x).max())
        scale16 = np.float16(max(maximum / np.float32(127.0), np.float32(2.0 ** -24)))
        scale = np.float32(scale16)
        codes = np.clip(np.rint(x / scale), -127, 127).astype(np.int8)
        records[row, :d] = codes.view(np.uint8)
        records[row, d:] = np.frombuffer(scale16.tobytes(), dtype=np.uint8)
        decoded[row] = codes.astype(np.float32) * scale
    return records, decoded


def _float_statement(query, keys, values, first_context, d, gated=True):
    """The fixture's expectation (:986-1024): q, k, v and the probabilities
    rounded to bf16, sums in float32."""
    rows, heads = query.shape[:2]
    out = np.zeros((rows, heads, d), dtype=np.float32)
    kb, vb = _bf16(keys), _bf16(values)
    for row in range(rows):
        visible = first_context + row
        for head in range(heads):
            q = _bf16(query[row, head, :d])
            scores = (kb[:visible] * q).sum(axis=1, dtype=np.float32) / np.float32(np.sqrt(d))
            p = _bf16(np.exp(scores - scores.max()))
            numerator = (p[:, None] * vb[:visible]).sum(axis=0, dtype=np.float32)
            result = numerator / p.sum(dtype=np.float32)
            if gated:
                result = result / (1.0 + np.exp(-query[row, head, d:]))
            out[row, head] = result
    return out


def test_q8_records_equal_the_fixture_encoder_byte_for_byte():
    # q8_kv_attention_check: 8 tokens, 1 KV head, d = 256, page of 8 tokens
    rows, d, page_tokens = 8, 256, 8
    index = np.arange(rows * d, dtype=np.float32)
    key = (np.sin((index + 11) * np.float32(0.019)) *
           (np.float32(0.2) + (np.arange(rows * d) % 13).astype(np.float32) * np.float32(0.017)))
    value = (np.cos((index + 17) * np.float32(0.023)) *
             (np.float32(0.15) + (np.arange(rows * d) % 7).astype(np.float32) * np.float32(0.013)))
    key, value = key.astype(np.float32), value.astype(np.float32)
    page = np.zeros(ol.q8_layer_bytes(page_tokens, 1, d), dtype=np.uint8)
    assert page.size == 2 * page_tokens * (d + 2)            # :1043-1046
    for token in range(rows):
        ol.q8_store(page, 0, page_tokens, token, 0, 1, d,
                    key[token * d:(token + 1) * d], value[token * d:(token + 1) * d])
    want_k, decoded_k = _fixture_records(key, d)
    want_v, decoded_v = _fixture_records(value, d)
    assert np.array_equal(page[:rows * (d + 2)].reshape(rows, d + 2), want_k)
    assert np.array_equal(page[rows * (d + 2):].reshape(rows, d + 2), want_v)
    for token in range(rows):
        k, v = ol.q8_load(page, 0, page_tokens, token, 0, 1, d)
        assert np.array_equal(k, decoded_k[token]) and np.array_equal(v, decoded_v[token])

    # decode attention of the same fixture (:1090-1167): one query row over the
    # 8 tokens, 8 query heads, gated
    heads = 8
    query = (np.sin((np.arange(2 * heads * d, dtype=np.float32) + 5) * np.float32(0.007)) *
             np.float32(0.4)).astype(np.float32).reshape(1, heads, 2 * d)
    shape = ol.AttentionShape(1, heads, 1, d, rows, page_tokens, 0, 1)
    got = ol.attention_q8(shape, query, [page])
    want = _float_statement(query, decoded_k, decoded_v, rows, d)
    assert np.abs(got - want).max() < 2e-3


def test_q8_five_query_fixture():
    # q8_five_query_microbatch_check (:896-1033): 16 tokens, rows 5, first
    # context 12, 6 query heads, 1 KV head, d = 256
    context, first, rows, heads, d = 16, 12, 5, 6, 256
    index = np.arange(context * d, dtype=np.float32)
    key = (np.sin((index + 31) * np.float32(0.013)) *
           (np.float32(0.19) + (np.arange(context * d) % 11).astype(np.float32) * np.float32(0.009)))
    value = (np.cos((index + 23) * np.float32(0.017)) *
             (np.float32(0.17) + (np.arange(context * d) % 9).astype(np.float32) * np.float32(0.011)))
    query = (np.sin((np.arange(rows * 2 * heads * d, dtype=np.float32) + 7) * np.float32(0.005)) *
             np.float32(0.37)).astype(np.float32).reshape(rows, heads, 2 * d)
    page = np.zeros(ol.q8_layer_bytes(context, 1, d), dtype=np.uint8)
    for token in range(context):
        ol.q8_store(page, 0, context, token, 0, 1, d,
                    key[token * d:(token + 1) * d].astype(np.float32),
                    value[token * d:(token + 1) * d].astype(np.float32))
    _, decoded_k = _fixture_records(key, d)
    _, decoded_v = _fixture_records(value, d)
    shape = ol.AttentionShape(rows, heads, 1, d, first, context, 0, 1)
    got = ol.attention_q8(shape, query, [page])
    want = _float_statement(query, decoded_k, decoded_v, first, d)
    assert np.abs(got - want).max() < 2e-3
    # causal rule: the rows differ, the last row sees every token
    assert np.abs(got[0] - got[-1]).max() > 1e-4


def test_q8_attention_is_textbook_softmax_on_the_dequantised_cache():
    """Several KV heads, several pages, a layer offset inside the page, no gate:
    against a numpy softmax on what q8_load returns."""
    rng = np.random.default_rng(8)
    tokens, rows, Q, KV, d, page_tokens = 70, 3, 8, 2, 128, 32
    offset = 4096
    layer_bytes = ol.q8_layer_bytes(page_tokens, KV, d)
    pages = [np.zeros(offset + layer_bytes, dtype=np.uint8) for _ in range(3)]
    keys = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    values = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    for token in range(tokens):
        for head in range(KV):
            ol.q8_store(pages[token // page_tokens], offset, page_tokens, token, head,
                        KV, d, keys[token, head], values[token, head])
    dk = np.zeros((tokens, KV, d)); dv = np.zeros((tokens, KV, d))
    for token in range(tokens):
        for head in range(KV):
            dk[token, head], dv[token, head] = ol.q8_load(
                pages[token // page_tokens], offset, page_tokens, token, head, KV, d)
    assert np.abs(dk - keys).max() <= np.abs(keys).max() / 127 * 0.51
    query = rng.standard_normal((rows, Q, d)).astype(np.float32)
    first = tokens - (rows - 1)
    shape = ol.AttentionShape(rows, Q, KV, d, first, page_tokens, 0, 0)
    got = ol.attention_q8(shape, query, pages, offset)
    for row in range(rows):
        visible = first + row
        for head in range(Q):
            kv = head // (Q // KV)
            scores = dk[:visible, kv] @ query[row, head].astype(np.float64) / np.sqrt(d)
            p = np.exp(scores - scores.max())
            want = p @ dv[:visible, kv] / p.sum()
            assert np.abs(got[row, head] - want).max() < 1e-6
