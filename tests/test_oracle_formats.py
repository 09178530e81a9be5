"""Pins the oracle's number formats, FP4 decode, Q8 / Q4H quantisers and
token-selection rules against the reference's known answers and against
independent library routines (numpy float16, torch bfloat16)."""
import numpy as np
import torch

import oracle_lib as ol
import synth


def test_fp4_levels_and_nibble_order():
    # compiler/expert_pack/fp4_reference.py:12-29 (value table) and the byte
    # KATs of tests/compiler/test_fp4_quant.py:323-354
    levels = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    for code in range(16):
        expected = levels[code & 7] * (-1.0 if code & 8 else 1.0)
        assert ol.oracle().qo_fp4_value(code) == expected
        assert ol.oracle().qo_fp4_twice(code) == int(2 * expected)
    out = np.zeros(32, dtype=np.float64)
    payload = np.zeros(16, dtype=np.uint8)
    payload[0] = 0x02 | (0x0B << 4)   # values[0]=1.0, values[1]=-1.5
    payload[1] = 0x01 | (0x09 << 4)   # 0.5, -0.5
    payload[15] = 0x70                # values[31]=6.0
    scale = np.array([127], dtype=np.uint8)  # unit block scale
    ol.oracle().qo_fp4_decode_row(ol._p(payload), ol._p(scale), ol.c_int(0),
                                  ol.c_uint32(32), ol._p(out))
    assert out[0] == 1.0 and out[1] == -1.5 and out[2] == 0.5 and out[3] == -0.5
    assert out[30] == 0.0 and out[31] == 6.0


def test_ue8m0():
    f = ol.oracle().qo_ue8m0_value
    assert f(127) == 1.0 and f(128) == 2.0 and f(124) == 0.125
    assert f(254) == 2.0 ** 127
    assert f(0) == 2.0 ** -127      # transformer_kernels.cu:203-206
    assert f(1) == 2.0 ** -126


def test_f16_conversion_matches_numpy_everywhere():
    lib = ol.oracle()
    bits = np.arange(65536, dtype=np.uint16)
    expected = bits.view(np.float16).astype(np.float32)
    got = np.array([lib.qo_f16_value(int(b)) for b in bits], dtype=np.float32)
    finite = np.isfinite(expected)
    assert np.array_equal(got[finite], expected[finite])
    assert np.all(np.isnan(got[np.isnan(expected)]))
    rng = np.random.default_rng(0)
    values = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * 10.0 ** rng.integers(-9, 5, 20000),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, 2.0 ** -24, 2.0 ** -25,
                  2.0 ** -25 * 1.0000001, 2.0 ** -14, 6.1e-5, 5.96e-8, 3.0e-8],
                 dtype=np.float32)])
    with np.errstate(over="ignore"):
        want = values.astype(np.float16).view(np.uint16)
    have = np.array([lib.qo_f16_bits(float(v)) for v in values], dtype=np.uint16)
    assert np.array_equal(want, have)


def test_bf16_rounding_matches_torch():
    rng = np.random.default_rng(1)
    values = (rng.standard_normal(50000) * 10.0 ** rng.integers(-20, 20, 50000)
              ).astype(np.float32)
    want = torch.from_numpy(values).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(ol.bf16_round(values), want)
    got = np.array([ol.oracle().qo_bf16_round(float(v)) for v in values[:5000]],
                   dtype=np.float32)
    assert np.array_equal(got, want[:5000])


def test_q8_quantisation_known_answers():
    # rule of transformer_kernels.cu:912-946 / fp4_host_executor.cpp:141-152
    x = np.array([[0.0, 1.0, -2.0, 0.5, 1.27, -1.27 * 2, 0.0101]], dtype=np.float32)
    q, s = ol.quantize_q8_rows(x, 32)
    assert s[0] == np.float32(2.54) / np.float32(127.0)
    assert q[0, :7].tolist() == [0, 50, -100, 25, 64, -127, 1]   # 63.5 -> 64 (even)
    assert not q[0, 7:].any()
    q, s = ol.quantize_q8_rows(np.zeros((1, 5), dtype=np.float32), 32)
    assert s[0] == 1.0 and not q.any()
    # ties go to even: x/scale = 0.5 -> 0, 1.5 -> 2, 2.5 -> 2
    x = np.array([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5]], dtype=np.float32)
    q, s = ol.quantize_q8_rows(x, 32)
    assert s[0] == 1.0 and q[0, :6].tolist() == [127, 0, 2, 2, 0, -2]


def test_q4h_record_layout_and_encoding():
    # store_paged_kv_record<q4_per_head>, transformer_kernels.cu:251-288;
    # record size invariant d/2 + 2 bytes (dense_fp4_cuda_smoke.cpp:2531)
    page_tokens, kv_heads, d = 32, 4, 256
    assert ol.q4h_layer_bytes(page_tokens, kv_heads, d) == 32 * 4 * 2 * 130
    assert ol.q4h_layer_bytes(256, 8, 128) == 256 * 8 * 2 * 66
    page = np.zeros(ol.q4h_layer_bytes(page_tokens, kv_heads, d) * 2, dtype=np.uint8)
    key = np.zeros(d, dtype=np.float32)
    value = np.zeros(d, dtype=np.float32)
    key[0], key[1], key[2], key[3] = 7.0, -7.0, 3.49, 3.51      # scale exactly 1
    value[0], value[1], value[255] = 14.0, 1.0, -14.0           # scale exactly 2
    ol.q4h_store(page, 1, page_tokens, 32 + 5, 2, kv_heads, d, key, value)
    layer = ol.q4h_layer_bytes(page_tokens, kv_heads, d)
    records = page_tokens * kv_heads
    record = 2 * page_tokens + 5
    base = layer
    key_codes = page[base + record * 128: base + record * 128 + 128]
    assert key_codes[0] == (7 | (9 << 4))        # 7, -7 -> 0x9 in two's complement
    assert key_codes[1] == (3 | (4 << 4))        # rn(3.49)=3, rn(3.51)=4
    assert not key_codes[2:].any()
    key_scale = page[base + records * 128 + record * 2:][:2].view(np.uint16)[0]
    assert key_scale == np.float16(1.0).view(np.uint16)
    value_base = base + records * 128 + records * 2
    value_codes = page[value_base + record * 128: value_base + record * 128 + 128]
    assert value_codes[0] == (7 | (0 << 4))      # 14/2 = 7, rn(0.5) = 0 (even)
    assert value_codes[127] == (0 | (9 << 4))    # -7
    value_scale = page[value_base + records * 128 + record * 2:][:2].view(np.uint16)[0]
    assert value_scale == np.float16(2.0).view(np.uint16)
    assert not page[:layer].any()                # layer 0 untouched
    # zero vector: scale floors at 2^-24
    ol.q4h_store(page, 0, page_tokens, 0, 0, kv_heads, d, np.zeros(d, np.float32),
                 np.zeros(d, np.float32))
    assert page[records * 128: records * 128 + 2].view(np.uint16)[0] == 1
    k2, v2 = ol.q4h_load(page, 1, page_tokens, 37, 2, kv_heads, d)
    assert k2[0] == 7.0 and k2[1] == -7.0 and k2[2] == 3.0 and k2[3] == 4.0
    assert v2[0] == 14.0 and v2[255] == -14.0


def test_q4h_vectorised_encoder_matches_oracle_store():
    rng = np.random.default_rng(2)
    tokens, kv_heads, d, page_tokens = 70, 2, 128, 64
    keys = rng.standard_normal((tokens, kv_heads, d)).astype(np.float32)
    values = rng.standard_normal((tokens, kv_heads, d)).astype(np.float32)
    pages = synth.q4h_pages(keys, values, page_tokens, layers=2, layer=1)
    layer_bytes = ol.q4h_layer_bytes(page_tokens, kv_heads, d)
    expect = [np.zeros(layer_bytes * 2, dtype=np.uint8) for _ in range(2)]
    for t in range(tokens):
        for h in range(kv_heads):
            ol.q4h_store(expect[t // page_tokens], 1, page_tokens, t, h, kv_heads, d,
                         keys[t, h], values[t, h])
    for got, want in zip(pages, expect):
        assert np.array_equal(got, want)


def test_q4h_roundtrip_error_bound():
    rng = np.random.default_rng(3)
    d = 128
    page = np.zeros(ol.q4h_layer_bytes(64, 1, d), dtype=np.uint8)
    for trial in range(50):
        key = (rng.standard_normal(d) * 10.0 ** rng.integers(-3, 3)).astype(np.float32)
        value = rng.standard_normal(d).astype(np.float32)
        ol.q4h_store(page, 0, 64, trial, 0, 1, d, key, value)
        k2, v2 = ol.q4h_load(page, 0, 64, trial, 0, 1, d)
        for x, y in ((key, k2), (value, v2)):
            scale = float(np.float16(np.abs(x).max() / np.float32(7.0)))
            assert np.abs(x - y).max() <= 0.5 * scale * 1.001 + 7 * abs(
                scale - np.abs(x).max() / 7)


def test_argmax_and_topk_known_answers():
    nan = float("nan")
    # runtime/tools/dense_fp4_cuda_smoke.cpp:4313-4335
    logits = np.array([1.0, 7.0, nan, 7.0, -2.0, 4.5, 4.5, 9.0, 0.0], np.float32)
    values, indices = ol.topk(logits, 5)
    assert indices.tolist() == [7, 1, 3, 5, 6]
    assert values.tolist() == [9.0, 7.0, 7.0, 4.5, 4.5]
    assert ol.argmax(logits) == 7
    assert ol.argmax(np.array([nan, 2.0, 2.0], np.float32)) == 1   # tie -> lower
    assert ol.argmax(np.array([nan, nan], np.float32)) == 0xffffffff
    assert ol.argmax(np.array([-np.inf, -np.inf], np.float32)) == 0
    # :4337-4359, V = 248320 against a stable sort
    v = 248320
    i = np.arange(v, dtype=np.float32)
    big = (np.sin(i * np.float32(0.0137)) + np.float32(0.37) * np.cos(i * np.float32(0.0071))
           ).astype(np.float32)
    big[19] = 7.0
    big[127] = 7.0
    big[1021] = nan
    keyed = np.where(np.isnan(big), -np.inf, big).astype(np.float64)
    order = np.lexsort((np.arange(v), -keyed))
    order = order[~np.isnan(big[order])][:20]
    values, indices = ol.topk(big, 20)
    assert indices.tolist() == order.tolist()
    assert indices[:2].tolist() == [19, 127]


def test_presence_penalty_known_answer():
    # dense_fp4_cuda_smoke.cpp:4398-4412
    logits = np.array([3.0, 2.0, 1.0, -1.0], dtype=np.float32)
    emitted = np.array([0, 1, 1, 0], dtype=np.uint8)
    ol.oracle().qo_presence_penalty(ol._p(logits), ol._p(emitted), ol.c_uint32(4),
                                    ol.c_float(1.5))
    assert logits.tolist() == [3.0, 0.5, -0.5, -1.0]


def test_greedy_acceptance_rule():
    logits = np.full((5, 10), -1.0, dtype=np.float32)
    for row, token in enumerate([3, 4, 5, 6, 7]):
        logits[row, token] = 1.0
    assert ol.accept_greedy(logits, [3, 4, 5, 6]) == (4, 7)   # all accepted -> bonus
    assert ol.accept_greedy(logits, [3, 4, 9, 6]) == (2, 5)   # reject at depth 2
    assert ol.accept_greedy(logits, [0, 4, 5, 6]) == (0, 3)
