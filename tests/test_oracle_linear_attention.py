"""Pins the oracle's FP4 linear and attention statements: against independent
numpy float64 restatements built from library routines (table lookup + matmul,
scipy softmax), against the reference's closed-form smoke fixtures, and through
identities a wrong index or a dropped term would break."""
import numpy as np
import pytest
from scipy.special import softmax

import oracle_lib as ol
import synth


def test_fp4_linear_matches_numpy_matmul_both_schemes():
    rng = np.random.default_rng(0)
    for scheme in (ol.SCALE_UE8M0_BLOCK32, ol.SCALE_F16_BLOCK16):
        rows, padded, batch = 37, 96 if scheme == 1 else 128, 5
        codes, scales = synth.fp4_matrix(rng, rows, padded, scheme)
        act = ol.bf16_round(rng.standard_normal((batch, padded)).astype(np.float32))
        want = act.astype(np.float64) @ synth.dequantize(codes, scales, scheme).T
        got = ol.fp4_linear_f64(codes, scales, scheme, rows, padded, act)
        assert np.array_equal(got, want.astype(np.float32))


def test_block16_reduces_to_block32():
    """Equal power-of-two scales in adjacent 16-blocks == one UE8M0 block."""
    rng = np.random.default_rng(1)
    rows, padded = 16, 128
    codes = rng.integers(0, 256, (rows, padded // 2), dtype=np.uint8)
    exponents = rng.integers(120, 134, (rows, padded // 32))
    ue8m0 = exponents.astype(np.uint8)
    f16 = np.repeat(np.ldexp(1.0, exponents - 127), 2, axis=1).astype(np.float16
                                                                    ).view(np.uint16)
    act = ol.bf16_round(rng.standard_normal((3, padded)).astype(np.float32))
    a = ol.fp4_linear_f64(codes, ue8m0, 0, rows, padded, act)
    b = ol.fp4_linear_f64(codes, np.ascontiguousarray(f16), 1, rows, padded, act)
    assert np.array_equal(a, b)


def test_reference_dense_fixture_q8_and_bf16_forms_agree():
    """runtime/tools/dense_fp4_cuda_smoke.cpp:139-216: rows 67, cols 100 (pad
    128); the reference requires its kernels within 2e-4 of both expectations,
    so the integer statement and the closed form must agree on it."""
    rows, columns, padded, batch = 67, 100, 128, 9
    r = np.arange(rows)[:, None]
    blocks = np.arange(padded // 32)[None, :]
    scales = (124 + (r + blocks) % 7).astype(np.uint8)
    pair = np.arange(padded // 2)[None, :]
    low = (r + 3 * pair) % 16
    high = (5 * r + pair + 1) % 16
    codes = (low | (high << 4)).astype(np.uint8)
    x = (np.sin(np.arange(batch * columns, dtype=np.float32) * np.float32(0.071)) *
         np.float32(0.7)).astype(np.float32).reshape(batch, columns)
    q8, s = ol.quantize_q8_rows(x, padded)
    integer_form = ol.fp4_linear_block32_q8(codes, scales, rows, padded, q8, s)
    dequantised_act = (q8.astype(np.float32) * s[:, None]).astype(np.float32)
    closed_form = ol.fp4_linear_f64(codes, scales, 0, rows, padded, dequantised_act)
    assert np.abs(integer_form - closed_form).max() < 2e-4
    # the bf16 expectation of the same fixture: padded activations are zero
    padded_x = np.zeros((batch, padded), dtype=np.float32)
    padded_x[:, :columns] = ol.bf16_round(x)
    bf16_form = ol.fp4_linear_f64(codes, scales, 0, rows, padded, padded_x)
    want = padded_x.astype(np.float64) @ synth.dequantize(codes, scales, 0).T
    assert np.array_equal(bf16_form, want.astype(np.float32))
    # the two forms differ by at most the Q8 rounding of the activations:
    # |delta| <= (scale/2 + bf16 step) * sum_k |w_k|
    weights = np.abs(synth.dequantize(codes, scales, 0))[:, :columns].sum(1)
    bound = (0.5 * s[:, None] + 0.7 * 2.0 ** -8) * weights[None, :]
    assert np.all(np.abs(integer_form - bf16_form) <= bound)


def test_q8_linear_inner_sums_are_exact_integers():
    rng = np.random.default_rng(2)
    rows, padded = 8, 64
    codes = rng.integers(0, 256, (rows, padded // 2), dtype=np.uint8)
    scales = np.full((rows, padded // 32), 127, dtype=np.uint8)   # unit scales
    q8 = rng.integers(-127, 128, (2, padded), dtype=np.int8)
    out = ol.fp4_linear_block32_q8(codes, scales, rows, padded, q8,
                                   np.ones(2, dtype=np.float32))
    twice = 2.0 * synth.dequantize(codes, scales, 0)
    want = 0.5 * (q8.astype(np.float64) @ twice.T)
    assert np.array_equal(out.astype(np.float64), want)


def _dequantised_cache(pages, page_tokens, tokens, kv_heads, d, layer=0):
    keys = np.zeros((tokens, kv_heads, d), dtype=np.float64)
    values = np.zeros_like(keys)
    for t in range(tokens):
        for h in range(kv_heads):
            k, v = ol.q4h_load(pages[t // page_tokens], layer, page_tokens, t, h,
                               kv_heads, d)
            keys[t, h], values[t, h] = k, v
    return keys, values


def _textbook_attention(q, keys, values, first_context, group, gate=None):
    rows, heads, d = q.shape
    out = np.zeros((rows, heads, d))
    for r in range(rows):
        context = first_context + r
        for h in range(heads):
            kv = h // group
            scores = keys[:context, kv] @ q[r, h].astype(np.float64) / np.sqrt(d)
            out[r, h] = softmax(scores) @ values[:context, kv]
            if gate is not None:
                out[r, h] /= 1.0 + np.exp(-gate[r, h].astype(np.float64))
    return out


def test_q4h_attention_matches_textbook_softmax():
    rng = np.random.default_rng(3)
    rows, Q, KV, d, page_tokens, tokens = 5, 8, 2, 128, 64, 150
    keys = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    values = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    pages = synth.q4h_pages(keys, values, page_tokens)
    for gated in (False, True):
        stride = d * (2 if gated else 1)
        q = rng.standard_normal((rows, Q, stride)).astype(np.float32)
        shape = ol.AttentionShape(rows, Q, KV, d, tokens - 4, page_tokens, 0, int(gated))
        got = ol.attention_q4h(shape, q, pages, "f64")
        dk, dv = _dequantised_cache(pages, page_tokens, tokens, KV, d)
        want = _textbook_attention(q[..., :d], dk, dv, tokens - 4, Q // KV,
                                   q[..., d:] if gated else None)
        assert np.abs(got - want).max() < 1e-6


def test_causal_rule_row_sees_first_context_plus_row():
    """Changing a token at index first_context + r must change rows > r only."""
    rng = np.random.default_rng(4)
    rows, Q, KV, d, page_tokens, tokens = 5, 4, 1, 128, 64, 40
    keys = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    values = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    q = rng.standard_normal((rows, Q, d)).astype(np.float32)
    first = tokens - 4
    shape = ol.AttentionShape(rows, Q, KV, d, first, page_tokens, 0, 0)
    base = ol.attention_q4h(shape, q, synth.q4h_pages(keys, values, page_tokens), "f64")
    for r in range(rows - 1):
        changed_values = values.copy()
        changed_values[first + r] += 3.0
        out = ol.attention_q4h(shape, q, synth.q4h_pages(keys, changed_values,
                                                         page_tokens), "f64")
        assert np.array_equal(out[:r + 1], base[:r + 1])
        assert np.abs(out[r + 1:] - base[r + 1:]).max() > 1e-4


def test_reference_q4h_fixture_three_statements_agree():
    """Closed-form fixture of runtime/tools/dense_fp4_cuda_smoke.cpp:1601-1641
    (8 tokens, 24 Q / 4 KV heads, d 256, page 32, first_context 4, gated).  The
    reference requires its kernel within 2e-4 of the Q8/int8 statement and
    within 2e-3 of the float statement, so the two must agree within 2.2e-3,
    and the textbook result must be close to both."""
    stored, rows, first, Q, KV, d, page_tokens = 8, 5, 4, 24, 4, 256, 32
    index = np.arange(stored * KV * d, dtype=np.float32).reshape(stored, KV, d)
    dimension = np.arange(d, dtype=np.float32)
    keys = (np.sin((index + 11) * np.float32(0.013)) *
            (np.float32(0.08) + np.float32(0.006) * (dimension % 17))).astype(np.float32)
    values = (np.cos((index + 19) * np.float32(0.009)) *
              (np.float32(0.07) + np.float32(0.005) * (dimension % 23))).astype(np.float32)
    for token in range(stored):
        for head in range(KV):
            for block in range(d // 32):
                outlier = (token * 5 + head * 7 + block * 11 + 3) % 32
                sign = -1.0 if (token + head + block) & 1 else 1.0
                keys[token, head, block * 32 + outlier] = sign * (1.75 + 0.125 * (block + head))
    query = np.zeros((rows, Q, 2 * d), dtype=np.float32)
    for row in range(rows):
        for head in range(Q):
            base = (row * Q + head) * 2 * d
            dim = np.arange(d)
            query[row, head, :d] = (np.sin((base + dim + 1).astype(np.float32) * np.float32(0.005)) *
                                    (np.float32(0.11) + np.float32(0.002) * (dim % 13)))
            query[row, head, d:] = np.cos((row + head + dim + 1).astype(np.float32) *
                                          np.float32(0.017)) * np.float32(0.4)
    pages = synth.q4h_pages(keys, values, page_tokens)
    assert pages[0].size == page_tokens * KV * 2 * 130
    shape = ol.AttentionShape(rows, Q, KV, d, first, page_tokens, 0, 1)
    exact = ol.attention_q4h(shape, query, pages, "f64")
    integer = ol.attention_q4h(shape, query, pages, "int8")
    assert np.abs(exact - integer).max() < 2.2e-3
    dk, dv = _dequantised_cache(pages, page_tokens, stored, KV, d)
    want = _textbook_attention(query[..., :d], dk, dv, first, Q // KV, query[..., d:])
    assert np.abs(exact - want).max() < 1e-6


def test_f16_attention_reference_fixture():
    """host_fp16_attention_check, dense_fp4_cuda_smoke.cpp:3972-4006: rows 3,
    32 Q / 2 KV, d 32, page 4, first_context 5; threshold 5e-4 between the
    f16-probability statement and the textbook result."""
    rows, Q, KV, d, page_tokens, first, capacity = 3, 32, 2, 32, 4, 5, 8
    n = rows * Q * d * 2
    query = (np.sin(np.arange(1, n + 1, dtype=np.float32) * np.float32(0.013)) *
             np.float32(0.35)).reshape(rows, Q, 2 * d)
    cache = np.arange(capacity * KV * d, dtype=np.float32)
    keys = (np.cos((cache + 3) * np.float32(0.017)) * np.float32(0.4)).reshape(capacity, KV, d)
    values = (np.sin((cache + 5) * np.float32(0.019)) * np.float32(0.3)).reshape(capacity, KV, d)
    pages = synth.f16_pages(keys, values, page_tokens)
    shape = ol.AttentionShape(rows, Q, KV, d, first, page_tokens, 0, 1)
    exact = ol.attention_f16(shape, query, pages, False)
    rounded = ol.attention_f16(shape, query, pages, True)
    assert np.abs(exact - rounded).max() < 5e-4
    k16 = keys.astype(np.float16).astype(np.float64)
    v16 = values.astype(np.float16).astype(np.float64)
    want = _textbook_attention(query[..., :d], k16, v16, first, Q // KV, query[..., d:])
    assert np.abs(exact - want).max() < 1e-6


def test_split_combine_is_split_invariant():
    """The combine of per-split (max, sum, unnormalised out) partials equals the
    unsplit softmax for every split size (dense_fp4_cuda_smoke.cpp:4900-4908)."""
    rng = np.random.default_rng(6)
    rows, Q, KV, d, tokens = 3, 4, 2, 128, 90
    first = tokens - (rows - 1)
    keys = rng.standard_normal((tokens, KV, d))
    values = rng.standard_normal((tokens, KV, d))
    q = rng.standard_normal((rows, Q, d)).astype(np.float32)
    want = _textbook_attention(q, keys, values, first, Q // KV)
    for split_tokens in (16, 32, 64, 128):
        splits = (tokens + split_tokens - 1) // split_tokens
        maxima = np.full((rows, splits, Q), -np.inf, dtype=np.float32)
        sums = np.zeros((rows, splits, Q), dtype=np.float32)
        outs = np.zeros((rows, splits, Q, d), dtype=np.float32)
        for r in range(rows):
            context = first + r
            for s in range((context + split_tokens - 1) // split_tokens):
                lo, hi = s * split_tokens, min((s + 1) * split_tokens, context)
                for h in range(Q):
                    sc = keys[lo:hi, h // (Q // KV)] @ q[r, h].astype(np.float64) / np.sqrt(d)
                    m = sc.max()
                    p = np.exp(sc - m)
                    maxima[r, s, h], sums[r, s, h] = m, p.sum()
                    outs[r, s, h] = p @ values[lo:hi, h // (Q // KV)]
        out = np.zeros((rows, Q, d), dtype=np.float32)
        ol.oracle().qo_attention_combine(
            ol._p(maxima), ol._p(sums), ol._p(outs), None,
            ol.c_uint32(0), ol.c_uint32(rows), ol.c_uint32(Q), ol.c_uint32(d),
            ol.c_uint32(first), ol.c_uint32(split_tokens), ol.c_uint32(splits),
            ol._p(out))
        assert np.abs(out - want).max() < 2e-5


def test_rms_norm_and_rope_closed_forms():
    rng = np.random.default_rng(7)
    x = rng.standard_normal((3, 64)).astype(np.float32)
    w = rng.standard_normal(64).astype(np.float32)
    for zero_centered in (False, True):
        factor = 1.0 + w if zero_centered else w
        want = x / np.sqrt((x.astype(np.float64) ** 2).mean(1, keepdims=True) + 1e-5) * factor
        got = ol.rms_norm_rows(x, w, 1e-5, zero_centered)
        assert np.abs(got - want).max() < 1e-6
    # rotary: position 0 is the identity; rotation preserves pair norms; the
    # first rotary_dim dims follow (x*cos - x[i+half]*sin, x*cos + x[i-half]*sin)
    v = rng.standard_normal(128).astype(np.float32)
    assert np.allclose(ol.head_norm_rope(v, None, 128, 0, 1e-6, 1e6), v, atol=1e-7)
    for rotary_dim in (128, 64):
        out = ol.head_norm_rope(v, None, rotary_dim, 1234, 1e-6, 1e6)
        half = rotary_dim // 2
        i = np.arange(half)
        angle = 1234 * (1e6 ** (-2.0 * i / rotary_dim))
        want = v.astype(np.float64).copy()
        want[:half] = v[:half] * np.cos(angle) - v[half:rotary_dim] * np.sin(angle)
        want[half:rotary_dim] = v[half:rotary_dim] * np.cos(angle) + v[:half] * np.sin(angle)
        assert np.abs(out - want).max() < 1e-5
        assert np.array_equal(out[rotary_dim:], v[rotary_dim:])
    # per-head norm uses (1 + w)
    weight = rng.standard_normal(128).astype(np.float32) * 0.1
    normed = ol.head_norm_rope(v, weight, 128, 0, 1e-6, 1e6)
    want = v / np.sqrt((v.astype(np.float64) ** 2).mean() + 1e-6) * (1.0 + weight)
    assert np.abs(normed - want).max() < 1e-6


def test_silu_product_and_embedding():
    rng = np.random.default_rng(8)
    g = rng.standard_normal(100).astype(np.float32) * 4
    u = rng.standard_normal(100).astype(np.float32)
    want = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u
    assert np.abs(ol.silu_product(g, u) - want).max() < 1e-6
    rounded = ol.silu_product(g, u, True)
    assert np.array_equal(rounded, ol.bf16_round(rounded))
    for scheme in (0, 1):
        codes, scales = synth.fp4_matrix(rng, 50, 64, scheme)
        tokens = np.array([3, 49, 0, 3], dtype=np.uint32)
        got = ol.fp4_embedding(codes, scales, scheme, 64, 64, tokens)
        want = synth.dequantize(codes, scales, scheme)[tokens]
        assert np.array_equal(got, want.astype(np.float32))


@pytest.mark.skipif(ol.ref() is None or not hasattr(ol.ref(), "qref_fp4_swiglu"),
                    reason="oracle/_ref (built from the reference tree) is absent")
@pytest.mark.parametrize("bf16_intermediate", [False, True])
def test_q8_linear_matches_the_reference_cpu_executor(bf16_intermediate):
    """The reference's own all-core FP4 x Q8 SwiGLU executor
    (runtime/src/cpu/fp4_host_executor.cpp), compiled from its source, against
    the oracle's statement of the same three linears: Q8 rows -> gate/up ->
    silu(g)*u -> Q8 -> down."""
    rng = np.random.default_rng(21 + bf16_intermediate)
    hidden, intermediate, rows = 256, 448, 5
    scheme = ol.SCALE_UE8M0_BLOCK32
    gate = synth.fp4_matrix(rng, intermediate, hidden, scheme)
    up = synth.fp4_matrix(rng, intermediate, hidden, scheme)
    down = synth.fp4_matrix(rng, hidden, intermediate, scheme)
    x = rng.standard_normal((rows, hidden)).astype(np.float32)
    got, _ = ol.reference_fp4_swiglu(gate, up, down, hidden, intermediate, x,
                                     threads=3, bf16_intermediate=bf16_intermediate)
    q, s = ol.quantize_q8_rows(x, hidden)
    g = ol.fp4_linear_block32_q8(*gate, intermediate, hidden, q, s)
    u = ol.fp4_linear_block32_q8(*up, intermediate, hidden, q, s)
    act = (g / (1.0 + np.exp(-g.astype(np.float64)))).astype(np.float32) * u
    if bf16_intermediate:
        act = ol.bf16_round(act)
    q2, s2 = ol.quantize_q8_rows(act, intermediate)
    want = ol.fp4_linear_block32_q8(*down, hidden, intermediate, q2, s2)
    # identical integer block sums; F32 accumulation order and expf differ
    assert np.abs(got - want).max() <= 2e-4 * np.abs(want).max()
