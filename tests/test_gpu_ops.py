"""Small per-row kernels and token selection on the GPU against the oracle."""
import numpy as np
import pytest
import torch

import gpu_util as gu
import oracle_lib as ol
import qllm_hip as qh
import synth

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("columns", [256, 252, 5120])
@pytest.mark.parametrize("scheme", [0, 1])
def test_embedding_is_exact(device, scheme, columns):
    # 252 columns in 256 padded ones takes the one-column-per-thread kernel,
    # the multiples of eight the eight-columns-per-thread one.
    rng = np.random.default_rng(scheme)
    V, H = 300, (columns + 31) // 32 * 32
    codes, scales = synth.fp4_matrix(rng, V, H, scheme)
    tokens = np.array([0, 5, 299, 17, 5], dtype=np.uint32)
    want = ol.fp4_embedding(codes, scales, scheme, columns, H, tokens)
    tensors = [gu.device_tensor(x, device) for x in (codes, scales, tokens)]
    out = torch.zeros((5, columns), device=device)
    qh.call("qllm_fp4_embedding_batch",
            qh.fp4_matrix(tensors[0], tensors[1], V, columns, H, scheme),
            qh.ptr(tensors[2]), qh.ptr(out), 5, None)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), want)


@pytest.mark.parametrize("zero_centered", [0, 1])
def test_rms_norm(device, zero_centered):
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((5, 5120)) * 3).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(5120)).astype(np.float32)
    d_x, d_w = gu.device_tensor(x, device), gu.device_tensor(w, device)
    out_f32 = torch.zeros((5, 5120), device=device)
    out_bf16 = torch.zeros((5, 5120), dtype=torch.bfloat16, device=device)
    qh.call("qllm_rms_norm_batch", qh.ptr(d_x), qh.ptr(d_w), qh.ptr(out_f32),
            qh.ptr(out_bf16), 5120, 5, 5120, 1e-6, zero_centered, None)
    torch.cuda.synchronize()
    want = ol.rms_norm_rows(x, w, 1e-6, bool(zero_centered))
    assert np.abs(out_f32.cpu().numpy() - want).max() < 2e-5   # reference: 2e-5
    assert np.array_equal(out_bf16.float().cpu().numpy(),
                          ol.bf16_round(out_f32.cpu().numpy()))


@pytest.mark.parametrize("elements", [5120, 256])
def test_rms_norm_concat_is_two_norms_side_by_side(device, elements):
    """[RMSNorm(a) | RMSNorm(b)] in one launch: each half within the reference's
    2e-5 of the oracle before the bf16 rounding, and bit-equal to the two-call
    form it stands in for."""
    rng = np.random.default_rng(7)
    a = (rng.standard_normal((5, elements)) * 2).astype(np.float32)
    b = rng.standard_normal((5, elements)).astype(np.float32)
    wa = (1 + 0.1 * rng.standard_normal(elements)).astype(np.float32)
    wb = (0.1 * rng.standard_normal(elements)).astype(np.float32)
    d = [gu.device_tensor(x, device) for x in (a, wa, b, wb)]
    out = torch.zeros((5, 2 * elements), dtype=torch.bfloat16, device=device)
    qh.call("qllm_rms_norm_concat_batch", qh.ptr(d[0]), qh.ptr(d[1]), qh.ptr(d[2]),
            qh.ptr(d[3]), qh.ptr(out), 5, elements, 1e-6, 1, None)
    halves = []
    for x, w in ((d[0], d[1]), (d[2], d[3])):
        single = torch.zeros((5, elements), dtype=torch.bfloat16, device=device)
        qh.call("qllm_rms_norm_batch", qh.ptr(x), qh.ptr(w), None, qh.ptr(single),
                elements, 5, elements, 1e-6, 1, None)
        halves.append(single)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    assert np.array_equal(got[:, :elements], halves[0].float().cpu().numpy())
    assert np.array_equal(got[:, elements:], halves[1].float().cpu().numpy())
    for half, (x, w) in enumerate(((a, wa), (b, wb))):
        want = ol.rms_norm_rows(x, w, 1e-6, True)
        piece = got[:, half * elements:(half + 1) * elements]
        # bf16 keeps 8 significant bits: half an ulp is 2^-9 of the value
        assert (np.abs(piece - want) <= np.abs(want) * 2.0 ** -8 + 2e-5).all()


def test_add_silu_and_bf16_convert(device):
    rng = np.random.default_rng(3)
    a = rng.standard_normal(3000).astype(np.float32) * 3
    b = rng.standard_normal(3000).astype(np.float32)
    d_a, d_b = gu.device_tensor(a, device), gu.device_tensor(b, device)
    out = torch.zeros(3000, device=device)
    for bf16 in (0, 1):
        qh.call("qllm_silu_product", qh.ptr(d_a), qh.ptr(d_b), qh.ptr(out), 3000, bf16,
                None)
        torch.cuda.synchronize()
        want = ol.silu_product(a, b, bool(bf16))
        gu.assert_close(out.cpu().numpy(), want, rtol=1e-5 if not bf16 else 8e-3,
                        atol=1e-6, what="silu")
    # bf16 mode rounding points of the reference (dense_fp4_cuda_smoke.cpp:4424+)
    qh.call("qllm_add_in_place", qh.ptr(d_a), qh.ptr(d_b), 3000, 1, None)
    torch.cuda.synchronize()
    assert np.array_equal(d_a.cpu().numpy(), ol.bf16_round(a + b))
    x = rng.standard_normal((2, 100)).astype(np.float32)
    d_x = gu.device_tensor(x, device)
    converted = torch.ones((2, 128), dtype=torch.bfloat16, device=device)
    qh.call("qllm_convert_f32_to_bf16_batch", qh.ptr(d_x), qh.ptr(converted),
            converted.numel() * 2, 2, 100, 128, None)
    torch.cuda.synchronize()
    host = converted.float().cpu().numpy()
    assert np.array_equal(host[:, :100], ol.bf16_round(x)) and not host[:, 100:].any()


@pytest.mark.parametrize("V", [151936, 151937, 65536])
def test_argmax_ties_nan_and_large_vocabulary(device, V):
    # an odd row length leaves every second row off the 16-byte alignment the
    # vector loads need, so both load paths and the ragged last chunk are hit
    nan = float("nan")
    rng = np.random.default_rng(4)
    logits = rng.standard_normal((5, V)).astype(np.float32)
    logits[0, 77] = logits[0, V - 1000] = 9.0        # tie -> lower index
    logits[1, :] = nan
    logits[1, 5000] = -3.0                           # NaN never wins
    logits[2, :] = -np.inf                           # all -inf -> index 0
    logits[3, V - 1] = 12.0
    d_logits = gu.device_tensor(logits, device)
    out = torch.zeros(5, dtype=torch.int32, device=device)
    size = qh.call("qllm_argmax_workspace_bytes", V, 5)
    workspace = torch.zeros(size, dtype=torch.uint8, device=device)
    qh.call("qllm_argmax_batch", qh.ptr(d_logits), V, 5, qh.ptr(out), qh.ptr(workspace),
            size, None)
    torch.cuda.synchronize()
    want = [ol.argmax(logits[r]) for r in range(5)]
    assert out.cpu().numpy().astype(np.uint32).tolist() == want
    assert want[:4] == [77, 5000, 0, V - 1]


def test_topk_known_answers(device):
    nan = float("nan")

    def run(values, k):
        d_values = gu.device_tensor(values, device)
        out_v = torch.zeros(k, device=device)
        out_i = torch.zeros(k, dtype=torch.int32, device=device)
        size = qh.call("qllm_topk_workspace_bytes", len(values), k)
        workspace = torch.zeros(size, dtype=torch.uint8, device=device)
        qh.call("qllm_topk_logits", qh.ptr(d_values), len(values), k, qh.ptr(out_v),
                qh.ptr(out_i), qh.ptr(workspace), size, None)
        torch.cuda.synchronize()
        return out_v.cpu().numpy(), out_i.cpu().numpy().astype(np.uint32)

    # runtime/tools/dense_fp4_cuda_smoke.cpp:4313-4335
    values, indices = run(np.array([1.0, 7.0, nan, 7.0, -2.0, 4.5, 4.5, 9.0, 0.0],
                                   np.float32), 5)
    assert indices.tolist() == [7, 1, 3, 5, 6]
    assert values.tolist() == [9.0, 7.0, 7.0, 4.5, 4.5]
    # :4337-4359
    v = 248320
    i = np.arange(v, dtype=np.float32)
    big = (np.sin(i * np.float32(0.0137)) + np.float32(0.37) * np.cos(i * np.float32(0.0071))
           ).astype(np.float32)
    big[19] = big[127] = 7.0
    big[1021] = nan
    values, indices = run(big, 20)
    want_v, want_i = ol.topk(big, 20)
    assert indices.tolist() == want_i.tolist() and np.array_equal(values, want_v)
    rng = np.random.default_rng(5)
    random_logits = rng.standard_normal(151936).astype(np.float32)
    values, indices = run(random_logits, 64)
    want_v, want_i = ol.topk(random_logits, 64)
    assert indices.tolist() == want_i.tolist() and np.array_equal(values, want_v)


def test_presence_penalty_known_answer(device):
    logits = gu.device_tensor(np.array([3.0, 2.0, 1.0, -1.0], np.float32), device)
    emitted = gu.device_tensor(np.array([0, 1, 1, 0], np.uint8), device)
    qh.call("qllm_apply_presence_penalty", qh.ptr(logits), qh.ptr(emitted), 4, 1.5, None)
    torch.cuda.synchronize()
    assert logits.cpu().numpy().tolist() == [3.0, 0.5, -0.5, -1.0]


def test_presence_penalty_over_the_rows_of_a_verify_step(device):
    """Row r is penalised at the emitted tokens and at the drafts of the rows
    before it; the oracle does it row by row, marking a draft in between."""
    rng = np.random.default_rng(8)
    V, stride, rows = 151936, 151936 + 64, 5
    logits = rng.standard_normal((rows, stride)).astype(np.float32)
    emitted = (rng.random(V) < 0.01).astype(np.uint8)
    drafts = np.array([17, 90000, 17, V - 1], dtype=np.uint32)   # a repeated draft
    want = logits.copy()
    present = emitted.copy()
    for row in range(rows):
        want[row, :V] = ol.presence_penalty(logits[row, :V], present, 1.5)
        if row < rows - 1:
            present[drafts[row]] = 1
    d_logits = gu.device_tensor(logits, device)
    d_emitted = gu.device_tensor(emitted, device)
    d_drafts = gu.device_tensor(drafts, device)
    qh.call("qllm_apply_presence_penalty_rows", qh.ptr(d_logits), stride,
            qh.ptr(d_emitted), qh.ptr(d_drafts), rows, V, 1.5, None)
    # marks: tokens on the device, entries outside the vocabulary ignored
    marks = gu.device_tensor(np.array([5, V - 1, 0xffffffff, 5], np.uint32), device)
    qh.call("qllm_mark_presence", qh.ptr(d_emitted), qh.ptr(marks), 4, V, None)
    torch.cuda.synchronize()
    assert np.array_equal(d_logits.cpu().numpy(), want)      # padding untouched too
    marked = emitted.copy()
    marked[[5, V - 1]] = 1
    assert np.array_equal(d_emitted.cpu().numpy(), marked)


def test_query_q8_quantisation_is_byte_exact(device):
    rng = np.random.default_rng(6)
    rows, Q, d = 5, 24, 256
    q = rng.standard_normal((rows, Q, 2 * d)).astype(np.float32)
    want_q8, want_scales = ol.quantize_queries_q8(q, rows, Q, d, 2 * d)
    d_q = gu.device_tensor(q, device)
    q8 = torch.zeros((rows, Q, d), dtype=torch.int8, device=device)
    scales = torch.zeros((rows, Q), device=device)
    qh.call("qllm_quantize_gqa_queries_q8", qh.ptr(d_q), 2 * d, qh.ptr(q8),
            qh.ptr(scales), rows, Q, d, None)
    torch.cuda.synchronize()
    assert np.array_equal(q8.cpu().numpy(), want_q8)
    assert np.array_equal(scales.cpu().numpy(), want_scales)


@pytest.mark.parametrize("elements,count", [(5120, 3), (256, 1), (16384, 16), (5124, 2)])
def test_rms_norm_residual_adds_partials_in_order(device, elements, count):
    """hidden += partial 0 + partial 1 + ... (that order, F32) and the RMSNorm
    of the sum in bf16: the sum bit for bit, the norm equal to the plain norm
    kernel's on the same sum and within the reference's 2e-5 of the oracle."""
    rng = np.random.default_rng(elements + count)
    rows = 5
    hidden = (rng.standard_normal((rows, elements)) * 2).astype(np.float32)
    partials = rng.standard_normal((count, rows, elements)).astype(np.float32)
    w = (0.1 * rng.standard_normal(elements)).astype(np.float32)
    d_hidden, d_partials, d_w = (gu.device_tensor(x, device) for x in (hidden, partials, w))
    out = torch.zeros((rows, elements), dtype=torch.bfloat16, device=device)
    qh.call("qllm_rms_norm_residual_batch", qh.ptr(d_hidden), qh.ptr(d_partials), count,
            qh.ptr(d_w), qh.ptr(out), rows, elements, 1e-6, 1, None)
    total = hidden.copy()
    for part in partials:
        total = total + part
    torch.cuda.synchronize()
    assert np.array_equal(d_hidden.cpu().numpy(), total)
    plain = torch.zeros((rows, elements), dtype=torch.bfloat16, device=device)
    qh.call("qllm_rms_norm_batch", qh.ptr(d_hidden), qh.ptr(d_w), None, qh.ptr(plain),
            elements, rows, elements, 1e-6, 1, None)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    assert np.array_equal(got, plain.float().cpu().numpy())
    want = ol.rms_norm_rows(total, w, 1e-6, True)
    assert (np.abs(got - want) <= np.abs(want) * 2.0 ** -8 + 2e-5).all()
    for bad_elements, bad_count in ((elements + 2, count), (16388, count), (elements, 0),
                                    (elements, 17)):
        with pytest.raises(qh.QllmError):
            qh.call("qllm_rms_norm_residual_batch", qh.ptr(d_hidden), qh.ptr(d_partials),
                    bad_count, qh.ptr(d_w), qh.ptr(out), rows, bad_elements, 1e-6, 1, None)


def batched_topk(device, rows_of_values, k, stride=None):
    values = np.stack(rows_of_values).astype(np.float32)
    rows, count = values.shape
    stride = stride or count
    padded = np.full((rows, stride), 1e30, dtype=np.float32)   # never read
    padded[:, :count] = values
    d_values = gu.device_tensor(padded, device)
    out_v = torch.zeros((rows, k), device=device)
    out_i = torch.zeros((rows, k), dtype=torch.int32, device=device)
    size = qh.call("qllm_topk_batch_workspace_bytes", count, k, rows)
    workspace = torch.zeros(max(size, 4), dtype=torch.uint8, device=device)
    qh.call("qllm_topk_logits_batch", qh.ptr(d_values), count, stride, k, rows,
            qh.ptr(out_v), qh.ptr(out_i), qh.ptr(workspace), size, None)
    torch.cuda.synchronize()
    return out_v.cpu().numpy(), out_i.cpu().numpy().astype(np.uint32)


def check_against_oracle(device, rows_of_values, k, stride=None):
    values, indices = batched_topk(device, rows_of_values, k, stride)
    for row, source in enumerate(rows_of_values):
        want_v, want_i = ol.topk(np.asarray(source, dtype=np.float32), k)
        assert indices[row].tolist() == want_i.tolist(), row
        assert np.array_equal(values[row], want_v), row


def test_batched_topk_equals_the_oracle_row_by_row(device):
    """Threshold selection for all rows of a batch: bit-equal to the exact
    descending top-k of the oracle (ties to the lower id, NaN excluded)."""
    nan = float("nan")
    # runtime/tools/dense_fp4_cuda_smoke.cpp:4313-4335
    check_against_oracle(device, [[1.0, 7.0, nan, 7.0, -2.0, 4.5, 4.5, 9.0, 0.0]], 5)
    # :4337-4359, beside three other rows of the same length
    v = 248320
    i = np.arange(v, dtype=np.float32)
    big = (np.sin(i * np.float32(0.0137)) + np.float32(0.37) * np.cos(i * np.float32(0.0071))
           ).astype(np.float32)
    big[19] = big[127] = 7.0
    big[1021] = nan
    rng = np.random.default_rng(5)
    check_against_oracle(device, [big, rng.standard_normal(v), -big, np.sort(big)], 20)
    # the verify step's shape: 5 rows of the vocabulary inside a wider buffer
    logits = [rng.standard_normal(151936) * 3 for _ in range(5)]
    logits[1][1000:1064] = 50.0            # 64 equal winners
    logits[2][::7] = nan
    logits[3][:] = np.round(logits[3])     # many ties at the threshold
    check_against_oracle(device, logits, 64, stride=151936 + 64)
    check_against_oracle(device, logits[:2], 1)
    # the draft vocabulary, a short row, fewer chunks than k
    check_against_oracle(device, [rng.standard_normal(65536)], 64)
    check_against_oracle(device, [rng.standard_normal(4097), rng.standard_normal(4097)], 64)
    check_against_oracle(device, [rng.standard_normal(300)], 64)


def test_batched_topk_when_the_threshold_does_not_filter(device):
    """Large values packed into few chunks, or all values equal: more items
    reach the threshold than the candidate list holds and the rows fall back
    to the k rounds; fewer valid items than k pad with (-inf, no index)."""
    rng = np.random.default_rng(6)
    flat = np.zeros(151936, dtype=np.float32)
    ramp = np.arange(151936, dtype=np.float32)          # the top k end the row
    plateau = rng.standard_normal(151936).astype(np.float32)
    plateau[plateau > -1.0] = 2.5                       # most items tie for first
    check_against_oracle(device, [flat, ramp, -ramp, plateau], 64)
    few = np.full(9000, np.nan, dtype=np.float32)
    few[[3, 4000, 8999]] = [1.0, -np.inf, 1.0]
    values, indices = batched_topk(device, [few], 8)
    assert indices[0].tolist() == [3, 8999, 4000] + [0xffffffff] * 5
    assert values[0][:3].tolist() == [1.0, 1.0, -np.inf] and np.all(np.isneginf(values[0][3:]))


def test_batched_topk_rejects_what_it_does_not_take(device):
    values = torch.zeros((2, 1000), device=device)
    out_v = torch.zeros((2, 64), device=device)
    out_i = torch.zeros((2, 64), dtype=torch.int32, device=device)
    workspace = torch.zeros(1 << 16, dtype=torch.uint8, device=device)
    for count, stride, k, rows, bytes_ in ((1000, 1000, 65, 2, 1 << 16), (1000, 999, 8, 2, 1 << 16),
                                           (1000, 1000, 0, 2, 1 << 16), (1000, 1000, 8, 0, 1 << 16),
                                           (1000, 1000, 8, 2, 8), (7, 1000, 8, 2, 1 << 16)):
        with pytest.raises(qh.QllmError):
            qh.call("qllm_topk_logits_batch", qh.ptr(values), count, stride, k, rows,
                    qh.ptr(out_v), qh.ptr(out_i), qh.ptr(workspace), bytes_, None)


@pytest.mark.parametrize("zero_centered", [False, True])
@pytest.mark.parametrize("rows,elements", [(5, 5120), (1, 256), (8, 16384), (3, 1000)])
def test_norm_into_q8_equals_norm_then_quantise(device, rows, elements, zero_centered):
    """qllm_rms_norm_q8_batch against qllm_rms_norm_batch + qllm_quantize_q8_batch
    (bit-equal: the same operations on the same values) and against the
    oracle's Q8 of the oracle's norm (the reference's quantiser is byte-exact
    on equal inputs; the norms agree to F32 rounding, so a code may differ by
    one step where a value sits on a rounding boundary)."""
    rng = np.random.default_rng(rows + elements)
    x = (2.0 * rng.standard_normal((rows, elements))).astype(np.float32)
    weight = (0.2 * rng.standard_normal(elements)).astype(np.float32)
    d_x, d_w = gu.device_tensor(x, device), gu.device_tensor(weight, device)
    fused_q8 = torch.zeros((rows, elements), dtype=torch.int8, device=device)
    fused_scales = torch.zeros(rows, device=device)
    qh.call("qllm_rms_norm_q8_batch", qh.ptr(d_x), qh.ptr(d_w), qh.ptr(fused_q8),
            qh.ptr(fused_scales), rows, elements, 1e-6, int(zero_centered), None)
    normed = torch.zeros((rows, elements), device=device)
    qh.call("qllm_rms_norm_batch", qh.ptr(d_x), qh.ptr(d_w), qh.ptr(normed), None, 0, rows,
            elements, 1e-6, int(zero_centered), None)
    two_q8 = torch.zeros((rows, elements), dtype=torch.int8, device=device)
    two_scales = torch.zeros(rows, device=device)
    qh.call("qllm_quantize_q8_batch", qh.ptr(normed), qh.ptr(two_q8), qh.ptr(two_scales),
            rows, elements, elements, 0, None)
    torch.cuda.synchronize()
    assert np.array_equal(fused_q8.cpu().numpy(), two_q8.cpu().numpy())
    assert np.array_equal(fused_scales.cpu().numpy(), two_scales.cpu().numpy())
    # the quantiser itself, byte-exact against the oracle on the GPU's own norm
    want_q8, want_scales = ol.quantize_q8_rows(normed.cpu().numpy(), elements)
    assert np.array_equal(two_q8.cpu().numpy(), want_q8)
    assert np.array_equal(two_scales.cpu().numpy(), want_scales)
    reference = ol.rms_norm_rows(x, weight, 1e-6, zero_centered, False)
    q8, _ = ol.quantize_q8_rows(reference, elements)
    assert np.abs(q8.astype(np.int32) - want_q8.astype(np.int32)).max() <= 1


@pytest.mark.parametrize("rows,columns,padded", [(5, 17408, 17408), (5, 8192, 8192),
                                                 (2, 20480, 20480), (3, 100, 128)])
def test_wide_rows_quantise_byte_exactly(device, rows, columns, padded):
    rng = np.random.default_rng(columns)
    x = (3.0 * rng.standard_normal((rows, columns))).astype(np.float32)
    x[0, 7] = 0.0
    d_x = gu.device_tensor(x, device)
    d_q8 = torch.full((rows, padded), 5, dtype=torch.int8, device=device)
    d_s = torch.zeros(rows, device=device)
    qh.call("qllm_quantize_q8_batch", qh.ptr(d_x), qh.ptr(d_q8), qh.ptr(d_s), rows, columns,
            padded, 0, None)
    torch.cuda.synchronize()
    want_q8, want_scales = ol.quantize_q8_rows(x, padded)
    assert np.array_equal(d_q8.cpu().numpy(), want_q8)
    assert np.array_equal(d_s.cpu().numpy(), want_scales)


@pytest.mark.parametrize("scheme", [0, 1])
@pytest.mark.parametrize("rows,elements", [(1, 5120), (5, 256), (8, 1024)])
def test_lookup_with_two_norms_equals_the_three_launches(device, scheme, rows, elements):
    """[RMSNorm(embedding[token]) | RMSNorm(hidden)] straight from the FP4
    table: bit-equal to qllm_fp4_embedding_batch followed by
    qllm_rms_norm_concat_batch, and the first half within the reference's 2e-5
    (plus the bf16 rounding) of the oracle's norm of the oracle's lookup."""
    rng = np.random.default_rng(scheme * 7 + rows)
    V = 300
    codes, scales = synth.fp4_matrix(rng, V, elements, scheme)
    tokens = rng.integers(0, V, rows).astype(np.uint32)
    tokens[0] = V - 1
    hidden = (rng.standard_normal((rows, elements)) * 2).astype(np.float32)
    wa = (0.1 * rng.standard_normal(elements)).astype(np.float32)
    wb = (0.1 * rng.standard_normal(elements)).astype(np.float32)
    d = [gu.device_tensor(x, device) for x in (codes, scales, tokens, hidden, wa, wb)]
    table = qh.fp4_matrix(d[0], d[1], V, elements, elements, scheme)
    fused = torch.zeros((rows, 2 * elements), dtype=torch.bfloat16, device=device)
    presence = torch.zeros(V, dtype=torch.uint8, device=device)
    qh.call("qllm_rms_norm_concat_embedding_batch", table, qh.ptr(d[2]), qh.ptr(d[4]),
            qh.ptr(d[3]), qh.ptr(d[5]), qh.ptr(fused), rows, 1e-6, 1, qh.ptr(presence),
            None)
    looked_up = torch.zeros((rows, elements), device=device)
    qh.call("qllm_fp4_embedding_batch", table, qh.ptr(d[2]), qh.ptr(looked_up), rows, None)
    apart = torch.zeros_like(fused)
    qh.call("qllm_rms_norm_concat_batch", qh.ptr(looked_up), qh.ptr(d[4]), qh.ptr(d[3]),
            qh.ptr(d[5]), qh.ptr(apart), rows, elements, 1e-6, 1, None)
    torch.cuda.synchronize()
    assert torch.equal(fused, apart)
    # the batch's tokens, and only they, are marked present
    marked = np.zeros(V, dtype=np.uint8)
    marked[tokens] = 1
    assert np.array_equal(presence.cpu().numpy(), marked)
    embedding = ol.fp4_embedding(codes, scales, scheme, elements, elements, tokens)
    want = ol.rms_norm_rows(embedding, wa, 1e-6, True)
    got = fused.float().cpu().numpy()[:, :elements]
    assert (np.abs(got - want) <= np.abs(want) * 2.0 ** -8 + 2e-5).all()
    # a tiled table, an out-of-range width and missing operands are turned down
    bad = qh.fp4_matrix(d[0], d[1], V, elements, elements, scheme)
    bad.layout = 1
    for arguments in ((bad, qh.ptr(d[2]), qh.ptr(d[4]), qh.ptr(d[3]), qh.ptr(d[5]),
                       qh.ptr(fused), rows, 1e-6, 1, None, None),
                      (table, None, qh.ptr(d[4]), qh.ptr(d[3]), qh.ptr(d[5]),
                       qh.ptr(fused), rows, 1e-6, 1, None, None),
                      (table, qh.ptr(d[2]), qh.ptr(d[4]), qh.ptr(d[3]), qh.ptr(d[5]),
                       qh.ptr(fused), 0, 1e-6, 1, None, None)):
        with pytest.raises(qh.QllmError):
            qh.call("qllm_rms_norm_concat_embedding_batch", *arguments)


def test_norm_of_partial_sums_with_and_without_a_residual(device):
    """qllm_rms_norm_partials_batch: the sum goes where it is told (in place, or
    elsewhere with the residual left alone, or from zero without a residual),
    bit-equal to qllm_rms_norm_residual_batch on the same operands."""
    rng = np.random.default_rng(12)
    rows, elements, count = 5, 5120, 3
    hidden = rng.standard_normal((rows, elements)).astype(np.float32)
    partials = rng.standard_normal((count, rows, elements)).astype(np.float32)
    weight = (0.1 * rng.standard_normal(elements)).astype(np.float32)
    d_partials, d_weight = gu.device_tensor(partials, device), gu.device_tensor(weight, device)

    def run(residual, separate_sum):
        d_residual = None if residual is None else gu.device_tensor(residual, device)
        d_sum = (torch.full((rows, elements), 7.0, device=device)
                 if separate_sum or d_residual is None else d_residual)
        out = torch.zeros((rows, elements), dtype=torch.bfloat16, device=device)
        qh.call("qllm_rms_norm_partials_batch", qh.ptr(d_residual), qh.ptr(d_sum),
                qh.ptr(d_partials), count, qh.ptr(d_weight), qh.ptr(out), rows, elements,
                1e-6, 1, None)
        torch.cuda.synchronize()
        return d_residual, d_sum.cpu().numpy(), out.float().cpu().numpy()

    reference = gu.device_tensor(hidden, device)
    want_out = torch.zeros((rows, elements), dtype=torch.bfloat16, device=device)
    qh.call("qllm_rms_norm_residual_batch", qh.ptr(reference), qh.ptr(d_partials), count,
            qh.ptr(d_weight), qh.ptr(want_out), rows, elements, 1e-6, 1, None)
    torch.cuda.synchronize()
    want_sum = reference.cpu().numpy()
    assert np.array_equal(want_sum, ((hidden + partials[0]) + partials[1]) + partials[2])
    for separate in (False, True):
        residual, got_sum, got_out = run(hidden, separate)
        assert np.array_equal(got_sum, want_sum)
        assert np.array_equal(got_out, want_out.float().cpu().numpy())
        if separate:
            assert np.array_equal(residual.cpu().numpy(), hidden)
    _, got_sum, got_out = run(None, True)
    want = (partials[0] + partials[1]) + partials[2]
    assert np.array_equal(got_sum, want)
    normed = ol.rms_norm_rows(want, weight, 1e-6, True)
    assert (np.abs(got_out - normed) <= np.abs(normed) * 2.0 ** -8 + 2e-5).all()
