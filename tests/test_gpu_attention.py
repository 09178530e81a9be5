"""Q4H decode attention (split + combine) and the K/V store on the GPU,
through the C ABI, against the CPU oracle."""
import numpy as np
import pytest
import torch

import gpu_util as gu
import oracle_lib as ol
import qllm_hip as qh
import synth

pytestmark = pytest.mark.gpu


def run_case(device, rng, tokens, rows, Q, KV, d, page_tokens, split_tokens, gated,
             scale=1.0, layers=1, layer=0):
    first = tokens - (rows - 1)
    keys = (scale * rng.standard_normal((tokens, KV, d))).astype(np.float32)
    values = (scale * rng.standard_normal((tokens, KV, d))).astype(np.float32)
    pages = synth.q4h_pages(keys, values, page_tokens, layers, layer)
    stride = d * (2 if gated else 1)
    query = ol.bf16_round((scale * rng.standard_normal((rows, Q, stride))
                           ).astype(np.float32))
    shape = ol.AttentionShape(rows, Q, KV, d, first, page_tokens, layer, int(gated))
    want = ol.attention_q4h(shape, query, pages, "f64")
    got = gu.q4h_attention(device, pages, query, rows, Q, KV, d, first, page_tokens,
                           split_tokens, gated, layer)
    return got, want, (shape, query, pages)


@pytest.mark.parametrize("tokens,rows,Q,KV,d,page,split,gated", [
    (5, 5, 8, 2, 128, 64, 512, False),        # context of the rows alone
    (12, 5, 8, 1, 128, 64, 64, False),
    (100, 5, 64, 8, 128, 256, 64, False),     # several splits, 64Q/8KV heads
    (1000, 5, 64, 8, 128, 256, 256, False),
    (700, 5, 24, 4, 256, 256, 512, True),     # reference geometry, gated
    (3000, 1, 64, 8, 128, 256, 1024, False),  # single-row decode
    (257, 3, 16, 8, 128, 64, 128, True),
    (4100, 5, 64, 8, 128, 256, 512, False),
    # split 0: tiles dealt evenly over 32 workgroups per KV head
    (5, 5, 8, 2, 128, 64, 0, False),          # most waves have no tile at all
    (100, 5, 64, 8, 128, 256, 0, False),
    (4100, 5, 64, 8, 128, 256, 0, False),
    (20000, 5, 64, 8, 128, 256, 0, False),    # 2-3 tiles per wave
    (1500, 4, 24, 4, 256, 256, 0, True)])
def test_attention_matches_oracle(device, tokens, rows, Q, KV, d, page, split, gated):
    rng = np.random.default_rng(tokens + 7 * rows + Q)
    got, want, _ = run_case(device, rng, tokens, rows, Q, KV, d, page, split, gated)
    gu.assert_close(got, want, what="attention")


def test_attention_sharp_softmax_and_nonzero_layer(device):
    rng = np.random.default_rng(5)
    got, want, _ = run_case(device, rng, 200, 5, 8, 2, 128, 64, 512, False,
                            scale=2.4, layers=3, layer=2)
    gu.assert_close(got, want, what="attention, |q|,|k| ~ 2.4")


def test_reference_arithmetic_is_within_its_own_error(device):
    """The reference's production statement (Q8 query, int8 probabilities) is
    itself ~1e-2 away from exact attention on N(0,1) inputs; the kernel stays
    closer to the exact result than that statement does."""
    rng = np.random.default_rng(6)
    got, want, (shape, query, pages) = run_case(device, rng, 300, 5, 8, 1, 128, 64,
                                                512, False)
    reference_form = ol.attention_q4h(shape, query, pages, "int8")
    assert np.abs(got - want).max() < np.abs(reference_form - want).max()
    assert np.abs(got - reference_form).max() < 2e-2


def test_attention_is_split_invariant_at_32k(device):
    """Benchmark attention shape (5 rows, 64Q/8KV, d=128, L=32768): the result
    must not depend on the split size, and the causal rows must differ."""
    rng = np.random.default_rng(7)
    tokens, rows, Q, KV, d, page = 32768, 5, 64, 8, 128, 256
    keys = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    values = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    pages = synth.q4h_pages(keys, values, page)
    query = ol.bf16_round(rng.standard_normal((rows, Q, d)).astype(np.float32))
    first = tokens - 4
    results = [gu.q4h_attention(device, pages, query, rows, Q, KV, d, first, page,
                                split, False) for split in (1024, 4096, 32768, 0)]
    for other in results[1:]:
        assert np.abs(other - results[0]).max() < 2e-5
    # oracle on two KV heads' worth of query heads (full double precision)
    shape = ol.AttentionShape(rows, Q, KV, d, first, page, 0, 0)
    want = ol.attention_q4h(shape, query, pages, "f64")
    gu.assert_close(results[0], want, what="32K attention")


def test_kv_store_is_byte_exact(device):
    """Layout + encoding gate of the reference: 0 byte difference
    (runtime/tools/dense_fp4_cuda_smoke.cpp:4799)."""
    rng = np.random.default_rng(8)
    rows, KV, d, page_tokens, layers, layer, first = 70, 4, 256, 32, 2, 1, 5
    keys = (rng.standard_normal((rows, KV, d)) * 10.0 ** rng.integers(-2, 2, (rows, KV, 1))
            ).astype(np.float32)
    values = rng.standard_normal((rows, KV, d)).astype(np.float32)
    keys[3] = 0.0                                     # zero vector: scale floor
    layer_bytes = ol.q4h_layer_bytes(page_tokens, KV, d)
    n_pages = (first + rows + page_tokens - 1) // page_tokens
    want = [np.zeros(layer_bytes * layers, dtype=np.uint8) for _ in range(n_pages)]
    for r in range(rows):
        for h in range(KV):
            ol.q4h_store(want[(first + r) // page_tokens], layer, page_tokens,
                         first + r, h, KV, d, keys[r, h], values[r, h])
    d_pages = [torch.zeros(layer_bytes * layers, dtype=torch.uint8, device=device)
               for _ in range(n_pages)]
    table = torch.tensor([p.data_ptr() for p in d_pages], dtype=torch.int64,
                         device=device)
    d_keys, d_values = gu.device_tensor(keys, device), gu.device_tensor(values, device)
    qh.call("qllm_store_kv_paged_q4h_batch", qh.ptr(d_keys), qh.ptr(d_values),
            qh.ptr(table), layer, page_tokens, first, rows, KV, d, None)
    torch.cuda.synchronize()
    for got, expect in zip(d_pages, want):
        assert np.array_equal(got.cpu().numpy(), expect)


@pytest.mark.parametrize("gated,qk_norm,rotary", [(False, False, 128), (True, True, 64)])
def test_qkv_rope_cache_matches_oracle(device, gated, qk_norm, rotary):
    rng = np.random.default_rng(9)
    rows, Q, KV, d, page_tokens, first, layer = 5, 8, 2, 128, 64, 61, 1
    stride = d * (2 if gated else 1)
    q = rng.standard_normal((rows, Q, stride)).astype(np.float32)
    k = rng.standard_normal((rows, KV, d)).astype(np.float32)
    v = rng.standard_normal((rows, KV, d)).astype(np.float32)
    qw = (0.1 * rng.standard_normal(d)).astype(np.float32) if qk_norm else None
    kw = (0.1 * rng.standard_normal(d)).astype(np.float32) if qk_norm else None
    layer_bytes = ol.q4h_layer_bytes(page_tokens, KV, d)
    want_pages = [np.zeros(layer_bytes * 2, dtype=np.uint8) for _ in range(2)]
    want_q, want_k = q.copy(), k.copy()
    for r in range(rows):
        for h in range(Q):
            want_q[r, h, :d] = ol.head_norm_rope(q[r, h, :d], qw, rotary, first + r,
                                                 1e-6, 1e6)
        for h in range(KV):
            want_k[r, h] = ol.head_norm_rope(k[r, h], kw, rotary, first + r, 1e-6, 1e6)
    d_q, d_k, d_v = (gu.device_tensor(x, device) for x in (q, k, v))
    d_pages = [torch.zeros(layer_bytes * 2, dtype=torch.uint8, device=device)
               for _ in range(2)]
    table = torch.tensor([p.data_ptr() for p in d_pages], dtype=torch.int64,
                         device=device)
    d_qw = None if qw is None else gu.device_tensor(qw, device)
    d_kw = None if kw is None else gu.device_tensor(kw, device)
    qh.call("qllm_qkv_rope_cache_paged_q4h_batch", qh.ptr(d_q), stride, qh.ptr(d_k),
            qh.ptr(d_v), qh.ptr(d_qw), qh.ptr(d_kw), qh.ptr(table), layer, page_tokens,
            first, first, rows, Q, KV, d, rotary, 1e-6, 1e6, 0, None)
    torch.cuda.synchronize()
    got_k = d_k.cpu().numpy()
    assert np.abs(d_q.cpu().numpy() - want_q).max() < 8e-3 * 1e-3 + 2e-5
    assert np.abs(got_k - want_k).max() < 2e-5
    if gated:   # the gate half is untouched
        assert np.array_equal(d_q.cpu().numpy()[..., d:], q[..., d:])
    # the stored records are the exact encoding of the K the kernel produced
    for r in range(rows):
        for h in range(KV):
            ol.q4h_store(want_pages[(first + r) // page_tokens], layer, page_tokens,
                         first + r, h, KV, d, got_k[r, h], v[r, h])
    for got, expect in zip(d_pages, want_pages):
        assert np.array_equal(got.cpu().numpy(), expect)


def test_attention_rejects_unsupported_geometry(device):
    q = torch.zeros((5, 80, 128), device=device)
    launch = qh.Q4hAttentionLaunch(qh.ptr(q), 0, 0, qh.ptr(q), qh.ptr(q), qh.ptr(q),
                                   qh.ptr(q), qh.ptr(q), 10, 5, 0, 64, 80, 8, 128, 64,
                                   1, 128, 0, 0, None)
    with pytest.raises(qh.QllmError) as error:   # 5 rows x 10 grouped heads > 48
        qh.call("qllm_attention_paged_q4h", launch)
    assert error.value.code == 4


@pytest.mark.parametrize("total,first,Q,KV,d,gated,batch", [
    (23, 300, 64, 8, 128, False, 5),     # last batch has 3 rows
    (40, 1, 8, 2, 256, True, 5),         # the prompt starts the cache; d = 256
    (64, 4000, 64, 8, 128, False, 6),    # six rows per batch (48 matrix rows)
    (7, 70, 16, 8, 128, False, 1)])      # one row per batch
@pytest.mark.parametrize("splits", [8, 1])   # 1: the combine's single-split form
def test_batched_launch_equals_one_launch_per_batch(device, total, first, Q, KV, d,
                                                     gated, batch, splits):
    """Prompt prefill attends `total` consecutive rows in one launch, in
    batches of `batch` rows that each see the cache up to their own rows: bit
    for bit what one launch per batch computes, and the oracle's attention."""
    rng = np.random.default_rng(total + first)
    page_tokens = 64
    tokens = first + total - 1
    keys = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    values = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    pages = synth.q4h_pages(keys, values, page_tokens, 1, 0)
    stride = d * (2 if gated else 1)
    query = ol.bf16_round(rng.standard_normal((total, Q, stride)).astype(np.float32))
    d_pages = [gu.device_tensor(page, device) for page in pages]
    table = torch.tensor([page.data_ptr() for page in d_pages], dtype=torch.int64,
                         device=device)
    d_query = gu.device_tensor(query, device)
    maxima = torch.zeros((total, splits, Q), device=device)
    sums = torch.zeros_like(maxima)
    outputs = torch.zeros((total, splits, Q, d), device=device)
    out = torch.zeros((total, Q, d), device=device)
    launch = qh.Q4hAttentionLaunch(
        qh.ptr(d_query), 0, 0, qh.ptr(table), qh.ptr(out), qh.ptr(maxima), qh.ptr(sums),
        qh.ptr(outputs), first, total, 0, page_tokens, Q, KV, d, 0, splits, stride,
        int(gated), qh.OUT_F32, None)
    qh.call("qllm_attention_paged_q4h_batched", launch, batch)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    for row in range(0, total, batch):
        rows = min(batch, total - row)
        single = gu.q4h_attention(device, pages, query[row:row + rows], rows, Q, KV, d,
                                  first + row, page_tokens, 0, gated, balanced_splits=splits)
        assert np.array_equal(got[row:row + rows], single), row
    shape = ol.AttentionShape(total, Q, KV, d, first, page_tokens, 0, int(gated))
    gu.assert_close(got, ol.attention_q4h(shape, query, pages, "f64"), what="batched attention")
    if total * (Q // KV) > (32 if d == 256 else 48):
        with pytest.raises(qh.QllmError, match="exceeds"):     # one batch of everything
            qh.call("qllm_attention_paged_q4h_batched", launch, total)


@pytest.mark.parametrize("total,first,Q,KV,gated,batch,splits", [
    (100, 300, 64, 8, False, 6, 1),      # 17 batches: three workgroup layers, the last part empty
    (100, 300, 64, 8, False, 6, 3),      # the tiles cut over three splits
    (55, 1, 16, 8, True, 5, 1),          # the prompt starts the cache; gated; small groups
    (20, 4000, 64, 8, False, 6, 5),      # fewer than eight batches
    (300, 70, 40, 8, False, 6, 2)])      # group of five: 30 of 48 matrix rows
def test_prompt_attention_equals_the_batched_launch(device, total, first, Q, KV, gated,
                                                    batch, splits):
    """Eight batches per workgroup on shared tiles: the oracle's attention, and
    the batched launch's result up to the rounding of the probabilities."""
    d, page_tokens = 128, (256 if total == 300 else 64)   # tiles inside and across pages
    rng = np.random.default_rng(total * 7 + first)
    tokens = first + total - 1
    keys = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    values = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    pages = synth.q4h_pages(keys, values, page_tokens, 1, 0)
    stride = d * (2 if gated else 1)
    query = ol.bf16_round(rng.standard_normal((total, Q, stride)).astype(np.float32))
    d_pages = [gu.device_tensor(page, device) for page in pages]
    table = torch.tensor([page.data_ptr() for page in d_pages], dtype=torch.int64,
                         device=device)
    d_query = gu.device_tensor(query, device)
    results = {}
    for name in ("qllm_attention_paged_q4h_prompt", "qllm_attention_paged_q4h_batched"):
        maxima = torch.zeros((total, splits, Q), device=device)
        sums = torch.zeros_like(maxima)
        outputs = torch.zeros((total, splits, Q, d), device=device)
        out = torch.full((total, Q, d), float("nan"), device=device)
        launch = qh.Q4hAttentionLaunch(
            qh.ptr(d_query), 0, 0, qh.ptr(table), qh.ptr(out), qh.ptr(maxima),
            qh.ptr(sums), qh.ptr(outputs), first, total, 0, page_tokens, Q, KV, d, 0,
            splits, stride, int(gated), qh.OUT_F32, None)
        qh.call(name, launch, batch)
        torch.cuda.synchronize()
        results[name] = out.cpu().numpy()
    got, batched = results.values()
    shape = ol.AttentionShape(total, Q, KV, d, first, page_tokens, 0, int(gated))
    gu.assert_close(got, ol.attention_q4h(shape, query, pages, "f64"), what="prompt attention")
    # (binary16 probabilities are rounded relative to each wave's running
    # maximum, which the two launches reach by different routes: a few 1e-4)
    gu.assert_close(got, batched, rtol=3e-3, atol=3e-4, what="prompt vs batched")
    bad = qh.Q4hAttentionLaunch(
        qh.ptr(d_query), 0, 0, qh.ptr(table), qh.ptr(out), qh.ptr(maxima), qh.ptr(sums),
        qh.ptr(outputs), first, total, 0, page_tokens, Q, KV, d, 64, splits, stride,
        int(gated), qh.OUT_F32, None)
    with pytest.raises(qh.QllmError, match="invalid Q4H prompt attention"):
        qh.call("qllm_attention_paged_q4h_prompt", bad, batch)   # fixed split_tokens


def test_attention_at_131072_tokens_on_one_kv_head(device):
    """The long-context benchmark shape cut down to one KV head and its eight
    query heads (the heads are independent, so this is one eighth of the full
    launch): against the oracle in double precision, and the same result for
    every context partition."""
    rng = np.random.default_rng(131072)
    tokens, rows, Q, KV, d, page = 131072, 5, 8, 1, 128, 256
    keys = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    values = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    pages = synth.q4h_pages(keys, values, page)
    query = ol.bf16_round(rng.standard_normal((rows, Q, d)).astype(np.float32))
    first = tokens - 4
    results = [gu.q4h_attention(device, pages, query, rows, Q, KV, d, first, page,
                                split, False) for split in (4096, 16384, 0)]
    for other in results[1:]:
        assert np.abs(other - results[0]).max() < 2e-5
    shape = ol.AttentionShape(rows, Q, KV, d, first, page, 0, 0)
    want = ol.attention_q4h(shape, query, pages, "f64")
    gu.assert_close(results[0], want, what="131072-token attention")
    # the rows are causal among themselves: each sees one token more
    assert all(np.abs(results[0][r] - results[0][r + 1]).max() > 0 for r in range(rows - 1))


def unpack_query_operands(planes, scales, rows, Q, KV, d):
    """The prepared operands of qllm_qkv_rope_cache_paged_q4h_prepared back as
    (high, low) int8 [rows, Q, d] and the scale per (row, head)."""
    group = Q // KV
    row_tiles = (rows * group + 15) // 16
    steps = d // 64
    planes = planes.reshape(KV, row_tiles, steps, 2, 64, 16).view(np.int8)
    scales = scales.reshape(KV, row_tiles * 16)
    high = np.zeros((rows, Q, d), dtype=np.int8)
    low = np.zeros_like(high)
    scale = np.zeros((rows, Q), dtype=np.float32)
    for row in range(rows):
        for head in range(Q):
            kv, m = head // group, row * group + head % group
            scale[row, head] = scales[kv, m]
            for index in range(d):
                within, j = index % 128, index % 16
                step = 2 * (index // 128) + (within % 32) // 16
                lane = 16 * (within // 32) + m % 16
                slot = (j & 8) + ((j & 1) << 2) + ((j & 7) >> 1)
                high[row, head, index] = planes[kv, m // 16, step, 0, lane, slot]
                low[row, head, index] = planes[kv, m // 16, step, 1, lane, slot]
    return high, low, scale


@pytest.mark.parametrize("tokens,rows,Q,KV,d,page,gated", [
    (1000, 5, 64, 8, 128, 256, False),
    (700, 4, 24, 4, 256, 256, True),
    (300, 1, 16, 8, 128, 64, False),
    (130, 3, 16, 2, 128, 64, True)])
def test_prepared_query_operands_give_the_same_attention(device, tokens, rows, Q, KV, d,
                                                         page, gated):
    """The rotary kernel's query operands are what the attention kernel would
    have built from the rotated queries itself: same bytes, same output."""
    rng = np.random.default_rng(tokens + Q)
    first = tokens - (rows - 1)           # context of the first row, new tokens included
    keys = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    values = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    pages = synth.q4h_pages(keys, values, page, 1, 0)
    stride = d * (2 if gated else 1)
    q = rng.standard_normal((rows, Q, stride)).astype(np.float32)
    q[1 % rows, 3] *= 37.0                # rows of very different magnitude
    k = rng.standard_normal((rows, KV, d)).astype(np.float32)
    v = rng.standard_normal((rows, KV, d)).astype(np.float32)
    d_pages = [gu.device_tensor(p, device) for p in pages]
    table = torch.tensor([p.data_ptr() for p in d_pages], dtype=torch.int64, device=device)
    d_q, d_k, d_v = (gu.device_tensor(x, device) for x in (q, k, v))
    operand_bytes = qh.call("qllm_q4h_query_operand_bytes", rows, Q, KV, d)
    group = Q // KV
    row_tiles = (rows * group + 15) // 16
    assert operand_bytes == KV * row_tiles * (d // 64) * 2048
    operands = torch.zeros(operand_bytes, dtype=torch.uint8, device=device)
    scales = torch.zeros(KV * row_tiles * 16, dtype=torch.float32, device=device)
    qh.call("qllm_qkv_rope_cache_paged_q4h_prepared", None, 0, qh.ptr(d_q), stride,
            qh.ptr(d_k), qh.ptr(d_v), None, None, qh.ptr(table), 0, page, first - 1,
            first - 1, None, rows, Q, KV, d, d, 1e-6, 1e6, 0, qh.ptr(operands),
            qh.ptr(scales), None)
    torch.cuda.synchronize()
    rotated = d_q.cpu().numpy()
    high, low, scale = unpack_query_operands(operands.cpu().numpy(), scales.cpu().numpy(),
                                             rows, Q, KV, d)
    # 15 bits of each row's largest magnitude, exactly as the kernel rounds
    largest = np.abs(rotated[..., :d]).max(axis=-1)
    step = np.maximum(largest * np.float32(1.0 / 16319.0), np.float32(2.0 ** -100))
    quantized = np.rint(rotated[..., :d] * (np.float32(1.0) / step)[..., None])
    quantized = np.clip(quantized, -16319, 16319).astype(np.int32)
    assert np.array_equal(128 * high.astype(np.int32) + low, quantized)
    assert low.min() >= -64 and low.max() <= 63 and np.abs(high).max() <= 127
    factor = np.float32(1.4426950408889634 / (16.0 * np.sqrt(np.float32(d))))
    assert np.allclose(scale, step * factor, rtol=1e-6, atol=0)

    def attend(prepared):
        splits = 32
        maxima = torch.zeros((rows, splits, Q), device=device)
        sums = torch.zeros_like(maxima)
        outputs = torch.zeros((rows, splits, Q, d), device=device)
        out = torch.zeros((rows, Q, d), device=device)
        launch = qh.Q4hAttentionLaunch(
            qh.ptr(d_q), qh.ptr(operands) if prepared else 0,
            qh.ptr(scales) if prepared else 0, qh.ptr(table), qh.ptr(out),
            qh.ptr(maxima), qh.ptr(sums), qh.ptr(outputs), first, rows, 0, page, Q, KV,
            d, 0, splits, stride, int(gated), qh.OUT_F32, None)
        qh.call("qllm_attention_paged_q4h", launch)
        torch.cuda.synchronize()
        return out.cpu().numpy()

    assert np.array_equal(attend(True), attend(False))


@pytest.mark.parametrize("tokens,rows,Q,KV,d,page,gated,qk_norm,rotary,splits", [
    (1000, 5, 64, 8, 128, 256, False, False, 128, 32),
    (5, 5, 8, 2, 128, 64, False, True, 128, 32),       # the batch is the whole context
    (66, 5, 16, 2, 128, 64, True, True, 64, 32),       # batch across a tile and page edge
    (258, 4, 24, 4, 256, 256, True, True, 64, 32),     # reference geometry, page edge
    (4100, 1, 64, 8, 128, 256, False, False, 128, 32),
    (20000, 5, 64, 8, 128, 256, False, True, 128, 32),
    (700, 6, 8, 8, 128, 64, False, False, 128, 4)])    # one query head per KV head
def test_fused_rotary_attention_equals_the_two_launches(device, tokens, rows, Q, KV, d, page,
                                                        gated, qk_norm, rotary, splits):
    """qllm_attention_paged_q4h_fused (rotary, K/V store and attention in one
    launch, cos/sin from qllm_rope_table) against the rotary kernel followed by
    the attention kernel: same output bits, same page bytes."""
    rng = np.random.default_rng(tokens + rows + Q)
    first = tokens - (rows - 1)
    keys = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    values = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    pages = synth.q4h_pages(keys, values, page, 2, 1)
    stride = d * (2 if gated else 1)
    q = rng.standard_normal((rows, Q, stride)).astype(np.float32)
    k = rng.standard_normal((rows, KV, d)).astype(np.float32)
    v = rng.standard_normal((rows, KV, d)).astype(np.float32)
    qw = (0.1 * rng.standard_normal(d)).astype(np.float32) if qk_norm else None
    kw = (0.1 * rng.standard_normal(d)).astype(np.float32) if qk_norm else None
    d_qw = None if qw is None else gu.device_tensor(qw, device)
    d_kw = None if kw is None else gu.device_tensor(kw, device)
    group = Q // KV
    row_tiles = (rows * group + 15) // 16
    results = []
    for fused in (False, True):
        d_pages = [gu.device_tensor(p, device) for p in pages]
        table = torch.tensor([p.data_ptr() for p in d_pages], dtype=torch.int64,
                             device=device)
        d_q, d_k, d_v = (gu.device_tensor(x, device) for x in (q, k, v))
        maxima = torch.zeros((rows, splits, Q), device=device)
        sums = torch.zeros_like(maxima)
        outputs = torch.zeros((rows, splits, Q, d), device=device)
        out = torch.zeros((rows, Q, d), device=device)
        operands = torch.zeros(KV * row_tiles * (d // 64) * 2048, dtype=torch.uint8,
                               device=device)
        scales = torch.zeros(KV * row_tiles * 16, dtype=torch.float32, device=device)
        launch = qh.Q4hAttentionLaunch(
            qh.ptr(d_q), 0 if fused else qh.ptr(operands), 0 if fused else qh.ptr(scales),
            qh.ptr(table), qh.ptr(out), qh.ptr(maxima), qh.ptr(sums), qh.ptr(outputs),
            first, rows, 1, page, Q, KV, d, 0, splits, stride, int(gated), qh.OUT_F32, None)
        if fused:
            cos_sin = torch.zeros((rows, rotary // 2, 2), device=device)
            qh.call("qllm_rope_table", qh.ptr(cos_sin), rows, rotary, first - 1, 1e6, 0,
                    None, None)
            rope = qh.Q4hFusedRope(qh.ptr(d_k), qh.ptr(d_v), qh.ptr(d_qw), qh.ptr(d_kw),
                                   qh.ptr(cos_sin), rotary, 1e-6, first - 1, 0)
            qh.call("qllm_attention_paged_q4h_fused", launch, rope)
        else:
            qh.call("qllm_qkv_rope_cache_paged_q4h_prepared", None, 0, qh.ptr(d_q), stride,
                    qh.ptr(d_k), qh.ptr(d_v), qh.ptr(d_qw), qh.ptr(d_kw), qh.ptr(table), 1,
                    page, first - 1, first - 1, None, rows, Q, KV, d, rotary, 1e-6, 1e6, 0,
                    qh.ptr(operands), qh.ptr(scales), None)
            qh.call("qllm_attention_paged_q4h", launch)
        torch.cuda.synchronize()
        results.append((out.cpu().numpy(), [p.cpu().numpy() for p in d_pages]))
    (plain, plain_pages), (fused, fused_pages) = results
    assert np.array_equal(plain, fused)
    for index, (a, b) in enumerate(zip(plain_pages, fused_pages)):
        assert np.array_equal(a, b), index
    assert not np.array_equal(plain_pages[-1], pages[-1])   # the batch was stored
