"""Exact-F16 paged decode attention and its K/V store on the GPU, through the
C ABI, against the CPU oracle."""
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
    pages = synth.f16_pages(keys, values, page_tokens, layers, layer)
    stride = d * (2 if gated else 1)
    query = (scale * rng.standard_normal((rows, Q, stride))).astype(np.float32)
    shape = ol.AttentionShape(rows, Q, KV, d, first, page_tokens, layer, int(gated))
    got = gu.f16_attention(device, pages, query, rows, Q, KV, d, first, page_tokens,
                           split_tokens, gated, layer)
    return got, shape, query, pages


@pytest.mark.parametrize("tokens,rows,Q,KV,d,page,split,gated", [
    (5, 5, 8, 2, 128, 32, 512, False),        # context of the rows alone
    (12, 5, 8, 1, 128, 64, 32, False),
    (100, 5, 64, 8, 128, 256, 64, False),     # several splits, 64Q/8KV heads
    (1000, 5, 64, 8, 128, 256, 256, False),
    (700, 5, 24, 4, 256, 256, 512, True),     # reference geometry, gated
    (3000, 1, 64, 8, 128, 256, 1024, False),  # single-row decode
    (257, 3, 16, 8, 128, 64, 128, True),
    (5, 5, 8, 2, 128, 64, 0, False),          # balanced: most waves idle
    (4100, 5, 64, 8, 128, 256, 0, False),
    (1500, 4, 24, 4, 256, 256, 0, True)])
def test_f16_attention_matches_oracle(device, tokens, rows, Q, KV, d, page, split,
                                      gated):
    """rtol 1e-2, atol 1e-3 (F32 accumulate) against the
    reference's arithmetic (binary16 query and probabilities) and against
    exact attention on the same binary16 cache."""
    rng = np.random.default_rng(tokens + 7 * rows + Q)
    got, shape, query, pages = run_case(device, rng, tokens, rows, Q, KV, d, page,
                                        split, gated)
    gu.assert_close(got, ol.attention_f16(shape, query, pages, True),
                    what="F16 attention (reference rounding points)")
    gu.assert_close(got, ol.attention_f16(shape, query, pages, False),
                    what="F16 attention (exact)")


def test_f16_attention_sharp_softmax_and_nonzero_layer(device):
    rng = np.random.default_rng(5)
    got, shape, query, pages = run_case(device, rng, 200, 5, 8, 2, 128, 64, 512,
                                        False, scale=2.4, layers=3, layer=2)
    gu.assert_close(got, ol.attention_f16(shape, query, pages, True),
                    what="F16 attention, |q|,|k| ~ 2.4")


def test_f16_attention_ignores_uninitialised_tail(device):
    """Records past the context (the rest of the last page) may hold any bit
    pattern, NaN included, without reaching the result."""
    rng = np.random.default_rng(6)
    tokens, rows, Q, KV, d, page = 70, 5, 8, 2, 128, 64
    first = tokens - (rows - 1)
    keys = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    values = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    pages = synth.f16_pages(keys, values, page)
    query = rng.standard_normal((rows, Q, d)).astype(np.float32)
    shape = ol.AttentionShape(rows, Q, KV, d, first, page, 0, 0)
    want = ol.attention_f16(shape, query, pages, True)
    poisoned = [p.copy() for p in pages]
    tail = poisoned[1].view(np.uint16).reshape(2, page, KV, d)
    tail[:, tokens - page:] = 0x7e00          # NaN in K and V of unseen tokens
    got = gu.f16_attention(device, poisoned, query, rows, Q, KV, d, first, page, 64,
                           False)
    assert np.isfinite(got).all()
    gu.assert_close(got, want, what="F16 attention with a poisoned tail")


def test_f16_attention_is_split_invariant_at_16k(device):
    rng = np.random.default_rng(7)
    tokens, rows, Q, KV, d, page = 16384, 5, 64, 8, 128, 256
    keys = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    values = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    pages = synth.f16_pages(keys, values, page)
    query = rng.standard_normal((rows, Q, d)).astype(np.float32)
    first = tokens - 4
    results = [gu.f16_attention(device, pages, query, rows, Q, KV, d, first, page,
                                split, False) for split in (1024, 16384, 0)]
    for other in results[1:]:
        assert np.abs(other - results[0]).max() < 2e-5
    shape = ol.AttentionShape(rows, Q, KV, d, first, page, 0, 0)
    gu.assert_close(results[0], ol.attention_f16(shape, query, pages, True),
                    what="16K F16 attention")


def test_f16_store_matches_oracle_rounding(device):
    rng = np.random.default_rng(8)
    rows, KV, d, page_tokens, layers, layer, first = 70, 4, 128, 32, 2, 1, 5
    keys = (rng.standard_normal((rows, KV, d)) * 10.0 ** rng.integers(-3, 3, (rows, KV, 1))
            ).astype(np.float32)
    values = rng.standard_normal((rows, KV, d)).astype(np.float32)
    page_values = page_tokens * KV * d
    n_pages = (first + rows + page_tokens - 1) // page_tokens
    d_pages = [torch.zeros(layers * 2 * page_values, dtype=torch.float16, device=device)
               for _ in range(n_pages)]
    table = torch.tensor([p.data_ptr() for p in d_pages], dtype=torch.int64,
                         device=device)
    d_keys, d_values = gu.device_tensor(keys, device), gu.device_tensor(values, device)
    qh.call("qllm_store_kv_paged_f16_batch", qh.ptr(d_keys), qh.ptr(d_values),
            qh.ptr(table), layer, page_tokens, first, rows, KV, d, None)
    torch.cuda.synchronize()
    for r in range(rows):
        position = first + r
        page = d_pages[position // page_tokens].cpu().numpy()
        base = layer * 2 * page_values + (position % page_tokens) * KV * d
        assert np.array_equal(page[base: base + KV * d].view(np.uint16),
                              keys[r].astype(np.float16).ravel().view(np.uint16))
        assert np.array_equal(
            page[base + page_values: base + page_values + KV * d].view(np.uint16),
            values[r].astype(np.float16).ravel().view(np.uint16))


def test_f16_attention_rejects_unsupported_geometry(device):
    rng = np.random.default_rng(9)
    with pytest.raises(qh.QllmError):   # head_dim 32 (the reference fixture's)
        run_case(device, rng, 40, 3, 32, 2, 32, 32, 32, False)
    with pytest.raises(qh.QllmError):   # 6 rows x 8 heads per KV head = 3 tiles, 4th row tile
        run_case(device, rng, 40, 7, 8, 1, 128, 32, 32, False)


def test_batched_launch_equals_one_launch_per_batch(device):
    """All row batches of a prompt chunk in one launch: bit for bit what one
    launch per batch computes."""
    rng = np.random.default_rng(77)
    total, first, Q, KV, d, page_tokens, splits, batch = 23, 200, 16, 4, 128, 64, 8, 5
    tokens = first + total - 1
    keys = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    values = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    pages = synth.f16_pages(keys, values, page_tokens, 1, 0)
    query = ol.bf16_round(rng.standard_normal((total, Q, d)).astype(np.float32))
    d_pages = [gu.device_tensor(page, device) for page in pages]
    table = torch.tensor([page.data_ptr() for page in d_pages], dtype=torch.int64,
                         device=device)
    d_query = gu.device_tensor(query, device)
    maxima = torch.zeros((total, splits, Q), device=device)
    sums = torch.zeros_like(maxima)
    outputs = torch.zeros((total, splits, Q, d), device=device)
    out = torch.zeros((total, Q, d), device=device)
    launch = qh.F16AttentionLaunch(
        qh.ptr(d_query), qh.ptr(table), qh.ptr(out), qh.ptr(maxima), qh.ptr(sums),
        qh.ptr(outputs), first, total, 0, page_tokens, Q, KV, d, 0, splits, d, 0,
        qh.OUT_F32, None)
    qh.call("qllm_attention_paged_f16_batched", launch, batch)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    for row in range(0, total, batch):
        rows = min(batch, total - row)
        single = gu.f16_attention(device, pages, query[row:row + rows], rows, Q, KV, d,
                                  first + row, page_tokens, 0, False, balanced_splits=splits)
        assert np.array_equal(got[row:row + rows], single), row


def test_f16_attention_at_262144_tokens_on_one_kv_head(device):
    """The exact-F16 benchmark shape cut down to one KV head and its eight
    query heads: against the oracle (reference rounding points and exact), and
    the same result for every context partition."""
    rng = np.random.default_rng(262144)
    tokens, rows, Q, KV, d, page = 262144, 5, 8, 1, 128, 256
    first = tokens - (rows - 1)
    keys = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    values = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    pages = synth.f16_pages(keys, values, page)
    query = rng.standard_normal((rows, Q, d)).astype(np.float32)
    results = [gu.f16_attention(device, pages, query, rows, Q, KV, d, first, page, split,
                                False) for split in (8192, 65536, 0)]
    for other in results[1:]:
        assert np.abs(other - results[0]).max() < 2e-5
    shape = ol.AttentionShape(rows, Q, KV, d, first, page, 0, 0)
    gu.assert_close(results[0], ol.attention_f16(shape, query, pages, False),
                    what="262144-token F16 attention (exact)")


@pytest.mark.parametrize("tokens,rows,Q,KV,splits,gated", [
    (6000, 5, 64, 8, 4, False),      # six tiles per wave, three row tiles
    (2051, 3, 16, 8, 2, True),       # one row tile, ragged tail tile
    (40000, 4, 32, 4, 32, False)])   # two row tiles at 40K tokens
def test_pipelined_kernel_equals_the_plain_one(device, tokens, rows, Q, KV, splits, gated):
    """head_dim 128 launches take the kernel that keeps the next tile in flight;
    the batched entry point still runs the plain one.  Same tiles, same order
    of every sum: the outputs are bit-equal."""
    rng = np.random.default_rng(tokens)
    d, page_tokens = 128, 256
    first = tokens - (rows - 1)
    keys = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    values = rng.standard_normal((tokens, KV, d)).astype(np.float32)
    pages = synth.f16_pages(keys, values, page_tokens, 1, 0)
    stride = d * (2 if gated else 1)
    query = rng.standard_normal((rows, Q, stride)).astype(np.float32)
    pipelined = gu.f16_attention(device, pages, query, rows, Q, KV, d, first, page_tokens,
                                 0, gated, balanced_splits=splits)
    d_pages = [gu.device_tensor(page, device) for page in pages]
    table = torch.tensor([page.data_ptr() for page in d_pages], dtype=torch.int64,
                         device=device)
    d_query = gu.device_tensor(query, device)
    maxima = torch.zeros((rows, splits, Q), device=device)
    sums = torch.zeros_like(maxima)
    outputs = torch.zeros((rows, splits, Q, d), device=device)
    out = torch.zeros((rows, Q, d), device=device)
    launch = qh.F16AttentionLaunch(
        qh.ptr(d_query), qh.ptr(table), qh.ptr(out), qh.ptr(maxima), qh.ptr(sums),
        qh.ptr(outputs), first, rows, 0, page_tokens, Q, KV, d, 0, splits, stride,
        int(gated), qh.OUT_F32, None)
    qh.call("qllm_attention_paged_f16_batched", launch, rows)
    torch.cuda.synchronize()
    assert np.array_equal(pipelined, out.cpu().numpy())
