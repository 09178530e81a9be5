"""The proposer's Q8 KV cache on the GPU, through the C ABI: records byte-exact
against the CPU oracle, decode attention within rtol 1e-2 / atol 1e-3 of the
oracle's double-precision attention on the same records."""
import numpy as np
import pytest
import torch

import gpu_util as gu
import oracle_lib as ol
import qllm_hip as qh

pytestmark = pytest.mark.gpu


def build_cache(device, rng, tokens, KV, d, page_tokens, offset, scale=1.0, chunk=5):
    """Fills device pages through the store kernel (in micro-batches, as the
    proposer does) and the oracle's pages with the same rows."""
    layer_bytes = ol.q8_layer_bytes(page_tokens, KV, d)
    assert qh.load().qllm_q8_layer_bytes(page_tokens, KV, d) == layer_bytes
    n_pages = (tokens + page_tokens - 1) // page_tokens
    d_pages = [torch.zeros(offset + layer_bytes, dtype=torch.uint8, device=device)
               for _ in range(n_pages)]
    table = torch.tensor([page.data_ptr() for page in d_pages], dtype=torch.int64,
                         device=device)
    pages = [np.zeros(offset + layer_bytes, dtype=np.uint8) for _ in range(n_pages)]
    keys = (scale * rng.standard_normal((tokens, KV, d))).astype(np.float32)
    values = (scale * rng.standard_normal((tokens, KV, d))).astype(np.float32)
    keys[min(3, tokens - 1), 0] = 0.0                     # an all-zero record
    for first in range(0, tokens, chunk):
        count = min(chunk, tokens - first)
        gu.q8_store(device, d_pages, table, offset, page_tokens, first,
                    keys[first:first + count], values[first:first + count])
    for token in range(tokens):
        for head in range(KV):
            ol.q8_store(pages[token // page_tokens], offset, page_tokens, token, head,
                        KV, d, keys[token, head], values[token, head])
    return d_pages, table, pages


@pytest.mark.parametrize("tokens,KV,d,page_tokens,offset", [
    (70, 2, 128, 32, 0), (300, 4, 256, 64, 4096), (37, 8, 128, 256, 16)])
def test_q8_store_is_byte_exact(device, tokens, KV, d, page_tokens, offset):
    rng = np.random.default_rng(tokens + KV)
    d_pages, table, pages = build_cache(device, rng, tokens, KV, d, page_tokens, offset)
    for index, page in enumerate(pages):
        got = gu.q8_planes_to_records(d_pages[index].cpu().numpy(), offset,
                                      page_tokens, KV, d)
        want = page[offset:]
        assert np.array_equal(got, want), f"page {index}"
        assert not d_pages[index].cpu().numpy()[:offset].any()   # nothing before the layer


@pytest.mark.parametrize("tokens,rows,Q,KV,d,page,split,gated", [
    (5, 5, 8, 2, 128, 32, 512, False),        # context of the rows alone
    (12, 5, 8, 1, 128, 64, 32, False),
    (100, 5, 64, 8, 128, 256, 64, False),
    (1000, 5, 64, 8, 128, 256, 256, False),
    (700, 5, 24, 4, 256, 256, 512, True),     # reference geometry, gated
    (3000, 1, 64, 8, 128, 256, 1024, False),  # single-row decode (rollout passes)
    (257, 3, 16, 8, 128, 64, 128, True),
    (5, 5, 8, 2, 128, 64, 0, False),          # balanced: most waves idle
    (4100, 5, 64, 8, 128, 256, 0, False),
    (1500, 1, 24, 4, 256, 256, 0, True)])
def test_q8_attention_matches_oracle(device, tokens, rows, Q, KV, d, page, split, gated):
    rng = np.random.default_rng(tokens + 7 * rows + Q)
    offset = 1024
    d_pages, table, pages = build_cache(device, rng, tokens, KV, d, page, offset)
    first = tokens - (rows - 1)
    stride = d * (2 if gated else 1)
    query = rng.standard_normal((rows, Q, stride)).astype(np.float32)
    shape = ol.AttentionShape(rows, Q, KV, d, first, page, 0, int(gated))
    want = ol.attention_q8(shape, query, pages, offset)
    got = gu.q8_attention(device, d_pages, table, offset, query, rows, Q, KV, d, first,
                          page, split, gated)
    gu.assert_close(got, want, what="Q8 attention")


def test_q8_attention_reference_fixture(device):
    """q8_five_query_microbatch_check (dense_fp4_cuda_smoke.cpp:896-1033; its
    bound on the reference kernel is 2e-3), at head_dim 256 with one KV head,
    context padded to a 32-token page."""
    context, first, rows, heads, d, page = 16, 12, 5, 6, 256, 32
    index = np.arange(context * d, dtype=np.float32)
    key = (np.sin((index + 31) * np.float32(0.013)) *
           (np.float32(0.19) + (np.arange(context * d) % 11).astype(np.float32) * np.float32(0.009)))
    value = (np.cos((index + 23) * np.float32(0.017)) *
             (np.float32(0.17) + (np.arange(context * d) % 9).astype(np.float32) * np.float32(0.011)))
    query = (np.sin((np.arange(rows * 2 * heads * d, dtype=np.float32) + 7) * np.float32(0.005)) *
             np.float32(0.37)).astype(np.float32).reshape(rows, heads, 2 * d)
    keys = key.astype(np.float32).reshape(context, 1, d)
    values = value.astype(np.float32).reshape(context, 1, d)
    layer_bytes = ol.q8_layer_bytes(page, 1, d)
    d_page = torch.zeros(layer_bytes, dtype=torch.uint8, device=device)
    table = torch.tensor([d_page.data_ptr()], dtype=torch.int64, device=device)
    gu.q8_store(device, [d_page], table, 0, page, 0, keys, values)
    host = np.zeros(layer_bytes, dtype=np.uint8)
    for token in range(context):
        ol.q8_store(host, 0, page, token, 0, 1, d, keys[token, 0], values[token, 0])
    shape = ol.AttentionShape(rows, heads, 1, d, first, page, 0, 1)
    want = ol.attention_q8(shape, query, [host])
    got = gu.q8_attention(device, [d_page], table, 0, query, rows, heads, 1, d, first,
                          page, 32, True)
    assert np.abs(got - want).max() < 2e-3
    gu.assert_close(got, want, what="Q8 fixture")


def test_q8_attention_ignores_records_past_the_context(device):
    """Uninitialised records behind the last visible token (any bit pattern,
    NaN scales included) must not reach the result."""
    rng = np.random.default_rng(11)
    tokens, rows, Q, KV, d, page = 45, 5, 8, 2, 128, 64
    offset = 0
    d_pages, table, pages = build_cache(device, rng, tokens, KV, d, page, offset)
    first = tokens - (rows - 1)
    query = rng.standard_normal((rows, Q, d)).astype(np.float32)
    clean = gu.q8_attention(device, d_pages, table, offset, query, rows, Q, KV, d, first,
                            page, 32, False)
    # poison everything behind token `tokens`: codes 0x80.., scales NaN (0x7e00)
    host = d_pages[0].cpu().numpy().copy()
    codes = page * KV * d
    for kind in range(2):
        plane = host[kind * codes:(kind + 1) * codes].reshape(page, KV, d)
        plane[tokens:] = 0x80
        scales = host[2 * codes + kind * KV * page * 2:
                      2 * codes + (kind + 1) * KV * page * 2].view(np.uint16).reshape(KV, page)
        scales[:, tokens:] = 0x7e00
    d_pages[0].copy_(torch.from_numpy(host))
    poisoned = gu.q8_attention(device, d_pages, table, offset, query, rows, Q, KV, d,
                               first, page, 32, False)
    assert np.array_equal(clean, poisoned)


def test_q8_entry_points_reject_bad_arguments(device):
    page = torch.zeros(4096, dtype=torch.uint8, device=device)
    table = torch.tensor([page.data_ptr()], dtype=torch.int64, device=device)
    x = torch.zeros((1, 1, 128), device=device)
    with pytest.raises(qh.QllmError):          # offset not a multiple of 16
        qh.call("qllm_store_kv_paged_q8_batch", qh.ptr(x), qh.ptr(x), qh.ptr(table),
                8, 32, 0, 1, 1, 128, None)
    query = torch.zeros((1, 8, 128), device=device)
    out = torch.zeros((1, 8, 128), device=device)
    part = torch.zeros((1, 1, 8, 130), device=device)
    launch = qh.Q8AttentionLaunch(
        qh.ptr(query), qh.ptr(table), qh.ptr(out), qh.ptr(part), qh.ptr(part),
        qh.ptr(part), 0, 1, 1, 48, 8, 1, 128, 32, 1, 128, 0, qh.OUT_F32, None)
    with pytest.raises(qh.QllmError):          # page_tokens % 32
        qh.call("qllm_attention_paged_q8", launch)
    launch.page_tokens, launch.head_dim = 32, 64
    with pytest.raises(qh.QllmError):          # head_dim
        qh.call("qllm_attention_paged_q8", launch)


@pytest.mark.parametrize("total,first,Q,KV,d,batch,gated", [
    (23, 200, 16, 4, 128, 5, False), (40, 1, 64, 8, 128, 6, False),
    (9, 300, 24, 4, 256, 4, True)])
def test_q8_batched_launch_equals_one_launch_per_batch(device, total, first, Q, KV, d,
                                                       batch, gated):
    """All row batches of a prompt chunk in one launch: bit for bit what one
    launch per batch computes."""
    rng = np.random.default_rng(total + first)
    page_tokens, offset, splits = 64, 512, 8
    tokens = first + total - 1
    d_pages, table, pages = build_cache(device, rng, tokens, KV, d, page_tokens, offset)
    stride = d * (2 if gated else 1)
    query = rng.standard_normal((total, Q, stride)).astype(np.float32)
    d_query = gu.device_tensor(query, device)
    maxima = torch.zeros((total, splits, Q), device=device)
    sums = torch.zeros_like(maxima)
    outputs = torch.zeros((total, splits, Q, d), device=device)
    out = torch.zeros((total, Q, d), device=device)
    launch = qh.Q8AttentionLaunch(
        qh.ptr(d_query), qh.ptr(table), qh.ptr(out), qh.ptr(maxima), qh.ptr(sums),
        qh.ptr(outputs), offset, first, total, page_tokens, Q, KV, d, 0, splits, stride,
        int(gated), qh.OUT_F32, None)
    qh.call("qllm_attention_paged_q8_batched", launch, batch)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    for row in range(0, total, batch):
        rows = min(batch, total - row)
        single = gu.q8_attention(device, d_pages, table, offset, query[row:row + rows], rows,
                                 Q, KV, d, first + row, page_tokens, 0, gated,
                                 balanced_splits=splits)
        assert np.array_equal(got[row:row + rows], single), row
    if total * (Q // KV) > (32 if d == 256 else 48):
        with pytest.raises(qh.QllmError):
            qh.call("qllm_attention_paged_q8_batched", launch, total)


@pytest.mark.parametrize("deferred", [False, True])
@pytest.mark.parametrize("rows,Q,KV,d,rotary,gated,qk_norm", [
    (1, 24, 4, 256, 64, True, True),      # one rollout pass at the 27B geometry
    (5, 8, 2, 128, 128, False, False),
    (8, 16, 8, 128, 64, True, True)])
def test_rotary_with_q8_store_equals_the_two_launches(device, rows, Q, KV, d, rotary,
                                                      gated, qk_norm, deferred):
    """qllm_qkv_rope_store_q8_batch against the oracle's rotary, and bit-equal -
    queries, keys and cache bytes - to qllm_qkv_rope_batch followed by
    qllm_store_kv_paged_q8_batch; cache position and rotary position differ by
    one as in the proposer, given as arguments or as device words."""
    rng = np.random.default_rng(rows * 31 + Q)
    page_tokens, offset, cache_first = 64, 4096, 61       # the rows cross a page edge
    rotary_first = cache_first + 1
    stride = d * (2 if gated else 1)
    q = rng.standard_normal((rows, Q, stride)).astype(np.float32)
    k = rng.standard_normal((rows, KV, d)).astype(np.float32)
    v = rng.standard_normal((rows, KV, d)).astype(np.float32)
    qw = (0.1 * rng.standard_normal(d)).astype(np.float32) if qk_norm else None
    kw = (0.1 * rng.standard_normal(d)).astype(np.float32) if qk_norm else None
    d_qw = None if qw is None else gu.device_tensor(qw, device)
    d_kw = None if kw is None else gu.device_tensor(kw, device)
    layer_bytes = ol.q8_layer_bytes(page_tokens, KV, d)

    def pages():
        held = [torch.zeros(offset + layer_bytes, dtype=torch.uint8, device=device)
                for _ in range(2)]
        return held, torch.tensor([p.data_ptr() for p in held], dtype=torch.int64,
                                  device=device)

    one_q, one_k, d_v = (gu.device_tensor(x, device) for x in (q, k, v))
    one_pages, one_table = pages()
    words = torch.tensor([cache_first, rotary_first, 0, 0], dtype=torch.int32,
                         device=device)
    qh.call("qllm_qkv_rope_store_q8_batch", qh.ptr(one_q), stride, qh.ptr(one_k),
            qh.ptr(d_v), qh.ptr(d_qw), qh.ptr(d_kw), qh.ptr(one_table), offset,
            page_tokens, 0 if deferred else cache_first, 0 if deferred else rotary_first,
            qh.ptr(words) if deferred else None, rows, Q, KV, d, rotary, 1e-6, 1e6, 0,
            None)
    two_q, two_k = (gu.device_tensor(x, device) for x in (q, k))
    two_pages, two_table = pages()
    qh.call("qllm_qkv_rope_batch", qh.ptr(two_q), stride, qh.ptr(two_k), qh.ptr(d_qw),
            qh.ptr(d_kw), rotary_first, rows, Q, KV, d, rotary, 1e-6, 1e6, 0, None)
    qh.call("qllm_store_kv_paged_q8_batch", qh.ptr(two_k), qh.ptr(d_v),
            qh.ptr(two_table), offset, page_tokens, cache_first, rows, KV, d, None)
    torch.cuda.synchronize()
    assert torch.equal(one_q, two_q) and torch.equal(one_k, two_k)
    for one, two in zip(one_pages, two_pages):
        assert torch.equal(one, two)
    got_q, got_k = one_q.cpu().numpy(), one_k.cpu().numpy()
    for r in range(rows):
        for h in range(Q):
            want = ol.head_norm_rope(q[r, h, :d], qw, rotary, rotary_first + r, 1e-6, 1e6)
            assert np.abs(got_q[r, h, :d] - want).max() < 2e-5
        for h in range(KV):
            want = ol.head_norm_rope(k[r, h], kw, rotary, rotary_first + r, 1e-6, 1e6)
            assert np.abs(got_k[r, h] - want).max() < 2e-5
    if gated:
        assert np.array_equal(got_q[..., d:], q[..., d:])
    # the records are the oracle's encoding of the keys the kernel produced
    want_pages = [np.zeros(offset + layer_bytes, dtype=np.uint8) for _ in range(2)]
    for r in range(rows):
        for h in range(KV):
            ol.q8_store(want_pages[(cache_first + r) // page_tokens], offset, page_tokens,
                        cache_first + r, h, KV, d, got_k[r, h], v[r, h])
    for got, want in zip(one_pages, want_pages):
        assert np.array_equal(
            gu.q8_planes_to_records(got.cpu().numpy(), offset, page_tokens, KV, d),
            want[offset:])
