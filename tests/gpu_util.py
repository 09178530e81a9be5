"""Helpers shared by the GPU parity tests: torch tensors carry device memory,
the kernels are reached only through the C ABI (qllm_hip / qllm_provider)."""
import numpy as np
import torch

import oracle_lib as ol
import qllm_hip as qh

RTOL = 1e-2   # tolerance the hot path is held to for F32-accumulate outputs
ATOL = 1e-3


def device_tensor(array, device):
    return torch.from_numpy(np.ascontiguousarray(array)).to(device)


def assert_close(got, want, rtol=RTOL, atol=ATOL, what=""):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    error = np.abs(got - want)
    bound = atol + rtol * np.abs(want)
    worst = np.unravel_index(np.argmax(error - bound), error.shape)
    assert np.all(error <= bound), (
        f"{what}: {int((error > bound).sum())} of {error.size} outside "
        f"rtol={rtol} atol={atol}; worst at {worst}: got {got[worst]} want {want[worst]}")


def gemm(device, codes, scales, scheme, rows, padded, act_bf16_values, *,
         tiled=True, out_kind=qh.OUT_F32, residual=None, tile_rows=0):
    """qllm_fp4_gemm_bf16 on host numpy inputs; returns a numpy array.
    tile_rows 0 = full 32-row tiles."""
    batch = act_bf16_values.shape[0]
    d_codes = device_tensor(codes, device)
    d_scales = device_tensor(scales, device)
    d_act = device_tensor(ol.bf16_bits(act_bf16_values), device)
    matrix = qh.fp4_matrix(d_codes, d_scales, rows, padded, padded, scheme)
    keep = None
    if tiled:
        matrix, keep = qh.prepack(matrix, device, tile_rows)
    dtype = torch.bfloat16 if out_kind == qh.OUT_BF16 else torch.float32
    out = torch.zeros((batch, rows), dtype=dtype, device=device)
    d_residual = None if residual is None else device_tensor(residual, device)
    qh.call("qllm_fp4_gemm_bf16", matrix, qh.ptr(d_act), d_act.numel() * 2,
            qh.ptr(out), out_kind, qh.ptr(d_residual), batch, None)
    torch.cuda.synchronize()
    del keep
    return out.float().cpu().numpy()


def q4h_attention(device, pages, query, rows, query_heads, kv_heads, head_dim,
                  first_context, page_tokens, split_tokens, gated, layer=0,
                  out_kind=qh.OUT_F32, balanced_splits=32):
    """split_tokens 0 selects the balanced partition over `balanced_splits`
    workgroups per KV head."""
    stride = head_dim * (2 if gated else 1)
    d_pages = [device_tensor(page, device) for page in pages]
    table = torch.tensor([page.data_ptr() for page in d_pages], dtype=torch.int64,
                         device=device)
    d_query = device_tensor(query, device)
    context = first_context + rows - 1
    splits = ((context + split_tokens - 1) // split_tokens if split_tokens
              else balanced_splits)
    maxima = torch.zeros((rows, splits, query_heads), device=device)
    sums = torch.zeros_like(maxima)
    outputs = torch.zeros((rows, splits, query_heads, head_dim), device=device)
    dtype = torch.bfloat16 if out_kind == qh.OUT_BF16 else torch.float32
    out = torch.zeros((rows, query_heads, head_dim), dtype=dtype, device=device)
    launch = qh.Q4hAttentionLaunch(
        qh.ptr(d_query), 0, 0, qh.ptr(table), qh.ptr(out), qh.ptr(maxima),
        qh.ptr(sums), qh.ptr(outputs), first_context, rows, layer, page_tokens,
        query_heads, kv_heads, head_dim, split_tokens, splits, stride, int(gated),
        out_kind, None)
    qh.call("qllm_attention_paged_q4h", launch)
    torch.cuda.synchronize()
    return out.float().cpu().numpy()


def f16_attention(device, pages, query, rows, query_heads, kv_heads, head_dim,
                  first_context, page_tokens, split_tokens, gated, layer=0,
                  out_kind=qh.OUT_F32, balanced_splits=32):
    """qllm_attention_paged_f16 on host pages (list of uint8 arrays)."""
    stride = head_dim * (2 if gated else 1)
    d_pages = [device_tensor(page, device) for page in pages]
    table = torch.tensor([page.data_ptr() for page in d_pages], dtype=torch.int64,
                         device=device)
    d_query = device_tensor(query, device)
    context = first_context + rows - 1
    splits = ((context + split_tokens - 1) // split_tokens if split_tokens
              else balanced_splits)
    maxima = torch.zeros((rows, splits, query_heads), device=device)
    sums = torch.zeros_like(maxima)
    outputs = torch.zeros((rows, splits, query_heads, head_dim), device=device)
    dtype = torch.bfloat16 if out_kind == qh.OUT_BF16 else torch.float32
    out = torch.zeros((rows, query_heads, head_dim), dtype=dtype, device=device)
    launch = qh.F16AttentionLaunch(
        qh.ptr(d_query), qh.ptr(table), qh.ptr(out), qh.ptr(maxima), qh.ptr(sums),
        qh.ptr(outputs), first_context, rows, layer, page_tokens, query_heads,
        kv_heads, head_dim, split_tokens, splits, stride, int(gated), out_kind, None)
    qh.call("qllm_attention_paged_f16", launch)
    torch.cuda.synchronize()
    return out.float().cpu().numpy()


def q8_planes_to_records(page, offset, page_tokens, kv_heads, head_dim):
    """Re-lays one layer of a device Q8 page (code planes, then scale planes) as
    the reference's records: [K records | V records], record (slot*kv + head) =
    head_dim codes followed by the binary16 scale."""
    d = head_dim
    records = page_tokens * kv_heads
    codes = records * d
    layer = page[offset: offset + 2 * records * (d + 2)]
    out = np.zeros((2, records, d + 2), dtype=np.uint8)
    for kind in range(2):
        out[kind, :, :d] = layer[kind * codes:(kind + 1) * codes].reshape(records, d)
        scales = layer[2 * codes + kind * records * 2:
                       2 * codes + (kind + 1) * records * 2].view(np.uint16)
        scales = scales.reshape(kv_heads, page_tokens).T.reshape(records)   # -> [slot][head]
        out[kind, :, d:] = np.ascontiguousarray(scales).view(np.uint8).reshape(records, 2)
    return out.reshape(-1)


def q8_store(device, d_pages, table, offset, page_tokens, first_position, keys, values):
    """qllm_store_kv_paged_q8_batch for rows keys/values [rows, kv_heads, d]."""
    rows, kv_heads, d = keys.shape
    d_keys, d_values = device_tensor(keys, device), device_tensor(values, device)
    qh.call("qllm_store_kv_paged_q8_batch", qh.ptr(d_keys), qh.ptr(d_values),
            qh.ptr(table), offset, page_tokens, first_position, rows, kv_heads, d, None)
    torch.cuda.synchronize()


def q8_attention(device, d_pages, table, offset, query, rows, query_heads, kv_heads,
                 head_dim, first_context, page_tokens, split_tokens, gated,
                 out_kind=qh.OUT_F32, balanced_splits=32):
    stride = head_dim * (2 if gated else 1)
    d_query = device_tensor(query, device)
    context = first_context + rows - 1
    splits = ((context + split_tokens - 1) // split_tokens if split_tokens
              else balanced_splits)
    maxima = torch.zeros((rows, splits, query_heads), device=device)
    sums = torch.zeros_like(maxima)
    outputs = torch.zeros((rows, splits, query_heads, head_dim), device=device)
    dtype = torch.bfloat16 if out_kind == qh.OUT_BF16 else torch.float32
    out = torch.zeros((rows, query_heads, head_dim), dtype=dtype, device=device)
    launch = qh.Q8AttentionLaunch(
        qh.ptr(d_query), qh.ptr(table), qh.ptr(out), qh.ptr(maxima), qh.ptr(sums),
        qh.ptr(outputs), offset, first_context, rows, page_tokens, query_heads,
        kv_heads, head_dim, split_tokens, splits, stride, int(gated), out_kind, None)
    qh.call("qllm_attention_paged_q8", launch)
    torch.cuda.synchronize()
    return out.float().cpu().numpy()
