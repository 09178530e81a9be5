"""Seeded synthetic inputs for the parity tests (numpy, host side)."""
from __future__ import annotations

import numpy as np

import oracle_lib as ol

FP4_VALUES = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0,
                       -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0])


def fp4_matrix(rng, rows, padded, scheme):
    """Codes uniform over the 16 E2M1 codes; scales log-normal(0, 0.5) binary16
    per 16 columns, or UE8M0 codes in [124, 130] per 32 columns."""
    codes = rng.integers(0, 256, size=(rows, padded // 2), dtype=np.uint8)
    if scheme == ol.SCALE_F16_BLOCK16:
        scales = np.exp(0.5 * rng.standard_normal((rows, padded // 16))
                        ).astype(np.float16).view(np.uint16)
    else:
        scales = rng.integers(124, 131, size=(rows, padded // 32), dtype=np.uint8)
    return codes, scales


def dequantize(codes, scales, scheme):
    """Independent numpy dequantisation (table lookup), float64."""
    rows = codes.shape[0]
    low = FP4_VALUES[codes & 0x0f]
    high = FP4_VALUES[codes >> 4]
    values = np.empty((rows, codes.shape[1] * 2), dtype=np.float64)
    values[:, 0::2] = low
    values[:, 1::2] = high
    if scheme == ol.SCALE_F16_BLOCK16:
        s = scales.view(np.float16).astype(np.float64)
        return values * np.repeat(s, 16, axis=1)
    s = np.ldexp(1.0, scales.astype(np.int64) - 127)
    return values * np.repeat(s, 32, axis=1)


def q4h_encode_numpy(x):
    """Vectorised Q4H encoder: x [..., d] float32 -> (codes [..., d/2] u8,
    scale bits [...] u16)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    absmax = np.max(np.abs(x), axis=-1)
    scale16 = np.maximum(absmax / np.float32(7.0), np.float32(2.0 ** -24)
                         ).astype(np.float16)
    scale = scale16.astype(np.float32)[..., None]
    q = np.clip(np.rint(x / scale), -7, 7).astype(np.int32) & 0x0f
    codes = (q[..., 0::2] | (q[..., 1::2] << 4)).astype(np.uint8)
    return codes, scale16.view(np.uint16)


def q4h_pages(keys, values, page_tokens, layers=1, layer=0):
    """keys/values [tokens, kv_heads, d] -> list of uint8 pages laid out as
    K codes [kv][page_tokens][d/2] | K scales | V codes | V scales per layer."""
    tokens, kv_heads, d = keys.shape
    layer_bytes = ol.q4h_layer_bytes(page_tokens, kv_heads, d)
    n_pages = (tokens + page_tokens - 1) // page_tokens
    records = page_tokens * kv_heads
    kc, ks = q4h_encode_numpy(keys)
    vc, vs = q4h_encode_numpy(values)
    pages = []
    for page_index in range(n_pages):
        page = np.zeros(layer_bytes * layers, dtype=np.uint8)
        base = layer * layer_bytes
        first = page_index * page_tokens
        count = min(page_tokens, tokens - first)
        key_codes = page[base: base + records * (d // 2)].reshape(
            kv_heads, page_tokens, d // 2)
        off = base + records * (d // 2)
        key_scales = page[off: off + records * 2].view(np.uint16).reshape(
            kv_heads, page_tokens)
        off += records * 2
        value_codes = page[off: off + records * (d // 2)].reshape(
            kv_heads, page_tokens, d // 2)
        off += records * (d // 2)
        value_scales = page[off: off + records * 2].view(np.uint16).reshape(
            kv_heads, page_tokens)
        key_codes[:, :count] = kc[first:first + count].transpose(1, 0, 2)
        key_scales[:, :count] = ks[first:first + count].T
        value_codes[:, :count] = vc[first:first + count].transpose(1, 0, 2)
        value_scales[:, :count] = vs[first:first + count].T
        pages.append(page)
    return pages


def f16_pages(keys, values, page_tokens, layers=1, layer=0):
    """keys/values [tokens, kv_heads, d] -> list of uint8 pages holding, per
    layer, K [page_tokens][kv][d] then V [page_tokens][kv][d] in binary16."""
    tokens, kv_heads, d = keys.shape
    page_values = page_tokens * kv_heads * d
    n_pages = (tokens + page_tokens - 1) // page_tokens
    pages = []
    for page_index in range(n_pages):
        page = np.zeros(layers * 2 * page_values, dtype=np.float16)
        first = page_index * page_tokens
        count = min(page_tokens, tokens - first)
        base = layer * 2 * page_values
        page[base: base + count * kv_heads * d] = \
            keys[first:first + count].astype(np.float16).ravel()
        page[base + page_values: base + page_values + count * kv_heads * d] = \
            values[first:first + count].astype(np.float16).ravel()
        pages.append(page.view(np.uint8))
    return pages
