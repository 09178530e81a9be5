"""ctypes binding of the gfx950 kernel library's C ABI (include/qllm_kernels.h).

Plumbing for tests and the benchmark: device memory comes from torch tensors,
whose data pointers are handed to the C entry points unchanged.  There is no
fallback: importing works anywhere, but `load()` raises if the built library
is missing, and every call raises `QllmError` on a non-zero status.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import (POINTER, Structure, c_char_p, c_float, c_int32, c_size_t,
                    c_uint32, c_uint64, c_void_p)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.environ.get(
    "QLLM_HIP_LIBRARY",
    os.path.join(os.path.dirname(_HERE), "lib", "libqllm_hip.so"))

SCALE_UE8M0_BLOCK32 = 0
SCALE_F16_BLOCK16 = 1
OUT_F32 = 0
OUT_F32_BF16_ROUNDED = 1
OUT_BF16 = 2


class QllmError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"qllm status {code}: {message}")
        self.code = code


class Fp4Matrix(Structure):
    _fields_ = [("weights", c_void_p), ("scales", c_void_p),
                ("rows", c_uint32), ("columns", c_uint32),
                ("padded_columns", c_uint32), ("scale_scheme", c_uint32),
                ("layout", c_uint32), ("tile_rows", c_uint32)]


class RolloutStep(Structure):
    _fields_ = [("next_token", c_void_p), ("draft_tokens", c_void_p),
                ("capacity", c_uint32), ("rows", c_uint32),
                ("device_positions", c_void_p)]


class Q4hAttentionLaunch(Structure):
    _fields_ = [("query", c_void_p), ("q8_queries", c_void_p),
                ("query_scales", c_void_p), ("page_table", c_void_p),
                ("output", c_void_p), ("partial_maxima", c_void_p),
                ("partial_sums", c_void_p), ("partial_outputs", c_void_p),
                ("first_context_tokens", c_uint32), ("rows", c_uint32),
                ("full_attention_layer", c_uint32), ("page_tokens", c_uint32),
                ("query_heads", c_uint32), ("kv_heads", c_uint32),
                ("head_dim", c_uint32), ("split_tokens", c_uint32),
                ("maximum_splits", c_uint32), ("query_stride", c_uint32),
                ("output_gated", c_int32), ("output_kind", c_uint32),
                ("stream", c_void_p), ("device_positions", c_void_p)]


class Q4hFusedRope(Structure):
    _fields_ = [("key", c_void_p), ("value", c_void_p), ("q_norm_weight", c_void_p),
                ("k_norm_weight", c_void_p), ("rope_table", c_void_p),
                ("rotary_dim", c_uint32), ("epsilon", c_float),
                ("first_cache_position", c_uint32), ("bf16_activations", c_int32)]


class F16AttentionLaunch(Structure):
    _fields_ = [("query", c_void_p), ("device_pages", c_void_p),
                ("output", c_void_p), ("partial_maxima", c_void_p),
                ("partial_sums", c_void_p), ("partial_outputs", c_void_p),
                ("first_context_tokens", c_uint32), ("rows", c_uint32),
                ("device_page_layer", c_uint32),
                ("device_page_tokens", c_uint32), ("query_heads", c_uint32),
                ("kv_heads", c_uint32), ("head_dim", c_uint32),
                ("split_tokens", c_uint32), ("maximum_splits", c_uint32),
                ("query_stride", c_uint32), ("output_gated", c_int32),
                ("output_kind", c_uint32), ("stream", c_void_p)]


class Q8AttentionLaunch(Structure):
    _fields_ = [("query", c_void_p), ("device_pages", c_void_p),
                ("output", c_void_p), ("partial_maxima", c_void_p),
                ("partial_sums", c_void_p), ("partial_outputs", c_void_p),
                ("page_offset_bytes", c_size_t),
                ("first_context_tokens", c_uint32), ("rows", c_uint32),
                ("page_tokens", c_uint32), ("query_heads", c_uint32),
                ("kv_heads", c_uint32), ("head_dim", c_uint32),
                ("split_tokens", c_uint32), ("maximum_splits", c_uint32),
                ("query_stride", c_uint32), ("output_gated", c_int32),
                ("output_kind", c_uint32), ("stream", c_void_p),
                ("device_positions", c_void_p)]


# name -> (restype, argtypes); every symbol include/qllm_kernels.h declares.
SIGNATURES = {
    "qllm_last_error": (c_char_p, []),
    "qllm_version": (c_char_p, []),
    "qllm_quantize_q8_batch": (c_int32, [c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, c_int32, c_void_p]),
    "qllm_convert_f32_to_bf16_batch": (c_int32, [c_void_p, c_void_p, c_size_t, c_uint32, c_uint32, c_uint32, c_void_p]),
    "qllm_fp4_gemv_q8_batch": (c_int32, [POINTER(Fp4Matrix), c_void_p, c_void_p, c_void_p, c_uint32, c_int32, c_void_p]),
    "qllm_fp4_gemm_bf16": (c_int32, [POINTER(Fp4Matrix), c_void_p, c_size_t, c_void_p, c_uint32, c_void_p, c_uint32, c_void_p]),
    "qllm_fp4_gemm_bf16_partial": (c_int32, [POINTER(Fp4Matrix), c_void_p, c_size_t, c_void_p, c_uint32, c_uint32, c_void_p]),
    "qllm_fp4_gemm_bf16_split": (c_int32, [POINTER(Fp4Matrix), c_void_p, c_size_t, c_void_p, c_uint32, c_uint32, c_void_p]),
    "qllm_fp4_gemm_bf16_tall": (c_int32, [POINTER(Fp4Matrix), c_void_p, c_size_t, c_void_p, c_uint32, c_void_p, c_uint32, c_void_p]),
    "qllm_fp4_swiglu_bf16_tall": (c_int32, [POINTER(Fp4Matrix), POINTER(Fp4Matrix), c_void_p, c_size_t, c_void_p, c_uint32, c_void_p]),
    "qllm_fp4_gemm_bf16_tall_split": (c_int32, [POINTER(Fp4Matrix), c_void_p, c_size_t, c_void_p, c_uint32, c_uint32, c_void_p]),
    "qllm_fp4_swiglu_bf16": (c_int32, [POINTER(Fp4Matrix), POINTER(Fp4Matrix), c_void_p, c_size_t, c_void_p, c_uint32, c_void_p]),
    "qllm_fp4_gemm_balance_workspace_bytes": (c_size_t, []),
    "qllm_fp4_gemm_bf16_split_balanced": (c_int32, [POINTER(Fp4Matrix), c_void_p, c_size_t, c_void_p, c_uint32, c_uint32, c_void_p, c_size_t, c_void_p]),
    "qllm_fp4_swiglu_bf16_balanced": (c_int32, [POINTER(Fp4Matrix), POINTER(Fp4Matrix), c_void_p, c_size_t, c_void_p, c_uint32, c_void_p, c_size_t, c_void_p]),
    "qllm_fp4_gemm_q8": (c_int32, [POINTER(Fp4Matrix), c_void_p, c_void_p, c_void_p, c_uint32, c_void_p, c_uint32, c_void_p]),
    "qllm_fp4_gemm_q8_split": (c_int32, [POINTER(Fp4Matrix), c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_void_p, c_size_t, c_void_p]),
    "qllm_fp4_swiglu_q8": (c_int32, [POINTER(Fp4Matrix), POINTER(Fp4Matrix), c_void_p, c_void_p, c_void_p, c_uint32, c_void_p, c_size_t, c_void_p]),
    "qllm_fp4_packed_weight_bytes": (c_size_t, [c_uint32, c_uint32, c_uint32]),
    "qllm_fp4_packed_scale_bytes": (c_size_t, [c_uint32, c_uint32, c_uint32, c_uint32]),
    "qllm_fp4_prepack": (c_int32, [POINTER(Fp4Matrix), c_uint32, c_void_p, c_void_p, POINTER(Fp4Matrix), c_void_p]),
    "qllm_fp4_unpack_rows": (c_int32, [POINTER(Fp4Matrix), c_uint32, c_uint32, c_void_p, c_void_p, c_void_p]),
    "qllm_fp4_embedding_batch": (c_int32, [POINTER(Fp4Matrix), c_void_p, c_void_p, c_uint32, c_void_p]),
    "qllm_rms_norm_batch": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, c_float, c_int32, c_void_p]),
    "qllm_rms_norm_q8_batch": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_float, c_int32, c_void_p]),
    "qllm_rms_norm_residual_batch": (c_int32, [c_void_p, c_void_p, c_uint32, c_void_p, c_void_p, c_uint32, c_uint32, c_float, c_int32, c_void_p]),
    "qllm_rms_norm_partials_batch": (c_int32, [c_void_p, c_void_p, c_void_p, c_uint32, c_void_p, c_void_p, c_uint32, c_uint32, c_float, c_int32, c_void_p]),
    "qllm_rms_norm_partials_q8_batch": (c_int32, [c_void_p, c_void_p, c_void_p, c_uint32, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_float, c_int32, c_void_p]),
    "qllm_fp4_gemm_q8_partial": (c_int32, [POINTER(Fp4Matrix), c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_void_p]),
    "qllm_rms_norm_concat_batch": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_float, c_int32, c_void_p]),
    "qllm_rms_norm_concat_embedding_batch": (c_int32, [POINTER(Fp4Matrix), c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_float, c_int32, c_void_p, c_void_p]),
    "qllm_add_in_place": (c_int32, [c_void_p, c_void_p, c_uint32, c_int32, c_void_p]),
    "qllm_silu_product": (c_int32, [c_void_p, c_void_p, c_void_p, c_uint32, c_int32, c_void_p]),
    "qllm_q4h_layer_bytes": (c_size_t, [c_uint32, c_uint32, c_uint32]),
    "qllm_qkv_rope_cache_paged_q4h_batch": (c_int32, [c_void_p, c_uint32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_float, c_float, c_int32, c_void_p]),
    "qllm_qkv_rope_cache_paged_q4h_batch_deferred": (c_int32, [c_void_p, c_uint32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_float, c_float, c_int32, c_void_p]),
    "qllm_qkv_rope_cache_paged_q4h_from_partials": (c_int32, [c_void_p, c_uint32, c_void_p, c_uint32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_float, c_float, c_int32, c_void_p]),
    "qllm_qkv_rope_cache_paged_q4h_prepared": (c_int32, [c_void_p, c_uint32, c_void_p, c_uint32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_float, c_float, c_int32, c_void_p, c_void_p, c_void_p]),
    "qllm_q4h_query_operand_bytes": (c_size_t, [c_uint32, c_uint32, c_uint32, c_uint32]),
    "qllm_qkv_rope_batch": (c_int32, [c_void_p, c_uint32, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_float, c_float, c_int32, c_void_p]),
    "qllm_qkv_rope_batch_deferred": (c_int32, [c_void_p, c_uint32, c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_float, c_float, c_int32, c_void_p]),
    "qllm_store_kv_paged_q4h_batch": (c_int32, [c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_void_p]),
    "qllm_quantize_gqa_queries_q8": (c_int32, [c_void_p, c_uint32, c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, c_void_p]),
    "qllm_attention_paged_q4h": (c_int32, [POINTER(Q4hAttentionLaunch)]),
    "qllm_attention_paged_q4h_fused": (c_int32, [POINTER(Q4hAttentionLaunch), POINTER(Q4hFusedRope)]),
    "qllm_rope_table": (c_int32, [c_void_p, c_uint32, c_uint32, c_uint32, c_float, c_int32, c_void_p, c_void_p]),
    "qllm_attention_paged_q4h_batched": (c_int32, [POINTER(Q4hAttentionLaunch), c_uint32]),
    "qllm_attention_paged_q4h_prompt": (c_int32, [POINTER(Q4hAttentionLaunch), c_uint32]),
    "qllm_store_kv_paged_f16_batch": (c_int32, [c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_void_p]),
    "qllm_attention_paged_f16": (c_int32, [POINTER(F16AttentionLaunch)]),
    "qllm_attention_paged_f16_batched": (c_int32, [POINTER(F16AttentionLaunch), c_uint32]),
    "qllm_attention_paged_q8_batched": (c_int32, [POINTER(Q8AttentionLaunch), c_uint32]),
    "qllm_q8_layer_bytes": (c_size_t, [c_uint32, c_uint32, c_uint32]),
    "qllm_store_kv_paged_q8_batch": (c_int32, [c_void_p, c_void_p, c_void_p, c_size_t, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_void_p]),
    "qllm_store_kv_paged_q8_batch_deferred": (c_int32, [c_void_p, c_void_p, c_void_p, c_size_t, c_uint32, c_void_p, c_uint32, c_uint32, c_uint32, c_void_p]),
    "qllm_qkv_rope_store_q8_batch": (c_int32, [c_void_p, c_uint32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_uint32, c_uint32, c_uint32, c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_float, c_float, c_int32, c_void_p]),
    "qllm_fp4_head_workspace_bytes": (c_size_t, [POINTER(Fp4Matrix), c_uint32]),
    "qllm_fp4_head_argmax": (c_int32, [POINTER(Fp4Matrix), c_void_p, c_size_t, c_void_p, c_uint32, c_void_p, c_void_p, c_size_t, POINTER(RolloutStep), c_void_p]),
    "qllm_rollout_advance": (c_int32, [c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_void_p, c_void_p]),
    "qllm_attention_paged_q8": (c_int32, [POINTER(Q8AttentionLaunch)]),
    "qllm_argmax_workspace_bytes": (c_size_t, [c_uint32, c_uint32]),
    "qllm_argmax_batch": (c_int32, [c_void_p, c_uint32, c_uint32, c_void_p, c_void_p, c_size_t, c_void_p]),
    "qllm_argmax_static_capacity_bytes": (c_size_t, []),
    "qllm_argmax_batch_static": (c_int32, [c_void_p, c_uint32, c_uint32, c_void_p, c_void_p]),
    "qllm_topk_workspace_bytes": (c_size_t, [c_uint32, c_uint32]),
    "qllm_topk_logits": (c_int32, [c_void_p, c_uint32, c_uint32, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "qllm_topk_batch_workspace_bytes": (c_size_t, [c_uint32, c_uint32, c_uint32]),
    "qllm_topk_logits_batch": (c_int32, [c_void_p, c_uint32, c_size_t, c_uint32, c_uint32, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "qllm_apply_presence_penalty": (c_int32, [c_void_p, c_void_p, c_uint32, c_float, c_void_p]),
    "qllm_apply_presence_penalty_rows": (c_int32, [c_void_p, c_size_t, c_void_p, c_void_p, c_uint32, c_uint32, c_float, c_void_p]),
    "qllm_mark_presence": (c_int32, [c_void_p, c_void_p, c_uint32, c_uint32, c_void_p]),
    "qllm_fill_random": (c_int32, [c_void_p, c_size_t, c_uint32, c_uint64, c_void_p]),
}

class GemmSegment(ctypes.Structure):
    """Mirror of qllm_gemm_segment."""
    _fields_ = [("output", c_void_p), ("rows", c_uint32), ("output_kind", c_uint32)]


_STATUS_FUNCTIONS = {name for name, (restype, _) in SIGNATURES.items()
                     if restype is c_int32}
_library = None


def load() -> ctypes.CDLL:
    """Load the built library; raise if it has not been built."""
    global _library
    if _library is None:
        if not os.path.exists(LIBRARY_PATH):
            raise FileNotFoundError(
                f"{LIBRARY_PATH} is missing: build it with "
                "`make -C quantum-llm_amd` (or __graft_entry__.build())")
        library = ctypes.CDLL(LIBRARY_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            function = getattr(library, name)  # AttributeError if not exported
            function.restype = restype
            function.argtypes = argtypes
        _library = library
    return _library


def call(name: str, *arguments):
    """Call an entry point; raise QllmError on a non-zero status."""
    library = load()
    result = getattr(library, name)(*arguments)
    if name in _STATUS_FUNCTIONS and result != 0:
        raise QllmError(result, library.qllm_last_error().decode())
    return result


def ptr(tensor) -> int:
    """Device (or host) address of a torch tensor / None."""
    return 0 if tensor is None else tensor.data_ptr()


def fp4_matrix(weights, scales, rows, columns, padded_columns, scheme) -> Fp4Matrix:
    return Fp4Matrix(ptr(weights), ptr(scales), rows, columns, padded_columns,
                     scheme, 0, 0)


def prepack(matrix: Fp4Matrix, device, tile_rows=0):
    """Tiled device copy of a row-major matrix: (descriptor, keepalive).
    tile_rows 0 = full 32-row tiles."""
    import torch
    weight_bytes = call("qllm_fp4_packed_weight_bytes", matrix.rows,
                        matrix.padded_columns, tile_rows)
    scale_bytes = call("qllm_fp4_packed_scale_bytes", matrix.rows,
                       matrix.padded_columns, matrix.scale_scheme, tile_rows)
    weights = torch.empty(weight_bytes, dtype=torch.uint8, device=device)
    scales = torch.empty(scale_bytes, dtype=torch.uint8, device=device)
    packed = Fp4Matrix()
    call("qllm_fp4_prepack", ctypes.byref(matrix), tile_rows, ptr(weights), ptr(scales),
         ctypes.byref(packed), None)
    return packed, (weights, scales)
