"""ctypes access to the CPU oracle (oracle/libqllm_oracle.so) and, when it has
been built, to the shared library compiled from the reference's own host
sampling source (oracle/_ref/libqllm_ref.so).  Test infrastructure only."""
from __future__ import annotations

import ctypes
import os
import subprocess
from ctypes import (POINTER, Structure, c_double, c_float, c_int, c_size_t,
                    c_uint8, c_uint16, c_uint32, c_uint64, c_void_p)

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_PATH = os.path.join(ORACLE_DIR, "libqllm_oracle.so")
REF_PATH = os.path.join(ORACLE_DIR, "_ref", "libqllm_ref.so")

SCALE_UE8M0_BLOCK32 = 0
SCALE_F16_BLOCK16 = 1


class AttentionShape(Structure):
    _fields_ = [("rows", c_uint32), ("query_heads", c_uint32),
                ("kv_heads", c_uint32), ("head_dim", c_uint32),
                ("first_context_tokens", c_uint32), ("page_tokens", c_uint32),
                ("layer", c_uint32), ("output_gated", c_int)]


class TokenProbability(Structure):
    _fields_ = [("token", c_uint32), ("probability", c_double)]


class RejectionResult(Structure):
    _fields_ = [("accepted", c_int), ("token", c_uint32),
                ("target_probability", c_double),
                ("draft_probability", c_double)]


class VerifyResult(Structure):
    _fields_ = [("accepted", c_uint32), ("next_token", c_uint32),
                ("status", c_int)]


_oracle = None
_ref = None


def build_oracle() -> None:
    subprocess.run(["make", "-s", "-C", ORACLE_DIR], check=True)


def oracle() -> ctypes.CDLL:
    global _oracle
    if _oracle is None:
        if not os.path.exists(ORACLE_PATH):
            build_oracle()
        lib = ctypes.CDLL(ORACLE_PATH)
        lib.qo_bf16_round.restype = c_float
        lib.qo_bf16_round.argtypes = [c_float]
        lib.qo_bf16_bits.restype = c_uint16
        lib.qo_bf16_bits.argtypes = [c_float]
        lib.qo_f16_bits.restype = c_uint16
        lib.qo_f16_bits.argtypes = [c_float]
        lib.qo_f16_value.restype = c_float
        lib.qo_f16_value.argtypes = [c_uint16]
        lib.qo_fp4_value.restype = c_float
        lib.qo_fp4_value.argtypes = [c_uint8]
        lib.qo_fp4_twice.restype = c_int
        lib.qo_fp4_twice.argtypes = [c_uint8]
        lib.qo_ue8m0_value.restype = c_float
        lib.qo_ue8m0_value.argtypes = [c_uint8]
        lib.qo_q4h_layer_bytes.restype = c_size_t
        lib.qo_q4h_layer_bytes.argtypes = [c_uint32, c_uint32, c_uint32]
        lib.qo_argmax.restype = c_uint32
        lib.qo_argmax.argtypes = [c_void_p, c_uint32]
        lib.qo_topk.restype = c_uint32
        lib.qo_topk.argtypes = [c_void_p, c_uint32, c_uint32, c_void_p, c_void_p]
        lib.qo_counter_uniform.restype = c_double
        lib.qo_counter_uniform.argtypes = [c_uint64, c_uint32, c_uint32, c_uint32]
        lib.qo_accept_greedy.restype = VerifyResult
        lib.qo_accept_greedy.argtypes = [c_void_p, c_uint32, c_void_p, c_uint32]
        lib.qo_accept_stochastic.restype = VerifyResult
        lib.qo_accept_stochastic.argtypes = [
            POINTER(POINTER(TokenProbability)), c_void_p,
            POINTER(POINTER(TokenProbability)), c_void_p, c_void_p, c_uint32,
            c_uint64, c_uint32]
        lib.qo_num_threads.restype = c_int
        lib.qo_normal.restype = c_float
        lib.qo_normal.argtypes = [c_uint64, c_uint64]
        lib.qo_mix64.restype = c_uint64
        lib.qo_mix64.argtypes = [c_uint64, c_uint64]
        _oracle = lib
    return _oracle


def ref():
    """The reference's own sampling code, or None if it was not built."""
    global _ref
    if _ref is None and os.path.exists(REF_PATH):
        lib = ctypes.CDLL(REF_PATH)
        lib.qref_counter_uniform.restype = c_double
        lib.qref_counter_uniform.argtypes = [c_uint64, c_uint32, c_uint32, c_uint32]
        _ref = lib
    return _ref


def _p(array: np.ndarray):
    return array.ctypes.data_as(c_void_p)


def reference_fp4_swiglu(gate, up, down, hidden, intermediate, inputs, threads=1,
                         bf16_intermediate=False, repeats=1):
    """down(silu(gate x) * up x) by the reference's own CPU executor
    (runtime/src/cpu/fp4_host_executor.cpp) compiled into oracle/_ref.
    gate/up/down = (codes, scales) of ABI-3 matrices; returns (out, seconds of
    the best call).  Raises if the reference library was not built."""
    library = ref()
    if library is None or not hasattr(library, "qref_fp4_swiglu"):
        raise RuntimeError("oracle/_ref/libqllm_ref.so is not built")
    sections = [np.ascontiguousarray(part).view(np.uint8).ravel()
                for matrix in (gate, up, down) for part in matrix]
    offsets, cursor = [], 0
    for section in sections:
        offsets.append(cursor)
        cursor += (section.size + 63) // 64 * 64
    record = np.zeros(cursor, dtype=np.uint8)
    for offset, section in zip(offsets, sections):
        record[offset: offset + section.size] = section
    offsets = np.array(offsets, dtype=np.uint64)
    inputs = np.ascontiguousarray(inputs, dtype=np.float32)
    rows = inputs.shape[0]
    out = np.zeros((rows, hidden), dtype=np.float32)
    seconds = c_double(0.0)
    library.qref_fp4_swiglu.restype = c_int
    library.qref_fp4_swiglu.argtypes = [
        c_void_p, c_uint64, c_void_p, c_uint32, c_uint32, c_void_p, c_uint32,
        c_void_p, c_uint32, c_int, c_uint32, ctypes.POINTER(c_double)]
    status = library.qref_fp4_swiglu(_p(record), record.size, _p(offsets), hidden,
                                     intermediate, _p(inputs), rows, _p(out), threads,
                                     int(bf16_intermediate), repeats,
                                     ctypes.byref(seconds))
    if status != 0:
        raise RuntimeError(f"reference FP4 executor failed ({status})")
    return out, seconds.value


# ---- numpy-facing wrappers ------------------------------------------------

def bf16_round(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even to bf16 precision, kept as float32 (numpy bit ops)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32).astype(np.uint64)
    special = (bits & 0x7f800000) == 0x7f800000
    rounded = (bits + 0x7fff + ((bits >> 16) & 1)) & 0xffff0000
    out = np.where(special, bits, rounded).astype(np.uint32)
    return out.view(np.float32).reshape(x.shape)


def bf16_bits(x: np.ndarray) -> np.ndarray:
    return (bf16_round(x).view(np.uint32) >> 16).astype(np.uint16)


def bf16_from_bits(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << 16).view(np.float32)


def fp4_linear_f64(codes, scales, scheme, rows, padded, act, bf16_output=False):
    act = np.ascontiguousarray(act, dtype=np.float32)
    batch = act.shape[0]
    out = np.empty((batch, rows), dtype=np.float32)
    oracle().qo_fp4_linear_f64(_p(codes), _p(scales), c_int(scheme),
                               c_uint32(rows), c_uint32(padded), _p(act),
                               c_uint32(batch), _p(out), c_int(bf16_output))
    return out


def fp4_linear_block32_q8(codes, scales, rows, padded, q8, act_scales,
                          bf16_output=False):
    batch = q8.shape[0]
    out = np.empty((batch, rows), dtype=np.float32)
    oracle().qo_fp4_linear_block32_q8(_p(codes), _p(scales), c_uint32(rows),
                                      c_uint32(padded), _p(q8), _p(act_scales),
                                      c_uint32(batch), _p(out),
                                      c_int(bf16_output))
    return out


def quantize_q8_rows(x, padded, bf16_input=False):
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, columns = x.shape
    q = np.empty((rows, padded), dtype=np.int8)
    s = np.empty(rows, dtype=np.float32)
    oracle().qo_quantize_q8_rows(_p(x), c_uint32(rows), c_uint32(columns),
                                 c_uint32(padded), c_int(bf16_input), _p(q), _p(s))
    return q, s


def fp4_embedding(codes, scales, scheme, columns, padded, tokens):
    tokens = np.ascontiguousarray(tokens, dtype=np.uint32)
    out = np.empty((len(tokens), columns), dtype=np.float32)
    oracle().qo_fp4_embedding(_p(codes), _p(scales), c_int(scheme),
                              c_uint32(columns), c_uint32(padded), _p(tokens),
                              c_uint32(len(tokens)), _p(out))
    return out


def rms_norm_rows(x, weight, eps, zero_centered=False, bf16_output=False):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    w = None if weight is None else np.ascontiguousarray(weight, dtype=np.float32)
    oracle().qo_rms_norm_rows(_p(x), _p(w) if w is not None else None, _p(out),
                              c_uint32(x.shape[0]), c_uint32(x.shape[1]),
                              c_float(eps), c_int(zero_centered),
                              c_int(bf16_output))
    return out


def silu_product(gate, up, bf16_activations=False):
    gate = np.ascontiguousarray(gate, dtype=np.float32)
    up = np.ascontiguousarray(up, dtype=np.float32)
    out = np.empty_like(gate)
    oracle().qo_silu_product(_p(gate), _p(up), _p(out), c_uint32(gate.size),
                             c_int(bf16_activations))
    return out


def head_norm_rope(x, weight, rotary_dim, position, eps, theta, bf16=False):
    x = np.array(x, dtype=np.float32, copy=True)
    w = None if weight is None else np.ascontiguousarray(weight, dtype=np.float32)
    oracle().qo_head_norm_rope(_p(x), _p(w) if w is not None else None,
                               c_uint32(x.size), c_uint32(rotary_dim),
                               c_uint32(position), c_float(eps), c_float(theta),
                               c_int(bf16))
    return x


def q4h_layer_bytes(page_tokens, kv_heads, head_dim):
    return oracle().qo_q4h_layer_bytes(page_tokens, kv_heads, head_dim)


def q4h_store(page: np.ndarray, layer, page_tokens, position, kv_head,
              kv_heads, head_dim, key, value):
    key = np.ascontiguousarray(key, dtype=np.float32)
    value = np.ascontiguousarray(value, dtype=np.float32)
    oracle().qo_q4h_store(_p(page), c_uint32(layer), c_uint32(page_tokens),
                          c_uint32(position), c_uint32(kv_head),
                          c_uint32(kv_heads), c_uint32(head_dim), _p(key),
                          _p(value))


def q4h_load(page: np.ndarray, layer, page_tokens, position, kv_head, kv_heads,
             head_dim):
    key = np.empty(head_dim, dtype=np.float32)
    value = np.empty(head_dim, dtype=np.float32)
    oracle().qo_q4h_load(_p(page), c_uint32(layer), c_uint32(page_tokens),
                         c_uint32(position), c_uint32(kv_head),
                         c_uint32(kv_heads), c_uint32(head_dim), _p(key),
                         _p(value))
    return key, value


def q8_layer_bytes(page_tokens, kv_heads, head_dim):
    return 2 * page_tokens * kv_heads * (head_dim + 2)


def q8_store(page: np.ndarray, layer_offset, page_tokens, position, kv_head,
             kv_heads, head_dim, key, value):
    key = np.ascontiguousarray(key, dtype=np.float32)
    value = np.ascontiguousarray(value, dtype=np.float32)
    oracle().qo_q8_store(_p(page), c_size_t(layer_offset), c_uint32(page_tokens),
                         c_uint32(position), c_uint32(kv_head),
                         c_uint32(kv_heads), c_uint32(head_dim), _p(key),
                         _p(value))


def q8_load(page: np.ndarray, layer_offset, page_tokens, position, kv_head,
            kv_heads, head_dim):
    key = np.empty(head_dim, dtype=np.float32)
    value = np.empty(head_dim, dtype=np.float32)
    oracle().qo_q8_load(_p(page), c_size_t(layer_offset), c_uint32(page_tokens),
                        c_uint32(position), c_uint32(kv_head),
                        c_uint32(kv_heads), c_uint32(head_dim), _p(key),
                        _p(value))
    return key, value


def attention_q8(shape: AttentionShape, queries, pages, layer_offset=0):
    queries = np.ascontiguousarray(queries, dtype=np.float32)
    out = np.empty((shape.rows, shape.query_heads, shape.head_dim), np.float32)
    table = _page_table(pages)
    oracle().qo_attention_q8_f64(ctypes.byref(shape), c_size_t(layer_offset),
                                 _p(queries), table, _p(out))
    return out


def quantize_queries_q8(queries, rows, query_heads, head_dim, stride):
    queries = np.ascontiguousarray(queries, dtype=np.float32)
    q8 = np.empty((rows, query_heads, head_dim), dtype=np.int8)
    scales = np.empty((rows, query_heads), dtype=np.float32)
    oracle().qo_quantize_queries_q8(_p(queries), c_uint32(rows),
                                    c_uint32(query_heads), c_uint32(head_dim),
                                    c_uint32(stride), _p(q8), _p(scales))
    return q8, scales


def _page_table(pages):
    table = (c_void_p * len(pages))(*[p.ctypes.data for p in pages])
    return table


def attention_q4h(shape: AttentionShape, queries, pages, kind="f64"):
    queries = np.ascontiguousarray(queries, dtype=np.float32)
    out = np.empty((shape.rows, shape.query_heads, shape.head_dim), np.float32)
    table = _page_table(pages)
    fn = (oracle().qo_attention_q4h_f64 if kind == "f64"
          else oracle().qo_attention_q4h_int8)
    fn(ctypes.byref(shape), _p(queries), table, _p(out))
    return out


def attention_f16(shape: AttentionShape, queries, pages, f16_probabilities=False):
    queries = np.ascontiguousarray(queries, dtype=np.float32)
    out = np.empty((shape.rows, shape.query_heads, shape.head_dim), np.float32)
    table = _page_table(pages)
    oracle().qo_attention_f16_f64(ctypes.byref(shape), _p(queries), table,
                                  c_int(f16_probabilities), _p(out))
    return out


def argmax(values):
    values = np.ascontiguousarray(values, dtype=np.float32)
    return oracle().qo_argmax(_p(values), c_uint32(values.size))


def presence_penalty(logits, emitted, penalty):
    """logits - penalty where emitted (a copy; qo_presence_penalty)."""
    out = np.ascontiguousarray(logits, dtype=np.float32).copy()
    emitted = np.ascontiguousarray(emitted, dtype=np.uint8)
    oracle().qo_presence_penalty(_p(out), _p(emitted), c_uint32(out.size),
                                 ctypes.c_float(penalty))
    return out


def topk(values, k):
    values = np.ascontiguousarray(values, dtype=np.float32)
    out_v = np.empty(k, dtype=np.float32)
    out_i = np.empty(k, dtype=np.uint32)
    n = oracle().qo_topk(_p(values), c_uint32(values.size), c_uint32(k),
                         _p(out_v), _p(out_i))
    return out_v[:n], out_i[:n]


def _entries(tokens, probabilities):
    n = len(tokens)
    array = (TokenProbability * n)()
    for i in range(n):
        array[i].token = int(tokens[i])
        array[i].probability = float(probabilities[i])
    return array


def make_sampling_distribution(logits, tokens, temperature_ppm, top_p_ppm,
                               min_p_ppm, lib="oracle"):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    tokens = np.ascontiguousarray(tokens, dtype=np.uint32)
    n = len(logits)
    count = c_uint32(0)
    if lib == "oracle":
        entries = (TokenProbability * max(n, 1))()
        status = oracle().qo_make_sampling_distribution(
            _p(logits), _p(tokens), c_uint32(n), c_uint32(temperature_ppm),
            c_uint32(top_p_ppm), c_uint32(min_p_ppm), entries,
            ctypes.byref(count))
        if status:
            return status, [], []
        return 0, [entries[i].token for i in range(count.value)], \
            [entries[i].probability for i in range(count.value)]
    out_t = np.empty(max(n, 1), dtype=np.uint32)
    out_p = np.empty(max(n, 1), dtype=np.float64)
    status = ref().qref_make_sampling_distribution(
        _p(logits), _p(tokens), c_uint32(n), c_uint32(temperature_ppm),
        c_uint32(top_p_ppm), c_uint32(min_p_ppm), _p(out_t), _p(out_p),
        ctypes.byref(count))
    if status:
        return status, [], []
    return 0, out_t[:count.value].tolist(), out_p[:count.value].tolist()


def sample_distribution(tokens, probabilities, uniform, lib="oracle"):
    out = c_uint32(0)
    if lib == "oracle":
        status = oracle().qo_sample_distribution(
            _entries(tokens, probabilities), c_uint32(len(tokens)),
            c_double(uniform), ctypes.byref(out))
    else:
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        p = np.ascontiguousarray(probabilities, dtype=np.float64)
        status = ref().qref_sample_distribution(_p(t), _p(p), c_uint32(len(t)),
                                                c_double(uniform),
                                                ctypes.byref(out))
    return status, out.value


def rejection_sample(proposal, target, draft, u_accept, u_correct, lib="oracle"):
    """target/draft: (tokens, probabilities). Returns (status, accepted, token, p, q)."""
    if lib == "oracle":
        result = RejectionResult()
        status = oracle().qo_rejection_sample(
            c_uint32(proposal), _entries(*target), c_uint32(len(target[0])),
            _entries(*draft), c_uint32(len(draft[0])), c_double(u_accept),
            c_double(u_correct), ctypes.byref(result))
        return (status, bool(result.accepted), result.token,
                result.target_probability, result.draft_probability)
    tt = np.ascontiguousarray(target[0], dtype=np.uint32)
    tp = np.ascontiguousarray(target[1], dtype=np.float64)
    dt = np.ascontiguousarray(draft[0], dtype=np.uint32)
    dp = np.ascontiguousarray(draft[1], dtype=np.float64)
    accepted = c_int(0)
    token = c_uint32(0)
    p = c_double(0)
    q = c_double(0)
    status = ref().qref_rejection_sample(
        c_uint32(proposal), _p(tt), _p(tp), c_uint32(len(tt)), _p(dt), _p(dp),
        c_uint32(len(dt)), c_double(u_accept), c_double(u_correct),
        ctypes.byref(accepted), ctypes.byref(token), ctypes.byref(p),
        ctypes.byref(q))
    return status, bool(accepted.value), token.value, p.value, q.value


def counter_uniform(seed, position, stream, index=0, lib="oracle"):
    if lib == "oracle":
        return oracle().qo_counter_uniform(seed, position, stream, index)
    return ref().qref_counter_uniform(seed, position, stream, index)


def accept_greedy(logits, drafts):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    drafts = np.ascontiguousarray(drafts, dtype=np.uint32)
    r = oracle().qo_accept_greedy(_p(logits), c_uint32(logits.shape[1]),
                                  _p(drafts), c_uint32(len(drafts)))
    return r.accepted, r.next_token


def accept_stochastic(targets, drafts_dist, drafts, seed, position):
    """targets: list of (tokens, probs) of length n+1; drafts_dist: length n."""
    n = len(drafts)
    t_arrays = [_entries(*t) for t in targets]
    d_arrays = [_entries(*d) for d in drafts_dist]
    t_ptrs = (POINTER(TokenProbability) * (n + 1))(
        *[ctypes.cast(a, POINTER(TokenProbability)) for a in t_arrays])
    d_ptrs = (POINTER(TokenProbability) * max(n, 1))(
        *[ctypes.cast(a, POINTER(TokenProbability)) for a in d_arrays])
    t_counts = np.array([len(t[0]) for t in targets], dtype=np.uint32)
    d_counts = np.array([len(d[0]) for d in drafts_dist], dtype=np.uint32)
    tokens = np.ascontiguousarray(drafts, dtype=np.uint32)
    r = oracle().qo_accept_stochastic(t_ptrs, _p(t_counts), d_ptrs,
                                      _p(d_counts), _p(tokens), c_uint32(n),
                                      c_uint64(seed), c_uint32(position))
    return r.status, r.accepted, r.next_token
