"""ctypes binding of the provider's C ABI (include/qllm_provider.h).
Plumbing for tests and the benchmark; raises when the library is missing."""
from __future__ import annotations

import ctypes
import os
from ctypes import (POINTER, Structure, c_char_p, c_double, c_float, c_int32,
                    c_size_t, c_uint32, c_uint64, c_void_p)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.path.join(os.path.dirname(_HERE), "lib",
                            "libqllm_provider.so")


class ProviderError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"qllm provider status {code}: {message}")
        self.code = code


class DenseGeometry(Structure):
    _fields_ = [("hidden", c_uint32), ("intermediate", c_uint32),
                ("layers", c_uint32), ("query_heads", c_uint32),
                ("kv_heads", c_uint32), ("head_dim", c_uint32),
                ("rotary_dim", c_uint32), ("vocabulary", c_uint32),
                ("rope_theta", c_float), ("norm_epsilon", c_float),
                ("output_gated", c_int32), ("qk_norm", c_int32),
                ("zero_centered_norm", c_int32), ("scale_scheme", c_uint32),
                ("kv_encoding", c_uint32), ("kv_page_tokens", c_uint32),
                ("max_context", c_uint32), ("draft_depth", c_uint32),
                ("mtp_layers", c_uint32), ("draft_vocabulary", c_uint32),
                ("prefill_chunk_rows", c_uint32), ("activation_q8", c_uint32)]


SIGNATURES = {
    "qllm_provider_last_error": (c_char_p, []),
    "qllm_provider_create": (c_void_p, [POINTER(DenseGeometry)]),
    "qllm_provider_destroy": (None, [c_void_p]),
    "qllm_provider_capabilities": (c_uint32, [c_void_p, c_size_t]),
    "qllm_provider_stage_tensor": (c_int32, [c_void_p, c_char_p, c_char_p, c_uint32, c_uint32, c_uint32, c_void_p, c_size_t, c_void_p, c_size_t]),
    "qllm_provider_prepare": (c_int32, [c_void_p, c_char_p]),
    "qllm_provider_prepare_exact_decode": (c_int32, [c_void_p, c_char_p]),
    "qllm_provider_load_synthetic_weights": (c_int32, [c_void_p, c_uint64]),
    "qllm_provider_prefill_synthetic_kv": (c_int32, [c_void_p, c_uint32, c_uint64]),
    "qllm_provider_begin_request": (c_int32, [c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_uint64]),
    "qllm_provider_begin_request_with": (c_int32, [c_void_p, c_void_p, c_void_p, c_uint32]),
    "qllm_provider_synchronize": (c_int32, [c_void_p, c_uint32, c_uint32]),
    "qllm_provider_execute_program": (c_int32, [c_void_p, c_void_p, c_void_p, c_uint32, POINTER(c_uint32)]),
    "qllm_provider_synchronize_batch": (c_int32, [c_void_p, c_void_p, c_uint32, c_uint32, c_int32]),
    "qllm_provider_copy_matrix_rows": (c_int32, [c_void_p, c_char_p, c_uint32, c_uint32, c_void_p, c_void_p]),
    "qllm_provider_set_drafts": (c_int32, [c_void_p, c_void_p, c_uint32, c_void_p, c_void_p, c_void_p]),
    "qllm_provider_verify": (c_int32, [c_void_p, c_uint32, c_uint32, c_uint32, c_void_p, POINTER(c_uint32), POINTER(c_uint32), POINTER(c_uint32)]),
    "qllm_provider_run_target": (c_int32, [c_void_p, c_void_p, c_uint32, c_uint32]),
    "qllm_provider_capture_target": (c_int32, [c_void_p, c_void_p, c_uint32, c_uint32]),
    "qllm_provider_replay_target": (c_int32, [c_void_p]),
    "qllm_provider_synchronize_stream": (c_int32, [c_void_p]),
    "qllm_provider_copy_logits": (c_int32, [c_void_p, c_uint32, c_void_p]),
    "qllm_provider_copy_hidden": (c_int32, [c_void_p, c_uint32, c_void_p]),
    "qllm_provider_time_kernel": (c_int32, [c_void_p, c_char_p, c_uint32, c_uint32, POINTER(c_double), POINTER(c_uint64)]),
    "qllm_provider_kv_page_bytes": (c_uint64, [c_void_p]),
    "qllm_provider_copy_kv_page": (c_int32, [c_void_p, c_uint32, c_void_p]),
    "qllm_provider_copy_mtp_state": (c_int32, [c_void_p, c_void_p, c_void_p]),
    "qllm_provider_drafts": (c_uint32, [c_void_p, c_void_p, c_uint32]),
    "qllm_provider_draft_vocabulary": (c_uint32, [c_void_p]),
    "qllm_provider_logits": (c_void_p, [c_void_p]),
    "qllm_provider_hidden": (c_void_p, [c_void_p]),
    "qllm_provider_stream": (c_void_p, [c_void_p]),
    "qllm_provider_weight_bytes": (c_uint64, [c_void_p]),
    "qllm_provider_telemetry": (c_uint64, [c_void_p, c_char_p]),
    "qllm_sampling_make_distribution": (c_int32, [c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_void_p, c_void_p, POINTER(c_uint32)]),
    "qllm_sampling_sample": (c_int32, [c_void_p, c_void_p, c_uint32, c_double, POINTER(c_uint32)]),
    "qllm_sampling_rejection": (c_int32, [c_uint32, c_void_p, c_void_p, c_uint32, c_void_p, c_void_p, c_uint32, c_double, c_double, POINTER(c_int32), POINTER(c_uint32), POINTER(c_double), POINTER(c_double)]),
    "qllm_sampling_counter_uniform": (c_double, [c_uint64, c_uint32, c_uint32, c_uint32]),
    "qllm_provider_create_from_artifact": (c_void_p, [c_char_p, c_uint32, c_uint32, c_char_p, c_uint32]),
    "qllm_provider_prefill": (c_int32, [c_void_p, c_void_p, c_uint32, c_uint32, POINTER(c_uint32)]),
    "qllm_sha256": (c_int32, [c_void_p, c_size_t, c_void_p]),
    "qllm_sha256_portable": (c_int32, [c_void_p, c_size_t, c_void_p]),
    "qllm_artifact_open": (c_int32, [c_char_p, c_uint32, c_int32, POINTER(c_void_p)]),
    "qllm_artifact_close": (None, [c_void_p]),
    "qllm_artifact_tensor": (c_int32, [c_void_p, c_char_p, c_int32, POINTER(c_void_p), POINTER(c_uint64)]),
}

_library = None


def load():
    global _library
    if _library is None:
        if not os.path.exists(LIBRARY_PATH):
            raise FileNotFoundError(
                f"{LIBRARY_PATH} is missing: build it with "
                "`make -C quantum-llm_amd` (or __graft_entry__.build())")
        library = ctypes.CDLL(LIBRARY_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            function = getattr(library, name)
            function.restype = restype
            function.argtypes = argtypes
        _library = library
    return _library


def _check(status):
    if status != 0:
        raise ProviderError(status, load().qllm_provider_last_error().decode())


class Provider:
    """Thin object wrapper over the C handle."""

    def __init__(self, **geometry):
        self.geometry = DenseGeometry(**geometry)
        self.lib = load()
        self.handle = self.lib.qllm_provider_create(ctypes.byref(self.geometry))
        if not self.handle:
            raise ProviderError(10, self.lib.qllm_provider_last_error().decode())

    @classmethod
    def from_artifact(cls, root, geometry, max_context=0, kv_page_tokens=0,
                      kv_cache_dtype=None, mtp_draft_depth=0):
        """A provider loaded and prepared from an Expert Pack v1 directory;
        `geometry` (keyword dictionary) only describes it to this wrapper."""
        self = cls.__new__(cls)
        self.geometry = DenseGeometry(**geometry)
        self.lib = load()
        self.handle = self.lib.qllm_provider_create_from_artifact(
            os.fsencode(root), max_context, kv_page_tokens,
            kv_cache_dtype.encode() if kv_cache_dtype else None, mtp_draft_depth)
        if not self.handle:
            raise ProviderError(10, self.lib.qllm_provider_last_error().decode())
        return self

    def close(self):
        if self.handle:
            self.lib.qllm_provider_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def stage_fp4(self, role, codes, scales, rows, columns, quant_abi):
        _check(self.lib.qllm_provider_stage_tensor(
            self.handle, role.encode(), b"FP4_E2M1", quant_abi, rows, columns,
            codes.ctypes.data, codes.nbytes, scales.ctypes.data, scales.nbytes))

    def stage_f32(self, role, values):
        _check(self.lib.qllm_provider_stage_tensor(
            self.handle, role.encode(), b"F32", 0, values.size, 0,
            values.ctypes.data, values.nbytes, None, 0))

    def prepare(self, capability):
        _check(self.lib.qllm_provider_prepare(self.handle, capability.encode()))

    def prepare_exact_decode(self, capability):
        _check(self.lib.qllm_provider_prepare_exact_decode(
            self.handle, capability.encode()))

    def load_synthetic_weights(self, seed):
        _check(self.lib.qllm_provider_load_synthetic_weights(self.handle, seed))

    def prefill_synthetic_kv(self, tokens, seed):
        _check(self.lib.qllm_provider_prefill_synthetic_kv(self.handle, tokens, seed))

    def begin_request(self, temperature_ppm=0, top_p_ppm=1000000, top_k=0,
                      min_p_ppm=0, seed=0):
        _check(self.lib.qllm_provider_begin_request(
            self.handle, temperature_ppm, top_p_ppm, top_k, min_p_ppm, seed))

    def begin_request_with(self, **parameters):
        """create_request_state with the request's parameter map given by name."""
        import numpy as np
        names = (c_char_p * len(parameters))(*[n.encode() for n in parameters])
        values = np.array(list(parameters.values()), dtype=np.uint64)
        _check(self.lib.qllm_provider_begin_request_with(
            self.handle, names, values.ctypes.data, len(parameters)))

    def prefill(self, tokens, first_position=0):
        """Prompt prefill; returns the greedy prediction after the prompt."""
        import numpy as np
        tokens = np.ascontiguousarray(tokens, dtype=np.uint32)
        predicted = c_uint32()
        _check(self.lib.qllm_provider_prefill(self.handle, tokens.ctypes.data, tokens.size,
                                              first_position, ctypes.byref(predicted)))
        return predicted.value

    def execute_program(self, tokens, first_position):
        """The prepared program, operation by operation, on `tokens` at
        consecutive positions; returns the head's token for the last row."""
        import numpy as np
        tokens = np.ascontiguousarray(tokens, dtype=np.uint32)
        positions = np.arange(first_position, first_position + len(tokens),
                              dtype=np.uint32)
        selected = c_uint32()
        _check(self.lib.qllm_provider_execute_program(
            self.handle, tokens.ctypes.data, positions.ctypes.data, len(tokens),
            ctypes.byref(selected)))
        return selected.value

    def synchronize_batch(self, next_tokens, first_target_position, produce_final_draft):
        import numpy as np
        next_tokens = np.ascontiguousarray(next_tokens, dtype=np.uint32)
        _check(self.lib.qllm_provider_synchronize_batch(
            self.handle, next_tokens.ctypes.data, len(next_tokens),
            first_target_position, int(produce_final_draft)))

    def synchronize(self, token, position):
        _check(self.lib.qllm_provider_synchronize(self.handle, token, position))

    def set_drafts(self, tokens, distributions=None):
        import numpy as np
        tokens = np.ascontiguousarray(tokens, dtype=np.uint32)
        if distributions is None:
            _check(self.lib.qllm_provider_set_drafts(
                self.handle, tokens.ctypes.data, len(tokens), None, None, None))
            return
        counts = np.array([len(d[0]) for d in distributions], dtype=np.uint32)
        flat_tokens = np.concatenate(
            [np.asarray(d[0], dtype=np.uint32) for d in distributions])
        flat_probs = np.concatenate(
            [np.asarray(d[1], dtype=np.float64) for d in distributions])
        _check(self.lib.qllm_provider_set_drafts(
            self.handle, tokens.ctypes.data, len(tokens), counts.ctypes.data,
            flat_tokens.ctypes.data, flat_probs.ctypes.data))

    def verify(self, guaranteed_token, position, context_limit):
        import numpy as np
        emitted = np.zeros(16, dtype=np.uint32)
        count = c_uint32(0)
        next_token = c_uint32(0)
        advanced = c_uint32(0)
        _check(self.lib.qllm_provider_verify(
            self.handle, guaranteed_token, position, context_limit,
            emitted.ctypes.data, ctypes.byref(count), ctypes.byref(next_token),
            ctypes.byref(advanced)))
        return emitted[:count.value].tolist(), next_token.value, advanced.value

    def run_target(self, tokens, first_position):
        import numpy as np
        tokens = np.ascontiguousarray(tokens, dtype=np.uint32)
        _check(self.lib.qllm_provider_run_target(
            self.handle, tokens.ctypes.data, len(tokens), first_position))

    def capture_target(self, tokens, first_position):
        import numpy as np
        tokens = np.ascontiguousarray(tokens, dtype=np.uint32)
        _check(self.lib.qllm_provider_capture_target(
            self.handle, tokens.ctypes.data, len(tokens), first_position))

    def replay_target(self):
        _check(self.lib.qllm_provider_replay_target(self.handle))

    def synchronize_stream(self):
        _check(self.lib.qllm_provider_synchronize_stream(self.handle))

    def logits(self, rows):
        """Copy of the logits [rows, vocabulary] as a numpy array."""
        import numpy as np
        out = np.empty((rows, self.geometry.vocabulary), dtype=np.float32)
        _check(self.lib.qllm_provider_copy_logits(self.handle, rows,
                                                  out.ctypes.data))
        return out

    def hidden(self, rows):
        import numpy as np
        out = np.empty((rows, self.geometry.hidden), dtype=np.float32)
        _check(self.lib.qllm_provider_copy_hidden(self.handle, rows,
                                                  out.ctypes.data))
        return out

    def time_kernel(self, which, rounds, context_tokens=0):
        """(average microseconds per launch, launches) from HIP events."""
        microseconds = c_double(0.0)
        launches = c_uint64(0)
        _check(self.lib.qllm_provider_time_kernel(
            self.handle, which.encode(), rounds, context_tokens,
            ctypes.byref(microseconds), ctypes.byref(launches)))
        return microseconds.value, launches.value

    def kv_page(self, page_index):
        import numpy as np
        out = np.empty(self.lib.qllm_provider_kv_page_bytes(self.handle),
                       dtype=np.uint8)
        _check(self.lib.qllm_provider_copy_kv_page(self.handle, page_index,
                                                   out.ctypes.data))
        return out

    def matrix_rows(self, name, first_row, rows, padded_columns, scheme):
        """(codes [rows, K/2] u8, scales) of a weight matrix's rows, row-major."""
        import numpy as np
        codes = np.empty((rows, padded_columns // 2), dtype=np.uint8)
        scales = (np.empty((rows, padded_columns // 16), dtype=np.uint16) if scheme == 1
                  else np.empty((rows, padded_columns // 32), dtype=np.uint8))
        _check(self.lib.qllm_provider_copy_matrix_rows(
            self.handle, name.encode(), first_row, rows, codes.ctypes.data,
            scales.ctypes.data))
        return codes, scales

    def mtp_state(self):
        """(last hidden [hidden], draft logits [draft_vocabulary]) of the proposer."""
        import numpy as np
        hidden = np.empty(self.geometry.hidden, dtype=np.float32)
        logits = np.empty(self.lib.qllm_provider_draft_vocabulary(self.handle),
                          dtype=np.float32)
        _check(self.lib.qllm_provider_copy_mtp_state(
            self.handle, hidden.ctypes.data, logits.ctypes.data))
        return hidden, logits

    def drafts(self):
        import numpy as np
        tokens = np.zeros(16, dtype=np.uint32)
        count = self.lib.qllm_provider_drafts(self.handle, tokens.ctypes.data, 16)
        return tokens[:count].tolist()

    def weight_bytes(self):
        return self.lib.qllm_provider_weight_bytes(self.handle)

    def telemetry(self, name):
        return self.lib.qllm_provider_telemetry(self.handle, name.encode())

    def stream(self):
        return self.lib.qllm_provider_stream(self.handle)


def capabilities():
    library = load()
    buffer = ctypes.create_string_buffer(8192)
    count = library.qllm_provider_capabilities(buffer, len(buffer))
    raw = buffer.raw
    names = [part.decode() for part in raw.split(b"\0") if part][:count]
    return names


# ---- host sampling mathematics (no device needed) ----------------------------

def _arrays(tokens, probabilities):
    import numpy as np
    t = np.ascontiguousarray(tokens, dtype=np.uint32)
    p = np.ascontiguousarray(probabilities, dtype=np.float64)
    return t, p


def make_sampling_distribution(sorted_logits, sorted_tokens, temperature_ppm,
                               top_p_ppm, min_p_ppm):
    """Returns (tokens, probabilities); raises ProviderError on invalid input."""
    import numpy as np
    logits = np.ascontiguousarray(sorted_logits, dtype=np.float32)
    tokens = np.ascontiguousarray(sorted_tokens, dtype=np.uint32)
    out_tokens = np.zeros(max(len(tokens), 1), dtype=np.uint32)
    out_probabilities = np.zeros(max(len(tokens), 1), dtype=np.float64)
    count = c_uint32(0)
    _check(load().qllm_sampling_make_distribution(
        logits.ctypes.data, tokens.ctypes.data, len(tokens), temperature_ppm,
        top_p_ppm, min_p_ppm, out_tokens.ctypes.data,
        out_probabilities.ctypes.data, ctypes.byref(count)))
    return (out_tokens[:count.value].tolist(),
            out_probabilities[:count.value].tolist())


def sample_distribution(tokens, probabilities, uniform):
    t, p = _arrays(tokens, probabilities)
    token = c_uint32(0)
    _check(load().qllm_sampling_sample(t.ctypes.data, p.ctypes.data, len(t),
                                       uniform, ctypes.byref(token)))
    return token.value


def rejection_sample(proposal, target, draft, acceptance_uniform,
                     correction_uniform):
    """target / draft: (tokens, probabilities).  Returns (accepted, token,
    target probability, draft probability) of the proposal."""
    tt, tp = _arrays(*target)
    dt, dp = _arrays(*draft)
    accepted, token = c_int32(0), c_uint32(0)
    p, q = c_double(0.0), c_double(0.0)
    _check(load().qllm_sampling_rejection(
        proposal, tt.ctypes.data, tp.ctypes.data, len(tt), dt.ctypes.data,
        dp.ctypes.data, len(dt), acceptance_uniform, correction_uniform,
        ctypes.byref(accepted), ctypes.byref(token), ctypes.byref(p),
        ctypes.byref(q)))
    return bool(accepted.value), token.value, p.value, q.value


def counter_uniform(seed, position, stream, index=0):
    return load().qllm_sampling_counter_uniform(seed, position, stream, index)
