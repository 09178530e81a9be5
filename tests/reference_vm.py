"""ctypes access to oracle/_ref/libqllm_ref_vm.so: the reference's own common
VM (provider registry, program executor with its sessions and exact-decode
handle validation, artifact reader), compiled from the reference's sources,
with this repository's provider linked in as its one provider module."""
import ctypes
import os
from ctypes import (POINTER, byref, c_char_p, c_float, c_int, c_size_t, c_uint32,
                    c_uint64, c_void_p, create_string_buffer)

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIBRARY = os.path.join(ROOT, "oracle", "_ref", "libqllm_ref_vm.so")


class VmError(RuntimeError):
    pass


_library = None


def built():
    return os.path.exists(LIBRARY)


def library():
    """The library, or None when it was not built."""
    global _library
    if _library is None and os.path.exists(LIBRARY):
        lib = ctypes.CDLL(LIBRARY)
        lib.qvm_open.restype = c_void_p
        lib.qvm_open.argtypes = [c_char_p, c_uint32, c_uint32, c_char_p, c_uint32,
                                 c_uint32, c_char_p, c_size_t]
        lib.qvm_select_session.argtypes = [c_void_p, c_uint32]
        lib.qvm_end_session.argtypes = [c_void_p]
        lib.qvm_close.argtypes = [c_void_p]
        lib.qvm_error.restype = c_char_p
        lib.qvm_error.argtypes = [c_void_p]
        lib.qvm_service.argtypes = [c_void_p, c_char_p, c_size_t, POINTER(c_uint32),
                                    POINTER(c_uint32), POINTER(c_int), POINTER(c_int)]
        lib.qvm_begin_session.argtypes = [c_void_p, c_void_p, c_void_p, c_uint32]
        lib.qvm_execute.argtypes = [c_void_p, c_void_p, c_void_p, c_uint32,
                                    POINTER(c_uint32)]
        lib.qvm_exact_available.argtypes = [c_void_p]
        lib.qvm_synchronize.argtypes = [c_void_p, c_void_p, c_uint32, c_uint32, c_int]
        lib.qvm_exact_decode.argtypes = [c_void_p, c_uint32, c_uint32, c_uint32, c_void_p,
                                         POINTER(c_uint32), POINTER(c_uint32),
                                         POINTER(c_uint32)]
        lib.qvm_copy_logits.argtypes = [c_void_p, c_uint32, c_void_p]
        lib.qvm_telemetry.restype = c_uint64
        lib.qvm_telemetry.argtypes = [c_void_p, c_char_p]
        _library = lib
    return _library


class Machine:
    def __init__(self, root, max_context, kv_page_tokens, kv_cache_dtype="artifact",
                 mtp_draft_depth=0, vocabulary=0, capacity=1):
        self.lib = library()
        self.vocabulary = vocabulary
        message = create_string_buffer(2048)
        self.handle = self.lib.qvm_open(os.fsencode(root), max_context, kv_page_tokens,
                                        kv_cache_dtype.encode(), mtp_draft_depth, capacity,
                                        message, 2048)
        if not self.handle:
            raise VmError(message.value.decode())

    def _check(self, code):
        if code:
            raise VmError(self.lib.qvm_error(self.handle).decode())

    def close(self):
        if self.handle:
            self.lib.qvm_close(self.handle)
            self.handle = None

    def service(self):
        dtype = create_string_buffer(64)
        page, chunk, mtp, sampling = c_uint32(), c_uint32(), c_int(), c_int()
        self.lib.qvm_service(self.handle, dtype, 64, byref(page), byref(chunk), byref(mtp),
                             byref(sampling))
        return dict(kv_dtype=dtype.value.decode(), kv_page_tokens=page.value,
                    prefill_chunk_tokens=chunk.value, mtp_enabled=bool(mtp.value),
                    sampling_supported=bool(sampling.value))

    def select(self, session):
        """Which session (0 .. capacity; the last has no slot to count on) the
        calls that follow address."""
        self._check(self.lib.qvm_select_session(self.handle, session))

    def end_session(self):
        self._check(self.lib.qvm_end_session(self.handle))

    def begin_session(self, **parameters):
        names = (c_char_p * len(parameters))(*[n.encode() for n in parameters])
        values = np.array(list(parameters.values()), dtype=np.uint64)
        self._check(self.lib.qvm_begin_session(self.handle, names, values.ctypes.data,
                                               len(parameters)))

    def execute(self, tokens, first_position):
        tokens = np.ascontiguousarray(tokens, dtype=np.uint32)
        positions = np.arange(first_position, first_position + len(tokens), dtype=np.uint32)
        selected = c_uint32()
        self._check(self.lib.qvm_execute(self.handle, tokens.ctypes.data,
                                         positions.ctypes.data, len(tokens), byref(selected)))
        return selected.value

    def exact_available(self):
        return bool(self.lib.qvm_exact_available(self.handle))

    def synchronize(self, next_tokens, first_target_position, produce_final_draft):
        next_tokens = np.ascontiguousarray(next_tokens, dtype=np.uint32)
        self._check(self.lib.qvm_synchronize(self.handle, next_tokens.ctypes.data,
                                             len(next_tokens), first_target_position,
                                             int(produce_final_draft)))

    def exact_decode(self, guaranteed_token, position, context_limit):
        emitted = np.zeros(16, dtype=np.uint32)
        count, following, advanced = c_uint32(), c_uint32(), c_uint32()
        self._check(self.lib.qvm_exact_decode(self.handle, guaranteed_token, position,
                                              context_limit, emitted.ctypes.data, byref(count),
                                              byref(following), byref(advanced)))
        return emitted[:count.value].tolist(), following.value, advanced.value

    def logits(self, rows):
        out = np.empty((rows, self.vocabulary), dtype=np.float32)
        self._check(self.lib.qvm_copy_logits(self.handle, rows, out.ctypes.data))
        return out

    def telemetry(self, name):
        return self.lib.qvm_telemetry(self.handle, name.encode())
