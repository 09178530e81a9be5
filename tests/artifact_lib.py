"""ctypes access to the artifact reader of libqllm_provider.so and, where it
has been built, to the same functions of the reference itself
(oracle/_ref/libqllm_ref_artifact.so: the reference's own sources behind a
flat C shim).  Both return (status code, text): the canonical dump on success,
the status message otherwise."""
import ctypes
import os
from ctypes import (POINTER, byref, c_char_p, c_int, c_int32, c_size_t, c_uint32,
                    c_uint64, c_void_p, create_string_buffer)

import qllm_provider as qp

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REFERENCE_LIBRARY = os.path.join(ROOT, "oracle", "_ref", "libqllm_ref_artifact.so")
CAPACITY = 1 << 22


def product():
    return qp.load()


_reference = None


def reference():
    """The reference's reader, or None when it was not built."""
    global _reference
    if _reference is None and os.path.exists(REFERENCE_LIBRARY):
        lib = ctypes.CDLL(REFERENCE_LIBRARY)
        lib.qref_sha256.argtypes = [c_void_p, c_size_t, c_void_p]
        lib.qref_model_descriptor_parse.argtypes = [
            c_char_p, c_size_t, c_char_p, c_uint64, c_char_p, c_size_t, POINTER(c_size_t)]
        lib.qref_model_descriptor_load.argtypes = [
            c_char_p, c_uint64, c_char_p, c_char_p, c_uint64, c_char_p, c_size_t,
            POINTER(c_size_t)]
        lib.qref_model_program_bind.argtypes = [
            c_char_p, c_size_t, c_char_p, c_uint64, c_char_p, c_int, c_char_p, c_size_t,
            POINTER(c_size_t)]
        lib.qref_artifact_open.argtypes = [c_char_p, c_uint32, c_int, POINTER(c_void_p),
                                           c_char_p, c_size_t]
        lib.qref_artifact_close.argtypes = [c_void_p]
        lib.qref_artifact_dump.argtypes = [c_void_p, c_char_p, c_size_t, POINTER(c_size_t)]
        lib.qref_artifact_tensor.argtypes = [c_void_p, c_char_p, POINTER(c_void_p),
                                             POINTER(c_uint64), c_char_p, c_size_t]
        _reference = lib
    return _reference


def _text(buffer, length):
    return buffer.raw[:min(length.value, CAPACITY - 1)].decode()


class Product:
    name = "product"

    @staticmethod
    def sha256(data: bytes) -> bytes:
        out = create_string_buffer(32)
        assert product().qllm_sha256(data, len(data), out) == 0
        return out.raw

    @staticmethod
    def sha256_portable(data: bytes) -> bytes:
        out = create_string_buffer(32)
        assert product().qllm_sha256_portable(data, len(data), out) == 0
        return out.raw

    @staticmethod
    def parse(text: bytes, content_hash: bytes, namespace_base: int):
        lib = product()
        buffer, length = create_string_buffer(CAPACITY), c_size_t()
        code = lib.qllm_model_descriptor_parse(text, len(text), content_hash,
                                               namespace_base, buffer, CAPACITY, byref(length))
        return (code, _text(buffer, length)) if code == 0 else (
            code, lib.qllm_provider_last_error().decode())

    @staticmethod
    def load(path, expected_bytes, expected_sha, content_hash, namespace_base):
        lib = product()
        buffer, length = create_string_buffer(CAPACITY), c_size_t()
        code = lib.qllm_model_descriptor_load(os.fsencode(path), expected_bytes, expected_sha,
                                              content_hash, namespace_base, buffer, CAPACITY,
                                              byref(length))
        return (code, _text(buffer, length)) if code == 0 else (
            code, lib.qllm_provider_last_error().decode())

    @staticmethod
    def bind(text: bytes, content_hash: bytes, namespace_base: int, providers: str,
             executable: bool):
        """Report of registering `providers` and binding the program to them."""
        lib = product()
        buffer, length = create_string_buffer(CAPACITY), c_size_t()
        code = lib.qllm_model_program_bind(text, len(text), content_hash, namespace_base,
                                           providers.encode(), int(executable), buffer,
                                           CAPACITY, byref(length))
        assert code == 0, lib.qllm_provider_last_error().decode()
        return _text(buffer, length)

    class Artifact:
        def __init__(self, root, mtp_draft_depth=0, map_tensors=True):
            self.lib = product()
            self.handle = c_void_p()
            self.code = self.lib.qllm_artifact_open(os.fsencode(root), mtp_draft_depth,
                                                    int(map_tensors), byref(self.handle))
            self.message = "" if self.code == 0 else self.lib.qllm_provider_last_error().decode()

        def dump(self):
            buffer, length = create_string_buffer(CAPACITY), c_size_t()
            assert self.lib.qllm_artifact_dump(self.handle, buffer, CAPACITY, byref(length)) == 0
            return _text(buffer, length)

        def tensor(self, name, check_header=True):
            record, size = c_void_p(), c_uint64()
            code = self.lib.qllm_artifact_tensor(self.handle, name.encode(), int(check_header),
                                                 byref(record), byref(size))
            if code:
                return code, self.lib.qllm_provider_last_error().decode()
            return 0, ctypes.string_at(record.value, size.value)

        def close(self):
            if self.handle:
                self.lib.qllm_artifact_close(self.handle)
                self.handle = c_void_p()


class Reference:
    name = "reference"

    @staticmethod
    def sha256(data: bytes) -> bytes:
        out = create_string_buffer(32)
        reference().qref_sha256(data, len(data), out)
        return out.raw

    @staticmethod
    def parse(text: bytes, content_hash: bytes, namespace_base: int):
        buffer, length = create_string_buffer(CAPACITY), c_size_t()
        code = reference().qref_model_descriptor_parse(
            text, len(text), content_hash, namespace_base, buffer, CAPACITY, byref(length))
        return code, _text(buffer, length)

    @staticmethod
    def load(path, expected_bytes, expected_sha, content_hash, namespace_base):
        buffer, length = create_string_buffer(CAPACITY), c_size_t()
        code = reference().qref_model_descriptor_load(
            os.fsencode(path), expected_bytes, expected_sha, content_hash, namespace_base,
            buffer, CAPACITY, byref(length))
        return code, _text(buffer, length)

    @staticmethod
    def bind(text: bytes, content_hash: bytes, namespace_base: int, providers: str,
             executable: bool):
        buffer, length = create_string_buffer(CAPACITY), c_size_t()
        reference().qref_model_program_bind(text, len(text), content_hash, namespace_base,
                                            providers.encode(), int(executable), buffer,
                                            CAPACITY, byref(length))
        return _text(buffer, length)

    class Artifact:
        def __init__(self, root, mtp_draft_depth=0, map_tensors=True):
            self.lib = reference()
            self.handle = c_void_p()
            message = create_string_buffer(4096)
            self.code = self.lib.qref_artifact_open(os.fsencode(root), mtp_draft_depth,
                                                    int(map_tensors), byref(self.handle),
                                                    message, 4096)
            self.message = message.value.decode() if self.code else ""

        def dump(self):
            buffer, length = create_string_buffer(CAPACITY), c_size_t()
            self.lib.qref_artifact_dump(self.handle, buffer, CAPACITY, byref(length))
            return _text(buffer, length)

        def tensor(self, name, check_header=True):
            record, size = c_void_p(), c_uint64()
            message = create_string_buffer(4096)
            code = self.lib.qref_artifact_tensor(self.handle, name.encode(), byref(record),
                                                 byref(size), message, 4096)
            if code:
                return code, message.value.decode()
            return 0, ctypes.string_at(record.value, size.value)

        def close(self):
            if self.handle:
                self.lib.qref_artifact_close(self.handle)
                self.handle = c_void_p()
