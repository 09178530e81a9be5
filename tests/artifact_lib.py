"""ctypes access to the artifact reader of libqllm_provider.so and, where it
has been built, to the reader of the reference itself, each behind the same
printing shim (oracle/artifact_shim.cpp: oracle/libqllm_provider_probe.so over
the product's library, oracle/_ref/libqllm_ref_artifact.so over the reference's
own sources).  Both return (status code, text): the canonical dump on success,
the status message otherwise."""
import ctypes
import os
from ctypes import (POINTER, byref, c_char_p, c_int, c_int32, c_size_t, c_uint32,
                    c_uint64, c_void_p, create_string_buffer)

import qllm_provider as qp

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REFERENCE_LIBRARY = os.path.join(ROOT, "oracle", "_ref", "libqllm_ref_artifact.so")
PROBE_LIBRARY = os.path.join(ROOT, "oracle", "libqllm_provider_probe.so")
CAPACITY = 1 << 22


def product():
    return qp.load()


def _shim(path, prefix):
    """The printing shim at `path` with its functions under neutral names."""
    lib = ctypes.CDLL(path)

    class Functions:
        pass

    functions = Functions()
    for name, argtypes, restype in (
            ("sha256", [c_void_p, c_size_t, c_void_p], None),
            ("model_descriptor_parse", [c_char_p, c_size_t, c_char_p, c_uint64, c_char_p,
                                        c_size_t, POINTER(c_size_t)], c_int),
            ("model_descriptor_load", [c_char_p, c_uint64, c_char_p, c_char_p, c_uint64,
                                       c_char_p, c_size_t, POINTER(c_size_t)], c_int),
            ("model_program_bind", [c_char_p, c_size_t, c_char_p, c_uint64, c_char_p, c_int,
                                    c_char_p, c_size_t, POINTER(c_size_t)], None),
            ("artifact_open", [c_char_p, c_uint32, c_int, POINTER(c_void_p), c_char_p,
                               c_size_t], c_int),
            ("artifact_close", [c_void_p], None),
            ("artifact_dump", [c_void_p, c_char_p, c_size_t, POINTER(c_size_t)], None),
            ("artifact_tensor", [c_void_p, c_char_p, POINTER(c_void_p), POINTER(c_uint64),
                                 c_char_p, c_size_t], c_int)):
        function = getattr(lib, prefix + name)
        function.argtypes, function.restype = argtypes, restype
        setattr(functions, name, function)
    return functions


_reference = None
_probe = None


def reference():
    """The reference's reader, or None when it was not built."""
    global _reference
    if _reference is None and os.path.exists(REFERENCE_LIBRARY):
        _reference = _shim(REFERENCE_LIBRARY, "qref_")
    return _reference


def probe():
    """The shim over the product's reader (built by `make -C oracle probe`)."""
    global _probe
    if _probe is None:
        product()       # libqllm_provider.so first: the shim links against it
        if not os.path.exists(PROBE_LIBRARY):
            raise FileNotFoundError(f"{PROBE_LIBRARY} is missing: make -C oracle probe")
        _probe = _shim(PROBE_LIBRARY, "qprobe_")
    return _probe


def _text(buffer, length):
    return buffer.raw[:min(length.value, CAPACITY - 1)].decode()


class _ShimReader:
    """parse / load / bind and an artifact handle through a printing shim."""

    def __init__(self, functions):
        self.functions = functions

    def parse(self, text: bytes, content_hash: bytes, namespace_base: int):
        buffer, length = create_string_buffer(CAPACITY), c_size_t()
        code = self.functions().model_descriptor_parse(
            text, len(text), content_hash, namespace_base, buffer, CAPACITY, byref(length))
        return code, _text(buffer, length)

    def load(self, path, expected_bytes, expected_sha, content_hash, namespace_base):
        buffer, length = create_string_buffer(CAPACITY), c_size_t()
        code = self.functions().model_descriptor_load(
            os.fsencode(path), expected_bytes, expected_sha, content_hash, namespace_base,
            buffer, CAPACITY, byref(length))
        return code, _text(buffer, length)

    def bind(self, text: bytes, content_hash: bytes, namespace_base: int, providers: str,
             executable: bool):
        """Report of registering `providers` and binding the program to them."""
        buffer, length = create_string_buffer(CAPACITY), c_size_t()
        self.functions().model_program_bind(text, len(text), content_hash, namespace_base,
                                            providers.encode(), int(executable), buffer,
                                            CAPACITY, byref(length))
        return _text(buffer, length)


class _ShimArtifact:
    def __init__(self, functions, root, mtp_draft_depth=0, map_tensors=True):
        self.lib = functions
        self.handle = c_void_p()
        message = create_string_buffer(4096)
        self.code = self.lib.artifact_open(os.fsencode(root), mtp_draft_depth,
                                           int(map_tensors), byref(self.handle),
                                           message, 4096)
        self.message = message.value.decode() if self.code else ""

    def dump(self):
        buffer, length = create_string_buffer(CAPACITY), c_size_t()
        self.lib.artifact_dump(self.handle, buffer, CAPACITY, byref(length))
        return _text(buffer, length)

    def tensor(self, name, check_header=True):
        record, size = c_void_p(), c_uint64()
        message = create_string_buffer(4096)
        code = self.lib.artifact_tensor(self.handle, name.encode(), byref(record),
                                        byref(size), message, 4096)
        if code:
            return code, message.value.decode()
        return 0, ctypes.string_at(record.value, size.value)

    def close(self):
        if self.handle:
            self.lib.artifact_close(self.handle)
            self.handle = c_void_p()


class Product:
    """The product's reader: parse / load / bind results printed by the probe
    shim, the artifact handle through the library's own C ABI (open, tensor,
    close) with the index dump from the shim's handle on the same directory."""
    name = "product"
    _reader = _ShimReader(probe)
    parse = staticmethod(_reader.parse)
    load = staticmethod(_reader.load)
    bind = staticmethod(_reader.bind)

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

    class Artifact:
        def __init__(self, root, mtp_draft_depth=0, map_tensors=True):
            self.lib = product()
            self.handle = c_void_p()
            self.code = self.lib.qllm_artifact_open(os.fsencode(root), mtp_draft_depth,
                                                    int(map_tensors), byref(self.handle))
            self.message = "" if self.code == 0 else self.lib.qllm_provider_last_error().decode()
            self.printer = (_ShimArtifact(probe(), root, mtp_draft_depth, False)
                            if self.code == 0 else None)

        def dump(self):
            return self.printer.dump()

        def tensor(self, name, check_header=True):
            record, size = c_void_p(), c_uint64()
            code = self.lib.qllm_artifact_tensor(self.handle, name.encode(), int(check_header),
                                                 byref(record), byref(size))
            if code:
                return code, self.lib.qllm_provider_last_error().decode()
            return 0, ctypes.string_at(record.value, size.value)

        def close(self):
            if self.printer:
                self.printer.close()
                self.printer = None
            if self.handle:
                self.lib.qllm_artifact_close(self.handle)
                self.handle = c_void_p()


class Reference:
    name = "reference"
    _reader = _ShimReader(reference)
    parse = staticmethod(_reader.parse)
    load = staticmethod(_reader.load)
    bind = staticmethod(_reader.bind)

    @staticmethod
    def sha256(data: bytes) -> bytes:
        out = create_string_buffer(32)
        reference().sha256(data, len(data), out)
        return out.raw

    class Artifact(_ShimArtifact):
        def __init__(self, root, mtp_draft_depth=0, map_tensors=True):
            super().__init__(reference(), root, mtp_draft_depth, map_tensors)
