"""The built shared libraries exist in-tree and export every symbol the public
headers declare (no compute calls: this runs without a GPU)."""
import ctypes
import os
import re

import qllm_hip
import qllm_provider

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(qllm_[a-z0-9_]+)\s*\(", text)))


def test_kernel_library_exports_every_declared_symbol():
    library = ctypes.CDLL(qllm_hip.LIBRARY_PATH)
    names = declared_symbols("qllm_kernels.h")
    assert len(names) >= 25
    for name in names:
        assert hasattr(library, name), name
    assert sorted(qllm_hip.SIGNATURES) == names


def test_provider_library_exports_every_declared_symbol():
    library = ctypes.CDLL(qllm_provider.LIBRARY_PATH)
    names = declared_symbols("qllm_provider.h")
    for name in names:
        assert hasattr(library, name), name
    assert sorted(qllm_provider.SIGNATURES) == names


def test_capability_table_covers_the_dense_program():
    # capability strings the reference's dense program requires
    # (runtime/tools/dense_fp4_provider.cpp:996-1052)
    names = qllm_provider.capabilities()
    for required in ("embedding.lookup.fp4-block32.v1",
                     "block.full-attention.output-gated.v1",
                     "ffn.swiglu.dense.fp4-block32.v1",
                     "head.rmsnorm.token-select.fp4-block32.v1",
                     "decode.mtp.dense-full-attention.fp4-block32.exact.v2"):
        assert required in names


def test_version_and_error_text_without_a_device():
    library = qllm_hip.load()
    assert library.qllm_version().startswith(b"qllm-hip gfx950")
    # argument validation happens before any HIP call
    status = library.qllm_fp4_gemm_bf16(None, None, 0, None, 0, None, 0, None)
    assert status == 4
    assert b"invalid" in library.qllm_last_error()
    assert library.qllm_q4h_layer_bytes(256, 8, 128) == 256 * 8 * 2 * 66
