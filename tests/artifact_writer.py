"""Writes a small Expert Pack v1 artifact directory from host tensors, for the
artifact reader's tests.

The layout is the published one (docs/expert-pack-v1.md:8-36 of the
reference): `manifest.json`, `runtime-model.tsv` (schema-3 program, records as
runtime/src/model_descriptor.cpp:560-700 parses them), one dense QPack file of
4 KiB-aligned records, each a 256-byte little-endian header
(compiler/expert_pack/constants.py:72-92: magic, version, header bytes, flags,
quant ABI, rank, five dimensions, record bytes, data and scale ranges, SHA-256
of the name, SHA-256 of the payload) followed by 256-byte-aligned sections,
and `COMPLETED`.  The program is the dense full-attention one the reference's
compiler emits (compiler/expert_pack/adapters.py:1422-1760) without the
vision and recurrent operations.
"""
import hashlib
import json
import os
import struct

import numpy as np

PACK_ALIGNMENT = 4096
SECTION_ALIGNMENT = 256
HEADER_BYTES = 256
DENSE_HEADER = struct.Struct("<8sHHIIIIIIIIQQQQQ32s32s")
FLAG_ROW_MAJOR, FLAG_SYMMETRIC, FLAG_PER_ROW_SCALES = 1, 4, 8

# the value ABIs the artifact compiler declares (compiler/expert_pack/adapters.py:111-113)
TOKEN_ABI = "batch.token-id.u32.host.v1"
POSITION_ABI = "batch.position.u32.host.v1"
HIDDEN_ABI = "batch.hidden.f32.cuda.v1"


def _align(value, alignment):
    return (value + alignment - 1) // alignment * alignment


def f32_bits(value):
    return int(np.float32(value).view(np.uint32))


class PackWriter:
    """Accumulates dense records; `entries` is the manifest's tensor index."""

    def __init__(self, name="dense-00000.qpack"):
        self.name = name
        self.blob = bytearray()
        self.entries = []

    def _record(self, name, shape, quant_abi, flags, stored_dtype, data, scales):
        data_offset = HEADER_BYTES
        scale_offset = _align(data_offset + len(data), SECTION_ALIGNMENT) if scales else 0
        end = scale_offset + len(scales) if scales else data_offset + len(data)
        record_bytes = _align(end, PACK_ALIGNMENT)
        payload = bytearray(record_bytes - HEADER_BYTES)
        payload[0:len(data)] = data
        if scales:
            payload[scale_offset - HEADER_BYTES:scale_offset - HEADER_BYTES + len(scales)] = scales
        payload_hash = hashlib.sha256(payload).digest()
        dims = list(shape) + [0] * (5 - len(shape))
        header = DENSE_HEADER.pack(
            b"EPDENS01", 1, HEADER_BYTES, flags, quant_abi, len(shape), *dims,
            record_bytes, data_offset, len(data), scale_offset, len(scales),
            hashlib.sha256(name.encode()).digest(), payload_hash)
        offset = len(self.blob)
        assert offset % PACK_ALIGNMENT == 0
        self.blob += header + bytes(HEADER_BYTES - len(header)) + payload
        self.entries.append({
            "name": name, "pack": self.name, "offset": offset,
            "stored_bytes": record_bytes, "stored_dtype": stored_dtype,
            "quant_abi": quant_abi, "source_shape": list(shape),
            "sections": {"data": {"offset": data_offset, "bytes": len(data)},
                         "scales": {"offset": scale_offset, "bytes": len(scales)}},
            "payload_sha256": payload_hash.hex()})

    def add_f32(self, name, values):
        values = np.ascontiguousarray(values, dtype=np.float32)
        self._record(name, values.shape, 0, FLAG_ROW_MAJOR, "F32", values.tobytes(), b"")

    def add_fp4(self, name, codes, scales, rows, columns):
        """codes [rows, padded/2] uint8, scales [rows, padded/32] UE8M0."""
        codes = np.ascontiguousarray(codes, dtype=np.uint8)
        scales = np.ascontiguousarray(scales, dtype=np.uint8)
        padded = _align(columns, 32)
        assert codes.size == rows * padded // 2 and scales.size == rows * padded // 32
        self._record(name, (rows, columns), 3,
                     FLAG_ROW_MAJOR | FLAG_SYMMETRIC | FLAG_PER_ROW_SCALES,
                     "FP4_E2M1", codes.tobytes(), scales.tobytes())


def dense_program(model, tensor_names, mtp=True, draft_depth=4, draft_vocabulary=0,
                  max_context=4096, architecture="tiny.dense.fp4", activation_input=None):
    """runtime-model.tsv text for a TinyModel; `tensor_names` is filled with
    the tensor name -> (kind, payload) map the pack must hold."""
    m = model
    gated = m.output_gated
    attention = ("block.full-attention.output-gated.v1" if gated
                 else "block.full-attention.standard-gqa.v1")
    kernels = [("embedding.lookup.fp4-block32.v1", 1), (attention, 1),
               ("ffn.swiglu.dense.fp4-block32.v1", 1),
               ("head.rmsnorm.token-select.fp4-block32.v1", 1)]
    exact = "decode.mtp.dense-full-attention.fp4-block32.exact.v2"
    if mtp:
        kernels.append((exact, 2))
    # the activation contract as the compiler writes it
    # (compiler/expert_pack/compile.py:256-279): bf16 input is an attribute plus
    # a required kernel, Q8 - the default - is the absence of both
    if activation_input is None:
        activation_input = "q8" if getattr(m, "activation_q8", False) else "bf16"
    if activation_input == "bf16":
        kernels.append(("dense.activation-input.bfloat16.v1", 1))
    d, Q, KV, H, I, V = (m.head_dim, m.query_heads, m.kv_heads, m.hidden,
                         m.intermediate, m.vocabulary)
    q_rows = Q * d * (2 if gated else 1)

    def fp4(name, pair, rows, columns):
        tensor_names[name] = ("fp4", pair, rows, columns)
        return name

    def f32(name, values):
        tensor_names[name] = ("f32", values)
        return name

    lines = ["expert-runtime-model-v1",
             f"model\t3\t{architecture}\t{V}\t{max_context}\t{H}"]
    attributes = [
        ("attention_heads", Q), ("kv_heads", KV), ("head_dim", d),
        ("full_attention_layers", m.layers),
        ("norm_epsilon_f32_bits", f32_bits(m.eps)),
        ("rope_theta_f32_bits", f32_bits(m.rope_theta)),
        ("rotary_dimension", m.rotary_dim),
        ("zero_centered_norm", int(m.zero_centered)),
        ("mtp_layers", 1 if mtp else 0)]
    if activation_input == "bf16":
        attributes.append(("dense_activation_input_bf16", 1))
    lines += [f"attribute\t{key}\t{value}" for key, value in attributes]
    embedding = fp4("model.embed_tokens.weight", m.embedding, V, H)
    final_norm = f32("model.norm.weight", m.final_norm)
    head = fp4("lm_head.weight", m.head, V, H)
    lines += [f"model_tensor\ttoken_embedding\t{embedding}",
              f"model_tensor\tfinal_norm\t{final_norm}",
              f"model_tensor\toutput_head\t{head}",
              f"program_input\ttoken_ids\trequest.token_ids\t{TOKEN_ABI}",
              f"program_input\tpositions\trequest.positions\t{POSITION_ABI}",
              f"program_output\tnext_token_ids\tresponse.token_ids\t{TOKEN_ABI}"]
    lines += [f"kernel\t{capability}\t{abi}" for capability, abi in kernels]

    def block_tensors(prefix, weights):
        names = [("input_norm", f32(prefix + "input_layernorm.weight", weights["input_norm"])),
                 ("query_projection", fp4(prefix + "self_attn.q_proj.weight", weights["query"], q_rows, H)),
                 ("key_projection", fp4(prefix + "self_attn.k_proj.weight", weights["key"], KV * d, H)),
                 ("value_projection", fp4(prefix + "self_attn.v_proj.weight", weights["value"], KV * d, H)),
                 ("output_projection", fp4(prefix + "self_attn.o_proj.weight", weights["output"], H, Q * d))]
        if m.qk_norm:
            names += [("query_norm", f32(prefix + "self_attn.q_norm.weight", weights["query_norm"])),
                      ("key_norm", f32(prefix + "self_attn.k_norm.weight", weights["key_norm"]))]
        ffn = [("input_norm", f32(prefix + "post_attention_layernorm.weight", weights["post_attention_norm"])),
               ("gate_projection", fp4(prefix + "mlp.gate_proj.weight", weights["gate"], I, H)),
               ("up_projection", fp4(prefix + "mlp.up_proj.weight", weights["up"], I, H)),
               ("down_projection", fp4(prefix + "mlp.down_proj.weight", weights["down"], H, I))]
        return names, ffn

    if mtp:
        lines.append(f"exact_decode\t{exact}\t2\t{draft_depth + 1}")
        parameters = [("source_mtp_layers", 1), ("draft_depth", draft_depth),
                      ("draft_vocabulary_size", draft_vocabulary or min(V, 65536)),
                      ("mtp_kv_encoding", 1), ("embedding_first", 1), ("post_norm", 1)]
        lines += [f"exact_decode_parameter\t{key}\t{value}" for key, value in parameters]
        w = m.mtp
        bindings = [("token_embedding", embedding), ("output_head", head),
                    ("fusion_projection", fp4("mtp.fc.weight", w["fusion"], H, 2 * H)),
                    ("embedding_norm", f32("mtp.pre_fc_norm_embedding.weight", w["embedding_norm"])),
                    ("hidden_norm", f32("mtp.pre_fc_norm_hidden.weight", w["hidden_norm"])),
                    ("draft_norm", f32("mtp.norm.weight", w["draft_norm"]))]
        attention_names, ffn_names = block_tensors("mtp.layers.0.", w)
        bindings += [("layer.0." + role, name) for role, name in attention_names]
        bindings += [("layer.0." + ("post_attention_norm" if role == "input_norm" else role), name)
                     for role, name in ffn_names]
        lines += [f"exact_decode_tensor\t{role}\t{name}" for role, name in bindings]
    for layer in range(m.layers):
        lines.append(f"layer\t{layer}\t{attention}\t1\t-\t0")

    operations = []

    def operation(layer, capability, tensors, inputs, outputs):
        index = len(operations)
        operations.append(index)
        lines.append(f"operation\t{index}\t{'-' if layer is None else layer}\t{capability}\t1\t-\t0")
        lines.extend(f"operation_tensor\t{index}\t{role}\t{name}" for role, name in tensors)
        lines.extend(f"operation_input\t{index}\t{port}\t{value}\t{abi}" for port, value, abi in inputs)
        lines.extend(f"operation_output\t{index}\t{port}\t{value}\t{abi}" for port, value, abi in outputs)

    operation(None, "embedding.lookup.fp4-block32.v1", [("weight", embedding)],
              [("token_ids", "request.token_ids", TOKEN_ABI)],
              [("hidden", "hidden.0", HIDDEN_ABI)])
    for layer, block in enumerate(m.blocks):
        attention_names, ffn_names = block_tensors(f"model.layers.{layer}.", block)
        after = f"layer.{layer}.after_attention"
        operation(layer, attention, attention_names,
                  [("hidden", f"hidden.{layer}", HIDDEN_ABI),
                   ("positions", "request.positions", POSITION_ABI)],
                  [("hidden", after, HIDDEN_ABI)])
        operation(layer, "ffn.swiglu.dense.fp4-block32.v1", ffn_names,
                  [("hidden", after, HIDDEN_ABI)],
                  [("hidden", f"hidden.{layer + 1}", HIDDEN_ABI)])
    operation(None, "head.rmsnorm.token-select.fp4-block32.v1",
              [("norm", final_norm), ("weight", head)],
              [("hidden", f"hidden.{m.layers}", HIDDEN_ABI)],
              [("token_ids", "response.token_ids", TOKEN_ABI)])
    return "\n".join(lines) + "\n"


def write_artifact(root, model, mtp=True, draft_depth=4, draft_vocabulary=0,
                   max_context=4096, program_text=None, mutate_manifest=None,
                   completed=True, activation_input=None):
    """Writes the directory; returns the manifest dictionary."""
    os.makedirs(root, exist_ok=True)
    tensors = {}
    text = dense_program(model, tensors, mtp=mtp, draft_depth=draft_depth,
                         draft_vocabulary=draft_vocabulary, max_context=max_context,
                         activation_input=activation_input)
    if program_text is not None:
        text = program_text
    pack = PackWriter()
    for name, item in tensors.items():
        if item[0] == "f32":
            pack.add_f32(name, item[1])
        else:
            (codes, scales), rows, columns = item[1], item[2], item[3]
            pack.add_fp4(name, codes, scales, rows, columns)
    with open(os.path.join(root, pack.name), "wb") as handle:
        handle.write(pack.blob)
    program = text.encode()
    with open(os.path.join(root, "runtime-model.tsv"), "wb") as handle:
        handle.write(program)
    manifest = {
        "schema": "expert-pack-manifest-v1",
        "format": {"name": "expert-pack", "version": 1},
        "integrity": {"algorithm": "sha256",
                      "content_sha256": hashlib.sha256(bytes(pack.blob) + program).hexdigest()},
        "model_program": {"format": "expert-runtime-model-v1", "path": "runtime-model.tsv",
                          "bytes": len(program), "sha256": hashlib.sha256(program).hexdigest()},
        "packs": [{"name": pack.name, "kind": "dense", "bytes": len(pack.blob),
                   "sha256": hashlib.sha256(pack.blob).hexdigest()}],
        "tensors": pack.entries,
        "experts": [],
    }
    if mutate_manifest is not None:
        mutate_manifest(manifest)
    with open(os.path.join(root, "manifest.json"), "w") as handle:
        json.dump(manifest, handle, indent=1, sort_keys=True)
    if completed:
        with open(os.path.join(root, "COMPLETED"), "w") as handle:
            handle.write("ok\n")
    return manifest
