"""The Expert Pack v1 reader of the provider library (host only): manifest,
model program binding, pack index, mapped tensor store, record headers.

A small artifact is written by tests/artifact_writer.py (the published
layout) and read by the product and by the reference's own reader built from
its sources (oracle/_ref): both must list the same packs, tensors and program
and hand out the same record bytes, and must turn down the same broken
artifacts with the same status.
"""
import hashlib
import json
import os
import struct

import numpy as np
import pytest

import artifact_lib as al
import artifact_writer as aw
import oracle_lib as ol
import step_oracle

needs_reference = pytest.mark.skipif(al.reference() is None,
                                     reason="oracle/_ref/libqllm_ref_artifact.so is not built")
READERS = [al.Product] + ([al.Reference] if al.reference() is not None else [])


def tiny_model(seed=5):
    rng = np.random.default_rng(seed)
    return step_oracle.TinyModel(rng, 256, 512, 2, 8, 2, 128, 256, ol.SCALE_UE8M0_BLOCK32,
                                 output_gated=True, qk_norm=True, zero_centered=True,
                                 rotary_dim=64)


@pytest.fixture(scope="module")
def artifact(tmp_path_factory):
    root = tmp_path_factory.mktemp("artifact")
    manifest = aw.write_artifact(str(root), tiny_model())
    return str(root), manifest


def rewrite_manifest(root, edit):
    path = os.path.join(root, "manifest.json")
    with open(path) as handle:
        manifest = json.load(handle)
    edit(manifest)
    with open(path, "w") as handle:
        json.dump(manifest, handle)


def test_index_program_and_records(artifact):
    root, manifest = artifact
    opened = al.Product.Artifact(root)
    assert opened.code == 0, opened.message
    rows = [line.split("\t") for line in opened.dump().splitlines()]
    packs = [r for r in rows if r[0] == "pack"]
    assert len(packs) == 1 and packs[0][1:3] == ["dense-00000.qpack", "dense"]
    tensors = {r[1]: r for r in rows if r[0] == "tensor"}
    assert set(tensors) == {entry["name"] for entry in manifest["tensors"]}
    head = tensors["lm_head.weight"]
    assert head[5:8] == ["FP4_E2M1", "3", "256x256"]
    assert int(head[9]) == 256 * 256 // 2 and int(head[11]) == 256 * 256 // 32
    assert ["exact_decode_parameter", "draft_depth", "4"] in rows
    # every record: header agrees with the index, bytes are the file's
    with open(os.path.join(root, "dense-00000.qpack"), "rb") as handle:
        pack = handle.read()
    for entry in manifest["tensors"]:
        code, record = opened.tensor(entry["name"])
        assert code == 0, record
        assert record == pack[entry["offset"]:entry["offset"] + entry["stored_bytes"]]
        assert hashlib.sha256(record[256:]).hexdigest() == entry["payload_sha256"]
    assert opened.tensor("no.such.tensor") == (
        4, "artifact tensor is absent from the dense index")
    opened.close()


def test_draft_depth_policy(artifact):
    root, _ = artifact
    for reader in READERS:
        opened = reader.Artifact(root, mtp_draft_depth=2, map_tensors=False)
        assert opened.code == 0, opened.message
        dump = opened.dump()
        assert "exact_decode_parameter\tdraft_depth\t2\n" in dump
        assert [line.split("\t")[2:] for line in dump.splitlines()
                if line.startswith("exact_decode\t")] == [["2", "3"]]
        opened.close()
        refused = reader.Artifact(root, mtp_draft_depth=4096, map_tensors=False)
        assert (refused.code, refused.message) == (
            4, "artifact cannot apply the requested MTP depth")


@needs_reference
def test_reads_like_the_reference(artifact):
    root, manifest = artifact
    mine, theirs = al.Product.Artifact(root), al.Reference.Artifact(root)
    assert (mine.code, theirs.code) == (0, 0), (mine.message, theirs.message)
    assert mine.dump() == theirs.dump()
    for entry in manifest["tensors"]:
        assert mine.tensor(entry["name"]) == theirs.tensor(entry["name"])
    assert mine.tensor("absent", check_header=False) == theirs.tensor("absent")
    mine.close()
    theirs.close()


def broken_artifacts():
    """(name, edit of the directory after writing) -> expected status code."""
    def manifest_edit(edit):
        return lambda root: rewrite_manifest(root, edit)

    def set_path(value):
        return manifest_edit(lambda m: m["model_program"].__setitem__("path", value))

    def tensor_edit(index, key, value):
        return manifest_edit(lambda m: m["tensors"][index].__setitem__(key, value))

    def flip_pack_byte(root):
        path = os.path.join(root, "dense-00000.qpack")
        with open(path, "r+b") as handle:
            handle.seek(5000)
            byte = handle.read(1)
            handle.seek(5000)
            handle.write(bytes([byte[0] ^ 0x40]))

    def truncate_pack(root):
        path = os.path.join(root, "dense-00000.qpack")
        os.truncate(path, os.path.getsize(path) - 4096)

    def append_to_program(root):
        with open(os.path.join(root, "runtime-model.tsv"), "ab") as handle:
            handle.write(b"\n")

    return [
        ("no COMPLETED marker", lambda root: os.remove(os.path.join(root, "COMPLETED")), 4),
        ("no manifest", lambda root: os.remove(os.path.join(root, "manifest.json")), 4),
        ("manifest is not JSON", lambda root: open(os.path.join(root, "manifest.json"), "w").write("{"), 4),
        ("other format name", manifest_edit(lambda m: m["format"].__setitem__("name", "other-pack")), 4),
        ("other format version", manifest_edit(lambda m: m["format"].__setitem__("version", 2)), 4),
        ("format version is a string", manifest_edit(lambda m: m["format"].__setitem__("version", "1")), 4),
        ("no integrity", manifest_edit(lambda m: m.pop("integrity")), 4),
        ("short content hash", manifest_edit(lambda m: m["integrity"].__setitem__("content_sha256", "abcd")), 4),
        ("bad hex digit", manifest_edit(lambda m: m["integrity"].__setitem__("content_sha256", "g" * 64)), 4),
        ("program format", manifest_edit(lambda m: m["model_program"].__setitem__("format", "v2")), 4),
        ("program path escapes", set_path("../runtime-model.tsv"), 4),
        ("program path is absolute", set_path("/etc/passwd"), 4),
        ("program path is empty", set_path(""), 4),
        ("program grew", append_to_program, 4),
        ("program checksum", manifest_edit(lambda m: m["model_program"].__setitem__("sha256", "0" * 64)), 4),
        ("pack kind", manifest_edit(lambda m: m["packs"][0].__setitem__("kind", "sparse")), 4),
        ("pack size", manifest_edit(lambda m: m["packs"][0].__setitem__("bytes", 4096)), 4),
        ("pack listed twice", manifest_edit(lambda m: m["packs"].append(dict(m["packs"][0]))), 4),
        ("pack name escapes", manifest_edit(lambda m: m["packs"][0].__setitem__("name", "../x.qpack")), 4),
        ("pack truncated", truncate_pack, 4),
        ("pack byte flipped", flip_pack_byte, 8),
        ("tensor in unknown pack", tensor_edit(0, "pack", "dense-00001.qpack"), 4),
        ("tensor offset outside pack", tensor_edit(1, "offset", 1 << 40), 4),
        ("tensor larger than pack", tensor_edit(1, "stored_bytes", 1 << 40), 4),
        ("tensor encoding", tensor_edit(2, "stored_dtype", "FP8"), 4),
        ("tensor without shape", tensor_edit(2, "source_shape", []), 4),
        ("tensor dimension too wide", tensor_edit(2, "source_shape", [1 << 33]), 4),
        ("tensor negative offset", tensor_edit(2, "offset", -4096), 4),
        ("tensor data outside record", manifest_edit(
            lambda m: m["tensors"][3]["sections"]["data"].__setitem__("bytes", 1 << 30)), 4),
        ("tensor scales outside record", manifest_edit(
            lambda m: m["tensors"][0]["sections"]["scales"].__setitem__("offset", 1 << 30)), 4),
        ("tensor listed twice", manifest_edit(lambda m: m["tensors"].append(dict(m["tensors"][0]))), 4),
        ("expert records in a dense artifact", manifest_edit(lambda m: m["experts"].append({})), 4),
        ("no experts key", manifest_edit(lambda m: m.pop("experts")), 4),
    ]


@pytest.mark.parametrize("name,edit,code", broken_artifacts(),
                         ids=[case[0] for case in broken_artifacts()])
def test_broken_artifacts_are_turned_down(tmp_path, name, edit, code):
    root = str(tmp_path / "artifact")
    aw.write_artifact(root, tiny_model())
    edit(root)
    results = []
    for reader in READERS:
        opened = reader.Artifact(root)
        assert opened.code == code, (reader.name, opened.code, opened.message)
        results.append(opened.message)
    if len(results) == 2:
        mine, theirs = results
        # messages agree, except the wording of JSON-level complaints
        prefix = "invalid model artifact: "
        generic = ("must be", "missing required key", "JSON", "json", "expected")
        if any(word in theirs for word in generic):
            assert mine.split(": ")[0] == theirs.split(": ")[0]
        else:
            assert mine == theirs, (mine, theirs)
        assert mine.startswith(prefix) or not theirs.startswith(prefix)


def test_record_header_checks(tmp_path):
    """The 256-byte record header against its index entry: each corrupted field
    is named.  (The pack checksum in the manifest is updated with the
    corruption, so that the header check is what turns the record down.)"""
    root = str(tmp_path / "artifact")
    manifest = aw.write_artifact(root, tiny_model())
    pack_path = os.path.join(root, "dense-00000.qpack")
    entry = next(e for e in manifest["tensors"] if e["name"] == "lm_head.weight")
    with open(pack_path, "rb") as handle:
        original = handle.read()
    header = aw.DENSE_HEADER

    def with_header(**changes):
        fields = list(header.unpack(original[entry["offset"]:entry["offset"] + header.size]))
        names = ["magic", "version", "header_bytes", "flags", "quant_abi", "rank", "dim0",
                 "dim1", "dim2", "dim3", "dim4", "record_bytes", "data_offset", "data_bytes",
                 "scale_offset", "scale_bytes", "name_hash", "payload_hash"]
        for key, value in changes.items():
            fields[names.index(key)] = value
        blob = bytearray(original)
        blob[entry["offset"]:entry["offset"] + header.size] = header.pack(*fields)
        return blob

    cases = [
        (with_header(magic=b"EPDENS02"), "unknown dense record ABI"),
        (with_header(version=2), "unknown dense record ABI"),
        (with_header(header_bytes=128), "invalid dense header fields"),
        (with_header(record_bytes=entry["stored_bytes"] + 4096), "dense record/manifest size mismatch"),
        (with_header(flags=12), "dense record is not row-major"),
        (with_header(flags=1), "FP4 dense flags are incomplete"),
        (with_header(rank=6), "invalid dense rank"),
        (with_header(dim4=7), "invalid dense rank padding"),
        (with_header(dim0=128), "dense shape mismatch"),
        (with_header(quant_abi=1), "dense quantisation ABI mismatch"),
        (with_header(name_hash=bytes(32)), "dense name hash mismatch"),
        (with_header(data_bytes=100), "dense data section mismatch"),
        (with_header(scale_offset=entry["sections"]["scales"]["offset"] + 256), "dense scale section mismatch"),
        (with_header(payload_hash=bytes(32)), "dense payload/manifest checksum mismatch"),
    ]
    padded = bytearray(original)
    padded[entry["offset"] + 200] = 1
    cases.append((padded, "dense header padding is nonzero"))
    for blob, message in cases:
        with open(pack_path, "wb") as handle:
            handle.write(blob)
        rewrite_manifest(root, lambda m: m["packs"][0].__setitem__(
            "sha256", hashlib.sha256(blob).hexdigest()))
        opened = al.Product.Artifact(root)
        assert opened.code == 0, opened.message
        assert opened.tensor("lm_head.weight") == (4, message + ": lm_head.weight")
        assert opened.tensor("model.norm.weight")[0] == 0      # the other records are fine
        opened.close()
