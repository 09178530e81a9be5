"""The model-program parser and SHA-256 of the provider library (host only).

Pinned by: the FIPS 180-4 example digests and hashlib; the three programs the
reference's own tests parse, with the facts those tests assert
(tests/golden/model_programs/README.md); and, record for record, the
reference's own parser built from its sources (oracle/_ref) over those
programs, a generated dense program and a few thousand mutations of them:
same status code, same message, same descriptor.
"""
import hashlib
import os

import numpy as np
import pytest

import artifact_lib as al
import artifact_writer as aw
import oracle_lib as ol
import step_oracle

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "model_programs")
needs_reference = pytest.mark.skipif(al.reference() is None,
                                     reason="oracle/_ref/libqllm_ref_artifact.so is not built")


def golden(name):
    with open(os.path.join(GOLDEN, name), "rb") as handle:
        return handle.read()


def digest(first_byte):
    return bytes([first_byte]) + bytes(31)


def lines_of(dump):
    return [line.split("\t") for line in dump.splitlines()]


def tiny_program(mtp=True):
    rng = np.random.default_rng(3)
    model = step_oracle.TinyModel(rng, 256, 512, 2, 8, 2, 128, 256, ol.SCALE_UE8M0_BLOCK32,
                                  output_gated=True, qk_norm=True, zero_centered=True,
                                  rotary_dim=64)
    return aw.dense_program(model, {}, mtp=mtp).encode()


# ---- SHA-256 -----------------------------------------------------------------

def test_sha256_known_answers():
    # FIPS 180-4 examples: "abc", the empty message, the 448-bit message
    known = {
        b"abc": "ba7816bf8f01cfea414140de5dae2223b00361a396177a9cb410ff61f20015ad",
        b"": "e3b0c44298fc1c149afbf4c8996fb92427ae41e4649b934ca495991b7852b855",
        b"abcdbcdecdefdefgefghfghighijhijkijkljklmklmnlmnomnopnopq":
            "248d6a61d20638b8e5c026930c3e6039a33ce45964ff2167f6ecedd419db06c1",
    }
    for message, want in known.items():
        assert al.Product.sha256(message).hex() == want
        assert al.Product.sha256_portable(message).hex() == want


def test_sha256_matches_hashlib_across_block_boundaries():
    rng = np.random.default_rng(1)
    for size in [*range(0, 200), 1000, 4095, 4096, 4097, 1 << 20]:
        data = rng.integers(0, 256, size, dtype=np.uint8).tobytes()
        want = hashlib.sha256(data).digest()
        # with the CPU's SHA instructions where present, and without
        assert al.Product.sha256(data) == want, size
        assert al.Product.sha256_portable(data) == want, size


# ---- the reference's own fixtures --------------------------------------------

def test_schema1_fixture_facts():
    code, dump = al.Product.parse(golden("schema1_hybrid_sparse.tsv"), digest(0xa5), 0x9000)
    assert code == 0
    rows = lines_of(dump)
    assert rows[0] == ["model", "1", "fixture.hybrid.sparse", "64001", "262144", "6144"]
    assert rows[1] == ["content_hash", "a5" + "00" * 31]
    components = [r for r in rows if r[0] == "component"]
    assert len(components) == 1
    assert components[0][1:6] == ["decoder", str(0x9000), "2", "1000", "7"]
    assert components[0][-1] == "fp4.fixture.e2m1.group64"
    layers = [r for r in rows if r[0] == "layer"]
    assert layers[0][4] == "-" and layers[-1][4:] == ["decoder", "1"]
    duplicate = golden("schema1_hybrid_sparse.tsv") + b"layer_parameter\t1\twindow\t2048\n"
    code, message = al.Product.parse(duplicate, digest(0xa5), 0x9000)
    assert code == 4 and message == "malformed model descriptor line 14"


def test_schema2_fixture_facts():
    code, dump = al.Product.parse(golden("schema2_vendor_moe.tsv"), digest(0x5a), 0x4100)
    assert code == 0
    rows = lines_of(dump)
    assert rows[0][1] == "2"
    assert ["router_parameter", "decoder", "groups", "8"] in rows
    assert ["model_tensor", "token_embedding", "model.embed.weight"] in rows
    assert ["operation_tensor", "0", "input_norm", "model.layers.0.norm.weight"] in rows
    assert len([r for r in rows if r[0] == "operation"]) == 3


def test_schema3_fixture_facts_and_rejections():
    text = golden("schema3_callable_program.tsv")
    code, dump = al.Product.parse(text, digest(0x93), 0x9300)
    assert code == 0
    operations = [r for r in lines_of(dump) if r[0] == "operation"]
    model_level = str(2 ** 32 - 1)
    assert operations[0][2] == model_level and operations[-1][2] == model_level

    def rejected(old, new, message):
        assert old in text
        code, got = al.Product.parse(text.replace(old, new, 1), digest(0x93), 0x9300)
        assert (code, got) == (4, message)

    # the five corruptions the reference's test applies to the parsed descriptor
    rejected(b"operation_input\t1\thidden\tembedded.hidden", b"operation_input\t1\thidden\tfuture.hidden",
             "schema v3 operation input is unavailable or has the wrong ABI")
    rejected(b"operation_output\t1\thidden\ttransformed.hidden",
             b"operation_output\t1\thidden\tembedded.hidden",
             "schema v3 operation output has multiple producers")
    rejected(b"operation_input\t1\thidden\tembedded.hidden\tfixture.scalar.u64.v1",
             b"operation_input\t1\thidden\tembedded.hidden\tfixture.scalar.u32.v1",
             "schema v3 operation input is unavailable or has the wrong ABI")
    rejected(b"kernel\tfixture.exact-decode.v1\t1\n", b"",
             "exact decode program is invalid or unsupported")
    rejected(b"exact_decode\tfixture.exact-decode.v1\t1\t2", b"exact_decode\tfixture.exact-decode.v1\t1\t1",
             "exact decode program is invalid or unsupported")


def test_header_namespace_and_completeness():
    text = golden("schema1_hybrid_sparse.tsv")
    assert al.Product.parse(text, digest(1), 0) == (4, "model descriptor namespace base is zero")
    assert al.Product.parse(b"something-else\n" + text, digest(1), 1) == (
        4, "unknown model descriptor artifact header")
    assert al.Product.parse(b"expert-runtime-model-v1\n", digest(1), 1) == (
        4, "model descriptor artifact is incomplete")
    assert al.Product.parse(b"", digest(1), 1) == (4, "model descriptor artifact is incomplete")
    # blank lines and CRLF endings are tolerated; line numbers count every line
    crlf = text.replace(b"\n", b"\r\n\r\n")
    assert al.Product.parse(crlf, digest(0xa5), 0x9000)[1] == al.Product.parse(
        text, digest(0xa5), 0x9000)[1]
    broken = crlf.replace(b"kernel\tblock.fixture.windowed.v3\t3", b"kernel\tblock.fixture.windowed.v3\t+3")
    assert al.Product.parse(broken, digest(0xa5), 0x9000) == (4, "malformed model descriptor line 9")


def test_load_binds_size_and_checksum(tmp_path):
    text = golden("schema1_hybrid_sparse.tsv")
    path = tmp_path / "runtime-model.tsv"
    path.write_bytes(text)
    sha = hashlib.sha256(text).digest()
    code, dump = al.Product.load(path, len(text), sha, digest(0xa5), 0x9000)
    assert code == 0 and dump == al.Product.parse(text, digest(0xa5), 0x9000)[1]
    wrong = bytes([sha[0] ^ 1]) + sha[1:]
    assert al.Product.load(path, len(text), wrong, digest(0xa5), 0x9000) == (
        4, "model descriptor artifact checksum mismatch")
    assert al.Product.load(path, len(text) + 1, sha, digest(0xa5), 0x9000) == (
        4, "model descriptor artifact size is invalid")
    assert al.Product.load(tmp_path / "absent.tsv", len(text), sha, digest(0xa5), 0x9000) == (
        4, "model descriptor artifact size is invalid")


def test_generated_dense_program_parses():
    code, dump = al.Product.parse(tiny_program(), digest(7), 0x77)
    assert code == 0
    rows = lines_of(dump)
    assert ["attribute", "attention_heads", "8"] in rows
    assert ["exact_decode_parameter", "draft_depth", "4"] in rows
    assert [r[3] for r in rows if r[0] == "operation"] == [
        "embedding.lookup.fp4-block32.v1",
        "block.full-attention.output-gated.v1", "ffn.swiglu.dense.fp4-block32.v1",
        "block.full-attention.output-gated.v1", "ffn.swiglu.dense.fp4-block32.v1",
        "head.rmsnorm.token-select.fp4-block32.v1"]


# ---- against the reference's parser -------------------------------------------

PROGRAMS = [("schema1_hybrid_sparse.tsv", 0xa5, 0x9000), ("schema2_vendor_moe.tsv", 0x5a, 0x4100),
            ("schema3_callable_program.tsv", 0x93, 0x9300)]


def mutations(text, rng, count):
    """Single-edit corruptions of a program: lines dropped, repeated, moved,
    fields dropped, added, emptied, renamed or replaced by awkward numbers."""
    awkward = [b"", b"-", b"0", b"1", b"2", b"3", b"7", b"-1", b"+1", b"1 ", b" 1", b"01",
               b"4294967295", b"4294967296", b"18446744073709551615", b"18446744073709551616",
               b"1e3", b"0x10", b"decoder", b"other", b"a\rb"]
    lines = text.split(b"\n")[:-1]
    for _ in range(count):
        edited = list(lines)
        kind = rng.integers(0, 8)
        index = int(rng.integers(0, len(edited)))
        if kind == 0:
            del edited[index]
        elif kind == 1:
            edited.insert(int(rng.integers(0, len(edited) + 1)), edited[index])
        elif kind == 2:
            line = edited.pop(index)
            edited.insert(int(rng.integers(0, len(edited) + 1)), line)
        else:
            fields = edited[index].split(b"\t")
            field = int(rng.integers(0, len(fields)))
            if kind == 3:
                fields[field] = awkward[int(rng.integers(0, len(awkward)))]
            elif kind == 4:
                del fields[field]
            elif kind == 5:
                fields.insert(field, awkward[int(rng.integers(0, len(awkward)))])
            elif kind == 6:
                other = edited[int(rng.integers(0, len(edited)))].split(b"\t")
                fields[field] = other[int(rng.integers(0, len(other)))]
            else:
                fields[field] = fields[field] + b"x"
            edited[index] = b"\t".join(fields)
        ending = b"\r\n" if rng.integers(0, 8) == 0 else b"\n"
        yield ending.join(edited) + ending


@needs_reference
def test_sha256_equals_the_reference():
    rng = np.random.default_rng(2)
    for size in (0, 1, 55, 56, 63, 64, 65, 119, 120, 4096, 100001):
        data = rng.integers(0, 256, size, dtype=np.uint8).tobytes()
        assert al.Product.sha256(data) == al.Reference.sha256(data)


@needs_reference
@pytest.mark.parametrize("name,first,base", PROGRAMS)
def test_fixtures_parse_like_the_reference(name, first, base):
    text = golden(name)
    assert al.Product.parse(text, digest(first), base) == al.Reference.parse(
        text, digest(first), base)
    # namespace offsets that overflow the base are rejected alike
    top = 2 ** 64 - 1
    assert al.Product.parse(text, digest(first), top) == al.Reference.parse(
        text, digest(first), top)


@needs_reference
def test_generated_program_parses_like_the_reference():
    for mtp in (True, False):
        text = tiny_program(mtp)
        mine = al.Product.parse(text, digest(9), 0x1234)
        assert mine[0] == 0 and mine == al.Reference.parse(text, digest(9), 0x1234)


@needs_reference
def test_corrupted_programs_are_judged_like_the_reference():
    rng = np.random.default_rng(11)
    sources = [(golden(name), first, base) for name, first, base in PROGRAMS]
    sources.append((tiny_program(), 9, 0x1234))
    accepted = rejected = 0
    messages = set()
    for text, first, base in sources:
        for mutated in mutations(text, rng, 900):
            mine = al.Product.parse(mutated, digest(first), base)
            theirs = al.Reference.parse(mutated, digest(first), base)
            assert mine == theirs, mutated.decode(errors="replace")
            if mine[0] == 0:
                accepted += 1
            else:
                rejected += 1
                messages.add(mine[1].split(" line ")[0])
    # the corpus reaches the parser's and the validator's rejections, and edits
    # that leave a valid program
    assert accepted > 100 and rejected > 1500
    assert len(messages) >= 12, sorted(messages)


@needs_reference
def test_load_is_judged_like_the_reference(tmp_path):
    text = golden("schema3_callable_program.tsv")
    path = tmp_path / "runtime-model.tsv"
    path.write_bytes(text)
    sha = hashlib.sha256(text).digest()
    for size, checksum in ((len(text), sha), (len(text), bytes(32)), (len(text) - 1, sha), (0, sha)):
        assert al.Product.load(path, size, checksum, digest(0x93), 0x9300) == al.Reference.load(
            path, size, checksum, digest(0x93), 0x9300)
