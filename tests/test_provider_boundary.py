"""The provider boundary on the host (no GPU): capability negotiation and
program compilation against the reference's own registry, and the provider's
sources compiled against the reference's own headers.

Pinned by: the facts the reference's binding test asserts for its fixture
program (runtime/tests/cache_state_test.cpp:574-707: a metadata-only provider
wins the metadata binding, executable binding takes the two callable ones, four
SSA values, one input, one output, an exact-decode program), the selection
rules of runtime/src/execution_provider.cpp:38-131, and - report for report -
the reference's registry and compile_model_program built from their sources
(oracle/_ref) over the golden programs, a generated dense program and provider
sets that exercise priority, name ties, ABI ranges, missing kernels and
rejected registrations.
"""
import os
import subprocess

import pytest

import artifact_lib as al
import qllm_provider as qp
from test_model_descriptor import digest, golden, tiny_program

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REFERENCE_TREE = "/root/reference"
needs_reference = pytest.mark.skipif(al.reference() is None,
                                     reason="oracle/_ref/libqllm_ref_artifact.so is not built")

FIXTURE_PROVIDERS = "\n".join([
    "provider\tmetadata-only-high-priority\t100\t0",
    "capability\tfixture.embed.v7\t7\t7",
    "capability\tfixture.transform.v11\t11\t11",
    "capability\tfixture.head.v3\t3\t3",
    "capability\tfixture.exact-decode.v1\t1\t1",
    "provider\tcallable-edges\t20\t1",
    "capability\tfixture.embed.v7\t7\t7",
    "capability\tfixture.head.v3\t3\t3",
    "capability\tfixture.exact-decode.v1\t1\t1",
    "provider\tcallable-transform\t10\t1",
    "capability\tfixture.transform.v11\t11\t11",
]) + "\n"


def rows_of(report):
    return [line.split("\t") for line in report.splitlines()]


def dense_providers(**changes):
    """This library's own capability table as a provider description."""
    lines = ["provider\tmi355-dense-fp4\t200\t1"]
    for name in qp.capabilities():
        low, high = (2, 2) if ".exact.v2" in name else (1, 1)
        low, high = changes.get(name, (low, high))
        lines.append(f"capability\t{name}\t{low}\t{high}")
    return "\n".join(lines) + "\n"


def test_fixture_program_binds_as_the_reference_test_expects():
    text = golden("schema3_callable_program.tsv")
    metadata = rows_of(al.Product.bind(text, digest(0x93), 0x9300, FIXTURE_PROVIDERS, False))
    assert ["status", "bind", "0", ""] in metadata
    providers = [r for r in metadata if r[0] == "plan_provider"]
    assert providers == [["plan_provider", "metadata-only-high-priority", "0", "metadata"]]
    executable = rows_of(al.Product.bind(text, digest(0x93), 0x9300, FIXTURE_PROVIDERS, True))
    providers = [r for r in executable if r[0] == "plan_provider"]
    assert [r[1:] for r in providers] == [["callable-edges", "1", "callable"],
                                          ["callable-transform", "2", "callable"]]
    assert len([r for r in executable if r[0] == "value"]) == 4
    assert len([r for r in executable if r[0] == "input"]) == 1
    assert len([r for r in executable if r[0] == "output"]) == 1
    assert [r for r in executable if r[0] == "exact_decode"] == [["exact_decode", "3", "2"]]
    # kernel k: requirement k, the registry index of its provider, the position
    # of the capability inside that provider's table
    kernels = [r[1:] for r in executable if r[0] == "kernel"]
    assert kernels == [["0", "1", "0"], ["1", "2", "0"], ["2", "1", "1"], ["3", "1", "2"]]
    # SSA slots: the program input first, then every operation's output in order
    assert [r[1] for r in executable if r[0] == "value"] == [
        "request.token", "embedded.hidden", "transformed.hidden", "response.token"]
    assert ["operation_input", "1", "hidden", "1"] in executable
    assert ["operation_output", "2", "token", "3"] in executable
    assert ["output", "next_token", "3"] in executable


def test_selection_rules():
    text = golden("schema3_callable_program.tsv")

    def providers_with(*entries):
        lines = []
        for name, priority in entries:
            lines.append(f"provider\t{name}\t{priority}\t1")
            lines += ["capability\tfixture.embed.v7\t7\t7",
                      "capability\tfixture.transform.v11\t11\t11",
                      "capability\tfixture.head.v3\t3\t3",
                      "capability\tfixture.exact-decode.v1\t1\t1"]
        return "\n".join(lines) + "\n"

    def chosen(report):
        return [r[1] for r in rows_of(report) if r[0] == "plan_provider"]

    # higher priority wins; equal priority goes to the smaller name
    assert chosen(al.Product.bind(text, digest(1), 1, providers_with(("b", 5), ("a", 9)), True)) == ["a"]
    assert chosen(al.Product.bind(text, digest(1), 1, providers_with(("b", 5), ("a", 5)), True)) == ["a"]
    assert chosen(al.Product.bind(text, digest(1), 1, providers_with(("a", 5), ("b", 5)), True)) == ["a"]
    # an ABI outside the offered range is no offer
    narrow = providers_with(("a", 5)).replace("fixture.head.v3\t3\t3", "fixture.head.v3\t4\t6")
    report = rows_of(al.Product.bind(text, digest(1), 1, narrow, True))
    assert ["status", "bind", "4",
            "no execution provider implements required kernel: fixture.head.v3"] in report
    # registrations the registry turns down
    twice = providers_with(("a", 5), ("a", 6))
    assert ["add", "a", "4", "execution provider name is duplicated"] in rows_of(
        al.Product.bind(text, digest(1), 1, twice, True))
    empty = "provider\tnothing\t1\t1\n" + providers_with(("a", 5))
    assert ["add", "nothing", "4", "execution provider definition is incomplete"] in rows_of(
        al.Product.bind(text, digest(1), 1, empty, True))
    inverted = providers_with(("a", 5)).replace("fixture.embed.v7\t7\t7", "fixture.embed.v7\t7\t6")
    assert ["add", "a", "4", "execution provider capability is invalid or duplicated"] in rows_of(
        al.Product.bind(text, digest(1), 1, inverted, True))


def test_dense_program_compiles_against_this_providers_table():
    report = rows_of(al.Product.bind(tiny_program(), digest(7), 0x700, dense_providers(), True))
    assert ["status", "bind", "0", ""] in report
    operations = [r for r in report if r[0] == "operation"]
    assert len(operations) == 1 + 2 * 2 + 1            # embedding, 2 x (attention, ffn), head
    # every attention block reads the same positions slot, the program's second input
    positions = [r for r in report if r[0] == "operation_input" and r[2] == "positions"]
    assert len(positions) == 2 and {r[3] for r in positions} == {"0"}
    assert ["input", "positions", "0"] in report and ["input", "token_ids", "1"] in report


@needs_reference
def test_bind_reports_equal_the_references():
    programs = [(golden("schema3_callable_program.tsv"), digest(0x93), 0x9300),
                (golden("schema2_vendor_moe.tsv"), digest(0x5a), 0x4100),
                (golden("schema1_hybrid_sparse.tsv"), digest(0xa5), 0x9000),
                (tiny_program(), digest(7), 0x700),
                (tiny_program(mtp=False), digest(8), 0x800)]
    provider_sets = [FIXTURE_PROVIDERS, dense_providers(),
                     dense_providers(**{"ffn.swiglu.dense.fp4-block32.v1": (2, 3)}),
                     FIXTURE_PROVIDERS.replace("\t20\t1", "\t20\t0"),
                     FIXTURE_PROVIDERS.replace("callable-transform\t10", "callable-edges\t10"),
                     FIXTURE_PROVIDERS.replace("fixture.head.v3\t3\t3", "fixture.head.v3\t0\t3"),
                     "provider\tnothing\t1\t1\n" + FIXTURE_PROVIDERS, ""]
    # providers that serve every kernel of the two older fixtures
    for text, content, base in programs[1:3]:
        code, dump = al.Product.parse(text, content, base)
        assert code == 0
        kernels = [r for r in rows_of(dump) if r[0] == "kernel"]
        lines = ["provider\tgeneric\t7\t1"]
        lines += [f"capability\t{r[1]}\t1\t{max(int(r[2]), 1)}" for r in kernels]
        provider_sets.append("\n".join(dict.fromkeys(lines)) + "\n")
    compared = 0
    for text, content, base in programs:
        for providers in provider_sets:
            for executable in (False, True):
                ours = al.Product.bind(text, content, base, providers, executable)
                theirs = al.Reference.bind(text, content, base, providers, executable)
                assert ours == theirs, (providers, executable)
                compared += 1
    assert compared == len(programs) * len(provider_sets) * 2
    # and some of them do bind
    assert "status\tbind\t0\t" in al.Product.bind(*programs[1], provider_sets[-2], True)
    assert "status\tbind\t0\t" in al.Product.bind(*programs[2], provider_sets[-1], True)


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE_TREE, "runtime", "include")),
                    reason="the reference tree is not present")
@pytest.mark.parametrize("source", ["dense_fp4_provider.cpp", "artifact_provider.cpp",
                                    "execution_provider.cpp", "operation_handles.cpp",
                                    "speculative_sampling.cpp"])
def test_provider_sources_compile_against_the_reference_headers(source):
    """Swapping the include path: the reference's runtime/include in place of
    quantum-llm_amd/provider/include.  The provider object, the module factory
    and the boundary's helper sources must parse and type-check unchanged."""
    provider = os.path.join(ROOT, "quantum-llm_amd", "provider")
    command = ["g++", "-fsyntax-only", "-std=c++20", "-D__HIP_PLATFORM_AMD__",
               "-I" + os.path.join(REFERENCE_TREE, "runtime", "include"),
               "-I" + os.path.join(ROOT, "include"), "-I" + provider,
               "-I/opt/rocm/include", os.path.join(provider, source)]
    done = subprocess.run(command, capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-4000:]
