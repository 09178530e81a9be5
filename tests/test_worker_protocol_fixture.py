"""The worker protocol as the reference's own service tests state it
(tests/golden/worker_protocol.json, written from the literals of
tests/server/test_expert_server.py by tests/golden/make_worker_protocol_fixture.py):
the restatement of the service's reading of a ready line (worker_client.ServiceView)
must accept, reject and read those scripted workers exactly as the reference's
client does - that pins the rule the real worker's ready line is then held to
on the GPU (test_gpu_worker_slots.py)."""
import json
import os

import pytest

import worker_client as wc

FIXTURE = os.path.join(os.path.dirname(__file__), "golden", "worker_protocol.json")
with open(FIXTURE, encoding="utf-8") as source:
    PROTOCOL = json.load(source)


@pytest.mark.parametrize("case", PROTOCOL["ready_lines"],
                         ids=lambda case: f"{case['test']}-{case['ready']['kv_dtype']}")
def test_scripted_ready_lines_are_read_as_the_service_reads_them(case):
    if not case["accepted"]:
        with pytest.raises(wc.ContractError, match="runtime contract"):
            wc.ServiceView(case["ready"], case["launch"])
        return
    view = wc.ServiceView(case["ready"], case["launch"])
    for name, expected in case["attributes"].items():
        assert getattr(view, name) == expected, name


def test_the_fixture_covers_both_verdicts_and_every_generation():
    cases = PROTOCOL["ready_lines"]
    assert len(cases) >= 14 and any(not case["accepted"] for case in cases)
    assert {case["ready"]["protocol"] for case in cases} >= {4, 5, 6, 7, 9, 10, 11}


def test_sampling_group_is_serialised_as_the_service_serialises_it():
    """test_protocol8_serializes_request_sampling: temperature 1.0, top-p 0.95,
    top-k 20, min-p 0, no penalty, seed 1234."""
    line = next(item["line"] for item in PROTOCOL["command_lines"]
                if item["line"].startswith("\tSAMPLING"))
    view = wc.ServiceView.__new__(wc.ServiceView)
    view.sampling_supported = view.sampling_presence_penalty_supported = True
    fields = view.sampling_fields(1.0, 0.95, 20, 0.0, 0.0, 1234)
    assert "\t" + "\t".join(str(field) for field in fields) == line


@pytest.mark.parametrize("mutation, message", [
    (dict(capacity=2), "runtime contract"),
    (dict(kv_page_tokens=64), "runtime contract"),
    (dict(kv_dtype="int3"), "runtime contract"),
    (dict(placement_profile="latency"), "runtime contract"),
    (dict(sampling_supported=True, sampling_presence_penalty_supported=False),
     "runtime contract"),
    (dict(mtp_runtime_ready=True, mtp_resource_available=False), "without resources"),
])
def test_a_broken_field_is_turned_down(mutation, message):
    case = next(case for case in PROTOCOL["ready_lines"]
                if case["test"] == "test_protocol10_accepts_artifact_declared_bf16_latent_kv")
    with pytest.raises(wc.ContractError, match=message):
        wc.ServiceView({**case["ready"], **mutation}, case["launch"])
