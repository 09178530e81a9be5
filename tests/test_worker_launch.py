"""Launch contract of the worker process (runtime/src/worker_contract.cpp:67-180,
runtime/tools/moe_vm_runner.cpp:1472-1538): what it refuses before it touches
an artifact or the GPU.  Runs without a GPU."""
import os

import pytest

import worker_client as wc

pytestmark = pytest.mark.skipif(not os.path.exists(wc.BINARY), reason="worker not built")


def launch(*arguments):
    code, out, err = wc.run_to_exit(list(arguments))
    assert out == ""
    return code, err.strip()


def test_usage():
    assert launch()[0] == 64
    assert launch("/nowhere")[0] == 64
    code, err = launch("/nowhere", "--serve")
    assert code == 64 and err.startswith("usage: qllm-worker")


@pytest.mark.parametrize("change,message", [
    (dict(max_context=None), "missing worker option --max-context"),
    (dict(placement_profile=None), "missing worker option --placement-profile"),
    (dict(kv_page_tokens=0), "worker option is out of range"),
    (dict(max_context="12x"), "worker option is not an unsigned integer"),
    (dict(kv_cache_mib=0), "worker resource contract is invalid"),
    (dict(placement_profile="fast"), "worker resource contract is invalid"),
    (dict(routed_vram_policy="greedy"), "worker resource contract is invalid"),
    (dict(profile_gpu_phases=1), "boolean worker option profile-gpu-phases has a value"),
    (dict(ram_cache_gib=1 << 40), "worker resource byte count overflows"),
])
def test_launch_contract(change, message):
    code, err = launch("/nowhere", "--worker", *wc.launch_arguments(**change))
    assert code == 1 and err in ("qllm worker: invalid worker launch contract: " + message,
                                 "qllm worker: " + message)


def test_option_syntax():
    base = wc.launch_arguments()
    failures = {
        "positional": "worker launch contains a positional option",
        "--Max=1": "worker option name is not canonical",
        "---x=1": "worker option name is not canonical",
        "--capacity=": "worker option value is empty",
        "--capacity=1": "worker option is duplicated",
    }
    for argument, message in failures.items():
        code, err = launch("/nowhere", "--worker", *base, argument)
        assert code == 1 and err == "qllm worker: invalid worker launch contract: " + message
    code, err = launch("/nowhere", "--worker", *base, "--sm86-streams=2")
    assert code == 1
    assert err == "qllm worker: callable VM service does not accept provider-specific launch flags"


def test_missing_artifact_is_reported(tmp_path):
    code, err = launch(str(tmp_path / "absent"), "--worker", *wc.launch_arguments())
    assert code == 1 and err.startswith("qllm worker: ")
