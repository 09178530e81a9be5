"""The argmax entry point that allocates nothing (its stage-1 partials live in
a fixed device array inside the library) against qllm_argmax_batch with a
caller's workspace: same tokens on two calls in a row, the second smaller."""
import ctypes

import numpy as np
import pytest
import torch

import gpu_util as gu
import oracle_lib as ol
import qllm_hip as qh

pytestmark = pytest.mark.gpu


def with_workspace(d_logits, count, batch, device):
    out = torch.full((batch,), -1, dtype=torch.int32, device=device)
    size = qh.call("qllm_argmax_workspace_bytes", count, batch)
    workspace = torch.zeros(size, dtype=torch.uint8, device=device)
    qh.call("qllm_argmax_batch", qh.ptr(d_logits), count, batch, qh.ptr(out),
            qh.ptr(workspace), size, None)
    torch.cuda.synchronize()
    return out.cpu().numpy().astype(np.uint32)


def without_allocation(d_logits, count, batch, device, out):
    qh.call("qllm_argmax_batch_static", qh.ptr(d_logits), count, batch,
            qh.ptr(out), None)
    torch.cuda.synchronize()
    return out.cpu().numpy().astype(np.uint32)[:batch]


def test_static_argmax_equals_the_workspace_form_on_two_calls(device):
    rng = np.random.default_rng(11)
    nan = float("nan")
    large = rng.standard_normal((5, 151936)).astype(np.float32)
    large[0, 400] = large[0, 150000] = 8.0           # tie -> lower index
    large[1, :] = nan
    large[1, 90001] = -2.0                           # NaN never wins
    large[4, 151935] = 11.0
    small = rng.standard_normal((3, 3001)).astype(np.float32)
    small[2, 3000] = 7.5
    d_large, d_small = gu.device_tensor(large, device), gu.device_tensor(small, device)
    out = torch.full((8,), -1, dtype=torch.int32, device=device)   # allocated before the calls
    torch.cuda.synchronize()
    first = without_allocation(d_large, 151936, 5, device, out)
    second = without_allocation(d_small, 3001, 3, device, out)      # leftovers of the first call stay behind
    assert first.tolist() == with_workspace(d_large, 151936, 5, device).tolist()
    assert second.tolist() == with_workspace(d_small, 3001, 3, device).tolist()
    assert first.tolist() == [ol.argmax(large[r]) for r in range(5)]
    assert second.tolist() == [ol.argmax(small[r]) for r in range(3)]
    assert first[0] == 400 and first[1] == 90001 and second[2] == 3000


def test_static_argmax_rejects_what_does_not_fit(device):
    capacity = qh.call("qllm_argmax_static_capacity_bytes")
    assert capacity == 64 * 1024
    count = 2048 * 8192                       # 8192 partial blocks for one row: fits exactly
    assert qh.call("qllm_argmax_workspace_bytes", count, 1) == capacity
    values = torch.zeros(16, device=device)
    out = torch.zeros(8, dtype=torch.int32, device=device)
    with pytest.raises(qh.QllmError) as error:
        qh.call("qllm_argmax_batch_static", qh.ptr(values), count, 2, qh.ptr(out), None)
    assert error.value.code == 4 and "exceeds" in str(error.value)
    with pytest.raises(qh.QllmError):
        qh.call("qllm_argmax_batch_static", qh.ptr(values), count + 1, 1, qh.ptr(out), None)
