"""The FP4 GEMM for tall batches (prompt prefill) against the CPU oracle, and
against the small-batch kernel on the same rows."""
import ctypes

import numpy as np
import pytest
import torch

import gpu_util as gu
import oracle_lib as ol
import qllm_hip as qh
import synth

pytestmark = pytest.mark.gpu


def tall(device, codes, scales, scheme, rows, padded, act, out_kind=qh.OUT_F32,
         residual=None):
    batch = act.shape[0]
    d_codes, d_scales = gu.device_tensor(codes, device), gu.device_tensor(scales, device)
    d_act = gu.device_tensor(ol.bf16_bits(act), device)
    matrix, keep = qh.prepack(qh.fp4_matrix(d_codes, d_scales, rows, padded, padded, scheme),
                              device)
    dtype = torch.bfloat16 if out_kind == qh.OUT_BF16 else torch.float32
    out = torch.zeros((batch, rows), dtype=dtype, device=device)
    d_residual = None if residual is None else gu.device_tensor(residual, device)
    qh.call("qllm_fp4_gemm_bf16_tall", matrix, qh.ptr(d_act), d_act.numel() * 2,
            qh.ptr(out), out_kind, qh.ptr(d_residual), batch, None)
    torch.cuda.synchronize()
    return out.float().cpu().numpy()


@pytest.mark.parametrize("rows,padded,batch", [
    (256, 64, 128), (300, 1024, 9), (1024, 5120, 200), (77, 128, 333),
    (2048, 1024, 1024), (512, 8192, 130)])
@pytest.mark.parametrize("scheme", [ol.SCALE_UE8M0_BLOCK32, ol.SCALE_F16_BLOCK16])
def test_tall_gemm_matches_oracle(device, scheme, rows, padded, batch):
    """Ragged shapes: batches that are no multiple of 128, weight rows that are
    no multiple of 256 or 32, a single chunk of K."""
    rng = np.random.default_rng(rows + batch)
    codes, scales = synth.fp4_matrix(rng, rows, padded, scheme)
    act = ol.bf16_round(rng.standard_normal((batch, padded)).astype(np.float32))
    want = ol.fp4_linear_f64(codes, scales, scheme, rows, padded, act)
    got = tall(device, codes, scales, scheme, rows, padded, act)
    gu.assert_close(got, want, what="tall GEMM")
    if scheme == ol.SCALE_UE8M0_BLOCK32:
        # exact bf16 operands: only the F32 summation order separates the two
        error = np.abs(got - want).max() / np.abs(want).max()
        assert error < 2e-6 * np.sqrt(padded)


@pytest.mark.parametrize("scheme", [ol.SCALE_UE8M0_BLOCK32, ol.SCALE_F16_BLOCK16])
def test_tall_gemm_residual_and_bf16_output(device, scheme):
    rng = np.random.default_rng(5)
    rows, padded, batch = 640, 1024, 150
    codes, scales = synth.fp4_matrix(rng, rows, padded, scheme)
    act = ol.bf16_round(rng.standard_normal((batch, padded)).astype(np.float32))
    residual = rng.standard_normal((batch, rows)).astype(np.float32)
    want = ol.fp4_linear_f64(codes, scales, scheme, rows, padded, act)
    got = tall(device, codes, scales, scheme, rows, padded, act, residual=residual)
    gu.assert_close(got, want + residual, what="tall GEMM + residual")
    got = tall(device, codes, scales, scheme, rows, padded, act, out_kind=qh.OUT_BF16)
    gu.assert_close(got, want, rtol=1e-2, atol=1e-3, what="tall GEMM bf16")


@pytest.mark.parametrize("scheme", [ol.SCALE_UE8M0_BLOCK32, ol.SCALE_F16_BLOCK16])
def test_tall_gemm_rows_equal_the_small_batch_kernel(device, scheme):
    """The same five rows through the verify-step kernel and through the tall
    one (as rows 123..127 of a batch of 128)."""
    rng = np.random.default_rng(8)
    rows, padded = 1024, 5120
    codes, scales = synth.fp4_matrix(rng, rows, padded, scheme)
    act = ol.bf16_round(rng.standard_normal((128, padded)).astype(np.float32))
    small = gu.gemm(device, codes, scales, scheme, rows, padded, act[123:128])
    big = tall(device, codes, scales, scheme, rows, padded, act)[123:128]
    gu.assert_close(big, small, rtol=2e-3, atol=2e-4, what="tall vs small-batch rows")


def test_tall_gemm_binary16_scales_at_the_ends_of_their_exact_range(device):
    """Block scales of 2^-13 and of 10912 (6 x 10912 = 65472 is the largest
    product binary16 holds): inside that range weight x scale is carried
    exactly by the two binary16 halves, so the tall kernel agrees with the
    oracle as tightly as for ordinary scales.  Scales below the range (6e-5)
    lose the low half's last bits: within 2^-11 of each product."""
    rng = np.random.default_rng(21)
    rows, padded, batch = 256, 1024, 130
    codes, _ = synth.fp4_matrix(rng, rows, padded, ol.SCALE_F16_BLOCK16)
    act = ol.bf16_round(rng.standard_normal((batch, padded)).astype(np.float32))
    for low, high, tolerance in ((2.0 ** -13, 10912.0, 2e-6), (6e-5, 8192.0, 2.0 ** -11)):
        values = np.where(rng.random((rows, padded // 16)) < 0.5, low, high)
        scales = values.astype(np.float16).view(np.uint16)
        want = ol.fp4_linear_f64(codes, scales, ol.SCALE_F16_BLOCK16, rows, padded, act)
        got = tall(device, codes, scales, ol.SCALE_F16_BLOCK16, rows, padded, act)
        assert np.isfinite(got).all()
        # the error bound is relative to the sum of |products|, not to the result
        magnitude = ol.fp4_linear_f64(codes & 0x77, scales, ol.SCALE_F16_BLOCK16, rows, padded,
                                      np.abs(act))
        assert (np.abs(got - want) <= tolerance * np.sqrt(padded) * magnitude + 1e-30).all()
        small = gu.gemm(device, codes, scales, ol.SCALE_F16_BLOCK16, rows, padded, act[:5])
        assert (np.abs(small - want[:5]) <= 2e-6 * np.sqrt(padded) * magnitude[:5] + 1e-30).all()


def test_tall_split_outputs(device):
    rng = np.random.default_rng(9)
    scheme, padded, batch = ol.SCALE_F16_BLOCK16, 1024, 140
    parts = [512, 64, 64]
    rows = sum(parts)
    codes, scales = synth.fp4_matrix(rng, rows, padded, scheme)
    act = ol.bf16_round(rng.standard_normal((batch, padded)).astype(np.float32))
    whole = tall(device, codes, scales, scheme, rows, padded, act)
    d_codes, d_scales = gu.device_tensor(codes, device), gu.device_tensor(scales, device)
    d_act = gu.device_tensor(ol.bf16_bits(act), device)
    matrix, keep = qh.prepack(qh.fp4_matrix(d_codes, d_scales, rows, padded, padded, scheme),
                              device)
    outs = [torch.zeros((batch, part), device=device) for part in parts]
    segments = (qh.GemmSegment * 3)(*[qh.GemmSegment(qh.ptr(o), part, qh.OUT_F32)
                                      for o, part in zip(outs, parts)])
    qh.call("qllm_fp4_gemm_bf16_tall_split", matrix, qh.ptr(d_act), d_act.numel() * 2,
            segments, 3, batch, None)
    torch.cuda.synchronize()
    first = 0
    for out, part in zip(outs, parts):
        assert np.array_equal(out.cpu().numpy(), whole[:, first:first + part])
        first += part
    bad = (qh.GemmSegment * 2)(qh.GemmSegment(qh.ptr(outs[0]), 520, qh.OUT_F32),
                               qh.GemmSegment(qh.ptr(outs[1]), 120, qh.OUT_F32))
    with pytest.raises(qh.QllmError, match="multiples of 32"):
        qh.call("qllm_fp4_gemm_bf16_tall_split", matrix, qh.ptr(d_act), d_act.numel() * 2,
                bad, 2, batch, None)


@pytest.mark.parametrize("rows,padded,batch", [(1024, 1024, 200), (300, 128, 77), (96, 64, 129)])
@pytest.mark.parametrize("scheme", [ol.SCALE_UE8M0_BLOCK32, ol.SCALE_F16_BLOCK16])
def test_tall_swiglu_equals_two_gemms_and_the_product(device, scheme, rows, padded, batch):
    """One launch over the gate and the up matrix against two tall GEMMs and
    the SiLU-product launch with bf16 rounding points: bit-equal, and against
    the oracle's F64 projections within bf16 rounding."""
    rng = np.random.default_rng(rows + padded + batch)
    act = ol.bf16_round(rng.standard_normal((batch, padded)).astype(np.float32))
    d_act = gu.device_tensor(ol.bf16_bits(act), device)
    matrices, keep, f32, f64 = [], [], [], []
    for _ in range(2):
        codes, scales = synth.fp4_matrix(rng, rows, padded, scheme)
        tensors = gu.device_tensor(codes, device), gu.device_tensor(scales, device)
        matrix, packed = qh.prepack(qh.fp4_matrix(*tensors, rows, padded, padded, scheme), device)
        out = torch.zeros((batch, rows), device=device)
        qh.call("qllm_fp4_gemm_bf16_tall", matrix, qh.ptr(d_act), d_act.numel() * 2,
                qh.ptr(out), qh.OUT_F32, None, batch, None)
        matrices.append(matrix); keep.append((tensors, packed)); f32.append(out)
        f64.append(ol.fp4_linear_f64(codes, scales, scheme, rows, padded, act))
    qh.call("qllm_silu_product", qh.ptr(f32[0]), qh.ptr(f32[1]), qh.ptr(f32[0]),
            batch * rows, 1, None)
    fused = torch.zeros((batch, rows), dtype=torch.bfloat16, device=device)
    qh.call("qllm_fp4_swiglu_bf16_tall", matrices[0], matrices[1], qh.ptr(d_act),
            d_act.numel() * 2, qh.ptr(fused), batch, None)
    torch.cuda.synchronize()
    got = fused.float().cpu().numpy()
    assert np.array_equal(got, f32[0].cpu().numpy())
    want = f64[0] / (1.0 + np.exp(np.minimum(-f64[0], 80.0))) * f64[1]
    gu.assert_close(got, want, rtol=2e-2, atol=2e-2 * np.abs(want).max(), what="tall SwiGLU")
    with pytest.raises(qh.QllmError, match="invalid tall FP4 SwiGLU"):
        qh.call("qllm_fp4_swiglu_bf16_tall", matrices[0], None, qh.ptr(d_act),
                d_act.numel() * 2, qh.ptr(fused), batch, None)


def test_tall_gemm_rejects_row_major(device):
    rng = np.random.default_rng(1)
    codes, scales = synth.fp4_matrix(rng, 64, 64, 0)
    d = [gu.device_tensor(x, device) for x in (codes, scales)]
    act = torch.zeros((16, 64), dtype=torch.bfloat16, device=device)
    out = torch.zeros((16, 64), device=device)
    matrix = qh.fp4_matrix(d[0], d[1], 64, 64, 64, 0)
    with pytest.raises(qh.QllmError, match="invalid tall"):
        qh.call("qllm_fp4_gemm_bf16_tall", matrix, qh.ptr(act), act.numel() * 2,
                qh.ptr(out), qh.OUT_F32, None, 16, None)
