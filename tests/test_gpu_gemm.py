"""FP4 GEMM parity on the GPU, through the C ABI, against the CPU oracle."""
import numpy as np
import pytest
import torch

import gpu_util as gu
import oracle_lib as ol
import qllm_hip as qh
import synth

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("scheme", [ol.SCALE_F16_BLOCK16, ol.SCALE_UE8M0_BLOCK32])
@pytest.mark.parametrize("rows,padded,batch", [
    (64, 256, 5), (100, 320, 5), (67, 96, 3), (33, 64, 1), (1024, 5120, 5),
    (512, 8192, 5), (256, 17408, 5), (333, 5120, 8), (4096, 1024, 2)])
def test_gemm_matches_oracle(device, scheme, rows, padded, batch):
    rng = np.random.default_rng(rows * 31 + padded + batch + scheme)
    codes, scales = synth.fp4_matrix(rng, rows, padded, scheme)
    act = ol.bf16_round(rng.standard_normal((batch, padded)).astype(np.float32))
    want = ol.fp4_linear_f64(codes, scales, scheme, rows, padded, act)
    row_major = gu.gemm(device, codes, scales, scheme, rows, padded, act, tiled=False)
    gu.assert_close(row_major, want, what="row-major")
    if padded % 64 == 0:
        tiled = gu.gemm(device, codes, scales, scheme, rows, padded, act, tiled=True)
        # the tiled copy moves bytes only: same arithmetic, same bits
        assert np.array_equal(tiled, row_major)


@pytest.mark.parametrize("tile_rows", [8, 20, 24, 32])
@pytest.mark.parametrize("rows,padded,batch", [(333, 5120, 5), (2000, 1024, 6),
                                               (40, 128, 7), (17, 64, 8)])
@pytest.mark.parametrize("scheme", [ol.SCALE_UE8M0_BLOCK32, ol.SCALE_F16_BLOCK16])
def test_gemm_tile_heights(device, scheme, tile_rows, rows, padded, batch):
    """Every tile height of the streaming layout (partial last tile included)
    computes the same rows; only the summation order over K may differ."""
    rng = np.random.default_rng(rows + tile_rows)
    codes, scales = synth.fp4_matrix(rng, rows, padded, scheme)
    act = ol.bf16_round(rng.standard_normal((batch, padded)).astype(np.float32))
    want = ol.fp4_linear_f64(codes, scales, scheme, rows, padded, act)
    got = gu.gemm(device, codes, scales, scheme, rows, padded, act,
                  tile_rows=tile_rows)
    gu.assert_close(got, want, what=f"tile height {tile_rows}")


@pytest.mark.parametrize("tile_rows", [8, 20, 32])
@pytest.mark.parametrize("scheme", [ol.SCALE_UE8M0_BLOCK32, ol.SCALE_F16_BLOCK16])
def test_rows_read_back_from_the_tiled_layout(device, scheme, tile_rows):
    """qllm_fp4_unpack_rows undoes qllm_fp4_prepack for any row range (and is a
    plain copy for a row-major matrix)."""
    rng = np.random.default_rng(tile_rows + scheme)
    rows, padded = 333, 1024
    codes, scales = synth.fp4_matrix(rng, rows, padded, scheme)
    d_codes, d_scales = gu.device_tensor(codes, device), gu.device_tensor(scales, device)
    plain = qh.fp4_matrix(d_codes, d_scales, rows, padded, padded, scheme)
    tiled, keep = qh.prepack(plain, device, tile_rows)
    for matrix in (tiled, plain):
        for first, count in ((0, rows), (0, 1), (rows - 1, 1), (17, 40), (31, 2), (300, 33)):
            out_codes = torch.full((count, padded // 2), 0xee, dtype=torch.uint8, device=device)
            out_scales = torch.full((count, scales.shape[1] * scales.itemsize), 0xee,
                                    dtype=torch.uint8, device=device)
            qh.call("qllm_fp4_unpack_rows", matrix, first, count, qh.ptr(out_codes),
                    qh.ptr(out_scales), None)
            torch.cuda.synchronize()
            assert np.array_equal(out_codes.cpu().numpy(), codes[first:first + count])
            assert np.array_equal(out_scales.cpu().numpy().view(scales.dtype),
                                  scales[first:first + count])
    with pytest.raises(qh.QllmError):
        qh.call("qllm_fp4_unpack_rows", tiled, rows, 1, qh.ptr(d_codes), qh.ptr(d_scales), None)
    del keep


@pytest.mark.parametrize("padded,tiled", [(5120, True), (5120, False), (96, False)])
def test_split_gemm_equals_separate_calls(device, padded, tiled):
    """q, k and v stored as one matrix: each output segment carries exactly the
    bits of a separate call on that projection."""
    import ctypes
    rng = np.random.default_rng(padded + tiled)
    scheme, batch, parts = ol.SCALE_F16_BLOCK16, 5, (256, 64, 72)
    rows = sum(parts)
    codes, scales = synth.fp4_matrix(rng, rows, padded, scheme)
    act = ol.bf16_round(rng.standard_normal((batch, padded)).astype(np.float32))
    d_codes, d_scales = gu.device_tensor(codes, device), gu.device_tensor(scales, device)
    d_act = gu.device_tensor(ol.bf16_bits(act), device)
    matrix = qh.fp4_matrix(d_codes, d_scales, rows, padded, padded, scheme)
    if tiled:
        matrix, keep = qh.prepack(matrix, device)
    outputs = [torch.zeros((batch, part), device=device) for part in parts]
    segments = (qh.GemmSegment * 3)(*[
        qh.GemmSegment(qh.ptr(out), part, qh.OUT_F32)
        for out, part in zip(outputs, parts)])
    qh.call("qllm_fp4_gemm_bf16_split", matrix, qh.ptr(d_act), d_act.numel() * 2,
            ctypes.cast(segments, ctypes.c_void_p), 3, batch, None)
    torch.cuda.synchronize()
    first = 0
    for out, part in zip(outputs, parts):
        separate = gu.gemm(device, codes[first:first + part], scales[first:first + part],
                           scheme, part, padded, act, tiled=tiled and padded % 64 == 0)
        got = out.cpu().numpy()
        want = ol.fp4_linear_f64(codes[first:first + part], scales[first:first + part],
                                 scheme, part, padded, act)
        gu.assert_close(got, want, what="split segment")
        if padded % 64:
            assert np.array_equal(got, separate)
        else:   # K is split over four or eight waves depending on the tile count
            assert np.abs(got - separate).max() <= 2e-5 * np.abs(want).max()
        first += part
    with pytest.raises(qh.QllmError):
        segments[2].rows += 1
        qh.call("qllm_fp4_gemm_bf16_split", matrix, qh.ptr(d_act), d_act.numel() * 2,
                ctypes.cast(segments, ctypes.c_void_p), 3, batch, None)


def test_gemm_config1_shape_and_output_kinds(device):
    """Benchmark shape of one linear: [17408, 5120], M=5, binary16 scale per 16, bf16 out."""
    rng = np.random.default_rng(1)
    rows, padded, batch, scheme = 17408, 5120, 5, ol.SCALE_F16_BLOCK16
    codes, scales = synth.fp4_matrix(rng, rows, padded, scheme)
    act = ol.bf16_round(rng.standard_normal((batch, padded)).astype(np.float32))
    want = ol.fp4_linear_f64(codes, scales, scheme, rows, padded, act)
    got = gu.gemm(device, codes, scales, scheme, rows, padded, act)
    gu.assert_close(got, want, what="f32 out")
    got_bf16 = gu.gemm(device, codes, scales, scheme, rows, padded, act,
                       out_kind=qh.OUT_BF16)
    assert np.array_equal(got_bf16, ol.bf16_round(got))
    rounded = gu.gemm(device, codes, scales, scheme, rows, padded, act,
                      out_kind=qh.OUT_F32_BF16_ROUNDED)
    assert np.array_equal(rounded, got_bf16)
    residual = rng.standard_normal((batch, rows)).astype(np.float32)
    with_residual = gu.gemm(device, codes, scales, scheme, rows, padded, act,
                            residual=residual)
    gu.assert_close(with_residual, want + residual, what="residual")


def test_gemm_is_linear_in_the_activations(device):
    """Size-independent property at the lm_head shape: W(a+b) = Wa + Wb when the
    sum is exactly representable (powers of two)."""
    rng = np.random.default_rng(2)
    rows, padded, scheme = 151936, 5120, ol.SCALE_F16_BLOCK16
    codes = torch.empty((rows, padded // 2), dtype=torch.uint8, device=device)
    scales = torch.empty((rows, padded // 16), dtype=torch.float16, device=device)
    qh.call("qllm_fill_random", qh.ptr(codes), codes.numel(), 0, 11, None)
    qh.call("qllm_fill_random", qh.ptr(scales), scales.numel(), 3, 12, None)
    matrix, keep = qh.prepack(qh.fp4_matrix(codes, scales, rows, padded, padded, scheme),
                              device)
    a = (2.0 ** rng.integers(-2, 3, (2, padded))).astype(np.float32)
    a[1] *= rng.choice([-1.0, 1.0], padded).astype(np.float32)
    stacked = np.stack([a[0], a[1], np.zeros(padded, np.float32)])
    d_act = gu.device_tensor(ol.bf16_bits(stacked), device)
    out = torch.zeros((3, rows), device=device)
    qh.call("qllm_fp4_gemm_bf16", matrix, qh.ptr(d_act), d_act.numel() * 2,
            qh.ptr(out), qh.OUT_F32, None, 3, None)
    torch.cuda.synchronize()
    host = out.cpu().numpy()
    assert not host[2].any()                      # zero activations -> zero
    # spot-check 64 rows against the oracle (rows fetched back from the device)
    pick = rng.choice(rows, 64, replace=False)
    sub_codes = codes.cpu().numpy()[pick]
    sub_scales = scales.view(torch.uint16).cpu().numpy()[pick]
    want = ol.fp4_linear_f64(sub_codes, sub_scales, scheme, 64, padded, stacked)
    gu.assert_close(host[:, pick], want, what="lm_head rows")


@pytest.mark.parametrize("scheme", [ol.SCALE_F16_BLOCK16, ol.SCALE_UE8M0_BLOCK32])
def test_fused_swiglu_matches_oracle(device, scheme):
    rng = np.random.default_rng(3 + scheme)
    rows, padded, batch = 1024, 5120, 5
    gate = synth.fp4_matrix(rng, rows, padded, scheme)
    up = synth.fp4_matrix(rng, rows, padded, scheme)
    act = ol.bf16_round(0.02 * rng.standard_normal((batch, padded)).astype(np.float32))
    g = ol.fp4_linear_f64(*gate, scheme, rows, padded, act)
    u = ol.fp4_linear_f64(*up, scheme, rows, padded, act)
    want = ol.silu_product(g, u, True)
    tensors = [gu.device_tensor(x, device) for x in (*gate, *up)]
    gate_m, keep_g = qh.prepack(qh.fp4_matrix(tensors[0], tensors[1], rows, padded,
                                              padded, scheme), device)
    up_m, keep_u = qh.prepack(qh.fp4_matrix(tensors[2], tensors[3], rows, padded,
                                            padded, scheme), device)
    d_act = gu.device_tensor(ol.bf16_bits(act), device)
    out = torch.zeros((batch, rows), dtype=torch.bfloat16, device=device)
    qh.call("qllm_fp4_swiglu_bf16", gate_m, up_m, qh.ptr(d_act), d_act.numel() * 2,
            qh.ptr(out), batch, None)
    torch.cuda.synchronize()
    # one bf16 step of slack on top of the F32 tolerance
    gu.assert_close(out.float().cpu().numpy(), want, rtol=1e-2, atol=1e-3,
                    what="swiglu")


def test_q8_gemv_matches_reference_integer_statement(device):
    """Reference arithmetic (ABI 3 weights x Q8 activations), fixture of
    runtime/tools/dense_fp4_cuda_smoke.cpp:139-216, threshold 2e-4 (:4911)."""
    rows, columns, padded, batch = 67, 100, 128, 5
    r = np.arange(rows)[:, None]
    scales = (124 + (r + np.arange(padded // 32)[None, :]) % 7).astype(np.uint8)
    pair = np.arange(padded // 2)[None, :]
    codes = (((r + 3 * pair) % 16) | (((5 * r + pair + 1) % 16) << 4)).astype(np.uint8)
    x = (np.sin(np.arange(batch * columns, dtype=np.float32) * np.float32(0.071)) *
         np.float32(0.7)).astype(np.float32).reshape(batch, columns)
    want_q8, want_scales = ol.quantize_q8_rows(x, padded)
    d_x = gu.device_tensor(x, device)
    d_q8 = torch.zeros((batch, padded), dtype=torch.int8, device=device)
    d_s = torch.zeros(batch, device=device)
    qh.call("qllm_quantize_q8_batch", qh.ptr(d_x), qh.ptr(d_q8), qh.ptr(d_s), batch,
            columns, padded, 0, None)
    torch.cuda.synchronize()
    assert np.array_equal(d_q8.cpu().numpy(), want_q8)          # byte-exact
    assert np.array_equal(d_s.cpu().numpy(), want_scales)
    want = ol.fp4_linear_block32_q8(codes, scales, rows, padded, want_q8, want_scales)
    d_codes, d_scales = gu.device_tensor(codes, device), gu.device_tensor(scales, device)
    out = torch.zeros((batch, rows), device=device)
    qh.call("qllm_fp4_gemv_q8_batch",
            qh.fp4_matrix(d_codes, d_scales, rows, columns, padded, 0), qh.ptr(d_q8),
            qh.ptr(d_s), qh.ptr(out), batch, 0, None)
    torch.cuda.synchronize()
    assert np.abs(out.cpu().numpy() - want).max() < 2e-4


@pytest.mark.parametrize("rows,columns,batch", [(17408, 5120, 5), (1000, 5100, 8),
                                                (64, 33, 1)])
def test_q8_gemv_at_model_shapes_and_ragged_k(device, rows, columns, batch):
    """The Q8-activation form (the reference's default arithmetic: integer
    block sums, one F32 scale FMA per 32-block) at the SwiGLU projection's
    shape and with a K that is not a multiple of the block: against the integer
    statement of the oracle, 2e-4 as the reference's own gate."""
    rng = np.random.default_rng(rows + columns)
    padded = (columns + 31) // 32 * 32
    codes, scales = synth.fp4_matrix(rng, rows, padded, ol.SCALE_UE8M0_BLOCK32)
    x = rng.standard_normal((batch, columns)).astype(np.float32)
    want_q8, want_scales = ol.quantize_q8_rows(x, padded)
    d_x = gu.device_tensor(x, device)
    d_q8 = torch.zeros((batch, padded), dtype=torch.int8, device=device)
    d_s = torch.zeros(batch, device=device)
    qh.call("qllm_quantize_q8_batch", qh.ptr(d_x), qh.ptr(d_q8), qh.ptr(d_s), batch,
            columns, padded, 0, None)
    torch.cuda.synchronize()
    assert np.array_equal(d_q8.cpu().numpy(), want_q8)
    assert not want_q8[:, columns:].any()                       # padding quantises to 0
    want = ol.fp4_linear_block32_q8(codes, scales, rows, padded, want_q8, want_scales)
    d_codes, d_scales = gu.device_tensor(codes, device), gu.device_tensor(scales, device)
    out = torch.zeros((batch, rows), device=device)
    qh.call("qllm_fp4_gemv_q8_batch",
            qh.fp4_matrix(d_codes, d_scales, rows, columns, padded, 0), qh.ptr(d_q8),
            qh.ptr(d_s), qh.ptr(out), batch, 0, None)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.abs(got - want).max() <= 2e-4 * max(1.0, np.abs(want).max())


def test_invalid_arguments_are_rejected(device):
    with pytest.raises(qh.QllmError) as error:
        qh.call("qllm_fp4_gemm_bf16", qh.fp4_matrix(None, None, 4, 4, 32, 0), None, 0,
                None, 0, None, 5, None)
    assert error.value.code == 4
    codes = torch.zeros(64 * 32, dtype=torch.uint8, device=device)
    scales = torch.zeros(64 * 4, dtype=torch.uint8, device=device)
    act = torch.zeros((9, 64), dtype=torch.bfloat16, device=device)
    out = torch.zeros((9, 64), device=device)
    with pytest.raises(qh.QllmError):   # batch > 8
        qh.call("qllm_fp4_gemm_bf16", qh.fp4_matrix(codes, scales, 64, 64, 64, 0),
                qh.ptr(act), act.numel() * 2, qh.ptr(out), 0, None, 9, None)


@pytest.mark.parametrize("scheme", [ol.SCALE_F16_BLOCK16, ol.SCALE_UE8M0_BLOCK32])
@pytest.mark.parametrize("rows,padded,batch,splits", [
    (5120, 17408, 5, 3), (5120, 8192, 5, 3), (333, 5120, 8, 2), (64, 128, 1, 2),
    (100, 320, 3, 5), (512, 1024, 5, 16), (40, 64, 2, 1)])
def test_k_split_partials_add_up_to_the_product(device, scheme, rows, padded, batch, splits):
    """K cut over several workgroups per tile: partial s is the product over
    the split's own chunks of 64 columns (checked against the oracle on that
    column range), so the partials add up to the whole product."""
    rng = np.random.default_rng(rows + padded + splits + scheme)
    codes, scales = synth.fp4_matrix(rng, rows, padded, scheme)
    act = ol.bf16_round(rng.standard_normal((batch, padded)).astype(np.float32))
    tensors = (gu.device_tensor(codes, device), gu.device_tensor(scales, device))
    matrix, keep = qh.prepack(qh.fp4_matrix(tensors[0], tensors[1], rows, padded, padded,
                                            scheme), device)
    d_act = gu.device_tensor(ol.bf16_bits(act), device)
    partials = torch.full((splits, batch, rows), np.nan, device=device)
    qh.call("qllm_fp4_gemm_bf16_partial", matrix, qh.ptr(d_act), d_act.numel() * 2,
            qh.ptr(partials), splits, batch, None)
    torch.cuda.synchronize()
    got = partials.cpu().numpy()
    chunks = padded // 64
    pick = rng.choice(rows, min(rows, 48), replace=False)
    for split in range(splits):
        first, last = split * chunks // splits * 64, (split + 1) * chunks // splits * 64
        masked = np.zeros_like(act)
        masked[:, first:last] = act[:, first:last]
        want = ol.fp4_linear_f64(codes[pick], scales[pick], scheme, len(pick), padded, masked)
        gu.assert_close(got[split][:, pick], want, what=f"partial {split}")
    whole = gu.gemm(device, codes, scales, scheme, rows, padded, act, tiled=True)
    # F32 sums of up to 17408 terms of magnitude ~10 in two different orders
    gu.assert_close(got.astype(np.float64).sum(axis=0), whole, rtol=1e-5, atol=2e-3,
                    what="sum of the partials")


def test_k_split_rejects_what_it_does_not_take(device):
    rng = np.random.default_rng(9)
    rows, padded, batch = 64, 128, 5
    codes, scales = synth.fp4_matrix(rng, rows, padded, ol.SCALE_F16_BLOCK16)
    tensors = (gu.device_tensor(codes, device), gu.device_tensor(scales, device))
    row_major = qh.fp4_matrix(tensors[0], tensors[1], rows, padded, padded,
                              ol.SCALE_F16_BLOCK16)
    tiled, keep = qh.prepack(row_major, device)
    d_act = torch.zeros((batch, padded), dtype=torch.bfloat16, device=device)
    partials = torch.zeros((16, batch, rows), device=device)
    for matrix, splits, rows_in_batch in ((row_major, 2, batch), (tiled, 0, batch),
                                          (tiled, 3, batch), (tiled, 17, batch),
                                          (tiled, 2, 9)):
        with pytest.raises(qh.QllmError):
            qh.call("qllm_fp4_gemm_bf16_partial", matrix, qh.ptr(d_act), d_act.numel() * 2,
                    qh.ptr(partials), splits, rows_in_batch, None)


# ---- balanced tail: the tiles past the last full round over the CUs cut along K ----

def _balance_workspace(device):
    size = qh.call("qllm_fp4_gemm_balance_workspace_bytes")
    return torch.zeros(size, dtype=torch.uint8, device=device), size


@pytest.mark.parametrize("scheme", [ol.SCALE_F16_BLOCK16, ol.SCALE_UE8M0_BLOCK32])
@pytest.mark.parametrize("rows,padded,batch", [(17408, 5120, 5), (10240, 1024, 5),
                                               (8224, 512, 8), (9000, 128, 1)])
def test_balanced_swiglu_matches_oracle_and_the_plain_launch(device, scheme, rows, padded,
                                                             batch):
    """Gate/up with a ragged last round: cut tiles against the oracle, uncut
    tiles bit-equal to the plain launch, the same bits on every run and the
    workspace's counters back at zero."""
    rng = np.random.default_rng(rows + padded + scheme)
    gate = synth.fp4_matrix(rng, rows, padded, scheme)
    up = synth.fp4_matrix(rng, rows, padded, scheme)
    act = ol.bf16_round(0.02 * rng.standard_normal((batch, padded)).astype(np.float32))
    tensors = [gu.device_tensor(x, device) for x in (*gate, *up)]
    gate_m, keep_g = qh.prepack(qh.fp4_matrix(tensors[0], tensors[1], rows, padded,
                                              padded, scheme), device)
    up_m, keep_u = qh.prepack(qh.fp4_matrix(tensors[2], tensors[3], rows, padded,
                                            padded, scheme), device)
    d_act = gu.device_tensor(ol.bf16_bits(act), device)
    workspace, size = _balance_workspace(device)
    plain = torch.zeros((batch, rows), dtype=torch.bfloat16, device=device)
    qh.call("qllm_fp4_swiglu_bf16", gate_m, up_m, qh.ptr(d_act), d_act.numel() * 2,
            qh.ptr(plain), batch, None)
    runs = []
    for _ in range(3):
        out = torch.zeros((batch, rows), dtype=torch.bfloat16, device=device)
        qh.call("qllm_fp4_swiglu_bf16_balanced", gate_m, up_m, qh.ptr(d_act),
                d_act.numel() * 2, qh.ptr(out), batch, qh.ptr(workspace), size, None)
        torch.cuda.synchronize()
        runs.append(out.view(torch.uint16).cpu().numpy())
        assert int(workspace[:4096].view(torch.int32).abs().sum()) == 0
    assert np.array_equal(runs[0], runs[1]) and np.array_equal(runs[0], runs[2])
    units = torch.cuda.get_device_properties(device).multi_processor_count
    tiles = (rows + 31) // 32
    uncut = (tiles - tiles % units) * 32 if tiles > units else rows
    assert np.array_equal(runs[0][:, :uncut], plain.view(torch.uint16).cpu().numpy()[:, :uncut])
    # a sample of rows against the oracle (all of the cut ones)
    pick = np.unique(np.concatenate([rng.choice(rows, 256, replace=False),
                                     np.arange(min(uncut, rows - 1), rows)]))
    g = ol.fp4_linear_f64(gate[0][pick], gate[1][pick], scheme, len(pick), padded, act)
    u = ol.fp4_linear_f64(up[0][pick], up[1][pick], scheme, len(pick), padded, act)
    got = ol.bf16_from_bits(runs[0])[:, pick]
    gu.assert_close(got, ol.silu_product(g, u, True), rtol=1e-2, atol=1e-3, what="balanced swiglu")
    del keep_g, keep_u


@pytest.mark.parametrize("scheme", [ol.SCALE_F16_BLOCK16, ol.SCALE_UE8M0_BLOCK32])
def test_balanced_split_projection_matches_oracle(device, scheme):
    """q/k/v of the 27B shape ([8192 + 1024 + 1024, 5120], 320 tiles): the 64
    tiles past the first round are cut in four."""
    rng = np.random.default_rng(41 + scheme)
    rows, padded, batch = 10240, 5120, 5
    codes, scales = synth.fp4_matrix(rng, rows, padded, scheme)
    act = ol.bf16_round(rng.standard_normal((batch, padded)).astype(np.float32))
    tensors = [gu.device_tensor(x, device) for x in (codes, scales)]
    matrix, keep = qh.prepack(qh.fp4_matrix(tensors[0], tensors[1], rows, padded, padded,
                                            scheme), device)
    d_act = gu.device_tensor(ol.bf16_bits(act), device)
    workspace, size = _balance_workspace(device)
    parts = [8192, 1024, 1024]
    outs = [torch.zeros((batch, part), device=device) for part in parts]
    segments = (qh.GemmSegment * 3)(*[qh.GemmSegment(qh.ptr(o), part, qh.OUT_F32)
                                      for o, part in zip(outs, parts)])
    for _ in range(2):
        qh.call("qllm_fp4_gemm_bf16_split_balanced", matrix, qh.ptr(d_act),
                d_act.numel() * 2, segments, 3, batch, qh.ptr(workspace), size, None)
    torch.cuda.synchronize()
    got = np.concatenate([o.cpu().numpy() for o in outs], axis=1)
    pick = np.unique(np.concatenate([rng.choice(rows, 384, replace=False),
                                     np.arange(8192, rows, 7)]))
    want = ol.fp4_linear_f64(codes[pick], scales[pick], scheme, len(pick), padded, act)
    gu.assert_close(got[:, pick], want, what="balanced q/k/v")
    plain = gu.gemm(device, codes, scales, scheme, rows, padded, act)
    assert np.array_equal(got[:, :8192], plain[:, :8192])
    np.testing.assert_allclose(got, plain, rtol=1e-4, atol=1e-3)
    assert int(workspace[:4096].view(torch.int32).abs().sum()) == 0
    del keep


def test_balanced_launch_rejects_a_bad_workspace(device):
    rng = np.random.default_rng(2)
    codes, scales = synth.fp4_matrix(rng, 64, 128, ol.SCALE_F16_BLOCK16)
    tensors = [gu.device_tensor(x, device) for x in (codes, scales)]
    matrix, keep = qh.prepack(qh.fp4_matrix(tensors[0], tensors[1], 64, 128, 128,
                                            ol.SCALE_F16_BLOCK16), device)
    buffer = torch.zeros(4096, device=device)
    with pytest.raises(qh.QllmError):
        qh.call("qllm_fp4_swiglu_bf16_balanced", matrix, matrix, qh.ptr(buffer), 5 * 256,
                qh.ptr(buffer), 5, qh.ptr(buffer), 1024, None)
    with pytest.raises(qh.QllmError):
        qh.call("qllm_fp4_swiglu_bf16_balanced", matrix, matrix, qh.ptr(buffer), 5 * 256,
                qh.ptr(buffer), 5, 0, 1 << 22, None)
    del keep


# ---- the reference's default activation contract (Q8 rows) on the matrix cores ----

def _q8_case(device, rng, rows, columns, batch, x=None):
    padded = (columns + 63) // 64 * 64
    codes, scales = synth.fp4_matrix(rng, rows, padded, ol.SCALE_UE8M0_BLOCK32)
    if x is None:
        x = rng.standard_normal((batch, columns)).astype(np.float32)
    q8, act_scales = ol.quantize_q8_rows(x, padded)
    tensors = [gu.device_tensor(t, device) for t in (codes, scales)]
    matrix, keep = qh.prepack(qh.fp4_matrix(tensors[0], tensors[1], rows, columns, padded,
                                            ol.SCALE_UE8M0_BLOCK32), device)
    return (codes, scales, padded, q8, act_scales, matrix, (tensors, keep),
            gu.device_tensor(q8, device), gu.device_tensor(act_scales, device))


def test_q8_matrix_core_gemm_on_the_reference_fixture(device):
    """dense_fp4_cuda_smoke.cpp:139-216 (67 x 100 padded to 128, five rows of
    0.7 sin(0.071 i)), its own threshold 2e-4 (:4911), through the streaming
    layout and the matrix cores."""
    rows, columns, padded, batch = 67, 100, 128, 5
    r = np.arange(rows)[:, None]
    scales = (124 + (r + np.arange(padded // 32)[None, :]) % 7).astype(np.uint8)
    pair = np.arange(padded // 2)[None, :]
    codes = (((r + 3 * pair) % 16) | (((5 * r + pair + 1) % 16) << 4)).astype(np.uint8)
    x = (np.sin(np.arange(batch * columns, dtype=np.float32) * np.float32(0.071)) *
         np.float32(0.7)).astype(np.float32).reshape(batch, columns)
    q8, act_scales = ol.quantize_q8_rows(x, padded)
    want = ol.fp4_linear_block32_q8(codes, scales, rows, padded, q8, act_scales)
    d_codes, d_scales = gu.device_tensor(codes, device), gu.device_tensor(scales, device)
    matrix, keep = qh.prepack(qh.fp4_matrix(d_codes, d_scales, rows, columns, padded, 0), device)
    d_q8, d_s = gu.device_tensor(q8, device), gu.device_tensor(act_scales, device)
    out = torch.zeros((batch, rows), device=device)
    qh.call("qllm_fp4_gemv_q8_batch", matrix, qh.ptr(d_q8), qh.ptr(d_s), qh.ptr(out), batch,
            0, None)
    torch.cuda.synchronize()
    assert np.abs(out.cpu().numpy() - want).max() < 2e-4
    del keep


@pytest.mark.parametrize("rows,columns,batch", [
    (17408, 5120, 5), (5120, 17408, 5), (10240, 5120, 5), (5120, 8192, 5), (320, 192, 1),
    (1000, 1000, 8), (96, 64, 3)])
def test_q8_matrix_core_gemm_matches_the_integer_statement(device, rows, columns, batch):
    """Model shapes (gate/up, down, q/k/v, o) and ragged ones against
    qo_fp4_linear_block32_q8 - integer block sums, one F32 FMA per block - at
    the reference's own 2e-4; with a residual and the three output kinds."""
    rng = np.random.default_rng(rows * 7 + columns)
    codes, scales, padded, q8, act_scales, matrix, keep, d_q8, d_s = _q8_case(
        device, rng, rows, columns, batch)
    want = ol.fp4_linear_block32_q8(codes, scales, rows, padded, q8, act_scales)
    bound = 2e-4 * max(1.0, np.abs(want).max())
    out = torch.zeros((batch, rows), device=device)
    qh.call("qllm_fp4_gemm_q8", matrix, qh.ptr(d_q8), qh.ptr(d_s), qh.ptr(out), qh.OUT_F32,
            None, batch, None)
    torch.cuda.synchronize()
    assert np.abs(out.cpu().numpy() - want).max() <= bound
    residual = rng.standard_normal((batch, rows)).astype(np.float32)
    d_residual = gu.device_tensor(residual, device)
    qh.call("qllm_fp4_gemm_q8", matrix, qh.ptr(d_q8), qh.ptr(d_s), qh.ptr(d_residual),
            qh.OUT_F32, qh.ptr(d_residual), batch, None)
    rounded = torch.zeros((batch, rows), device=device)
    qh.call("qllm_fp4_gemm_q8", matrix, qh.ptr(d_q8), qh.ptr(d_s), qh.ptr(rounded),
            qh.OUT_F32_BF16_ROUNDED, None, batch, None)
    torch.cuda.synchronize()
    assert np.abs(d_residual.cpu().numpy() - (want + residual)).max() <= bound + 1e-5
    assert np.array_equal(rounded.cpu().numpy(), ol.bf16_round(out.cpu().numpy()))
    del keep


def test_q8_matrix_core_head_on_sampled_vocabulary_rows(device):
    """lm_head [151936, 5120] x Q8 rows: the whole launch, 512 sampled rows
    against the integer statement."""
    rows, columns, batch = 151936, 5120, 5
    codes = torch.randint(0, 256, (rows, columns // 2), dtype=torch.uint8, device=device)
    scales = torch.randint(118, 124, (rows, columns // 32), dtype=torch.uint8, device=device)
    matrix, keep = qh.prepack(qh.fp4_matrix(codes, scales, rows, columns, columns, 0), device)
    rng = np.random.default_rng(9)
    x = rng.standard_normal((batch, columns)).astype(np.float32)
    q8, act_scales = ol.quantize_q8_rows(x, columns)
    d_q8, d_s = gu.device_tensor(q8, device), gu.device_tensor(act_scales, device)
    out = torch.zeros((batch, rows), device=device)
    qh.call("qllm_fp4_gemm_q8", matrix, qh.ptr(d_q8), qh.ptr(d_s), qh.ptr(out), qh.OUT_F32,
            None, batch, None)
    torch.cuda.synchronize()
    pick = np.sort(rng.choice(rows, 512, replace=False))
    index = torch.from_numpy(pick).to(device)
    want = ol.fp4_linear_block32_q8(codes[index].cpu().numpy(), scales[index].cpu().numpy(),
                                    len(pick), columns, q8, act_scales)
    got = out.cpu().numpy()[:, pick]
    assert np.abs(got - want).max() <= 2e-4 * max(1.0, np.abs(want).max())
    del keep


def test_q8_split_and_swiglu_forms(device):
    """q/k/v as three segments equal the one-output launch bit for bit; the
    fused gate/up launch stores silu(gate) * up in F32 from the same sums."""
    rng = np.random.default_rng(77)
    rows, columns, batch = 1536, 1024, 5
    codes, scales, padded, q8, act_scales, matrix, keep, d_q8, d_s = _q8_case(
        device, rng, rows, columns, batch)
    whole = torch.zeros((batch, rows), device=device)
    qh.call("qllm_fp4_gemm_q8", matrix, qh.ptr(d_q8), qh.ptr(d_s), qh.ptr(whole), qh.OUT_F32,
            None, batch, None)
    parts = [1024, 256, 256]
    outs = [torch.zeros((batch, part), device=device) for part in parts]
    segments = (qh.GemmSegment * 3)(*[qh.GemmSegment(qh.ptr(o), part, qh.OUT_F32)
                                      for o, part in zip(outs, parts)])
    qh.call("qllm_fp4_gemm_q8_split", matrix, qh.ptr(d_q8), qh.ptr(d_s), segments, 3, batch,
            None, 0, None)
    up_codes, up_scales = synth.fp4_matrix(rng, rows, padded, ol.SCALE_UE8M0_BLOCK32)
    up_tensors = [gu.device_tensor(t, device) for t in (up_codes, up_scales)]
    up_matrix, keep_up = qh.prepack(qh.fp4_matrix(up_tensors[0], up_tensors[1], rows, columns,
                                                  padded, 0), device)
    fused = torch.zeros((batch, rows), device=device)
    qh.call("qllm_fp4_swiglu_q8", matrix, up_matrix, qh.ptr(d_q8), qh.ptr(d_s),
            qh.ptr(fused), batch, None, 0, None)
    torch.cuda.synchronize()
    assert np.array_equal(np.concatenate([o.cpu().numpy() for o in outs], axis=1),
                          whole.cpu().numpy())
    gate = ol.fp4_linear_block32_q8(codes, scales, rows, padded, q8, act_scales)
    up = ol.fp4_linear_block32_q8(up_codes, up_scales, rows, padded, q8, act_scales)
    want = ol.silu_product(gate, up, False)
    got = fused.cpu().numpy()
    assert np.abs(got - want).max() <= 2e-4 * max(1.0, np.abs(want).max())
    del keep, keep_up


@pytest.mark.parametrize("rows,columns,batch,splits", [(5120, 17408, 5, 3), (5120, 8192, 5, 3),
                                                       (320, 1024, 8, 2), (64, 128, 1, 2)])
def test_q8_k_split_partials_add_up_to_the_integer_statement(device, rows, columns, batch,
                                                             splits):
    """qllm_fp4_gemm_q8_partial: split s holds the blocks of its share of K times
    the row scale; added in index order they are the reference's sum within its
    2e-4 (the F32 additions are regrouped, nothing else), and
    qllm_rms_norm_partials_q8_batch finishes residual + sum and leaves the
    bytes qllm_rms_norm_q8_batch leaves for the same row."""
    rng = np.random.default_rng(rows + columns)
    codes, scales, padded, q8, act_scales, matrix, keep, d_q8, d_s = _q8_case(
        device, rng, rows, columns, batch)
    partials = torch.zeros((splits, batch, rows), device=device)
    qh.call("qllm_fp4_gemm_q8_partial", matrix, qh.ptr(d_q8), qh.ptr(d_s), qh.ptr(partials),
            splits, batch, None)
    torch.cuda.synchronize()
    want = ol.fp4_linear_block32_q8(codes, scales, rows, padded, q8, act_scales)
    parts = partials.cpu().numpy()
    total = parts[0].copy()
    for index in range(1, splits):
        total += parts[index]
    assert np.abs(total - want).max() <= 2e-4 * max(1.0, np.abs(want).max())
    assert all(np.abs(parts[index]).max() > 0 for index in range(splits))
    if rows % 4 == 0 and rows <= 16384:
        residual = rng.standard_normal((batch, rows)).astype(np.float32)
        weight = (0.1 * rng.standard_normal(rows)).astype(np.float32)
        d_residual, d_weight = gu.device_tensor(residual, device), gu.device_tensor(weight, device)
        summed = torch.zeros((batch, rows), device=device)
        out = torch.zeros((batch, rows), dtype=torch.int8, device=device)
        out_scales = torch.zeros(batch, device=device)
        qh.call("qllm_rms_norm_partials_q8_batch", qh.ptr(d_residual), qh.ptr(summed),
                qh.ptr(partials), splits, qh.ptr(d_weight), qh.ptr(out), qh.ptr(out_scales),
                batch, rows, 1e-6, 1, None)
        torch.cuda.synchronize()
        expected_sum = residual.copy()
        for index in range(splits):
            expected_sum += parts[index]
        assert np.array_equal(summed.cpu().numpy(), expected_sum)
        assert np.array_equal(d_residual.cpu().numpy(), residual)
        d_sum = gu.device_tensor(expected_sum, device)
        plain = torch.zeros_like(out)
        plain_scales = torch.zeros_like(out_scales)
        qh.call("qllm_rms_norm_q8_batch", qh.ptr(d_sum), qh.ptr(d_weight), qh.ptr(plain),
                qh.ptr(plain_scales), batch, rows, 1e-6, 1, None)
        torch.cuda.synchronize()
        assert torch.equal(out, plain) and torch.equal(out_scales, plain_scales)
    with pytest.raises(qh.QllmError):      # more splits than chunks of K
        qh.call("qllm_fp4_gemm_q8_partial", matrix, qh.ptr(d_q8), qh.ptr(d_s),
                qh.ptr(partials), padded // 64 + 1, batch, None)
    del keep


def test_q8_matrix_core_gemm_rejects_what_it_does_not_take(device):
    rng = np.random.default_rng(3)
    codes, scales, padded, q8, act_scales, matrix, keep, d_q8, d_s = _q8_case(
        device, rng, 64, 128, 2)
    out = torch.zeros((2, 64), device=device)
    f16_codes, f16_scales = synth.fp4_matrix(rng, 64, 128, ol.SCALE_F16_BLOCK16)
    tensors = [gu.device_tensor(t, device) for t in (f16_codes, f16_scales)]
    f16_matrix, keep2 = qh.prepack(qh.fp4_matrix(tensors[0], tensors[1], 64, 128, 128,
                                                 ol.SCALE_F16_BLOCK16), device)
    with pytest.raises(qh.QllmError):      # binary16 block-16 scales have no Q8 form
        qh.call("qllm_fp4_gemm_q8", f16_matrix, qh.ptr(d_q8), qh.ptr(d_s), qh.ptr(out),
                qh.OUT_F32, None, 2, None)
    with pytest.raises(qh.QllmError):      # no scales
        qh.call("qllm_fp4_gemm_q8", matrix, qh.ptr(d_q8), None, qh.ptr(out), qh.OUT_F32,
                None, 2, None)
    with pytest.raises(qh.QllmError):      # batch > 8
        qh.call("qllm_fp4_gemm_q8", matrix, qh.ptr(d_q8), qh.ptr(d_s), qh.ptr(out),
                qh.OUT_F32, None, 9, None)
    del keep, keep2


def _head_argmax(device, matrix, act, batch, advance=None):
    rows = matrix.rows
    logits = torch.full((batch, rows), -7.0, device=device)
    tokens = torch.full((batch,), 12345, dtype=torch.int32, device=device)
    need = qh.call("qllm_fp4_head_workspace_bytes", matrix, batch)
    workspace = torch.zeros(need, dtype=torch.uint8, device=device)
    d_act = gu.device_tensor(ol.bf16_bits(act), device)
    qh.call("qllm_fp4_head_argmax", matrix, qh.ptr(d_act), d_act.numel() * 2,
            qh.ptr(logits), batch, qh.ptr(tokens), qh.ptr(workspace), need, advance, None)
    torch.cuda.synchronize()
    return logits, tokens.cpu().numpy().astype(np.uint32)


def _two_pass_argmax(device, logits):
    batch, rows = logits.shape
    tokens = torch.zeros(batch, dtype=torch.int32, device=device)
    need = qh.call("qllm_argmax_workspace_bytes", rows, batch)
    workspace = torch.zeros(need, dtype=torch.uint8, device=device)
    qh.call("qllm_argmax_batch", qh.ptr(logits), rows, batch, qh.ptr(tokens),
            qh.ptr(workspace), need, None)
    torch.cuda.synchronize()
    return tokens.cpu().numpy().astype(np.uint32)


@pytest.mark.parametrize("tiled", [True, False])
@pytest.mark.parametrize("scheme", [ol.SCALE_UE8M0_BLOCK32, ol.SCALE_F16_BLOCK16])
@pytest.mark.parametrize("rows,padded,batch", [(1000, 1024, 5), (4099, 512, 8), (31, 64, 1),
                                               (20000, 256, 3)])
def test_head_with_argmax_equals_projection_then_argmax(device, scheme, rows, padded, batch,
                                                        tiled):
    """The head's projection with the arg-max taken in its epilogue: logits bit
    for bit those of the plain projection, tokens those of qllm_argmax_batch
    on them and of numpy on the oracle's ordering; vocabulary sizes that end
    inside a tile."""
    rng = np.random.default_rng(rows + padded + batch + scheme)
    codes, scales = synth.fp4_matrix(rng, rows, padded, scheme)
    act = ol.bf16_round(rng.standard_normal((batch, padded)).astype(np.float32))
    tensors = [gu.device_tensor(t, device) for t in (codes, scales)]
    matrix = qh.fp4_matrix(tensors[0], tensors[1], rows, padded, padded, scheme)
    keep = None
    if tiled:
        matrix, keep = qh.prepack(matrix, device)
    logits, tokens = _head_argmax(device, matrix, act, batch)
    plain = gu.gemm(device, codes, scales, scheme, rows, padded, act, tiled=tiled)
    got = logits.cpu().numpy()
    assert np.array_equal(got, plain)
    assert np.array_equal(tokens, _two_pass_argmax(device, logits))
    assert np.array_equal(tokens, got.argmax(axis=1).astype(np.uint32))
    del keep


def test_head_with_argmax_ties_and_nan(device):
    """Equal logits go to the lower row wherever the rows lie (same tile, other
    tiles); a row whose scale is NaN never wins; a head of NaN rows only selects
    nothing (0xffffffff), as qllm_argmax_batch does."""
    rng = np.random.default_rng(5)
    rows, padded, batch = 700, 256, 4
    codes, scales = synth.fp4_matrix(rng, rows, padded, ol.SCALE_UE8M0_BLOCK32)
    act = ol.bf16_round(rng.standard_normal((batch, padded)).astype(np.float32))
    reference = ol.fp4_linear_f64(codes, scales, ol.SCALE_UE8M0_BLOCK32, rows, padded, act)
    winner = int(reference[0].argmax())
    for copy in (3, 40, 650):                  # the same row thrice more: exact ties
        if copy != winner:
            codes[copy], scales[copy] = codes[winner], scales[winner]
    scales[1, 0] = 255                         # UE8M0 NaN: row 1 is NaN for every batch row
    tensors = [gu.device_tensor(t, device) for t in (codes, scales)]
    matrix, keep = qh.prepack(qh.fp4_matrix(tensors[0], tensors[1], rows, padded, padded,
                                            ol.SCALE_UE8M0_BLOCK32), device)
    logits, tokens = _head_argmax(device, matrix, act, batch)
    got = logits.cpu().numpy()
    assert np.isnan(got[:, 1]).all()
    assert tokens[0] == min(winner, 3)
    assert np.array_equal(tokens, _two_pass_argmax(device, logits))
    assert np.array_equal(tokens, np.nanargmax(got, axis=1).astype(np.uint32))
    scales[:, 0] = 255
    d_scales = gu.device_tensor(scales, device)
    matrix, keep = qh.prepack(qh.fp4_matrix(tensors[0], d_scales, rows, padded, padded,
                                            ol.SCALE_UE8M0_BLOCK32), device)
    logits, tokens = _head_argmax(device, matrix, act, batch)
    assert np.isnan(logits.cpu().numpy()).all()
    assert (tokens == 0xFFFFFFFF).all()
    assert np.array_equal(tokens, _two_pass_argmax(device, logits))
    del keep


def test_head_with_argmax_hands_the_winner_to_the_next_pass(device):
    """With a rollout step the selection kernel also does what
    qllm_rollout_advance does: next token, draft list entry, positions."""
    rng = np.random.default_rng(6)
    rows, padded = 5000, 512
    codes, scales = synth.fp4_matrix(rng, rows, padded, ol.SCALE_UE8M0_BLOCK32)
    act = ol.bf16_round(rng.standard_normal((1, padded)).astype(np.float32))
    tensors = [gu.device_tensor(t, device) for t in (codes, scales)]
    matrix, keep = qh.prepack(qh.fp4_matrix(tensors[0], tensors[1], rows, padded, padded,
                                            ol.SCALE_UE8M0_BLOCK32), device)
    for slot, capacity in ((1, 4), (4, 4)):    # a free draft entry; a full list
        state = []
        for fused in (True, False):
            next_token = torch.full((1,), 77, dtype=torch.int32, device=device)
            drafts = torch.full((4,), 99, dtype=torch.int32, device=device)
            positions = torch.tensor([10, 11, 12, slot], dtype=torch.int32, device=device)
            step = qh.RolloutStep(qh.ptr(next_token), qh.ptr(drafts), capacity, 3,
                                  qh.ptr(positions))
            if fused:
                logits, tokens = _head_argmax(device, matrix, act, 1, step)
            else:
                logits, tokens = _head_argmax(device, matrix, act, 1)
                selected = torch.tensor(tokens.astype(np.int32), device=device)
                qh.call("qllm_rollout_advance", qh.ptr(selected), qh.ptr(next_token),
                        qh.ptr(drafts), capacity, 3, qh.ptr(positions), None)
                torch.cuda.synchronize()
            state.append((tokens.tolist(), next_token.tolist(), drafts.tolist(),
                          positions.tolist()))
        assert state[0] == state[1]
        token = state[0][0][0]
        assert token == int(logits.cpu().numpy()[0].argmax())
        assert state[0][1] == [token]
        assert state[0][2] == [token if entry == slot else 99 for entry in range(4)]
        assert state[0][3] == [13, 14, 15, slot + 1]
    del keep


def test_head_with_argmax_rejects_what_it_does_not_take(device):
    rng = np.random.default_rng(8)
    rows, padded = 64, 128
    codes, scales = synth.fp4_matrix(rng, rows, padded, ol.SCALE_UE8M0_BLOCK32)
    tensors = [gu.device_tensor(t, device) for t in (codes, scales)]
    matrix = qh.fp4_matrix(tensors[0], tensors[1], rows, padded, padded,
                           ol.SCALE_UE8M0_BLOCK32)
    act = torch.zeros((2, padded), dtype=torch.bfloat16, device=device)
    logits = torch.zeros((2, rows), device=device)
    tokens = torch.zeros(2, dtype=torch.int32, device=device)
    need = qh.call("qllm_fp4_head_workspace_bytes", matrix, 2)
    workspace = torch.zeros(need, dtype=torch.uint8, device=device)
    step = qh.RolloutStep(qh.ptr(tokens), qh.ptr(tokens), 1, 1, qh.ptr(tokens))

    def status(*arguments):
        return qh.load().qllm_fp4_head_argmax(*arguments)

    good = [matrix, qh.ptr(act), act.numel() * 2, qh.ptr(logits), 2, qh.ptr(tokens),
            qh.ptr(workspace), need, None, None]
    assert status(*good) == 0
    torch.cuda.synchronize()
    for index, value in ((7, need - 1), (4, 9), (4, 0), (2, act.numel() * 2 - 1),
                         (5, None), (6, None), (8, step)):   # a rollout step takes one row
        bad = list(good)
        bad[index] = value
        assert status(*bad) == 4, index        # QLLM_INVALID_ARGUMENT
