"""GPU parity of the batched matMul/matMulAdd operator against the CPU oracle, through the C-ABI.

Bars: int8 -> int32 bit-exact; fp16 and e4m3 within max(2 ulp-fp16, 1e-3 relative,
2^-18 * sum|terms|) of the fp32-accumulated oracle (oracle_binding.float_parity_violations)."""
import json
import os

import numpy as np
import pytest
import torch

import oracle_binding as ob
from gpu_util import DEV, as_bytes, fp16_inputs, fp16_weights, matrix_in_layout, to_dev
from slang_amd import coopvec as cv
from slang_amd.coopvec import Activation, CoopVecComponentType as CT, CoopVecMatrixLayout as ML

pytestmark = pytest.mark.gpu

G = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "coopvec_goldens.json")))


# ---- the reference's golden vectors through the GPU path ------------------------------------

def test_goldens_fp16():
    g = G["matmul_f16"]
    x = to_dev(np.array([g["input"]], np.float16))
    W = as_bytes(to_dev(np.array(g["matrix_row_major_4x4"], np.float16)))
    b = as_bytes(to_dev(np.array(G["matmul_bias_f16"]["bias"], np.float16)))
    y = cv.coopVecMatMul(x, CT.Float16, W, 0, CT.Float16, ML.RowMajor, False, 8, M=4)
    assert y.cpu().numpy()[0].tolist() == g["expected"]
    y = cv.coopVecMatMulAdd(x, CT.Float16, W, 0, CT.Float16, b, 0, CT.Float16, ML.RowMajor, False, 8, M=4)
    assert y.cpu().numpy()[0].tolist() == G["matmul_bias_f16"]["expected"]
    acc = to_dev(np.array([G["matmul_f16_mut"]["initial"]], np.float16))
    cv.coopVecMatMul(x, CT.Float16, W, 0, CT.Float16, ML.RowMajor, False, 8, M=4, out=acc, accumulate=True)
    assert acc.cpu().numpy()[0].tolist() == G["matmul_f16_mut"]["expected"]
    acc = to_dev(np.array([G["matmul_bias_f16_mut"]["initial"]], np.float16))
    cv.coopVecMatMulAdd(x, CT.Float16, W, 0, CT.Float16, b, 0, CT.Float16, ML.RowMajor, False, 8, M=4,
                        out=acc, accumulate=True)
    assert acc.cpu().numpy()[0].tolist() == G["matmul_bias_f16_mut"]["expected"]


def test_goldens_int8_packed():
    g = G["matmul_i8_packed"]
    x = to_dev(np.array([g["input_bytes"]], np.int8).view(np.int32))          # one packed element
    W = as_bytes(to_dev(np.array(g["matrix_row_major_4x4_bytes"], np.int8)))
    b = as_bytes(to_dev(np.array(G["matmul_bias_i8_packed"]["bias_int32"], np.int32)))
    y = cv.coopVecMatMulPacked(x, CT.SignedInt8Packed, 4, W, 0, CT.SignedInt8, ML.RowMajor, False, 4, M=4)
    assert y.cpu().numpy()[0].tolist() == g["expected"]
    y = cv.coopVecMatMulAddPacked(x, CT.SignedInt8Packed, 4, W, 0, CT.SignedInt8, b, 0, CT.SignedInt32,
                                  ML.RowMajor, False, 4, M=4)
    assert y.cpu().numpy()[0].tolist() == G["matmul_bias_i8_packed"]["expected"]
    acc = to_dev(np.array([G["matmul_i8_packed_mut"]["initial"]], np.int32))
    cv.coopVecMatMulPacked(x, CT.SignedInt8Packed, 4, W, 0, CT.SignedInt8, ML.RowMajor, False, 4, M=4,
                           out=acc, accumulate=True)
    assert acc.cpu().numpy()[0].tolist() == G["matmul_i8_packed_mut"]["expected"]
    acc = to_dev(np.array([G["matmul_bias_i8_packed_mut"]["initial"]], np.int32))
    cv.coopVecMatMulAddPacked(x, CT.SignedInt8Packed, 4, W, 0, CT.SignedInt8, b, 0, CT.SignedInt32,
                              ML.RowMajor, False, 4, M=4, out=acc, accumulate=True)
    assert acc.cpu().numpy()[0].tolist() == G["matmul_bias_i8_packed_mut"]["expected"]
    with pytest.raises(cv.CoopVecError):     # static_assert hlsl.meta.slang:32965
        cv.coopVecMatMul(x, CT.SignedInt8Packed, W, 0, CT.SignedInt8, ML.RowMajor, False, 4, M=4)


# ---- fp16 ---------------------------------------------------------------------------------

def run_fp16(x, W, b, layout, stride=0, act=Activation.NoActivation, slope=0.0, result=CT.Float16):
    M, K = W.shape
    wb = to_dev(matrix_in_layout(W, CT.Float16, layout, stride))
    bb = as_bytes(to_dev(b)) if b is not None else None
    st = stride if stride else (K * 2 if layout == ML.RowMajor else M * 2)
    xd = to_dev(x)
    if b is None:
        return cv.coopVecMatMul(xd, CT.Float16, wb, 0, CT.Float16, layout, False, st, M=M, resultType=result)
    return cv.coopVecMatMulAdd(xd, CT.Float16, wb, 0, CT.Float16, bb, 0, CT.Float16, layout, False, st, M=M,
                               resultType=result, activation=act, leakySlope=slope)


@pytest.mark.parametrize("layout", [ML.RowMajor, ML.ColumnMajor, ML.InferencingOptimal, ML.TrainingOptimal])
def test_fp16_64x64_all_layouts(layout):
    # the single-layer config: inputs N(0,1), weights N(0,1/64), bias U[-0.1,0.1]; ragged batch
    rng = np.random.default_rng(42)
    B, M, K = 4096 + 37, 64, 64
    x, W = fp16_inputs(rng, B, K), fp16_weights(rng, M, K)
    b = rng.uniform(-0.1, 0.1, M).astype(np.float16)
    y = run_fp16(x, W, b, layout).cpu().numpy()
    ref, ab = ob.ref_matmul_f32(x, ob.F16, W, ob.F16, ob.ROW, K * 2, M, K, b, ob.F16)
    bad = ob.float_parity_violations(y, ref, ab)
    assert not bad.any(), "%d of %d outside tolerance" % (bad.sum(), bad.size)
    # the layout only changes where the bytes come from: results are bit-identical to RowMajor
    y0 = run_fp16(x, W, b, ML.RowMajor).cpu().numpy()
    assert (y.view(np.uint16) == y0.view(np.uint16)).all()


@pytest.mark.parametrize("M,K", [(1, 16), (16, 2), (16, 16), (40, 24), (5, 7), (128, 128), (100, 70),
                                 (64, 8), (1, 64), (8, 64), (33, 17), (128, 32), (32, 128)])
def test_fp16_shapes(M, K):
    rng = np.random.default_rng(M * 1000 + K)
    B = 333
    x, W = fp16_inputs(rng, B, K), fp16_weights(rng, M, K)
    b = rng.uniform(-0.1, 0.1, M).astype(np.float16)
    ref, ab = ob.ref_matmul_f32(x, ob.F16, W, ob.F16, ob.ROW, K * 2, M, K, b, ob.F16)
    for layout in (ML.RowMajor, ML.InferencingOptimal):
        y = run_fp16(x, W, b, layout).cpu().numpy()
        assert y.shape == (B, M)
        assert not ob.float_parity_violations(y, ref, ab).any()


def test_fp16_strided_matrix_offsets_and_vector_strides():
    rng = np.random.default_rng(5)
    B, M, K = 200, 24, 40
    x, W = fp16_inputs(rng, B, K), fp16_weights(rng, M, K)
    b = rng.uniform(-0.1, 0.1, M).astype(np.float16)
    ref, ab = ob.ref_matmul_f32(x, ob.F16, W, ob.F16, ob.ROW, K * 2, M, K, b, ob.F16)
    # row stride with padding, matrix and bias at non-zero (64-byte aligned) offsets in one buffer
    stride = K * 2 + 48
    wbytes = matrix_in_layout(W, CT.Float16, ML.RowMajor, stride)
    buf = np.full(256 + len(wbytes) + 192, 0xEE, np.uint8)
    buf[128:128 + len(wbytes)] = wbytes
    boff = 128 + (len(wbytes) + 63) // 64 * 64
    buf[boff:boff + M * 2] = b.view(np.uint8)
    d = to_dev(buf)
    # input rows padded to 96 halfs (16-byte aligned) and to 41 halfs (2-byte aligned only)
    for pad in (96, 41):
        xp = np.zeros((B, pad), np.float16); xp[:, :K] = x
        xd = to_dev(xp)[:, :K]
        out = torch.zeros(B, M + 3, dtype=torch.float16, device=DEV)[:, :M]
        cv.coopVecMatMulAdd(xd, CT.Float16, d, 128, CT.Float16, d, boff, CT.Float16, ML.RowMajor, False, stride,
                            M=M, out=out)
        assert not ob.float_parity_violations(out.cpu().numpy(), ref, ab).any()


def test_fp16_activations_result_types_and_transpose():
    rng = np.random.default_rng(6)
    B, M, K = 500, 64, 32
    x, W = fp16_inputs(rng, B, K), fp16_weights(rng, M, K)
    b = rng.uniform(-0.1, 0.1, M).astype(np.float16)
    ref, ab = ob.ref_matmul_f32(x, ob.F16, W, ob.F16, ob.ROW, K * 2, M, K, b, ob.F16)
    y = run_fp16(x, W, b, ML.RowMajor).cpu().numpy()
    yr = run_fp16(x, W, b, ML.RowMajor, act=Activation.ReLU).cpu().numpy()
    assert (yr == np.maximum(y, np.float16(0))).all()
    slope = float(np.float16(0.001))
    yl = run_fp16(x, W, b, ML.InferencingOptimal, act=Activation.LeakyReLU, slope=slope).cpu().numpy()
    want = np.maximum(y, (y.astype(np.float32) * np.float32(slope)).astype(np.float16))
    assert (yl.view(np.uint16) == want.view(np.uint16)).all()
    # fp32 result type: no final rounding
    y32 = run_fp16(x, W, b, ML.RowMajor, result=CT.Float32).cpu().numpy()
    assert y32.dtype == np.float32
    assert np.max(np.abs(y32 - ref) / np.maximum(ab, 1e-30)) < 2.0 ** -18
    assert (y32.astype(np.float16) == y).mean() > 0.999
    # transpose with an Optimal layout: memory holds the K x M matrix W^T
    wT = to_dev(matrix_in_layout(np.ascontiguousarray(W.T), CT.Float16, ML.InferencingOptimal))
    yt = cv.coopVecMatMulAdd(to_dev(x), CT.Float16, wT, 0, CT.Float16, as_bytes(to_dev(b)), 0, CT.Float16,
                             ML.InferencingOptimal, True, 0, M=M).cpu().numpy()
    assert (yt.view(np.uint16) == y.view(np.uint16)).all()
    # ColumnMajor storage of W^T with the same stride is RowMajor W (fflayer.slang:46-55)
    yc = cv.coopVecMatMul(to_dev(x), CT.Float16, as_bytes(to_dev(W)), 0, CT.Float16, ML.RowMajor, False, K * 2, M=M)
    yd = cv.coopVecMatMul(to_dev(x), CT.Float16, as_bytes(to_dev(np.ascontiguousarray(W.T))), 0, CT.Float16,
                          ML.ColumnMajor, False, M * 2, M=M)
    assert torch.equal(yc, yd)


def test_empty_and_tiny_batches():
    rng = np.random.default_rng(8)
    M, K = 64, 64
    W = fp16_weights(rng, M, K)
    wb = as_bytes(to_dev(W))
    x0 = torch.zeros(0, K, dtype=torch.float16, device=DEV)
    y0 = cv.coopVecMatMul(x0, CT.Float16, wb, 0, CT.Float16, ML.RowMajor, False, K * 2, M=M)
    assert y0.shape == (0, M)
    for B in (1, 15, 16, 17, 63, 64, 65, 255, 257):
        x = fp16_inputs(rng, B, K)
        y = cv.coopVecMatMul(to_dev(x), CT.Float16, wb, 0, CT.Float16, ML.RowMajor, False, K * 2, M=M)
        ref, ab = ob.ref_matmul_f32(x, ob.F16, W, ob.F16, ob.ROW, K * 2, M, K)
        assert not ob.float_parity_violations(y.cpu().numpy(), ref, ab).any()


# ---- int8 ---------------------------------------------------------------------------------

@pytest.mark.parametrize("layout", [ML.ColumnMajor, ML.InferencingOptimal, ML.RowMajor])
def test_int8_128x128_bit_exact(layout):
    rng = np.random.default_rng(43)
    B, M, K = 2051, 128, 128
    x = rng.integers(-128, 128, (B, K), dtype=np.int8)
    W = rng.integers(-127, 128, (M, K), dtype=np.int8)
    b = rng.integers(-65536, 65537, M).astype(np.int32)
    want = ob.ref_matmul_i32(x, W.view(np.uint8).ravel(), ob.ROW, K, M, K, b)
    wb = to_dev(matrix_in_layout(W, CT.SignedInt8, layout))
    st = K if layout == ML.RowMajor else M
    y = cv.coopVecMatMulAdd(to_dev(x), CT.SignedInt8, wb, 0, CT.SignedInt8, as_bytes(to_dev(b)), 0,
                            CT.SignedInt32, layout, False, st, M=M)
    assert (y.cpu().numpy() == want).all()
    # the packed form reads the same bytes
    yp = cv.coopVecMatMulAddPacked(to_dev(x.view(np.int32)), CT.SignedInt8Packed, K, wb, 0, CT.SignedInt8,
                                   as_bytes(to_dev(b)), 0, CT.SignedInt32, layout, False, st, M=M)
    assert (yp.cpu().numpy() == want).all()
    # extreme values: every product at its maximum magnitude
    xe = np.full((16, K), -128, np.int8); We = np.full((M, K), -127, np.int8)
    ye = cv.coopVecMatMul(to_dev(xe), CT.SignedInt8, as_bytes(to_dev(We)), 0, CT.SignedInt8, ML.RowMajor, False, K, M=M)
    assert (ye.cpu().numpy() == 128 * 127 * K).all()


@pytest.mark.parametrize("M,K", [(4, 4), (16, 64), (3, 5), (128, 256), (100, 72), (64, 12)])
def test_int8_shapes(M, K):
    rng = np.random.default_rng(M + 7 * K)
    B = 100
    x = rng.integers(-128, 128, (B, K), dtype=np.int8)
    W = rng.integers(-127, 128, (M, K), dtype=np.int8)
    b = rng.integers(-65536, 65537, M).astype(np.int32)
    want = ob.ref_matmul_i32(x, W.view(np.uint8).ravel(), ob.ROW, K, M, K, b)
    for layout in (ML.RowMajor, ML.ColumnMajor, ML.InferencingOptimal):
        wb = to_dev(matrix_in_layout(W, CT.SignedInt8, layout))
        st = K if layout == ML.RowMajor else M
        y = cv.coopVecMatMulAdd(to_dev(x), CT.SignedInt8, wb, 0, CT.SignedInt8, as_bytes(to_dev(b)), 0,
                                CT.SignedInt32, layout, False, st, M=M)
        assert (y.cpu().numpy() == want).all()


# ---- e4m3 ---------------------------------------------------------------------------------

@pytest.mark.parametrize("M,K", [(64, 32), (64, 64), (8, 64), (16, 16), (128, 128), (24, 40)])
def test_e4m3_layers(M, K):
    rng = np.random.default_rng(44 + M + K)
    B = 1000
    x = ob.encode_e4m3(rng.standard_normal((B, K)) * 0.5)
    W = ob.encode_e4m3(rng.standard_normal((M, K)) * 0.5)
    b = rng.uniform(-0.1, 0.1, M).astype(np.float16)
    ref, ab = ob.ref_matmul_f32(x, ob.E4M3, W, ob.E4M3, ob.ROW, K, M, K, b, ob.F16)
    for layout in (ML.RowMajor, ML.InferencingOptimal):
        wb = to_dev(matrix_in_layout(W, CT.FloatE4M3, layout))
        # default: e4m3 decoded to fp16 operands, fp32-grade accumulation -> the common float bar
        y = cv.coopVecMatMulAdd(to_dev(x), CT.FloatE4M3, wb, 0, CT.FloatE4M3, as_bytes(to_dev(b)), 0, CT.Float16,
                                layout, False, K, M=M)
        assert not ob.float_parity_violations(y.cpu().numpy(), ref, ab).any()
        # fp8 matrix pipeline: the hardware keeps ~11 bits below the largest product of an
        # instruction, so the cancellation floor is 2^-12 * sum|terms| instead of 2^-18
        yn = cv.coopVecMatMulAdd(to_dev(x), CT.FloatE4M3, wb, 0, CT.FloatE4M3, as_bytes(to_dev(b)), 0, CT.Float16,
                                 layout, False, K, M=M, flags=cv.FLAG_FP8_MATRIX_PIPELINE)
        assert not ob.float_parity_violations(yn.cpu().numpy(), ref, ab * np.float32(2.0 ** 6)).any()
    # every e4m3 code is decoded as the oracle decodes it, on both pipelines: identity weights
    codes = np.array([c for c in range(256) if (c & 0x7f) != 0x7f], np.uint8)
    xin = np.zeros((len(codes), 16), np.uint8); xin[:, 0] = codes
    eye = ob.encode_e4m3(np.eye(16))
    for flags in (0, cv.FLAG_FP8_MATRIX_PIPELINE):
        y = cv.coopVecMatMul(to_dev(xin), CT.FloatE4M3, as_bytes(to_dev(eye)), 0, CT.FloatE4M3, ML.RowMajor, False, 16,
                             M=16, resultType=CT.Float32, flags=flags).cpu().numpy()
        assert (y[:, 0] == ob.decode_e4m3(codes)).all()


# ---- full-size configurations: size-independent properties ----------------------------------

def test_full_size_fp16_single_layer():
    # batch 2^22 of the 64x64 layer: sampled oracle check, layout equality, determinism
    torch.manual_seed(1234)
    B, M, K = 1 << 22, 64, 64
    x = torch.randn(B, K, device=DEV).half()
    rng = np.random.default_rng(1234)
    W = fp16_weights(rng, M, K); b = rng.uniform(-0.1, 0.1, M).astype(np.float16)
    wrow = as_bytes(to_dev(W)); bb = as_bytes(to_dev(b))
    wopt = to_dev(matrix_in_layout(W, CT.Float16, ML.InferencingOptimal))
    y1 = cv.coopVecMatMulAdd(x, CT.Float16, wrow, 0, CT.Float16, bb, 0, CT.Float16, ML.RowMajor, False, K * 2, M=M)
    y2 = cv.coopVecMatMulAdd(x, CT.Float16, wopt, 0, CT.Float16, bb, 0, CT.Float16, ML.InferencingOptimal, False, 0, M=M)
    y3 = cv.coopVecMatMulAdd(x, CT.Float16, wrow, 0, CT.Float16, bb, 0, CT.Float16, ML.RowMajor, False, K * 2, M=M)
    assert torch.equal(y1.view(torch.int16), y2.view(torch.int16))
    assert torch.equal(y1.view(torch.int16), y3.view(torch.int16))
    idx = torch.from_numpy(np.concatenate([rng.integers(0, B, 8192), [0, 1, B - 2, B - 1]])).to(DEV)
    xs = x[idx].cpu().numpy(); ys = y1[idx].cpu().numpy()
    ref, ab = ob.ref_matmul_f32(xs, ob.F16, W, ob.F16, ob.ROW, K * 2, M, K, b, ob.F16)
    assert not ob.float_parity_violations(ys, ref, ab).any()
    # linearity in the bias: y(b) - y(0) == b wherever no rounding interferes is not exact in fp16,
    # so use an exact one: doubling the inputs doubles the pre-bias result (power-of-two scaling)
    y0 = cv.coopVecMatMul(x[:65536], CT.Float16, wrow, 0, CT.Float16, ML.RowMajor, False, K * 2, M=M)
    y0x2 = cv.coopVecMatMul(x[:65536] * 2, CT.Float16, wrow, 0, CT.Float16, ML.RowMajor, False, K * 2, M=M)
    normal = y0.abs() >= 2.0 ** -13          # fp16 subnormals lose a bit that the doubled result keeps
    assert torch.equal((y0 * 2)[normal].view(torch.int16), y0x2[normal].view(torch.int16))
    assert normal.float().mean().item() > 0.999


def test_full_size_int8():
    # batch 2^22 of 128x128 int8: sampled oracle check + exact linearity W(x1+x2) = Wx1 + Wx2
    B, M, K = 1 << 22, 128, 128
    g = torch.Generator(device=DEV); g.manual_seed(99)
    x1 = torch.randint(-64, 64, (B, K), device=DEV, dtype=torch.int8, generator=g)
    x2 = torch.randint(-64, 64, (B, K), device=DEV, dtype=torch.int8, generator=g)
    rng = np.random.default_rng(99)
    W = rng.integers(-127, 128, (M, K), dtype=np.int8)
    b = rng.integers(-65536, 65537, M).astype(np.int32)
    wcol = to_dev(matrix_in_layout(W, CT.SignedInt8, ML.ColumnMajor))
    wopt = to_dev(matrix_in_layout(W, CT.SignedInt8, ML.InferencingOptimal))
    bb = as_bytes(to_dev(b))
    f = lambda x, w, layout, bias: (cv.coopVecMatMulAdd(x, CT.SignedInt8, w, 0, CT.SignedInt8, bb, 0, CT.SignedInt32,
                                                        layout, False, M, M=M) if bias else
                                    cv.coopVecMatMul(x, CT.SignedInt8, w, 0, CT.SignedInt8, layout, False, M, M=M))
    y1 = f(x1, wcol, ML.ColumnMajor, True)
    y1o = f(x1, wopt, ML.InferencingOptimal, True)
    assert torch.equal(y1, y1o)
    idx = torch.from_numpy(rng.integers(0, B, 4096)).to(DEV)
    want = ob.ref_matmul_i32(x1[idx].cpu().numpy(), W.view(np.uint8).ravel(), ob.ROW, K, M, K, b)
    assert (y1[idx].cpu().numpy() == want).all()
    del y1o
    s = f(x1 + x2, wopt, ML.InferencingOptimal, False)
    a = f(x1, wopt, ML.InferencingOptimal, False)
    a += f(x2, wopt, ML.InferencingOptimal, False)
    assert torch.equal(s, a)
