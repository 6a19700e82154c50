"""GPU parity of the wider matMul surface, through the C-ABI: unsigned bytes (bit-exact against the
Slang fallback operator and the integer reference), fp16 vectors interpreted as e4m3, e5m2,
bfloat16, and shapes beyond 128 rows / 128 columns.

Float bars: fp16/fp32 results within max(2 ulp-fp16, 1e-3 relative, 2^-18 * sum|terms|) of the
fp32-accumulated oracle; bfloat16 results within max(2 ulp-bf16, 2^-18 * sum|terms|) (a bfloat16
ulp is 2^-7 relative, so the 1e-3 term cannot apply to that result type)."""
import numpy as np
import pytest
import torch

import oracle_binding as ob
from gpu_util import DEV, as_bytes, fp16_inputs, fp16_weights, matrix_in_layout, to_dev
from slang_amd import coopvec as cv
from slang_amd.coopvec import Activation, CoopVecComponentType as CT, CoopVecMatrixLayout as ML

pytestmark = pytest.mark.gpu


# ---- unsigned bytes ------------------------------------------------------------------------

def _bytes(rng, shape, ct):
    return (rng.integers(0, 256, shape, dtype=np.uint8) if ct == CT.UnsignedInt8
            else rng.integers(-128, 128, shape, dtype=np.int8))


@pytest.mark.parametrize("xct,wct", [(CT.UnsignedInt8, CT.UnsignedInt8), (CT.UnsignedInt8, CT.SignedInt8),
                                     (CT.SignedInt8, CT.UnsignedInt8)])
@pytest.mark.parametrize("M,K,B", [(128, 128, 2051), (64, 64, 515), (3, 5, 37), (100, 72, 260), (128, 256, 300),
                                   (16, 16, 64)])
def test_unsigned_bytes_bit_exact(xct, wct, M, K, B):
    rng = np.random.default_rng(1000 + M + 3 * K + int(xct) + 7 * int(wct))
    x = _bytes(rng, (B, K), xct)
    W = _bytes(rng, (M, K), wct)
    b = rng.integers(-65536, 65537, M).astype(np.int32)
    want = ob.ref_matmul_i32(x.view(np.uint8), W.view(np.uint8).ravel(), ob.ROW, K, M, K, b, x_ct=int(xct), w_ct=int(wct))
    for layout in (ML.RowMajor, ML.ColumnMajor, ML.InferencingOptimal):
        wb = to_dev(matrix_in_layout(W, wct, layout))
        st = K if layout == ML.RowMajor else M
        y = cv.coopVecMatMulAdd(to_dev(x), xct, wb, 0, wct, as_bytes(to_dev(b)), 0, CT.SignedInt32, layout, False, st, M=M)
        assert (y.cpu().numpy() == want).all(), (layout, cv.lastKernelName())
    # extremes: every product at its largest, 255 * 255 (or 255 * -128)
    xe = np.full((16, K), 255 if xct == CT.UnsignedInt8 else -128, np.int64)
    We = np.full((M, K), 255 if wct == CT.UnsignedInt8 else -128, np.int64)
    npx = np.uint8 if xct == CT.UnsignedInt8 else np.int8
    npw = np.uint8 if wct == CT.UnsignedInt8 else np.int8
    ye = cv.coopVecMatMul(to_dev(xe.astype(npx)), xct, as_bytes(to_dev(We.astype(npw))), 0, wct, ML.RowMajor, False, K, M=M)
    assert (ye.cpu().numpy() == int(xe[0, 0]) * int(We[0, 0]) * K).all()


def test_unsigned_bytes_against_the_slang_operator():
    # the Slang fallback itself, T = uint32 and T = int32 (hlsl.meta.slang:32893-32907), ReLU on uint is the identity
    rng = np.random.default_rng(77)
    B, M, K = 48, 24, 40
    x = rng.integers(0, 256, (B, K), dtype=np.uint8)
    W = rng.integers(0, 256, (M, K), dtype=np.uint8)
    bu = rng.integers(0, 1 << 20, M).astype(np.uint32)
    want = ob.slang_matmul(x, ob.U8, ob.U8, K, ob.U32, M, W.ravel(), ob.U8, ob.ROW, K, bu, ob.U32)
    y = cv.coopVecMatMulAdd(to_dev(x), CT.UnsignedInt8, as_bytes(to_dev(W)), 0, CT.UnsignedInt8, as_bytes(to_dev(bu.view(np.int32))), 0,
                            CT.UnsignedInt32, ML.RowMajor, False, K, M=M, resultType=CT.UnsignedInt32,
                            activation=Activation.ReLU)
    assert (y.view(torch.int32).cpu().numpy().view(np.uint32) == want).all()
    # the accumulate member form on unsigned bytes
    acc0 = rng.integers(-1000, 1000, (B, M)).astype(np.int32)
    acc = to_dev(acc0.copy())
    cv.coopVecMatMul(to_dev(x), CT.UnsignedInt8, as_bytes(to_dev(W)), 0, CT.UnsignedInt8, ML.RowMajor, False, K, M=M,
                     out=acc, accumulate=True)
    plain = ob.ref_matmul_i32(x, W.ravel(), ob.ROW, K, M, K, None, x_ct=ob.U8, w_ct=ob.U8)
    assert (acc.cpu().numpy() == acc0 + plain).all()


@pytest.mark.parametrize("interp", [CT.UnsignedInt8Packed, CT.SignedInt8Packed])
@pytest.mark.parametrize("wct", [CT.UnsignedInt8, CT.SignedInt8])
def test_packed_bytes_are_sign_extended_for_both_packed_kinds(interp, wct):
    # hlsl.meta.slang:32850-32855 unpacks through int8_t whatever the packed kind says
    rng = np.random.default_rng(5 + int(interp) + int(wct))
    B, M, K = 40, 32, 64
    xb = rng.integers(0, 256, (B, K), dtype=np.uint8)           # includes bytes >= 128
    x = xb.view(np.uint32)
    W = _bytes(rng, (M, K), wct)
    b = rng.integers(-65536, 65537, M).astype(np.int32)
    want = ob.slang_matmul(x, ob.U32, int(interp), K, ob.S32, M, W.view(np.uint8).ravel(), int(wct), ob.ROW, K, b, ob.S32)
    # independent statement of the same rule
    assert (want.astype(np.int64) == (xb.view(np.int8).astype(np.int64) @ W.astype(np.int64).T + b)).all()
    y = cv.coopVecMatMulAddPacked(to_dev(x.view(np.int32)), interp, K, as_bytes(to_dev(W)), 0, wct, as_bytes(to_dev(b)), 0,
                                  CT.SignedInt32, ML.RowMajor, False, K, M=M)
    assert (y.cpu().numpy() == want).all()


# ---- fp16 vectors interpreted as e4m3 --------------------------------------------------------

@pytest.mark.parametrize("M,K", [(64, 64), (128, 128), (24, 40), (64, 32)])
def test_fp16_vectors_interpreted_as_e4m3(M, K):
    rng = np.random.default_rng(90 + M + K)
    B = 1000
    xh = (rng.standard_normal((B, K)) * 0.7).astype(np.float16)
    xh[0, :8] = [1000.0, -1000.0, 448.0, 464.0, -480.0, 2.0 ** -10, 0.0, -0.0]      # saturation and tiny values
    xq = ob.encode_e4m3(xh.astype(np.float32))        # what the operator must see: the oracle's saturating quantiser
    W = ob.encode_e4m3(rng.standard_normal((M, K)) * 0.5)
    b = rng.uniform(-0.1, 0.1, M).astype(np.float16)
    ref, ab = ob.ref_matmul_f32(xq, ob.E4M3, W, ob.E4M3, ob.ROW, K, M, K, b, ob.F16)
    for layout in (ML.RowMajor, ML.InferencingOptimal):
        wb = to_dev(matrix_in_layout(W, CT.FloatE4M3, layout))
        y = cv.coopVecMatMulAdd(to_dev(xh), CT.FloatE4M3, wb, 0, CT.FloatE4M3, as_bytes(to_dev(b)), 0, CT.Float16,
                                layout, False, K, M=M)
        assert not ob.float_parity_violations(y.cpu().numpy(), ref, ab).any()
    # the quantisation itself, element by element: identity weights, fp32 result, every fp16 in a sweep
    sweep = np.arange(0, 65536, 7, dtype=np.uint16).view(np.float16)
    sweep = sweep[np.isfinite(sweep)]
    xin = np.zeros((len(sweep), 16), np.float16); xin[:, 0] = sweep
    eye = ob.encode_e4m3(np.eye(16))
    y = cv.coopVecMatMul(to_dev(xin), CT.FloatE4M3, as_bytes(to_dev(eye)), 0, CT.FloatE4M3, ML.RowMajor, False, 16,
                         M=16, resultType=CT.Float32).cpu().numpy()
    assert (y[:, 0] == ob.decode_e4m3(ob.encode_e4m3(sweep.astype(np.float32)))).all()


# ---- e5m2 ----------------------------------------------------------------------------------

def _e5m2_codes(rng, shape, max_exp=15):
    sign = rng.integers(0, 2, shape).astype(np.uint8) << 7
    exp = rng.integers(0, max_exp + 1, shape).astype(np.uint8) << 2
    man = rng.integers(0, 4, shape).astype(np.uint8)
    return (sign | exp | man).astype(np.uint8)


@pytest.mark.parametrize("M,K", [(64, 64), (128, 128), (24, 40), (16, 16)])
def test_e5m2(M, K):
    rng = np.random.default_rng(300 + M + K)
    B = 1000
    x = _e5m2_codes(rng, (B, K))
    W = _e5m2_codes(rng, (M, K), max_exp=13)
    b = rng.uniform(-0.1, 0.1, M).astype(np.float16)
    ref, ab = ob.ref_matmul_f32(x, ob.E5M2, W, ob.E5M2, ob.ROW, K, M, K, b, ob.F16)
    # the oracle's decoder against the definition (high byte of a binary16)
    ref0, _ = ob.ref_matmul_f32(x[:4], ob.E5M2, W, ob.E5M2, ob.ROW, K, M, K)
    assert np.allclose(ref0, ob.e5m2_to_f32(x[:4]) @ ob.e5m2_to_f32(W).T, rtol=1e-5, atol=1e-6)
    for layout in (ML.RowMajor, ML.ColumnMajor, ML.InferencingOptimal):
        wb = to_dev(matrix_in_layout(W, CT.FloatE5M2, layout))
        st = K if layout == ML.RowMajor else M
        y = cv.coopVecMatMulAdd(to_dev(x), CT.FloatE5M2, wb, 0, CT.FloatE5M2, as_bytes(to_dev(b)), 0, CT.Float16,
                                layout, False, st, M=M)
        assert not ob.float_parity_violations(y.cpu().numpy(), ref, ab).any()
    # every finite e5m2 code decodes exactly
    codes = np.array([c for c in range(256) if (c & 0x7c) != 0x7c], np.uint8)
    xin = np.zeros((len(codes), 16), np.uint8); xin[:, 0] = codes
    eye = np.where(np.eye(16) > 0, 0x3c, 0).astype(np.uint8)       # 1.0 in e5m2
    y = cv.coopVecMatMul(to_dev(xin), CT.FloatE5M2, as_bytes(to_dev(eye)), 0, CT.FloatE5M2, ML.RowMajor, False, 16,
                         M=16, resultType=CT.Float32).cpu().numpy()
    assert (y[:, 0] == ob.e5m2_to_f32(codes)).all()


# ---- bfloat16 --------------------------------------------------------------------------------

def _bf16_ulp(ref):
    e = np.floor(np.log2(np.maximum(np.abs(ref), 2.0 ** -126)))
    return np.exp2(e - 7).astype(np.float32)


def _bf16_tensor(bits):
    return to_dev(bits.view(np.int16)).view(torch.bfloat16)


@pytest.mark.parametrize("M,K", [(64, 64), (128, 128), (24, 40), (16, 32)])
def test_bfloat16(M, K):
    rng = np.random.default_rng(500 + M + K)
    B = 1000
    xb = ob.bf16_bits(rng.standard_normal((B, K)))
    Wb = ob.bf16_bits(rng.standard_normal((M, K)) / np.sqrt(K))
    bb = ob.bf16_bits(rng.uniform(-0.1, 0.1, M))
    ref, ab = ob.ref_matmul_f32(xb, ob.BF16, Wb.view(np.uint8).ravel(), ob.BF16, ob.ROW, 2 * K, M, K, bb, ob.BF16)
    # the oracle's bf16 decoding against the definition, in float64
    ref64 = ob.bf16_to_f32(xb[:8]).astype(np.float64) @ ob.bf16_to_f32(Wb).astype(np.float64).T + ob.bf16_to_f32(bb)
    assert np.allclose(ref[:8], ref64, rtol=1e-5, atol=1e-6)
    for layout in (ML.RowMajor, ML.ColumnMajor, ML.InferencingOptimal, ML.TrainingOptimal):
        wb = to_dev(matrix_in_layout(Wb, CT.BFloat16, layout))
        st = 2 * K if layout == ML.RowMajor else 2 * M
        y32 = cv.coopVecMatMulAdd(_bf16_tensor(xb), CT.BFloat16, wb, 0, CT.BFloat16, as_bytes(_bf16_tensor(bb)), 0,
                                  CT.BFloat16, layout, False, st, M=M, resultType=CT.Float32)
        assert not ob.float_parity_violations(y32.cpu().numpy(), ref, ab).any()
        y = cv.coopVecMatMulAdd(_bf16_tensor(xb), CT.BFloat16, wb, 0, CT.BFloat16, as_bytes(_bf16_tensor(bb)), 0,
                                CT.BFloat16, layout, False, st, M=M, activation=Activation.ReLU)
        got = y.float().cpu().numpy()
        want = np.maximum(ref, 0)
        tol = np.maximum(2 * _bf16_ulp(want), ab * np.float32(2.0 ** -18))
        assert (np.abs(got - want) <= tol).all()
        assert (got >= 0).all()


# ---- fp32 vectors against a Float32 matrix -----------------------------------------------------

@pytest.mark.parametrize("M,K", [(64, 64), (128, 128), (24, 40), (16, 32), (4, 4), (200, 300)])
def test_float32_matrix(M, K):
    rng = np.random.default_rng(600 + M + K)
    B = 500
    x = rng.standard_normal((B, K)).astype(np.float32)
    W = (rng.standard_normal((M, K)) / np.sqrt(K)).astype(np.float32)
    b = rng.uniform(-0.5, 0.5, M).astype(np.float32)
    ref, ab = ob.ref_matmul_f32(x, ob.F32, W.view(np.uint8).ravel(), ob.F32, ob.ROW, 4 * K, M, K, b, ob.F32)
    ref64 = x.astype(np.float64) @ W.astype(np.float64).T + b
    bound = (K + 1) * 2.0 ** -23 * ab            # fp32 products and sums, any order
    assert (np.abs(ref - ref64) <= bound).all()   # the oracle against the definition
    for layout in (ML.RowMajor, ML.ColumnMajor, ML.InferencingOptimal, ML.TrainingOptimal):
        wb = to_dev(matrix_in_layout(W, CT.Float32, layout))
        st = 4 * K if layout == ML.RowMajor else 4 * M
        y = cv.coopVecMatMulAdd(to_dev(x), CT.Float32, wb, 0, CT.Float32, as_bytes(to_dev(b)), 0, CT.Float32, layout,
                                False, st, M=M, resultType=CT.Float32)
        assert y.dtype == torch.float32 and "f32" in cv.lastKernelName()
        got = y.cpu().numpy()
        assert (np.abs(got - ref64) <= bound).all(), layout
        assert not ob.float_parity_violations(got, ref, ab).any()
    # transposed use (memory holds K x M), ReLU; then the bias-less operator
    wt = to_dev(matrix_in_layout(np.ascontiguousarray(W.T), CT.Float32, ML.InferencingOptimal))
    y = cv.coopVecMatMulAdd(to_dev(x), CT.Float32, wt, 0, CT.Float32, as_bytes(to_dev(b)), 0, CT.Float32,
                            ML.InferencingOptimal, True, 0, M=M, resultType=CT.Float32, activation=Activation.ReLU)
    assert (np.abs(y.cpu().numpy() - np.maximum(ref64, 0)) <= bound).all()
    y = cv.coopVecMatMul(to_dev(x), CT.Float32, wt, 0, CT.Float32, ML.InferencingOptimal, True, 0, M=M, resultType=CT.Float32)
    assert (np.abs(y.cpu().numpy() - (ref64 - b)) <= bound).all()


def test_float32_matrix_equals_the_slang_operator_on_exact_data():
    # small integers: every product and sum is exact in fp32, so any summation order gives the operator's result
    rng = np.random.default_rng(77)
    M, K, B = 20, 12, 64
    x = rng.integers(-8, 9, (B, K)).astype(np.float32)
    W = rng.integers(-8, 9, (M, K)).astype(np.float32)
    b = rng.integers(-100, 100, M).astype(np.float32)
    want = ob.slang_matmul(x, ob.F32, ob.F32, K, ob.F32, M, W.view(np.uint8).ravel(), ob.F32, ob.ROW, 4 * K, b, ob.F32)
    assert np.array_equal(want, x @ W.T + b)
    y = cv.coopVecMatMulAdd(to_dev(x), CT.Float32, to_dev(W.view(np.uint8).ravel()), 0, CT.Float32, as_bytes(to_dev(b)), 0,
                            CT.Float32, ML.RowMajor, False, 4 * K, M=M, resultType=CT.Float32)
    assert np.array_equal(y.cpu().numpy(), want)
    # on the matrix pipeline a Float32 matrix takes fp32 vectors only; fp16 vectors against it run as the scalar
    # definition (exact data: the same result)
    y = cv.coopVecMatMul(to_dev(x.astype(np.float16)), CT.Float16, to_dev(W.view(np.uint8).ravel()), 0, CT.Float32,
                         ML.RowMajor, False, 4 * K, M=M, resultType=CT.Float32)
    assert cv.lastKernelName().startswith("matmulScalarKernel"), cv.lastKernelName()
    assert np.array_equal(y.cpu().numpy(), x @ W.T)


# ---- beyond 128 rows / 128 columns --------------------------------------------------------------

@pytest.mark.parametrize("M,K", [(256, 64), (200, 128), (64, 256), (128, 512), (300, 200), (16, 1024), (520, 72)])
def test_fp16_large_shapes(M, K):
    rng = np.random.default_rng(700 + M + K)
    B = 333
    x = fp16_inputs(rng, B, K)
    W = fp16_weights(rng, M, K)
    b = rng.uniform(-0.5, 0.5, M).astype(np.float16)
    ref, ab = ob.ref_matmul_f32(x, ob.F16, W.view(np.uint8).ravel(), ob.F16, ob.ROW, 2 * K, M, K, b, ob.F16)
    for layout in (ML.RowMajor, ML.ColumnMajor, ML.InferencingOptimal, ML.TrainingOptimal):
        wb = to_dev(matrix_in_layout(W, CT.Float16, layout))
        st = 2 * K if layout == ML.RowMajor else 2 * M
        y = cv.coopVecMatMulAdd(to_dev(x), CT.Float16, wb, 0, CT.Float16, as_bytes(to_dev(b)), 0, CT.Float16, layout,
                                False, st, M=M)
        assert not ob.float_parity_violations(y.cpu().numpy(), ref, ab).any(), (layout, cv.lastKernelName())
    # transposed use of an optimal-layout matrix: memory holds K x M
    wt = to_dev(matrix_in_layout(np.ascontiguousarray(W.T), CT.Float16, ML.InferencingOptimal))
    y = cv.coopVecMatMulAdd(to_dev(x), CT.Float16, wt, 0, CT.Float16, as_bytes(to_dev(b)), 0, CT.Float16,
                            ML.InferencingOptimal, True, 0, M=M)
    assert not ob.float_parity_violations(y.cpu().numpy(), ref, ab).any()


@pytest.mark.parametrize("M,K", [(256, 128), (128, 512), (130, 700)])
def test_int8_large_shapes_bit_exact(M, K):
    rng = np.random.default_rng(800 + M + K)
    B = 200
    for xct, wct in ((CT.SignedInt8, CT.SignedInt8), (CT.UnsignedInt8, CT.UnsignedInt8)):
        x = _bytes(rng, (B, K), xct)
        W = _bytes(rng, (M, K), wct)
        b = rng.integers(-65536, 65537, M).astype(np.int32)
        want = ob.ref_matmul_i32(x.view(np.uint8), W.view(np.uint8).ravel(), ob.ROW, K, M, K, b, x_ct=int(xct), w_ct=int(wct))
        for layout in (ML.RowMajor, ML.InferencingOptimal):
            wb = to_dev(matrix_in_layout(W, wct, layout))
            y = cv.coopVecMatMulAdd(to_dev(x), xct, wb, 0, wct, as_bytes(to_dev(b)), 0, CT.SignedInt32, layout, False, K, M=M)
            assert (y.cpu().numpy() == want).all(), (xct, layout, cv.lastKernelName())


def test_e4m3_large_shape_and_limit():
    rng = np.random.default_rng(900)
    B, M, K = 200, 160, 384
    x = ob.encode_e4m3(rng.standard_normal((B, K)) * 0.5)
    W = ob.encode_e4m3(rng.standard_normal((M, K)) * 0.5)
    ref, ab = ob.ref_matmul_f32(x, ob.E4M3, W, ob.E4M3, ob.ROW, K, M, K)
    y = cv.coopVecMatMul(to_dev(x), CT.FloatE4M3, as_bytes(to_dev(W)), 0, CT.FloatE4M3, ML.RowMajor, False, K, M=M)
    assert not ob.float_parity_violations(y.cpu().numpy(), ref, ab).any()
    # k beyond what one 16-row block can keep in LDS answers NOT_AVAILABLE, never a wrong result
    K2 = 4096 + 32
    with pytest.raises(cv.CoopVecError) as e:
        cv.coopVecMatMul(torch.zeros((4, K2), dtype=torch.float16, device=DEV), CT.Float16,
                         torch.zeros(16 * K2 * 2, dtype=torch.uint8, device=DEV), 0, CT.Float16, ML.RowMajor, False, 2 * K2, M=16)
    assert e.value.result == cv.SLANG_E_NOT_AVAILABLE
    # fp32: the widest k (2048) works, one more k-tile does not
    K3, M3 = 2048, 20
    x3 = rng.standard_normal((50, K3)).astype(np.float32)
    W3 = (rng.standard_normal((M3, K3)) / np.sqrt(K3)).astype(np.float32)
    y3 = cv.coopVecMatMul(to_dev(x3), CT.Float32, as_bytes(to_dev(W3)), 0, CT.Float32, ML.RowMajor, False, 4 * K3, M=M3,
                          resultType=CT.Float32)
    want3 = x3.astype(np.float64) @ W3.astype(np.float64).T
    ab3 = np.abs(x3).astype(np.float64) @ np.abs(W3).astype(np.float64).T
    assert (np.abs(y3.cpu().numpy() - want3) <= (K3 + 1) * 2.0 ** -23 * ab3).all()
    with pytest.raises(cv.CoopVecError) as e:
        cv.coopVecMatMul(torch.zeros((4, K3 + 16), dtype=torch.float32, device=DEV), CT.Float32,
                         torch.zeros(16 * (K3 + 16) * 4, dtype=torch.uint8, device=DEV), 0, CT.Float32, ML.RowMajor, False,
                         4 * (K3 + 16), M=16, resultType=CT.Float32)
    assert e.value.result == cv.SLANG_E_NOT_AVAILABLE


def test_non_finite_inputs_stay_within_their_sample():
    # every sample is a column of the matrix-core product: an Inf or NaN element changes that sample's
    # outputs only, and there it yields what the scalar definition yields (w * Inf, 0 * Inf = NaN, NaN)
    rng = np.random.default_rng(12)
    B, M, K = 300, 48, 64
    x = fp16_inputs(rng, B, K)
    W = fp16_weights(rng, M, K)
    W[7, 3] = 0.0                                           # 0 * Inf
    clean = cv.coopVecMatMul(to_dev(x), CT.Float16, as_bytes(to_dev(W)), 0, CT.Float16, ML.RowMajor, False, 2 * K, M=M,
                             resultType=CT.Float32).cpu().numpy()
    xb = x.copy()
    xb[5, 3] = np.inf
    xb[9, 0] = np.nan
    xb[200, 63] = -np.inf
    got = cv.coopVecMatMul(to_dev(xb), CT.Float16, as_bytes(to_dev(W)), 0, CT.Float16, ML.RowMajor, False, 2 * K, M=M,
                           resultType=CT.Float32).cpu().numpy()
    touched = np.zeros(B, bool); touched[[5, 9, 200]] = True
    assert np.array_equal(got[~touched], clean[~touched])
    with np.errstate(invalid="ignore", over="ignore"):
        want = xb[touched].astype(np.float32) @ W.astype(np.float32).T
    assert np.array_equal(np.isnan(got[touched]), np.isnan(want))
    assert np.array_equal(got[touched][~np.isnan(want)], want[~np.isnan(want)])      # +-inf where the definition says so


def test_query_lists_what_matmul_accepts():
    combos = cv.querySupportedCombinations()
    keys = {(c["inputType"], c["inputInterpretation"], c["matrixInterpretation"], c["resultType"]) for c in combos}
    for want in [(CT.UnsignedInt8, CT.UnsignedInt8, CT.UnsignedInt8, CT.UnsignedInt32),
                 (CT.UnsignedInt32, CT.UnsignedInt8Packed, CT.SignedInt8, CT.SignedInt32),
                 (CT.Float16, CT.FloatE4M3, CT.FloatE4M3, CT.Float16),
                 (CT.FloatE5M2, CT.FloatE5M2, CT.FloatE5M2, CT.Float16),
                 (CT.BFloat16, CT.BFloat16, CT.BFloat16, CT.BFloat16),
                 (CT.Float32, CT.Float32, CT.Float32, CT.Float32)]:
        assert tuple(int(v) for v in want) in keys


def test_float32_blocks_in_registers_and_in_lds():
    # Up to 64 rows and 64 columns an fp32 block stays in registers (the kernels of the 16-bit types, their streaming form
    # for whole aligned vectors); anything larger is staged in LDS.  Large and ragged batches, padded vector rows, `+=`.
    rng = np.random.default_rng(4242)
    for M, K, B, pad in ((64, 64, 70001, 0), (64, 32, 4096, 0), (8, 64, 1000, 4), (33, 17, 999, 0), (64, 64, 513, 3), (128, 64, 2000, 0),
                         (64, 128, 2000, 0)):
        x = rng.standard_normal((B, K)).astype(np.float32)
        W = (rng.standard_normal((M, K)) / np.sqrt(K)).astype(np.float32)
        b = rng.uniform(-0.5, 0.5, M).astype(np.float32)
        ref64 = x.astype(np.float64) @ W.astype(np.float64).T + b
        mag = np.abs(x.astype(np.float64)) @ np.abs(W.astype(np.float64)).T + np.abs(b)
        bound = (K + 1) * 2.0 ** -23 * mag
        wide = torch.zeros((B, K + pad), dtype=torch.float32, device=DEV); wide[:, :K] = to_dev(x)
        y = cv.coopVecMatMulAdd(wide[:, :K], CT.Float32, as_bytes(to_dev(W)), 0, CT.Float32, as_bytes(to_dev(b)), 0, CT.Float32,
                                ML.RowMajor, False, 4 * K, M=M, resultType=CT.Float32)
        name = cv.lastKernelName()
        assert name.startswith("matmulKernel<f32" if M <= 64 and K <= 64 else "matmulLargeKernel<f32"), (M, K, name)
        if (M, K, pad) == (64, 64, 0):
            assert "streaming" in name, name
        assert (np.abs(y.cpu().numpy() - ref64) <= bound).all(), (M, K, B)
        # the member form: this += W x (no bias)
        acc0 = rng.standard_normal((B, M)).astype(np.float32)
        out = to_dev(acc0)
        cv.coopVecMatMul(wide[:, :K], CT.Float32, as_bytes(to_dev(W)), 0, CT.Float32, ML.RowMajor, False, 4 * K, M=M,
                         resultType=CT.Float32, out=out, accumulate=True)
        want = acc0.astype(np.float64) + (ref64 - b)
        assert (np.abs(out.cpu().numpy() - want) <= bound + 2.0 ** -23 * np.abs(want)).all(), (M, K, B, "accumulate")
