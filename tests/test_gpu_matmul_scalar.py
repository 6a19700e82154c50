"""GPU parity of coopVecMatMul[Add] for the combinations without a matrix instruction (16- and 32-bit
integers, mixed integer / float forms), which run as the scalar definition of the operator
(hlsl.meta.slang:32835-32912, :33043-33103) in matmulScalarKernel.

Integer results and fp32 results are compared bit for bit with the Slang fallback itself
(oracle: cvo_slang_matmul; for fp32 it multiplies and adds in the same order with the same roundings);
half results against the same operator evaluated in fp32 on operands cast to half, with the float bar."""
import numpy as np
import pytest
import torch

import oracle_binding as ob
from gpu_util import DEV, as_bytes, to_dev
from slang_amd import coopvec as cv
from slang_amd.coopvec import Activation, CoopVecMatrixLayout as ML

pytestmark = pytest.mark.gpu

NP = {ob.F16: np.float16, ob.F32: np.float32, ob.F64: np.float64, ob.S8: np.int8, ob.U8: np.uint8, ob.S16: np.int16,
      ob.U16: np.uint16, ob.S32: np.int32, ob.U32: np.uint32, ob.S64: np.int64, ob.U64: np.uint64}


def values(rng, ct, shape, small=False):
    if ct in (ob.F16, ob.F32, ob.F64):
        return (rng.standard_normal(shape) * (2.0 if small else 8.0)).astype(NP[ct])
    info = np.iinfo(NP[ct])
    lo, hi = (max(info.min, -6), min(info.max, 6)) if small else (info.min, info.max)
    return rng.integers(lo, hi, shape, dtype=NP[ct], endpoint=True)


def dev(a):
    t = torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(a.shape[0], -1)).to(DEV)
    dt = {np.dtype(np.float16): torch.float16, np.dtype(np.float32): torch.float32, np.dtype(np.int8): torch.int8,
          np.dtype(np.uint8): torch.uint8, np.dtype(np.int16): torch.int16, np.dtype(np.uint16): torch.uint16,
          np.dtype(np.int32): torch.int32, np.dtype(np.uint32): torch.uint32, np.dtype(np.int64): torch.int64,
          np.dtype(np.uint64): torch.uint64, np.dtype(np.float64): torch.float64}[a.dtype]
    return t.view(dt)


INT_CASES = [  # (input, matrix, bias, result)
    (ob.S16, ob.S16, ob.S32, ob.S32), (ob.U16, ob.S16, None, ob.S32), (ob.S32, ob.S32, ob.S32, ob.S32),
    (ob.U32, ob.U32, ob.U32, ob.U32), (ob.S8, ob.S16, ob.S16, ob.S32), (ob.S16, ob.U8, ob.S8, ob.U32),
    (ob.S32, ob.U16, None, ob.U32), (ob.U8, ob.S32, ob.U16, ob.S32),
    # 64-bit arms of the switch (hlsl.meta.slang:32873-32903): 64-bit matrices, vectors and results
    (ob.S64, ob.S64, ob.S64, ob.S64), (ob.U64, ob.U64, None, ob.U64), (ob.S16, ob.S64, ob.S32, ob.S64),
    (ob.S64, ob.S8, ob.U64, ob.S32), (ob.U32, ob.U64, ob.S16, ob.U32), (ob.S32, ob.S32, ob.S64, ob.S64),
]


@pytest.mark.parametrize("in_ct,w_ct,b_ct,r_ct", INT_CASES)
@pytest.mark.parametrize("layout", [ML.RowMajor, ML.ColumnMajor])
def test_integer_combinations_bit_exact(in_ct, w_ct, b_ct, r_ct, layout):
    # full-range operands: the sums wrap modulo 2^32 exactly as the reference's int32 / uint32 arithmetic does
    rng = np.random.default_rng(in_ct * 100 + w_ct * 10 + r_ct)
    B, k, M = 300, 37, 21
    x = values(rng, in_ct, (B, k)); W = values(rng, w_ct, (M, k))
    bias = values(rng, b_ct, (M,)) if b_ct is not None else None
    Wm = np.ascontiguousarray(W if layout == ML.RowMajor else W.T)
    stride = Wm.shape[1] * W.itemsize
    ref = ob.slang_matmul(x, in_ct, in_ct, k, r_ct, M, Wm.view(np.uint8).reshape(-1), w_ct, int(layout), stride,
                          bias, b_ct if b_ct is not None else -1)
    wd = as_bytes(to_dev(Wm))
    if bias is None:
        y = cv.coopVecMatMul(dev(x), in_ct, wd, 0, w_ct, layout, False, stride, M=M, resultType=r_ct)
    else:
        y = cv.coopVecMatMulAdd(dev(x), in_ct, wd, 0, w_ct, as_bytes(to_dev(bias)), 0, b_ct, layout, False, stride, M=M, resultType=r_ct)
    assert cv.lastKernelName().startswith("matmulScalarKernel"), cv.lastKernelName()
    got = y.cpu().numpy().view(NP[r_ct])
    assert np.array_equal(got, ref)


FLOAT_CASES = [  # (input, matrix, bias, result)
    (ob.F32, ob.S8, ob.F32, ob.F32), (ob.F32, ob.F16, None, ob.F32), (ob.F16, ob.F32, ob.F16, ob.F32),
    (ob.S16, ob.F32, ob.F32, ob.F32), (ob.F32, ob.S16, ob.S8, ob.F32), (ob.U8, ob.F16, ob.F16, ob.F32),
    (ob.F64, ob.F64, ob.F64, ob.F64), (ob.F32, ob.F64, None, ob.F64), (ob.S32, ob.F16, ob.F64, ob.F64),
    (ob.F64, ob.S64, ob.F32, ob.F32), (ob.S64, ob.F32, ob.S64, ob.F64),
]


@pytest.mark.parametrize("in_ct,w_ct,b_ct,r_ct", FLOAT_CASES)
def test_float_results_equal_the_scalar_definition(in_ct, w_ct, b_ct, r_ct):
    # T = float / double: every product and every sum rounded to T, j ascending, bias last: the same bits as the fallback
    rng = np.random.default_rng(in_ct * 100 + w_ct * 10 + 7)
    B, k, M = 257, 45, 19
    x = values(rng, in_ct, (B, k), small=True); W = values(rng, w_ct, (M, k), small=True)
    bias = values(rng, b_ct, (M,), small=True) if b_ct is not None else None
    stride = k * W.itemsize
    ref = ob.slang_matmul(x, in_ct, in_ct, k, r_ct, M, W.view(np.uint8).reshape(-1), w_ct, ob.ROW, stride, bias,
                          b_ct if b_ct is not None else -1)
    wd = as_bytes(to_dev(W))
    if bias is None:
        y = cv.coopVecMatMul(dev(x), in_ct, wd, 0, w_ct, ML.RowMajor, False, stride, M=M, resultType=r_ct)
    else:
        y = cv.coopVecMatMulAdd(dev(x), in_ct, wd, 0, w_ct, as_bytes(to_dev(bias)), 0, b_ct, ML.RowMajor, False, stride, M=M, resultType=r_ct)
    assert cv.lastKernelName().startswith("matmulScalarKernel"), cv.lastKernelName()
    bits = np.uint64 if r_ct == ob.F64 else np.uint32
    assert np.array_equal(y.cpu().numpy().view(bits), ref.view(bits))
    # and the definition itself: fp64 of the same operands agrees to fp32 accuracy
    z = x.astype(np.float64) @ W.astype(np.float64).T + (bias.astype(np.float64) if bias is not None else 0.0)
    terms = np.abs(x.astype(np.float64)) @ np.abs(W.astype(np.float64)).T + 1.0
    assert (np.abs(ref.astype(np.float64) - z) <= 2.0 ** (-48 if r_ct == ob.F64 and ob.F16 not in (in_ct, w_ct) else -20) * terms).all()


@pytest.mark.parametrize("in_ct,w_ct", [(ob.F32, ob.F32), (ob.F16, ob.S16), (ob.S32, ob.F16), (ob.F32, ob.U8)])
@pytest.mark.parametrize("act", [Activation.NoActivation, Activation.ReLU, Activation.LeakyReLU])
def test_half_results(in_ct, w_ct, act):
    # T = half: operands cast to half (nearest even), products and sums in fp32, one rounding of the result,
    # then the activation in half -- the rule of the matrix-pipeline kernels
    rng = np.random.default_rng(in_ct * 10 + w_ct + int(act))
    B, k, M = 200, 64, 24
    x = values(rng, in_ct, (B, k), small=True); W = values(rng, w_ct, (M, k), small=True)
    bias = (rng.standard_normal(M) * 0.5).astype(np.float16)
    xh = x.astype(np.float16).astype(np.float32); Wh = W.astype(np.float16).astype(np.float32)
    acc = np.zeros((B, M), np.float32)
    for j in range(k):
        acc = acc + (xh[:, j:j + 1] * Wh[:, j][None, :]).astype(np.float32)
    acc = acc + bias.astype(np.float32)[None, :]
    ref = acc.astype(np.float16)
    slope = np.float16(0.125)
    if act == Activation.ReLU:
        ref = np.maximum(ref, np.float16(0))
    elif act == Activation.LeakyReLU:
        ref = np.maximum(ref, (ref * slope).astype(np.float16))
    stride = k * W.itemsize
    y = cv.coopVecMatMulAdd(dev(x), in_ct, as_bytes(to_dev(W)), 0, w_ct, as_bytes(to_dev(bias)), 0, ob.F16, ML.RowMajor, False,
                            stride, M=M, resultType=ob.F16, activation=act, leakySlope=float(slope))
    assert cv.lastKernelName().startswith("matmulScalarKernel"), cv.lastKernelName()
    got = y.cpu().numpy()
    assert np.array_equal(got.view(np.uint16), ref.view(np.uint16))


def test_accumulate_forms_strides_and_row_blocks():
    # a = a + matMul(...) (hlsl.meta.slang:31510-31520) in int32; padded vector strides; more rows and a longer k
    # than one LDS block holds (rows are staged in blocks)
    rng = np.random.default_rng(5)
    B, k, M = 130, 700, 40           # 12288 / 700 = 17 rows per block -> 16
    x = values(rng, ob.S16, (B, k)); W = values(rng, ob.S16, (M, k))
    ref = ob.slang_matmul(x, ob.S16, ob.S16, k, ob.S32, M, W.view(np.uint8).reshape(-1), ob.S16, ob.ROW, 2 * k)
    xin = torch.zeros((B, k + 6), dtype=torch.int16, device=DEV); xin[:, :k] = dev(x)
    out = torch.full((B, M + 3), 1000, dtype=torch.int32, device=DEV)
    cv.coopVecMatMul(xin[:, :k], ob.S16, as_bytes(to_dev(W)), 0, ob.S16, ML.RowMajor, False, 2 * k, M=M, resultType=ob.S32,
                     out=out[:, :M], accumulate=True)
    assert "rows/block=16" in cv.lastKernelName(), cv.lastKernelName()
    got = out.cpu().numpy()
    assert np.array_equal(got[:, :M], ref + 1000)
    assert (got[:, M:] == 1000).all()


PACKED_CASES = [  # (packed kind, element type of the vector, matrix, bias, result)
    (ob.S8P, ob.U32, ob.S16, ob.S32, ob.S32), (ob.U8P, ob.S32, ob.U16, None, ob.U32), (ob.S8P, ob.S32, ob.S32, ob.S64, ob.S64),
    (ob.U8P, ob.U32, ob.F16, ob.F32, ob.F32), (ob.S8P, ob.U32, ob.F32, None, ob.F32), (ob.S8P, ob.U32, ob.F64, ob.F64, ob.F64),
    (ob.U8P, ob.U32, ob.S8, ob.S32, ob.S64), (ob.S8P, ob.S32, ob.U8, ob.F16, ob.F32),
]


@pytest.mark.parametrize("interp,in_ct,w_ct,b_ct,r_ct", PACKED_CASES)
def test_packed_vectors_against_every_matrix_type(interp, in_ct, w_ct, b_ct, r_ct):
    # coopVecMatMulPacked: four bytes per 32-bit element, sign-extended for both packed kinds
    # (hlsl.meta.slang:32844-32856), then the scalar definition in the result type: the same bits as the fallback
    rng = np.random.default_rng(interp * 1000 + w_ct * 10 + r_ct)
    B, k, M = 260, 44, 17
    x = rng.integers(0, 2 ** 32, (B, k // 4), dtype=np.uint64).astype(np.uint32).view(NP[in_ct])
    W = values(rng, w_ct, (M, k), small=w_ct in (ob.F16, ob.F32, ob.F64))
    bias = values(rng, b_ct, (M,), small=True) if b_ct is not None else None
    stride = k * W.itemsize
    ref = ob.slang_matmul(x, in_ct, interp, k, r_ct, M, W.view(np.uint8).reshape(-1), w_ct, ob.ROW, stride, bias,
                          b_ct if b_ct is not None else -1)
    wd = as_bytes(to_dev(W))
    if bias is None:
        y = cv.coopVecMatMulPacked(dev(x), interp, k, wd, 0, w_ct, ML.RowMajor, False, stride, M=M, resultType=r_ct)
    else:
        y = cv.coopVecMatMulAddPacked(dev(x), interp, k, wd, 0, w_ct, as_bytes(to_dev(bias)), 0, b_ct, ML.RowMajor, False,
                                      stride, M=M, resultType=r_ct)
    assert cv.lastKernelName().startswith("matmulScalarKernel"), cv.lastKernelName()
    bits = {2: np.uint16, 4: np.uint32, 8: np.uint64}[ref.itemsize]
    assert np.array_equal(y.cpu().numpy().view(bits), ref.view(bits))
    # and the unpacking itself: byte j of the vector is (x[j / 4] >> 8 (j % 4)) as a signed byte
    if r_ct in (ob.S32, ob.S64) and b_ct is None:
        xb = x.view(np.int8).astype(np.int64)
        assert np.array_equal(ref.astype(np.int64), (xb @ W.astype(np.int64).T).astype(NP[r_ct]).astype(np.int64))


@pytest.mark.parametrize("in_ct,interp,w_ct,r_ct", [(ob.F32, ob.F16, ob.F16, ob.F32), (ob.S16, ob.S8, ob.S16, ob.S32),
                                                    (ob.F16, ob.S16, ob.F32, ob.F32), (ob.U8, ob.F32, ob.S32, ob.S64)])
def test_plain_interpretation_of_another_type_changes_nothing(in_ct, interp, w_ct, r_ct):
    # the scalar definition casts the stored elements to the result type and never reads a plain
    # inputInterpretation (hlsl.meta.slang:32839-32843)
    rng = np.random.default_rng(in_ct * 100 + interp)
    B, k, M = 140, 30, 12
    x = values(rng, in_ct, (B, k), small=True); W = values(rng, w_ct, (M, k), small=True)
    stride = k * W.itemsize
    ref = ob.slang_matmul(x, in_ct, interp, k, r_ct, M, W.view(np.uint8).reshape(-1), w_ct, ob.ROW, stride)
    wd = as_bytes(to_dev(W))
    y = cv.coopVecMatMul(dev(x), interp, wd, 0, w_ct, ML.RowMajor, False, stride, M=M, resultType=r_ct)
    assert cv.lastKernelName().startswith("matmulScalarKernel"), cv.lastKernelName()
    same = cv.coopVecMatMul(dev(x), in_ct, wd, 0, w_ct, ML.RowMajor, False, stride, M=M, resultType=r_ct)
    bits = {4: np.uint32, 8: np.uint64}[ref.itemsize]
    assert np.array_equal(y.cpu().numpy().view(bits), ref.view(bits))
    if cv.lastKernelName().startswith("matmulScalarKernel"):
        assert torch.equal(y, same)


def test_what_stays_unavailable():
    x = torch.zeros((4, 8), dtype=torch.int16, device=DEV)
    W = torch.zeros(64, dtype=torch.int16, device=DEV).view(torch.uint8)
    with pytest.raises(cv.CoopVecError) as e:          # no Optimal layouts for 16-bit integers
        cv.coopVecMatMul(x, ob.S16, W, 0, ob.S16, ML.InferencingOptimal, False, 0, M=4, resultType=ob.S32)
    assert e.value.result == cv.SLANG_E_NOT_AVAILABLE
    with pytest.raises(cv.CoopVecError) as e:          # smooth activations: matrix-pipeline combinations only
        cv.coopVecMatMulAdd(x, ob.S16, W, 0, ob.S16, torch.zeros(8, dtype=torch.uint8, device=DEV), 0, ob.F16, ML.RowMajor, False, 16,
                            M=4, resultType=ob.F16, activation=Activation.Tanh)
    assert e.value.result == cv.SLANG_E_NOT_AVAILABLE
