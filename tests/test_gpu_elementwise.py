"""GPU parity of the element-wise CoopVec surface (cvElementwise / cvElementwiseBackward) and of the
neural module's activations fused behind matMulAdd, through the C-ABI.

Bars: fp32 elements 1e-5 relative (+1e-6 absolute) against the oracle's double evaluation (the GPU's
transcendental functions are a few fp32 ulps wide); fp16 elements 2 ulp-fp16; the reference's own
CHECK values (tests/autodiff/coopvec.slang) to their printed precision; tie rules exact."""
import json
import os

import numpy as np
import pytest
import torch

import elementwise_tape as T
import oracle_binding as ob
from gpu_util import DEV, as_bytes, to_dev
from slang_amd import coopvec as cv
from slang_amd.coopvec import Activation, CoopVecComponentType as CT, CoopVecMatrixLayout as ML, FeedForwardLayer
from test_oracle_elementwise import CASES, G

pytestmark = pytest.mark.gpu


class GpuOps:
    def forward(self, op, a, b, c, param):
        return cv.elementwise(op, a, b, c, param=param)

    def backward(self, op, d_out, a, b, c, param):
        return cv.elementwiseBackward(op, d_out, a, b, c, param=param)


def make(dtype):
    def f(v):
        arr = np.full((1, 4), v, dtype) if np.isscalar(v) else np.array([v], dtype)
        return to_dev(arr)
    return f


@pytest.mark.parametrize("name", CASES)
def test_reference_goldens_on_gpu(name):
    case = G[name]
    primal, dx, dy, tangent = T.run_case(GpuOps(), name, case, make(np.float32))
    assert np.allclose(primal.cpu().numpy()[0], case["primal"], rtol=5e-6, atol=1e-6)
    for got, key in ((dx, "dx"), (dy, "dy"), (tangent, "tangent")):
        if key in case:
            assert np.allclose(got.cpu().numpy()[0], case[key], rtol=5e-6, atol=1e-6), (key, got)


def _operands(rng, op, B, N, dtype):
    x = rng.uniform(-3, 3, (B, N))
    y = rng.uniform(-3, 3, (B, N))
    z = rng.uniform(-3, 3, (B, N))
    if op in (T.LOG, T.LOG2):
        x = np.abs(x) + 0.05
    if op == T.DIV:
        y = np.where(np.abs(y) < 0.25, 0.25, y)
    if op == T.CLAMP:
        y, z = np.minimum(y, z) - 0.5, np.maximum(y, z) + 0.5
    if op in (T.MIN, T.MAX, T.STEP, T.RELU):
        x[::7] = y[::7]                       # ties
        if op == T.RELU:
            x[::5] = 0.0
    nops = T.N_OPERANDS.get(op, 1)
    ops = [x.astype(dtype), y.astype(dtype) if nops >= 2 else None, z.astype(dtype) if nops >= 3 else None]
    return ops


def _close(got, want, dtype):
    got = got.astype(np.float64); want = want.astype(np.float64)
    if dtype == np.float32:
        return np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-6
    return np.abs(got - want) <= 2.0 * ob.f16_ulp(want.astype(np.float32)) + 1e-7


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("shape", [(1000, 64), (333, 5)])
def test_every_operator_against_oracle(dtype, shape):
    rng = np.random.default_rng(11 + shape[1])
    B, N = shape
    for op in range(24):
        a, b, c = _operands(rng, op, B, N, dtype)
        da, db, dc = [to_dev(v) if v is not None else None for v in (a, b, c)]
        got = cv.elementwise(op, da, db, dc, param=0.1).cpu().numpy()
        want = ob.elementwise(op, a, b, c, 0.1)
        ok = _close(got, want, dtype)
        assert ok.all(), (op, dtype, got[~ok][:4], want[~ok][:4])
        g = rng.uniform(-2, 2, (B, N)).astype(dtype)
        grads = cv.elementwiseBackward(op, to_dev(g), da, db, dc, param=0.1)
        wants = ob.elementwise_backward(op, g, a, b, c, 0.1)
        for k, (gg, ww) in enumerate(zip(grads, wants)):
            if ww is None:
                assert gg is None
                continue
            ok = _close(gg.cpu().numpy(), ww, dtype)
            if dtype == np.float16:      # a product of two rounded factors: one more ulp
                ok |= np.abs(gg.cpu().numpy().astype(np.float64) - ww.astype(np.float64)) <= 3.0 * ob.f16_ulp(ww.astype(np.float32))
            assert ok.all(), (op, k, dtype)


def test_half_fma_is_rounded_once_and_scale_takes_a_scalar_of_the_element_type():
    # fma on half vectors: a*b = 1.5 + 1.5 ulp exactly (a tie of the half grid), c = -2^-24 pulls the exact sum below the
    # tie, so the correctly rounded result is the lower neighbour 0x3E01; a float fma lands on the tie (its own tie, to
    # even) and a second rounding to half would give 0x3E02
    a = np.full((3, 8), 1.0009765625, np.float16); b = np.full((3, 8), 1.5, np.float16)
    c = np.full((3, 8), -2.0 ** -24, np.float16)
    got = cv.elementwise(T.FMA, to_dev(a), to_dev(b), to_dev(c)).cpu().numpy()
    assert (got.view(np.uint16) == 0x3E01).all(), hex(int(got.view(np.uint16)[0, 0]))
    assert (ob.elementwise(T.FMA, a, b, c, 0.0).view(np.uint16) == 0x3E01).all()
    wide = cv.elementwise(T.FMA, to_dev(a[:, :5]), to_dev(b[:, :5]), to_dev(c[:, :5])).cpu().numpy()      # the strided kernel
    assert (wide.view(np.uint16) == 0x3E01).all()
    # vector * scalar (hlsl.meta.slang:32004): the scalar is converted to the element type first
    rng = np.random.default_rng(3)
    x = rng.uniform(-4, 4, (100, 16)).astype(np.float16)
    k = 0.3                                   # not a half: half(0.3) = 0.300048828125
    got = cv.elementwise(T.SCALE, to_dev(x), param=k).cpu().numpy()
    want = (x.astype(np.float32) * np.float32(np.float16(k))).astype(np.float16)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    g = rng.uniform(-1, 1, x.shape).astype(np.float16)
    da, _, _ = cv.elementwiseBackward(T.SCALE, to_dev(g), to_dev(x), param=k)
    assert np.array_equal(da.cpu().numpy().view(np.uint16), (g.astype(np.float32) * np.float32(np.float16(k))).astype(np.float16).view(np.uint16))
    xf = x.astype(np.float32)
    assert np.array_equal(cv.elementwise(T.SCALE, to_dev(xf), param=k).cpu().numpy(), xf * np.float32(k))


def test_strided_rows_and_in_place():
    rng = np.random.default_rng(5)
    B, N = 257, 24
    big = to_dev(rng.uniform(-2, 2, (B, 40)).astype(np.float32))
    a = big[:, 8:8 + N]                      # rows 160 bytes apart, 96 used
    out = torch.zeros(B, 48, dtype=torch.float32, device=DEV)
    cv.elementwise(T.TANH, a, out=out[:, :N])
    assert np.allclose(out[:, :N].cpu().numpy(), np.tanh(a.cpu().numpy().astype(np.float64)), rtol=1e-5, atol=1e-6)
    assert (out[:, N:] == 0).all()
    x = to_dev(rng.uniform(-2, 2, (B, N)).astype(np.float16))
    want = ob.elementwise(T.SILU, x.cpu().numpy())
    cv.elementwise(T.SILU, x, out=x)         # in place
    assert _close(x.cpu().numpy(), want, np.float16).all()


def test_elementwise_argument_validation():
    x = torch.zeros(4, 8, dtype=torch.float32, device=DEV)
    with pytest.raises(cv.CoopVecError) as e:
        cv.elementwise(99, x)
    assert e.value.result == cv.SLANG_E_INVALID_ARG
    with pytest.raises(cv.CoopVecError) as e:
        cv.elementwise(T.ADD, x)             # binary operator without b
    assert e.value.result == cv.SLANG_E_INVALID_ARG
    with pytest.raises(cv.CoopVecError) as e:
        cv.elementwise(T.TANH, x.to(torch.int32))     # integer vectors: arithmetic, min, max, clamp only
    assert e.value.result == cv.SLANG_E_NOT_AVAILABLE
    with pytest.raises(cv.CoopVecError) as e:
        cv.elementwiseBackward(T.NEG, x.to(torch.float64), x.to(torch.float64))
    assert e.value.result == cv.SLANG_E_NOT_AVAILABLE
    assert cv.elementwise(T.NEG, x[:0]).shape == (0, 8)


ACT_OF = {Activation.Sigmoid: T.SIGMOID, Activation.Tanh: T.TANH, Activation.Exp: T.EXP, Activation.Sine: T.SIN,
          Activation.SiLU: T.SILU, Activation.QuickGELU: T.QUICK_GELU}


@pytest.mark.parametrize("act", list(ACT_OF))
def test_activation_fused_behind_matmul_add(act):
    # out = act(half(W x + b)): the activation sees the fp16 carrier, as FFLayer.eval applies
    # IActivation.eval to the layer's output vector (layers.slang:90-110)
    rng = np.random.default_rng(int(act))
    B, M, K = 2000, 48, 40
    x = rng.uniform(-1, 1, (B, K)).astype(np.float16)
    W = (rng.standard_normal((M, K)) / np.sqrt(K)).astype(np.float16)
    b = rng.uniform(-0.5, 0.5, M).astype(np.float16)
    y = cv.coopVecMatMulAdd(to_dev(x), CT.Float16, as_bytes(to_dev(W)), 0, CT.Float16, as_bytes(to_dev(b)), 0, CT.Float16,
                            ML.RowMajor, False, K * 2, M=M, activation=act).cpu().numpy()
    z = cv.coopVecMatMulAdd(to_dev(x), CT.Float16, as_bytes(to_dev(W)), 0, CT.Float16, as_bytes(to_dev(b)), 0, CT.Float16,
                            ML.RowMajor, False, K * 2, M=M).cpu().numpy()
    want = ob.elementwise(ACT_OF[act], z)
    assert _close(y, want, np.float16).all()
    # fp32 result type
    y32 = cv.coopVecMatMulAdd(to_dev(x), CT.Float16, as_bytes(to_dev(W)), 0, CT.Float16, as_bytes(to_dev(b)), 0, CT.Float16,
                              ML.RowMajor, False, K * 2, M=M, activation=act, resultType=CT.Float32).cpu().numpy()
    z32 = cv.coopVecMatMulAdd(to_dev(x), CT.Float16, as_bytes(to_dev(W)), 0, CT.Float16, as_bytes(to_dev(b)), 0, CT.Float16,
                              ML.RowMajor, False, K * 2, M=M, resultType=CT.Float32).cpu().numpy()
    assert _close(y32, ob.elementwise(ACT_OF[act], z32), np.float32).all()


def test_mlp_with_smooth_activations_equals_layer_chain():
    # tanh / SiLU hidden layers, sigmoid output: the fused forward equals the chain of single layers
    rng = np.random.default_rng(21)
    dims = [12, 64, 40, 3]
    acts = [Activation.Tanh, Activation.SiLU, Activation.Sigmoid]
    layers, h = [], None
    B = 1500
    x = to_dev(rng.uniform(-1, 1, (B, dims[0])).astype(np.float16))
    h = x
    for i, act in enumerate(acts):
        fi, fo = dims[i], dims[i + 1]
        W = (rng.standard_normal((fo, fi)) / np.sqrt(fi)).astype(np.float16)
        b = rng.uniform(-0.2, 0.2, fo).astype(np.float16)
        wb, bb = as_bytes(to_dev(W)), as_bytes(to_dev(b))
        layers.append(FeedForwardLayer(fi, fo, wb, bb, ML.RowMajor, fi * 2, act, 0.0))
        h = cv.coopVecMatMulAdd(h, CT.Float16, wb, 0, CT.Float16, bb, 0, CT.Float16, ML.RowMajor, False, fi * 2, M=fo,
                                activation=act)
    y = cv.mlpForward(layers, x)
    assert torch.equal(y.view(torch.int16), h.view(torch.int16))
    assert ((y > 0) & (y < 1)).all()
    with pytest.raises(cv.CoopVecError) as e:        # no derivative of these inside the fused training step
        for L in layers:
            L.weightsGrad = torch.zeros(L.inputSize * L.outputSize * 4, dtype=torch.uint8, device=DEV)
            L.biasesGrad = torch.zeros(L.outputSize * 4, dtype=torch.uint8, device=DEV)
            L.gradLayout = ML.RowMajor
        cv.mlpTrainStepWorkspaceSize(layers, B) and cv.mlpTrainStep(layers, x, None)
    assert e.value.result == cv.SLANG_E_NOT_AVAILABLE


# ---------------------------------------------------------------------------------------------
# integer and fp64 vectors; conversions between element types
# ---------------------------------------------------------------------------------------------

INT_TYPES = [np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64]


def _torch_dtype(np_dtype):
    return {np.dtype(np.int8): torch.int8, np.dtype(np.uint8): torch.uint8, np.dtype(np.int16): torch.int16,
            np.dtype(np.uint16): torch.uint16, np.dtype(np.int32): torch.int32, np.dtype(np.uint32): torch.uint32,
            np.dtype(np.int64): torch.int64, np.dtype(np.uint64): torch.uint64, np.dtype(np.float16): torch.float16,
            np.dtype(np.float32): torch.float32, np.dtype(np.float64): torch.float64}[np.dtype(np_dtype)]


def _dev_typed(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(a.shape[0], -1)).to(DEV).view(_torch_dtype(a.dtype))


def _wrap(v, dtype):
    info = np.iinfo(dtype)
    span = int(info.max) - int(info.min) + 1
    return (v - int(info.min)) % span + int(info.min)


def _int_ref(op, a, b, c, dtype):
    """The operator on Python integers (unbounded), wrapped to the element type: independent of any machine arithmetic."""
    info = np.iinfo(dtype)
    out = np.empty(a.shape, dtype)
    for idx in np.ndindex(a.shape):
        x, y, z = int(a[idx]), int(b[idx]), int(c[idx])
        if op == T.ADD: v = x + y
        elif op == T.SUB: v = x - y
        elif op == T.MUL: v = x * y
        elif op == T.DIV:
            # C's quotient (towards zero); x / 0 = 0 by this library's definition, MIN / -1 wraps to MIN
            v = 0 if y == 0 else (abs(x) // abs(y)) * (1 if (x < 0) == (y < 0) else -1)
        elif op == T.NEG: v = -x
        elif op == T.MIN: v = min(x, y)
        elif op == T.MAX: v = max(x, y)
        elif op == T.CLAMP: v = min(max(x, y), z)
        out[idx] = _wrap(v, dtype)
    return out


@pytest.mark.parametrize("dtype", INT_TYPES)
def test_integer_vectors_bit_exact(dtype):
    # Slang declares arithmetic, min, max and clamp on CoopVec<integer, N> (slang-ir-lower-coopvec.cpp:188-192,
    # hlsl.meta.slang:32115-32229): two's complement, wrapping
    rng = np.random.default_rng(np.dtype(dtype).itemsize * 2 + (np.dtype(dtype).kind == "u"))
    info = np.iinfo(dtype)
    B, N = 37, 11
    def draw():
        v = rng.integers(info.min, info.max, (B, N), dtype=dtype, endpoint=True)
        small = rng.random((B, N)) < 0.3
        v[small] = rng.integers(max(info.min, -3), 4, int(small.sum()), dtype=dtype)     # small values, zeros, -1
        return v
    a, b, c = draw(), draw(), draw()
    a[0, :3] = info.min; b[0, 0] = dtype(-1) if info.min < 0 else dtype(1); b[0, 1] = 0
    for op in (T.ADD, T.SUB, T.MUL, T.DIV, T.NEG, T.MIN, T.MAX, T.CLAMP):
        lo, hi = (np.minimum(b, c), np.maximum(b, c)) if op == T.CLAMP else (b, c)
        got = cv.elementwise(op, _dev_typed(a), _dev_typed(lo), _dev_typed(hi)).cpu().numpy().view(dtype)
        assert cv.lastKernelName().startswith("elementwiseArithKernel"), cv.lastKernelName()
        assert np.array_equal(got, _int_ref(op, a, lo, hi, dtype)), op


def test_fp64_vectors():
    rng = np.random.default_rng(64)
    a, b, c = (rng.standard_normal((50, 9)) for _ in range(3))
    b[0, 0] = a[0, 0]
    lo, hi = np.minimum(b, c), np.maximum(b, c)
    ops = {T.ADD: a + b, T.SUB: a - b, T.MUL: a * b, T.DIV: a / b, T.NEG: -a, T.MIN: np.minimum(a, b), T.MAX: np.maximum(a, b),
           T.STEP: (b >= a).astype(np.float64)}
    for op, want in ops.items():
        got = cv.elementwise(op, _dev_typed(a), _dev_typed(b), _dev_typed(c)).cpu().numpy()
        assert np.array_equal(got, want), op          # IEEE operations: the same bits
    got = cv.elementwise(T.CLAMP, _dev_typed(a), _dev_typed(lo), _dev_typed(hi)).cpu().numpy()
    assert np.array_equal(got, np.clip(a, lo, hi))
    got = cv.elementwise(T.FMA, _dev_typed(a), _dev_typed(b), _dev_typed(c)).cpu().numpy()
    import math
    want = np.array([[math.fma(x, y, z) for x, y, z in zip(ra, rb, rc)] for ra, rb, rc in zip(a, b, c)]) if hasattr(math, "fma") else None
    if want is not None:
        assert np.array_equal(got, want)
    else:             # one rounding: within half an ulp of the exact value, which a*b + c in long double brackets
        exact = a.astype(np.longdouble) * b.astype(np.longdouble) + c.astype(np.longdouble)
        assert (np.abs(got.astype(np.longdouble) - exact) <= np.spacing(np.abs(got)) * 0.5 + np.abs(exact) * 2.0 ** -63).all()


ALL_TYPES = INT_TYPES + [np.float16, np.float32, np.float64]


@pytest.mark.parametrize("src", ALL_TYPES)
def test_copy_from_converts_between_all_plain_types(src):
    # CoopVec<T,N>(CoopVec<U,N>) (hlsl.meta.slang:30683-30730): numpy's astype is C's conversion for values the
    # target can hold (integers wrap, floats truncate towards zero, to float: one rounding to nearest even)
    rng = np.random.default_rng(np.dtype(src).itemsize + 10 * (np.dtype(src).kind == "f"))
    B, N = 61, 17
    if np.dtype(src).kind == "f":
        x = (rng.standard_normal((B, N)) * rng.choice([0.01, 1.0, 100.0], (B, N))).astype(src)
        x[0, :4] = [0.5, -0.5, 2.5, -3.99]
    else:
        info = np.iinfo(src)
        x = rng.integers(info.min, info.max, (B, N), dtype=src, endpoint=True)
        small = rng.random((B, N)) < 0.5
        x[small] = rng.integers(max(info.min, -100), 100, int(small.sum()), dtype=src)
    for dst in ALL_TYPES:
        xs = x
        if np.dtype(src).kind == "f" and np.dtype(dst).kind != "f":
            info = np.iinfo(dst)           # values the target holds; the rest is pinned by the next test
            xs = np.clip(x, max(info.min, -100), min(info.max, 100)).astype(src)
        with np.errstate(over="ignore"):
            want = xs.astype(dst)
        got = cv.copyFrom(_dev_typed(xs), {np.int8: CT.SignedInt8, np.uint8: CT.UnsignedInt8, np.int16: CT.SignedInt16,
                                           np.uint16: CT.UnsignedInt16, np.int32: CT.SignedInt32, np.uint32: CT.UnsignedInt32,
                                           np.int64: CT.SignedInt64, np.uint64: CT.UnsignedInt64, np.float16: CT.Float16,
                                           np.float32: CT.Float32, np.float64: CT.Float64}[dst])
        assert cv.lastKernelName().startswith("vectorCastKernel"), cv.lastKernelName()
        bits = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[np.dtype(dst).itemsize]
        assert np.array_equal(got.cpu().numpy().view(bits), want.view(bits)), (src, dst)


def test_copy_from_single_rounding_and_the_values_c_leaves_open():
    # double -> half in one rounding: 1 + 2^-11 + 2^-30 lies above the tie between 1 and 1 + 2^-10; rounding to
    # float first would land on the tie and then on 1
    x = np.array([[1.0 + 2.0 ** -11 + 2.0 ** -30, 1.0 + 2.0 ** -11, 65519.999, 65520.0, -1e300, 1e-8, 2.0 ** -25 * (1 + 1e-12)]], np.float64)
    got = cv.copyFrom(_dev_typed(x), CT.Float16).cpu().numpy()
    with np.errstate(over="ignore"):
        assert np.array_equal(got.view(np.uint16), x.astype(np.float16).view(np.uint16))
    assert got[0, 0] == np.float16(1.0 + 2.0 ** -10) and got[0, 1] == np.float16(1.0)
    # float -> integer outside the target: NaN -> 0, saturation at 32 bits (64 for 64-bit targets), then the low bits
    f = np.array([[np.nan, 1e20, -1e20, 300.7, -129.9, 4294967295.5]], np.float64)
    assert cv.copyFrom(_dev_typed(f), CT.SignedInt32).cpu().numpy().tolist() == [[0, 2 ** 31 - 1, -2 ** 31, 300, -129, 2 ** 31 - 1]]
    assert cv.copyFrom(_dev_typed(f), CT.UnsignedInt32).cpu().numpy().view(np.uint32).tolist() == [[0, 2 ** 32 - 1, 0, 300, 0, 2 ** 32 - 1]]
    assert cv.copyFrom(_dev_typed(f), CT.SignedInt8).cpu().numpy().tolist() == [[0, -1, 0, 44, 127, -1]]
    assert cv.copyFrom(_dev_typed(f), CT.SignedInt64).cpu().numpy().tolist() == [[0, 2 ** 63 - 1, -2 ** 63, 300, -129, 4294967295]]
    assert cv.copyFrom(_dev_typed(f), CT.UnsignedInt64).cpu().numpy().view(np.uint64).tolist() == [[0, 2 ** 64 - 1, 0, 300, 0, 4294967295]]
    # strided rows, and nothing written past a row
    src = torch.arange(5 * 12, dtype=torch.int32, device=DEV).reshape(5, 12)
    out = torch.full((5, 16), -1.0, dtype=torch.float32, device=DEV)
    cv.copyFrom(src[:, 2:9], CT.Float32, out=out[:, :7])
    assert torch.equal(out[:, :7], src[:, 2:9].to(torch.float32)) and (out[:, 7:] == -1).all()
    with pytest.raises(cv.CoopVecError) as e:
        cv.copyFrom(torch.zeros(2, 4, dtype=torch.uint8, device=DEV).view(torch.float8_e4m3fn), CT.Float32)
    assert e.value.result == cv.SLANG_E_NOT_AVAILABLE


def test_copy_from_bfloat16():
    # bfloat16 is the high half of binary32: to it, one rounding to nearest even of the exact source value; from it, exact
    rng = np.random.default_rng(16)
    x32 = (rng.standard_normal((50, 33)) * rng.choice([1e-3, 1.0, 1e4], (50, 33))).astype(np.float32)
    x32[0, :3] = [1.0 + 2.0 ** -8, 1.0 + 2.0 ** -8 + 2.0 ** -20, 3.3895314e38]           # a tie, just above it, near the top
    got = cv.copyFrom(to_dev(x32), CT.BFloat16)
    assert got.dtype == torch.bfloat16
    assert np.array_equal(got.view(torch.int16).cpu().numpy().view(np.uint16), ob.bf16_bits(x32))
    back = cv.copyFrom(got, CT.Float32).cpu().numpy()
    assert np.array_equal(back.view(np.uint32), ob.bf16_bits(x32).astype(np.uint32) << 16)
    # double -> bfloat16 in one rounding: above the tie by less than float resolves
    d = np.array([[1.0 + 2.0 ** -8 + 2.0 ** -40, 1.0 + 2.0 ** -8, -(1.0 + 3 * 2.0 ** -8 + 2.0 ** -45)]], np.float64)
    got = cv.copyFrom(_dev_typed(d), CT.BFloat16).float().cpu().numpy()
    assert got.tolist() == [[1.0 + 2.0 ** -7, 1.0, -(1.0 + 2.0 ** -6)]]
    # 64-bit integers beyond 2^53: (2^8 + 1) 2^55 is a tie of the 8 significant bits (-> 2^63, the even one), one more
    # rounds up -- a conversion through double alone would land on the tie
    big = np.array([[257 << 55, (257 << 55) + 1, 3 << 56]], np.uint64)
    got = cv.copyFrom(_dev_typed(big), CT.BFloat16).float().cpu().numpy().astype(np.float64)
    assert got.tolist() == [[float(1 << 63), float(129 << 56), float(3 << 56)]]
    ints = rng.integers(-70000, 70000, (20, 9), dtype=np.int32)
    got = cv.copyFrom(_dev_typed(ints), CT.BFloat16)
    assert np.array_equal(got.view(torch.int16).cpu().numpy().view(np.uint16), ob.bf16_bits(ints.astype(np.float32)))
    assert cv.copyFrom(got, CT.SignedInt32).cpu().numpy().tolist() == ob.bf16_to_f32(ob.bf16_bits(ints.astype(np.float32))).astype(np.int32).tolist()
