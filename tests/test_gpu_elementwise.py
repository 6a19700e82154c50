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
    for op in range(23):
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
        cv.elementwise(T.NEG, x.to(torch.int32))
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
