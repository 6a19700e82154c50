"""The fused training step whose waves share a tile of samples by kind of work (CV_FLAG_TRAIN_SPLIT_BY_ROLE), through the
C-ABI: against the fp64-accumulating CPU oracle to the bar of the default kernels (per layer ||dW - dW_ref||_F <= 1e-3
||dW_ref||_F, same for db and the loss), against the default kernels (same rounding points: the fp32 sums differ in their
order only), and run to run bit for bit."""
import numpy as np
import pytest
import torch

import oracle_binding as ob
from gpu_util import to_dev
from slang_amd import coopvec as cv
from slang_amd.coopvec import Activation, CoopVecComponentType as CT, CoopVecMatrixLayout as ML
from test_gpu_train import build, make_specs, read_grads, rel_err

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dims,B,targets", [([8, 64, 64, 64, 64, 1], 16384 + 21, True), ([8, 64, 64, 64, 64, 1], 40000, False),
                                            ([16, 64, 5], 16384, True), ([6, 64, 64, 16], 20001, True),
                                            ([12, 64, 64, 64, 3], 17000, False)])
def test_role_split_kernel_against_oracle_and_default_kernels(dims, B, targets):
    rng = np.random.default_rng(sum(dims) + B)
    specs = make_specs(rng, dims)
    x = rng.uniform(-1, 1, (B, dims[0])).astype(np.float16)
    t = None
    if targets:
        t = np.ascontiguousarray(np.sin(x.astype(np.float32).sum(1, keepdims=True)).astype(np.float16).repeat(dims[-1], 1))
    layers = build(specs)
    lmax = torch.zeros(1, dtype=torch.float32, device="cuda")
    _, loss = cv.mlpTrainStep(layers, to_dev(x), to_dev(t) if targets else None, lossMax=lmax, flags=cv.FLAG_TRAIN_SPLIT_BY_ROLE)
    assert cv.lastKernelName().startswith("mlpTrainTeamKernel"), cv.lastKernelName()
    dW, dB = read_grads(layers, specs, CT.Float32, ML.RowMajor)
    other = build(specs)
    lmax2 = torch.zeros(1, dtype=torch.float32, device="cuda")
    _, loss2 = cv.mlpTrainStep(other, to_dev(x), to_dev(t) if targets else None, lossMax=lmax2)
    assert cv.lastKernelName().startswith(("mlpTrainPairKernel", "mlpTrainKernel")), cv.lastKernelName()
    oW, oB = read_grads(other, specs, CT.Float32, ML.RowMajor)
    for l in range(len(specs)):
        assert rel_err(dW[l], oW[l]) <= 1e-3 and rel_err(dB[l], oB[l]) <= 1e-3, l
    assert abs(loss.item() - loss2.item()) <= 1e-4 * abs(loss2.item())
    assert lmax.item() == lmax2.item()
    rW, rB, rloss = ob.ref_mlp_train(specs, x, t, 1.0, tie_rule=True)
    for l in range(len(specs)):
        assert rel_err(dW[l], rW[l]) <= 1e-3, (l, rel_err(dW[l], rW[l]))
        assert rel_err(dB[l], rB[l]) <= 1e-3, (l, rel_err(dB[l], rB[l]))
    assert abs(loss.item() - rloss) <= 1e-3 * rloss
    again = build(specs)
    cv.mlpTrainStep(again, to_dev(x), to_dev(t) if targets else None, flags=cv.FLAG_TRAIN_SPLIT_BY_ROLE)
    for a, b in zip(layers, again):
        assert torch.equal(a.weightsGrad, b.weightsGrad) and torch.equal(a.biasesGrad, b.biasesGrad)


def test_role_split_flag_falls_back_where_the_kernel_does_not_apply():
    # small batches, other widths, leaky ReLU: the flag changes nothing
    rng = np.random.default_rng(5)
    for dims, B, act in (([8, 64, 64, 1], 1000, Activation.ReLU), ([8, 32, 32, 4], 20000, Activation.ReLU),
                         ([8, 64, 64, 1], 20000, Activation.LeakyReLU)):
        specs = make_specs(rng, dims, act=act, slope=0.25 if act == Activation.LeakyReLU else 0.0)
        x = rng.uniform(-1, 1, (B, dims[0])).astype(np.float16)
        a, b = build(specs), build(specs)
        cv.mlpTrainStep(a, to_dev(x), None, flags=cv.FLAG_TRAIN_SPLIT_BY_ROLE)
        assert not cv.lastKernelName().startswith("mlpTrainTeamKernel"), cv.lastKernelName()
        cv.mlpTrainStep(b, to_dev(x), None)
        for p, q in zip(a, b):
            assert torch.equal(p.weightsGrad, q.weightsGrad) and torch.equal(p.biasesGrad, q.biasesGrad)


def test_role_split_kernel_tie_rule():
    # Pre-activations of exactly +0, negative and positive values: max() sends half the gradient at a tie
    # (diff.meta.slang:2258-2277).  Sparse weights of -1, 0, 1 and a power-of-two loss scale keep every value a small
    # multiple of 2^-5, so that every sum is exact whatever its order: both kernels and the oracle agree bit for bit.
    rng = np.random.default_rng(9)
    dims, B = [8, 64, 64, 2], 16384
    specs = []
    for i in range(len(dims) - 1):
        fo, fi = dims[i + 1], dims[i]
        W = np.zeros((fo, fi), np.float16)
        for r in range(fo):
            W[r, rng.choice(fi, 2, replace=False)] = rng.choice(np.array([-1, 1], np.float16), 2)
        b = rng.integers(-1, 2, fo).astype(np.float16)
        if i + 2 < len(dims):
            W[::3] = 0; b[::3] = 0              # rows of zeros in W and b: a pre-activation of +0 for every sample
        specs.append(dict(W=W, b=b, act=int(Activation.NoActivation if i == len(dims) - 2 else Activation.ReLU), slope=0.0))
    x = rng.integers(-1, 2, (B, dims[0])).astype(np.float16)
    t = rng.integers(-2, 3, (B, dims[-1])).astype(np.float16)
    a, b = build(specs), build(specs)
    scale = 1.0 / 16
    cv.mlpTrainStep(a, to_dev(x), to_dev(t), lossScale=scale, flags=cv.FLAG_TRAIN_SPLIT_BY_ROLE)
    assert cv.lastKernelName().startswith("mlpTrainTeamKernel"), cv.lastKernelName()
    cv.mlpTrainStep(b, to_dev(x), to_dev(t), lossScale=scale)
    aW, aB = read_grads(a, specs, CT.Float32, ML.RowMajor)
    bW, bB = read_grads(b, specs, CT.Float32, ML.RowMajor)
    rW, rB, _ = ob.ref_mlp_train(specs, x, t, scale, tie_rule=True)
    nW, nB, _ = ob.ref_mlp_train(specs, x, t, scale, tie_rule=False)
    for l in range(len(specs)):
        assert np.array_equal(aW[l], bW[l]) and np.array_equal(aB[l], bB[l]), l
        assert np.array_equal(aW[l], rW[l]) and np.array_equal(aB[l], rB[l]), l
    assert not np.array_equal(nB[0], rB[0])     # the rule matters on this data
