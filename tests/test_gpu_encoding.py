"""GPU parity of the input encodings in front of the MLP, through the C-ABI.

The example's encoding (network.slang:35-38) and loss (network.slang:58-75) are evaluated in half; the
test restates them with numpy float16 arithmetic (IEEE half, one rounding per operation) and feeds the
encoded vectors / targets to the un-encoded entry points, which the other tests hold to the oracle:
encoded and un-encoded launches must agree bit for bit."""
import numpy as np
import pytest
import torch

import oracle_binding as ob
from gpu_util import DEV, as_bytes, to_dev
from slang_amd import coopvec as cv
from slang_amd.coopvec import Activation, CoopVecComponentType as CT, CoopVecMatrixLayout as ML, FeedForwardLayer, InputEncoding
from test_gpu_train import build, make_specs, read_grads

pytestmark = pytest.mark.gpu


def encode_xy_squares(xy32: np.ndarray) -> np.ndarray:
    h = xy32.astype(np.float16)                                # (half2)inputs[tid], kernels.slang:19
    return np.concatenate([h, h * h], axis=1)                  # CoopVec<half,4>(x, y, x*x, y*y), network.slang:37


def groundtruth(xy32: np.ndarray) -> np.ndarray:
    h = xy32.astype(np.float16)
    x, y = h[:, 0], h[:, 1]
    one, two, hlf, c12 = np.float16(1), np.float16(2), np.float16(0.5), np.float16(1.2)
    return np.stack([(x + y) / (one + y * y), two * x + y, hlf * x * x + c12 * y, x + hlf * y * y], axis=1)   # network.slang:67-75


@pytest.mark.parametrize("dims,B", [([4, 16, 4], 1000), ([4, 64, 64, 4], 4099), ([4, 24, 9], 333)])
def test_forward_with_example_encoding(dims, B):
    rng = np.random.default_rng(sum(dims))
    specs = make_specs(rng, dims, act=Activation.LeakyReLU, slope=float(np.float16(0.001)))
    xy = rng.uniform(0, 1, (B, 2)).astype(np.float32)
    layers = build(specs)
    y_enc = cv.mlpForward(layers, to_dev(xy), inputEncoding=InputEncoding.XYSquares)
    y_ref = cv.mlpForward(layers, to_dev(encode_xy_squares(xy)))
    assert torch.equal(y_enc.view(torch.int16), y_ref.view(torch.int16))
    # strided float2 samples (two of every four floats)
    wide = to_dev(np.concatenate([xy, -xy], axis=1))
    y_str = cv.mlpForward(layers, wide[:, :2], inputEncoding=InputEncoding.XYSquares)
    assert torch.equal(y_str.view(torch.int16), y_ref.view(torch.int16))


@pytest.mark.parametrize("dims,B", [([4, 16, 4], 16), ([4, 16, 4], 2000), ([4, 64, 64, 4], 1500)])
def test_training_step_with_example_encoding_and_loss(dims, B):
    # learnGradient of the example: float2 samples in, encoding, loss against groundtruth(x, y) -- all in the kernel
    rng = np.random.default_rng(B)
    specs = make_specs(rng, dims, act=Activation.LeakyReLU, slope=float(np.float16(0.001)))
    specs[-1]["act"] = int(Activation.LeakyReLU)            # the example activates the last layer too (fflayer.slang:60-66)
    specs[-1]["slope"] = float(np.float16(0.001))
    xy = rng.uniform(0, 1, (B, 2)).astype(np.float32)
    la = build(specs, CT.Float32, ML.TrainingOptimal)
    _, loss_a = cv.mlpTrainStep(la, to_dev(xy), None, inputEncoding=InputEncoding.XYSquares)
    lb = build(specs, CT.Float32, ML.TrainingOptimal)
    _, loss_b = cv.mlpTrainStep(lb, to_dev(encode_xy_squares(xy)), to_dev(groundtruth(xy)))
    for a, b in zip(la, lb):
        assert torch.equal(a.weightsGrad, b.weightsGrad) and torch.equal(a.biasesGrad, b.biasesGrad)
    assert loss_a.item() == loss_b.item()
    # and the un-encoded launch is the one the oracle checks
    dW, dB = read_grads(lb, specs, CT.Float32, ML.TrainingOptimal)
    rW, rB, rloss = ob.ref_mlp_train(specs, encode_xy_squares(xy), groundtruth(xy), 1.0, tie_rule=True)
    for l in range(len(specs)):
        assert np.linalg.norm(dW[l] - rW[l]) <= 1e-3 * np.linalg.norm(rW[l])
    assert abs(loss_a.item() - rloss) <= 1e-3 * rloss


def test_encoding_argument_validation():
    rng = np.random.default_rng(0)
    layers = build(make_specs(rng, [8, 16, 4]))
    xy = torch.zeros(10, 2, dtype=torch.float32, device=DEV)
    with pytest.raises(cv.CoopVecError) as e:
        cv.mlpForward(layers, xy, inputEncoding=InputEncoding.XYSquares)     # first layer must take 4 inputs
    assert e.value.result == cv.SLANG_E_NOT_AVAILABLE
    layers = build(make_specs(rng, [4, 16, 3]))
    with pytest.raises(cv.CoopVecError) as e:
        cv.mlpTrainStep(layers, xy, None, inputEncoding=InputEncoding.XYSquares)    # the example's loss has 4 outputs
    assert e.value.result == cv.SLANG_E_INVALID_ARG
