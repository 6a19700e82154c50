"""GPU parity of the fused training step against the fp64-accumulating CPU oracle, through the C-ABI.

Bar (fp16 carrier, fp32 accumulation of the gradients on the GPU, fp64 in the oracle): per layer
||dW_gpu - dW_ref||_F <= 1e-3 * ||dW_ref||_F (same for db), plus bitwise run-to-run determinism.
With explicit targets every rounding point of the oracle is reproduced; the residual differences
are hidden units whose fp32 sum fell within one rounding of an fp16 boundary."""
import json
import os

import numpy as np
import pytest
import torch

import oracle_binding as ob
from gpu_util import DEV, as_bytes, matrix_in_layout, to_dev
from slang_amd import coopvec as cv
from slang_amd.coopvec import Activation, CoopVecComponentType as CT, CoopVecMatrixLayout as ML, FeedForwardLayer

pytestmark = pytest.mark.gpu
G = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "coopvec_goldens.json")))


def build(specs, grad_ct=CT.Float32, grad_layout=ML.RowMajor, preset=None):
    layers = []
    gdt = torch.float32 if grad_ct == CT.Float32 else torch.float16
    for li, s in enumerate(specs):
        out, fan_in = s["W"].shape
        size = cv.getCooperativeVectorMatrixSize(out, fan_in, grad_ct, grad_layout)
        wg = torch.zeros(size, dtype=torch.uint8, device=DEV)
        bg = torch.zeros(out, dtype=gdt, device=DEV)
        if preset is not None:
            bg += preset
        layers.append(FeedForwardLayer(fan_in, out, as_bytes(to_dev(s["W"])),
                                       as_bytes(to_dev(s["b"])) if s["b"] is not None else None,
                                       ML.RowMajor, fan_in * 2, s["act"], s.get("slope", 0.0),
                                       wg, bg.view(torch.uint8), grad_layout, 0))
    return layers


def read_grads(layers, specs, grad_ct, grad_layout):
    dW, dB = [], []
    npdt = np.float32 if grad_ct == CT.Float32 else np.float16
    for L, s in zip(layers, specs):
        out, fan_in = s["W"].shape
        raw = L.weightsGrad.cpu().numpy()
        back = np.zeros((out, fan_in), npdt)
        rc = ob.lib().cvo_layout_convert(ob.ptr(back), out, fan_in, int(grad_ct), ob.ROW, 0, ob.ptr(raw), int(grad_ct),
                                         int(grad_layout), 0)
        assert rc == 0
        dW.append(back.astype(np.float64))
        dB.append(L.biasesGrad.cpu().numpy().view(npdt).astype(np.float64))
    return dW, dB


def rel_err(a, b):
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)


def make_specs(rng, dims, act=Activation.ReLU, slope=0.0, bias=True):
    specs = []
    for i in range(len(dims) - 1):
        fi, fo = dims[i], dims[i + 1]
        W = (rng.standard_normal((fo, fi)) * np.sqrt(2.0 / fi)).astype(np.float16)
        b = rng.uniform(-0.1, 0.1, fo).astype(np.float16) if bias else None
        last = i == len(dims) - 2
        specs.append(dict(W=W, b=b, act=int(Activation.NoActivation if last else act), slope=slope))
    return specs


def test_ffn_closed_form_backward():
    # tests/neural/basic-ilayer-ffn-backward-test.slang: dW1=[-3,4,6,-8], db1=[-2,4], dW2=[6,-7.25], db2=1
    f, bwd = G["ffn_forward"], G["ffn_backward"]
    specs = [dict(W=np.array(f["W1"], np.float16), b=np.array(f["b1"], np.float16), act=0),
             dict(W=np.array(f["W2"], np.float16), b=np.array(f["b2"], np.float16), act=0)]
    layers = build(specs)
    x = to_dev(np.array([f["x"]], np.float16))
    t = to_dev(np.array([[-41.0]], np.float16))          # seed 2*(y - t) = 1 with y = -40.5
    _, loss = cv.mlpTrainStep(layers, x, t)
    dW, dB = read_grads(layers, specs, CT.Float32, ML.RowMajor)
    assert dW[0].tolist() == bwd["dW1"] and dB[0].tolist() == bwd["db1"]
    assert dW[1].tolist() == bwd["dW2"] and dB[1].tolist() == bwd["db2"]
    assert loss.item() == 0.25


@pytest.mark.parametrize("dims,B", [([8, 64, 64, 64, 64, 1], 4096 + 21), ([4, 16, 4], 1000), ([2, 16, 16, 16, 1], 2048),
                                    ([8, 32, 32, 4], 777), ([20, 64, 64, 8], 1500), ([8, 64, 64, 64, 5], 900),
                                    ([8, 32, 4], 300), ([8, 32, 32, 32, 4], 1500), ([8, 32, 32, 32, 32, 2], 2100), ([24, 32, 32, 32, 8], 1000),
                                    ([8, 64, 4], 513), ([24, 64, 64, 64, 6], 1200),
                                    # hidden layers of different widths, and widths between the tile counts the kernels are built
                                    # for: the widest one decides, the others are padded to it
                                    ([8, 16, 64, 4], 1500), ([20, 48, 24, 5], 700), ([8, 48, 48, 48, 3], 900), ([5, 40, 2], 333)])
def test_train_step_against_oracle(dims, B):
    rng = np.random.default_rng(sum(dims) + B)
    specs = make_specs(rng, dims)
    x = rng.uniform(-1, 1, (B, dims[0])).astype(np.float16)
    t = np.sin(x.astype(np.float32).sum(1, keepdims=True)).astype(np.float16).repeat(dims[-1], 1)
    t = np.ascontiguousarray(t)
    layers = build(specs)
    _, loss = cv.mlpTrainStep(layers, to_dev(x), to_dev(t))
    # one launch for the whole step (plus the reduction): hidden layers of 16, 32 or 64 units all have a fused kernel
    assert cv.lastKernelName().startswith(("mlpTrainPairKernel", "mlpTrainKernel")), cv.lastKernelName()
    dW, dB = read_grads(layers, specs, CT.Float32, ML.RowMajor)
    rW, rB, rloss = ob.ref_mlp_train(specs, x, t, 1.0, tie_rule=True)
    for l in range(len(specs)):
        assert rel_err(dW[l], rW[l]) <= 1e-3, (l, rel_err(dW[l], rW[l]))
        assert rel_err(dB[l], rB[l]) <= 1e-3, (l, rel_err(dB[l], rB[l]))
    assert abs(loss.item() - rloss) <= 1e-3 * rloss
    # the layer-by-layer step gives the same gradients to its own bar
    if max(dims) <= 32:
        general = build(specs)
        cv.mlpTrainStep(general, to_dev(x), to_dev(t), flags=cv.FLAG_LAYERWISE_TRAINING)
        gW, gB = read_grads(general, specs, CT.Float32, ML.RowMajor)
        for l in range(len(specs)):
            assert rel_err(gW[l], dW[l]) <= 1e-3 and rel_err(gB[l], dB[l]) <= 1e-3
    # bitwise determinism, and "+=" semantics: a second step doubles the (fp32) gradients exactly
    before = [L.weightsGrad.clone() for L in layers]
    layers2 = build(specs)
    cv.mlpTrainStep(layers2, to_dev(x), to_dev(t))
    for a, b in zip(before, layers2):
        assert torch.equal(a, b.weightsGrad)
    cv.mlpTrainStep(layers, to_dev(x), to_dev(t))
    for a, L in zip(before, layers):
        assert torch.equal(a.view(torch.float32) * 2, L.weightsGrad.view(torch.float32))


def test_train_step_sin_target_in_kernel():
    # the training configuration: 8 -> 64 x4 -> 1, ReLU, He init, inputs U[-1,1]^8, target sin(sum x)
    rng = np.random.default_rng(5)
    dims = [8, 64, 64, 64, 64, 1]
    B = 8192
    specs = make_specs(rng, dims, bias=False)
    x = rng.uniform(-1, 1, (B, 8)).astype(np.float16)
    layers = build(specs, grad_layout=ML.TrainingOptimal)
    _, loss = cv.mlpTrainStep(layers, to_dev(x), None)
    dW, dB = read_grads(layers, specs, CT.Float32, ML.TrainingOptimal)
    rW, rB, rloss = ob.ref_mlp_train(specs, x, None, 1.0, tie_rule=True)
    for l in range(len(specs)):
        assert rel_err(dW[l], rW[l]) <= 1e-3, (l, rel_err(dW[l], rW[l]))
        assert rel_err(dB[l], rB[l]) <= 1e-3
    assert abs(loss.item() - rloss) <= 1e-3 * rloss


def gradient_term_sums(specs, x, t):
    """sum over the batch of |dZ_l[s][i] * X_l[s][j]| (and of |dZ_l[s][i]| for the biases) of a ReLU network with an MSE
    loss, carriers rounded to half like the kernels': the scale against which an element of a gradient is
    cancellation-dominated or not."""
    a = [x.astype(np.float32)]
    zs = []
    for s in specs:
        z = a[-1] @ s["W"].astype(np.float32).T + (s["b"].astype(np.float32) if s["b"] is not None else 0.0)
        z = z.astype(np.float16).astype(np.float32)
        zs.append(z)
        a.append(np.maximum(z, 0) if s["act"] == int(Activation.ReLU) else z)
    g = (2.0 * (a[-1] - t.astype(np.float32))).astype(np.float16).astype(np.float32)
    tW, tB = [None] * len(specs), [None] * len(specs)
    for l in reversed(range(len(specs))):
        dz = g * (zs[l] > 0) if specs[l]["act"] == int(Activation.ReLU) else g
        tW[l] = np.abs(dz).T.astype(np.float64) @ np.abs(a[l]).astype(np.float64)
        tB[l] = np.abs(dz).sum(0).astype(np.float64)
        g = (dz @ specs[l]["W"].astype(np.float32)).astype(np.float16).astype(np.float32)
    return tW, tB


def test_train_step_gradients_element_by_element():
    # Per element of every gradient of the training configuration (8 -> 64 x4 -> 1, batch 2^14 here), against the
    # fp64-accumulating oracle: of the elements that are not cancellation-dominated, |g| >= 2^-8 * sum|terms| (13 018 of
    # the 13 121), at least 99.9 % agree to 2 ulp of fp16 at their own magnitude (about 1e-3 relative; seen: all but 4),
    # and every element agrees to max(6 ulp, 2^-14 * sum|terms|).  The stragglers are units that few samples activate:
    # there a single sample in which the two sides rounded a carrier to neighbouring halves (a hidden unit or the
    # network's output whose fp32 sum lies on an fp16 boundary; the loss gradient 2(y - t) then moves by an ulp of y,
    # which is several ulp of a small difference) is a visible part of the sum.
    rng = np.random.default_rng(2020)
    dims = [8, 64, 64, 64, 64, 1]
    B = 1 << 14
    specs = make_specs(rng, dims)
    x = rng.uniform(-1, 1, (B, dims[0])).astype(np.float16)
    t = np.sin(x.astype(np.float32).sum(1, keepdims=True)).astype(np.float16)
    layers = build(specs, grad_layout=ML.TrainingOptimal)
    cv.mlpTrainStep(layers, to_dev(x), to_dev(t))
    assert cv.lastKernelName().startswith("mlpTrainPairKernel"), cv.lastKernelName()
    dW, dB = read_grads(layers, specs, CT.Float32, ML.TrainingOptimal)
    rW, rB, _ = ob.ref_mlp_train(specs, x, t, 1.0, tie_rule=True)
    tW, tB = gradient_term_sums(specs, x, t)
    checked = beyond_ulp = 0
    for l in range(len(specs)):
        for got, ref, terms in ((dW[l], rW[l], tW[l]), (dB[l], rB[l], tB[l])):
            solid = np.abs(ref) >= 2.0 ** -8 * terms
            err = np.abs(got - ref)
            ulp_bar = 2.0 * ob.f16_ulp(ref.astype(np.float32)).astype(np.float64)
            bad = err > np.maximum(3.0 * ulp_bar, 2.0 ** -14 * terms)
            assert not bad.any(), "layer %d: %d of %d elements outside the bar" % (l, bad.sum(), bad.size)
            checked += int(solid.sum())
            beyond_ulp += int((solid & (err > ulp_bar)).sum())
    assert beyond_ulp <= checked // 1000, (beyond_ulp, checked)
    assert checked > 12000      # nearly all of the 13 121 elements are not cancellation-dominated


@pytest.mark.parametrize("dims,B,flags", [([8, 64, 64, 64, 64, 1], 5000, 0), ([4, 16, 4], 16, 0), ([8, 32, 32, 6], 777, 0),
                                          ([8, 64, 64, 64, 64, 1], 3000, cv.FLAG_LAYERWISE_TRAINING), ([20, 50, 7], 300, 0)])
def test_loss_max_is_the_largest_per_sample_loss(dims, B, flags):
    # lossMax: what learnGradient leaves in its loss buffer (WaveActiveMax + atomic max, kernels.slang:21-26), from the
    # paired kernel, the one-wave kernel and the layer-by-layer step; gradients and lossSum are what they are without it
    rng = np.random.default_rng(sum(dims) + B)
    specs = make_specs(rng, dims)
    x = rng.uniform(-1, 1, (B, dims[0])).astype(np.float16)
    t = rng.uniform(-1, 1, (B, dims[-1])).astype(np.float16)
    layers = build(specs)
    lmax = torch.full((1,), -1.0, dtype=torch.float32, device=DEV)
    _, loss = cv.mlpTrainStep(layers, to_dev(x), to_dev(t), lossMax=lmax, flags=flags)
    y = cv.mlpForward(gpu_fwd_layers(specs), to_dev(x)).cpu().numpy()
    diff = (y.astype(np.float32) - t.astype(np.float32)).astype(np.float16).astype(np.float32)
    per_sample = (diff * diff).sum(1, dtype=np.float64)
    assert abs(lmax.item() - per_sample.max()) <= 1e-5 * per_sample.max(), (lmax.item(), per_sample.max())
    assert abs(loss.item() - per_sample.sum()) <= 1e-4 * per_sample.sum()
    layers2 = build(specs)
    _, loss2 = cv.mlpTrainStep(layers2, to_dev(x), to_dev(t), flags=flags)
    assert loss2.item() == loss.item()
    for a, b in zip(layers, layers2):
        assert torch.equal(a.weightsGrad, b.weightsGrad) and torch.equal(a.biasesGrad, b.biasesGrad)


def gpu_fwd_layers(specs):
    return [FeedForwardLayer(s["W"].shape[1], s["W"].shape[0], as_bytes(to_dev(s["W"])),
                             as_bytes(to_dev(s["b"])) if s["b"] is not None else None, ML.RowMajor, s["W"].shape[1] * 2,
                             s["act"], s.get("slope", 0.0)) for s in specs]


def test_nan_loss_voids_the_whole_step():
    # A workgroup whose loss partial is NaN voids the step: the loss outputs and every gradient sum the step adds
    # are NaN (this is how a pair meeting that timed out reports itself; a NaN sample takes the same path)
    rng = np.random.default_rng(4)
    dims, B = [8, 64, 64, 64, 64, 1], 4096
    specs = make_specs(rng, dims)
    x = rng.uniform(-1, 1, (B, dims[0])).astype(np.float16)
    x[1234, 3] = np.nan
    layers = build(specs)
    lmax = torch.zeros(1, dtype=torch.float32, device=DEV)
    _, loss = cv.mlpTrainStep(layers, to_dev(x), None, lossMax=lmax)
    assert cv.lastKernelName().startswith("mlpTrainPairKernel")
    assert np.isnan(loss.item()) and np.isnan(lmax.item())
    for L in layers:
        assert torch.isnan(L.weightsGrad.view(torch.float32)).all() and torch.isnan(L.biasesGrad.view(torch.float32)).all()


def test_train_tie_rule_and_leaky_relu():
    # a hidden unit at exactly z = 0 gets half of the gradient (diff.meta.slang:2258-2277)
    specs = [dict(W=np.array([[1.0], [0.5]] + [[0.0]] * 14, np.float16), b=np.array([-1.0, 0.25] + [0.0] * 14, np.float16), act=1),
             dict(W=np.array([[2.0, 1.0] + [0.0] * 14], np.float16), b=None, act=0)]
    layers = build(specs)
    x = to_dev(np.array([[1.0]], np.float16))            # z = [0, 0.75, 0...]: y = 0.75
    t = to_dev(np.array([[0.25]], np.float16))           # dL/dy = 1
    cv.mlpTrainStep(layers, x, t)
    dW, dB = read_grads(layers, specs, CT.Float32, ML.RowMajor)
    rW, rB, _ = ob.ref_mlp_train(specs, np.array([[1.0]], np.float16), np.array([[0.25]], np.float16), 1.0, True)
    assert dB[0].tolist() == rB[0].tolist() and dB[0][0] == 1.0 and dB[0][1] == 1.0   # 0.5*2 and 1*1
    assert dW[0].tolist() == rW[0].tolist()
    # leaky ReLU network (the example's activation on hidden layers)
    rng = np.random.default_rng(9)
    slope = float(np.float16(0.001))
    specs = make_specs(rng, [4, 16, 4], act=Activation.LeakyReLU, slope=slope)
    B = 512
    x = rng.uniform(0, 1, (B, 4)).astype(np.float16)
    t = rng.uniform(-1, 1, (B, 4)).astype(np.float16)
    layers = build(specs)
    cv.mlpTrainStep(layers, to_dev(x), to_dev(t))
    dW, dB = read_grads(layers, specs, CT.Float32, ML.RowMajor)
    rW, rB, _ = ob.ref_mlp_train(specs, x, t, 1.0, True)
    for l in range(2):
        assert rel_err(dW[l], rW[l]) <= 1e-3 and rel_err(dB[l], rB[l]) <= 1e-3


def test_train_tie_rule_wide_network():
    # 8 -> 64 -> 64 -> 1 with ReLU (the kernel instantiation the training configuration uses), one
    # sample, all values dyadic so that every sum is exact in fp16 and fp32 on both sides.  Layer 0 is
    # crafted so that hidden unit 0 has z = +0, unit 1 has a negative sum that rounds to -0 in fp16
    # (-2^-14 * 2^-14), unit 2 is negative and unit 3 positive; Slang's max() rule gives the tied
    # units half of the gradient whatever the sign of the zero (diff.meta.slang:2258-2277).
    rng = np.random.default_rng(314)
    tiny = np.float16(2.0 ** -14)
    W0 = np.zeros((64, 8), np.float16)
    W0[1, 0] = -tiny; W0[2, 0] = -1.0; W0[3, 1] = 1.0
    x = np.zeros((1, 8), np.float16); x[0, 0] = tiny; x[0, 1] = 1.0
    W1 = rng.choice(np.array([-1, -0.5, -0.25, 0.25, 0.5, 1], np.float16), (64, 64))
    W1[:4, 3] = [0.0, 0.5, -1.0, 0.25]          # layer 1 gets a tie, two positives and a negative of its own
    W2 = rng.choice(np.array([-1, -0.5, 0.5, 1], np.float16), (1, 64))
    specs = [dict(W=W0, b=np.zeros(64, np.float16), act=1), dict(W=W1, b=None, act=1), dict(W=W2, b=None, act=0)]
    a1 = np.maximum(W1[:, 3].astype(np.float64), 0)
    y = float((W2.astype(np.float64) @ a1)[0])
    t = np.array([[y - 0.5]], np.float16)                # dL/dy = 2 * 0.5 = 1
    assert float(t[0, 0]) == y - 0.5
    layers = build(specs, grad_layout=ML.TrainingOptimal)
    _, loss = cv.mlpTrainStep(layers, to_dev(x), to_dev(t))
    dW, dB = read_grads(layers, specs, CT.Float32, ML.TrainingOptimal)
    rW, rB, rloss = ob.ref_mlp_train(specs, x, t, 1.0, tie_rule=True)
    assert loss.item() == 0.25 == rloss
    for l in range(3):
        assert np.array_equal(dW[l], rW[l]) and np.array_equal(dB[l], rB[l]), l
    # the rule itself, against the upstream gradient g0 = W1^T dz1 of layer 0's outputs
    dz1 = W2[0].astype(np.float64) * np.where(W1[:, 3] > 0, 1.0, np.where(W1[:, 3] == 0, 0.5, 0.0))
    g0 = W1.astype(np.float64).T @ dz1
    assert dB[0][0] == 0.5 * g0[0] and dB[0][1] == 0.5 * g0[1] and dB[0][2] == 0.0 and dB[0][3] == g0[3]
    assert g0[0] != 0 and g0[1] != 0 and g0[2] != 0
    # without the tie rule the oracle disagrees, i.e. the check above has teeth
    nW, nB, _ = ob.ref_mlp_train(specs, x, t, 1.0, tie_rule=False)
    assert not np.array_equal(nB[0], rB[0])


def test_train_fp16_training_optimal_gradients_and_convert():
    # the example's flow: fp16 TrainingOptimal weight gradients, then one convert call to RowMajor
    rng = np.random.default_rng(10)
    dims = [4, 16, 4]
    specs = make_specs(rng, dims)
    B = 64
    x = rng.uniform(0, 1, (B, 4)).astype(np.float16)
    t = rng.uniform(-1, 1, (B, 4)).astype(np.float16)
    layers = build(specs, CT.Float16, ML.TrainingOptimal, preset=None)
    cv.mlpTrainStep(layers, to_dev(x), to_dev(t), lossScale=1.0 / 64, gradType=CT.Float16)
    rW, rB, _ = ob.ref_mlp_train(specs, x, t, 1.0 / 64, True)
    for l, (L, s) in enumerate(zip(layers, specs)):
        out, fan_in = s["W"].shape
        row = torch.zeros(out * fan_in * 2, dtype=torch.uint8, device=DEV)
        size = cv.getCooperativeVectorMatrixSize(out, fan_in, CT.Float16, ML.TrainingOptimal)
        cv.convertCooperativeVectorMatrix(row, [cv.CooperativeVectorMatrixDesc(out, fan_in, CT.Float16, ML.RowMajor, out * fan_in * 2, 0, fan_in * 2)],
                                          L.weightsGrad, [cv.CooperativeVectorMatrixDesc(out, fan_in, CT.Float16, ML.TrainingOptimal, size, 0, 0)])
        got = row.cpu().numpy().view(np.float16).reshape(out, fan_in).astype(np.float64)
        assert np.max(np.abs(got - rW[l])) <= 2e-3 * np.max(np.abs(rW[l])) + 1e-6


@pytest.mark.parametrize("dims,B,act,slope", [
    ([8, 16, 64, 4], 1500, Activation.ReLU, 0.0),           # hidden widths differ
    ([20, 48, 24, 5], 700, Activation.ReLU, 0.0),           # the shapes of the general forward kernel's test
    ([3, 7, 33, 2], 333, Activation.LeakyReLU, 0.25),
    ([12, 100, 100, 9], 1000, Activation.LeakyReLU, 0.1),
    ([64, 160, 96, 32], 900, Activation.ReLU, 0.0),         # wider than 128
    ([8, 64, 64, 64, 64, 1], 2000, Activation.ReLU, 0.0),   # a fused shape, forced through the general step below
    ([16, 128, 128, 128, 4], 600, Activation.ReLU, 0.0),    # three 128-wide hidden layers: no fused kernel
])
@pytest.mark.parametrize("grad_ct,grad_layout", [(CT.Float32, ML.RowMajor), (CT.Float16, ML.TrainingOptimal)])
def test_general_training_step_against_oracle(dims, B, act, slope, grad_ct, grad_layout):
    rng = np.random.default_rng(sum(dims) + B + int(grad_ct))
    specs = make_specs(rng, dims, act=act, slope=slope)
    x = rng.uniform(-1, 1, (B, dims[0])).astype(np.float16)
    t = rng.uniform(-1, 1, (B, dims[-1])).astype(np.float16)
    layers = build(specs, grad_ct, grad_layout)
    fused_shape = max(dims[1:-1]) <= 128      # these also have a fused kernel: the general step is asked for
    flags = cv.FLAG_LAYERWISE_TRAINING if fused_shape else 0
    _, loss = cv.mlpTrainStep(layers, to_dev(x), to_dev(t), gradType=grad_ct, flags=flags)
    assert "layer-by-layer" in cv.lastKernelName()
    dW, dB = read_grads(layers, specs, grad_ct, grad_layout)
    rW, rB, rloss = ob.ref_mlp_train(specs, x, t, 1.0, tie_rule=True)
    tol = 1e-3 if grad_ct == CT.Float32 else 2e-3      # fp16 gradient storage rounds each element once more
    for l in range(len(specs)):
        assert rel_err(dW[l], rW[l]) <= tol, (l, rel_err(dW[l], rW[l]))
        assert rel_err(dB[l], rB[l]) <= tol, (l, rel_err(dB[l], rB[l]))
    assert abs(loss.item() - rloss) <= 1e-3 * rloss
    # bitwise determinism
    layers2 = build(specs, grad_ct, grad_layout)
    cv.mlpTrainStep(layers2, to_dev(x), to_dev(t), gradType=grad_ct, flags=flags)
    for a, b in zip(layers, layers2):
        assert torch.equal(a.weightsGrad, b.weightsGrad) and torch.equal(a.biasesGrad, b.biasesGrad)
    if fused_shape:
        # the fused kernel on the same step: same rounding points, only the order of the fp32 sums differs
        layers3 = build(specs, grad_ct, grad_layout)
        _, loss3 = cv.mlpTrainStep(layers3, to_dev(x), to_dev(t), gradType=grad_ct)
        assert ("mlpTrain" in cv.lastKernelName() and "layer-by-layer" not in cv.lastKernelName()) == (len(dims) <= 4 or max(dims[1:-1]) <= 64)
        fW, fB = read_grads(layers3, specs, grad_ct, grad_layout)
        for l in range(len(specs)):
            assert rel_err(fW[l], dW[l]) <= (1e-4 if grad_ct == CT.Float32 else 1e-3)
            assert rel_err(fB[l], dB[l]) <= (1e-4 if grad_ct == CT.Float32 else 1e-3)
        assert abs(loss3.item() - loss.item()) <= 1e-5 * loss.item()


def test_general_training_step_tie_rule_and_sin_target():
    # hidden pre-activations that are exactly zero take half the gradient (Slang's max rule), also on the
    # layer-by-layer step; targets == None selects sin(sum of the inputs)
    rng = np.random.default_rng(31)
    dims = [8, 16, 40, 3]
    B = 512
    specs = make_specs(rng, dims, bias=False)
    specs[0]["W"][:4] = 0                                   # four hidden units of layer 0 are always exactly 0
    x = rng.uniform(-1, 1, (B, 8)).astype(np.float16)
    layers = build(specs)
    _, loss = cv.mlpTrainStep(layers, to_dev(x), None, flags=cv.FLAG_LAYERWISE_TRAINING)
    assert "layer-by-layer" in cv.lastKernelName()
    dW, dB = read_grads(layers, specs, CT.Float32, ML.RowMajor)
    rW, rB, rloss = ob.ref_mlp_train(specs, x, None, 1.0, tie_rule=True)
    nW, nB, _ = ob.ref_mlp_train(specs, x, None, 1.0, tie_rule=False)
    assert np.abs(rB[0][:4]).min() > 0 and np.abs(nB[0][:4]).max() == 0      # the rule matters here
    for l in range(len(specs)):
        assert rel_err(dW[l], rW[l]) <= 1e-3 and rel_err(dB[l], rB[l]) <= 1e-3
    assert abs(loss.item() - rloss) <= 1e-3 * rloss


def test_train_argument_validation():
    rng = np.random.default_rng(0)
    specs = make_specs(rng, [8, 16, 4])
    layers = build(specs)
    x = torch.zeros(10, 8, dtype=torch.float16, device=DEV)
    need = cv.mlpTrainStepWorkspaceSize(layers, 10)
    assert need > 0
    with pytest.raises(cv.CoopVecError) as e:
        cv.mlpTrainStep(layers, x, None, workspace=torch.zeros(need - 16, dtype=torch.uint8, device=DEV))
    assert e.value.result == cv.SLANG_E_BUFFER_TOO_SMALL
    # layer sizes outside the fused shapes take the layer-by-layer step, whose workspace grows with the batch
    specs = make_specs(rng, [8, 16, 160, 4])
    assert cv.mlpTrainStepWorkspaceSize(build(specs), 4096) > cv.mlpTrainStepWorkspaceSize(build(specs), 16) > 0
    with pytest.raises(cv.CoopVecError) as e:      # one layer has nothing to chain
        cv.mlpTrainStepWorkspaceSize(build(make_specs(rng, [8, 4])), 10)
    assert e.value.result == cv.SLANG_E_NOT_AVAILABLE


def test_full_size_training_step_properties():
    # the training configuration at its full batch (2^20): bitwise determinism, scaling of the
    # gradients with the loss scale, and agreement with the oracle on a leading slice
    rng = np.random.default_rng(2020)
    dims = [8, 64, 64, 64, 64, 1]
    B = 1 << 20
    specs = make_specs(rng, dims, bias=False)
    g = torch.Generator(device=DEV); g.manual_seed(5)
    x = (torch.rand(B, 8, device=DEV, generator=g) * 2 - 1).half()
    TO = ML.TrainingOptimal      # the configuration's gradient destinations: fp32 TrainingOptimal
    la, lb, lc = build(specs, grad_layout=TO), build(specs, grad_layout=TO), build(specs, grad_layout=TO)
    _, loss_a = cv.mlpTrainStep(la, x, None)
    _, loss_b = cv.mlpTrainStep(lb, x, None)
    cv.mlpTrainStep(lc, x, None, lossScale=0.5)
    for a, b, c in zip(la, lb, lc):
        assert torch.equal(a.weightsGrad, b.weightsGrad) and torch.equal(a.biasesGrad, b.biasesGrad)
        # scaling is exact except where a carrier gradient is subnormal in fp16
        fa, fc = a.weightsGrad.view(torch.float32), c.weightsGrad.view(torch.float32)
        assert (fa * 0.5 - fc).norm().item() <= 1e-3 * fc.norm().item()
    assert loss_a.item() == loss_b.item()
    # the first 4096 samples against the fp64 oracle (same kernel, smaller batch)
    n = 4096
    ls = build(specs, grad_layout=TO)
    cv.mlpTrainStep(ls, x[:n], None)
    dW, dB = read_grads(ls, specs, CT.Float32, TO)
    rW, rB, _ = ob.ref_mlp_train(specs, x[:n].cpu().numpy(), None, 1.0, True)
    for l in range(len(specs)):
        assert rel_err(dW[l], rW[l]) <= 1e-3
    # additivity over a split of the batch (fp32 sums in a different order: relative 1e-5)
    l1 = build(specs, grad_layout=TO)
    cv.mlpTrainStep(l1, x[: B // 2], None)
    cv.mlpTrainStep(l1, x[B // 2:], None)        # "+=" into the same buffers
    for a, s in zip(la, l1):
        fa, fs = a.weightsGrad.view(torch.float32), s.weightsGrad.view(torch.float32)
        assert (fa - fs).norm().item() <= 1e-5 * fa.norm().item()


@pytest.mark.parametrize("dims,B,targets,grad_ct,grad_layout", [
    ([16, 128, 128, 8], 4096 + 37, True, CT.Float32, ML.RowMajor),
    ([16, 128, 128, 8], 3000, False, CT.Float16, ML.TrainingOptimal),
    ([7, 128, 3], 1111, True, CT.Float32, ML.TrainingOptimal),            # rows of 14 bytes
    ([24, 120, 128, 16], 2500, True, CT.Float32, ML.RowMajor),            # two input tiles, a hidden layer of 120
    ([32, 128, 1], 700, False, CT.Float32, ML.RowMajor),
    ([16, 80, 100, 8], 1300, True, CT.Float32, ML.RowMajor),              # padded to 128
    ([12, 100, 30, 9], 1000, True, CT.Float32, ML.TrainingOptimal),
])
def test_train_step_128_wide_hidden_layers(dims, B, targets, grad_ct, grad_layout):
    # one or two ReLU hidden layers, the wider of 65..128 units: the fused kernel in which four waves share the dW accumulators
    rng = np.random.default_rng(sum(dims) + B)
    specs = make_specs(rng, dims)
    x = rng.uniform(-1, 1, (B, dims[0])).astype(np.float16)
    t = rng.uniform(-1, 1, (B, dims[-1])).astype(np.float16) if targets else None
    layers = build(specs, grad_ct, grad_layout)
    lmax = torch.zeros(1, dtype=torch.float32, device=DEV)
    _, loss = cv.mlpTrainStep(layers, to_dev(x), to_dev(t) if targets else None, gradType=grad_ct, lossMax=lmax)
    assert cv.lastKernelName().startswith("mlpTrainQuadKernel"), cv.lastKernelName()
    dW, dB = read_grads(layers, specs, grad_ct, grad_layout)
    rW, rB, rloss = ob.ref_mlp_train(specs, x, t, 1.0, tie_rule=True)
    tol = 1e-3 if grad_ct == CT.Float32 else 2e-3
    for l in range(len(specs)):
        assert rel_err(dW[l], rW[l]) <= tol, (l, rel_err(dW[l], rW[l]))
        assert rel_err(dB[l], rB[l]) <= tol, (l, rel_err(dB[l], rB[l]))
    assert abs(loss.item() - rloss) <= 1e-3 * rloss
    # the layer-by-layer step on the same data: same rounding points, other order of the fp32 sums
    general = build(specs, grad_ct, grad_layout)
    lmax2 = torch.zeros(1, dtype=torch.float32, device=DEV)
    _, loss2 = cv.mlpTrainStep(general, to_dev(x), to_dev(t) if targets else None, gradType=grad_ct, flags=cv.FLAG_LAYERWISE_TRAINING,
                               lossMax=lmax2)
    assert "layer-by-layer" in cv.lastKernelName()
    gW, gB = read_grads(general, specs, grad_ct, grad_layout)
    for l in range(len(specs)):
        assert rel_err(gW[l], dW[l]) <= tol and rel_err(gB[l], dB[l]) <= tol, l
    assert abs(loss2.item() - loss.item()) <= 1e-4 * loss.item()
    assert abs(lmax2.item() - lmax.item()) <= 1e-3 * lmax.item()
    # bitwise determinism
    again = build(specs, grad_ct, grad_layout)
    cv.mlpTrainStep(again, to_dev(x), to_dev(t) if targets else None, gradType=grad_ct)
    for a, b in zip(layers, again):
        assert torch.equal(a.weightsGrad, b.weightsGrad) and torch.equal(a.biasesGrad, b.biasesGrad)


def test_train_step_128_wide_tie_rule_and_other_activations():
    # exact small numbers: pre-activations of +0 take half the gradient; the fused kernel and the oracle agree bit for bit
    rng = np.random.default_rng(17)
    dims, B = [16, 128, 128, 2], 640
    specs = []
    for i in range(len(dims) - 1):
        fo, fi = dims[i + 1], dims[i]
        W = np.zeros((fo, fi), np.float16)
        for r in range(fo):
            W[r, rng.choice(fi, 2, replace=False)] = rng.choice(np.array([-1, 1], np.float16), 2)
        b = rng.integers(-1, 2, fo).astype(np.float16)
        if i + 2 < len(dims):
            W[::3] = 0; b[::3] = 0
        specs.append(dict(W=W, b=b, act=int(Activation.NoActivation if i == len(dims) - 2 else Activation.ReLU), slope=0.0))
    x = rng.integers(-1, 2, (B, dims[0])).astype(np.float16)
    t = rng.integers(-2, 3, (B, dims[-1])).astype(np.float16)
    layers = build(specs)
    cv.mlpTrainStep(layers, to_dev(x), to_dev(t), lossScale=1.0 / 16)
    assert cv.lastKernelName().startswith("mlpTrainQuadKernel"), cv.lastKernelName()
    dW, dB = read_grads(layers, specs, CT.Float32, ML.RowMajor)
    rW, rB, _ = ob.ref_mlp_train(specs, x, t, 1.0 / 16, tie_rule=True)
    nW, nB, _ = ob.ref_mlp_train(specs, x, t, 1.0 / 16, tie_rule=False)
    for l in range(len(specs)):
        assert np.array_equal(dW[l], rW[l]) and np.array_equal(dB[l], rB[l]), l
    assert not np.array_equal(nB[0], rB[0])
    # leaky ReLU (on one layer, ReLU on the other): the fused kernel's second instantiation, against the oracle and the
    # layer-by-layer step
    leaky = make_specs(rng, [16, 128, 128, 8], act=Activation.LeakyReLU, slope=0.125)
    leaky[1]["act"] = int(Activation.ReLU)
    xs = rng.uniform(-1, 1, (1500, 16)).astype(np.float16)
    ts = rng.uniform(-1, 1, (1500, 8)).astype(np.float16)
    L2, L3 = build(leaky), build(leaky)
    _, loss = cv.mlpTrainStep(L2, to_dev(xs), to_dev(ts))
    assert cv.lastKernelName().startswith("mlpTrainQuadKernel") and "leaky" in cv.lastKernelName(), cv.lastKernelName()
    cv.mlpTrainStep(L3, to_dev(xs), to_dev(ts), flags=cv.FLAG_LAYERWISE_TRAINING)
    assert "layer-by-layer" in cv.lastKernelName()
    aW, aB = read_grads(L2, leaky, CT.Float32, ML.RowMajor)
    gW, gB = read_grads(L3, leaky, CT.Float32, ML.RowMajor)
    rW, rB, rloss = ob.ref_mlp_train(leaky, xs, ts, 1.0, tie_rule=True)
    for l in range(3):
        assert rel_err(aW[l], rW[l]) <= 1e-3 and rel_err(aB[l], rB[l]) <= 1e-3, l
        assert rel_err(aW[l], gW[l]) <= 1e-3 and rel_err(aB[l], gB[l]) <= 1e-3, l
    assert abs(loss.item() - rloss) <= 1e-3 * rloss
    # a last layer with ReLU or leaky ReLU stays on that instantiation (test_activation_behind_the_last_layer_...); any
    # other activation there has no fused kernel for these widths
    leaky[2]["act"] = int(Activation.ReLU)
    cv.mlpTrainStep(build(leaky), to_dev(xs), to_dev(ts))
    assert cv.lastKernelName().startswith("mlpTrainQuadKernel") and "leaky" in cv.lastKernelName(), cv.lastKernelName()


def test_fused_and_layer_by_layer_steps_agree_on_random_shapes():
    # networks drawn at random within what the fused kernels take (up to 32 inputs, 16 outputs, four hidden layers of up to 64
    # units or two of up to 128, ReLU or leaky ReLU, hidden layers of different widths): the step the library picks and the
    # layer-by-layer step have the same rounding points and differ in the order of their fp32 sums only
    rng = np.random.default_rng(20260)
    fused = 0
    for case in range(40):
        wide = case % 4 == 3
        nhid = int(rng.integers(1, 3 if wide else 5))
        top = 128 if wide else 64
        dims = [int(rng.integers(1, 33))] + [int(rng.integers(top // 2 + 1 if h == 0 else 3, top + 1)) for h in range(nhid)] + [int(rng.integers(1, 17))]
        leaky = case % 3 == 1
        B = int(rng.integers(1, 700))
        specs = make_specs(rng, dims, act=Activation.LeakyReLU if leaky else Activation.ReLU, slope=0.125 if leaky else 0.0,
                           bias=case % 5 != 0)
        x = rng.uniform(-1, 1, (B, dims[0])).astype(np.float16)
        t = rng.uniform(-1, 1, (B, dims[-1])).astype(np.float16) if case % 2 else None
        a, b = build(specs), build(specs)
        _, la = cv.mlpTrainStep(a, to_dev(x), to_dev(t) if t is not None else None)
        name = cv.lastKernelName()
        fused += "layer-by-layer" not in name
        _, lb = cv.mlpTrainStep(b, to_dev(x), to_dev(t) if t is not None else None, flags=cv.FLAG_LAYERWISE_TRAINING)
        aW, aB = read_grads(a, specs, CT.Float32, ML.RowMajor)
        bW, bB = read_grads(b, specs, CT.Float32, ML.RowMajor)
        for l in range(len(specs)):
            scaleW, scaleB = max(np.linalg.norm(bW[l]), 1e-6), max(np.linalg.norm(bB[l]), 1e-6)
            assert np.linalg.norm(aW[l] - bW[l]) <= 1e-3 * scaleW, (case, dims, B, name, l)
            assert np.linalg.norm(aB[l] - bB[l]) <= 1e-3 * scaleB, (case, dims, B, name, l)
        assert abs(la.item() - lb.item()) <= 1e-4 * max(abs(lb.item()), 1e-6), (case, dims, B, name)
    assert fused == 40


@pytest.mark.parametrize("grad_ct,grad_layout", [(CT.Float32, ML.TrainingOptimal), (CT.Float32, ML.RowMajor), (CT.Float16, ML.ColumnMajor)])
@pytest.mark.parametrize("dims,B", [([4, 16, 4], 16), ([8, 16, 16, 3], 50), ([12, 16, 16, 16, 1], 64), ([4, 16, 4], 1)])
def test_step_of_a_single_workgroup(dims, B, grad_ct, grad_layout):
    # A batch of at most four tiles (the example's 16 samples) is one workgroup of the one-wave kernel, which adds its sums
    # to the gradients itself: "+=" onto what the buffers hold, lossSum and lossMax, the same step twice gives the same
    # bits, and a sample that is not finite voids every sum of the step.
    rng = np.random.default_rng(sum(dims) * 7 + B)
    specs = make_specs(rng, dims, act=Activation.LeakyReLU, slope=float(np.float16(0.01)))
    x = rng.uniform(-1, 1, (B, dims[0])).astype(np.float16)
    t = rng.uniform(-1, 1, (B, dims[-1])).astype(np.float16)
    rW, rB, rLoss = ob.ref_mlp_train(specs, x, t, 0.5, True)
    runs = []
    for _ in range(2):
        layers = build(specs, grad_ct, grad_layout, preset=1.0)
        lmax = torch.full((1,), -1.0, dtype=torch.float32, device=DEV)
        _, loss = cv.mlpTrainStep(layers, to_dev(x), to_dev(t), lossScale=0.5, gradType=grad_ct, lossMax=lmax)
        assert cv.lastKernelName().startswith("mlpTrainKernel") and "Reduce" not in cv.lastKernelName().split("+")[0]
        dW, dB = read_grads(layers, specs, grad_ct, grad_layout)
        runs.append((loss.item(), lmax.item(), dW, dB))
    tol = 2e-3 if grad_ct == CT.Float32 else 1e-2
    loss0, lmax0, dW, dB = runs[0]
    assert loss0 == runs[1][0] and lmax0 == runs[1][1]
    for l in range(len(specs)):
        assert np.array_equal(dW[l], runs[1][2][l]) and np.array_equal(dB[l], runs[1][3][l])
        assert rel_err(dW[l], rW[l]) < tol, (l, rel_err(dW[l], rW[l]))
        assert rel_err(dB[l] - 1.0, rB[l]) < tol + (0 if grad_ct == CT.Float32 else 2e-2), (l, rel_err(dB[l] - 1.0, rB[l]))     # the preset stayed
    assert abs(loss0 - rLoss) <= 2e-3 * abs(rLoss) and 0 < lmax0 <= loss0 + 1e-6
    # not finite: everything the step adds is NaN
    x[B // 2, 1] = np.inf
    layers = build(specs, grad_ct, grad_layout, preset=1.0)
    lmax = torch.zeros(1, dtype=torch.float32, device=DEV)
    _, loss = cv.mlpTrainStep(layers, to_dev(x), to_dev(t), lossScale=0.5, gradType=grad_ct, lossMax=lmax)
    assert np.isnan(loss.item()) and np.isnan(lmax.item())
    dW, dB = read_grads(layers, specs, grad_ct, grad_layout)
    for l in range(len(specs)):
        valid = np.ones_like(dW[l], bool)
        assert np.isnan(dW[l]).all() and np.isnan(dB[l]).all()


@pytest.mark.parametrize("dims,B", [([8, 64, 64, 64, 64, 1], 4099), ([8, 32, 32, 32, 4], 1500), ([20, 64, 64, 8], 777), ([8, 48, 24, 3], 640)])
def test_leaky_relu_networks_on_the_paired_kernel(dims, B):
    # hidden layers with leaky ReLU (the example's activation, fflayer.slang:60-66), also mixed with ReLU layers: the paired
    # kernel, held against the oracle, against the one-wave kernel (taken by vectors at a 2-byte pitch), and to the tie rule
    rng = np.random.default_rng(sum(dims) * 3 + B)
    slope = float(np.float16(0.01))
    specs = make_specs(rng, dims, act=Activation.LeakyReLU, slope=slope)
    if len(specs) > 2:
        specs[1]["act"] = int(Activation.ReLU); specs[1]["slope"] = 0.0        # a ReLU layer among the leaky ones
    if B % 2:      # the example's layers all carry the activation, the last one too (fflayer.slang:60-66); or a ReLU there
        specs[-1]["act"] = int(Activation.LeakyReLU if B % 3 else Activation.ReLU); specs[-1]["slope"] = slope if B % 3 else 0.0
    x = rng.uniform(-1, 1, (B, dims[0])).astype(np.float16)
    x[5] = 0                                                                     # (pre-activations equal to the biases)
    t = rng.uniform(-1, 1, (B, dims[-1])).astype(np.float16)
    layers = build(specs)
    _, loss = cv.mlpTrainStep(layers, to_dev(x), to_dev(t), lossScale=0.25)
    assert cv.lastKernelName().startswith("mlpTrainPairKernel") and "leaky-or-relu" in cv.lastKernelName(), cv.lastKernelName()
    dW, dB = read_grads(layers, specs, CT.Float32, ML.RowMajor)
    rW, rB, rloss = ob.ref_mlp_train(specs, x, t, 0.25, tie_rule=True)
    for l in range(len(specs)):
        assert rel_err(dW[l], rW[l]) <= 1e-3, (l, rel_err(dW[l], rW[l]))
        assert rel_err(dB[l], rB[l]) <= 1e-3, (l, rel_err(dB[l], rB[l]))
    assert abs(loss.item() - rloss) <= 1e-3 * rloss
    # the same step on the one-wave kernel
    wide = torch.zeros((B, dims[0] + 1), dtype=torch.float16, device=DEV); wide[:, :dims[0]] = to_dev(x)
    other = build(specs)
    _, loss1 = cv.mlpTrainStep(other, wide[:, :dims[0]], to_dev(t), lossScale=0.25)
    assert cv.lastKernelName().startswith("mlpTrainKernel"), cv.lastKernelName()
    oW, oB = read_grads(other, specs, CT.Float32, ML.RowMajor)
    for l in range(len(specs)):
        assert rel_err(dW[l], oW[l]) <= 2e-6 and rel_err(dB[l], oB[l]) <= 2e-6, (l, rel_err(dW[l], oW[l]), rel_err(dB[l], oB[l]))
    assert abs(loss.item() - loss1.item()) <= 1e-6 * abs(loss1.item())
    # bitwise determinism
    again = build(specs)
    cv.mlpTrainStep(again, to_dev(x), to_dev(t), lossScale=0.25)
    for a, b in zip(layers, again):
        assert torch.equal(a.weightsGrad, b.weightsGrad) and torch.equal(a.biasesGrad, b.biasesGrad)


def test_leaky_tie_rule_on_the_paired_kernel():
    # a hidden unit at exactly z = 0 of a leaky layer passes (1 + slope) / 2 of the gradient (diff.meta.slang:2258-2277 on
    # max(z, z * slope)); the oracle with the tie rule switched off disagrees
    slope = 0.25
    W0 = np.zeros((32, 8), np.float16); W0[0, 0] = 1.0; W0[1, 0] = 0.5; W0[2, 0] = -1.0
    b0 = np.zeros(32, np.float16); b0[0] = -1.0; b0[1] = 0.25; b0[2] = 0.5
    W1 = np.zeros((1, 32), np.float16); W1[0, 0] = 2.0; W1[0, 1] = 1.0; W1[0, 2] = 4.0
    specs = [dict(W=W0, b=b0, act=int(Activation.LeakyReLU), slope=slope), dict(W=W1, b=None, act=0, slope=0.0)]
    B = 64
    x = np.zeros((B, 8), np.float16); x[:, 0] = 1.0             # z = [0, 0.75, -0.5, 0 ...]
    t = np.zeros((B, 1), np.float16)
    layers = build(specs)
    cv.mlpTrainStep(layers, to_dev(x), to_dev(t), lossScale=1.0 / B)
    assert cv.lastKernelName().startswith("mlpTrainPairKernel") and "leaky" in cv.lastKernelName(), cv.lastKernelName()
    dW, dB = read_grads(layers, specs, CT.Float32, ML.RowMajor)
    rW, rB, _ = ob.ref_mlp_train(specs, x, t, 1.0 / B, True)
    nW, nB, _ = ob.ref_mlp_train(specs, x, t, 1.0 / B, False)
    assert np.allclose(dB[0], rB[0], rtol=1e-3, atol=1e-6) and not np.allclose(rB[0][:1], nB[0][:1], rtol=1e-3)
    y = 0.75 + 4.0 * (-0.5 * slope)                             # the network's output
    assert abs(dB[0][0] - 2 * y * 2.0 * (1 + slope) / 2) <= 1e-2 * abs(dB[0][0])
    assert abs(dB[0][2] - 2 * y * 4.0 * slope) <= 1e-2 * abs(dB[0][2])


@pytest.mark.parametrize("last", [Activation.LeakyReLU, Activation.ReLU])
def test_activation_behind_the_last_layer_on_the_four_wave_kernel(last):
    # a 128-wide network of the example's layers (the activation behind every layer, fflayer.slang:60-66) stays fused
    rng = np.random.default_rng(130 + int(last))
    dims, B = [16, 128, 100, 8], 1500
    slope = float(np.float16(0.01))
    specs = make_specs(rng, dims, act=Activation.LeakyReLU, slope=slope)
    specs[-1]["act"] = int(last); specs[-1]["slope"] = slope if last == Activation.LeakyReLU else 0.0
    x = rng.uniform(-1, 1, (B, dims[0])).astype(np.float16)
    t = rng.uniform(-1, 1, (B, dims[-1])).astype(np.float16)
    layers = build(specs)
    _, loss = cv.mlpTrainStep(layers, to_dev(x), to_dev(t), lossScale=0.25)
    assert cv.lastKernelName().startswith("mlpTrainQuadKernel"), cv.lastKernelName()
    dW, dB = read_grads(layers, specs, CT.Float32, ML.RowMajor)
    rW, rB, rloss = ob.ref_mlp_train(specs, x, t, 0.25, tie_rule=True)
    for l in range(len(specs)):
        assert rel_err(dW[l], rW[l]) <= 1e-3 and rel_err(dB[l], rB[l]) <= 1e-3, (l, rel_err(dW[l], rW[l]), rel_err(dB[l], rB[l]))
    assert abs(loss.item() - rloss) <= 1e-3 * rloss
    # the layer-by-layer step agrees to its own bar
    general = build(specs)
    cv.mlpTrainStep(general, to_dev(x), to_dev(t), lossScale=0.25, flags=cv.FLAG_LAYERWISE_TRAINING)
    gW, gB = read_grads(general, specs, CT.Float32, ML.RowMajor)
    for l in range(len(specs)):
        assert rel_err(gW[l], dW[l]) <= 1e-3 and rel_err(gB[l], dB[l]) <= 1e-3
