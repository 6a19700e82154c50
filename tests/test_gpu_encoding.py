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


# ---- grid hashes and the permutohedral encoder ---------------------------------------------------
import json
import os

NG = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "neural_goldens.json")))


def test_grid_hash_goldens_and_random_positions():
    # integer work: bit-exact against tests/neural/hash-function-test.slang and the oracle
    pos = NG["hash"]["positions"]
    got = []
    for t in (cv.HashType.Prime, cv.HashType.CoherentPrime, cv.HashType.ReversedPrime, cv.HashType.BaseConvert, cv.HashType.Rng):
        for d in "1234":
            p = torch.tensor([pos[d]], dtype=torch.int32, device=DEV)
            got.append(int(cv.gridHash(t, p).cpu().numpy().view(np.uint32)[0]))
    p3 = torch.tensor([pos["3"]], dtype=torch.int32, device=DEV)
    got.append(int(cv.gridHash(cv.HashType.Prime, p3).cpu().numpy().view(np.uint32)[0]))
    got.append(int(cv.gridHash(cv.HashType.BaseConvert, p3).cpu().numpy().view(np.uint32)[0]))
    assert got == NG["hash"]["expected"]
    rng = np.random.default_rng(1)
    for dims in (1, 2, 3, 5, 7):
        grid = rng.integers(0, 2 ** 32, (3000, dims), dtype=np.uint64).astype(np.uint32)
        gd = to_dev(grid.view(np.int32))
        for t in range(5):
            want = np.array([ob.grid_hash(t, row) for row in grid[:300]], np.uint32)
            assert np.array_equal(cv.gridHash(t, gd).cpu().numpy().view(np.uint32)[:300], want), (t, dims)


def _reference_setup():
    from test_oracle_encoders import reference_setup
    return reference_setup()


def test_permuto_encoder_reference_data():
    # tests/neural/permuto-encoder-test.slang and -backward: the reference's expected values, to its epsilon
    P = NG["permuto"]; cfg = P["config"]
    pos, table, levels, max_level = _reference_setup()
    enc = cv.PermutoEncoder(2, 2, 8, 4, baseScale=cfg["baseScale"], log2PerLevelScale=cfg["log2PerLevelScale"],
                            maxLevelRatio=cfg["maxLevelRatio"], seed=cfg["seed"])
    out = enc.encode(to_dev(pos), to_dev(table)).cpu().numpy()
    want = np.array(P["expectedForward"]).reshape(16, 8)
    assert np.abs(out[P["verifyPositions"]] - want).max() <= cfg["epsilon"]
    assert np.array_equal(out, ob.permuto_encode(levels, 2, max_level, pos, table))      # same fp32 operations, same order
    d_pos, d_table = enc.backward(to_dev(pos), to_dev(table), torch.ones(256, 8, device=DEV))
    want_pos = np.array(P["expectedDLdPos"]).reshape(16, 2)
    got_pos = d_pos.cpu().numpy()[P["verifyPositions"]]
    assert (np.abs(got_pos - want_pos) <= cfg["epsilon"] + 1e-5 * np.abs(want_pos)).all()
    assert np.abs(d_table.cpu().numpy()[P["verifyParamIndices"]] - np.array(P["expectedDLdParams"])).max() <= cfg["epsilon"]


@pytest.mark.parametrize("D,F,levels_n", [(1, 1, 3), (3, 4, 6), (4, 2, 8), (6, 8, 2), (8, 2, 4)])
def test_permuto_encoder_against_oracle(D, F, levels_n):
    rng = np.random.default_rng(D * 100 + F)
    log2 = 10
    enc = cv.PermutoEncoder(D, F, log2, levels_n, baseScale=2.0, log2PerLevelScale=0.8, maxLevelRatio=0.8, seed=7)
    levels = ob.permuto_levels(D, log2, levels_n, 2.0, 0.8, 7)
    max_level = float(np.float32(0.8) * np.float32(levels_n))
    B = 5000
    pos = rng.uniform(0, 1, (B, D)).astype(np.float32)
    table = rng.standard_normal(enc.featureTableElements).astype(np.float32)
    out = enc.encode(to_dev(pos), to_dev(table)).cpu().numpy()
    assert np.array_equal(out, ob.permuto_encode(levels, F, max_level, pos, table))
    g = rng.standard_normal((B, levels_n * F)).astype(np.float32)
    d_pos, d_table = enc.backward(to_dev(pos), to_dev(table), to_dev(g))
    r_pos, r_table = ob.permuto_encode_backward(levels, F, max_level, pos, table, g)
    assert np.linalg.norm(d_pos.cpu().numpy() - r_pos) <= 1e-4 * np.linalg.norm(r_pos)
    assert np.linalg.norm(d_table.cpu().numpy() - r_table) <= 1e-4 * np.linalg.norm(r_table)
    # fp16 data: every product and sum rounded to half, as the generic T of the reference does
    enc16 = cv.PermutoEncoder(D, F, log2, levels_n, baseScale=2.0, log2PerLevelScale=0.8, maxLevelRatio=0.8, seed=7, dtype=torch.float16)
    p16, t16 = pos.astype(np.float16), table.astype(np.float16)
    o16 = enc16.encode(to_dev(p16), to_dev(t16)).cpu().numpy()
    assert np.array_equal(o16, ob.permuto_encode(levels, F, max_level, p16, t16))


@pytest.mark.parametrize("D,F,levels_n,log2", [(2, 2, 5, 8), (3, 8, 3, 6), (4, 1, 7, 12), (2, 4, 16, 4), (3, 2, 8, 14), (5, 4, 2, 9)])
def test_permuto_encoder_kernel_choices(D, F, levels_n, log2):
    # one thread per (position, level) with the table in LDS or in memory, level counts that are no power of two,
    # positions outside the unit cube, output rows at a pitch, and the one-thread-per-position kernel for what the
    # other does not take (more than four dimensions, entries over 16 bytes, unaligned buffers): all bit for bit the oracle
    rng = np.random.default_rng(D * 1000 + F * 10 + levels_n)
    levels = ob.permuto_levels(D, log2, levels_n, 1.5, 0.7, 99)
    max_level = float(np.float32(1.1) * np.float32(levels_n))
    B = 3001
    pos = rng.uniform(-4, 4, (B, D)).astype(np.float32)
    for dt, npdt in ((torch.float32, np.float32), (torch.float16, np.float16)):
        enc = cv.PermutoEncoder(D, F, log2, levels_n, baseScale=1.5, log2PerLevelScale=0.7, maxLevelRatio=1.1, seed=99, dtype=dt)
        p, t = pos.astype(npdt), rng.standard_normal(enc.featureTableElements).astype(npdt)
        want = ob.permuto_encode(levels, F, max_level, p, t)
        out = enc.encode(to_dev(p), to_dev(t))
        name = cv.lastKernelName()
        pairs = D <= 4 and F * np.dtype(npdt).itemsize <= 16
        assert name.startswith("permutoEncodePairsKernel" if pairs else "permutoEncodeKernel"), name
        assert np.array_equal(out.cpu().numpy(), want)
        # rows at a pitch of one extra entry; then a table that starts one element into its allocation
        wide = torch.zeros(B, levels_n * F + F, dtype=dt, device=DEV)
        enc.encode(to_dev(p), to_dev(t), out=wide[:, :levels_n * F])
        assert np.array_equal(wide[:, :levels_n * F].cpu().numpy(), want) and not wide[:, levels_n * F:].any()
        shifted = torch.zeros(t.size + 1, dtype=dt, device=DEV)
        shifted[1:] = to_dev(t)
        out2 = enc.encode(to_dev(p), shifted[1:])
        assert np.array_equal(out2.cpu().numpy(), want)
        if F > 1:
            assert cv.lastKernelName().startswith("permutoEncodeKernel"), cv.lastKernelName()


def test_encoder_feeds_the_mlp():
    # encode positions, run the decoder MLP on the fp16 features: the neural-texture shape
    rng = np.random.default_rng(8)
    enc = cv.PermutoEncoder(3, 2, 12, 8, baseScale=4.0, log2PerLevelScale=1.0, dtype=torch.float16)
    B = 4096
    pos = to_dev(rng.uniform(0, 1, (B, 3)).astype(np.float16))
    table = to_dev((rng.standard_normal(enc.featureTableElements) * 0.5).astype(np.float16))
    feats = enc.encode(pos, table)
    specs = make_specs(rng, [16, 64, 64, 3])
    layers = build(specs)
    y = cv.mlpForward(layers, feats)
    ref = ob.ref_mlp_forward(specs, feats.cpu().numpy(), ob.F16)
    assert (np.abs(y.cpu().numpy().astype(np.float32) - ref.astype(np.float32)) <= 2e-2 * np.abs(ref.astype(np.float32)) + 2e-2).mean() > 0.999


@pytest.mark.parametrize("D,F,levels_n,log2,dims,B,kernel", [
    (3, 2, 8, 12, [16, 64, 64, 3], 4099, "permutoWide16Kernel"),     # the neural-texture shape; table (128 KB) and network in LDS
    (2, 2, 16, 8, [32, 32, 4], 777, "permutoWide16Kernel"),
    (4, 2, 8, 10, [16, 64, 8], 64, "permutoWide16Kernel"),
    (3, 2, 16, 11, [32, 64, 64, 1], 3000, "permutoWide16Kernel"),
    (2, 4, 4, 8, [16, 32, 5], 17, "permutoMlpKernel"),               # four features per entry
    (4, 1, 12, 10, [12, 128, 128, 7], 1000, "permutoMlpKernel"),     # 128-wide layers; a first layer narrower than its 16-column tile
    (3, 2, 8, 15, [16, 64, 64, 3], 2500, "permutoMlpKernel"),        # a 1 MB table stays in memory
    (1, 2, 16, 6, [32, 48, 16, 1], 1, "permutoMlpKernel"),
])
def test_encoder_and_network_in_one_kernel(D, F, levels_n, log2, dims, B, kernel):
    # cvPermutoMlpForward == cvPermutoEncode followed by cvMlpForward, bit for bit, on the 32-sample-tile kernel where the
    # decoder allows it and on the run-time-size kernel otherwise (or when asked for)
    rng = np.random.default_rng(D * 100 + F * 10 + len(dims))
    enc = cv.PermutoEncoder(D, F, log2, levels_n, baseScale=2.0, log2PerLevelScale=0.9, maxLevelRatio=0.9, seed=5, dtype=torch.float16)
    pos = to_dev(rng.uniform(-1, 2, (B, D)).astype(np.float16))
    table = to_dev((rng.standard_normal(enc.featureTableElements) * 0.5).astype(np.float16))
    specs = make_specs(rng, dims)
    if kernel == "permutoMlpKernel":
        specs[0]["act"], specs[0]["slope"] = 2, float(np.float16(0.01))      # a leaky layer among the ReLU ones
    layers = build(specs)
    feats = enc.encode(pos, table)
    want = cv.mlpForward(layers, feats)
    got = enc.encodeAndEval(pos, table, layers)
    name = cv.lastKernelName()
    assert name.startswith(kernel + "<D=%d,F=%d" % (D, F)), name
    if kernel == "permutoMlpKernel":
        assert name.endswith("memory>" if log2 == 15 else "LDS>"), name
    assert torch.equal(got, want)
    got16 = enc.encodeAndEval(pos, table, layers, flags=cv.FLAG_FORWARD_TILE16)
    assert cv.lastKernelName().startswith("permutoMlpKernel"), cv.lastKernelName()
    assert torch.equal(got16, want)
    levels = ob.permuto_levels(D, log2, levels_n, 2.0, 0.9, 5)
    max_level = float(np.float32(0.9) * np.float32(levels_n))
    f_ref = ob.permuto_encode(levels, F, max_level, pos.cpu().numpy(), table.cpu().numpy())
    assert np.array_equal(feats.cpu().numpy(), f_ref)
    # rows of the result at a pitch
    wide = torch.full((B, dims[-1] + 3), 7.0, dtype=torch.float16, device=DEV)
    enc.encodeAndEval(pos, table, layers, out=wide[:, :dims[-1]])
    assert torch.equal(wide[:, :dims[-1]], want) and bool((wide[:, dims[-1]:] == 7.0).all())


def test_encoder_and_network_argument_checks():
    rng = np.random.default_rng(3)
    enc = cv.PermutoEncoder(3, 2, 8, 4, baseScale=1.0, log2PerLevelScale=1.0, dtype=torch.float16)
    pos = to_dev(rng.uniform(0, 1, (8, 3)).astype(np.float16))
    table = to_dev(rng.standard_normal(enc.featureTableElements).astype(np.float16))
    with pytest.raises(cv.CoopVecError) as e:          # first layer does not match the encoder's output
        enc.encodeAndEval(pos, table, build(make_specs(rng, [16, 32, 4])))
    assert e.value.result == cv.SLANG_E_INVALID_ARG
    with pytest.raises(cv.CoopVecError) as e:          # a single layer is not a network
        enc.encodeAndEval(pos, table, build(make_specs(rng, [8, 4])))
    assert e.value.result == cv.SLANG_E_NOT_AVAILABLE
    enc5 = cv.PermutoEncoder(5, 2, 8, 4, baseScale=1.0, log2PerLevelScale=1.0, dtype=torch.float16)
    with pytest.raises(cv.CoopVecError) as e:          # five dimensions: the two-call form
        enc5.encodeAndEval(to_dev(rng.uniform(0, 1, (8, 5)).astype(np.float16)),
                           to_dev(rng.standard_normal(enc5.featureTableElements).astype(np.float16)), build(make_specs(rng, [8, 16, 4])))
    assert e.value.result == cv.SLANG_E_NOT_AVAILABLE
