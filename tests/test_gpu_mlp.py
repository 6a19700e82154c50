"""GPU parity of the fused forward MLP against the CPU oracle, through the C-ABI.

Three checks per network:
  (1) chain rule of parity: the fused kernel equals, bit for bit, the chain of single-layer GPU
      operators (each of which is held to the float bar against the oracle in test_gpu_matmul.py);
  (2) end to end against the oracle that applies the same rounding points (fp32 accumulate ->
      fp16 -> activation -> [e4m3 re-quantisation]): max(2 ulp-fp16, 1e-3 relative) on the final
      fp16, with the propagated summation-order floor 2^-18 * sum|terms| of the last layer;
  (3) every sample outside that bar is explained: at the first layer where the GPU's carrier differs
      from the oracle's (their inputs to that layer are identical), each differing hidden unit's sum,
      recomputed in fp64, lies within the summation-order floor of a point where rounding to fp16
      changes its result -- the two sides rounded a boundary case differently and the later layers
      amplified it.  A sample that violates the bar without such a unit fails the test.
"""
import numpy as np
import pytest
import torch

import oracle_binding as ob
from gpu_util import DEV, as_bytes, matrix_in_layout, to_dev
from slang_amd import coopvec as cv
from slang_amd.coopvec import Activation, CoopVecComponentType as CT, CoopVecMatrixLayout as ML, FeedForwardLayer

pytestmark = pytest.mark.gpu


def make_net(rng, dims, wtype, act=Activation.ReLU, slope=0.0, bias="zero", init="fan_in"):
    specs = []
    for i in range(len(dims) - 1):
        fan_in, out = dims[i], dims[i + 1]
        std = np.sqrt(2.0 / fan_in) if init == "he" else (0.5 if init == "half" else np.sqrt(1.0 / fan_in))
        Wf = rng.standard_normal((out, fan_in)) * std
        W = Wf.astype(np.float16) if wtype == CT.Float16 else ob.encode_e4m3(Wf)
        if bias == "zero":
            b = np.zeros(out, np.float16)
        elif bias == "none":
            b = None
        else:
            b = rng.uniform(-0.1, 0.1, out).astype(np.float16)
        last = i == len(dims) - 2
        specs.append(dict(W=W, b=b, act=int(Activation.NoActivation if last else act), slope=slope))
    return specs


def gpu_layers(specs, wtype, layout):
    layers = []
    for s in specs:
        out, fan_in = s["W"].shape
        wb = to_dev(matrix_in_layout(s["W"], wtype, layout))
        esz = s["W"].dtype.itemsize
        layers.append(FeedForwardLayer(fan_in, out, wb, as_bytes(to_dev(s["b"])) if s["b"] is not None else None,
                                       layout, fan_in * esz if layout == ML.RowMajor else 0,
                                       s["act"], s["slope"]))
    return layers


def chain_of_single_layers(specs, x_dev, wtype, flags=0, hidden=None):
    """The same network as separate coopVecMatMulAdd launches; fp16 between layers, re-quantised
    to e4m3 on the host side of each launch for e4m3 networks.  `hidden` (a list) receives every
    layer's fp16 output."""
    h = x_dev
    for s in specs:
        out, fan_in = s["W"].shape
        wb = as_bytes(to_dev(s["W"]))
        esz = s["W"].dtype.itemsize
        if wtype == CT.FloatE4M3 and h.dtype == torch.float16:
            h = h.float().clamp(-448, 448).to(torch.float8_e4m3fn)
        args = (h, wtype, wb, 0, wtype)
        kw = dict(M=out, activation=s["act"], leakySlope=s["slope"], flags=flags)
        if s["b"] is not None:
            h = cv.coopVecMatMulAdd(*args, as_bytes(to_dev(s["b"])), 0, CT.Float16, ML.RowMajor, False, fan_in * esz, **kw)
        else:
            bz = torch.zeros(out, dtype=torch.float16, device=DEV).view(torch.uint8)
            h = cv.coopVecMatMulAdd(*args, bz, 0, CT.Float16, ML.RowMajor, False, fan_in * esz, **kw)
        if hidden is not None:
            hidden.append(h.cpu().numpy())
    return h


def _weights_f64(s):
    W = s["W"]
    return W.astype(np.float64) if W.dtype == np.float16 else ob.decode_e4m3(W).astype(np.float64)


def end_to_end_ok(y, specs, x, x_ct, gpu_hidden, floor=2.0 ** -18):
    """Fraction of outputs inside the bar; asserts that every sample outside it is a rounding-boundary
    case of a hidden unit (check (3) of the module docstring).  `floor` is the accumulation floor of
    the pipeline that produced `gpu_hidden`, relative to sum|terms|."""
    ref, acts = ob.ref_mlp_forward(specs, x, x_ct, want_acts=True)
    # floor from the last layer's terms: |W| . |a_prev|
    prev = acts[-2].astype(np.float32) if len(acts) > 1 else None
    Wl = np.abs(_weights_f64(specs[-1])).astype(np.float32)
    ab = np.abs(prev) @ Wl.T
    bad = ob.float_parity_violations(y, ref.astype(np.float32), ab, floor)
    e4m3 = specs[0]["W"].dtype != np.float16
    x64 = x.astype(np.float64) if x_ct == ob.F16 else ob.decode_e4m3(x).astype(np.float64)
    for s in np.nonzero(bad.any(axis=1))[0]:
        first = None
        for l in range(len(specs) - 1):
            if not np.array_equal(gpu_hidden[l][s].astype(np.float32), acts[l][s].astype(np.float32)):
                first = l
                break
        assert first is not None, "sample %d violates the bar although every hidden carrier equals the oracle's" % s
        src = x64[s] if first == 0 else acts[first - 1][s].astype(np.float64)
        if e4m3 and first > 0:      # the carrier is re-quantised in front of the layer
            src = ob.decode_e4m3(ob.encode_e4m3(src)).astype(np.float64)
        W = _weights_f64(specs[first])
        b = specs[first]["b"]
        z = W @ src + (b.astype(np.float64) if b is not None else 0.0)
        terms = np.abs(W) @ np.abs(src) + (np.abs(b.astype(np.float64)) if b is not None else 0.0)
        units = np.nonzero(gpu_hidden[first][s].astype(np.float32) != acts[first][s].astype(np.float32))[0]
        dist = ob.f16_midpoint_distance(z[units])
        assert (dist <= floor * terms[units] + 2.0 ** -30).all(), \
            "sample %d layer %d: hidden units %s differ from the oracle away from a rounding boundary" % (s, first, units)
        # and the two sides are neighbours in fp16
        d = np.abs(gpu_hidden[first][s][units].astype(np.float32) - acts[first][s][units].astype(np.float32))
        assert (d <= ob.f16_ulp(acts[first][s][units].astype(np.float32)) * (1.0 if floor <= 2.0 ** -17 else 64.0)).all()
    ob.note_end_to_end(bad.sum(), bad.size)
    return 1.0 - bad.mean(), bad


@pytest.mark.parametrize("layout", [ML.RowMajor, ML.InferencingOptimal])
def test_small_fp16_mlp_config(layout):
    # 2 -> 16 -> 16 -> 16 -> 1, ReLU on hidden layers, batch 65536, inputs U[0,1)^2,
    # weights N(0, 1/fan_in) as fp16, zero biases
    rng = np.random.default_rng(2024)
    dims = [2, 16, 16, 16, 1]
    B = 65536
    specs = make_net(rng, dims, CT.Float16)
    x = rng.uniform(0, 1, (B, 2)).astype(np.float16)
    xd = to_dev(x)
    y = cv.mlpForward(gpu_layers(specs, CT.Float16, layout), xd)
    assert y.shape == (B, 1)
    hid = []
    yc = chain_of_single_layers(specs, xd, CT.Float16, hidden=hid)
    assert torch.equal(y.view(torch.int16), yc.view(torch.int16))
    frac, bad = end_to_end_ok(y.cpu().numpy(), specs, x, ob.F16, hid)
    assert frac >= 0.999, "only %.5f within tolerance" % frac


def test_example_network_leaky_relu():
    # the example's 4 -> 16 -> 4 with max(z, 0.001 z) after *every* layer (fflayer.slang:60-66),
    # parameters U[-1,1], inputs (x, y, x^2, y^2) (network.slang:35-38)
    rng = np.random.default_rng(1072)
    slope = float(np.float16(0.001))
    specs = []
    for fan_in, out in ((4, 16), (16, 4)):
        specs.append(dict(W=rng.uniform(-1, 1, (out, fan_in)).astype(np.float16),
                          b=rng.uniform(-1, 1, out).astype(np.float16), act=int(Activation.LeakyReLU), slope=slope))
    B = 1000
    xy = rng.uniform(0, 1, (B, 2)).astype(np.float16)
    x = np.concatenate([xy, (xy.astype(np.float32) ** 2).astype(np.float16)], axis=1)
    xd = to_dev(x)
    y = cv.mlpForward(gpu_layers(specs, CT.Float16, ML.RowMajor), xd)
    hid = []
    yc = chain_of_single_layers(specs, xd, CT.Float16, hidden=hid)
    assert torch.equal(y.view(torch.int16), yc.view(torch.int16))
    frac, _ = end_to_end_ok(y.cpu().numpy(), specs, x, ob.F16, hid)
    assert frac >= 0.999


@pytest.mark.parametrize("dims", [[8, 64, 64, 64, 64, 1], [32, 64, 64, 8], [64, 64, 64, 64], [5, 30, 30, 3],
                                  [40, 64, 64, 64], [16, 32, 32, 32, 20], [3, 60, 7]])
def test_fp16_mlp_shapes(dims):
    rng = np.random.default_rng(sum(dims))
    B = 2000 + 13
    specs = make_net(rng, dims, CT.Float16, bias="rand", init="he")
    x = rng.uniform(-1, 1, (B, dims[0])).astype(np.float16)
    xd = to_dev(x)
    y = cv.mlpForward(gpu_layers(specs, CT.Float16, ML.InferencingOptimal), xd)
    hid = []
    yc = chain_of_single_layers(specs, xd, CT.Float16, hidden=hid)
    assert torch.equal(y.view(torch.int16), yc.view(torch.int16))
    frac, _ = end_to_end_ok(y.cpu().numpy(), specs, x, ob.F16, hid)
    assert frac >= 0.999


@pytest.mark.parametrize("flags", [0, cv.FLAG_FP8_MATRIX_PIPELINE])
def test_e4m3_decoder_config(flags):
    # 32 -> 64 -> 64 -> 8, weights and inputs 0.5*N(0,1) saturate-cast to e4m3, activations
    # fp16 -> ReLU -> e4m3, fp16 output (a 2^16 slice of the 2^24 batch)
    rng = np.random.default_rng(4096)
    dims = [32, 64, 64, 8]
    B = 1 << 16
    specs = make_net(rng, dims, CT.FloatE4M3, bias="none", init="half")
    x = ob.encode_e4m3(rng.standard_normal((B, 32)) * 0.5)
    xd = to_dev(x)
    for layout in (ML.RowMajor, ML.InferencingOptimal):
        y = cv.mlpForward(gpu_layers(specs, CT.FloatE4M3, layout), xd, weightType=CT.FloatE4M3, flags=flags)
        hid = []
        yc = chain_of_single_layers(specs, xd, CT.FloatE4M3, flags, hidden=hid)
        assert torch.equal(y.view(torch.int16), yc.view(torch.int16))
    # the fp8 matrix pipeline's documented accumulation floor is 2^-12 * sum|terms| per layer
    frac, bad = end_to_end_ok(y.cpu().numpy(), specs, x, ob.E4M3, hid, floor=2.0 ** -18 if flags == 0 else 2.0 ** -12)
    if flags == 0:
        # fp32-grade accumulation: the oracle's bar
        assert frac >= 0.999, "only %.5f within tolerance" % frac
    else:
        # fp8 matrix pipeline: products far below the largest one of an instruction are truncated,
        # which moves some hidden units across an e4m3 rounding boundary; report, and require the
        # bulk to agree
        assert frac >= 0.80, "only %.5f within tolerance" % frac


@pytest.mark.parametrize("flags", [0, cv.FLAG_FP8_MATRIX_PIPELINE])
@pytest.mark.parametrize("B", [4096, 50])       # streaming kernel / tail path
def test_e4m3_saturation_and_fp16_overflow(flags, B):
    # hidden sums beyond +-448 saturate when the carrier is re-quantised (also through an fp16
    # overflow: inf -> 448), while an overflow of the network's own fp16 output stays inf
    rng = np.random.default_rng(448)
    dims = [32, 64, 64, 8]
    specs = make_net(rng, dims, CT.FloatE4M3, act=Activation.NoActivation, bias="none", init="half")
    for s in specs[:-1]:
        s["act"] = int(Activation.NoActivation)
    specs[0]["W"][:8] = ob.encode_e4m3(np.full((8, 32), 448.0))         # rows that overflow fp16 (+)
    specs[0]["W"][8:16] = ob.encode_e4m3(np.full((8, 32), -448.0))      # ... and (-)
    specs[0]["W"][16:24] = ob.encode_e4m3(np.full((8, 32), 2.0))        # beyond 448, within fp16
    specs[2]["W"][0] = ob.encode_e4m3(np.full(64, 448.0))               # output row that can overflow fp16
    xf = rng.standard_normal((B, 32)) * 0.5
    xf[::3] = 448.0
    xf[1::7] = -448.0
    x = ob.encode_e4m3(xf)
    xd = to_dev(x)
    y = cv.mlpForward(gpu_layers(specs, CT.FloatE4M3, ML.InferencingOptimal), xd, weightType=CT.FloatE4M3, flags=flags)
    hid = []
    yc = chain_of_single_layers(specs, xd, CT.FloatE4M3, flags, hidden=hid)
    assert torch.equal(y.view(torch.int16), yc.view(torch.int16))
    ref, acts = ob.ref_mlp_forward(specs, x, ob.E4M3, want_acts=True)
    got = y.cpu().numpy()
    assert np.isinf(ref).any() and np.isinf(acts[0]).any()              # the case is exercised
    assert np.array_equal(np.isinf(got), np.isinf(ref))
    assert np.array_equal(got[np.isinf(ref)], ref[np.isinf(ref)])       # same sign of inf
    if flags == 0:
        fin = np.isfinite(ref)
        bad = ob.float_parity_violations(got[fin], ref[fin].astype(np.float32),
                                         (np.abs(acts[1].astype(np.float32)) @ np.abs(ob.decode_e4m3(specs[2]["W"])).T)[fin])
        assert bad.mean() <= 1e-3


@pytest.mark.parametrize("dims,B", [([32, 64, 64, 8], 4096), ([32, 64, 64, 8], 77), ([20, 48, 24, 5], 300), ([64, 64, 64, 64], 1000)])
@pytest.mark.parametrize("flags", [0, cv.FLAG_FP8_MATRIX_PIPELINE])
def test_e4m3_network_with_fp16_vectors(dims, B, flags):
    # CoopVec<half> + inputInterpretation FloatE4M3: the vectors are quantised (saturating, nearest
    # even) as they are loaded, so the result is bit for bit that of the pre-quantised bytes
    rng = np.random.default_rng(sum(dims) + B)
    specs = make_net(rng, dims, CT.FloatE4M3, bias="none", init="half")
    xh = (rng.standard_normal((B, dims[0])) * 0.7).astype(np.float16)
    xh[0, :6] = [1000.0, -1000.0, 464.0, -480.0, 2.0 ** -10, -0.0]
    xq = ob.encode_e4m3(xh.astype(np.float32))          # the oracle's quantiser
    for layout in (ML.RowMajor, ML.InferencingOptimal):
        layers = gpu_layers(specs, CT.FloatE4M3, layout)
        y_bytes = cv.mlpForward(layers, to_dev(xq), weightType=CT.FloatE4M3, flags=flags)
        y_half = cv.mlpForward(layers, to_dev(xh), weightType=CT.FloatE4M3, flags=flags)
        assert torch.equal(y_half.view(torch.int16), y_bytes.view(torch.int16)), cv.lastKernelName()
    # strided fp16 vectors (the element-wise load path)
    wide = torch.zeros((B, dims[0] + 3), dtype=torch.float16, device=DEV)
    wide[:, :dims[0]] = to_dev(xh)
    y_str = cv.mlpForward(layers, wide[:, :dims[0]], weightType=CT.FloatE4M3, flags=flags)
    assert torch.equal(y_str.view(torch.int16), y_bytes.view(torch.int16))


@pytest.mark.parametrize("dims,B", [([32, 64, 8], 4097), ([32, 64, 64, 8], 100003), ([32, 64, 64, 64, 8], 2048),
                                    ([32, 32, 8], 33), ([32, 32, 32, 32, 4], 1000), ([32, 64, 64, 16], 777),
                                    ([32, 64, 64, 32], 1501), ([32, 64, 12], 64), ([32, 64, 64, 8], 1), ([32, 64, 64, 8], 31)])
@pytest.mark.parametrize("last_relu", [False, True])
def test_e4m3_networks_on_32_sample_tiles(dims, B, last_relu):
    # e4m3 networks with 32-byte input rows and ReLU hidden layers of 32 or 64 units run on 32-sample
    # tiles (v_mfma_f32_32x32x16_f16, rows loaded straight in operand order, tiles drawn from a counter):
    # same bits as the chain of single-layer operators for every depth, output width, layout and ragged batch
    rng = np.random.default_rng(sum(dims) * 7 + B)
    specs = make_net(rng, dims, CT.FloatE4M3, bias="none", init="half")
    if last_relu:
        specs[-1]["act"] = int(Activation.ReLU)
    x = ob.encode_e4m3(rng.standard_normal((B, 32)) * 0.5)
    xd = to_dev(x)
    hid = []
    yc = chain_of_single_layers(specs, xd, CT.FloatE4M3, hidden=hid)
    for layout in (ML.RowMajor, ML.ColumnMajor, ML.InferencingOptimal):
        y = cv.mlpForward(gpu_layers(specs, CT.FloatE4M3, layout), xd, weightType=CT.FloatE4M3)
        assert cv.lastKernelName().startswith("mlpWideKernel"), cv.lastKernelName()
        assert torch.equal(y.view(torch.int16), yc.view(torch.int16)), layout
    frac, _ = end_to_end_ok(y.cpu().numpy(), specs, x, ob.E4M3, hid)
    assert frac >= 0.99
    # a padded output buffer: rows at a stride, nothing written between them
    wide = torch.full((B, dims[-1] + 4), -7.0, dtype=torch.float16, device=DEV)
    cv.mlpForward(gpu_layers(specs, CT.FloatE4M3, ML.RowMajor), xd, weightType=CT.FloatE4M3, out=wide[:, :dims[-1]])
    assert torch.equal(wide[:, :dims[-1]].contiguous().view(torch.int16), yc.view(torch.int16))
    assert (wide[:, dims[-1]:] == -7.0).all()


@pytest.mark.parametrize("dims,B", [([32, 64, 64, 8], 5000), ([32, 64, 8], 33), ([32, 32, 32, 4], 1), ([32, 64, 64, 64, 8], 700),
                                    ([32, 64, 64, 32], 257)])
def test_fp16_vectors_on_32_sample_tiles(dims, B):
    # CoopVec<half> + inputInterpretation FloatE4M3 on the 32-sample kernel: rows of 64 bytes, quantised
    # (saturating, nearest even) after they are split between the lane halves; bit for bit the result of
    # pre-quantised bytes, which in turn equals the chain of single-layer operators
    rng = np.random.default_rng(sum(dims) + B)
    specs = make_net(rng, dims, CT.FloatE4M3, bias="none", init="half")
    xh = (rng.standard_normal((B, 32)) * 0.7).astype(np.float16)
    xh[0, :8] = [1000.0, -1000.0, 464.0, -480.0, 2.0 ** -10, -0.0, 65504.0, np.inf]
    xq = ob.encode_e4m3(np.clip(xh.astype(np.float32), -448.0, 448.0))
    layers = gpu_layers(specs, CT.FloatE4M3, ML.InferencingOptimal)
    y_bytes = cv.mlpForward(layers, to_dev(xq), weightType=CT.FloatE4M3)
    y_half = cv.mlpForward(layers, to_dev(xh), weightType=CT.FloatE4M3)
    assert cv.lastKernelName().startswith("mlpWideKernel") and "fp16-vectors" in cv.lastKernelName(), cv.lastKernelName()
    assert torch.equal(y_half.view(torch.int16), y_bytes.view(torch.int16))
    yc = chain_of_single_layers(specs, to_dev(xq), CT.FloatE4M3)
    assert torch.equal(y_half.view(torch.int16), yc.view(torch.int16))


@pytest.mark.parametrize("dims,B", [([32, 64, 64, 8], 3000), ([32, 64, 16], 65), ([32, 32, 32, 32, 8], 500), ([32, 64, 64, 64, 32], 129)])
@pytest.mark.parametrize("fp16_vectors", [False, True])
def test_biases_on_32_sample_tiles(dims, B, fp16_vectors):
    # biases enter the 32-sample kernel as one more k-step (bias x 1.0 into zeroed accumulators), which
    # leaves float(bias) where the 16-sample kernels seed their accumulators: same bits as the chain.
    # One layer has no bias (a null pointer next to layers that have one).
    rng = np.random.default_rng(sum(dims) + 3 * B)
    specs = make_net(rng, dims, CT.FloatE4M3, bias="rand", init="half")
    specs[1]["b"] = None
    x = ob.encode_e4m3(rng.standard_normal((B, 32)) * 0.5)
    xd = to_dev(x)
    xin = to_dev(ob.decode_e4m3(x).astype(np.float16)) if fp16_vectors else xd
    hid = []
    yc = chain_of_single_layers(specs, xd, CT.FloatE4M3, hidden=hid)
    for layout in (ML.RowMajor, ML.InferencingOptimal):
        y = cv.mlpForward(gpu_layers(specs, CT.FloatE4M3, layout), xin, weightType=CT.FloatE4M3)
        name = cv.lastKernelName()
        assert name.startswith("mlpWideKernel") and ",bias" in name and ("fp16-vectors" in name) == fp16_vectors, name
        assert torch.equal(y.view(torch.int16), yc.view(torch.int16)), layout
    frac, _ = end_to_end_ok(y.cpu().numpy(), specs, x, ob.E4M3, hid)
    assert frac >= 0.99


@pytest.mark.parametrize("dims,B", [([8, 64, 64, 64, 64, 1], 100003), ([8, 64, 64, 64, 64, 1], 1), ([8, 64, 1], 63), ([8, 32, 32, 3], 65),
                                    ([16, 64, 64, 8], 4097), ([16, 32, 32, 32, 32, 20], 1000), ([16, 64, 32], 31),
                                    ([32, 64, 64, 64, 8], 5000), ([32, 64, 64, 64, 16], 129), ([32, 32, 32, 32, 7], 33), ([32, 64, 64, 64, 64, 4], 2049),
                                    ([16, 64, 64, 64, 2], 70001)])
@pytest.mark.parametrize("bias", ["rand", "none"])
def test_fp16_networks_on_32_sample_tiles(dims, B, bias):
    # fp16 networks with 8, 16 or 32 inputs in contiguous rows and ReLU hidden layers of 32 or 64 units run on
    # 32-sample tiles (v_mfma_f32_32x32x16_f16, all weights in registers, biases as the C operand of a layer's first
    # matrix instruction): same bits as the chain of single-layer operators and as the kernels on 16-sample tiles, for
    # every depth, output width, weight layout and ragged batch; one layer without a bias next to layers that have one
    rng = np.random.default_rng(sum(dims) * 11 + B)
    specs = make_net(rng, dims, CT.Float16, bias=bias, init="he")
    if bias == "rand" and len(specs) > 2:
        specs[1]["b"] = None
    x = rng.uniform(-1, 1, (B, dims[0])).astype(np.float16)
    xd = to_dev(x)
    hid = []
    yc = chain_of_single_layers(specs, xd, CT.Float16, hidden=hid)
    for layout in (ML.RowMajor, ML.ColumnMajor, ML.InferencingOptimal):
        y = cv.mlpForward(gpu_layers(specs, CT.Float16, layout), xd)
        name = cv.lastKernelName()
        assert name.startswith("mlpWide16Kernel") and ((",bias" in name) == (bias == "rand")), name
        assert torch.equal(y.view(torch.int16), yc.view(torch.int16)), layout
    y16 = cv.mlpForward(gpu_layers(specs, CT.Float16, ML.RowMajor), xd, flags=cv.FLAG_FORWARD_TILE16)
    assert not cv.lastKernelName().startswith("mlpWide16Kernel"), cv.lastKernelName()
    assert torch.equal(y16.view(torch.int16), yc.view(torch.int16))
    frac, _ = end_to_end_ok(y.cpu().numpy(), specs, x, ob.F16, hid)      # (every outlier is checked to be a boundary case)
    assert frac >= 0.99
    # a ReLU behind the last layer, and a padded output buffer: rows at a stride, nothing written between them
    specs[-1]["act"] = int(Activation.ReLU)
    wide = torch.full((B, dims[-1] + 3), -7.0, dtype=torch.float16, device=DEV)
    cv.mlpForward(gpu_layers(specs, CT.Float16, ML.RowMajor), xd, out=wide[:, :dims[-1]])
    assert cv.lastKernelName().startswith("mlpWide16Kernel"), cv.lastKernelName()
    assert torch.equal(wide[:, :dims[-1]].contiguous().view(torch.int16), torch.clamp_min(yc, 0).view(torch.int16))
    assert (wide[:, dims[-1]:] == -7.0).all()


def test_fp16_32_sample_tiles_fall_back():
    # a ReLU layer among leaky ones, rows at a stride and other widths stay on the 16-sample kernels (same results either way)
    rng = np.random.default_rng(99)
    dims, B = [8, 64, 64, 1], 500
    x = rng.uniform(-1, 1, (B, 8)).astype(np.float16)
    specs = make_net(rng, dims, CT.Float16, act=Activation.LeakyReLU, slope=0.01, bias="rand", init="he")
    specs[0]["act"] = Activation.ReLU
    y = cv.mlpForward(gpu_layers(specs, CT.Float16, ML.RowMajor), to_dev(x))
    assert not cv.lastKernelName().startswith("mlpWide16Kernel"), cv.lastKernelName()
    assert torch.equal(y.view(torch.int16), chain_of_single_layers(specs, to_dev(x), CT.Float16).view(torch.int16))
    specs = make_net(rng, dims, CT.Float16, bias="rand", init="he")
    strided = torch.zeros((B, 12), dtype=torch.float16, device=DEV)
    strided[:, :8] = to_dev(x)
    y = cv.mlpForward(gpu_layers(specs, CT.Float16, ML.RowMajor), strided[:, :8])
    assert not cv.lastKernelName().startswith("mlpWide16Kernel"), cv.lastKernelName()
    y2 = cv.mlpForward(gpu_layers(specs, CT.Float16, ML.RowMajor), to_dev(x))
    assert cv.lastKernelName().startswith("mlpWide16Kernel"), cv.lastKernelName()
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16))


def test_32_sample_tiles_keep_the_summation_order():
    # The last layer's fp32 sums reach the fp16 output without any coarser rounding in between, so they
    # show the order in which the 8-element chunks of k meet the accumulator: with hidden values and
    # weights log-uniform over 2^-9 .. 2^4 the terms of one sum span far more than fp32 holds, most
    # accumulations are inexact, and a different order moves the fp16 result in about one output of 10^4.
    # The 32-sample kernel feeds the chunks in the order of the 16-sample operators: same bits on 6.4 million
    # outputs.  (Layer 0 passes the inputs through: units 0..31 = relu(x), 32..63 = relu(-x), exact.)
    rng = np.random.default_rng(1234)
    B = 200000
    mag = lambda shape: np.exp2(rng.uniform(-9, 4, shape)) * rng.choice([-1.0, 1.0], shape)
    W0 = np.zeros((64, 32)); W0[np.arange(32), np.arange(32)] = 1.0; W0[32 + np.arange(32), np.arange(32)] = -1.0
    W1 = ob.encode_e4m3(mag((32, 64)))
    specs = [dict(W=ob.encode_e4m3(W0), b=None, act=int(Activation.ReLU), slope=0.0),
             dict(W=W1, b=None, act=int(Activation.NoActivation), slope=0.0)]
    x = ob.encode_e4m3(mag((B, 32)))
    xd = to_dev(x)
    yc = chain_of_single_layers(specs, xd, CT.FloatE4M3)
    y = cv.mlpForward(gpu_layers(specs, CT.FloatE4M3, ML.RowMajor), xd, weightType=CT.FloatE4M3)
    assert cv.lastKernelName().startswith("mlpWideKernel"), cv.lastKernelName()
    assert torch.equal(y.view(torch.int16), yc.view(torch.int16))
    # the case is exercised: summing the k axis in another order, in fp32, changes fp16 results
    n = B
    xf = ob.decode_e4m3(x[:n]).astype(np.float32)
    hf = np.concatenate([np.maximum(xf, 0), np.maximum(-xf, 0)], axis=1)
    wf = ob.decode_e4m3(W1).astype(np.float32)
    fwd = np.zeros((n, 32), np.float32); bwd = np.zeros((n, 32), np.float32)
    for k in range(64):
        fwd += hf[:, k:k + 1] * wf[:, k][None, :]
        bwd += hf[:, 63 - k:64 - k] * wf[:, 63 - k][None, :]
    assert (fwd != bwd).mean() > 0.05
    assert (fwd.astype(np.float16) != bwd.astype(np.float16)).sum() >= 5


@pytest.mark.parametrize("B", [4096, 50])
def test_e4m3_saturation_on_32_sample_tiles(B):
    # ReLU networks (the 32-sample kernel): hidden sums beyond 448, also through an fp16 overflow, saturate
    # to 448 when the carrier is re-quantised; an overflow of the network's own fp16 output stays inf
    rng = np.random.default_rng(449)
    specs = make_net(rng, [32, 64, 64, 8], CT.FloatE4M3, bias="none", init="half")
    specs[0]["W"][:8] = ob.encode_e4m3(np.full((8, 32), 448.0))         # rows that overflow fp16
    specs[0]["W"][16:24] = ob.encode_e4m3(np.full((8, 32), 2.0))        # beyond 448, within fp16
    specs[1]["W"][:, :8] = ob.encode_e4m3(np.abs(rng.standard_normal((64, 8))) * 0.5)
    specs[2]["W"][0] = ob.encode_e4m3(np.full(64, 448.0))               # output row that can overflow fp16
    xf = rng.standard_normal((B, 32)) * 0.5
    xf[::3] = 448.0
    x = ob.encode_e4m3(xf)
    xd = to_dev(x)
    y = cv.mlpForward(gpu_layers(specs, CT.FloatE4M3, ML.InferencingOptimal), xd, weightType=CT.FloatE4M3)
    assert cv.lastKernelName().startswith("mlpWideKernel"), cv.lastKernelName()
    yc = chain_of_single_layers(specs, xd, CT.FloatE4M3)
    assert torch.equal(y.view(torch.int16), yc.view(torch.int16))
    ref, acts = ob.ref_mlp_forward(specs, x, ob.E4M3, want_acts=True)
    got = y.cpu().numpy()
    assert np.isinf(ref).any() and np.isinf(acts[0]).any()              # the case is exercised
    assert np.array_equal(np.isinf(got), np.isinf(ref))
    assert np.array_equal(got[np.isinf(ref)], ref[np.isinf(ref)])


def test_forward_plan_equals_mlp_forward():
    # the prepared call (descriptor marshalled once) is the same C-ABI call: same bits, same errors
    rng = np.random.default_rng(21)
    for wtype, dims in ((CT.Float16, [2, 16, 16, 16, 1]), (CT.FloatE4M3, [32, 64, 64, 8])):
        specs = make_net(rng, dims, wtype, bias="rand" if wtype == CT.Float16 else "none", init="he" if wtype == CT.Float16 else "half")
        layers = gpu_layers(specs, wtype, ML.RowMajor)
        if wtype == CT.Float16:
            xd = to_dev(rng.uniform(-1, 1, (1000, dims[0])).astype(np.float16))
        else:
            xd = to_dev(ob.encode_e4m3(rng.standard_normal((1000, dims[0])) * 0.5))
        plan = cv.MlpForwardPlan(layers, weightType=wtype)
        y0 = cv.mlpForward(layers, xd, weightType=wtype)
        y1 = plan(xd)
        out = torch.empty_like(y0)
        y2 = plan(xd[:333], out=out[:333])
        assert torch.equal(y0.view(torch.int16), y1.view(torch.int16))
        assert torch.equal(y0[:333].view(torch.int16), y2.view(torch.int16))
        if wtype == CT.FloatE4M3:       # the same plan takes fp16 vectors (quantised on load)
            xh = to_dev(ob.decode_e4m3(xd.cpu().numpy()).astype(np.float16))
            assert torch.equal(plan(xh).view(torch.int16), y0.view(torch.int16))
            assert torch.equal(plan(xd).view(torch.int16), y0.view(torch.int16))
        with pytest.raises(cv.CoopVecError):
            plan(xd[:, ::2])


def test_forward_in_a_hip_graph():
    # a launch-bound loop of small forward passes recorded into one HIP graph: the library launches on the
    # capturing stream and allocates nothing; every replay, with eager work in between, gives the eager result
    rng = np.random.default_rng(41)
    specs = make_net(rng, [2, 16, 16, 16, 1], CT.Float16, act=Activation.ReLU)
    layers = gpu_layers(specs, CT.Float16, ML.RowMajor)
    B = 4096
    x = torch.zeros(B, 2, dtype=torch.float16, device=DEV)
    outs = [torch.zeros(B, 1, dtype=torch.float16, device=DEV) for _ in range(3)]
    plan = cv.MlpForwardPlan(layers)
    plan(x, outs[0])                                   # first call outside the capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for o in outs:
            plan(x, o)
    for seed in range(4):
        xn = to_dev(np.random.default_rng(seed).uniform(0, 1, (B, 2)).astype(np.float16))
        want = cv.mlpForward(layers, xn)               # eager work between the replays
        x.copy_(xn)
        for o in outs:
            o.fill_(-1)
        g.replay()
        torch.cuda.synchronize()
        for o in outs:
            assert torch.equal(o.view(torch.int16), want.view(torch.int16)), seed


def test_mlp_argument_validation():
    rng = np.random.default_rng(0)
    specs = make_net(rng, [8, 16, 4], CT.Float16)
    layers = gpu_layers(specs, CT.Float16, ML.RowMajor)
    x = torch.zeros(10, 8, dtype=torch.float16, device=DEV)
    assert cv.mlpForward(layers, x[:0]).shape == (0, 4)
    layers[1].inputSize = 15
    with pytest.raises(cv.CoopVecError) as e:
        cv.mlpForward(layers, x)
    assert e.value.result == cv.SLANG_E_INVALID_ARG
    # beyond 128 wide there is no fused kernel
    specs = make_net(rng, [8, 144, 4], CT.Float16)
    with pytest.raises(cv.CoopVecError) as e:
        cv.mlpForward(gpu_layers(specs, CT.Float16, ML.RowMajor), x)
    assert e.value.result == cv.SLANG_E_NOT_AVAILABLE


@pytest.mark.parametrize("wtype", [CT.Float16, CT.FloatE4M3])
@pytest.mark.parametrize("dims", [[8, 16, 64, 4], [100, 128, 96, 50, 3], [5, 7], [33, 17, 128, 128, 1], [64, 128, 128, 16]])
def test_general_kernel_for_arbitrary_shapes(dims, wtype):
    # no built-in tile shape matches these: the general kernel (weights in LDS, run-time sizes)
    if len(dims) == 2:
        dims = dims + [dims[-1]]
    rng = np.random.default_rng(sum(dims) + int(wtype))
    B = 777
    act = Activation.LeakyReLU if wtype == CT.Float16 else Activation.ReLU
    specs = make_net(rng, dims, wtype, act=act, slope=float(np.float16(0.01)), bias="rand",
                     init="he" if wtype == CT.Float16 else "half")
    if wtype == CT.Float16:
        x = rng.uniform(-1, 1, (B, dims[0])).astype(np.float16)
        xd = to_dev(x); xct = ob.F16
    else:
        x = ob.encode_e4m3(rng.standard_normal((B, dims[0])) * 0.5)
        xd = to_dev(x); xct = ob.E4M3
    for layout in (ML.RowMajor, ML.InferencingOptimal):
        y = cv.mlpForward(gpu_layers(specs, wtype, layout), xd, weightType=wtype)
        hid = []
        yc = chain_of_single_layers(specs, xd, wtype, hidden=hid)
        assert torch.equal(y.view(torch.int16), yc.view(torch.int16))
    # deeper and wider chains give more hidden units a chance to sit on a rounding boundary
    frac, _ = end_to_end_ok(y.cpu().numpy(), specs, x, xct, hid)
    assert frac >= 0.99


def test_full_size_e4m3_decoder():
    # batch 2^24 of the 32 -> 64 -> 64 -> 8 e4m3 decoder: sampled oracle check, layout equality,
    # determinism, and agreement of the two halves with one full launch (tiling independence)
    B = 1 << 24
    rng = np.random.default_rng(77)
    specs = make_net(rng, [32, 64, 64, 8], CT.FloatE4M3, bias="none", init="half")
    g = torch.Generator(device=DEV); g.manual_seed(77)
    x = (torch.randn(B, 32, device=DEV, generator=g) * 0.5).to(torch.float8_e4m3fn)
    lo = gpu_layers(specs, CT.FloatE4M3, ML.InferencingOptimal)
    lr = gpu_layers(specs, CT.FloatE4M3, ML.RowMajor)
    y1 = cv.mlpForward(lo, x, weightType=CT.FloatE4M3)
    y2 = cv.mlpForward(lr, x, weightType=CT.FloatE4M3)
    assert torch.equal(y1.view(torch.int16), y2.view(torch.int16))
    y3 = cv.mlpForward(lo, x, weightType=CT.FloatE4M3)
    assert torch.equal(y1.view(torch.int16), y3.view(torch.int16))
    half = B // 2 + 48          # an offset that is not a multiple of the kernel's slot size
    ya = cv.mlpForward(lo, x[:half], weightType=CT.FloatE4M3)
    yb = cv.mlpForward(lo, x[half:], weightType=CT.FloatE4M3)
    assert torch.equal(y1[:half].view(torch.int16), ya.view(torch.int16))
    assert torch.equal(y1[half:].view(torch.int16), yb.view(torch.int16))
    idx = torch.from_numpy(np.concatenate([rng.integers(0, B, 8192), [0, 1, B - 2, B - 1]])).to(DEV)
    xs = x[idx].view(torch.uint8).cpu().numpy()
    hid = []
    ys = chain_of_single_layers(specs, x[idx].contiguous(), CT.FloatE4M3, hidden=hid)
    assert torch.equal(ys.view(torch.int16), y1[idx].view(torch.int16))
    frac, _ = end_to_end_ok(y1[idx].cpu().numpy(), specs, xs, ob.E4M3, hid)
    assert frac >= 0.999, frac


def test_fused_forward_equals_the_chain_of_single_layers_on_random_shapes():
    # Networks drawn at random (every layer up to 128 wide, one to five layers, ReLU or leaky ReLU, with and without
    # biases, fp16 and e4m3 weights, RowMajor and InferencingOptimal, batches that end inside a tile): whichever kernel
    # cvMlpForward picks, its result equals the chain of coopVecMatMulAdd launches bit for bit.
    rng = np.random.default_rng(20261)
    kernels = set()
    for case in range(48):
        wtype = CT.FloatE4M3 if case % 3 == 2 else CT.Float16
        nl = int(rng.integers(2, 6))
        shape_kind = case % 4
        if shape_kind == 0:      # the shapes of the specialised kernels
            width = int(rng.choice([16, 32, 64]))
            dims = [int(rng.choice([8, 16, 32]))] + [width] * (nl - 1) + [int(rng.integers(1, 17))]
        else:
            dims = [int(rng.integers(1, 129)) for _ in range(nl + 1)]
        leaky = wtype == CT.Float16 and case % 5 == 1
        specs = make_net(rng, dims, wtype, act=Activation.LeakyReLU if leaky else Activation.ReLU, slope=0.0625 if leaky else 0.0,
                         bias=("rand", "none", "zero")[case % 3], init="he" if wtype == CT.Float16 else "half")
        B = int(rng.integers(1, 3000))
        if wtype == CT.Float16:
            xd = to_dev(rng.uniform(-1, 1, (B, dims[0])).astype(np.float16))
        else:
            xd = to_dev(ob.encode_e4m3(rng.standard_normal((B, dims[0])) * 0.5))
        layout = ML.InferencingOptimal if case % 2 else ML.RowMajor
        y = cv.mlpForward(gpu_layers(specs, wtype, layout), xd, weightType=wtype)
        kernels.add(cv.lastKernelName().split("<")[0])
        yc = chain_of_single_layers(specs, xd, wtype)
        assert torch.equal(y.view(torch.int16), yc.view(torch.int16)), (case, dims, B, cv.lastKernelName())
    assert len(kernels) >= 3, kernels


@pytest.mark.parametrize("layout", [ML.RowMajor, ML.InferencingOptimal, ML.ColumnMajor])
def test_small_networks_on_the_lean_instantiations(layout):
    # Networks of 16-wide layers run on mlpForwardKernel's lean instantiations when their matrices are RowMajor with
    # rows of whole dwords or already in fragment order and the input vectors are whole aligned dwords; everything else
    # (ColumnMajor, rows or vectors of an odd number of halfs, a 6-byte pitch) stays on the general one.  Either way the
    # result equals the chain of single layers bit for bit, for batches of one sample, of one super-tile per wave, and
    # of several.
    rng = np.random.default_rng(411)
    lean_seen = 0
    for dims in ([2, 16, 16, 16, 1], [4, 16, 4], [16, 16, 16, 16, 16], [6, 10, 12, 3], [8, 16, 1], [3, 16, 16, 2], [2, 16, 5, 4]):
        for bias in ("rand", "none"):
            specs = make_net(rng, dims, CT.Float16, act=Activation.ReLU, bias=bias, init="he")
            layers = gpu_layers(specs, CT.Float16, layout)
            for B, pitch in ((1, 0), (15, 0), (64, 0), (65, 2), (1000, 0), (1000, 1), (70001, 0), (300000, 2)):
                full = to_dev(rng.uniform(-1, 1, (B, dims[0] + pitch)).astype(np.float16))
                xd = full[:, :dims[0]]
                y = cv.mlpForward(layers, xd, weightType=CT.Float16)
                name = cv.lastKernelName()
                whole = (dims[0] * 2) % 4 == 0 and ((dims[0] + pitch) * 2) % 4 == 0
                rows = all((d * 2) % 4 == 0 for d in dims[:-1])
                expect_lean = whole and (layout == ML.InferencingOptimal or (layout == ML.RowMajor and rows))
                if name.startswith("mlpForwardKernel"):      # (some of these shapes belong to the run-time-size kernel)
                    assert ("lean" in name) == expect_lean, (dims, B, pitch, name)
                    lean_seen += expect_lean
                yc = chain_of_single_layers(specs, xd.contiguous(), CT.Float16)
                assert torch.equal(y.view(torch.int16), yc.view(torch.int16)), (dims, bias, B, pitch, name)
    assert lean_seen > 0 or layout == ML.ColumnMajor


def test_lean_instantiation_with_padded_weight_rows():
    # RowMajor rows with a pitch beyond their length (whole dwords: lean; an odd number of halfs: general)
    rng = np.random.default_rng(412)
    dims = [4, 16, 12, 16, 2]
    specs = make_net(rng, dims, CT.Float16, act=Activation.ReLU, bias="rand", init="he")
    xd = to_dev(rng.uniform(-1, 1, (777, dims[0])).astype(np.float16))
    yc = chain_of_single_layers(specs, xd, CT.Float16)
    for pad, lean in ((2, True), (6, True), (1, False)):
        layers = []
        for s in specs:
            out, fan_in = s["W"].shape
            padded = np.zeros((out, fan_in + pad), np.float16)
            padded[:, :fan_in] = s["W"]
            padded[:, fan_in:] = 7.0            # (never read)
            layers.append(FeedForwardLayer(fan_in, out, as_bytes(to_dev(padded)), as_bytes(to_dev(s["b"])), ML.RowMajor,
                                           (fan_in + pad) * 2, s["act"], s["slope"]))
        y = cv.mlpForward(layers, xd, weightType=CT.Float16)
        if cv.lastKernelName().startswith("mlpForwardKernel"):
            assert ("lean" in cv.lastKernelName()) == lean, (pad, cv.lastKernelName())
        assert torch.equal(y.view(torch.int16), yc.view(torch.int16)), pad


@pytest.mark.parametrize("dims,B", [([8, 64, 64, 64, 64, 1], 100003), ([16, 32, 32, 32, 4], 4097), ([32, 64, 64, 64, 8], 5000), ([8, 32, 3], 129),
                                    ([16, 64, 64, 16], 70001)])
@pytest.mark.parametrize("bias", ["rand", "none"])
def test_leaky_fp16_networks_on_32_sample_tiles(dims, B, bias):
    # hidden layers that are all leaky ReLU (the example's activation) run on the 32-sample-tile kernel too: equal to the
    # chain of single layers bit for bit, and inside the oracle bar; one ReLU layer among them sends the call elsewhere
    rng = np.random.default_rng(sum(dims) + B)
    slope = 0.01
    specs = make_net(rng, dims, CT.Float16, act=Activation.LeakyReLU, slope=slope, bias=bias, init="he")
    if bias == "none":      # the example's layers all carry the activation, the last one too (fflayer.slang:60-66)
        specs[-1]["act"] = int(Activation.LeakyReLU)
    x = rng.uniform(-1, 1, (B, dims[0])).astype(np.float16)
    xd = to_dev(x)
    y = cv.mlpForward(gpu_layers(specs, CT.Float16, ML.RowMajor), xd, weightType=CT.Float16)
    assert cv.lastKernelName().startswith("mlpWide16Kernel") and "leaky" in cv.lastKernelName(), cv.lastKernelName()
    yc = chain_of_single_layers(specs, xd, CT.Float16)
    assert torch.equal(y.view(torch.int16), yc.view(torch.int16))
    # End to end against the oracle: the bar on the outputs.  (What lies outside stems from hidden sums at a rounding
    # boundary, which the two sides round differently; behind a leaky unit such a flip is scaled by the slope, so the
    # neighbour test that end_to_end_ok applies to ReLU networks does not fit here.)
    ref, acts = ob.ref_mlp_forward(specs, x, ob.F16, want_acts=True)
    ab = np.abs(acts[-2].astype(np.float32)) @ np.abs(specs[-1]["W"].astype(np.float32)).T
    bad = ob.float_parity_violations(y.cpu().numpy(), ref.astype(np.float32), ab, 2.0 ** -18)
    assert 1.0 - bad.mean() >= 0.99, 1.0 - bad.mean()
    if len(specs) > 2:
        specs[1]["act"] = Activation.ReLU
        y = cv.mlpForward(gpu_layers(specs, CT.Float16, ML.RowMajor), xd, weightType=CT.Float16)
        assert not cv.lastKernelName().startswith("mlpWide16Kernel"), cv.lastKernelName()
        assert torch.equal(y.view(torch.int16), chain_of_single_layers(specs, xd, CT.Float16).view(torch.int16))
