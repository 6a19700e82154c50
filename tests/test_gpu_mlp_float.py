"""GPU parity of the fused forward MLP whose carrier is not half: networks of one type T = float (the neural
module's FFLayer<float, ...> chain, source/standard-modules/neural/layers.slang:34-110) or bfloat16
(this library's extension), through cvMlpForward / cvNeuralMlpForward.

The bar: bit-equal with the chain of single-layer operators (coopVecMatMulAdd + activation in T, pinned against the
oracle in test_gpu_matmul.py), and within the float tolerance of the same network evaluated in float64
(T = float: 2^-18 of the layer-wise magnitude sums; T = bfloat16: its 2^-8 roundings per layer)."""
import numpy as np
import pytest
import torch

import oracle_binding as ob
from gpu_util import DEV, as_bytes, to_dev
from slang_amd import coopvec as cv
from slang_amd.coopvec import Activation, CoopVecComponentType as CT, CoopVecMatrixLayout as ML, FeedForwardLayer

pytestmark = pytest.mark.gpu

TORCH = {CT.Float32: torch.float32, CT.BFloat16: torch.bfloat16}


def to_T(a64, ct):
    """float64 array -> device tensor of type T (bfloat16: nearest even)"""
    if ct == CT.Float32:
        return to_dev(a64.astype(np.float32))
    return to_dev(ob.bf16_bits(a64.astype(np.float32)).view(np.int16)).view(torch.bfloat16)


def from_T(t):
    return t.float().cpu().numpy().astype(np.float64)


def act64(z, act, slope):
    if act == Activation.ReLU: return np.maximum(z, 0)
    if act == Activation.LeakyReLU: return np.maximum(z, z * slope)
    if act == Activation.Tanh: return np.tanh(z)
    if act == Activation.Sigmoid: return 1 / (1 + np.exp(-z))
    return z


def build(rng, dims, ct, acts, layout, bias=True):
    """device layers in `layout` + the same parameters, as T rounded them, in float64"""
    layers, params = [], []
    esz = 4 if ct == CT.Float32 else 2
    for l in range(len(dims) - 1):
        fi, fo = dims[l], dims[l + 1]
        Wd = to_T(rng.standard_normal((fo, fi)) * np.sqrt(2.0 / fi), ct)
        bd = to_T(rng.standard_normal(fo) * 0.1, ct) if bias and l != 1 else None     # one layer without a bias
        wbytes = as_bytes(Wd.contiguous())
        stride = fi * esz
        if layout != ML.RowMajor:
            size = cv.getCooperativeVectorMatrixSize(fo, fi, ct, layout)
            dst = torch.zeros(size, dtype=torch.uint8, device=DEV)
            D = cv.CooperativeVectorMatrixDesc
            cv.convertCooperativeVectorMatrix(dst, [D(fo, fi, ct, layout, size, 0, 0)], wbytes, [D(fo, fi, ct, ML.RowMajor, fo * stride, 0, stride)])
            wbytes, stride = dst, 0
        layers.append(FeedForwardLayer(fi, fo, wbytes, as_bytes(bd) if bd is not None else None, layout, stride, acts[l], 0.125))
        params.append((from_T(Wd), from_T(bd) if bd is not None else None, Wd, bd))
    return layers, params


def chain(params, x, ct, acts):
    """the same network as single-layer operators"""
    esz = 4 if ct == CT.Float32 else 2
    for (_, _, Wd, bd), act in zip(params, acts):
        fo, fi = Wd.shape
        if bd is not None:
            x = cv.coopVecMatMulAdd(x, ct, as_bytes(Wd.contiguous()), 0, ct, as_bytes(bd), 0, ct, ML.RowMajor, False, fi * esz, M=fo,
                                    resultType=ct, activation=act, leakySlope=0.125)
        else:
            x = cv.coopVecMatMul(x, ct, as_bytes(Wd.contiguous()), 0, ct, ML.RowMajor, False, fi * esz, M=fo, resultType=ct)
            assert act == Activation.NoActivation
    return x


@pytest.mark.parametrize("ct", [CT.Float32, CT.BFloat16])
@pytest.mark.parametrize("dims", [[8, 64, 64, 4], [5, 13, 7, 19], [100, 128, 50, 3], [32, 16, 16, 16, 16, 1]])
def test_float_networks_equal_the_chain_of_single_layer_operators(ct, dims):
    rng = np.random.default_rng(sum(dims) + int(ct))
    B = 1000
    L = len(dims) - 1
    acts = [[Activation.ReLU, Activation.NoActivation, Activation.LeakyReLU, Activation.Tanh, Activation.Sigmoid][l % 5] for l in range(L)]
    acts[1] = Activation.NoActivation
    x64 = rng.uniform(-1, 1, (B, dims[0]))
    xd = to_T(x64, ct)
    ys = []
    for layout in (ML.RowMajor, ML.InferencingOptimal, ML.TrainingOptimal):
        layers, params = build(np.random.default_rng(7), dims, ct, acts, layout)
        y = cv.mlpForward(layers, xd, weightType=ct)
        assert cv.lastKernelName().startswith("mlpFloatKernel"), cv.lastKernelName()
        assert y.dtype == TORCH[ct] and y.shape == (B, dims[-1])
        ys.append(y)
    bits = torch.int32 if ct == CT.Float32 else torch.int16
    assert torch.equal(ys[0].view(bits), ys[1].view(bits)) and torch.equal(ys[0].view(bits), ys[2].view(bits))
    yc = chain(params, xd, ct, acts)
    assert torch.equal(ys[0].view(bits), yc.view(bits))
    # the network itself, in float64 on the parameters as T holds them
    h = from_T(xd)
    mag = np.abs(h)
    for (W, b, _, _), act in zip(params, acts):
        z = h @ W.T + (b if b is not None else 0.0)
        mag = mag @ np.abs(W).T + (np.abs(b) if b is not None else 0.0)       # bound of the layer's terms, carried along
        h = act64(z, act, 0.125)
    eps = 2.0 ** -18 if ct == CT.Float32 else 2.0 ** -7 * L
    assert (np.abs(from_T(ys[0]) - h) <= eps * (mag + 1.0)).all()


def test_plan_strides_and_validation():
    rng = np.random.default_rng(3)
    dims, acts = [6, 24, 10], [Activation.ReLU, Activation.NoActivation]
    layers, params = build(rng, dims, CT.Float32, acts, ML.RowMajor)
    B = 300
    big = to_dev(rng.uniform(-1, 1, (B, 16)).astype(np.float32))
    x = big[:, 3:9]                        # rows 64 bytes apart, 4-byte aligned only
    out = torch.full((B, 12), -7.0, dtype=torch.float32, device=DEV)
    plan = cv.MlpForwardPlan(layers, weightType=CT.Float32)
    plan(x, out=out[:, :10])
    assert torch.equal(out[:, :10], cv.mlpForward(layers, x.contiguous(), weightType=CT.Float32)) and (out[:, 10:] == -7).all()
    with pytest.raises(cv.CoopVecError) as e:          # vectors of another type than the network's
        cv.mlpForward(layers, x.to(torch.float16), weightType=CT.Float32)
    assert e.value.result == cv.SLANG_E_NOT_AVAILABLE


def test_fp32_parameter_block_of_the_neural_module():
    # NetworkParameterLayoutConverter<float, ...> + FFLayer<float, ...>.eval: from the portable and from the optimal
    # block, equal to the un-blocked network on the same parameters
    rng = np.random.default_rng(11)
    dims, mask = [5, 13, 7, 19], 0b101
    conv = cv.NetworkParameterLayoutConverter(torch.float32, mask, *dims)
    portable = (rng.standard_normal(conv.ElementCountLogical) * 0.4).astype(np.float32)
    pd = to_dev(portable)
    opt = conv.toOptimalLayout(pd)
    B = 500
    x = to_dev(rng.uniform(-1, 1, (B, 5)).astype(np.float32))
    acts = [Activation.ReLU, Activation.Tanh, Activation.NoActivation]
    y_lin = conv.eval(pd, x, optimalLayout=False, activations=acts)
    y_opt = conv.eval(opt, x, optimalLayout=True, activations=acts)
    assert y_lin.dtype == torch.float32
    assert torch.equal(y_lin.view(torch.int32), y_opt.view(torch.int32))
    h, off = x.cpu().numpy().astype(np.float64), 0
    for k in range(3):
        fi, fo = dims[k], dims[k + 1]
        W = portable[off:off + fi * fo].reshape(fo, fi).astype(np.float64); off += fi * fo
        z = h @ W.T
        if (mask >> k) & 1:
            z = z + portable[off:off + fo].astype(np.float64); off += fo
        h = act64(z, acts[k], 0.0)
    assert np.allclose(y_lin.cpu().numpy(), h, rtol=1e-5, atol=1e-5)
    # bwd_diff through the block: the gradients land at the parameters' offsets, the same from both layouts
    t = to_dev(rng.standard_normal((B, dims[-1])).astype(np.float32))
    g_lin = torch.zeros_like(pd); g_opt = torch.zeros_like(opt)
    acts_t = [Activation.ReLU, Activation.LeakyReLU, Activation.NoActivation]
    l1 = conv.trainStep(pd, g_lin, x, t, optimalLayout=False, activations=acts_t, leakySlopes=[0, 0.125, 0])
    l2 = conv.trainStep(opt, g_opt, x, t, optimalLayout=True, activations=acts_t, leakySlopes=[0, 0.125, 0])
    assert torch.equal(l1, l2)
    assert torch.equal(conv.toPortableLayout(g_opt).view(torch.int32), g_lin.view(torch.int32))
    want_loss, want_g = backprop64(portable, dims, mask, acts_t, 0.125, x.cpu().numpy(), t.cpu().numpy(), 1.0)
    assert abs(float(l1) - want_loss) <= 1e-5 * want_loss
    got = g_lin.cpu().numpy().astype(np.float64)
    assert np.linalg.norm(got - want_g) <= 1e-5 * np.linalg.norm(want_g)


def backprop64(portable, dims, mask, acts, slope, x, t, loss_scale):
    """The step in float64 on a portable parameter block: (loss sum, gradient block of the same layout)."""
    L = len(dims) - 1
    Ws, bs, off = [], [], 0
    for k in range(L):
        fi, fo = dims[k], dims[k + 1]
        Ws.append(portable[off:off + fi * fo].reshape(fo, fi).astype(np.float64)); off += fi * fo
        if (mask >> k) & 1:
            bs.append(portable[off:off + fo].astype(np.float64)); off += fo
        else:
            bs.append(None)
    hs, zs = [x.astype(np.float64)], []
    for k in range(L):
        z = hs[-1] @ Ws[k].T + (bs[k] if bs[k] is not None else 0.0)
        zs.append(z); hs.append(act64(z, acts[k], slope))
    diff = hs[-1] - t.astype(np.float64)
    loss = float((diff ** 2).sum())
    g = 2.0 * diff * loss_scale
    out = np.zeros(portable.shape, np.float64)
    grads = []
    for k in range(L - 1, -1, -1):
        z = zs[k]
        if acts[k] == Activation.ReLU: d = np.where(z > 0, 1.0, np.where(z == 0, 0.5, 0.0))
        elif acts[k] == Activation.LeakyReLU: d = np.where(z > 0, 1.0, np.where(z == 0, 0.5 + 0.5 * slope, slope))
        else: d = 1.0
        dz = g * d
        grads.append((dz.T @ hs[k], dz.sum(axis=0)))
        g = dz @ Ws[k]
    grads.reverse()
    off = 0
    for k in range(L):
        fi, fo = dims[k], dims[k + 1]
        out[off:off + fi * fo] = grads[k][0].reshape(-1); off += fi * fo
        if (mask >> k) & 1:
            out[off:off + fo] = grads[k][1]; off += fo
    return loss, out


@pytest.mark.parametrize("grad_layout", [ML.RowMajor, ML.TrainingOptimal])
def test_fp32_training_step_against_float64(grad_layout):
    # learnGradient for a network of float (layer by layer): loss and every gradient against float64 backpropagation
    # on the same fp32 parameters; "+=" into pre-filled destinations; bitwise reproducible
    rng = np.random.default_rng(17)
    dims, mask = [6, 20, 13, 3], 0b111
    acts = [Activation.ReLU, Activation.LeakyReLU, Activation.NoActivation]
    n_par = sum(dims[k] * dims[k + 1] + dims[k + 1] for k in range(3))
    portable = (rng.standard_normal(n_par) * 0.5).astype(np.float32)
    B = 3000
    x = rng.uniform(-1, 1, (B, dims[0])).astype(np.float32); t = rng.standard_normal((B, dims[-1])).astype(np.float32)
    want_loss, want_g = backprop64(portable, dims, mask, acts, 0.125, x, t, 0.5)

    def run():
        layers, views, off = [], [], 0
        for k in range(3):
            fi, fo = dims[k], dims[k + 1]
            W = portable[off:off + fi * fo]; off += fi * fo
            b = portable[off:off + fo]; off += fo
            gsize = cv.getCooperativeVectorMatrixSize(fo, fi, CT.Float32, grad_layout, fi * 4)
            wg = torch.zeros(gsize, dtype=torch.uint8, device=DEV)
            bg = torch.full((fo,), 1.0, dtype=torch.float32, device=DEV)          # pre-filled: the step adds
            layers.append(FeedForwardLayer(fi, fo, as_bytes(to_dev(W)), as_bytes(to_dev(b)), ML.RowMajor, fi * 4, acts[k], 0.125,
                                           wg, as_bytes(bg), grad_layout, fi * 4 if grad_layout == ML.RowMajor else 0))
            views.append((wg, bg, gsize))
        _, loss = cv.mlpTrainStep(layers, to_dev(x), to_dev(t), lossScale=0.5, weightType=CT.Float32)
        assert "layer-by-layer" in cv.lastKernelName()
        out = []
        for k, (wg, bg, gsize) in enumerate(views):
            fi, fo = dims[k], dims[k + 1]
            if grad_layout != ML.RowMajor:
                row = torch.zeros(fo * fi * 4, dtype=torch.uint8, device=DEV)
                D = cv.CooperativeVectorMatrixDesc
                cv.convertCooperativeVectorMatrix(row, [D(fo, fi, CT.Float32, ML.RowMajor, fo * fi * 4, 0, fi * 4)],
                                                  wg, [D(fo, fi, CT.Float32, grad_layout, gsize, 0, 0)])
                wg = row
            out.append(wg.view(torch.float32).cpu().numpy().copy()); out.append(bg.cpu().numpy().copy() - 1.0)
        return float(loss), np.concatenate(out)

    loss1, g1 = run()
    loss2, g2 = run()
    assert loss1 == loss2 and np.array_equal(g1.view(np.uint32), g2.view(np.uint32))
    assert abs(loss1 - want_loss) <= 1e-5 * want_loss
    assert np.linalg.norm(g1.astype(np.float64) - want_g) <= 2e-5 * np.linalg.norm(want_g)
    assert (np.abs(g1.astype(np.float64) - want_g) <= 1e-4 * (np.abs(want_g) + np.abs(want_g).mean())).all()
