"""The neural module's whole-network parameter layouts: the numpy oracle against what the reference's
tests fix, the library's size arithmetic (CPU), and the GPU converter / FFLayer front against the oracle."""
import os
import sys

import numpy as np
import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(REPO, "oracle"))
import neural_layout as nl          # noqa: E402
import oracle_binding as ob        # noqa: E402

# (bias mask, dims, logical, physical): buffer sizes of tests/neural/network-parameter-layout-converter-buffer.slang
# :52-94 and of tools/gfx-unit-test/neural-slang-network-converter.cpp:21-22,42-46
REFERENCE_COUNTS = [
    (1, [4, 2], 10, 272),
    (0x200000001, [1] * 35, 36, 9248),
    (1, [17, 33], 594, 1584),
    (0x8000000000000001, [1] * 65, 66, 17408),
    (0b1010, [4, 5, 3, 2, 6], 62, 1088),
    (0b101, [5, 13, 7, 19], 321, 1088),
]


@pytest.mark.parametrize("mask,dims,logical,physical", REFERENCE_COUNTS)
def test_counts_match_the_reference_buffers(mask, dims, logical, physical):
    assert nl.network_counts(mask, dims) == (logical, physical)
    if len(dims) - 1 <= 64:
        import ctypes
        from slang_amd import _lib
        d = _lib.CvNeuralNetworkDesc()
        d.layerCount = len(dims) - 1
        for i, v in enumerate(dims):
            d.dims[i] = v
        d.biasMask, d.elementType, d.order = mask, 3, 0
        l, p = ctypes.c_size_t(0), ctypes.c_size_t(0)
        assert _lib.load().cvNeuralNetworkSize(ctypes.byref(d), ctypes.byref(l), ctypes.byref(p)) == 0
        assert (l.value, p.value) == (logical, physical)


def test_oversized_layer_is_refused():
    # the converter kernels index a layer's elements with 32-bit integers: 2^31 padded elements or more are refused
    import ctypes
    from slang_amd import _lib
    d = _lib.CvNeuralNetworkDesc()
    d.layerCount = 2
    d.dims[0], d.dims[1], d.dims[2] = 8, 65536, 32768         # the second layer has 2^31 weights
    d.biasMask, d.elementType, d.order = 0, 3, 0
    l, p = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert _lib.load().cvNeuralNetworkSize(ctypes.byref(d), ctypes.byref(l), ctypes.byref(p)) < 0
    d.dims[2] = 16384                                          # 2^30: fine
    assert _lib.load().cvNeuralNetworkSize(ctypes.byref(d), ctypes.byref(l), ctypes.byref(p)) == 0
    assert l.value == 8 * 65536 + 65536 * 16384


def host_test_network():
    mask, dims = 0b101, [5, 13, 7, 19]
    portable = np.array([nl.make_portable_value(i) for i in range(321)], np.float32)
    return mask, dims, portable


def test_metal_and_spirv_orders_by_independent_formulations():
    mask, dims, portable = host_test_network()
    metal = nl.to_optimal(portable, mask, dims, nl.PADDED_ROW_MAJOR)
    spirv = nl.to_optimal(portable, mask, dims, nl.TILED_ROW_MAJOR)
    lo = po = 0
    for k in range(3):
        n_in, n_out = dims[k], dims[k + 1]
        has_bias = bool((mask >> k) & 1)
        pin, pout = nl.align16(n_in), nl.align16(n_out)
        W = portable[lo:lo + n_in * n_out].reshape(n_out, n_in)
        padded = np.zeros((pout, pin), np.float32); padded[:n_out, :n_in] = W
        assert np.array_equal(metal[po:po + pin * pout], padded.ravel())                       # padded row-major
        tiles = padded.reshape(pout // 16, 16, pin // 16, 16).transpose(0, 2, 1, 3).ravel()   # 16x16 tiles, row-major inside
        assert np.array_equal(spirv[po:po + pin * pout], tiles)
        bias = np.zeros(pout, np.float32)
        if has_bias:
            bias[:n_out] = portable[lo + n_in * n_out: lo + n_in * n_out + n_out]
        assert np.array_equal(metal[po + pin * pout: po + pin * pout + pout], bias)
        lo += n_in * n_out + (n_out if has_bias else 0)
        po += pin * pout + pout
    assert lo == 321 and po == 1088


def test_cuda_and_native_orders_are_bijections_with_known_points():
    # rowMajorToCudaNativeLayout evaluated by hand for a few coordinates (converter :59-72)
    assert [nl.row_major_to_cuda_native(r, c) for r, c in ((0, 0), (1, 0), (2, 0), (8, 0), (0, 8), (0, 1), (15, 15))] == \
        [0, 1, 8, 2, 4, 32, 255]
    for order in (nl.CUDA_MATRIX_B, nl.NATIVE, nl.TILED_ROW_MAJOR, nl.PADDED_ROW_MAJOR):
        for n_in, n_out in ((16, 16), (17, 33), (5, 13)):
            offs = {nl.physical_weight_offset(order, n_in, n_out, o, i) for o in range(n_out) for i in range(n_in)}
            assert len(offs) == n_in * n_out and max(offs) < nl.align16(n_in) * nl.align16(n_out)
    # NATIVE inside one layer is the TrainingOptimal map of the C oracle
    for n_in, n_out in ((17, 33), (5, 13), (64, 64)):
        for o in range(n_out):
            for i in range(0, n_in, 3):
                assert nl.physical_weight_offset(nl.NATIVE, n_in, n_out, o, i) * 2 == \
                    ob.lib().cvo_layout_elem_offset(n_out, n_in, ob.F16, ob.TRAIN_OPT, 0, o, i)


@pytest.mark.parametrize("order", [nl.NATIVE, nl.TILED_ROW_MAJOR, nl.PADDED_ROW_MAJOR, nl.CUDA_MATRIX_B])
def test_oracle_round_trip(order):
    for mask, dims, logical, physical in REFERENCE_COUNTS[:1] + REFERENCE_COUNTS[2:3] + REFERENCE_COUNTS[4:]:
        portable = (np.arange(logical) + 1).astype(np.float32)
        opt = nl.to_optimal(portable, mask, dims, order)
        assert opt.size == physical and np.count_nonzero(opt) == logical
        assert np.array_equal(nl.to_portable(opt, mask, dims, order), portable)


# ---- GPU ------------------------------------------------------------------------------------------

@pytest.mark.gpu
@pytest.mark.parametrize("order", [nl.NATIVE, nl.TILED_ROW_MAJOR, nl.PADDED_ROW_MAJOR, nl.CUDA_MATRIX_B])
@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_gpu_converter_matches_oracle(order, dtype):
    import torch
    from slang_amd import coopvec as cv
    tdt = getattr(torch, dtype); ndt = getattr(np, dtype)
    for mask, dims, logical, physical in REFERENCE_COUNTS[:1] + REFERENCE_COUNTS[2:3] + REFERENCE_COUNTS[4:]:
        conv = cv.NetworkParameterLayoutConverter(tdt, mask, *dims, order=order)
        assert (conv.ElementCountLogical, conv.ElementCountPhysical) == (logical, physical)
        portable = np.array([nl.make_portable_value(i) for i in range(logical)], ndt)
        pd = torch.from_numpy(portable).cuda()
        opt = torch.full((physical,), 7.0, dtype=tdt, device="cuda")      # stale contents: padding must be overwritten with 0
        conv.toOptimalLayout(pd, opt)
        assert np.array_equal(opt.cpu().numpy(), nl.to_optimal(portable, mask, dims, order))
        back = conv.toPortableLayout(opt)
        assert np.array_equal(back.cpu().numpy(), portable)
    # the long masks (bits 33 and 63) through the library
    for mask, dims, logical, physical in (REFERENCE_COUNTS[1], REFERENCE_COUNTS[3][:1] + ([1] * 65, 66, 17408)):
        conv = cv.NetworkParameterLayoutConverter(tdt, mask, *dims, order=order)
        portable = (np.arange(logical) + 1).astype(ndt)
        opt = conv.toOptimalLayout(torch.from_numpy(portable).cuda())
        assert np.array_equal(opt.cpu().numpy(), nl.to_optimal(portable, mask, dims, order))


@pytest.mark.gpu
def test_fflayer_chain_over_a_parameter_block():
    # FFLayer.eval chain (layers.slang:90-110) from the portable block and from the optimal block: same
    # result, equal to the un-blocked fused MLP on the same weights
    import torch
    from gpu_util import DEV, as_bytes, to_dev
    from slang_amd import coopvec as cv
    from slang_amd.coopvec import Activation, CoopVecMatrixLayout as ML, FeedForwardLayer
    rng = np.random.default_rng(6)
    dims, mask = [5, 13, 7, 19], 0b101
    conv = cv.NetworkParameterLayoutConverter(torch.float16, mask, *dims)
    portable = (rng.standard_normal(conv.ElementCountLogical) * 0.4).astype(np.float16)
    pd = to_dev(portable)
    opt = conv.toOptimalLayout(pd)
    B = 777
    x = to_dev(rng.uniform(-1, 1, (B, 5)).astype(np.float16))
    acts = [Activation.ReLU, Activation.Tanh, Activation.NoActivation]
    y_lin = conv.eval(pd, x, optimalLayout=False, activations=acts)
    y_opt = conv.eval(opt, x, optimalLayout=True, activations=acts)
    assert torch.equal(y_lin.view(torch.int16), y_opt.view(torch.int16))
    layers, off = [], 0
    for k in range(3):
        fi, fo = dims[k], dims[k + 1]
        W = portable[off:off + fi * fo]; off += fi * fo
        b = None
        if (mask >> k) & 1:
            b = portable[off:off + fo]; off += fo
        layers.append(FeedForwardLayer(fi, fo, as_bytes(to_dev(W)), as_bytes(to_dev(b)) if b is not None else None,
                                       ML.RowMajor, fi * 2, acts[k], 0.0))
    y_ref = cv.mlpForward(layers, x)
    assert torch.equal(y_lin.view(torch.int16), y_ref.view(torch.int16))


@pytest.mark.gpu
def test_training_through_a_parameter_block():
    # gradients land in a block laid out like the parameters (portable and optimal), equal after conversion
    import torch
    from gpu_util import to_dev
    from slang_amd import coopvec as cv
    from slang_amd.coopvec import Activation
    rng = np.random.default_rng(12)
    dims, mask = [4, 16, 4], 0b01
    conv = cv.NetworkParameterLayoutConverter(torch.float16, mask, *dims)
    portable = (rng.standard_normal(conv.ElementCountLogical) * 0.5).astype(np.float16)
    pd = to_dev(portable); opt = conv.toOptimalLayout(pd)
    B = 64
    x = to_dev(rng.uniform(0, 1, (B, 4)).astype(np.float16))
    t = to_dev(rng.uniform(-1, 1, (B, 4)).astype(np.float16))
    acts = [Activation.ReLU, Activation.NoActivation]
    g_lin = torch.zeros_like(pd); g_opt = torch.zeros_like(opt)
    l1 = conv.trainStep(pd, g_lin, x, t, optimalLayout=False, activations=acts, lossScale=1.0 / B)
    l2 = conv.trainStep(opt, g_opt, x, t, optimalLayout=True, activations=acts, lossScale=1.0 / B)
    assert l1.item() == l2.item() and l1.item() > 0
    assert torch.equal(conv.toPortableLayout(g_opt).view(torch.int16), g_lin.view(torch.int16))
    assert g_lin.abs().sum().item() > 0
    # layer 1 has no bias: its slot in the optimal gradient block stays untouched (zero)
    assert (g_opt[nl.layer_counts(4, 16, True)[1] + 16 * 16:] == 0).all()
