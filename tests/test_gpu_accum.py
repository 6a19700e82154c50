"""GPU parity of the batched outer-product / reduce-sum accumulate operators, through the C-ABI."""
import json
import os

import numpy as np
import pytest
import torch

import oracle_binding as ob
from gpu_util import DEV, as_bytes, matrix_in_layout, to_dev
from slang_amd import coopvec as cv
from slang_amd.coopvec import CoopVecComponentType as CT, CoopVecMatrixLayout as ML

pytestmark = pytest.mark.gpu
G = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "coopvec_goldens.json")))


def test_outer_product_golden():
    # tests/cooperative-vector/outer-product.slang: a=[1..4], b=[1..8], 111 pre-stored at [0]
    g = G["outer_product_f16"]
    a = to_dev(np.array([g["a"]], np.float16)); b = to_dev(np.array([g["b"]], np.float16))
    mat = np.zeros(32, np.float16); mat[0] = g["prestored_at_0"]
    d = to_dev(mat).view(torch.uint8)
    cv.coopVecOuterProductAccumulate(a, b, d, 0, 16, ML.RowMajor, CT.Float16)
    assert d.view(torch.float16).cpu().numpy().tolist() == g["expected_row_major_4x8"]
    # TrainingOptimal destination (the layout the reference requires on hardware), read back by convert
    size = cv.getCooperativeVectorMatrixSize(4, 8, CT.Float16, ML.TrainingOptimal)
    t = torch.zeros(size, dtype=torch.uint8, device=DEV)
    cv.coopVecOuterProductAccumulate(a, b, t, 0, 0, ML.TrainingOptimal, CT.Float16)
    row = torch.zeros(64, dtype=torch.uint8, device=DEV)
    cv.convertCooperativeVectorMatrix(row, [cv.CooperativeVectorMatrixDesc(4, 8, CT.Float16, ML.RowMajor, 64, 0, 16)],
                                      t, [cv.CooperativeVectorMatrixDesc(4, 8, CT.Float16, ML.TrainingOptimal, size, 0, 0)])
    want = list(g["expected_row_major_4x8"]); want[0] = 1.0
    assert row.view(torch.float16).cpu().numpy().tolist() == want


def test_reduce_sum_goldens():
    g = G["reduce_sum_f16"]
    v = to_dev(np.array([g["v"]], np.float16))
    buf = np.zeros(4, np.float16); buf[0] = g["prestored_at_0"]
    d = to_dev(buf)
    cv.coopVecReduceSumAccumulate(v, d.view(torch.uint8), 0)
    assert d.cpu().numpy().tolist() == g["expected"]
    # 8 threads x [1,1,1,1] -> [8,8,8,8]: accumulation across threads (reduce-sum-accumulate-sm610.slang)
    g8 = G["reduce_sum_8threads"]
    v8 = to_dev(np.array([g8["v"]] * g8["threads"], np.float16))
    d = torch.zeros(4, dtype=torch.float16, device=DEV)
    cv.coopVecReduceSumAccumulate(v8, d.view(torch.uint8), 0)
    assert d.cpu().numpy().tolist() == g8["expected"]
    # 128 threads x (i+1)/128 -> i+1 (tests/neural/bias-sum-reduce.slang)
    v = to_dev(np.tile(((np.arange(8) + 1) / 128.0).astype(np.float16), (128, 1)))
    d = torch.zeros(8, dtype=torch.float32, device=DEV)
    cv.coopVecReduceSumAccumulate(v, d.view(torch.uint8), 0, bufferType=CT.Float32)
    assert d.cpu().numpy().tolist() == (np.arange(8) + 1.0).tolist()


@pytest.mark.parametrize("M,N,B", [(64, 8, 5000), (64, 64, 4099), (1, 64, 777), (16, 4, 33), (100, 70, 1500), (128, 128, 2048)])
@pytest.mark.parametrize("layout,ct", [(ML.RowMajor, CT.Float32), (ML.TrainingOptimal, CT.Float32), (ML.ColumnMajor, CT.Float16)])
def test_outer_product_against_fp64(M, N, B, layout, ct):
    rng = np.random.default_rng(M * 131 + N + B)
    a = (rng.standard_normal((B, M)) * 0.25).astype(np.float16)
    b = rng.uniform(-1, 1, (B, N)).astype(np.float16)
    want = a.astype(np.float64).T @ b.astype(np.float64)
    npdt = np.float32 if ct == CT.Float32 else np.float16
    init = rng.standard_normal((M, N)).astype(npdt)
    d = to_dev(matrix_in_layout(init, ct, layout))
    cv.coopVecOuterProductAccumulate(to_dev(a), to_dev(b), d, 0, 0, layout, ct)
    back = np.zeros((M, N), npdt)
    assert ob.lib().cvo_layout_convert(ob.ptr(back), M, N, int(ct), ob.ROW, 0, ob.ptr(d.cpu().numpy()), int(ct), int(layout), 0) == 0
    got = back.astype(np.float64) - init.astype(np.float64)
    tol = 1e-3 if ct == CT.Float32 else 4e-3      # fp16 destination: one more rounding of sum + init
    assert np.linalg.norm(got - want) <= tol * np.linalg.norm(want)
    # closed form of tests/neural/outerproduct-accumulate-tiled-test.slang: sum_s (c_s * u) (x) w = (sum c_s) u (x) w
    if layout == ML.RowMajor:
        d2 = torch.zeros(M * N, dtype=torch.float32, device=DEV)
        cv.coopVecOuterProductAccumulate(to_dev(a), to_dev(b), d2.view(torch.uint8), 0, N * 4, ML.RowMajor, CT.Float32)
        d3 = torch.zeros(M * N, dtype=torch.float32, device=DEV)
        cv.coopVecOuterProductAccumulate(to_dev(a), to_dev(b), d3.view(torch.uint8), 0, N * 4, ML.RowMajor, CT.Float32)
        assert torch.equal(d2, d3)                 # bitwise run-to-run determinism


@pytest.mark.parametrize("N,B", [(64, 5000), (1, 100), (8, 33), (100, 4099), (256, 1000)])
def test_reduce_sum_against_fp64(N, B):
    rng = np.random.default_rng(N + B)
    v = rng.uniform(-1, 1, (B, N)).astype(np.float16)
    want = v.astype(np.float64).sum(0)
    d = torch.ones(N, dtype=torch.float32, device=DEV)
    cv.coopVecReduceSumAccumulate(to_dev(v), d.view(torch.uint8), 0, bufferType=CT.Float32)
    got = d.cpu().numpy().astype(np.float64) - 1.0
    assert np.max(np.abs(got - want)) <= 1e-4 * max(1.0, np.abs(want).max()) + 1e-3
    d2 = torch.ones(N, dtype=torch.float32, device=DEV)
    cv.coopVecReduceSumAccumulate(to_dev(v), d2.view(torch.uint8), 0, bufferType=CT.Float32)
    assert torch.equal(d, d2)


def test_outer_product_infinite_element_stays_within_its_fragment():
    # One infinite b[s][j].  The reference's per-element a[i]*b[j] (hlsl.meta.slang:33261-33315) makes
    # column j of the destination non-finite and nothing else.  Here the sample-major -> feature-major
    # transposition multiplies a fragment of 32 features by a 0/1 selection matrix on the MFMA, and
    # 0 * Inf = NaN: the columns that share j's 32-feature fragment become NaN as well.  Everything
    # outside that fragment stays exact.
    rng = np.random.default_rng(99)
    M, N, B, j = 64, 64, 1000, 5
    a = (rng.standard_normal((B, M)) * 0.25).astype(np.float16)
    b = rng.uniform(-1, 1, (B, N)).astype(np.float16)
    b[123, j] = np.inf
    d = torch.zeros(M * N, dtype=torch.float32, device=DEV)
    cv.coopVecOuterProductAccumulate(to_dev(a), to_dev(b), d.view(torch.uint8), 0, N * 4, ML.RowMajor, CT.Float32)
    got = d.cpu().numpy().reshape(M, N).astype(np.float64)
    bad_cols = np.nonzero(~np.isfinite(got).all(axis=0))[0]
    assert j in bad_cols and len(bad_cols) <= 32
    ok = np.setdiff1d(np.arange(N), bad_cols)
    want = a.astype(np.float64).T @ b.astype(np.float64)[:, ok]
    assert np.linalg.norm(got[:, ok] - want) <= 1e-3 * np.linalg.norm(want)


def test_accumulate_argument_validation():
    a = torch.zeros(4, 8, dtype=torch.float16, device=DEV)
    m = torch.zeros(1024, dtype=torch.uint8, device=DEV)
    with pytest.raises(cv.CoopVecError) as e:
        cv.coopVecOuterProductAccumulate(a, a, m, 0, 16, ML.RowMajor, CT.SignedInt8Packed)
    assert e.value.result == cv.SLANG_E_INVALID_ARG          # static_assert hlsl.meta.slang:33237
    with pytest.raises(cv.CoopVecError) as e:
        cv.coopVecOuterProductAccumulate(a, a, m, 0, 8, ML.RowMajor, CT.Float16)     # stride < row
    assert e.value.result == cv.SLANG_E_INVALID_ARG
    with pytest.raises(cv.CoopVecError) as e:
        cv.coopVecOuterProductAccumulate(a, a, m, 0, 16, ML.RowMajor, CT.Float16, workspace=torch.zeros(16, dtype=torch.uint8, device=DEV))
    assert e.value.result == cv.SLANG_E_BUFFER_TOO_SMALL
    cv.coopVecReduceSumAccumulate(a[:0], m, 0)               # empty batch: nothing to do
