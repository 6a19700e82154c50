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


# ---------------------------------------------------------------------------------------------
# every other plain element type: the scalar definition (hlsl.meta.slang:33261-33315, :33344-33352)
# ---------------------------------------------------------------------------------------------

NPT = {CT.Float16: np.float16, CT.Float32: np.float32, CT.Float64: np.float64, CT.SignedInt8: np.int8,
       CT.UnsignedInt8: np.uint8, CT.SignedInt16: np.int16, CT.UnsignedInt16: np.uint16, CT.SignedInt32: np.int32,
       CT.UnsignedInt32: np.uint32, CT.SignedInt64: np.int64, CT.UnsignedInt64: np.uint64}
TORCHT = {np.dtype(np.float16): torch.float16, np.dtype(np.float32): torch.float32, np.dtype(np.float64): torch.float64,
          np.dtype(np.int8): torch.int8, np.dtype(np.uint8): torch.uint8, np.dtype(np.int16): torch.int16,
          np.dtype(np.uint16): torch.uint16, np.dtype(np.int32): torch.int32, np.dtype(np.uint32): torch.uint32,
          np.dtype(np.int64): torch.int64, np.dtype(np.uint64): torch.uint64}


def typed(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(a.shape[0], -1)).to(DEV).view(TORCHT[a.dtype])


def draw(rng, ct, shape, small=False):
    dt = NPT[ct]
    if np.dtype(dt).kind == "f":
        return (rng.standard_normal(shape) * 2.0).astype(dt)
    info = np.iinfo(dt)
    lo, hi = (max(info.min, -9), min(info.max, 9)) if small else (info.min, info.max)
    return rng.integers(lo, hi, shape, dtype=dt, endpoint=True)


INT_PAIRS = [(CT.SignedInt8, CT.SignedInt32), (CT.UnsignedInt8, CT.UnsignedInt16), (CT.SignedInt16, CT.SignedInt64),
             (CT.SignedInt32, CT.SignedInt8), (CT.UnsignedInt32, CT.UnsignedInt64), (CT.SignedInt64, CT.SignedInt64),
             (CT.UnsignedInt16, CT.SignedInt32), (CT.UnsignedInt64, CT.UnsignedInt8), (CT.SignedInt32, CT.SignedInt32)]


@pytest.mark.parametrize("t_ct,m_ct", INT_PAIRS)
@pytest.mark.parametrize("layout", [ML.RowMajor, ML.ColumnMajor])
def test_outer_product_integer_types_bit_exact(t_ct, m_ct, layout):
    # product in T (wraps to T's width), cast to the matrix type (sign- or zero-extended, or cut), summed modulo the
    # matrix type's width: numpy's same-type integer arithmetic is exactly that, and the order of the samples is free
    rng = np.random.default_rng(int(t_ct) * 100 + int(m_ct))
    B, M, N = 777, 7, 5
    a = draw(rng, t_ct, (B, M)); b = draw(rng, t_ct, (B, N))
    mt = NPT[m_ct]
    before = draw(rng, m_ct, (M, N))
    with np.errstate(over="ignore"):
        prod = (a[:, :, None] * b[:, None, :]).astype(mt)             # [B, M, N], wrapped twice
        want = before + prod.sum(axis=0, dtype=mt)
    stored = np.ascontiguousarray(before if layout == ML.RowMajor else before.T)
    d = as_bytes(to_dev(stored))
    stride = stored.shape[1] * stored.itemsize
    cv.coopVecOuterProductAccumulate(typed(a), typed(b), d, 0, stride, layout, m_ct)
    assert cv.lastKernelName().startswith("outerScalarKernel"), cv.lastKernelName()
    got = d.cpu().numpy().view(mt).reshape(stored.shape)
    got = got if layout == ML.RowMajor else got.T
    assert np.array_equal(got, want)


FLOAT_PAIRS = [(CT.Float32, CT.Float32), (CT.Float32, CT.Float64), (CT.Float64, CT.Float64), (CT.Float64, CT.Float32),
               (CT.Float16, CT.Float64), (CT.Float32, CT.Float16), (CT.SignedInt16, CT.Float32), (CT.UnsignedInt8, CT.Float64)]


@pytest.mark.parametrize("t_ct,m_ct", FLOAT_PAIRS)
def test_outer_product_float_destinations(t_ct, m_ct):
    # the products (rounded to T) summed over the batch: float64 of the same products, with the float bar of the
    # destination type on the sum of magnitudes
    rng = np.random.default_rng(int(t_ct) * 100 + int(m_ct) + 1)
    B, M, N = 1500, 9, 6
    a = draw(rng, t_ct, (B, M), small=True); b = draw(rng, t_ct, (B, N), small=True)
    mt = NPT[m_ct]
    before = rng.standard_normal((M, N)).astype(mt)
    with np.errstate(over="ignore"):
        prod = (a[:, :, None] * b[:, None, :]).astype(np.float64)      # the product in T, exactly representable in float64
    want = before.astype(np.float64) + prod.sum(axis=0)
    mag = np.abs(before.astype(np.float64)) + np.abs(prod).sum(axis=0)
    d = as_bytes(to_dev(before))
    cv.coopVecOuterProductAccumulate(typed(a), typed(b), d, 0, N * before.itemsize, ML.RowMajor, m_ct)
    # (fp32 vectors into an fp32 matrix have a kernel on the matrix pipeline; every other pair is the scalar definition)
    kernel = "outerProductF32Kernel" if (t_ct, m_ct) == (CT.Float32, CT.Float32) else "outerScalarKernel"
    assert cv.lastKernelName().startswith(kernel), cv.lastKernelName()
    got = d.cpu().numpy().view(mt).reshape(M, N).astype(np.float64)
    eps = {np.float16: 2.0 ** -10, np.float32: 2.0 ** -20, np.float64: 2.0 ** -48}[mt]
    assert (np.abs(got - want) <= eps * mag).all()


def test_outer_product_float_vectors_into_integers_and_optimal_layout():
    rng = np.random.default_rng(99)
    B, M, N = 300, 6, 4
    a = (rng.standard_normal((B, M)) * 3).astype(np.float32); b = (rng.standard_normal((B, N)) * 3).astype(np.float32)
    # cast<int>(product): towards zero, per product
    want = np.trunc((a[:, :, None] * b[:, None, :]).astype(np.float32)).astype(np.int64).sum(axis=0).astype(np.int32)
    d = torch.zeros(M * N, dtype=torch.int32, device=DEV)
    cv.coopVecOuterProductAccumulate(typed(a), typed(b), as_bytes(d), 0, N * 4, ML.RowMajor, CT.SignedInt32)
    assert np.array_equal(d.cpu().numpy().reshape(M, N), want)
    # fp32 vectors into an fp32 TrainingOptimal matrix (the layout the reference asks for on hardware), read back by convert
    size = cv.getCooperativeVectorMatrixSize(M, N, CT.Float32, ML.TrainingOptimal)
    t = torch.zeros(size, dtype=torch.uint8, device=DEV)
    cv.coopVecOuterProductAccumulate(typed(a), typed(b), t, 0, 0, ML.TrainingOptimal, CT.Float32)
    row = torch.zeros(M * N * 4, dtype=torch.uint8, device=DEV)
    D = cv.CooperativeVectorMatrixDesc
    cv.convertCooperativeVectorMatrix(row, [D(M, N, CT.Float32, ML.RowMajor, M * N * 4, 0, N * 4)],
                                      t, [D(M, N, CT.Float32, ML.TrainingOptimal, size, 0, 0)])
    ref = a.astype(np.float64).T @ b.astype(np.float64)
    assert np.allclose(row.view(torch.float32).cpu().numpy().reshape(M, N), ref, rtol=1e-5, atol=1e-4)


def test_scalar_accumulate_equals_the_slang_operator_sample_by_sample():
    # the fallback itself (oracle: cvo_slang_*), applied to one sample after the other: exact for integer
    # destinations, and for a single sample also for fp32
    rng = np.random.default_rng(5)
    B, M, N = 40, 4, 6
    for t_ct, m_ct, o_t, o_m in ((CT.SignedInt32, CT.SignedInt32, ob.S32, ob.S32), (CT.UnsignedInt32, CT.UnsignedInt8, ob.U32, ob.U8),
                                 (CT.Float32, CT.SignedInt32, ob.F32, ob.S32), (CT.SignedInt32, CT.SignedInt8, ob.S32, ob.S8)):
        a = draw(rng, t_ct, (B, M), small=True); b = draw(rng, t_ct, (B, N), small=True)
        mat = draw(rng, m_ct, (M, N))
        ref = mat.copy()
        for s in range(B):
            assert ob.lib().cvo_slang_outer_product_accumulate(ob.ptr(a[s]), M, ob.ptr(b[s]), N, o_t, ob.ptr(ref), 0, N * ref.itemsize,
                                                               ob.ROW, o_m, ob.HALF_RNE) == 0
        d = as_bytes(to_dev(mat))
        cv.coopVecOuterProductAccumulate(typed(a), typed(b), d, 0, N * mat.itemsize, ML.RowMajor, m_ct)
        assert np.array_equal(d.cpu().numpy().view(mat.dtype).reshape(M, N), ref), (t_ct, m_ct)
    a = draw(rng, CT.Float32, (1, M)); b = draw(rng, CT.Float32, (1, N)); mat = draw(rng, CT.Float32, (M, N))
    ref = mat.copy()
    assert ob.lib().cvo_slang_outer_product_accumulate(ob.ptr(a[0]), M, ob.ptr(b[0]), N, ob.F32, ob.ptr(ref), 0, N * 4, ob.ROW, ob.F32, ob.HALF_RNE) == 0
    d = as_bytes(to_dev(mat))
    cv.coopVecOuterProductAccumulate(typed(a), typed(b), d, 0, N * 4, ML.RowMajor, CT.Float32)
    assert np.array_equal(d.cpu().numpy().view(np.uint32), ref.view(np.uint32).reshape(-1))
    # reduce-sum: the destination has the vectors' type
    for t_ct, o_t in ((CT.SignedInt32, ob.S32), (CT.UnsignedInt32, ob.U32)):
        v = draw(rng, t_ct, (B, 9)); buf = draw(rng, t_ct, (9,))
        ref = buf.copy()
        for s in range(B):
            assert ob.lib().cvo_slang_reduce_sum_accumulate(ob.ptr(v[s]), 9, o_t, ob.ptr(ref), 0, ob.HALF_RNE) == 0
        d = as_bytes(to_dev(buf))
        cv.coopVecReduceSumAccumulate(typed(v), d, 0)
        assert cv.lastKernelName().startswith("outerScalarKernel"), cv.lastKernelName()
        assert np.array_equal(d.cpu().numpy().view(buf.dtype), ref)


@pytest.mark.parametrize("t_ct", [CT.SignedInt8, CT.UnsignedInt16, CT.SignedInt64, CT.UnsignedInt64, CT.Float32, CT.Float64])
def test_reduce_sum_every_plain_type(t_ct):
    rng = np.random.default_rng(int(t_ct) + 300)
    B, N = 5000, 37
    v = draw(rng, t_ct, (B, N)); buf = draw(rng, t_ct, (N,))
    dt = NPT[t_ct]
    d = as_bytes(to_dev(buf))
    padded = torch.zeros((B, N + 3), dtype=TORCHT[np.dtype(dt)], device=DEV); padded[:, :N] = typed(v)     # strided rows
    cv.coopVecReduceSumAccumulate(padded[:, :N], d, 0)
    got = d.cpu().numpy().view(dt)
    if np.dtype(dt).kind == "f":
        want = buf.astype(np.float64) + v.astype(np.float64).sum(axis=0)
        mag = np.abs(buf.astype(np.float64)) + np.abs(v.astype(np.float64)).sum(axis=0)
        assert (np.abs(got.astype(np.float64) - want) <= (2.0 ** -20 if dt == np.float32 else 2.0 ** -48) * mag).all()
    else:
        with np.errstate(over="ignore"):
            assert np.array_equal(got, buf + v.sum(axis=0, dtype=dt))      # modulo 2^width
    with pytest.raises(cv.CoopVecError) as e:                              # the buffer has the vectors' type
        cv.coopVecReduceSumAccumulate(typed(v), d, 0, bufferType=CT.Float16 if t_ct != CT.Float16 else CT.Float32)
    assert e.value.result == cv.SLANG_E_NOT_AVAILABLE


# ---------------------------------------------------------------------------------------------
# fp32 vectors into fp32 destinations: the kernel on v_mfma_f32_16x16x4_f32
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("M,N,B", [(9, 6, 1), (9, 6, 5), (64, 64, 4096), (70, 33, 1500), (128, 16, 70001), (1, 1, 333), (16, 17, 19),
                                   (17, 16, 64), (130, 129, 300)])
@pytest.mark.parametrize("layout", [ML.RowMajor, ML.ColumnMajor, ML.TrainingOptimal])
def test_fp32_outer_product_against_fp64(M, N, B, layout):
    rng = np.random.default_rng(M * 1000 + N * 10 + B)
    a = (rng.standard_normal((B, M)) * 2).astype(np.float32); b = (rng.standard_normal((B, N)) * 2).astype(np.float32)
    before = rng.standard_normal((M, N)).astype(np.float32)
    prod = a.astype(np.float64)[:, :, None] * b.astype(np.float64)[:, None, :]
    want = before.astype(np.float64) + prod.sum(axis=0)
    mag = np.abs(before.astype(np.float64)) + np.abs(prod).sum(axis=0)
    D = cv.CooperativeVectorMatrixDesc
    stride = {ML.RowMajor: N * 4, ML.ColumnMajor: M * 4, ML.TrainingOptimal: 0}[layout]
    size = cv.getCooperativeVectorMatrixSize(M, N, CT.Float32, layout, stride)
    row_desc = D(M, N, CT.Float32, ML.RowMajor, M * N * 4, 0, N * 4)
    results = []
    for _ in range(2):
        d = torch.zeros(size, dtype=torch.uint8, device=DEV)
        cv.convertCooperativeVectorMatrix(d, [D(M, N, CT.Float32, layout, size, 0, stride)], as_bytes(to_dev(before)), [row_desc])
        # strided vectors: rows of a wider array
        wide_a = torch.zeros((B, M + 3), dtype=torch.float32, device=DEV); wide_a[:, :M] = to_dev(a)
        cv.coopVecOuterProductAccumulate(wide_a[:, :M], to_dev(b), d, 0, stride, layout, CT.Float32)
        assert cv.lastKernelName().startswith("outerProductF32Kernel"), cv.lastKernelName()
        row = torch.zeros(M * N * 4, dtype=torch.uint8, device=DEV)
        cv.convertCooperativeVectorMatrix(row, [row_desc], d, [D(M, N, CT.Float32, layout, size, 0, stride)])
        results.append(row.view(torch.float32).cpu().numpy().reshape(M, N).copy())
    assert np.array_equal(results[0].view(np.uint32), results[1].view(np.uint32))          # no atomics: the same bits every time
    assert (np.abs(results[0].astype(np.float64) - want) <= 2.0 ** -20 * mag).all()


def test_fp32_outer_product_one_sample_is_the_operator_itself():
    # one sample: matrix[i][j] += a[i] * b[j] with the product rounded to float, the bits of the Slang fallback
    rng = np.random.default_rng(77)
    M, N = 37, 21
    a = draw(rng, CT.Float32, (1, M)); b = draw(rng, CT.Float32, (1, N)); mat = draw(rng, CT.Float32, (M, N))
    ref = mat.copy()
    assert ob.lib().cvo_slang_outer_product_accumulate(ob.ptr(a[0]), M, ob.ptr(b[0]), N, ob.F32, ob.ptr(ref), 0, N * 4, ob.ROW, ob.F32, ob.HALF_RNE) == 0
    d = as_bytes(to_dev(mat))
    cv.coopVecOuterProductAccumulate(typed(a), typed(b), d, 0, N * 4, ML.RowMajor, CT.Float32)
    assert np.array_equal(d.cpu().numpy().view(np.uint32), ref.view(np.uint32).reshape(-1))


def test_fp32_outer_product_infinite_element_stays_in_its_row_and_column():
    # an infinity in the last sample of a ragged batch: the samples past the end that the kernel's loads repeat contribute
    # nothing, and rows and columns without the infinite element stay finite
    rng = np.random.default_rng(78)
    B, M, N = 21, 20, 18
    a = (rng.standard_normal((B, M))).astype(np.float32); b = (rng.standard_normal((B, N))).astype(np.float32)
    a[B - 1, 3] = np.inf
    b[B - 1, 5] = 0.0
    d = torch.zeros(M * N, dtype=torch.float32, device=DEV)
    cv.coopVecOuterProductAccumulate(to_dev(a), to_dev(b), d.view(torch.uint8), 0, N * 4, ML.RowMajor, CT.Float32)
    got = d.cpu().numpy().reshape(M, N)
    with np.errstate(invalid="ignore"):
        want = (a.astype(np.float64)[:, :, None] * b.astype(np.float64)[:, None, :]).sum(axis=0)
    fin = np.isfinite(want)
    assert np.array_equal(np.isfinite(got), fin) and np.array_equal(np.isnan(got), np.isnan(want))
    assert not fin[3].any() and fin[np.arange(M) != 3].all()
    assert np.allclose(got[fin], want[fin], rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("N,B", [(1, 7), (9, 5000), (64, 100000), (200, 333), (16, 16)])
def test_fp32_reduce_sum_against_fp64(N, B):
    rng = np.random.default_rng(N * 31 + B)
    v = (rng.standard_normal((B, N)) * 3).astype(np.float32)
    buf = rng.standard_normal(N).astype(np.float32)
    want = buf.astype(np.float64) + v.astype(np.float64).sum(axis=0)
    mag = np.abs(buf.astype(np.float64)) + np.abs(v.astype(np.float64)).sum(axis=0)
    out = []
    for _ in range(2):
        d = as_bytes(to_dev(buf))
        cv.coopVecReduceSumAccumulate(to_dev(v), d, 0)
        assert cv.lastKernelName().startswith("outerProductF32Kernel"), cv.lastKernelName()
        out.append(d.cpu().numpy().view(np.float32).copy())
    assert np.array_equal(out[0].view(np.uint32), out[1].view(np.uint32))
    assert (np.abs(out[0].astype(np.float64) - want) <= 2.0 ** -20 * mag).all()
