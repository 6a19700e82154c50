"""Pins the CPU oracle against the reference's own golden vectors (tests/golden/README.md lists
the reference test each one comes from) and against what the mathematics fixes."""
import json
import os

import numpy as np
import pytest

import oracle_binding as ob
from oracle_binding import F16, F32, S8, S32, U32, S8P, ROW, COL, INF_OPT, TRAIN_OPT, HALF_RNE, HALF_SLANG

G = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "coopvec_goldens.json")))
L = ob.lib()


def slang_matmul(inp, U, packedK, inInterp, k, T, M, mat, matOff, matInterp, layout, transpose, stride,
                 bias=None, biasInterp=-1, init=None, half_mode=HALF_RNE):
    res_dtype = np.float16 if T == F16 else (np.float32 if T == F32 else np.int32)
    res = np.zeros(M, res_dtype) if init is None else np.array(init, res_dtype)
    rc = L.cvo_slang_matmul(ob.ptr(inp), U, packedK, inInterp, k, ob.ptr(res), T, M, ob.ptr(mat), matOff,
                            matInterp, layout, int(transpose), stride,
                            ob.ptr(bias) if bias is not None else None, 0, biasInterp,
                            int(init is not None), half_mode)
    return rc, res


W16 = np.array(G["matmul_f16"]["matrix_row_major_4x4"], np.float16)
X16 = np.array(G["matmul_f16"]["input"], np.float16)
W8 = np.array(G["matmul_i8_packed"]["matrix_row_major_4x4_bytes"], np.int8)
X8 = np.array(G["matmul_i8_packed"]["input_bytes"], np.int8)


@pytest.mark.parametrize("half_mode", [HALF_RNE, HALF_SLANG])
def test_slang_matmul_f16_goldens(half_mode):
    rc, r = slang_matmul(X16, F16, 4, F16, 4, F16, 4, W16, 0, F16, ROW, False, 8, half_mode=half_mode)
    assert rc == 0 and r.tolist() == G["matmul_f16"]["expected"]
    b = np.array(G["matmul_bias_f16"]["bias"], np.float16)
    rc, r = slang_matmul(X16, F16, 4, F16, 4, F16, 4, W16, 0, F16, ROW, False, 8, b, F16, half_mode=half_mode)
    assert rc == 0 and r.tolist() == G["matmul_bias_f16"]["expected"]
    rc, r = slang_matmul(X16, F16, 4, F16, 4, F16, 4, W16, 0, F16, ROW, False, 8,
                         init=G["matmul_f16_mut"]["initial"], half_mode=half_mode)
    assert rc == 0 and r.tolist() == G["matmul_f16_mut"]["expected"]
    rc, r = slang_matmul(X16, F16, 4, F16, 4, F16, 4, W16, 0, F16, ROW, False, 8, b, F16,
                         init=G["matmul_bias_f16_mut"]["initial"], half_mode=half_mode)
    assert rc == 0 and r.tolist() == G["matmul_bias_f16_mut"]["expected"]


def test_slang_matmul_i8_packed_goldens():
    xp = X8.view(np.uint32)
    rc, r = slang_matmul(xp, U32, 1, S8P, 4, S32, 4, W8, 0, S8, ROW, False, 4)
    assert rc == 0 and r.tolist() == G["matmul_i8_packed"]["expected"]
    rc, r = slang_matmul(xp, U32, 1, S8P, 4, S32, 4, W8, 0, S8, ROW, False, 4,
                         init=G["matmul_i8_packed_mut"]["initial"])
    assert rc == 0 and r.tolist() == G["matmul_i8_packed_mut"]["expected"]
    b = np.array(G["matmul_bias_i8_packed"]["bias_int32"], np.int32)
    rc, r = slang_matmul(xp, U32, 1, S8P, 4, S32, 4, W8, 0, S8, ROW, False, 4, b, S32)
    assert rc == 0 and r.tolist() == G["matmul_bias_i8_packed"]["expected"]
    rc, r = slang_matmul(xp, U32, 1, S8P, 4, S32, 4, W8, 0, S8, ROW, False, 4, b, S32,
                         init=G["matmul_bias_i8_packed_mut"]["initial"])
    assert rc == 0 and r.tolist() == G["matmul_bias_i8_packed_mut"]["expected"]


def test_slang_packed_sign_extension_and_byte_order():
    # element i = byte i%4 of word i/4, sign-extended (hlsl.meta.slang:32850-32855)
    x = np.array([-1, 2, -128, 127, 5, -6, 7, -8], np.int8)
    W = np.arange(1, 17, dtype=np.int8).reshape(2, 8)
    rc, r = slang_matmul(x.view(np.uint32), U32, 2, S8P, 8, S32, 2, W, 0, S8, ROW, False, 8)
    assert rc == 0
    assert r.tolist() == (W.astype(np.int64) @ x.astype(np.int64)).tolist()


def test_slang_static_assert_rules():
    # packed matrix interpretation is rejected (:32803); fp8 has no stride case (:32666-32668)
    rc, _ = slang_matmul(X8.view(np.uint32), U32, 1, S8P, 4, S32, 4, W8, 0, S8P, ROW, False, 4)
    assert rc != 0
    rc, _ = slang_matmul(X16, F16, 4, F16, 4, F16, 4, W16, 0, ob.E4M3, ROW, False, 8)
    assert rc != 0
    # non-packed input needs k == vector length (:32798)
    rc, _ = slang_matmul(X16, F16, 4, F16, 3, F16, 4, W16, 0, F16, ROW, False, 8)
    assert rc != 0
    assert L.cvo_component_type_stride(ob.E4M3) == -1 and L.cvo_component_type_stride(F16) == 2
    assert L.cvo_component_type_stride(S8P) == 4 and L.cvo_component_packing_factor(S8P) == 4
    assert L.cvo_component_scalar_type(ob.E4M3) == 17 and L.cvo_component_scalar_type(S8P) == 10


def test_slang_column_major_is_transpose():
    # ColumnMajor with the same stride reads the transpose (:32862-32864; fflayer.slang:46-55)
    rng = np.random.default_rng(1)
    W = rng.integers(-8, 8, (6, 4)).astype(np.float16)     # 6 rows x 4 cols, row-major, stride 8
    g = rng.integers(-4, 4, 6).astype(np.float16)
    rc, r = slang_matmul(g, F16, 6, F16, 6, F16, 4, W, 0, F16, COL, False, 8)
    assert rc == 0
    assert r.astype(np.float64).tolist() == (W.astype(np.float64).T @ g.astype(np.float64)).tolist()
    # every non-ColumnMajor layout is read as row-major by the fallback
    x = rng.integers(-4, 4, 4).astype(np.float16)
    for layout in (ROW, INF_OPT, TRAIN_OPT):
        rc, r = slang_matmul(x, F16, 4, F16, 4, F16, 6, W, 0, F16, layout, False, 8)
        assert rc == 0 and r.astype(np.float64).tolist() == (W.astype(np.float64) @ x.astype(np.float64)).tolist()


def test_slang_fp16_accumulates_in_half():
    # result[i] += w*v in half: 2048 + 1 is not representable, so 1's added after 2048 are lost
    x = np.array([1, 1, 1, 1], np.float16)
    W = np.array([[2048, 1, 1, 1]], np.float16)
    rc, r = slang_matmul(x, F16, 4, F16, 4, F16, 1, W, 0, F16, ROW, False, 8)
    assert rc == 0 and float(r[0]) == 2048.0
    # with an fp32 result type the same sum is exact
    rc, r = slang_matmul(x, F16, 4, F16, 4, F32, 1, W, 0, F16, ROW, False, 8)
    assert rc == 0 and float(r[0]) == 2051.0
    # the two `half` flavours differ exactly on ties: 2049 -> 2048 (even) vs 2050 (away)
    W2 = np.array([[2048, 1, 0, 0]], np.float16)
    _, r_rne = slang_matmul(x, F16, 4, F16, 4, F16, 1, W2, 0, F16, ROW, False, 8, half_mode=HALF_RNE)
    _, r_soft = slang_matmul(x, F16, 4, F16, 4, F16, 1, W2, 0, F16, ROW, False, 8, half_mode=HALF_SLANG)
    assert float(r_rne[0]) == 2048.0 and float(r_soft[0]) == 2050.0


def test_slang_outer_product_golden():
    g = G["outer_product_f16"]
    a = np.array(g["a"], np.float16); b = np.array(g["b"], np.float16)
    mat = np.zeros(32, np.float16); mat[0] = g["prestored_at_0"]
    # the golden is the row-major 4x8 image; on the fallback every non-ColumnMajor layout
    # is addressed row-major with the given stride (8 halfs = 16 bytes here)
    rc = L.cvo_slang_outer_product_accumulate(ob.ptr(a), 4, ob.ptr(b), 8, F16, ob.ptr(mat), 0, 16, TRAIN_OPT, F16, HALF_RNE)
    assert rc == 0 and mat.tolist() == g["expected_row_major_4x8"]
    # ColumnMajor stores the transpose
    mat = np.zeros(32, np.float16)
    rc = L.cvo_slang_outer_product_accumulate(ob.ptr(a), 4, ob.ptr(b), 8, F16, ob.ptr(mat), 0, 8, COL, F16, HALF_RNE)
    assert rc == 0
    assert mat.reshape(8, 4).astype(np.float64).tolist() == np.outer(b, a).astype(np.float64).tolist()
    # fp32 destination
    m32 = np.zeros(32, np.float32)
    rc = L.cvo_slang_outer_product_accumulate(ob.ptr(a), 4, ob.ptr(b), 8, F16, ob.ptr(m32), 0, 32, ROW, F32, HALF_RNE)
    assert rc == 0 and m32.reshape(4, 8).tolist() == np.outer(a, b).astype(np.float32).tolist()


def test_slang_reduce_sum_goldens():
    g = G["reduce_sum_f16"]
    v = np.array(g["v"], np.float16)
    buf = np.zeros(4, np.float16); buf[0] = g["prestored_at_0"]
    assert L.cvo_slang_reduce_sum_accumulate(ob.ptr(v), 4, F16, ob.ptr(buf), 0, HALF_RNE) == 0
    assert buf.tolist() == g["expected"]
    g8 = G["reduce_sum_8threads"]
    buf = np.zeros(4, np.float16); v = np.array(g8["v"], np.float16)
    for _ in range(g8["threads"]):
        L.cvo_slang_reduce_sum_accumulate(ob.ptr(v), 4, F16, ob.ptr(buf), 0, HALF_RNE)
    assert buf.tolist() == g8["expected"]
    # closed form of tests/neural/bias-sum-reduce.slang: 128 threads x (i+1)/128 -> i+1
    buf = np.zeros(8, np.float32)
    v = ((np.arange(8) + 1) / 128.0).astype(np.float32)
    for _ in range(128):
        L.cvo_slang_reduce_sum_accumulate(ob.ptr(v), 8, F32, ob.ptr(buf), 0, HALF_RNE)
    assert buf.tolist() == (np.arange(8) + 1.0).tolist()


def test_slang_dispatch_matches_single_thread_calls():
    rng = np.random.default_rng(3)
    B, M, K = 600, 5, 8
    x = rng.standard_normal((B, K)).astype(np.float16)
    W = rng.standard_normal((M, K)).astype(np.float16)
    b = rng.standard_normal(M).astype(np.float16)
    out = np.zeros((B, M), np.float16)
    rc = L.cvo_slang_dispatch_matmul_add(0, (B + 255) // 256, B, ob.ptr(x), K * 2, F16, K, F16, K,
                                         ob.ptr(out), M * 2, F16, M, ob.ptr(W), 0, F16, ROW, 0, K * 2,
                                         ob.ptr(b), 0, F16, HALF_RNE)
    assert rc == 0
    for s in (0, 255, 256, 599):
        _, r = slang_matmul(x[s].copy(), F16, K, F16, K, F16, M, W, 0, F16, ROW, False, K * 2, b, F16)
        assert r.tolist() == out[s].tolist()
    # group range is honoured: only group 1 written
    out2 = np.zeros((B, M), np.float16)
    L.cvo_slang_dispatch_matmul_add(1, 2, B, ob.ptr(x), K * 2, F16, K, F16, K, ob.ptr(out2), M * 2, F16, M,
                                    ob.ptr(W), 0, F16, ROW, 0, K * 2, ob.ptr(b), 0, F16, HALF_RNE)
    assert not out2[:256].any() and (out2[256:512] == out[256:512]).all() and not out2[512:].any()


# ---- parity reference ---------------------------------------------------------------------

def test_ref_matmul_goldens_and_fp64():
    out, _ = ob.ref_matmul_f32(X16.reshape(1, 4), F16, W16, F16, ROW, 8, 4, 4)
    assert out[0].tolist() == G["matmul_f16"]["expected"]
    b = np.array(G["matmul_bias_f16"]["bias"], np.float16)
    out, _ = ob.ref_matmul_f32(X16.reshape(1, 4), F16, W16, F16, ROW, 8, 4, 4, b, F16)
    assert out[0].tolist() == G["matmul_bias_f16"]["expected"]
    oi = ob.ref_matmul_i32(X8.reshape(1, 4), W8, ROW, 4, 4, 4, np.array([5, 6, 7, 8], np.int32))
    assert oi[0].tolist() == G["matmul_bias_i8_packed"]["expected"]
    # brute force in fp64 on random shapes, all layouts of the same logical matrix
    rng = np.random.default_rng(7)
    for (M, K) in [(3, 5), (16, 16), (64, 64), (17, 33), (128, 40)]:
        x = rng.standard_normal((9, K)).astype(np.float16)
        W = (rng.standard_normal((M, K)) / np.sqrt(K)).astype(np.float16)
        b = rng.uniform(-0.1, 0.1, M).astype(np.float16)
        want = x.astype(np.float64) @ W.astype(np.float64).T + b.astype(np.float64)
        for layout in (ROW, COL, INF_OPT, TRAIN_OPT):
            size = L.cvo_layout_matrix_size(M, K, F16, layout, 0)
            buf = np.zeros(size, np.uint8)
            assert L.cvo_layout_convert(ob.ptr(buf), M, K, F16, layout, 0, ob.ptr(W), F16, ROW, 0) == 0
            got, ab = ob.ref_matmul_f32(x, F16, buf, F16, layout, 0, M, K, b, F16)
            assert np.max(np.abs(got - want)) <= 1e-5 * max(1.0, np.max(ab))
    # fp32 vectors against a Float32 matrix, the same way (and the Slang operator itself on data it computes exactly)
    for (M, K) in [(4, 4), (24, 40), (64, 64)]:
        x = rng.standard_normal((9, K)).astype(np.float32)
        W = (rng.standard_normal((M, K)) / np.sqrt(K)).astype(np.float32)
        b = rng.uniform(-0.1, 0.1, M).astype(np.float32)
        want = x.astype(np.float64) @ W.astype(np.float64).T + b.astype(np.float64)
        for layout in (ROW, COL, INF_OPT, TRAIN_OPT):
            size = L.cvo_layout_matrix_size(M, K, F32, layout, 0)
            buf = np.zeros(size, np.uint8)
            assert L.cvo_layout_convert(ob.ptr(buf), M, K, F32, layout, 0, ob.ptr(W), F32, ROW, 0) == 0
            got, ab = ob.ref_matmul_f32(x, F32, buf, F32, layout, 0, M, K, b, F32)
            assert (np.abs(got - want) <= (K + 1) * 2.0 ** -23 * ab).all()
    xi = rng.integers(-8, 9, (3, 12)).astype(np.float32)
    Wi = rng.integers(-8, 9, (20, 12)).astype(np.float32)
    bi = rng.integers(-100, 100, 20).astype(np.float32)
    assert np.array_equal(ob.slang_matmul(xi, F32, F32, 12, F32, 20, Wi.view(np.uint8).ravel(), F32, ROW, 48, bi, F32),
                          xi @ Wi.T + bi)
    # integer path: exact, and wraps like int32 only beyond 2^31 (never at these sizes)
    x = rng.integers(-128, 128, (5, 128), dtype=np.int8)
    W = rng.integers(-127, 128, (128, 128), dtype=np.int8)
    b = rng.integers(-65536, 65537, 128).astype(np.int32)
    for layout, buf, stride in ((ROW, W, 128), (COL, np.ascontiguousarray(W.T), 128)):
        got = ob.ref_matmul_i32(x, buf.view(np.uint8).ravel(), layout, stride, 128, 128, b)
        assert (got.astype(np.int64) == x.astype(np.int64) @ W.astype(np.int64).T + b).all()


def test_ref_mlp_forward_ffn_closed_form():
    f = G["ffn_forward"]
    specs = [dict(W=np.array(f["W1"], np.float16), b=np.array(f["b1"], np.float16)),
             dict(W=np.array(f["W2"], np.float16), b=np.array(f["b2"], np.float16))]
    x = np.array([f["x"]], np.float16)
    y, acts = ob.ref_mlp_forward(specs, x, F16, want_acts=True)
    assert acts[0][0].tolist() == f["h"] and y[0].tolist() == f["y"]
    # ReLU and leaky ReLU follow max(z,0) / max(z, z*slope) in half
    specs[0]["act"] = ob.ACT_RELU
    _, acts = ob.ref_mlp_forward(specs, x, F16, want_acts=True)
    assert acts[0][0].tolist() == [6.0, 0.0]
    specs[0]["act"] = ob.ACT_LEAKY; specs[0]["slope"] = float(np.float16(0.001))
    _, acts = ob.ref_mlp_forward(specs, x, F16, want_acts=True)
    assert acts[0][0].tolist() == [6.0, float(np.float16(np.float32(-7.25) * np.float32(np.float16(0.001))))]


def test_ref_mlp_train_ffn_closed_form():
    f, bwd = G["ffn_forward"], G["ffn_backward"]
    specs = [dict(W=np.array(f["W1"], np.float16), b=np.array(f["b1"], np.float16)),
             dict(W=np.array(f["W2"], np.float16), b=np.array(f["b2"], np.float16))]
    x = np.array([f["x"]], np.float16)
    # seed dL/dy = 2*(y - t)*scale = 1 with y = -40.5, t = -41
    t = np.array([[-41.0]], np.float16)
    dW, dB, loss = ob.ref_mlp_train(specs, x, t, 1.0)
    assert dW[0].tolist() == bwd["dW1"] and dB[0].tolist() == bwd["db1"]
    assert dW[1].tolist() == bwd["dW2"] and dB[1].tolist() == bwd["db2"]
    assert loss == 0.25


def test_ref_mlp_train_finite_differences():
    # small values so that fp16 carrier rounding stays far below the finite-difference step
    rng = np.random.default_rng(11)
    dims = [3, 4, 4, 2]
    B = 7
    Ws = [rng.integers(-3, 4, (dims[i + 1], dims[i])).astype(np.float64) / 4 for i in range(3)]
    bs = [rng.integers(-2, 3, dims[i + 1]).astype(np.float64) / 4 for i in range(3)]
    x = rng.integers(-4, 5, (B, 3)).astype(np.float64) / 4
    t = rng.integers(-4, 5, (B, 2)).astype(np.float64) / 4

    def loss64(Ws_, bs_):
        h = x
        for i in range(3):
            h = h @ Ws_[i].T + bs_[i]
            if i < 2:
                h = np.maximum(h, 0)
        return np.sum((h - t) ** 2)

    specs = [dict(W=Ws[i].astype(np.float16), b=bs[i].astype(np.float16),
                  act=ob.ACT_RELU if i < 2 else ob.ACT_NONE) for i in range(3)]
    dW, dB, loss = ob.ref_mlp_train(specs, x.astype(np.float16), t.astype(np.float16), 1.0, tie_rule=False)
    assert abs(loss - loss64(Ws, bs)) < 1e-6
    # central finite differences of the fp64 model (weights where no ReLU sits within the
    # step of its kink); the oracle rounds its carriers to fp16, hence the 1% tolerance
    eps = 2.0 ** -10
    h = x
    zmin = np.inf
    for i in range(3):
        h = h @ Ws[i].T + bs[i]
        if i < 2:
            zmin = min(zmin, np.abs(h[h != 0]).min()); h = np.maximum(h, 0)
    assert zmin > 8 * eps
    for l in range(3):
        for idx in [(0, 0), (dims[l + 1] - 1, dims[l] - 1), (1, 1)]:
            Wp = [w.copy() for w in Ws]; Wm = [w.copy() for w in Ws]
            Wp[l][idx] += eps; Wm[l][idx] -= eps
            fd = (loss64(Wp, bs) - loss64(Wm, bs)) / (2 * eps)
            # units sitting exactly on the kink make the two one-sided slopes differ: skip those
            one_sided = (loss64(Wp, bs) - loss64(Ws, bs)) / eps
            if abs(one_sided - fd) > 0.05 * max(1.0, abs(fd)):
                continue
            assert abs(fd - dW[l][idx]) < 1e-2 * max(1.0, abs(fd)), (l, idx, fd, dW[l][idx])
    # float64 backprop with the "0 at a tie" rule; fp16 carriers of the oracle give ~1e-3 relative
    h = [x]
    z = []
    for i in range(3):
        zi = h[-1] @ Ws[i].T + bs[i]; z.append(zi)
        h.append(np.maximum(zi, 0) if i < 2 else zi)
    g = 2 * (h[-1] - t)
    for i in (2, 1, 0):
        if i < 2:
            g = g * (z[i] > 0)
        wantW, wantB = g.T @ h[i], g.sum(0)
        assert np.max(np.abs(dW[i] - wantW)) <= 3e-3 * np.max(np.abs(wantW))
        assert np.max(np.abs(dB[i] - wantB)) <= 3e-3 * np.max(np.abs(wantB))
        g = g @ Ws[i]


def test_ref_max_tie_rule():
    # z == 0 at the hidden unit: Slang's max derivative gives 0.5 each (diff.meta.slang:2258-2277)
    specs = [dict(W=np.array([[1.0]], np.float16), b=np.array([-1.0], np.float16), act=ob.ACT_RELU),
             dict(W=np.array([[2.0]], np.float16), b=None)]
    x = np.array([[1.0]], np.float16)
    t = np.array([[-0.5]], np.float16)         # y = 0, dL/dy = 2*(0+0.5) = 1
    dW, dB, _ = ob.ref_mlp_train(specs, x, t, 1.0, tie_rule=True)
    assert dB[0].tolist() == [1.0] and dW[0].tolist() == [[1.0]]      # 0.5 * (2*1)
    dW, dB, _ = ob.ref_mlp_train(specs, x, t, 1.0, tie_rule=False)
    assert dB[0].tolist() == [0.0]


def test_slang_matmul_with_64_bit_types_against_exact_arithmetic():
    """The 64-bit arms of the fallback's switch (hlsl.meta.slang:32873-32903) in the oracle: int64 / uint64
    results equal Python's exact integers modulo 2^64 (full-range operands, so the sums wrap), float64
    results equal numpy's float64 products and sums taken in the same order, and casts between widths
    follow C (sign extension, truncation to the low bits, nearest-even float conversions)."""
    rng = np.random.default_rng(64)
    B, k, M = 5, 13, 7
    NPT = {ob.S8: np.int8, ob.U16: np.uint16, ob.S32: np.int32, ob.S64: np.int64, ob.U64: np.uint64, ob.F32: np.float32, ob.F64: np.float64}

    def rand(ct, shape):
        if ct in (ob.F32, ob.F64):
            return rng.standard_normal(shape).astype(NPT[ct]) * 3
        info = np.iinfo(NPT[ct])
        return rng.integers(info.min, info.max, shape, dtype=NPT[ct], endpoint=True)

    for in_ct, w_ct, b_ct, r_ct in ((ob.S64, ob.S64, ob.S64, ob.S64), (ob.U64, ob.S32, ob.U16, ob.U64), (ob.S8, ob.U64, ob.S64, ob.S64),
                                    (ob.S64, ob.U64, ob.S32, ob.S32)):
        x, W, bias = rand(in_ct, (B, k)), rand(w_ct, (M, k)), rand(b_ct, (M,))
        got = ob.slang_matmul(x, in_ct, in_ct, k, r_ct, M, W.view(np.uint8).reshape(-1), w_ct, ob.ROW, k * W.itemsize, bias, b_ct)
        bits = 32 if r_ct == ob.S32 else 64
        mod = 1 << bits
        for b in range(B):
            for i in range(M):
                # cast<T> of each operand first (the low bits), then exact arithmetic modulo 2^bits
                acc = sum((int(W[i, j]) % mod) * (int(x[b, j]) % mod) for j in range(k)) + int(bias[i]) % mod
                assert int(got[b, i]) % mod == acc % mod
    for in_ct, w_ct, b_ct in ((ob.F64, ob.F64, ob.F64), (ob.F32, ob.F64, ob.S32), (ob.S32, ob.F64, ob.F32)):
        x, W, bias = rand(in_ct, (B, k)), rand(w_ct, (M, k)), rand(b_ct, (M,))
        got = ob.slang_matmul(x, in_ct, in_ct, k, ob.F64, M, W.view(np.uint8).reshape(-1), w_ct, ob.ROW, k * W.itemsize, bias, b_ct)
        acc = np.zeros((B, M), np.float64)
        for j in range(k):
            acc = acc + x[:, j:j + 1].astype(np.float64) * W[:, j][None, :].astype(np.float64)
        acc = acc + bias.astype(np.float64)[None, :]
        assert np.array_equal(got.view(np.uint64), acc.view(np.uint64))
    # a 64-bit matrix under a float result: cast<float>(int64) rounds to nearest even
    W = np.array([[(1 << 53) + 1, -(1 << 40) - 1]], np.int64); x = np.array([[1.0, 1.0]], np.float32)
    got = ob.slang_matmul(x, ob.F32, ob.F32, 2, ob.F32, 1, W.view(np.uint8).reshape(-1), ob.S64, ob.ROW, 16)
    assert got[0, 0] == np.float32(np.float32(float((1 << 53) + 1)) + np.float32(float(-(1 << 40) - 1)))
