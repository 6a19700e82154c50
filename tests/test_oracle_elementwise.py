"""The oracle's element-wise operators and their reverse-mode rules, pinned by the reference's own
test (tests/autodiff/coopvec.slang: every CHECK value of the element-wise blocks, reverse and forward
mode) and, for what that leaves open (the activations, operands away from the test's points), by
central differences and textbook identities."""
import json
import os

import numpy as np
import pytest

import elementwise_tape as T
import oracle_binding as ob

G = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "coopvec_goldens.json")))["autodiff_coopvec"]
CASES = ["compound", "common_math", "division_negation", "additional_math", "forward_arithmetic", "same_operand",
         "min_max_clamp_fma"]


class OracleOps:
    def __init__(self, dtype):
        self.dtype = dtype
        self.ct = ob.F32 if dtype == np.float32 else ob.F16

    def forward(self, op, a, b, c, param):
        return ob.elementwise(op, a, b, c, param)

    def backward(self, op, d_out, a, b, c, param):
        return ob.elementwise_backward(op, d_out, a, b, c, param)


def make(dtype):
    def f(v):
        return np.full(4, v, dtype) if np.isscalar(v) else np.array(v, dtype)
    return f


@pytest.mark.parametrize("name", CASES)
def test_reference_goldens_fp32(name):
    case = G[name]
    primal, dx, dy, tangent = T.run_case(OracleOps(np.float32), name, case, make(np.float32))
    # the CHECK lines are prefixes of the printed floats (six to seven significant digits)
    assert np.allclose(primal, case["primal"], rtol=5e-6, atol=1e-6)
    for got, key in ((dx, "dx"), (dy, "dy"), (tangent, "tangent")):
        if key in case:
            assert got is not None and np.allclose(got, case[key], rtol=5e-6, atol=1e-6), (key, got)


def test_gradients_against_central_differences():
    rng = np.random.default_rng(3)
    n = 64
    x = rng.uniform(0.3, 2.0, n).astype(np.float32)
    y = rng.uniform(0.3, 2.0, n).astype(np.float32)
    z = rng.uniform(2.1, 3.0, n).astype(np.float32)
    g = rng.uniform(-1, 1, n).astype(np.float32)
    h = 1e-3
    for op in range(23):
        if op == T.STEP:
            continue
        nops = T.N_OPERANDS.get(op, 1)
        ops = [x, y if nops >= 2 else None, z if nops >= 3 else None]
        if op == T.CLAMP:
            ops = [x, np.full(n, 0.8, np.float32), np.full(n, 1.5, np.float32)]
        grads = ob.elementwise_backward(op, g, ops[0], ops[1], ops[2], 0.1)
        for k in range(nops):
            if op == T.CLAMP and k > 0:
                continue
            lo = [o.astype(np.float64) if o is not None else None for o in ops]
            hi = [o.astype(np.float64) if o is not None else None for o in ops]
            lo[k] = lo[k] - h; hi[k] = hi[k] + h
            f = lambda v: ob.elementwise(op, *[o.astype(np.float32) if o is not None else None for o in v], 0.1).astype(np.float64)
            num = (f(hi) - f(lo)) / (2 * h) * g
            kink = np.zeros(n, bool)
            if op in (T.MIN, T.MAX):
                kink = np.abs(x - y) < 4 * h
            if op == T.CLAMP:
                kink = (np.abs(x - 0.8) < 4 * h) | (np.abs(x - 1.5) < 4 * h)
            assert np.allclose(grads[k][~kink], num[~kink], rtol=2e-2, atol=2e-3), (op, k)


def test_half_results_are_rounded_once_and_scale():
    # the oracle rounds its double results to half in one step: a*b + c = (1.5 + 1.5 ulp) - 2^-24 is below the tie
    a = np.full(4, 1.0009765625, np.float16); b = np.full(4, 1.5, np.float16); c = np.full(4, -2.0 ** -24, np.float16)
    assert (ob.elementwise(T.FMA, a, b, c, 0.0).view(np.uint16) == 0x3E01).all()
    c0 = np.zeros(4, np.float16)
    assert (ob.elementwise(T.FMA, a, b, c0, 0.0).view(np.uint16) == 0x3E02).all()       # the exact tie goes to even
    x = np.array([1.0, -2.5, 3.0, 0.1], np.float16)
    assert np.array_equal(ob.elementwise(T.SCALE, x, None, None, 0.3), (x.astype(np.float32) * np.float32(np.float16(0.3))).astype(np.float16))
    xf = x.astype(np.float32)
    assert np.array_equal(ob.elementwise(T.SCALE, xf, None, None, 0.3), (xf.astype(np.float64) * np.float64(np.float32(0.3))).astype(np.float32))
    da, _, _ = ob.elementwise_backward(T.SCALE, np.ones(4, np.float32), xf, None, None, 2.0)
    assert (da == 2.0).all()


def test_tie_rules_and_identities():
    one = np.ones(4, np.float32)
    x = np.array([1.0, 2.0, 3.0, -1.0], np.float32)
    y = np.array([1.0, 3.0, 2.0, -1.0], np.float32)
    dmax = ob.elementwise_backward(T.MAX, one, x, y, None, 0.0)
    dmin = ob.elementwise_backward(T.MIN, one, x, y, None, 0.0)
    assert dmax[0].tolist() == [0.5, 0.0, 1.0, 0.5] and dmax[1].tolist() == [0.5, 1.0, 0.0, 0.5]   # diff.meta.slang:2266-2273
    assert dmin[0].tolist() == [0.5, 1.0, 0.0, 0.5] and dmin[1].tolist() == [0.5, 0.0, 1.0, 0.5]
    lo, hi = np.full(4, 1.0, np.float32), np.full(4, 2.0, np.float32)
    dcl = ob.elementwise_backward(T.CLAMP, one, np.array([0.5, 1.0, 2.0, 2.5], np.float32), lo, hi, 0.0)
    assert dcl[0].tolist() == [0, 1, 1, 0] and dcl[1].tolist() == [1, 0, 0, 0] and dcl[2].tolist() == [0, 0, 0, 1]
    # relu is max(x, 0): half of the gradient at exactly 0 (activations.slang:25-42 through the max rule)
    assert ob.elementwise_backward(T.RELU, one, np.array([-1, 0, 0.0, 2], np.float32), None, None, 0.0)[0].tolist() == [0, 0.5, 0.5, 1]
    # activations against their textbook forms
    v = np.linspace(-6, 6, 25).astype(np.float32)
    sig = 1 / (1 + np.exp(-v.astype(np.float64)))
    assert np.allclose(ob.elementwise(T.SIGMOID, v, None, None, 0.0), sig, rtol=1e-6)
    assert np.allclose(ob.elementwise(T.SILU, v, None, None, 0.0), v * sig, rtol=1e-6, atol=1e-7)
    assert np.allclose(ob.elementwise(T.QUICK_GELU, v, None, None, 0.0), v / (1 + np.exp(-1.702 * v.astype(np.float64))), rtol=1e-6, atol=1e-7)
    assert np.allclose(ob.elementwise(T.LEAKY_RELU, v, None, None, 0.01), np.where(v < 0, 0.01 * v, v), rtol=1e-6)
    assert ob.elementwise(T.STEP, np.array([1, 1, 1], np.float32), np.array([0.5, 1, 2], np.float32), None, 0.0).tolist() == [0, 1, 1]
    # fp16: one rounding of the exact value
    vh = v.astype(np.float16)
    assert np.array_equal(ob.elementwise(T.TANH, vh, None, None, 0.0), np.tanh(vh.astype(np.float64)).astype(np.float16))
