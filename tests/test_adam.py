"""The example's Adam update (adam.slang:20-36, kernels.slang:29-45): oracle against the closed
form of the first steps, GPU kernel against the oracle.  The reference ships no golden for the
optimizer, so the oracle is pinned by mathematics only (parity unpinned against the reference)."""
import numpy as np
import pytest

import oracle_binding as ob


def h(x):
    return np.float32(np.float16(np.float32(x)))


def test_oracle_first_step_closed_form():
    # first step from zero state: mean = (1-b1) g, var = (1-b2) g^2, bias-corrected ratio ~ sign(g):
    # every parameter moves by about lr against the gradient's sign
    g = np.array([0.5, -0.25, 2.0, -3.0, 1e-2], np.float16)
    p = np.array([1.0, 1.0, -1.0, 0.0, 0.5], np.float16)
    st = np.zeros(5, ob.ADAM_STATE_DTYPE)
    p0 = p.copy()
    ob.slang_adam_step(st, p, g.copy())
    assert (st["iteration"] == 1).all()
    # step by step in half, as the source spells it
    b1, b2, eps, lr = h(0.9), h(0.999), h(1e-7), h(0.01)
    for i in range(5):
        gi = np.float32(g[i])
        mean = h(h(b1 * 0) + h(h(1 - b1) * gi))
        var = h(h(b2 * 0) + h(h(h(1 - b2) * gi) * gi))
        mhat = h(mean / h(1 - h(np.float32(b1) ** 1)))
        vhat = h(var / h(1 - h(np.float32(b2) ** 1)))
        want = np.float16(np.float32(p0[i]) - h(h(lr * mhat) / h(np.sqrt(h(max(np.float32(0), vhat) + eps)))))
        assert p[i] == want
        assert abs(float(p0[i]) - float(p[i]) - 0.01 * np.sign(gi)) < 2e-3
    # NaN gradients are cleared and skipped, infinities clipped to +-10000, gradients zeroed
    g = np.array([np.nan, np.inf, -np.inf, 1.0], np.float16)
    p = np.ones(4, np.float16); st = np.zeros(4, ob.ADAM_STATE_DTYPE)
    ob.slang_adam_step(st, p, g)
    assert (g == 0).all() and st["iteration"].tolist() == [0, 1, 1, 1]
    # in half, (1-b2)*10000*10000 overflows: variance = inf, so the step itself is 0 -- faithful to
    # the source's arithmetic; the state still advances
    assert p[0] == 1.0 and p[1] == 1.0 and p[2] == 1.0
    assert np.isinf(st["variance"][1:3].view(np.float16)).all() and st["mean"][3] != 0


@pytest.mark.gpu
def test_gpu_adam_matches_oracle():
    import torch
    from slang_amd import coopvec as cv
    rng = np.random.default_rng(7)
    n = 5000
    p = rng.uniform(-1, 1, n).astype(np.float16)
    st = np.zeros(n, ob.ADAM_STATE_DTYPE)
    pd = torch.from_numpy(p.copy()).cuda()
    sd = torch.zeros(n * 8, dtype=torch.uint8, device="cuda")
    mism = 0
    for it in range(12):
        g = (rng.standard_normal(n) * 10.0 ** rng.integers(-4, 3, n)).astype(np.float16)
        g[::97] = np.nan; g[5::101] = np.inf; g[7::103] = -np.inf
        gd = torch.from_numpy(g.copy()).cuda()
        cv.adjustParameters(sd, pd, gd)
        ob.slang_adam_step(st, p, g)
        assert (gd.cpu().numpy() == 0).all()
        got = pd.cpu().numpy()
        # identical arithmetic; only powf may differ by an fp32 ulp between the two maths libraries
        mism = max(mism, int((got.view(np.uint16) != p.view(np.uint16)).sum()))
        assert np.max(np.abs(got.astype(np.float32) - p.astype(np.float32))) <= 2e-3
        stg = sd.cpu().numpy().view(ob.ADAM_STATE_DTYPE)
        assert (stg["iteration"] == st["iteration"]).all()
        # continue from the GPU's state so that differences do not accumulate in the comparison
        p = got.copy(); st = stg.copy()
    assert mism <= n // 100
