"""The example's Adam update (adam.slang:20-36, kernels.slang:29-45).

The reference ships no golden for the optimizer, so the oracle is pinned by what the mathematics
of Adam fixes over several steps (bounds stated per test; all arithmetic is fp16, so they are a few
fp16 roundings wide), and the GPU kernel is then held to the oracle bit for bit -- except where the
two maths libraries round pow() differently, which the test proves element by element."""
import numpy as np
import pytest

import oracle_binding as ob

LR, B1, B2 = 0.01, 0.9, 0.999


def ulp16(v):
    return float(ob.f16_ulp(np.array([v], np.float32))[0])


def test_constant_gradient_moves_by_lr_every_step():
    # constant g: mean_n = (1-b1^n) g and var_n = (1-b2^n) g^2, so the bias-corrected moments are g
    # and g^2 at every step and the update is lr*g/(|g|+eps) = lr*sign(g).  This needs the state to
    # carry over and the correction to use pow(beta, iteration) with the running count: without
    # carry-over step 2 would move by 0.53*lr, with a constant exponent by 1.34*lr.
    # Bound: 3 % of lr for the half roundings of mean, variance, both corrections, sqrt and the
    # quotient (each 2^-11 relative, variance halved by the root) plus the rounding of p itself.
    # Gradients are chosen so that (1-b2) g^2 is a normal fp16 number: below that the source's own
    # arithmetic loses the variance to subnormal rounding.
    g = np.array([0.5, -1.5, 2.0, -3.0, 0.75, -40.0], np.float16)
    p = np.zeros(6, np.float16)
    st = np.zeros(6, ob.ADAM_STATE_DTYPE)
    for n in range(1, 17):
        before = p.astype(np.float64)
        ob.slang_adam_step(st, p, g.copy())
        assert (st["iteration"] == n).all()
        step = before - p.astype(np.float64)
        for i in range(6):
            assert abs(step[i] - LR * np.sign(float(g[i]))) <= 0.03 * LR + ulp16(p[i]), (n, i, step[i])


def test_impulse_response_separates_the_two_betas():
    # one gradient g, then zeros: mean_n = b1^(n-1)(1-b1) g, var_n = b2^(n-1)(1-b2) g^2, so step n moves by
    #   lr * [b1^(n-1)(1-b1)/(1-b1^n)] / sqrt(b2^(n-1)(1-b2)/(1-b2^n)) * sign(g)
    # (0.670 lr at n = 2; 0.726 lr if the betas were swapped).  Betas as fp16 values, as the source has them.
    b1, b2 = float(np.float16(B1)), float(np.float16(B2))
    g0 = np.array([1.0, -0.5, 8.0], np.float16)
    p = np.zeros(3, np.float16)
    st = np.zeros(3, ob.ADAM_STATE_DTYPE)
    for n in range(1, 9):
        g = g0.copy() if n == 1 else np.zeros(3, np.float16)
        before = p.astype(np.float64)
        ob.slang_adam_step(st, p, g)
        want = LR * (b1 ** (n - 1) * (1 - b1) / (1 - b1 ** n)) / np.sqrt(b2 ** (n - 1) * (1 - b2) / (1 - b2 ** n))
        step = before - p.astype(np.float64)
        for i in range(3):
            assert abs(step[i] - want * np.sign(float(g0[i]))) <= 0.03 * LR + ulp16(p[i]), (n, i, step[i], want)
        assert (g == 0).all() and (st["iteration"] == n).all()


def test_nan_skips_and_infinities_clip():
    # kernels.slang:39-43: a NaN gradient is cleared and the parameter's state is left alone (no
    # iteration, no decay); adam.slang:23-29: +-inf count as +-10000
    g = np.array([np.nan, np.inf, -np.inf, 1.0], np.float16)
    p = np.ones(4, np.float16); st = np.zeros(4, ob.ADAM_STATE_DTYPE)
    ob.slang_adam_step(st, p, g)
    assert (g == 0).all() and st["iteration"].tolist() == [0, 1, 1, 1]
    # in half, (1-b2)*10000*10000 overflows: variance = inf and the step itself is 0 -- faithful to
    # the source's arithmetic; the state still advances
    assert p[0] == 1.0 and p[1] == 1.0 and p[2] == 1.0 and p[3] < 1.0
    assert np.isinf(st["variance"][1:3].view(np.float16)).all() and st["mean"][3] != 0
    # a NaN in the middle of a run: the other steps behave as if it had not been there
    pa = np.zeros(1, np.float16); sa = np.zeros(1, ob.ADAM_STATE_DTYPE)
    pb = np.zeros(1, np.float16); sb = np.zeros(1, ob.ADAM_STATE_DTYPE)
    for n in range(6):
        ob.slang_adam_step(sa, pa, np.array([0.5], np.float16))
        if n == 2:
            ob.slang_adam_step(sb, pb, np.array([np.nan], np.float16))
        ob.slang_adam_step(sb, pb, np.array([0.5], np.float16))
    assert pa[0] == pb[0] and sa.tobytes() == sb.tobytes()


@pytest.mark.gpu
@pytest.mark.parametrize("n", [5000, 5003])      # four parameters per thread, and the kernel for any count
def test_gpu_adam_matches_oracle(n):
    import torch
    from slang_amd import coopvec as cv
    rng = np.random.default_rng(7)
    p = rng.uniform(-1, 1, n).astype(np.float16)
    st = np.zeros(n, ob.ADAM_STATE_DTYPE)
    pd = torch.from_numpy(p.copy()).cuda()
    sd = torch.zeros(n * 8, dtype=torch.uint8, device="cuda")
    pow_cases = 0
    for it in range(12):
        g = (rng.standard_normal(n) * 10.0 ** rng.integers(-4, 3, n)).astype(np.float16)
        g[::97] = np.nan; g[5::101] = np.inf; g[7::103] = -np.inf
        gd = torch.from_numpy(g.copy()).cuda()
        cv.adjustParameters(sd, pd, gd)
        # the oracle with pow() as the host library rounds it, and with its fp32 value one or two ulps
        # to either side for each beta: the only operation the two libraries may round differently
        variants = {}
        for n1 in range(-2, 3):
            for n2 in range(-2, 3):
                pv, sv, gv = p.copy(), st.copy(), g.copy()
                ob.slang_adam_step(sv, pv, gv, pow_nudge=(n1, n2))
                variants[(n1, n2)] = (pv, sv)
        assert (gd.cpu().numpy() == 0).all()
        got = pd.cpu().numpy()
        stg = sd.cpu().numpy().view(ob.ADAM_STATE_DTYPE)
        ref_p, ref_s = variants[(0, 0)]
        # state: no pow() involved, bit-equal always
        assert stg.tobytes() == ref_s.tobytes()
        differs = got.view(np.uint16) != ref_p.view(np.uint16)
        if differs.any():
            explained = np.zeros(n, bool)
            for pv, _ in variants.values():
                explained |= got.view(np.uint16) == pv.view(np.uint16)
            assert explained[differs].all(), "parameters differ from the oracle beyond the rounding of pow()"
            pow_cases += int(differs.sum())
        # continue from the GPU's state so that differences do not accumulate in the comparison
        p = got.copy(); st = stg.copy()
    assert pow_cases <= n // 100


@pytest.mark.gpu
def test_gpu_adam_with_step_counts_that_differ_between_parameters():
    # the kernel evaluates pow(beta, t) once per workgroup for the count its first state holds; a parameter with another
    # count must get its own powers: states with random counts, one step, against the oracle
    import torch
    from slang_amd import coopvec as cv
    rng = np.random.default_rng(11)
    n = 3000
    p = rng.uniform(-1, 1, n).astype(np.float16)
    st = np.zeros(n, ob.ADAM_STATE_DTYPE)
    st["iteration"] = rng.integers(0, 60, n)
    st["iteration"][:1200] = 17                      # a whole workgroup with one count, then mixed ones
    st["mean"] = rng.uniform(-0.1, 0.1, n).astype(np.float16)
    st["variance"] = rng.uniform(0, 0.01, n).astype(np.float16)
    g = (rng.standard_normal(n) * 0.1).astype(np.float16)
    pd = torch.from_numpy(p.copy()).cuda()
    sd = torch.from_numpy(st.copy().view(np.uint8)).cuda()
    gd = torch.from_numpy(g.copy()).cuda()
    cv.adjustParameters(sd, pd, gd)
    got, stg = pd.cpu().numpy(), sd.cpu().numpy().view(ob.ADAM_STATE_DTYPE)
    variants = []
    for n1 in range(-2, 3):
        for n2 in range(-2, 3):
            pv, sv, gv = p.copy(), st.copy(), g.copy()
            ob.slang_adam_step(sv, pv, gv, pow_nudge=(n1, n2))
            variants.append((pv, sv, (n1, n2)))
    ref_p, ref_s = [(pv, sv) for pv, sv, k in variants if k == (0, 0)][0]
    assert stg.tobytes() == ref_s.tobytes()
    differs = got.view(np.uint16) != ref_p.view(np.uint16)
    explained = np.zeros(n, bool)
    for pv, _, _ in variants:
        explained |= got.view(np.uint16) == pv.view(np.uint16)
    assert explained[differs].all() and differs.sum() <= n // 100


@pytest.mark.gpu
@pytest.mark.parametrize("grad_type", ["f16", "f32"])
def test_network_adam_step_equals_convert_plus_adam(grad_type):
    # cvMlpAdamStep reads every layer's gradient where the training step left it (TrainingOptimal here) and updates
    # weights and biases in one launch: same bits as the example's convert (TrainingOptimal -> RowMajor) followed by
    # adjustParameters over the row-major gradients, over several steps (the states carry over), NaN / inf
    # gradients included; and it leaves the gradient buffers at zero
    import torch
    from slang_amd import coopvec as cv
    from slang_amd.coopvec import Activation, CoopVecComponentType as CT, CoopVecMatrixLayout as ML, FeedForwardLayer
    from slang_amd.coopvec import CooperativeVectorMatrixDesc as D
    rng = np.random.default_rng(17)
    dims = [4, 16, 20, 3]
    gct, gdt, gnp = (CT.Float16, torch.float16, np.float16) if grad_type == "f16" else (CT.Float32, torch.float32, np.float32)
    dev = "cuda"
    W = [torch.from_numpy(rng.uniform(-1, 1, (dims[i + 1], dims[i])).astype(np.float16)).to(dev) for i in range(3)]
    Bv = [torch.from_numpy(rng.uniform(-1, 1, dims[i + 1]).astype(np.float16)).to(dev) for i in range(3)]
    Bv[1] = None                                   # a layer without biases
    Wref = [w.clone() for w in W]; Bref = [b.clone() if b is not None else None for b in Bv]
    wst = [torch.zeros(w.numel() * 8, dtype=torch.uint8, device=dev) for w in W]
    bst = [torch.zeros(b.numel() * 8, dtype=torch.uint8, device=dev) if b is not None else None for b in Bv]
    wst_ref = [t.clone() for t in wst]; bst_ref = [t.clone() if t is not None else None for t in bst]
    sizes = [cv.getCooperativeVectorMatrixSize(dims[i + 1], dims[i], gct, ML.TrainingOptimal) for i in range(3)]
    for step in range(4):
        layers, gref = [], []
        for i in range(3):
            fo, fi = dims[i + 1], dims[i]
            g = (rng.standard_normal((fo, fi)) * 10.0 ** rng.integers(-3, 2, (fo, fi))).astype(gnp)
            g[0, 0] = np.nan; g[1 % fo, 1] = np.inf
            grow = torch.from_numpy(g).to(dev)
            gopt = torch.zeros(sizes[i], dtype=torch.uint8, device=dev)
            esz = grow.element_size()
            cv.convertCooperativeVectorMatrix(gopt, [D(fo, fi, gct, ML.TrainingOptimal, sizes[i], 0, 0)],
                                              grow.contiguous().view(torch.uint8).flatten(), [D(fo, fi, gct, ML.RowMajor, fo * fi * esz, 0, fi * esz)])
            bg = torch.from_numpy((rng.standard_normal(fo) * 0.1).astype(gnp)).to(dev) if Bv[i] is not None else None
            layers.append(FeedForwardLayer(fi, fo, W[i].view(torch.uint8).flatten(), Bv[i].view(torch.uint8) if Bv[i] is not None else None,
                                           ML.RowMajor, fi * 2, Activation.ReLU, 0.0, gopt,
                                           bg.view(torch.uint8) if bg is not None else None, ML.TrainingOptimal, 0))
            gref.append((grow.to(torch.float16).clone(), bg.to(torch.float16).clone() if bg is not None else None))
        cv.mlpAdjustParameters(layers, wst, bst, gradType=gct)
        assert cv.lastKernelName().startswith("adamLayersKernel")
        for i in range(3):
            cv.adjustParameters(wst_ref[i], Wref[i].view(-1), gref[i][0].contiguous().view(-1))
            if Bref[i] is not None:
                cv.adjustParameters(bst_ref[i], Bref[i], gref[i][1])
            assert torch.equal(W[i].view(torch.int16), Wref[i].view(torch.int16)), (step, i)
            assert torch.equal(wst[i], wst_ref[i]), (step, i)
            if Bv[i] is not None:
                assert torch.equal(Bv[i].view(torch.int16), Bref[i].view(torch.int16)) and torch.equal(bst[i], bst_ref[i])
                assert (layers[i].biasesGrad == 0).all()
            assert (layers[i].weightsGrad == 0).all()
    with pytest.raises(cv.CoopVecError):
        cv.mlpAdjustParameters(layers, wst[:2] + [None], bst, gradType=gct)
