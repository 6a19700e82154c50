"""cvMlpTrainStepNoAlloc (the entry point that allocates nothing) against cvMlpTrainStep, through the
C-ABI: bit-identical gradients and loss on two calls in a row, the second with a smaller batch (the
library's scratch array keeps the first call's partials), and the size limit's error."""
import numpy as np
import pytest
import torch

from gpu_util import DEV, to_dev
from slang_amd import coopvec as cv
from slang_amd.coopvec import CoopVecComponentType as CT, CoopVecMatrixLayout as ML
from test_gpu_train import build, make_specs

pytestmark = pytest.mark.gpu


def _grads(layers):
    return [(L.weightsGrad.clone(), L.biasesGrad.clone()) for L in layers]


@pytest.mark.parametrize("dims", [[8, 64, 64, 64, 64, 1], [4, 16, 4]])
def test_no_alloc_matches_workspace_entry_point(dims):
    rng = np.random.default_rng(77)
    specs = make_specs(rng, dims)
    for B in (8192 + 5, 1000):          # second call: smaller input, same scratch array
        x = to_dev(rng.uniform(-1, 1, (B, dims[0])).astype(np.float16))
        t = to_dev(rng.uniform(-1, 1, (B, dims[-1])).astype(np.float16))
        ref_layers = build(specs, CT.Float32, ML.TrainingOptimal)
        _, ref_loss = cv.mlpTrainStep(ref_layers, x, t)
        got_layers = build(specs, CT.Float32, ML.TrainingOptimal)
        got_loss = torch.zeros(1, dtype=torch.float32, device=DEV)
        before = torch.cuda.memory_stats()["allocation.all.allocated"]
        cv.mlpTrainStepNoAlloc(got_layers, x, t, got_loss)
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == before   # torch's allocator untouched
        torch.cuda.synchronize()
        for (rw, rb), (gw, gb) in zip(_grads(ref_layers), _grads(got_layers)):
            assert torch.equal(rw, gw) and torch.equal(rb, gb)
        assert ref_loss.item() == got_loss.item()


def test_no_alloc_validates_like_the_workspace_entry_point():
    rng = np.random.default_rng(1)
    layers = build(make_specs(rng, [8, 16, 64, 4]))      # no fused specialisation: same error as cvMlpTrainStep
    x = torch.zeros(10, 8, dtype=torch.float16, device=DEV)
    loss = torch.zeros(1, dtype=torch.float32, device=DEV)
    with pytest.raises(cv.CoopVecError) as e:
        cv.mlpTrainStepNoAlloc(layers, x, None, loss)
    assert e.value.result == cv.SLANG_E_NOT_AVAILABLE
