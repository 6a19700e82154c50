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


def test_no_alloc_on_the_layer_by_layer_step_and_its_limit():
    # layer sizes without a fused kernel take the layer-by-layer step, whose scratch grows with the batch:
    # a small batch fits the built-in array (same result as cvMlpTrainStep, bit for bit), a large one does not
    rng = np.random.default_rng(1)
    specs = make_specs(rng, [8, 16, 160, 4])
    x = to_dev(rng.uniform(-1, 1, (300, 8)).astype(np.float16))
    ref_layers, layers = build(specs), build(specs)
    _, ref_loss = cv.mlpTrainStep(ref_layers, x, None)
    loss = torch.zeros(1, dtype=torch.float32, device=DEV)
    cv.mlpTrainStepNoAlloc(layers, x, None, loss)
    for r, g in zip(ref_layers, layers):
        assert torch.equal(r.weightsGrad, g.weightsGrad) and torch.equal(r.biasesGrad, g.biasesGrad)
    assert ref_loss.item() == loss.item()
    big = torch.zeros(1 << 17, 8, dtype=torch.float16, device=DEV)
    assert cv.mlpTrainStepWorkspaceSize(layers, big.shape[0]) > cv.NOALLOC_SCRATCH_BYTES
    with pytest.raises(cv.CoopVecError) as e:
        cv.mlpTrainStepNoAlloc(layers, big, None, loss)
    assert e.value.result == cv.SLANG_E_NOT_AVAILABLE


def test_no_alloc_entry_point_under_graph_capture():
    # A hipMalloc / hipFree inside the library would be invisible to torch's allocator statistics, but not to a stream
    # capture, which such a call breaks: after one call outside capture (the scratch array's address is looked up then),
    # the entry point is recorded into a HIP graph and replayed three times, with eager work and synchronisations in
    # between; every replay gives the gradients and the loss of cvMlpTrainStep, bit for bit.
    rng = np.random.default_rng(8)
    dims, B = [8, 64, 64, 64, 64, 1], 5000
    specs = make_specs(rng, dims)
    x = to_dev(rng.uniform(-1, 1, (B, dims[0])).astype(np.float16))
    t = to_dev(rng.uniform(-1, 1, (B, dims[-1])).astype(np.float16))
    ref_layers = build(specs, CT.Float32, ML.TrainingOptimal)
    _, ref_loss = cv.mlpTrainStep(ref_layers, x, t)
    layers = build(specs, CT.Float32, ML.TrainingOptimal)
    loss = torch.zeros(1, dtype=torch.float32, device=DEV)
    cv.mlpTrainStepNoAlloc(layers, x, t, loss)          # outside capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        cv.mlpTrainStepNoAlloc(layers, x, t, loss)
    for replay in range(3):
        for L in layers:                                  # eager work between the replays: the gradients start from zero
            L.weightsGrad.zero_(); L.biasesGrad.zero_()
        loss.fill_(-1.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for r, g in zip(ref_layers, layers):
            assert torch.equal(r.weightsGrad, g.weightsGrad) and torch.equal(r.biasesGrad, g.biasesGrad), replay
        assert ref_loss.item() == loss.item()
