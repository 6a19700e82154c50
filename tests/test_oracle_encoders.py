"""The oracle's grid hashes and permutohedral encoder against the data the reference's own tests hold
(tests/golden/neural_goldens.json, copied from tests/neural/hash-function-test.slang,
permuto-reference-data.slang and permuto-encoder-precomputed-constants.slang)."""
import json
import os

import numpy as np

import oracle_binding as ob

G = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "neural_goldens.json")))
P = G["permuto"]
CFG = P["config"]


def reference_setup():
    """The configuration of tests/neural/permuto-encoder-test.slang: 16x16 cell centres in [0,1]^2,
    feature table value[i] = i."""
    gs = CFG["gridSize"]
    idx = np.arange(gs * gs)
    pos = np.stack([((idx % gs) + 0.5) / gs, ((idx // gs) + 0.5) / gs], axis=1).astype(np.float32)
    n_table = (1 << CFG["log2HashmapSize"]) * CFG["levels"] * CFG["featureDimPerEntry"]
    table = np.arange(n_table, dtype=np.float32)
    levels = ob.permuto_levels(CFG["dimensions"], CFG["log2HashmapSize"], CFG["levels"], CFG["baseScale"],
                               CFG["log2PerLevelScale"], CFG["seed"])
    max_level = np.float32(CFG["maxLevelRatio"]) * np.float32(CFG["levels"])
    return pos, table, levels, float(max_level)


def test_hash_goldens():
    pos = G["hash"]["positions"]
    want = G["hash"]["expected"]
    got = []
    for t in (ob.HASH_PRIME, ob.HASH_COHERENT_PRIME, ob.HASH_REVERSED_PRIME, ob.HASH_BASE_CONVERT, ob.HASH_RNG):
        for d in "1234":
            got.append(ob.grid_hash(t, pos[d]))
    got.append(ob.grid_hash(ob.HASH_PRIME, pos["3"]))
    got.append(ob.grid_hash(ob.HASH_BASE_CONVERT, pos["3"]))
    assert got == want


def test_level_constants():
    _, _, levels, max_level = reference_setup()
    assert abs(max_level - 4.4) < 1e-6
    for l in range(CFG["levels"]):
        lv = levels[l]
        assert lv.currentLevelIndex == l and lv.offsetOfFeatureTable == P["offsets"][l] and lv.featureTableSize == P["tableSizes"][l]
        assert abs(lv.scale - P["scales"][l]) <= 2e-6 * P["scales"][l]
        for d in range(2):
            assert abs(lv.scalesPerDim[d] - P["scalesPerDim"][2 * l + d]) <= 2e-6 * P["scalesPerDim"][2 * l + d]
            assert abs(lv.shiftsPerDim[d] - P["shiftsPerDim"][2 * l + d]) <= 2e-6     # printed with six decimals


def test_forward_reference_values():
    pos, table, levels, max_level = reference_setup()
    out = ob.permuto_encode(levels, CFG["featureDimPerEntry"], max_level, pos, table)
    want = np.array(P["expectedForward"]).reshape(16, 8)
    got = out[P["verifyPositions"]]
    assert np.abs(got - want).max() <= CFG["epsilon"], np.abs(got - want).max()
    # barycentric weights sum to one: with table value[i] = i the two features of an entry differ by exactly 1
    assert np.allclose(out[:, 1::2] - out[:, 0::2], 1.0, atol=2e-3)


def test_backward_reference_values():
    pos, table, levels, max_level = reference_setup()
    d_out = np.ones((pos.shape[0], 8), np.float32)
    d_pos, d_table = ob.permuto_encode_backward(levels, CFG["featureDimPerEntry"], max_level, pos, table, d_out)
    want_pos = np.array(P["expectedDLdPos"]).reshape(16, 2)
    # the reference data are fp32 results of magnitude 1e4: its epsilon 0.1 plus one part in 1e5
    assert (np.abs(d_pos[P["verifyPositions"]] - want_pos) <= CFG["epsilon"] + 1e-5 * np.abs(want_pos)).all()
    want_par = np.array(P["expectedDLdParams"])
    assert np.abs(d_table[P["verifyParamIndices"]] - want_par).max() <= CFG["epsilon"]
    # every sample spreads a total weight of 1 per level and feature over the table
    assert abs(d_table.sum() - pos.shape[0] * 8) < 1e-6 * pos.shape[0] * 8


def test_levels_beyond_max_level_are_zero_and_fp16_follows_fp32():
    pos, table, levels, _ = reference_setup()
    out = ob.permuto_encode(levels, 2, 1.5, pos, table)           # levels 2 and 3 are >= maxLevel + 1e-3
    assert (out[:, 4:] == 0).all() and (out[:, :4] != 0).any()
    small = (table / 64).astype(np.float16)
    o16 = ob.permuto_encode(levels, 2, 4.4, pos.astype(np.float16), small)
    o32 = ob.permuto_encode(levels, 2, 4.4, pos.astype(np.float16).astype(np.float32), small.astype(np.float32))
    assert np.abs(o16.astype(np.float32) - o32).max() <= 0.02 * np.abs(o32).max()


def test_library_level_preparation_matches_reference_constants_without_gpu():
    # cvPermutoPrepareLevels runs on the host: checked here against the reference's precomputed constants
    import ctypes
    from slang_amd import _lib
    d = _lib.CvPermutoDesc()
    d.dimensions, d.featureDimensionPerEntry, d.log2HashmapSize, d.maxLevels, d.elementType = 2, 2, 8, 4, 3
    assert _lib.load().cvPermutoPrepareLevels(ctypes.byref(d), CFG["baseScale"], CFG["log2PerLevelScale"], CFG["maxLevelRatio"], CFG["seed"]) == 0
    assert abs(d.maxLevel - 4.4) < 1e-6
    levels = ob.permuto_levels(2, 8, 4, CFG["baseScale"], CFG["log2PerLevelScale"], CFG["seed"])
    for l in range(4):
        lv = d.levelInfo[l]
        assert (lv.currentLevelIndex, lv.offsetOfFeatureTable, lv.featureTableSize) == (l, P["offsets"][l], P["tableSizes"][l])
        assert abs(lv.scale - P["scales"][l]) <= 2e-6 * P["scales"][l]
        for k in range(2):
            assert abs(lv.scalesPerDim[k] - P["scalesPerDim"][2 * l + k]) <= 2e-6 * P["scalesPerDim"][2 * l + k]
            assert abs(lv.shiftsPerDim[k] - P["shiftsPerDim"][2 * l + k]) <= 2e-6
            assert lv.shiftsPerDim[k] == levels[l].shiftsPerDim[k]           # same PCG32 stream as the oracle
