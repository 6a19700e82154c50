"""GPU layout converter against the oracle's byte images, through the C-ABI."""
import numpy as np
import pytest
import torch

import oracle_binding as ob
from gpu_util import DEV, matrix_in_layout, to_dev
from slang_amd import coopvec as cv
from slang_amd.coopvec import CoopVecComponentType as CT, CoopVecMatrixLayout as ML, CooperativeVectorMatrixDesc as Desc

pytestmark = pytest.mark.gpu

SHAPES = [(13, 5), (7, 13), (19, 7), (33, 17), (5, 4), (16, 16), (64, 64), (128, 128), (1, 64), (64, 8), (100, 70)]
NP = {CT.Float16: np.float16, CT.SignedInt8: np.int8, CT.FloatE4M3: np.uint8, CT.Float32: np.float32}


def portable_value(i):
    return ((37 * i + 19) % 257 - 128) / 8.0     # neural-slang-network-converter.cpp:153-235


@pytest.mark.parametrize("rows,cols", SHAPES)
@pytest.mark.parametrize("ct", [CT.Float16, CT.SignedInt8, CT.FloatE4M3, CT.Float32])
def test_convert_matches_oracle_and_round_trips(rows, cols, ct):
    vals = np.array([portable_value(i) for i in range(rows * cols)]).reshape(rows, cols)
    W = (vals * 8).astype(np.int8).view(NP[ct]) if NP[ct] in (np.int8, np.uint8) else vals.astype(NP[ct])
    esz = W.dtype.itemsize
    src = to_dev(W).view(torch.uint8).flatten()
    layouts = [ML.ColumnMajor, ML.InferencingOptimal] + ([ML.TrainingOptimal] if ct in (CT.Float16, CT.Float32) else [])
    for layout in layouts:
        size = cv.getCooperativeVectorMatrixSize(rows, cols, ct, layout)
        dst = torch.full((size + 64,), 0xCD, dtype=torch.uint8, device=DEV)
        cv.convertCooperativeVectorMatrix(dst, [Desc(rows, cols, ct, layout, size, 0, 0)],
                                          src, [Desc(rows, cols, ct, ML.RowMajor, rows * cols * esz, 0, cols * esz)])
        want = matrix_in_layout(W, ct, layout)
        got = dst.cpu().numpy()
        assert (got[:size] == want).all()
        assert (got[size:] == 0xCD).all()                       # nothing written past the matrix
        back = torch.zeros(rows * cols * esz, dtype=torch.uint8, device=DEV)
        cv.convertCooperativeVectorMatrix(back, [Desc(rows, cols, ct, ML.RowMajor, rows * cols * esz, 0, 0)],
                                          dst, [Desc(rows, cols, ct, layout, size, 0, 0)])
        assert (back.cpu().numpy() == W.view(np.uint8).ravel()).all()


def test_convert_batched_like_the_example():
    # one call converts every layer's TrainingOptimal gradient to RowMajor inside the same buffer
    # (mlp-training-coopvec.cpp:203-236), sub-allocations rounded to 64 bytes (:273-279)
    sizes = [4, 16, 4]
    rng = np.random.default_rng(3)
    off = 0
    def alloc(n):
        nonlocal off
        o = off; off += (n + 63) // 64 * 64; return o
    row_offs, train_offs, train_sizes, mats = [], [], [], []
    for i in range(2):
        row_offs.append(alloc(sizes[i] * sizes[i + 1] * 2))
    for i in range(2):
        sz = cv.getCooperativeVectorMatrixSize(sizes[i + 1], sizes[i], CT.Float16, ML.TrainingOptimal)
        train_sizes.append(sz); train_offs.append(alloc(sz))
    host = np.zeros(off, np.uint8)
    for i in range(2):
        Wg = rng.standard_normal((sizes[i + 1], sizes[i])).astype(np.float16); mats.append(Wg)
        host[train_offs[i]:train_offs[i] + train_sizes[i]] = matrix_in_layout(Wg, CT.Float16, ML.TrainingOptimal)
    buf = to_dev(host)
    srcs = [Desc(sizes[i + 1], sizes[i], CT.Float16, ML.TrainingOptimal, train_sizes[i], train_offs[i]) for i in range(2)]
    dsts = [Desc(sizes[i + 1], sizes[i], CT.Float16, ML.RowMajor, sizes[i] * sizes[i + 1] * 2, row_offs[i], sizes[i] * 2)
            for i in range(2)]
    cv.convertCooperativeVectorMatrix(buf, dsts, buf, srcs, 2)
    out = buf.cpu().numpy()
    for i in range(2):
        got = out[row_offs[i]:row_offs[i] + mats[i].size * 2].view(np.float16).reshape(mats[i].shape)
        assert (got == mats[i]).all()
    with pytest.raises(cv.CoopVecError) as e:
        cv.convertCooperativeVectorMatrix(buf, [Desc(4, 4, CT.Float16, ML.RowMajor, 32, off - 16, 8)],
                                          buf, [Desc(4, 4, CT.Float16, ML.RowMajor, 32, 0, 8)])
    assert e.value.result == cv.SLANG_E_BUFFER_TOO_SMALL


def test_convert_fp32_to_fp16_and_strided_destination():
    rows, cols = 9, 20
    W = np.random.default_rng(0).standard_normal((rows, cols)).astype(np.float32)
    src = to_dev(W).view(torch.uint8).flatten()
    stride = cols * 2 + 24
    size = cv.getCooperativeVectorMatrixSize(rows, cols, CT.Float16, ML.RowMajor, stride)
    dst = torch.full((size,), 0x77, dtype=torch.uint8, device=DEV)
    cv.convertCooperativeVectorMatrix(dst, [Desc(rows, cols, CT.Float16, ML.RowMajor, size, 0, stride)],
                                      src, [Desc(rows, cols, CT.Float32, ML.RowMajor, rows * cols * 4, 0, 0)])
    got = dst.cpu().numpy()
    for r in range(rows):
        row = got[r * stride:r * stride + cols * 2].view(np.float16)
        assert (row == W[r].astype(np.float16)).all()
        if r + 1 < rows:
            assert (got[r * stride + cols * 2:(r + 1) * stride] == 0x77).all()   # stride padding untouched
