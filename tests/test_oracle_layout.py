"""Invariants of the matrix layouts.  The reference leaves InferencingOptimal/TrainingOptimal to
the vendor driver, so they are pinned by invariants only (round trip, bijection into the declared
size, zero padding, size rules) plus the shape cases the reference's converter tests use
(tools/gfx-unit-test/neural-slang-network-converter.cpp:36-47: 5->13, 13->7, 7->19;
tests/neural/network-parameter-layout-converter-buffer.slang: 17->33 multi-tile, 4->5->3->2->6)."""
import numpy as np
import pytest

import oracle_binding as ob
from oracle_binding import F16, F32, S8, U8, E4M3, ROW, COL, INF_OPT, TRAIN_OPT

L = ob.lib()

SHAPES = [(13, 5), (7, 13), (19, 7), (33, 17), (5, 4), (3, 5), (2, 3), (6, 2), (16, 16), (64, 64),
          (128, 128), (1, 64), (64, 8), (8, 64), (64, 32), (16, 2), (1, 1), (100, 70)]


def portable_value(i):
    # the deterministic fill rule of neural-slang-network-converter.cpp:153-235
    return ((37 * i + 19) % 257 - 128) / 8.0


@pytest.mark.parametrize("rows,cols", SHAPES)
@pytest.mark.parametrize("ct", [F16, S8, E4M3, F32])
def test_optimal_layout_is_a_bijection_into_its_size(rows, cols, ct):
    for layout in (INF_OPT, TRAIN_OPT):
        if layout == TRAIN_OPT and ct not in (F16, F32):
            assert L.cvo_layout_matrix_size(rows, cols, ct, layout, 0) == 0
            continue
        size = L.cvo_layout_matrix_size(rows, cols, ct, layout, 0)
        esz = {F16: 2, S8: 1, E4M3: 1, F32: 4}[ct]
        assert size >= rows * cols * esz and size % 64 == 0
        offs = np.array([[L.cvo_layout_elem_offset(rows, cols, ct, layout, 0, r, c) for c in range(cols)]
                         for r in range(rows)])
        assert offs.min() >= 0 and offs.max() + esz <= size
        assert (offs % esz == 0).all()
        assert len(np.unique(offs)) == rows * cols


@pytest.mark.parametrize("rows,cols", SHAPES)
def test_round_trip_and_zero_padding(rows, cols):
    vals = np.array([portable_value(i) for i in range(rows * cols)], np.float16).reshape(rows, cols)
    for layout in (COL, INF_OPT, TRAIN_OPT):
        size = L.cvo_layout_matrix_size(rows, cols, F16, layout, 0)
        buf = np.full(size, 0xAB, np.uint8)
        assert L.cvo_layout_convert(ob.ptr(buf), rows, cols, F16, layout, 0, ob.ptr(vals), F16, ROW, 0) == 0
        back = np.zeros((rows, cols), np.float16)
        assert L.cvo_layout_convert(ob.ptr(back), rows, cols, F16, ROW, 0, ob.ptr(buf), F16, layout, 0) == 0
        assert (back.view(np.uint16) == vals.view(np.uint16)).all()
        if layout != COL:
            # everything that is not a logical element reads as zero
            used = np.zeros(size, bool)
            for r in range(rows):
                for c in range(cols):
                    o = L.cvo_layout_elem_offset(rows, cols, F16, layout, 0, r, c)
                    used[o:o + 2] = True
            assert not buf[~used].any()


def test_strided_row_and_column_major():
    rows, cols = 5, 7
    W = np.arange(rows * cols, dtype=np.float16).reshape(rows, cols)
    assert L.cvo_layout_matrix_size(rows, cols, F16, ROW, 32) == 4 * 32 + 14
    assert L.cvo_layout_matrix_size(rows, cols, F16, ROW, 8) == 0          # stride < row
    assert L.cvo_layout_elem_offset(rows, cols, F16, ROW, 32, 2, 3) == 2 * 32 + 6
    assert L.cvo_layout_elem_offset(rows, cols, F16, COL, 16, 2, 3) == 3 * 16 + 4
    assert L.cvo_layout_elem_offset(rows, cols, F16, ROW, 0, 5, 0) == -1   # out of range
    buf = np.zeros(L.cvo_layout_matrix_size(rows, cols, F16, COL, 16), np.uint8)
    assert L.cvo_layout_convert(ob.ptr(buf), rows, cols, F16, COL, 16, ob.ptr(W), F16, ROW, 0) == 0
    v = buf.view(np.float16)
    for r in range(rows):
        for c in range(cols):
            assert v[(c * 16 + r * 2) // 2] == W[r, c]


def test_inferencing_optimal_fragment_structure():
    # lane group g owns input columns [g*GS,(g+1)*GS) and output rows [g*4MT,(g+1)*4MT):
    # all elements of one (row block, column block) pair land in one 16-lane group's slots
    rows, cols = 64, 64
    epl, gs, mt4 = 8, 16, 16
    for r in range(rows):
        for c in range(cols):
            off = L.cvo_layout_elem_offset(rows, cols, F16, INF_OPT, 0, r, c) // 2
            s = off % epl; lane = (off // epl) % 64; f = off // (epl * 64)
            kt, t = f % 2, f // 2
            g, i = lane // 16, lane % 16
            assert c == g * gs + kt * epl + s
            assert r == (i // 4) * mt4 + 4 * t + i % 4
    # int8 fragments carry 16 k-slots per lane
    off = L.cvo_layout_elem_offset(128, 128, S8, INF_OPT, 0, 0, 17)
    assert off == ((0 * 2 + 1) * 64 + 0) * 16 + 1


def test_f16_f32_conversion_and_type_rules():
    rows, cols = 9, 20
    W = (np.random.default_rng(0).standard_normal((rows, cols))).astype(np.float32)
    size = L.cvo_layout_matrix_size(rows, cols, F16, TRAIN_OPT, 0)
    buf = np.zeros(size, np.uint8)
    assert L.cvo_layout_convert(ob.ptr(buf), rows, cols, F16, TRAIN_OPT, 0, ob.ptr(W), F32, ROW, 0) == 0
    back = np.zeros((rows, cols), np.float32)
    assert L.cvo_layout_convert(ob.ptr(back), rows, cols, F32, ROW, 0, ob.ptr(buf), F16, TRAIN_OPT, 0) == 0
    assert (back == W.astype(np.float16).astype(np.float32)).all()
    # int8 <-> fp16 is not a layout conversion
    assert L.cvo_layout_convert(ob.ptr(buf), rows, cols, S8, ROW, 0, ob.ptr(W), F32, ROW, 0) != 0
    assert L.cvo_layout_matrix_size(4, 4, ob.S8P, ROW, 0) == 0
    assert L.cvo_layout_matrix_size(0, 4, F16, ROW, 0) == 0
