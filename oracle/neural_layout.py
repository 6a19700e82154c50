"""CPU oracle (numpy) for the neural module's whole-network parameter layouts.

TEST INFRASTRUCTURE ONLY: imported by tests/ alone; the shipped library never uses it.

Restates NetworkParameterLayoutConverter (source/standard-modules/neural/
network-parameter-layout-converter.slang): layer sizes :96-135, the three target orders :137-172 and
their inverses :219-262, per-layer conversion with zero padding and the always-reserved bias slot
:288-440, and the host-side statement of the same rules in
tools/gfx-unit-test/neural-slang-network-converter.cpp:78-235.

Pinned by: the element counts the reference's tests allocate (321/1088 in the host test; 10/272,
36/9248, 594/1584, 66/17408, 62/1088 in tests/neural/network-parameter-layout-converter-buffer.slang);
independent numpy formulations of the Metal (pad) and SPIR-V (tile/transpose) orders; bijection and
hand-evaluated points of the CUDA order; round trips.  The NATIVE order is this library's own
(PARITY UNPINNED against the reference, which has no gfx950 target): pinned by round trip, bijection and
agreement with the TrainingOptimal map of oracle/coopvec_oracle.c.
"""
from __future__ import annotations

import numpy as np

NATIVE, TILED_ROW_MAJOR, PADDED_ROW_MAJOR, CUDA_MATRIX_B = range(4)


def align16(v: int) -> int:
    return (v + 15) // 16 * 16


def row_major_to_cuda_native(row: int, col: int) -> int:
    """rowMajorToCudaNativeLayout, converter :59-72."""
    row_group = 0 if row < 8 else 1
    row_in_group = row - 8 * row_group
    tid_local, pair = row_in_group // 2, row_in_group % 2
    sub = 0 if col < 8 else 1
    gid = col - 8 * sub
    return (gid * 4 + tid_local) * 8 + sub * 4 + row_group * 2 + pair


def physical_weight_offset(order: int, in_size: int, out_size: int, o: int, i: int) -> int:
    pin, pout = align16(in_size), align16(out_size)
    ot, it, oi, ii = o // 16, i // 16, o % 16, i % 16
    if order == CUDA_MATRIX_B:          # :155-160
        return (it * (pout // 16) + ot) * 256 + row_major_to_cuda_native(ii, oi)
    if order == TILED_ROW_MAJOR:        # :161-166
        return (ot * (pin // 16) + it) * 256 + oi * 16 + ii
    if order == PADDED_ROW_MAJOR:       # :167-170
        return o * pin + i
    # NATIVE: accumulator-native 16x16 tiles (lane 16g+j holds rows 4g..4g+3 of column j), tile grid row-major
    return (ot * (pin // 16) + it) * 256 + (16 * (oi // 4) + ii) * 4 + (oi & 3)


def layer_counts(in_size: int, out_size: int, has_bias: bool):
    logical = in_size * out_size + (out_size if has_bias else 0)                       # :109-113
    physical = align16(in_size) * align16(out_size) + align16(out_size)                # :120-123
    return logical, physical


def network_counts(bias_mask: int, dims):
    l = p = 0
    for k in range(len(dims) - 1):
        a, b = layer_counts(dims[k], dims[k + 1], bool((bias_mask >> k) & 1))
        l += a; p += b
    return l, p


def to_optimal(portable: np.ndarray, bias_mask: int, dims, order: int) -> np.ndarray:
    l_total, p_total = network_counts(bias_mask, dims)
    assert portable.size >= l_total
    out = np.zeros(p_total, portable.dtype)
    lo = po = 0
    for k in range(len(dims) - 1):
        n_in, n_out = dims[k], dims[k + 1]
        has_bias = bool((bias_mask >> k) & 1)
        wl, wp = n_in * n_out, align16(n_in) * align16(n_out)
        for o in range(n_out):
            for i in range(n_in):
                out[po + physical_weight_offset(order, n_in, n_out, o, i)] = portable[lo + o * n_in + i]
            if has_bias:
                out[po + wp + o] = portable[lo + wl + o]
        a, b = layer_counts(n_in, n_out, has_bias)
        lo += a; po += b
    return out


def to_portable(optimal: np.ndarray, bias_mask: int, dims, order: int) -> np.ndarray:
    l_total, p_total = network_counts(bias_mask, dims)
    assert optimal.size >= p_total
    out = np.zeros(l_total, optimal.dtype)
    lo = po = 0
    for k in range(len(dims) - 1):
        n_in, n_out = dims[k], dims[k + 1]
        has_bias = bool((bias_mask >> k) & 1)
        wl, wp = n_in * n_out, align16(n_in) * align16(n_out)
        for o in range(n_out):
            for i in range(n_in):
                out[lo + o * n_in + i] = optimal[po + physical_weight_offset(order, n_in, n_out, o, i)]
            if has_bias:
                out[lo + wl + o] = optimal[po + wp + o]
        a, b = layer_counts(n_in, n_out, has_bias)
        lo += a; po += b
    return out


def make_portable_value(index: int) -> float:
    """makePortableValue of the reference's host test (neural-slang-network-converter.cpp:153-157)."""
    return float((index * 37 + 19) % 257 - 128) * 0.125
