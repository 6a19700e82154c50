"""Helpers shared by the GPU parity tests: seeded inputs, buffers, oracle-side mirrors."""
from __future__ import annotations

import numpy as np
import torch

import oracle_binding as ob
from slang_amd import coopvec as cv
from slang_amd.coopvec import CoopVecComponentType as CT, CoopVecMatrixLayout as ML

DEV = "cuda"

NP_OF_CT = {CT.Float16: np.float16, CT.Float32: np.float32, CT.SignedInt8: np.int8, CT.FloatE4M3: np.uint8,
            CT.SignedInt32: np.int32}


def to_dev(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def as_bytes(t: torch.Tensor) -> torch.Tensor:
    return t.contiguous().view(torch.uint8).flatten()


def matrix_in_layout(W: np.ndarray, ct: int, layout: int, stride: int = 0) -> np.ndarray:
    """Bytes of the logical matrix W (row-major numpy) in `layout`, produced by the oracle."""
    rows, cols = W.shape
    size = ob.lib().cvo_layout_matrix_size(rows, cols, int(ct), int(layout), stride)
    assert size > 0
    buf = np.zeros(size, np.uint8)
    src = np.ascontiguousarray(W)
    rc = ob.lib().cvo_layout_convert(ob.ptr(buf), rows, cols, int(ct), int(layout), stride,
                                     ob.ptr(src), int(ct), ob.ROW, 0)
    assert rc == 0
    return buf


def fp16_inputs(rng, B, K, scale=1.0):
    return (rng.standard_normal((B, K)) * scale).astype(np.float16)


def fp16_weights(rng, M, K):
    return (rng.standard_normal((M, K)) / np.sqrt(K)).astype(np.float16)
