"""Host-side mirror of Slang's cooperative-vector operator surface, served by the gfx950 library.

Names, argument order and argument meaning follow the Slang declarations
(source/slang/hlsl.meta.slang:32954 coopVecMatMul, :32786 coopVecMatMulPacked,
:33160 coopVecMatMulAdd, :32983 coopVecMatMulAddPacked, :33227 coopVecOuterProductAccumulate,
:33330 coopVecReduceSumAccumulate) and the two slang-rhi calls the example makes
(examples/mlp-training-coopvec/mlp-training-coopvec.cpp:305 getCooperativeVectorMatrixSize,
:227 convertCooperativeVectorMatrix).

Where Slang has one CoopVec<T,N> per shader thread, these functions take a batch: a 2-D torch
tensor [batch, N] on the GPU, one row per thread.  Buffers (ByteAddressBuffer in Slang) are 1-D
torch tensors used as raw bytes.  torch only supplies device memory and the stream; all
arithmetic happens in the HIP library, and every function raises if that library is missing.
"""
from __future__ import annotations

import ctypes
import enum
from dataclasses import dataclass
from typing import Optional, Sequence

import torch

from . import _lib


class CoopVecMatrixLayout(enum.IntEnum):
    """hlsl.meta.slang:32547-32553"""
    RowMajor = 0
    ColumnMajor = 1
    InferencingOptimal = 2
    TrainingOptimal = 3


class CoopVecComponentType(enum.IntEnum):
    """hlsl.meta.slang:32558-32575; BFloat16 is this library's extension (the reference knows
    bfloat16 as a scalar type only, SLANG_SCALAR_TYPE_BFLOAT16, include/slang.h:2155)."""
    FloatE4M3 = 0
    FloatE5M2 = 1
    Float16 = 2
    Float32 = 3
    Float64 = 4
    SignedInt8 = 5
    SignedInt16 = 6
    SignedInt32 = 7
    SignedInt64 = 8
    SignedInt8Packed = 9
    UnsignedInt8 = 10
    UnsignedInt16 = 11
    UnsignedInt32 = 12
    UnsignedInt64 = 13
    UnsignedInt8Packed = 14
    BFloat16 = 15


class RhiCooperativeVectorComponentType(enum.IntEnum):
    """rhi::CooperativeVectorComponentType (include/slang-gfx.h:1748-1765): the numbering the example's
    host code holds (mlp-training-coopvec.cpp:212,220,308).  Convert with componentTypeFromRhi before
    calling into this module, whose functions all take CoopVecComponentType."""
    Float16 = 0
    Float32 = 1
    Float64 = 2
    SInt8 = 3
    SInt16 = 4
    SInt32 = 5
    SInt64 = 6
    UInt8 = 7
    UInt16 = 8
    UInt32 = 9
    UInt64 = 10
    SInt8Packed = 11
    UInt8Packed = 12
    FloatE4M3 = 13
    FloatE5M2 = 14


def componentTypeFromRhi(rhiComponentType: int) -> CoopVecComponentType:
    v = _lib.load().cvComponentTypeFromRhi(int(rhiComponentType))
    if v < 0:
        raise CoopVecError(SLANG_E_INVALID_ARG, "not an rhi::CooperativeVectorComponentType: %d" % int(rhiComponentType))
    return CoopVecComponentType(v)


def componentTypeToRhi(componentType: int) -> RhiCooperativeVectorComponentType:
    v = _lib.load().cvComponentTypeToRhi(int(componentType))
    if v < 0:
        raise CoopVecError(SLANG_E_INVALID_ARG, "not a CoopVecComponentType: %d" % int(componentType))
    return RhiCooperativeVectorComponentType(v)


FLAG_FP8_MATRIX_PIPELINE = 1   # CV_FLAG_FP8_MATRIX_PIPELINE of include/coopvec.h
FLAG_LAYERWISE_TRAINING = 2    # CV_FLAG_LAYERWISE_TRAINING
FLAG_FORWARD_TILE16 = 4         # CV_FLAG_FORWARD_TILE16: keep cvMlpForward to the kernels on 16-sample tiles
FLAG_TRAIN_SPLIT_BY_ROLE = 8    # CV_FLAG_TRAIN_SPLIT_BY_ROLE: cvMlpTrainStep on the kernel whose waves share a tile by kind of work


class Activation(enum.IntEnum):
    """CvActivation: NoActivation..LeakyReLU as the example spells them (fflayer.slang:60-66), the rest
    the neural module's (source/standard-modules/neural/activations.slang)."""
    NoActivation = 0
    ReLU = 1
    LeakyReLU = 2
    Sigmoid = 3
    Tanh = 4
    Exp = 5
    Sine = 6
    SiLU = 7
    QuickGELU = 8


class ElementwiseOp(enum.IntEnum):
    """CvElementwiseOp: the per-component operators and functions of CoopVec<T,N>
    (hlsl.meta.slang:32043-32421, slang-ir-lower-coopvec.cpp:113-166) and the neural activations."""
    Add = 0
    Sub = 1
    Mul = 2
    Div = 3
    Neg = 4
    Min = 5
    Max = 6
    Clamp = 7
    Step = 8
    Sin = 9
    Cos = 10
    Exp = 11
    Log = 12
    Log2 = 13
    Exp2 = 14
    Tanh = 15
    Atan = 16
    Fma = 17
    ReLU = 18
    LeakyReLU = 19
    Sigmoid = 20
    SiLU = 21
    QuickGELU = 22
    Scale = 23      # vector * scalar (hlsl.meta.slang:32004): a * T(param)


# SlangResult values (include/slang.h:1400-1464)
SLANG_OK = 0
SLANG_FAIL = -2147467259            # 0x80004005
SLANG_E_NOT_IMPLEMENTED = -2147467263   # 0x80004001
SLANG_E_INVALID_ARG = -2147024809   # 0x80070057
SLANG_E_BUFFER_TOO_SMALL = -2113929215  # 0x82000001
SLANG_E_INTERNAL_FAIL = -2113929210     # 0x82000006
SLANG_E_NOT_AVAILABLE = -2113929209     # 0x82000007


class CoopVecError(RuntimeError):
    """A failed library call; `.result` is the SlangResult-compatible code."""

    def __init__(self, result: int, message: str):
        super().__init__("%s (SlangResult 0x%08x)" % (message, result & 0xFFFFFFFF))
        self.result = result


def _check(rc: int) -> None:
    if rc < 0:
        raise CoopVecError(rc, _lib.load().cvGetLastErrorMessage().decode("utf-8", "replace"))


def _stream_handle(stream) -> ctypes.c_void_p:
    if stream is None:
        stream = torch.cuda.current_stream()
    if isinstance(stream, torch.cuda.Stream):
        return ctypes.c_void_p(stream.cuda_stream)
    return ctypes.c_void_p(int(stream))


_TORCH_TO_CT = {
    torch.float16: CoopVecComponentType.Float16,
    torch.bfloat16: CoopVecComponentType.BFloat16,
    torch.float32: CoopVecComponentType.Float32,
    torch.int8: CoopVecComponentType.SignedInt8,
    torch.uint8: CoopVecComponentType.UnsignedInt8,
    torch.int16: CoopVecComponentType.SignedInt16,
    torch.int32: CoopVecComponentType.SignedInt32,
    torch.int64: CoopVecComponentType.SignedInt64,
    torch.float64: CoopVecComponentType.Float64,
}
if hasattr(torch, "uint64"):
    _TORCH_TO_CT[torch.uint64] = CoopVecComponentType.UnsignedInt64
if hasattr(torch, "uint32"):
    _TORCH_TO_CT[torch.uint32] = CoopVecComponentType.UnsignedInt32
if hasattr(torch, "uint16"):
    _TORCH_TO_CT[torch.uint16] = CoopVecComponentType.UnsignedInt16
if hasattr(torch, "float8_e4m3fn"):
    _TORCH_TO_CT[torch.float8_e4m3fn] = CoopVecComponentType.FloatE4M3
if hasattr(torch, "float8_e5m2"):
    _TORCH_TO_CT[torch.float8_e5m2] = CoopVecComponentType.FloatE5M2

_CT_TO_TORCH = {
    CoopVecComponentType.Float16: torch.float16,
    CoopVecComponentType.BFloat16: torch.bfloat16,
    CoopVecComponentType.Float32: torch.float32,
    CoopVecComponentType.SignedInt8: torch.int8,
    CoopVecComponentType.UnsignedInt8: torch.uint8,
    CoopVecComponentType.SignedInt16: torch.int16,
    CoopVecComponentType.SignedInt32: torch.int32,
    CoopVecComponentType.SignedInt64: torch.int64,
    CoopVecComponentType.Float64: torch.float64,
}
if hasattr(torch, "uint16"):
    _CT_TO_TORCH[CoopVecComponentType.UnsignedInt16] = torch.uint16
if hasattr(torch, "uint32"):
    _CT_TO_TORCH[CoopVecComponentType.UnsignedInt32] = torch.uint32
if hasattr(torch, "uint64"):
    _CT_TO_TORCH[CoopVecComponentType.UnsignedInt64] = torch.uint64


def lastKernelName() -> str:
    """Name and specialisation of the kernel(s) the last launching call on this thread dispatched."""
    return _lib.load().cvGetLastKernelName().decode()


def componentPackingFactor(componentType: int) -> int:
    """hlsl.meta.slang:32578-32587"""
    return _lib.load().cvComponentPackingFactor(int(componentType))


def componentTypeStride(componentType: int) -> int:
    return _lib.load().cvComponentTypeStride(int(componentType))


def querySupportedCombinations():
    lib = _lib.load()
    n = lib.cvQuerySupportedCombinations(None, 0)
    arr = (_lib.CvCombination * n)()
    lib.cvQuerySupportedCombinations(arr, n)
    return [dict(inputType=CoopVecComponentType(c.inputType),
                 inputInterpretation=CoopVecComponentType(c.inputInterpretation),
                 inputPackingFactor=c.inputPackingFactor,
                 matrixInterpretation=CoopVecComponentType(c.matrixInterpretation),
                 biasInterpretation=CoopVecComponentType(c.biasInterpretation),
                 resultType=CoopVecComponentType(c.resultType),
                 transpose=bool(c.transpose)) for c in arr]


# ---------------------------------------------------------------------------------------------
# host surface
# ---------------------------------------------------------------------------------------------

def getCooperativeVectorMatrixSize(rowCount: int, colCount: int, componentType: int, layout: int,
                                   rowColumnStride: int = 0) -> int:
    """Bytes needed for a matrix (rhi::IDevice::getCooperativeVectorMatrixSize,
    mlp-training-coopvec.cpp:305-311)."""
    out = ctypes.c_size_t(0)
    _check(_lib.load().cvGetMatrixSize(rowCount, colCount, int(componentType), int(layout),
                                       rowColumnStride, ctypes.byref(out)))
    return out.value


@dataclass
class CooperativeVectorMatrixDesc:
    """Fields of rhi::CooperativeVectorMatrixDesc as the example fills them
    (mlp-training-coopvec.cpp:204-225)."""
    rowCount: int = 0
    colCount: int = 0
    componentType: int = CoopVecComponentType.Float16
    layout: int = CoopVecMatrixLayout.RowMajor
    size: int = 0
    offset: int = 0
    rowColumnStride: int = 0

    def _c(self) -> "_lib.CvMatrixDesc":
        return _lib.CvMatrixDesc(self.rowCount, self.colCount, int(self.componentType), int(self.layout),
                                 self.size, self.offset, self.rowColumnStride)


def _buffer_ptr(buf: torch.Tensor, what: str) -> int:
    if not isinstance(buf, torch.Tensor) or not buf.is_cuda:
        raise CoopVecError(SLANG_E_INVALID_ARG, "%s must be a GPU tensor" % what)
    if not buf.is_contiguous():
        raise CoopVecError(SLANG_E_INVALID_ARG, "%s must be contiguous" % what)
    return buf.data_ptr()


def convertCooperativeVectorMatrix(dstBuffer: torch.Tensor, dstDescs: Sequence[CooperativeVectorMatrixDesc],
                                   srcBuffer: torch.Tensor, srcDescs: Sequence[CooperativeVectorMatrixDesc],
                                   matrixCount: Optional[int] = None, stream=None) -> None:
    """rhi::ICommandEncoder::convertCooperativeVectorMatrix (mlp-training-coopvec.cpp:227-232)."""
    n = len(srcDescs) if matrixCount is None else matrixCount
    if len(dstDescs) < n or len(srcDescs) < n:
        raise CoopVecError(SLANG_E_INVALID_ARG, "fewer descs than matrixCount")
    d = (_lib.CvMatrixDesc * max(n, 1))(*[x._c() for x in dstDescs[:n]])
    s = (_lib.CvMatrixDesc * max(n, 1))(*[x._c() for x in srcDescs[:n]])
    for descs, buf, what in ((dstDescs[:n], dstBuffer, "dst"), (srcDescs[:n], srcBuffer, "src")):
        nbytes = buf.numel() * buf.element_size()
        for i, x in enumerate(descs):
            if x.offset + x.size > nbytes:
                raise CoopVecError(SLANG_E_BUFFER_TOO_SMALL,
                                   "%s desc %d: offset+size %d exceeds the buffer (%d bytes)"
                                   % (what, i, x.offset + x.size, nbytes))
    _check(_lib.load().cvConvertMatrices(_stream_handle(stream), _buffer_ptr(dstBuffer, "dstBuffer"), d,
                                         _buffer_ptr(srcBuffer, "srcBuffer"), s, n))


# ---------------------------------------------------------------------------------------------
# operator surface
# ---------------------------------------------------------------------------------------------

def _vector_info(v: torch.Tensor, interpretation: int, what: str):
    if not isinstance(v, torch.Tensor) or not v.is_cuda or v.dim() != 2:
        raise CoopVecError(SLANG_E_INVALID_ARG, "%s must be a 2-D GPU tensor [batch, N]" % what)
    if v.stride(1) != 1:
        raise CoopVecError(SLANG_E_INVALID_ARG, "%s: elements of one vector must be contiguous" % what)
    ct = _TORCH_TO_CT.get(v.dtype)
    if ct is None:
        raise CoopVecError(SLANG_E_NOT_AVAILABLE, "%s: unsupported element dtype %s" % (what, v.dtype))
    # a byte tensor interpreted as an 8-bit float carries elements of that type
    if ct == CoopVecComponentType.UnsignedInt8 and interpretation in (CoopVecComponentType.FloatE4M3,
                                                                    CoopVecComponentType.FloatE5M2):
        ct = CoopVecComponentType(interpretation)
    return ct, v.stride(0) * v.element_size()


def _matmul(input, inputInterpretation, k, matrix, matrixOffset, matrixInterpretation, bias, biasOffset,
            biasInterpretation, memoryLayout, transpose, matrixStride, M, resultType, activation, leakySlope,
            accumulate, out, stream, flags=0):
    lib = _lib.load()
    inCt, inStride = _vector_info(input, inputInterpretation, "input")
    batch = input.shape[0]
    if resultType is None:
        resultType = (CoopVecComponentType.SignedInt32 if inCt in (
            CoopVecComponentType.SignedInt8, CoopVecComponentType.UnsignedInt8, CoopVecComponentType.SignedInt16,
            CoopVecComponentType.UnsignedInt16, CoopVecComponentType.SignedInt32,
            CoopVecComponentType.UnsignedInt32) else
            CoopVecComponentType.SignedInt64 if inCt in (CoopVecComponentType.SignedInt64, CoopVecComponentType.UnsignedInt64) else
            CoopVecComponentType.Float64 if inCt == CoopVecComponentType.Float64 else
            CoopVecComponentType.Float32 if inCt == CoopVecComponentType.Float32 else
            CoopVecComponentType.BFloat16 if inCt == CoopVecComponentType.BFloat16 else CoopVecComponentType.Float16)
    if out is None:
        if accumulate:
            raise CoopVecError(SLANG_E_INVALID_ARG, "the accumulate forms need `out` (the vector added to)")
        dt = _CT_TO_TORCH.get(CoopVecComponentType(resultType))
        if dt is None:
            raise CoopVecError(SLANG_E_NOT_AVAILABLE, "unsupported result type %s" % resultType)
        out = torch.empty((batch, M), dtype=dt, device=input.device)
    outCt, outStride = _vector_info(out, resultType, "out")
    if out.shape[0] != batch or out.shape[1] != M or outCt != resultType:
        raise CoopVecError(SLANG_E_INVALID_ARG, "out must be [batch, M] of the result type")
    d = _lib.CvMatMulDesc()
    d.input = input.data_ptr(); d.inputStride = inStride
    d.inputType = int(inCt); d.inputInterpretation = int(inputInterpretation); d.k = int(k)
    d.output = out.data_ptr(); d.outputStride = outStride
    d.resultType = int(resultType); d.m = int(M)
    d.matrix = _buffer_ptr(matrix, "matrix"); d.matrixOffset = int(matrixOffset)
    d.matrixInterpretation = int(matrixInterpretation); d.layout = int(memoryLayout)
    d.transpose = 1 if transpose else 0; d.matrixStride = int(matrixStride)
    if bias is not None:
        d.bias = _buffer_ptr(bias, "bias"); d.biasOffset = int(biasOffset)
        d.biasInterpretation = int(biasInterpretation)
    else:
        d.bias = None; d.biasOffset = 0; d.biasInterpretation = -1
    d.activation = int(activation); d.leakySlope = float(leakySlope)
    d.accumulate = 1 if accumulate else 0; d.batch = batch; d.flags = int(flags)
    _check(lib.cvMatMul(_stream_handle(stream), ctypes.byref(d)))
    return out


def coopVecMatMulPacked(input: torch.Tensor, inputInterpretation: int, k: int, matrix: torch.Tensor,
                        matrixOffset: int, matrixInterpretation: int, memoryLayout: int, transpose: bool,
                        matrixStride: int, *, M: int, resultType: Optional[int] = None,
                        out: Optional[torch.Tensor] = None, accumulate: bool = False, stream=None,
                        flags: int = 0):
    """coopVecMatMulPacked<T,M,PackedK,U> (hlsl.meta.slang:32786-32796); accumulate=True is the
    member form matMulAccumPacked (:31476)."""
    return _matmul(input, inputInterpretation, k, matrix, matrixOffset, matrixInterpretation, None, 0, -1,
                   memoryLayout, transpose, matrixStride, M, resultType, Activation.NoActivation, 0.0,
                   accumulate, out, stream, flags)


def coopVecMatMul(input: torch.Tensor, inputInterpretation: int, matrix: torch.Tensor, matrixOffset: int,
                  matrixInterpretation: int, memoryLayout: int, transpose: bool, matrixStride: int, *,
                  M: int, resultType: Optional[int] = None, out: Optional[torch.Tensor] = None,
                  accumulate: bool = False, stream=None, flags: int = 0):
    """coopVecMatMul<T,M,K,U> (hlsl.meta.slang:32954-32963)."""
    if componentPackingFactor(inputInterpretation) != 1:   # static_assert :32965
        raise CoopVecError(SLANG_E_INVALID_ARG,
                           "for packed inputInterpretation values please use coopVecMatMulPacked and specify k manually")
    return coopVecMatMulPacked(input, inputInterpretation, input.shape[1], matrix, matrixOffset,
                               matrixInterpretation, memoryLayout, transpose, matrixStride, M=M,
                               resultType=resultType, out=out, accumulate=accumulate, stream=stream,
                               flags=flags)


def coopVecMatMulAddPacked(input: torch.Tensor, inputInterpretation: int, k: int, matrix: torch.Tensor,
                           matrixOffset: int, matrixInterpretation: int, bias: torch.Tensor, biasOffset: int,
                           biasInterpretation: int, memoryLayout: int, transpose: bool, matrixStride: int, *,
                           M: int, resultType: Optional[int] = None, out: Optional[torch.Tensor] = None,
                           accumulate: bool = False, activation: int = Activation.NoActivation,
                           leakySlope: float = 0.0, stream=None, flags: int = 0):
    """coopVecMatMulAddPacked<T,M,PackedK,U> (hlsl.meta.slang:32983-32996)."""
    return _matmul(input, inputInterpretation, k, matrix, matrixOffset, matrixInterpretation, bias, biasOffset,
                   biasInterpretation, memoryLayout, transpose, matrixStride, M, resultType, activation,
                   leakySlope, accumulate, out, stream, flags)


def coopVecMatMulAdd(input: torch.Tensor, inputInterpretation: int, matrix: torch.Tensor, matrixOffset: int,
                     matrixInterpretation: int, bias: torch.Tensor, biasOffset: int, biasInterpretation: int,
                     memoryLayout: int, transpose: bool, matrixStride: int, *, M: int,
                     resultType: Optional[int] = None, out: Optional[torch.Tensor] = None,
                     accumulate: bool = False, activation: int = Activation.NoActivation,
                     leakySlope: float = 0.0, stream=None, flags: int = 0):
    """coopVecMatMulAdd<T,M,K,U> (hlsl.meta.slang:33160-33173)."""
    if componentPackingFactor(inputInterpretation) != 1:
        raise CoopVecError(SLANG_E_INVALID_ARG,
                           "for packed inputInterpretation values please use coopVecMatMulAddPacked and specify k manually")
    return coopVecMatMulAddPacked(input, inputInterpretation, input.shape[1], matrix, matrixOffset,
                                  matrixInterpretation, bias, biasOffset, biasInterpretation, memoryLayout,
                                  transpose, matrixStride, M=M, resultType=resultType, out=out,
                                  accumulate=accumulate, activation=activation, leakySlope=leakySlope,
                                  stream=stream, flags=flags)


# ---------------------------------------------------------------------------------------------
# element-wise surface
# ---------------------------------------------------------------------------------------------

def _ew_operand(t: Optional[torch.Tensor], like: torch.Tensor, what: str):
    if t is None:
        return None, 0
    if not t.is_cuda or t.dim() != 2 or t.stride(1) != 1 or t.shape != like.shape or t.dtype != like.dtype:
        raise CoopVecError(SLANG_E_INVALID_ARG, "%s must be a GPU tensor [batch, N] of the same shape and dtype" % what)
    return t.data_ptr(), t.stride(0) * t.element_size()


def elementwise(op: int, a: torch.Tensor, b: Optional[torch.Tensor] = None, c: Optional[torch.Tensor] = None, *,
                param: float = 0.0, out: Optional[torch.Tensor] = None, stream=None) -> torch.Tensor:
    """op(a, b, c) per component of every CoopVec of the batch (fp16 or fp32 tensors [batch, N]; integer and
    fp64 tensors for the arithmetic operators, min, max and clamp):
    e.g. elementwise(ElementwiseOp.Clamp, x, lo, hi) is Slang's clamp(x, lo, hi)."""
    ct = _TORCH_TO_CT.get(a.dtype)
    if out is None:
        out = torch.empty_like(a, memory_format=torch.contiguous_format)
    pa, sa = _ew_operand(a, a, "a"); pb, sb = _ew_operand(b, a, "b"); pc, sc = _ew_operand(c, a, "c")
    po, so = _ew_operand(out, a, "out")
    _check(_lib.load().cvElementwise(_stream_handle(stream), int(op), int(ct) if ct is not None else -1, a.shape[1],
                                     a.shape[0], pa, sa, pb, sb, pc, sc, po, so, float(param)))
    return out


def copyFrom(other: torch.Tensor, T: int, *, out: Optional[torch.Tensor] = None, stream=None) -> torch.Tensor:
    """CoopVec<T,N>(CoopVec<U,N>) / CoopVec.copyFrom (hlsl.meta.slang:30683-30730) for every vector of the batch:
    the elements of `other` converted to component type T."""
    src_ct, src_stride = _vector_info(other, -1, "other")
    if out is None:
        dt = _CT_TO_TORCH.get(CoopVecComponentType(T))
        if dt is None:
            raise CoopVecError(SLANG_E_NOT_AVAILABLE, "unsupported element type %s" % T)
        out = torch.empty(other.shape, dtype=dt, device=other.device)
    dst_ct, dst_stride = _vector_info(out, -1, "out")
    if out.shape != other.shape or dst_ct != T:
        raise CoopVecError(SLANG_E_INVALID_ARG, "out must have the shape of `other` and element type T")
    _check(_lib.load().cvVectorCast(_stream_handle(stream), other.shape[1], other.shape[0], other.data_ptr(), src_stride,
                                    int(src_ct), out.data_ptr(), dst_stride, int(dst_ct)))
    return out


def elementwiseBackward(op: int, dOut: torch.Tensor, a: torch.Tensor, b: Optional[torch.Tensor] = None,
                        c: Optional[torch.Tensor] = None, *, param: float = 0.0, stream=None):
    """Reverse-mode derivative of elementwise(op, a, b, c) by Slang's rules (diff.meta.slang:1948-2470):
    returns (dA, dB, dC), None for operands the operator does not take."""
    ct = _TORCH_TO_CT.get(a.dtype)
    grads = [torch.empty_like(a, memory_format=torch.contiguous_format) if t is not None else None for t in (a, b, c)]
    pa, sa = _ew_operand(a, a, "a"); pb, sb = _ew_operand(b, a, "b"); pc, sc = _ew_operand(c, a, "c")
    pg, sg = _ew_operand(dOut, a, "dOut")
    ptrs = [_ew_operand(g, a, "grad") for g in grads]
    _check(_lib.load().cvElementwiseBackward(_stream_handle(stream), int(op), int(ct) if ct is not None else -1,
                                             a.shape[1], a.shape[0], pa, sa, pb, sb, pc, sc, pg, sg,
                                             ptrs[0][0], ptrs[0][1], ptrs[1][0], ptrs[1][1], ptrs[2][0], ptrs[2][1],
                                             float(param)))
    return tuple(grads)


# ---------------------------------------------------------------------------------------------
# input encoders of the neural module
# ---------------------------------------------------------------------------------------------

class HashType(enum.IntEnum):
    """hash-function.slang:6-13"""
    Prime = 0
    CoherentPrime = 1
    ReversedPrime = 2
    Rng = 3
    BaseConvert = 4


def gridHash(hashType: int, positions: torch.Tensor, *, stream=None) -> torch.Tensor:
    """gridHash<Type, Dimensions> (hash-function.slang:134-151) of integer grid positions [batch, D]."""
    if positions.dtype not in (torch.int32, getattr(torch, "uint32", torch.int32)) or positions.dim() != 2 or positions.stride(1) != 1:
        raise CoopVecError(SLANG_E_INVALID_ARG, "positions must be a 32-bit integer GPU tensor [batch, D]")
    out = torch.empty(positions.shape[0], dtype=torch.int32, device=positions.device)
    _check(_lib.load().cvGridHash(_stream_handle(stream), int(hashType), positions.shape[1], positions.data_ptr(),
                                  positions.stride(0) * 4, out.data_ptr(), positions.shape[0]))
    return out


class PermutoEncoder:
    """PermutoEncoder<T, Dimensions, FeatureDimensionPerEntry, Log2HashmapSize, MaxLevels>
    (permuto-encoder.slang:8-20) with its HyperParameters prepared as prepareLevelInfo does (:339-368)."""

    def __init__(self, dimensions: int, featureDimensionPerEntry: int, log2HashmapSize: int, maxLevels: int, *,
                 baseScale: float, log2PerLevelScale: float, maxLevelRatio: float = 1.1, seed: int = 1337,
                 dtype: torch.dtype = torch.float32):
        self.desc = _lib.CvPermutoDesc()
        self.desc.dimensions = dimensions
        self.desc.featureDimensionPerEntry = featureDimensionPerEntry
        self.desc.log2HashmapSize = log2HashmapSize
        self.desc.maxLevels = maxLevels
        self.desc.elementType = int(_TORCH_TO_CT.get(dtype, -1))
        self.dtype = dtype
        _check(_lib.load().cvPermutoPrepareLevels(ctypes.byref(self.desc), baseScale, log2PerLevelScale, maxLevelRatio, seed))

    @property
    def featureTableElements(self) -> int:
        return (1 << self.desc.log2HashmapSize) * self.desc.maxLevels * self.desc.featureDimensionPerEntry

    @property
    def outputSize(self) -> int:
        return self.desc.maxLevels * self.desc.featureDimensionPerEntry

    def encode(self, positions: torch.Tensor, featureTable: torch.Tensor, *, out: Optional[torch.Tensor] = None, stream=None):
        """encode (:319-337) of every row of positions [batch, Dimensions]."""
        if positions.dtype != self.dtype or featureTable.dtype != self.dtype or positions.dim() != 2 or positions.stride(1) != 1:
            raise CoopVecError(SLANG_E_INVALID_ARG, "positions [batch, D] and featureTable must have the encoder's dtype")
        if featureTable.numel() < self.featureTableElements or not featureTable.is_contiguous():
            raise CoopVecError(SLANG_E_BUFFER_TOO_SMALL, "featureTable holds fewer than %d elements" % self.featureTableElements)
        if out is None:
            out = torch.empty(positions.shape[0], self.outputSize, dtype=self.dtype, device=positions.device)
        es = positions.element_size()
        _check(_lib.load().cvPermutoEncode(_stream_handle(stream), ctypes.byref(self.desc), positions.data_ptr(),
                                           positions.stride(0) * es, featureTable.data_ptr(), out.data_ptr(),
                                           out.stride(0) * es, positions.shape[0]))
        return out

    def encodeAndEval(self, positions: torch.Tensor, featureTable: torch.Tensor, layers, *,
                      out: Optional[torch.Tensor] = None, flags: int = 0, stream=None) -> torch.Tensor:
        """network.eval(encoder.encode(position)) for every row of positions, in one kernel: what a Slang thread does
        when it hands encode's result (:319-337) to its network; the encoded vectors never reach memory.  Same bits as
        mlpForward(layers, self.encode(positions, featureTable)); half encoders and networks only."""
        if positions.dtype != self.dtype or featureTable.dtype != self.dtype or positions.dim() != 2 or positions.stride(1) != 1:
            raise CoopVecError(SLANG_E_INVALID_ARG, "positions [batch, D] and featureTable must have the encoder's dtype")
        if featureTable.numel() < self.featureTableElements or not featureTable.is_contiguous():
            raise CoopVecError(SLANG_E_BUFFER_TOO_SMALL, "featureTable holds fewer than %d elements" % self.featureTableElements)
        batch = positions.shape[0]
        if out is None:
            out = torch.empty((batch, layers[-1].outputSize), dtype=torch.float16, device=positions.device)
        outCt, outStride = _vector_info(out, CoopVecComponentType.Float16, "out")
        d, keep = _mlp_desc(layers, CoopVecComponentType.Float16, CoopVecComponentType.Float32, flags, 0)
        es = positions.element_size()
        _check(_lib.load().cvPermutoMlpForward(_stream_handle(stream), ctypes.byref(self.desc), positions.data_ptr(),
                                               positions.stride(0) * es, featureTable.data_ptr(), ctypes.byref(d),
                                               out.data_ptr(), outStride, batch))
        return out

    def backward(self, positions: torch.Tensor, featureTable: torch.Tensor, dOut: torch.Tensor, *,
                 dFeatureTable: Optional[torch.Tensor] = None, wantPositionGrad: bool = True, stream=None):
        """bwd_diff of encode: returns (dPositions or None, dFeatureTable); the table gradient is added to."""
        if dFeatureTable is None:
            dFeatureTable = torch.zeros_like(featureTable)
        dPos = torch.empty_like(positions, memory_format=torch.contiguous_format) if wantPositionGrad else None
        es = positions.element_size()
        _check(_lib.load().cvPermutoEncodeBackward(_stream_handle(stream), ctypes.byref(self.desc), positions.data_ptr(),
                                                   positions.stride(0) * es, featureTable.data_ptr(), dOut.data_ptr(),
                                                   dOut.stride(0) * es, dPos.data_ptr() if dPos is not None else None,
                                                   dPos.stride(0) * es if dPos is not None else 0,
                                                   dFeatureTable.data_ptr(), positions.shape[0]))
        return dPos, dFeatureTable


# ---------------------------------------------------------------------------------------------
# fused MLP: the example's FeedForwardLayer chain
# ---------------------------------------------------------------------------------------------

@dataclass
class FeedForwardLayer:
    """One layer of the example's network (examples/mlp-training-coopvec/fflayer.slang:7-67):
    device buffers for weights / weightsGrad / biases / biasesGrad plus what is constexpr in Slang."""
    inputSize: int
    outputSize: int
    weights: torch.Tensor                  # raw bytes (any dtype), layout `weightLayout`
    biases: Optional[torch.Tensor] = None  # fp16 [outputSize]
    weightLayout: int = CoopVecMatrixLayout.RowMajor
    weightStride: int = 0
    activation: int = Activation.NoActivation
    leakySlope: float = 0.0
    weightsGrad: Optional[torch.Tensor] = None
    biasesGrad: Optional[torch.Tensor] = None
    gradLayout: int = CoopVecMatrixLayout.TrainingOptimal
    gradStride: int = 0


class InputEncoding(enum.IntEnum):
    """CvInputEncoding: XYSquares is the example's MyNetwork::encodeInput (network.slang:35-38) on
    float2 samples: layer 0 sees (x, y, x*x, y*y) in half."""
    NoEncoding = 0
    XYSquares = 1


def _mlp_carrier_type(weightType: int) -> CoopVecComponentType:
    if weightType in (CoopVecComponentType.Float32, CoopVecComponentType.BFloat16):
        return CoopVecComponentType(weightType)
    return CoopVecComponentType.Float16


def _mlp_desc(layers: Sequence[FeedForwardLayer], weightType: int, gradType: int, flags: int,
              inputEncoding: int = 0):
    arr = (_lib.CvMlpLayer * len(layers))()
    for i, L in enumerate(layers):
        arr[i].weights = _buffer_ptr(L.weights, "weights")
        arr[i].weightsGrad = _buffer_ptr(L.weightsGrad, "weightsGrad") if L.weightsGrad is not None else None
        arr[i].biases = _buffer_ptr(L.biases, "biases") if L.biases is not None else None
        arr[i].biasesGrad = _buffer_ptr(L.biasesGrad, "biasesGrad") if L.biasesGrad is not None else None
        arr[i].inputSize = L.inputSize; arr[i].outputSize = L.outputSize
        arr[i].weightLayout = int(L.weightLayout); arr[i].weightStride = int(L.weightStride)
        arr[i].gradLayout = int(L.gradLayout); arr[i].gradStride = int(L.gradStride)
        arr[i].activation = int(L.activation); arr[i].leakySlope = float(L.leakySlope)
    d = _lib.CvMlpDesc()
    d.layers = arr; d.numLayers = len(layers)
    d.inputType = int(weightType); d.weightType = int(weightType)
    carrier = _mlp_carrier_type(weightType)      # half, or T for networks of one type T = float / bfloat16
    d.biasType = int(carrier); d.outputType = int(carrier)
    d.gradType = int(gradType); d.flags = int(flags); d.inputEncoding = int(inputEncoding)
    if inputEncoding:
        d.inputType = int(CoopVecComponentType.Float32)
    return d, arr


def mlpForward(layers: Sequence[FeedForwardLayer], input: torch.Tensor, *,
               weightType: int = CoopVecComponentType.Float16, out: Optional[torch.Tensor] = None,
               flags: int = 0, inputEncoding: int = 0, stream=None) -> torch.Tensor:
    """network.eval over a batch: every layer is coopVecMatMulAdd + activation with CoopVec<half>
    between layers (network.slang:41-47), fused into one kernel.  weightType Float32 / BFloat16: a network
    of that one type (vectors, biases, results), the neural module's FFLayer<float, ...> chain."""
    inCt, inStride = _vector_info(input, weightType, "input")
    batch = input.shape[0]
    carrier = _mlp_carrier_type(weightType)
    if out is None:
        out = torch.empty((batch, layers[-1].outputSize), dtype=_CT_TO_TORCH[carrier], device=input.device)
    outCt, outStride = _vector_info(out, carrier, "out")
    if outCt != carrier:
        raise CoopVecError(SLANG_E_INVALID_ARG, "out must have the network's result type")
    d, keep = _mlp_desc(layers, weightType, CoopVecComponentType.Float32, flags, inputEncoding)
    d.inputType = int(inCt)
    _check(_lib.load().cvMlpForward(_stream_handle(stream), ctypes.byref(d), input.data_ptr(), inStride,
                                    out.data_ptr(), outStride, batch))
    return out


class MlpForwardPlan:
    """mlpForward with the network description marshalled once.

    The example's host program fills its constant buffer of per-layer device addresses once and
    dispatches many times (mlp-training-coopvec.cpp:146-161, :319-334); a C caller of cvMlpForward does
    the same with one CvMlpDesc.  This is that pattern for the Python mirror: the descriptor is built
    here, a call only passes the vectors.  The layers' buffers must stay alive and in place (the plan
    keeps references), and a change of a FeedForwardLayer after the plan was made is not seen."""

    def __init__(self, layers: Sequence[FeedForwardLayer], *, weightType: int = CoopVecComponentType.Float16,
                 flags: int = 0, inputEncoding: int = 0):
        self._layers = list(layers)
        self._weightType = weightType
        self._desc, self._keep = _mlp_desc(self._layers, weightType, CoopVecComponentType.Float32, flags, inputEncoding)
        self._ref = ctypes.byref(self._desc)
        self._fn = _lib.load().cvMlpForward
        self._outputSize = self._layers[-1].outputSize
        self._carrier = _mlp_carrier_type(weightType)
        self._outDtype = _CT_TO_TORCH[self._carrier]
        self._inCt = None

    def __call__(self, input: torch.Tensor, out: Optional[torch.Tensor] = None, stream=None) -> torch.Tensor:
        inCt, inStride = _vector_info(input, self._weightType, "input")
        if inCt != self._inCt:
            self._desc.inputType = int(inCt)
            self._inCt = inCt
        batch = input.shape[0]
        if out is None:
            out = torch.empty((batch, self._outputSize), dtype=self._outDtype, device=input.device)
        outCt, outStride = _vector_info(out, self._carrier, "out")
        if outCt != self._carrier:
            raise CoopVecError(SLANG_E_INVALID_ARG, "out must have the network's result type")
        rc = self._fn(_stream_handle(stream), self._ref, input.data_ptr(), inStride, out.data_ptr(), outStride, batch)
        if rc < 0:
            _check(rc)
        return out


def mlpTrainStepWorkspaceSize(layers: Sequence[FeedForwardLayer], batch: int,
                              gradType: int = CoopVecComponentType.Float32, flags: int = 0, inputEncoding: int = 0,
                              weightType: int = CoopVecComponentType.Float16) -> int:
    d, keep = _mlp_desc(layers, weightType, gradType, flags, inputEncoding)
    out = ctypes.c_size_t(0)
    _check(_lib.load().cvMlpTrainStepWorkspaceSize(ctypes.byref(d), batch, ctypes.byref(out)))
    return out.value


def mlpTrainStep(layers: Sequence[FeedForwardLayer], input: torch.Tensor, targets: Optional[torch.Tensor] = None, *,
                 lossScale: float = 1.0, gradType: int = CoopVecComponentType.Float32,
                 workspace: Optional[torch.Tensor] = None, lossSum: Optional[torch.Tensor] = None,
                 inputEncoding: int = 0, flags: int = 0, weightType: int = CoopVecComponentType.Float16,
                 lossMax: Optional[torch.Tensor] = None, stream=None):
    """learnGradient over a batch (kernels.slang:9-27): forward, bwd_diff of the squared-error loss,
    weight gradients accumulated into every layer's weightsGrad (coopVecOuterProductAccumulate,
    fflayer.slang:35-41) and bias gradients into biasesGrad (coopVecReduceSumAccumulate, :44),
    deterministically.  Returns (workspace, lossSum) so that both can be reused.  weightType Float32: a network
    of float (vectors, targets, parameters), stepped layer by layer with Float32 gradients.  lossMax (one float32 on
    the device) receives the largest per-sample loss, the figure learnGradient leaves in its loss buffer
    (kernels.slang:21-26)."""
    _, inStride = _vector_info(input, weightType, "input")
    batch = input.shape[0]
    d, keep = _mlp_desc(layers, weightType, gradType, flags, inputEncoding)
    if lossMax is not None:
        if lossMax.dtype != torch.float32 or lossMax.numel() < 1:
            raise CoopVecError(SLANG_E_INVALID_ARG, "lossMax must be a float32 tensor")
        d.lossMax = lossMax.data_ptr()
    lib = _lib.load()
    if workspace is None:
        need = ctypes.c_size_t(0)
        _check(lib.cvMlpTrainStepWorkspaceSize(ctypes.byref(d), batch, ctypes.byref(need)))
        workspace = torch.empty(need.value, dtype=torch.uint8, device=input.device)
    if lossSum is None:
        lossSum = torch.zeros(1, dtype=torch.float32, device=input.device)
    tptr, tstride = None, 0
    if targets is not None:
        _, tstride = _vector_info(targets, weightType, "targets")
        tptr = targets.data_ptr()
    _check(lib.cvMlpTrainStep(_stream_handle(stream), ctypes.byref(d), input.data_ptr(), inStride, tptr, tstride,
                              float(lossScale), batch, lossSum.data_ptr(), workspace.data_ptr(),
                              workspace.numel() * workspace.element_size()))
    return workspace, lossSum


NOALLOC_SCRATCH_BYTES = 16 << 20   # CV_NOALLOC_SCRATCH_BYTES of include/coopvec.h


def mlpTrainStepNoAlloc(layers: Sequence[FeedForwardLayer], input: torch.Tensor, targets: Optional[torch.Tensor],
                        lossSum: torch.Tensor, *, lossScale: float = 1.0,
                        gradType: int = CoopVecComponentType.Float32, stream=None) -> None:
    """mlpTrainStep for callers that cannot allocate: the gradient partials go to an array inside
    the library's device image, nothing is allocated (lossSum is the caller's, too).  Calls that
    overlap on one GPU race on that array."""
    _, inStride = _vector_info(input, CoopVecComponentType.Float16, "input")
    d, keep = _mlp_desc(layers, CoopVecComponentType.Float16, gradType, 0)
    tptr, tstride = None, 0
    if targets is not None:
        _, tstride = _vector_info(targets, CoopVecComponentType.Float16, "targets")
        tptr = targets.data_ptr()
    _check(_lib.load().cvMlpTrainStepNoAlloc(_stream_handle(stream), ctypes.byref(d), input.data_ptr(), inStride,
                                             tptr, tstride, float(lossScale), input.shape[0],
                                             lossSum.data_ptr() if lossSum is not None else None))


# ---------------------------------------------------------------------------------------------
# training operators over a batch
# ---------------------------------------------------------------------------------------------

def coopVecOuterProductAccumulate(a: torch.Tensor, b: torch.Tensor, matrix: torch.Tensor, matrixOffset: int,
                                  matrixStride: int, memoryLayout: int, matrixInterpretation: int, *,
                                  workspace: Optional[torch.Tensor] = None, stream=None) -> None:
    """coopVecOuterProductAccumulate<T,M,N> (hlsl.meta.slang:33227-33235) for every row of the batch:
    matrix[i][j] += sum_s a[s][i]*b[s][j], without atomics and bitwise reproducible."""
    lib = _lib.load()
    ta, sa = _vector_info(a, CoopVecComponentType.Float16, "a")
    tb, sb = _vector_info(b, CoopVecComponentType.Float16, "b")
    if a.shape[0] != b.shape[0] or ta != tb:
        raise CoopVecError(SLANG_E_INVALID_ARG, "a and b must have the same batch and element type")
    batch, m, n = a.shape[0], a.shape[1], b.shape[1]
    if workspace is None:
        need = ctypes.c_size_t(0)
        _check(lib.cvOuterProductAccumulateWorkspaceSize(m, n, batch, ctypes.byref(need)))
        workspace = torch.empty(max(need.value, 16), dtype=torch.uint8, device=a.device)
    _check(lib.cvOuterProductAccumulate(_stream_handle(stream), a.data_ptr(), sa, m, b.data_ptr(), sb, n, int(ta), batch,
                                        _buffer_ptr(matrix, "matrix"), int(matrixOffset), int(matrixStride),
                                        int(memoryLayout), int(matrixInterpretation), workspace.data_ptr(),
                                        workspace.numel() * workspace.element_size()))


def coopVecReduceSumAccumulate(v: torch.Tensor, buffer: torch.Tensor, offset: int, *,
                               bufferType: Optional[int] = None, workspace: Optional[torch.Tensor] = None,
                               stream=None) -> None:
    """coopVecReduceSumAccumulate<T,N> (hlsl.meta.slang:33330-33334) for every row of the batch:
    buffer[i] += sum_s v[s][i].  The reference's destination type is the vector's type; bufferType
    Float32 gives the fp32 accumulation buffers the training configuration asks for."""
    lib = _lib.load()
    tv, sv = _vector_info(v, CoopVecComponentType.Float16, "v")
    batch, n = v.shape
    if bufferType is None:
        bufferType = tv
    if workspace is None:
        need = ctypes.c_size_t(0)
        _check(lib.cvReduceSumAccumulateWorkspaceSize(n, batch, ctypes.byref(need)))
        workspace = torch.empty(max(need.value, 16), dtype=torch.uint8, device=v.device)
    _check(lib.cvReduceSumAccumulate(_stream_handle(stream), v.data_ptr(), sv, n, int(tv), batch,
                                     _buffer_ptr(buffer, "buffer"), int(offset), int(bufferType),
                                     workspace.data_ptr(), workspace.numel() * workspace.element_size()))


# ---------------------------------------------------------------------------------------------
# the neural module's network parameter block
# ---------------------------------------------------------------------------------------------

class NeuralWeightOrder(enum.IntEnum):
    """CvNeuralWeightOrder: Native is this library's; the others are the reference's SPIR-V, Metal and
    CUDA orders (network-parameter-layout-converter.slang:137-172)."""
    Native = 0
    TiledRowMajor = 1
    PaddedRowMajor = 2
    CudaMatrixB = 3


class NetworkParameterLayoutConverter:
    """NetworkParameterLayoutConverter<T, BiasMask, D0, D1, ...>
    (network-parameter-layout-converter.slang:469-555) plus the FFLayer chain over the block."""

    def __init__(self, dtype: torch.dtype, biasMask: int, *dims: int, order: int = NeuralWeightOrder.Native):
        self.desc = _lib.CvNeuralNetworkDesc()
        self.desc.layerCount = len(dims) - 1
        for i, d in enumerate(dims):
            self.desc.dims[i] = d
        self.desc.biasMask = biasMask
        self.desc.elementType = int(_TORCH_TO_CT.get(dtype, -1))
        self.desc.order = int(order)
        self.dtype = dtype
        l, p = ctypes.c_size_t(0), ctypes.c_size_t(0)
        _check(_lib.load().cvNeuralNetworkSize(ctypes.byref(self.desc), ctypes.byref(l), ctypes.byref(p)))
        self.ElementCountLogical, self.ElementCountPhysical = l.value, p.value
        self.BytesLogical = l.value * torch.empty(0, dtype=dtype).element_size()
        self.BytesPhysical = p.value * torch.empty(0, dtype=dtype).element_size()

    def _buf(self, t, count, what):
        if t.dtype != self.dtype or not t.is_cuda or not t.is_contiguous() or t.numel() < count:
            raise CoopVecError(SLANG_E_BUFFER_TOO_SMALL, "%s must be a contiguous GPU tensor of at least %d %s" % (what, count, self.dtype))
        return t.data_ptr()

    def toOptimalLayout(self, portable: torch.Tensor, optimal: Optional[torch.Tensor] = None, *, stream=None) -> torch.Tensor:
        if optimal is None:
            optimal = torch.empty(self.ElementCountPhysical, dtype=self.dtype, device=portable.device)
        _check(_lib.load().cvNeuralToOptimalLayout(_stream_handle(stream), ctypes.byref(self.desc),
                                                   self._buf(portable, self.ElementCountLogical, "portable"),
                                                   self._buf(optimal, self.ElementCountPhysical, "optimal")))
        return optimal

    def toPortableLayout(self, optimal: torch.Tensor, portable: Optional[torch.Tensor] = None, *, stream=None) -> torch.Tensor:
        if portable is None:
            portable = torch.empty(self.ElementCountLogical, dtype=self.dtype, device=optimal.device)
        _check(_lib.load().cvNeuralToPortableLayout(_stream_handle(stream), ctypes.byref(self.desc),
                                                    self._buf(optimal, self.ElementCountPhysical, "optimal"),
                                                    self._buf(portable, self.ElementCountLogical, "portable")))
        return portable

    def _acts(self, activations, slopes):
        n = self.desc.layerCount
        a = (ctypes.c_int32 * n)(*[int(x) for x in (activations or [0] * n)])
        s = (ctypes.c_float * n)(*[float(x) for x in (slopes or [0.0] * n)])
        return a, s

    def eval(self, params: torch.Tensor, input: torch.Tensor, *, optimalLayout: bool, activations=None, leakySlopes=None,
             out: Optional[torch.Tensor] = None, stream=None) -> torch.Tensor:
        """The FFLayer chain (layers.slang:90-110) over the block; vectors and results have the block's element type."""
        _, inStride = _vector_info(input, self.desc.elementType, "input")
        if input.dtype != self.dtype or (out is not None and out.dtype != self.dtype):
            raise CoopVecError(SLANG_E_INVALID_ARG, "input and out must have the network's element type")
        if out is None:
            out = torch.empty(input.shape[0], self.desc.dims[self.desc.layerCount], dtype=self.dtype, device=input.device)
        a, s = self._acts(activations, leakySlopes)
        count = self.ElementCountPhysical if optimalLayout else self.ElementCountLogical
        _check(_lib.load().cvNeuralMlpForward(_stream_handle(stream), ctypes.byref(self.desc), 1 if optimalLayout else 0,
                                              self._buf(params, count, "params"), a, s, input.data_ptr(), inStride,
                                              out.data_ptr(), out.stride(0) * out.element_size(), input.shape[0]))
        return out

    def trainStep(self, params: torch.Tensor, paramGrads: torch.Tensor, input: torch.Tensor, targets: Optional[torch.Tensor], *,
                  optimalLayout: bool, activations=None, leakySlopes=None, lossScale: float = 1.0, stream=None) -> torch.Tensor:
        """bwd_diff through the chain; gradients accumulate in `paramGrads`, laid out like `params`; vectors and
        targets have the block's element type."""
        _, inStride = _vector_info(input, self.desc.elementType, "input")
        if input.dtype != self.dtype or (targets is not None and targets.dtype != self.dtype):
            raise CoopVecError(SLANG_E_INVALID_ARG, "input and targets must have the network's element type")
        a, s = self._acts(activations, leakySlopes)
        count = self.ElementCountPhysical if optimalLayout else self.ElementCountLogical
        need = ctypes.c_size_t(0)
        lib = _lib.load()
        _check(lib.cvNeuralMlpTrainStepWorkspaceSize(ctypes.byref(self.desc), input.shape[0], ctypes.byref(need)))
        ws = torch.empty(need.value, dtype=torch.uint8, device=input.device)
        loss = torch.zeros(1, dtype=torch.float32, device=input.device)
        tptr, tstride = None, 0
        if targets is not None:
            _, tstride = _vector_info(targets, self.desc.elementType, "targets")
            tptr = targets.data_ptr()
        _check(lib.cvNeuralMlpTrainStep(_stream_handle(stream), ctypes.byref(self.desc), 1 if optimalLayout else 0,
                                        self._buf(params, count, "params"), self._buf(paramGrads, count, "paramGrads"), a, s,
                                        input.data_ptr(), inStride, tptr, tstride, float(lossScale), input.shape[0],
                                        loss.data_ptr(), ws.data_ptr(), need.value))
        return loss


# ---------------------------------------------------------------------------------------------
# parameter update of the example
# ---------------------------------------------------------------------------------------------

ADAM_STATE_BYTES = 8    # {half mean; half variance; int iteration}, adam.slang:5-10


def adjustParameters(adamStates: torch.Tensor, params: torch.Tensor, gradients: torch.Tensor, count: Optional[int] = None,
                     *, beta1: float = 0.9, beta2: float = 0.999, epsilon: float = 1e-7, learningRate: float = 0.01,
                     stream=None) -> None:
    """The adjustParameters kernel of the example (kernels.slang:29-45): one Adam step in half on
    `count` fp16 parameters; gradients are zeroed.  adamStates: raw bytes, 8 per parameter."""
    if count is None:
        count = params.numel()
    if params.dtype != torch.float16 or gradients.dtype != torch.float16:
        raise CoopVecError(SLANG_E_INVALID_ARG, "params and gradients must be fp16")
    if (adamStates.numel() * adamStates.element_size() < count * ADAM_STATE_BYTES or params.numel() < count
            or gradients.numel() < count):
        raise CoopVecError(SLANG_E_BUFFER_TOO_SMALL, "buffers smaller than count")
    _check(_lib.load().cvAdamStep(_stream_handle(stream), _buffer_ptr(adamStates, "adamStates"),
                                  _buffer_ptr(params, "params"), _buffer_ptr(gradients, "gradients"), int(count),
                                  beta1, beta2, epsilon, learningRate))


def mlpAdjustParameters(layers: Sequence[FeedForwardLayer], weightStates: Sequence[torch.Tensor],
                        biasStates: Optional[Sequence[Optional[torch.Tensor]]] = None, *,
                        gradType: int = CoopVecComponentType.Float16, beta1: float = 0.9, beta2: float = 0.999,
                        epsilon: float = 1e-7, learningRate: float = 0.01, stream=None) -> None:
    """adjustParameters for a whole network in one launch, straight from the gradient buffers mlpTrainStep fills (any
    layout, TrainingOptimal included): what the example does with convertCooperativeVectorMatrix + adjustParameters
    (mlp-training-coopvec.cpp:203-250).  Every gradient element read is left at zero.  weightStates[l] / biasStates[l]:
    raw bytes, 8 per parameter, weights in row-major order."""
    d, keep = _mlp_desc(layers, CoopVecComponentType.Float16, gradType, 0)
    n = len(layers)
    ws = (ctypes.c_void_p * n)(*[_buffer_ptr(t, "weightStates") for t in weightStates])
    bs = (ctypes.c_void_p * n)(*[(_buffer_ptr(t, "biasStates") if t is not None else None)
                                 for t in (biasStates if biasStates is not None else [None] * n)])
    _check(_lib.load().cvMlpAdamStep(_stream_handle(stream), ctypes.byref(d), ws, bs, beta1, beta2, epsilon, learningRate))
