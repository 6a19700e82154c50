"""Loader for the gfx950 shared library.  There is no CPU fallback: if the library is
missing or cannot be loaded every operator raises."""
from __future__ import annotations

import ctypes
import os

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
# COOPVEC_MI355X_LIB points at another build of the same library (e.g. a tuning variant)
LIB_PATH = os.environ.get("COOPVEC_MI355X_LIB") or os.path.join(_PKG_DIR, "libcoopvec_mi355x.so")

_lib = None


class CoopVecLibraryMissing(ImportError):
    pass


def load() -> ctypes.CDLL:
    """Return the loaded library, loading it on first use."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise CoopVecLibraryMissing(
            "%s is not built; run `python -m slang_amd.build` (needs hipcc). "
            "There is no CPU fallback for the cooperative-vector operators." % LIB_PATH)
    # torch ships the HIP runtime this process uses for device memory and streams; importing it
    # first makes the library bind to that same runtime instance (same SONAME).
    import torch  # noqa: F401
    _lib = ctypes.CDLL(LIB_PATH)
    _declare(_lib)
    return _lib


class CvMatrixDesc(ctypes.Structure):
    _fields_ = [("rowCount", ctypes.c_uint32), ("colCount", ctypes.c_uint32),
                ("componentType", ctypes.c_int32), ("layout", ctypes.c_int32),
                ("size", ctypes.c_size_t), ("offset", ctypes.c_size_t),
                ("rowColumnStride", ctypes.c_size_t)]


class CvCombination(ctypes.Structure):
    _fields_ = [("inputType", ctypes.c_int32), ("inputInterpretation", ctypes.c_int32),
                ("inputPackingFactor", ctypes.c_uint32), ("matrixInterpretation", ctypes.c_int32),
                ("biasInterpretation", ctypes.c_int32), ("resultType", ctypes.c_int32),
                ("transpose", ctypes.c_int32)]


class CvMatMulDesc(ctypes.Structure):
    _fields_ = [("input", ctypes.c_void_p), ("inputStride", ctypes.c_size_t),
                ("inputType", ctypes.c_int32), ("inputInterpretation", ctypes.c_int32),
                ("k", ctypes.c_int32),
                ("output", ctypes.c_void_p), ("outputStride", ctypes.c_size_t),
                ("resultType", ctypes.c_int32), ("m", ctypes.c_int32),
                ("matrix", ctypes.c_void_p), ("matrixOffset", ctypes.c_size_t),
                ("matrixInterpretation", ctypes.c_int32), ("layout", ctypes.c_int32),
                ("transpose", ctypes.c_int32), ("matrixStride", ctypes.c_uint32),
                ("bias", ctypes.c_void_p), ("biasOffset", ctypes.c_size_t),
                ("biasInterpretation", ctypes.c_int32),
                ("activation", ctypes.c_int32), ("leakySlope", ctypes.c_float),
                ("accumulate", ctypes.c_int32), ("batch", ctypes.c_uint32), ("flags", ctypes.c_uint32)]


class CvMlpLayer(ctypes.Structure):
    _fields_ = [("weights", ctypes.c_void_p), ("weightsGrad", ctypes.c_void_p),
                ("biases", ctypes.c_void_p), ("biasesGrad", ctypes.c_void_p),
                ("inputSize", ctypes.c_int32), ("outputSize", ctypes.c_int32),
                ("weightLayout", ctypes.c_int32), ("weightStride", ctypes.c_uint32),
                ("gradLayout", ctypes.c_int32), ("gradStride", ctypes.c_uint32),
                ("activation", ctypes.c_int32), ("leakySlope", ctypes.c_float)]


class CvMlpDesc(ctypes.Structure):
    _fields_ = [("layers", ctypes.POINTER(CvMlpLayer)), ("numLayers", ctypes.c_int32),
                ("inputType", ctypes.c_int32), ("weightType", ctypes.c_int32),
                ("biasType", ctypes.c_int32), ("outputType", ctypes.c_int32),
                ("gradType", ctypes.c_int32), ("flags", ctypes.c_uint32), ("inputEncoding", ctypes.c_int32),
                ("lossMax", ctypes.c_void_p)]


PERMUTO_MAX_DIMS, PERMUTO_MAX_LEVELS = 8, 16


class CvPermutoLevelInfo(ctypes.Structure):
    _fields_ = [("currentLevelIndex", ctypes.c_uint32), ("offsetOfFeatureTable", ctypes.c_uint32),
                ("featureTableSize", ctypes.c_uint32), ("scale", ctypes.c_float),
                ("scalesPerDim", ctypes.c_float * PERMUTO_MAX_DIMS), ("shiftsPerDim", ctypes.c_float * PERMUTO_MAX_DIMS)]


class CvPermutoDesc(ctypes.Structure):
    _fields_ = [("dimensions", ctypes.c_int32), ("featureDimensionPerEntry", ctypes.c_int32),
                ("log2HashmapSize", ctypes.c_uint32), ("maxLevels", ctypes.c_uint32),
                ("elementType", ctypes.c_int32), ("maxLevel", ctypes.c_float),
                ("levelInfo", CvPermutoLevelInfo * PERMUTO_MAX_LEVELS)]


NEURAL_MAX_LAYERS = 64


class CvNeuralNetworkDesc(ctypes.Structure):
    _fields_ = [("layerCount", ctypes.c_int32), ("dims", ctypes.c_int32 * (NEURAL_MAX_LAYERS + 1)),
                ("biasMask", ctypes.c_uint64), ("elementType", ctypes.c_int32), ("order", ctypes.c_int32)]


# name -> (restype, argtypes); every function include/coopvec.h declares
SIGNATURES = {
    "cvGetVersion": (ctypes.c_uint32, []),
    "cvGetLastErrorMessage": (ctypes.c_char_p, []),
    "cvGetLastKernelName": (ctypes.c_char_p, []),
    "cvComponentPackingFactor": (ctypes.c_int32, [ctypes.c_int32]),
    "cvComponentScalarType": (ctypes.c_int32, [ctypes.c_int32]),
    "cvComponentTypeStride": (ctypes.c_int32, [ctypes.c_int32]),
    "cvComponentTypeFromRhi": (ctypes.c_int32, [ctypes.c_int32]),
    "cvComponentTypeToRhi": (ctypes.c_int32, [ctypes.c_int32]),
    "cvQuerySupportedCombinations": (ctypes.c_uint32, [ctypes.POINTER(CvCombination), ctypes.c_uint32]),
    "cvGetMatrixSize": (ctypes.c_int32, [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_int32, ctypes.c_int32,
                                         ctypes.c_size_t, ctypes.POINTER(ctypes.c_size_t)]),
    "cvConvertMatrices": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_void_p, ctypes.POINTER(CvMatrixDesc),
                                           ctypes.c_void_p, ctypes.POINTER(CvMatrixDesc), ctypes.c_uint32]),
    "cvMatMul": (ctypes.c_int32, [ctypes.c_void_p, ctypes.POINTER(CvMatMulDesc)]),
    "cvOuterProductAccumulateWorkspaceSize": (ctypes.c_int32, [ctypes.c_int32, ctypes.c_int32, ctypes.c_uint32,
                                                               ctypes.POINTER(ctypes.c_size_t)]),
    "cvOuterProductAccumulate": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int32,
                                                  ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int32, ctypes.c_int32,
                                                  ctypes.c_uint32, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint32,
                                                  ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_size_t]),
    "cvReduceSumAccumulateWorkspaceSize": (ctypes.c_int32, [ctypes.c_int32, ctypes.c_uint32,
                                                            ctypes.POINTER(ctypes.c_size_t)]),
    "cvReduceSumAccumulate": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int32,
                                               ctypes.c_int32, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_size_t,
                                               ctypes.c_int32, ctypes.c_void_p, ctypes.c_size_t]),
    "cvElementwise": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_uint32,
                                       ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_size_t,
                                       ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float]),
    "cvVectorCast": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_int32, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_size_t,
                                      ctypes.c_int32, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int32]),
    "cvElementwiseBackward": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_uint32,
                                               ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_size_t,
                                               ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_size_t,
                                               ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_size_t,
                                               ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float]),
    "cvGridHash": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_size_t,
                                    ctypes.c_void_p, ctypes.c_uint32]),
    "cvPermutoPrepareLevels": (ctypes.c_int32, [ctypes.POINTER(CvPermutoDesc), ctypes.c_float, ctypes.c_float, ctypes.c_float,
                                                ctypes.c_uint32]),
    "cvPermutoEncode": (ctypes.c_int32, [ctypes.c_void_p, ctypes.POINTER(CvPermutoDesc), ctypes.c_void_p, ctypes.c_size_t,
                                         ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint32]),
    "cvPermutoMlpForward": (ctypes.c_int32, [ctypes.c_void_p, ctypes.POINTER(CvPermutoDesc), ctypes.c_void_p, ctypes.c_size_t,
                                             ctypes.c_void_p, ctypes.POINTER(CvMlpDesc), ctypes.c_void_p, ctypes.c_size_t,
                                             ctypes.c_uint32]),
    "cvPermutoEncodeBackward": (ctypes.c_int32, [ctypes.c_void_p, ctypes.POINTER(CvPermutoDesc), ctypes.c_void_p, ctypes.c_size_t,
                                                 ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p,
                                                 ctypes.c_size_t, ctypes.c_void_p, ctypes.c_uint32]),
    "cvNeuralNetworkSize": (ctypes.c_int32, [ctypes.POINTER(CvNeuralNetworkDesc), ctypes.POINTER(ctypes.c_size_t),
                                             ctypes.POINTER(ctypes.c_size_t)]),
    "cvNeuralToOptimalLayout": (ctypes.c_int32, [ctypes.c_void_p, ctypes.POINTER(CvNeuralNetworkDesc), ctypes.c_void_p, ctypes.c_void_p]),
    "cvNeuralToPortableLayout": (ctypes.c_int32, [ctypes.c_void_p, ctypes.POINTER(CvNeuralNetworkDesc), ctypes.c_void_p, ctypes.c_void_p]),
    "cvNeuralMlpForward": (ctypes.c_int32, [ctypes.c_void_p, ctypes.POINTER(CvNeuralNetworkDesc), ctypes.c_int32, ctypes.c_void_p,
                                            ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_float), ctypes.c_void_p,
                                            ctypes.c_size_t, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint32]),
    "cvNeuralMlpTrainStepWorkspaceSize": (ctypes.c_int32, [ctypes.POINTER(CvNeuralNetworkDesc), ctypes.c_uint32,
                                                           ctypes.POINTER(ctypes.c_size_t)]),
    "cvNeuralMlpTrainStep": (ctypes.c_int32, [ctypes.c_void_p, ctypes.POINTER(CvNeuralNetworkDesc), ctypes.c_int32, ctypes.c_void_p,
                                              ctypes.c_void_p, ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_float),
                                              ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float,
                                              ctypes.c_uint32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]),
    "cvMlpForward": (ctypes.c_int32, [ctypes.c_void_p, ctypes.POINTER(CvMlpDesc), ctypes.c_void_p, ctypes.c_size_t,
                                      ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint32]),
    "cvMlpTrainStepWorkspaceSize": (ctypes.c_int32, [ctypes.POINTER(CvMlpDesc), ctypes.c_uint32,
                                                     ctypes.POINTER(ctypes.c_size_t)]),
    "cvMlpTrainStep": (ctypes.c_int32, [ctypes.c_void_p, ctypes.POINTER(CvMlpDesc), ctypes.c_void_p, ctypes.c_size_t,
                                        ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float, ctypes.c_uint32,
                                        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]),
    "cvMlpTrainStepNoAlloc": (ctypes.c_int32, [ctypes.c_void_p, ctypes.POINTER(CvMlpDesc), ctypes.c_void_p,
                                               ctypes.c_size_t, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float,
                                               ctypes.c_uint32, ctypes.c_void_p]),
    "cvAdamStep": (ctypes.c_int32, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint32,
                                    ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_float]),
    "cvMlpAdamStep": (ctypes.c_int32, [ctypes.c_void_p, ctypes.POINTER(CvMlpDesc), ctypes.POINTER(ctypes.c_void_p),
                                       ctypes.POINTER(ctypes.c_void_p), ctypes.c_float, ctypes.c_float, ctypes.c_float,
                                       ctypes.c_float]),
}


def _declare(lib: ctypes.CDLL) -> None:
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)   # AttributeError if the library lacks a declared symbol
        fn.restype = restype
        fn.argtypes = argtypes
