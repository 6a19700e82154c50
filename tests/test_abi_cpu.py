"""The C-ABI library without a GPU: it loads, exports every symbol include/coopvec.h declares,
answers the host-side queries and rejects bad arguments with SlangResult codes.  No kernel runs."""
import ctypes
import os
import re

import numpy as np
import pytest

import oracle_binding as ob

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

from slang_amd import _lib  # noqa: E402

pytestmark = pytest.mark.skipif(not os.path.exists(_lib.LIB_PATH),
                                reason="library not built (python -m slang_amd.build)")

OK, FAIL, E_NOTIMPL, E_INVALID, E_TOOSMALL, E_INTERNAL, E_NOTAVAIL = (
    0, -2147467259, -2147467263, -2147024809, -2113929215, -2113929210, -2113929209)


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def test_every_declared_symbol_is_exported(lib):
    header = open(os.path.join(REPO, "include", "coopvec.h")).read()
    declared = set(re.findall(r"CV_API\s+[\w\s\*]+?\b(cv\w+)\s*\(", header))
    assert len(declared) >= 15
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    for name in declared:
        assert hasattr(lib, name), name


def test_result_codes_match_slang(lib):
    header = open(os.path.join(REPO, "include", "coopvec.h")).read()
    vals = dict(re.findall(r"#define (CV_\w+)\s+\(\(CvResult\)(0x[0-9a-fA-F]+|0)\)", header))
    # include/slang.h:1400-1464: SLANG_MAKE_ERROR(fac, code) = 0x80000000 | fac<<16 | code
    def mk(fac, code):
        return 0x80000000 | (fac << 16) | code
    assert int(vals["CV_FAIL"], 16) == mk(0, 0x4005)
    assert int(vals["CV_E_NOT_IMPLEMENTED"], 16) == mk(0, 0x4001)
    assert int(vals["CV_E_INVALID_ARG"], 16) == mk(7, 0x57)
    assert int(vals["CV_E_BUFFER_TOO_SMALL"], 16) == mk(0x200, 1)
    assert int(vals["CV_E_INTERNAL_FAIL"], 16) == mk(0x200, 6)
    assert int(vals["CV_E_NOT_AVAILABLE"], 16) == mk(0x200, 7)


def test_type_tables_match_oracle(lib):
    O = ob.lib()
    for ct in range(15):
        assert lib.cvComponentPackingFactor(ct) == O.cvo_component_packing_factor(ct)
        assert lib.cvComponentScalarType(ct) == O.cvo_component_scalar_type(ct)
    # storage size: same as the fallback's stride table where that has a case; fp8 = 1 byte
    for ct in range(2, 15):
        assert lib.cvComponentTypeStride(ct) == O.cvo_component_type_stride(ct)
    assert lib.cvComponentTypeStride(0) == 1 and lib.cvComponentTypeStride(1) == 1
    assert lib.cvComponentTypeStride(99) == -1


@pytest.mark.parametrize("rows,cols", [(4, 4), (16, 4), (4, 16), (64, 64), (128, 128), (13, 5), (33, 17), (1, 64), (64, 8)])
def test_matrix_size_matches_oracle(lib, rows, cols):
    O = ob.lib()
    for ct in (ob.F16, ob.S8, ob.E4M3, ob.F32):
        for layout in range(4):
            out = ctypes.c_size_t(0)
            rc = lib.cvGetMatrixSize(rows, cols, ct, layout, 0, ctypes.byref(out))
            want = O.cvo_layout_matrix_size(rows, cols, ct, layout, 0)
            if want == 0:
                assert rc < 0
            else:
                assert rc == OK and out.value == want
                if layout >= 2:
                    assert out.value % 64 == 0
    out = ctypes.c_size_t(0)
    assert lib.cvGetMatrixSize(rows, cols, ob.F16, 0, cols * 2 + 64, ctypes.byref(out)) == OK
    assert out.value == (rows - 1) * (cols * 2 + 64) + cols * 2


def test_example_allocation_arithmetic(lib):
    # the example's buffer plan (mlp-training-coopvec.cpp:265-315) for 4 -> 16 -> 4:
    # every sub-allocation is rounded up to 64 bytes
    sizes = [4, 16, 4]
    off = 0
    def alloc(n):
        nonlocal off
        o = off; off += (n + 63) // 64 * 64; return o
    for i in range(2):
        alloc(sizes[i] * sizes[i + 1] * 2); alloc(sizes[i + 1] * 2)
    assert off == 128 + 64 + 128 + 64
    grad_off = off
    for i in range(2):
        alloc(sizes[i] * sizes[i + 1] * 2); alloc(sizes[i + 1] * 2)
    train_off = off
    for i in range(2):
        out = ctypes.c_size_t(0)
        assert lib.cvGetMatrixSize(sizes[i + 1], sizes[i], ob.F16, ob.TRAIN_OPT, 0, ctypes.byref(out)) == OK
        assert out.value == 512          # one 16x16 fp16 tile
        assert alloc(out.value) % 64 == 0
    assert (grad_off, train_off, off) == (384, 768, 1792)


def test_get_matrix_size_errors(lib):
    out = ctypes.c_size_t(7)
    assert lib.cvGetMatrixSize(4, 4, ob.F16, 0, 0, None) == E_INVALID
    assert lib.cvGetMatrixSize(0, 4, ob.F16, 0, 0, ctypes.byref(out)) == E_INVALID and out.value == 0
    assert lib.cvGetMatrixSize(4, 4, ob.F16, 7, 0, ctypes.byref(out)) == E_INVALID
    assert lib.cvGetMatrixSize(4, 4, ob.S8P, 0, 0, ctypes.byref(out)) == E_NOTAVAIL
    assert lib.cvGetMatrixSize(4, 4, ob.S8, ob.TRAIN_OPT, 0, ctypes.byref(out)) == E_NOTAVAIL
    assert lib.cvGetMatrixSize(4, 4, ob.F16, 0, 2, ctypes.byref(out)) == E_INVALID   # stride < row
    assert b"stride" in lib.cvGetLastErrorMessage()


def test_supported_combinations(lib):
    n = lib.cvQuerySupportedCombinations(None, 0)
    arr = (_lib.CvCombination * n)()
    assert lib.cvQuerySupportedCombinations(arr, n) == n
    combos = {(c.inputType, c.inputInterpretation, c.inputPackingFactor, c.matrixInterpretation,
               c.biasInterpretation, c.resultType) for c in arr}
    assert (ob.F16, ob.F16, 1, ob.F16, ob.F16, ob.F16) in combos
    assert (ob.U32, ob.S8P, 4, ob.S8, ob.S32, ob.S32) in combos     # packed int8, as in
    # tools/slang-unit-test/unit-test-cooperative-type-metadata.cpp:667-701 (inputPackingFactor 4)
    assert (ob.E4M3, ob.E4M3, 1, ob.E4M3, ob.F16, ob.F16) in combos
    # combinations without a matrix instruction run as the scalar definition
    assert (ob.S16, ob.S16, 1, ob.S32, ob.S32, ob.S32) in combos
    assert (ob.F32, ob.F32, 1, ob.S8, ob.F16, ob.F32) in combos
    assert (ob.F64, ob.F64, 1, ob.S64, ob.U64, ob.F64) in combos
    assert (ob.BF16, ob.BF16, 1, ob.F16, ob.F16, ob.F16) not in combos
    # packed bytes against any plain matrix type; a plain interpretation the scalar definition ignores is
    # accepted by cvMatMul and listed once, under the stored type
    assert (ob.U32, ob.S8P, 4, ob.F16, ob.F16, ob.F32) in combos
    assert (ob.S32, ob.U8P, 4, ob.S16, ob.S32, ob.S64) in combos
    assert (ob.F32, ob.F16, 1, ob.S16, ob.F32, ob.F32) not in combos


def _desc(**kw):
    d = _lib.CvMatMulDesc()
    base = dict(input=0x1000, inputStride=128, inputType=ob.F16, inputInterpretation=ob.F16, k=64,
                output=0x2000, outputStride=128, resultType=ob.F16, m=64, matrix=0x3000, matrixOffset=0,
                matrixInterpretation=ob.F16, layout=0, transpose=0, matrixStride=128, bias=None, biasOffset=0,
                biasInterpretation=-1, activation=0, leakySlope=0.0, accumulate=0, batch=16)
    base.update(kw)
    for k, v in base.items():
        setattr(d, k, v)
    return d


def test_matmul_argument_validation(lib):
    f = lambda **kw: lib.cvMatMul(None, ctypes.byref(_desc(**kw)))
    assert lib.cvMatMul(None, None) == E_INVALID
    assert f(batch=0) == OK                                   # empty batch: nothing to do
    assert f(input=None) == E_INVALID
    assert f(matrix=None) == E_INVALID
    assert f(m=0) == E_INVALID and f(k=-1) == E_INVALID
    assert f(layout=5) == E_INVALID
    assert f(matrixInterpretation=ob.S8P) == E_INVALID        # static_assert hlsl.meta.slang:32803
    assert f(bias=0x4000, biasInterpretation=ob.U8P) == E_INVALID   # :33004
    assert f(transpose=1) == E_INVALID                        # RowMajor + transpose, :32947
    assert f(accumulate=1, activation=1) == E_INVALID
    assert f(activation=9) == E_INVALID
    assert f(inputType=ob.BF16, inputInterpretation=ob.BF16) == E_NOTAVAIL     # bfloat16 only with a bfloat16 matrix
    assert f(matrixInterpretation=ob.E5M2, matrixStride=64) == E_NOTAVAIL      # 8-bit floats only with their own vectors
    assert f(inputType=ob.F32, inputInterpretation=ob.S8P, inputStride=256) == E_NOTAVAIL   # packed bytes live in 32-bit integers
    assert b"unsupported combination" in lib.cvGetLastErrorMessage()
    assert f(inputType=ob.F16, inputInterpretation=ob.E5M2) == E_NOTAVAIL      # fp16 vectors quantise to e4m3 only
    assert b"unsupported combination" in lib.cvGetLastErrorMessage()
    assert f(matrixInterpretation=ob.E4M3, matrixStride=64, inputType=ob.F32, inputInterpretation=ob.F32,
             inputStride=256) == E_NOTAVAIL                                    # 8-bit floats only with their own vectors
    assert f(matrixInterpretation=ob.S16, layout=2) == E_NOTAVAIL              # no Optimal layout for 16-bit integers
    assert f(matrixInterpretation=ob.S16, resultType=ob.S32, outputStride=256, activation=2) == E_NOTAVAIL   # leaky ReLU on integers
    assert f(inputType=ob.U32, inputInterpretation=ob.S8P, matrixInterpretation=ob.S8, resultType=ob.S32,
             k=6) == E_NOTAVAIL                               # packed needs k == 4*PackedK (:32846)
    assert f(input=0x1001) == E_INVALID                       # misaligned vector
    assert f(inputStride=64) == E_INVALID                     # stride smaller than the vector
    assert f(matrixStride=64) == E_INVALID                    # stride smaller than a row
    assert f(matrix=0x3002, layout=2) == E_INVALID            # Optimal layouts need 16-byte alignment
    assert f(m=4096) == E_NOTAVAIL or f(m=4096) == E_INVALID  # beyond the kernel table / stride
    assert b"cvMatMul" in lib.cvGetLastErrorMessage()


def test_convert_argument_validation(lib):
    D = _lib.CvMatrixDesc
    src = (D * 1)(D(4, 8, ob.F16, ob.ROW, 64, 0, 16))
    dst = (D * 1)(D(4, 8, ob.F16, ob.TRAIN_OPT, 512, 1024, 0))
    f = lambda s=src, d=dst, n=1, sb=0x10000, db=0x10000: lib.cvConvertMatrices(None, db, d, sb, s, n)
    assert f(n=0) == OK
    assert f(sb=None) == E_INVALID
    assert f(d=(D * 1)(D(4, 9, ob.F16, ob.TRAIN_OPT, 512, 1024, 0))) == E_INVALID      # shape mismatch
    assert f(d=(D * 1)(D(4, 8, ob.F16, ob.TRAIN_OPT, 256, 1024, 0))) == E_TOOSMALL      # dst size too small
    assert f(s=(D * 1)(D(4, 8, ob.F16, ob.ROW, 32, 0, 16))) == E_TOOSMALL               # src size too small
    assert f(d=(D * 1)(D(4, 8, ob.S8, ob.ROW, 512, 1024, 0))) == E_NOTAVAIL             # fp16 -> int8
    assert f(d=(D * 1)(D(4, 8, ob.S8, ob.TRAIN_OPT, 512, 1024, 0))) == E_NOTAVAIL       # no such layout
    assert f(d=(D * 1)(D(4, 8, ob.F16, ob.TRAIN_OPT, 512, 32, 0))) == E_INVALID         # ranges overlap
    assert f(n=65) == E_INVALID


def test_library_missing_is_loud(monkeypatch, tmp_path):
    import importlib
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    monkeypatch.setattr(_lib, "_lib", None)
    with pytest.raises(ImportError):
        _lib.load()


def test_rhi_component_type_numbering(lib):
    # rhi::CooperativeVectorComponentType (include/slang-gfx.h:1748-1765), the values the example's host
    # code passes (mlp-training-coopvec.cpp:212,220,308), against the shader-side enum this ABI takes
    rhi_names = ["Float16", "Float32", "Float64", "SInt8", "SInt16", "SInt32", "SInt64", "UInt8", "UInt16",
                 "UInt32", "UInt64", "SInt8Packed", "UInt8Packed", "FloatE4M3", "FloatE5M2"]
    slang_names = {"Float16": "Float16", "Float32": "Float32", "Float64": "Float64", "SInt8": "SignedInt8",
                   "SInt16": "SignedInt16", "SInt32": "SignedInt32", "SInt64": "SignedInt64", "UInt8": "UnsignedInt8",
                   "UInt16": "UnsignedInt16", "UInt32": "UnsignedInt32", "UInt64": "UnsignedInt64",
                   "SInt8Packed": "SignedInt8Packed", "UInt8Packed": "UnsignedInt8Packed",
                   "FloatE4M3": "FloatE4M3", "FloatE5M2": "FloatE5M2"}
    from slang_amd.coopvec import CoopVecComponentType, RhiCooperativeVectorComponentType
    for value, name in enumerate(rhi_names):
        assert RhiCooperativeVectorComponentType[name] == value
        want = CoopVecComponentType[slang_names[name]]
        assert lib.cvComponentTypeFromRhi(value) == want
        assert lib.cvComponentTypeToRhi(int(want)) == value
    assert lib.cvComponentTypeFromRhi(15) == -1 and lib.cvComponentTypeFromRhi(-1) == -1
    assert lib.cvComponentTypeToRhi(15) == -1
    # the example's size query: rhi Float16 (0) must give the fp16 size, not the e4m3 size that the
    # raw value 0 means on this ABI
    fp16, raw0 = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert lib.cvGetMatrixSize(16, 4, lib.cvComponentTypeFromRhi(0), 0, 0, ctypes.byref(fp16)) == OK
    assert lib.cvGetMatrixSize(16, 4, 0, 0, 0, ctypes.byref(raw0)) == OK
    assert fp16.value == 16 * 4 * 2 and raw0.value == 16 * 4


def test_bench_traffic_figures_come_from_the_profile_summaries():
    # bench.py quotes `roofline.traffic` from lines `traffic[<workload>] = <bytes> B per step` of profiles/*.md:
    # every workload of the default run that has a summary must be found there, with a plausible figure
    import importlib.util
    import os
    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(repo, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    traffic = bench.profiled_traffic()
    for key in ("c1", "c2", "c2b", "c3", "c4", "c4h", "c4n", "c5", "op", "rs", "copy"):
        assert key in traffic, "no traffic[%s] line in profiles/" % key
        nbytes, path = traffic[key]
        assert nbytes > 100000 and os.path.exists(os.path.join(repo, path))
    assert set(bench.DEFAULT_RUN) <= set(bench.WORKLOADS) and bench.HEADLINE in bench.WORKLOADS
