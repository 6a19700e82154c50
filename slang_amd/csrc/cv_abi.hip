// cv_abi.hip -- the extern "C" entry points declared in include/coopvec.h: argument
// validation, specialisation lookup and kernel launches.  No device memory is allocated here.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <vector>

#include "../../include/coopvec.h"
#include "cv_error.h"
#include "cv_kernels.h"

namespace {

thread_local char tlsError[512] = "";
thread_local char tlsKernel[256] = "";

CvResult fail(CvResult code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(tlsError, sizeof(tlsError), fmt, ap);
    va_end(ap);
    return code;
}

CvResult fromHip(hipError_t e, const char* what)
{
    if (e == hipSuccess) return CV_OK;
    return fail(CV_E_INTERNAL_FAIL, "%s: %s", what, hipGetErrorString(e));
}

// number of compute units of the current device (cached; immutable once read)
int currentDeviceCUs(CvResult* rc)
{
    static int cus[64];
    static std::once_flag once[64];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= 64) {
        *rc = fail(CV_E_NOT_AVAILABLE, "no usable HIP device: %s", hipGetErrorString(e));
        return 0;
    }
    std::call_once(once[dev], [dev] {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cus[dev] = n;
    });
    *rc = CV_OK;
    return cus[dev];
}

uint32_t alignOf(const void* p, size_t stride)
{
    uintptr_t v = (uintptr_t)p | (uintptr_t)stride | 16u;
    return (uint32_t)(v & (~v + 1));
}

// Scratch of cvMlpTrainStepNoAlloc: the per-workgroup gradient partials of the training step.  Every
// device the library runs on holds its own copy of this array at its own address; on the host the
// array's name is only a handle for hipGetSymbolAddress, never a device address.
static __device__ __align__(256) unsigned char scratch[CV_NOALLOC_SCRATCH_BYTES];

// Device address of `scratch` on the current device, looked up once per device.
void* scratchOfCurrentDevice(CvResult* rc)
{
    static void* ptr[64];
    static hipError_t err[64];
    static std::once_flag once[64];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= 64) {
        *rc = fail(CV_E_NOT_AVAILABLE, "no usable HIP device: %s", hipGetErrorString(e));
        return nullptr;
    }
    std::call_once(once[dev], [dev] {
        void* p = nullptr;
        err[dev] = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        ptr[dev] = err[dev] == hipSuccess ? p : nullptr;
    });
    if (err[dev] != hipSuccess || !ptr[dev]) {
        *rc = fail(CV_E_INTERNAL_FAIL, "address of the built-in scratch array on device %d: %s", dev, hipGetErrorString(err[dev]));
        return nullptr;
    }
    *rc = CV_OK;
    return ptr[dev];
}

bool isOptimal(int layout) { return layout == CV_LAYOUT_INFERENCING_OPTIMAL || layout == CV_LAYOUT_TRAINING_OPTIMAL; }

// What the matMul kernels implement: the matrix-core flavour that serves a combination of
// (type of the vectors in memory, inputInterpretation, matrixInterpretation, biasInterpretation or
// CV_COMPONENT_NONE, resultType), or false.  The table of cvQuerySupportedCombinations is this
// predicate evaluated over every combination, so the two cannot disagree (one exception, stated where the
// table is built: combinations that differ only by an interpretation the scalar definition ignores).
struct ComboKind {
    cv::MmaKind kind;
    bool inUnsigned, matUnsigned;
};

// combinations served by a matrix instruction
bool classifyMfmaCombo(int32_t inType, int32_t inInterp, int32_t matInterp, int32_t biasInterp, int32_t resType, ComboKind* out)
{
    const bool noBias = biasInterp == CV_COMPONENT_NONE;
    ComboKind k{cv::MmaKind::F16, false, false};
    const bool f16f32Res = resType == CV_FLOAT16 || resType == CV_FLOAT32;
    if (matInterp == CV_FLOAT16) {
        if (inType != CV_FLOAT16 || inInterp != CV_FLOAT16 || !f16f32Res) return false;
        if (!noBias && biasInterp != CV_FLOAT16 && biasInterp != CV_FLOAT32) return false;
        k.kind = cv::MmaKind::F16;
    } else if (matInterp == CV_FLOAT_E4M3) {
        if (inInterp != CV_FLOAT_E4M3 || !f16f32Res || (!noBias && biasInterp != CV_FLOAT16)) return false;
        if (inType == CV_FLOAT_E4M3) k.kind = cv::MmaKind::Fp8AsF16;
        else if (inType == CV_FLOAT16) k.kind = cv::MmaKind::F16VecAsE4M3;   // CoopVec<half> + interpretation
        else return false;
    } else if (matInterp == CV_FLOAT_E5M2) {
        if (inType != CV_FLOAT_E5M2 || inInterp != CV_FLOAT_E5M2 || !f16f32Res || (!noBias && biasInterp != CV_FLOAT16)) return false;
        k.kind = cv::MmaKind::Bf8AsF16;
    } else if (matInterp == CV_BFLOAT16) {
        if (inType != CV_BFLOAT16 || inInterp != CV_BFLOAT16) return false;
        if (resType != CV_BFLOAT16 && resType != CV_FLOAT32) return false;
        if (!noBias && biasInterp != CV_BFLOAT16 && biasInterp != CV_FLOAT32) return false;
        k.kind = cv::MmaKind::Bf16;
    } else if (matInterp == CV_FLOAT32) {
        // the all-fp32 form: CoopVec<float> with a Float32 matrix (hlsl.meta.slang:32870-32872)
        if (inType != CV_FLOAT32 || inInterp != CV_FLOAT32 || resType != CV_FLOAT32) return false;
        if (!noBias && biasInterp != CV_FLOAT32) return false;
        k.kind = cv::MmaKind::F32;
    } else if (matInterp == CV_SINT8 || matInterp == CV_UINT8) {
        if (resType != CV_SINT32 && resType != CV_UINT32) return false;
        if (!noBias && biasInterp != CV_SINT32 && biasInterp != CV_UINT32) return false;
        if (inInterp == CV_SINT8_PACKED || inInterp == CV_UINT8_PACKED) {
            // four bytes per 32-bit element; the reference's unpacking sign-extends for both packed
            // kinds (hlsl.meta.slang:32850-32855)
            if (inType != CV_UINT32 && inType != CV_SINT32) return false;
        } else if (inInterp == CV_SINT8 || inInterp == CV_UINT8) {
            if (inType != inInterp) return false;
            k.inUnsigned = inType == CV_UINT8;
        } else {
            return false;
        }
        k.matUnsigned = matInterp == CV_UINT8;
        k.kind = (k.inUnsigned || k.matUnsigned) ? cv::MmaKind::I8AnySign : cv::MmaKind::I8;
    } else {
        return false;
    }
    if (out) *out = k;
    return true;
}

// The scalar types the fallback's switch covers (hlsl.meta.slang:32866-32907).
bool isPlainScalar(int32_t ct)
{
    return ct == CV_FLOAT16 || ct == CV_FLOAT32 || ct == CV_FLOAT64 || ct == CV_SINT8 || ct == CV_UINT8 || ct == CV_SINT16 ||
           ct == CV_UINT16 || ct == CV_SINT32 || ct == CV_UINT32 || ct == CV_SINT64 || ct == CV_UINT64;
}

// Every combination of those types runs somewhere: on a matrix instruction where one exists, else as the
// scalar definition (cv_matmul_scalar.hip), results half / float / double / int32 / uint32 / int64 / uint64.
// The scalar definition casts the vector's elements, as they are stored, to the result type and never looks at
// a plain inputInterpretation (hlsl.meta.slang:32839-32843), so a plain interpretation other than the stored
// type changes nothing there; packed interpretations unpack four sign-extended bytes from each 32-bit element
// (:32844-32856) and go with every plain matrix type.
bool classifyCombo(int32_t inType, int32_t inInterp, int32_t matInterp, int32_t biasInterp, int32_t resType, ComboKind* out)
{
    if (classifyMfmaCombo(inType, inInterp, matInterp, biasInterp, resType, out)) return true;
    const bool resOk = resType == CV_FLOAT16 || resType == CV_FLOAT32 || resType == CV_FLOAT64 || resType == CV_SINT32 ||
                       resType == CV_UINT32 || resType == CV_SINT64 || resType == CV_UINT64;
    const bool packedIn = inInterp == CV_SINT8_PACKED || inInterp == CV_UINT8_PACKED;
    const bool inOk = packedIn ? (inType == CV_UINT32 || inType == CV_SINT32) : (isPlainScalar(inType) && isPlainScalar(inInterp));
    if (!inOk || !isPlainScalar(matInterp) || !resOk) return false;
    if (biasInterp != CV_COMPONENT_NONE && !isPlainScalar(biasInterp)) return false;
    if (out) *out = ComboKind{cv::MmaKind::Scalar, false, false};
    return true;
}

constexpr int32_t kNumComponentTypes = 16;   // CV_FLOAT_E4M3 .. CV_BFLOAT16

// every supported combination that carries a bias (each also covers the bias-less coopVecMatMul)
const std::vector<CvCombination>& comboTable()
{
    static std::vector<CvCombination> table;
    static std::once_flag once;
    std::call_once(once, [] {
        for (int32_t mat = 0; mat < kNumComponentTypes; ++mat)
            for (int32_t in = 0; in < kNumComponentTypes; ++in)
                for (int32_t interp = 0; interp < kNumComponentTypes; ++interp)
                    for (int32_t bias = 0; bias < kNumComponentTypes; ++bias)
                        for (int32_t res = 0; res < kNumComponentTypes; ++res) {
                            ComboKind kind;
                            if (!classifyCombo(in, interp, mat, bias, res, &kind)) continue;
                            // the scalar definition ignores a plain interpretation: the table lists each of
                            // those combinations once, under the stored type
                            if (kind.kind == cv::MmaKind::Scalar && interp != in && cvComponentPackingFactor(interp) == 1) continue;
                            CvCombination c;
                            c.inputType = in; c.inputInterpretation = interp;
                            c.inputPackingFactor = (uint32_t)cvComponentPackingFactor(interp);
                            c.matrixInterpretation = mat; c.biasInterpretation = bias; c.resultType = res;
                            c.transpose = 0;
                            table.push_back(c);
                        }
    });
    return table;
}

} // namespace

namespace cv {
CvResult failWith(CvResult code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(tlsError, sizeof(tlsError), fmt, ap);
    va_end(ap);
    return code;
}
void noteKernel(bool append, const char* fmt, ...)
{
    size_t at = 0;
    if (append) {
        at = strlen(tlsKernel);
        if (at + 4 < sizeof(tlsKernel)) { memcpy(tlsKernel + at, " + ", 4); at += 3; }
    }
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(tlsKernel + at, sizeof(tlsKernel) - at, fmt, ap);
    va_end(ap);
}
} // namespace cv

extern "C" {

CV_API const char* cvGetLastKernelName(void) { return tlsKernel; }

CV_API uint32_t cvGetVersion(void) { return (1u << 16) | 0u; }

CV_API const char* cvGetLastErrorMessage(void) { return tlsError; }

CV_API int32_t cvComponentPackingFactor(int32_t ct)
{
    return (ct == CV_SINT8_PACKED || ct == CV_UINT8_PACKED) ? 4 : 1;
}

CV_API int32_t cvComponentScalarType(int32_t ct)
{
    switch (ct) {   // SLANG_SCALAR_TYPE_* values, include/slang.h:2139-2157
    case CV_FLOAT_E4M3: return 17;
    case CV_FLOAT_E5M2: return 18;
    case CV_FLOAT16: return 7;
    case CV_FLOAT32: return 8;
    case CV_FLOAT64: return 9;
    case CV_SINT8: case CV_SINT8_PACKED: return 10;
    case CV_SINT16: return 12;
    case CV_SINT32: return 3;
    case CV_SINT64: return 5;
    case CV_UINT8: case CV_UINT8_PACKED: return 11;
    case CV_UINT16: return 13;
    case CV_UINT32: return 4;
    case CV_UINT64: return 6;
    case CV_BFLOAT16: return 16;
    }
    return -1;
}

CV_API int32_t cvComponentTypeStride(int32_t ct)
{
    const uint32_t s = cv::elemSize(ct);
    return s ? (int32_t)s : -1;
}

// rhi::CooperativeVectorComponentType (include/slang-gfx.h:1748-1765), indexed by its value
static const int32_t kRhiToCv[15] = {
    CV_FLOAT16, CV_FLOAT32, CV_FLOAT64, CV_SINT8, CV_SINT16, CV_SINT32, CV_SINT64,
    CV_UINT8, CV_UINT16, CV_UINT32, CV_UINT64, CV_SINT8_PACKED, CV_UINT8_PACKED, CV_FLOAT_E4M3, CV_FLOAT_E5M2,
};

CV_API int32_t cvComponentTypeFromRhi(int32_t rhi)
{
    return (rhi >= 0 && rhi < 15) ? kRhiToCv[rhi] : (int32_t)CV_COMPONENT_NONE;
}

CV_API int32_t cvComponentTypeToRhi(int32_t ct)
{
    for (int32_t i = 0; i < 15; ++i)
        if (kRhiToCv[i] == ct) return i;
    return -1;
}

CV_API uint32_t cvQuerySupportedCombinations(CvCombination* out, uint32_t capacity)
{
    const std::vector<CvCombination>& table = comboTable();
    for (size_t i = 0; i < table.size() && out && i < capacity; ++i) out[i] = table[i];
    return (uint32_t)table.size();
}

CV_API CvResult cvGetMatrixSize(uint32_t rowCount, uint32_t colCount, int32_t componentType,
                                int32_t layout, size_t rowColumnStride, size_t* outSize)
{
    if (!outSize) return fail(CV_E_INVALID_ARG, "cvGetMatrixSize: outSize is null");
    *outSize = 0;
    if (rowCount == 0 || colCount == 0) return fail(CV_E_INVALID_ARG, "cvGetMatrixSize: empty matrix %ux%u", rowCount, colCount);
    if (layout < 0 || layout > 3) return fail(CV_E_INVALID_ARG, "cvGetMatrixSize: unknown layout %d", layout);
    if (!cv::layoutSupports(componentType, layout))
        return fail(CV_E_NOT_AVAILABLE, "cvGetMatrixSize: component type %d has no layout %d", componentType, layout);
    const cv::MatrixShape s{rowCount, colCount, componentType, layout, isOptimal(layout) ? 0 : rowColumnStride};
    const size_t n = cv::matrixSize(s);
    if (!n) return fail(CV_E_INVALID_ARG, "cvGetMatrixSize: stride %zu is smaller than one row/column", rowColumnStride);
    *outSize = n;
    return CV_OK;
}

CV_API CvResult cvConvertMatrices(void* stream, void* dstBuffer, const CvMatrixDesc* dstDescs,
                                  const void* srcBuffer, const CvMatrixDesc* srcDescs, uint32_t count)
{
    if (count == 0) return CV_OK;
    if (!dstBuffer || !srcBuffer || !dstDescs || !srcDescs) return fail(CV_E_INVALID_ARG, "cvConvertMatrices: null argument");
    if (count > 64) return fail(CV_E_INVALID_ARG, "cvConvertMatrices: %u matrices in one call (limit 64)", count);
    for (uint32_t base = 0; base < count; base += cv::kMaxConvertItems) {
        cv::ConvertArgs args;
        args.count = (count - base < (uint32_t)cv::kMaxConvertItems) ? count - base : (uint32_t)cv::kMaxConvertItems;
        for (uint32_t i = 0; i < args.count; ++i) {
            const CvMatrixDesc& s = srcDescs[base + i];
            const CvMatrixDesc& d = dstDescs[base + i];
            if (s.rowCount != d.rowCount || s.colCount != d.colCount || s.rowCount == 0 || s.colCount == 0)
                return fail(CV_E_INVALID_ARG, "cvConvertMatrices[%u]: shapes differ or are empty (%ux%u -> %ux%u)",
                            base + i, s.rowCount, s.colCount, d.rowCount, d.colCount);
            if (!cv::layoutSupports(s.componentType, s.layout) || !cv::layoutSupports(d.componentType, d.layout))
                return fail(CV_E_NOT_AVAILABLE, "cvConvertMatrices[%u]: unsupported type/layout (%d,%d) -> (%d,%d)",
                            base + i, s.componentType, s.layout, d.componentType, d.layout);
            const bool f16f32 = (s.componentType == CV_FLOAT16 || s.componentType == CV_FLOAT32) &&
                                (d.componentType == CV_FLOAT16 || d.componentType == CV_FLOAT32);
            if (s.componentType != d.componentType && !f16f32)
                return fail(CV_E_NOT_AVAILABLE, "cvConvertMatrices[%u]: no conversion from component type %d to %d",
                            base + i, s.componentType, d.componentType);
            cv::ConvertItem& it = args.items[i];
            it.srcShape = cv::MatrixShape{s.rowCount, s.colCount, s.componentType, s.layout, isOptimal(s.layout) ? 0 : s.rowColumnStride};
            it.dstShape = cv::MatrixShape{d.rowCount, d.colCount, d.componentType, d.layout, isOptimal(d.layout) ? 0 : d.rowColumnStride};
            const size_t sNeed = cv::matrixSize(it.srcShape), dNeed = cv::matrixSize(it.dstShape);
            if (!sNeed || !dNeed) return fail(CV_E_INVALID_ARG, "cvConvertMatrices[%u]: stride smaller than a row/column", base + i);
            if (s.size < sNeed || d.size < dNeed)
                return fail(CV_E_BUFFER_TOO_SMALL, "cvConvertMatrices[%u]: desc.size too small (src %zu < %zu or dst %zu < %zu)",
                            base + i, s.size, sNeed, d.size, dNeed);
            const uint32_t esS = cv::elemSize(s.componentType), esD = cv::elemSize(d.componentType);
            if (s.offset % esS || d.offset % esD || s.rowColumnStride % esS || d.rowColumnStride % esD)
                return fail(CV_E_INVALID_ARG, "cvConvertMatrices[%u]: offset/stride not a multiple of the element size", base + i);
            if (dNeed > 0xffffffffull) return fail(CV_E_INVALID_ARG, "cvConvertMatrices[%u]: matrix too large", base + i);
            it.src = (const uint8_t*)srcBuffer + s.offset;
            it.dst = (uint8_t*)dstBuffer + d.offset;
            it.dstBytes = (uint32_t)dNeed;
            const uint8_t *s0 = it.src, *s1 = it.src + sNeed, *d0 = it.dst, *d1 = it.dst + dNeed;
            if (s0 < d1 && d0 < s1) return fail(CV_E_INVALID_ARG, "cvConvertMatrices[%u]: source and destination overlap", base + i);
        }
        CvResult rc = fromHip(cv::launchConvert((hipStream_t)stream, args), "cvConvertMatrices launch");
        if (CV_FAILED(rc)) return rc;
    }
    return CV_OK;
}

CV_API CvResult cvMatMul(void* stream, const CvMatMulDesc* d)
{
    if (!d) return fail(CV_E_INVALID_ARG, "cvMatMul: desc is null");
    if (d->batch == 0) return CV_OK;
    if (!d->input || !d->output || !d->matrix) return fail(CV_E_INVALID_ARG, "cvMatMul: null input/output/matrix");
    if (d->m <= 0 || d->k <= 0) return fail(CV_E_INVALID_ARG, "cvMatMul: m=%d k=%d", d->m, d->k);
    if (d->layout < 0 || d->layout > 3) return fail(CV_E_INVALID_ARG, "cvMatMul: unknown layout %d", d->layout);
    // static_asserts of the Slang signatures (hlsl.meta.slang:32798-32803, 33004)
    if (cvComponentPackingFactor(d->matrixInterpretation) != 1)
        return fail(CV_E_INVALID_ARG, "cvMatMul: can't use packed component type in matrixInterpretation");
    if (d->bias && cvComponentPackingFactor(d->biasInterpretation) != 1)
        return fail(CV_E_INVALID_ARG, "cvMatMul: can't use packed component type in biasInterpretation");
    if (d->transpose && !isOptimal(d->layout))   // hlsl.meta.slang:32947
        return fail(CV_E_INVALID_ARG, "cvMatMul: transpose must be false for RowMajor/ColumnMajor");
    if (d->accumulate && d->activation != CV_ACT_NONE)
        return fail(CV_E_INVALID_ARG, "cvMatMul: accumulate forms take no activation");
    if (d->activation < CV_ACT_NONE || d->activation > CV_ACT_QUICK_GELU)
        return fail(CV_E_INVALID_ARG, "cvMatMul: unknown activation %d", d->activation);
    const uint32_t packing = (uint32_t)cvComponentPackingFactor(d->inputInterpretation);
    if (packing != 1 && d->k % 4 != 0)   // fallback rule k == 4*PackedK (hlsl.meta.slang:32846)
        return fail(CV_E_NOT_AVAILABLE, "cvMatMul: packed input needs k to be a multiple of 4 (k=%d)", d->k);

    ComboKind combo;
    if (!classifyCombo(d->inputType, d->inputInterpretation, d->matrixInterpretation,
                       d->bias ? d->biasInterpretation : (int32_t)CV_COMPONENT_NONE, d->resultType, &combo))
        return fail(CV_E_NOT_AVAILABLE,
                    "cvMatMul: unsupported combination input %d as %d, matrix %d, bias %d, result %d",
                    d->inputType, d->inputInterpretation, d->matrixInterpretation,
                    d->bias ? d->biasInterpretation : -1, d->resultType);
    if (!cv::layoutSupports(d->matrixInterpretation, d->layout))
        return fail(CV_E_NOT_AVAILABLE, "cvMatMul: component type %d has no layout %d", d->matrixInterpretation, d->layout);

    cv::MatMulArgs a;
    memset(&a, 0, sizeof(a));
    // packed vectors are addressed as the bytes they hold; their 32-bit elements must be aligned
    const uint32_t inEsz = packing != 1 ? 1u : cv::elemSize(d->inputType);
    const uint32_t outEsz = cv::elemSize(d->resultType);
    if (packing != 1 && ((uintptr_t)d->input % 4 || d->inputStride % 4))
        return fail(CV_E_INVALID_ARG, "cvMatMul: packed vectors must be 4-byte aligned");
    if ((uintptr_t)d->input % inEsz || d->inputStride % inEsz || (uintptr_t)d->output % outEsz || d->outputStride % outEsz)
        return fail(CV_E_INVALID_ARG, "cvMatMul: vector address/stride not aligned to the element size");
    if (d->batch > 1 && (d->inputStride < (size_t)d->k * inEsz || d->outputStride < (size_t)d->m * outEsz))
        return fail(CV_E_INVALID_ARG, "cvMatMul: vector stride smaller than the vector");
    a.in = (const uint8_t*)d->input;
    a.out = (uint8_t*)d->output;
    a.inStride = d->inputStride;
    a.outStride = d->outputStride;
    a.mat = (const uint8_t*)d->matrix + d->matrixOffset;
    const uint32_t rows = d->transpose ? (uint32_t)d->k : (uint32_t)d->m;
    const uint32_t cols = d->transpose ? (uint32_t)d->m : (uint32_t)d->k;
    a.shape = cv::MatrixShape{rows, cols, d->matrixInterpretation, d->layout, isOptimal(d->layout) ? 0 : (size_t)d->matrixStride};
    if (cv::matrixSize(a.shape) == 0) return fail(CV_E_INVALID_ARG, "cvMatMul: matrixStride %u smaller than a row/column", d->matrixStride);
    const uint32_t wEsz = cv::elemSize(d->matrixInterpretation);
    if ((uintptr_t)a.mat % (isOptimal(d->layout) ? 16u : wEsz) || (!isOptimal(d->layout) && d->matrixStride % wEsz))
        return fail(CV_E_INVALID_ARG, "cvMatMul: matrix address/stride misaligned");
    a.transpose = d->transpose ? 1 : 0;
    a.m = d->m;
    a.k = d->k;
    a.inCt = d->inputType;
    if (d->bias) {
        a.bias = (const uint8_t*)d->bias + d->biasOffset;
        a.biasCt = d->biasInterpretation;
        if ((uintptr_t)a.bias % cv::elemSize(a.biasCt)) return fail(CV_E_INVALID_ARG, "cvMatMul: bias misaligned");
    }
    a.outCt = d->resultType;
    a.act = d->activation;
    if (d->resultType == CV_UINT32 && a.act == CV_ACT_RELU) a.act = CV_ACT_NONE;   // max(u, 0) == u
    // the slope is taken in the result's type where that is half: the example builds it as a vector of the layer's element
    // type (fflayer.slang:64, CoopVec<NFloat, OutputSize>(0.001h))
    a.slope = d->resultType == CV_FLOAT16 ? (float)(_Float16)d->leakySlope : d->leakySlope;
    a.accumulate = d->accumulate ? 1 : 0;
    a.batch = d->batch;
    a.inUnsigned = combo.inUnsigned ? 1 : 0;
    a.matUnsigned = combo.matUnsigned ? 1 : 0;
    a.inAlign = alignOf(d->input, d->inputStride);
    a.outAlign = alignOf(d->output, d->outputStride);

    CvResult rc;
    const int cus = currentDeviceCUs(&rc);
    if (CV_FAILED(rc)) return rc;
    cv::MmaKind kind = combo.kind;
    if (kind == cv::MmaKind::Fp8AsF16 && (d->flags & CV_FLAG_FP8_MATRIX_PIPELINE)) kind = cv::MmaKind::Fp8Native;
    if (kind == cv::MmaKind::Scalar) {
        if (packing != 1) a.inCt = CV_SINT8;      // the bytes of a packed vector, sign-extended for both packed kinds
        const bool floatRes = d->resultType == CV_FLOAT16 || d->resultType == CV_FLOAT32 || d->resultType == CV_FLOAT64;
        if (a.act > (floatRes ? CV_ACT_LEAKY_RELU : CV_ACT_RELU))
            return fail(CV_E_NOT_AVAILABLE, "cvMatMul: activation %d with input %d, matrix %d, result %d (this combination takes NONE, RELU%s)",
                        d->activation, d->inputType, d->matrixInterpretation, d->resultType, floatRes ? ", LEAKY_RELU" : "");
        const int kLimit = cv::elemSize(d->resultType) == 8 ? 6144 : 12288;
        if (d->k > kLimit)
            return fail(CV_E_NOT_AVAILABLE, "cvMatMul: k=%d (limit %d for input %d, matrix %d, result %d)", d->k, kLimit, d->inputType,
                        d->matrixInterpretation, d->resultType);
    }
    const hipError_t e = cv::launchMatMul((hipStream_t)stream, kind, a, cus);
    if (e == hipErrorInvalidValue)
        return fail(CV_E_NOT_AVAILABLE, "cvMatMul: k=%d is beyond what one 16-row block of the matrix can keep in LDS "
                    "(128 KiB: k <= 2048 for 32-bit types, 4096 for 16-bit ones, 8192 for 8-bit ones)", d->k);
    return fromHip(e, "cvMatMul launch");
}

CV_API CvResult cvOuterProductAccumulateWorkspaceSize(int32_t m, int32_t n, uint32_t batch, size_t* outBytes)
{
    if (!outBytes) return fail(CV_E_INVALID_ARG, "cvOuterProductAccumulateWorkspaceSize: outBytes is null");
    *outBytes = 0;
    if (m <= 0 || n <= 0) return fail(CV_E_INVALID_ARG, "cvOuterProductAccumulateWorkspaceSize: m=%d n=%d", m, n);
    CvResult rc;
    const int cus = currentDeviceCUs(&rc);
    if (CV_FAILED(rc)) return rc;
    const size_t fast = cv::outerWorkspaceBytes(m, n, batch ? batch : 1, cus), scalar = cv::accumScalarWorkspaceBytes(m, n, batch ? batch : 1);
    const size_t f32 = cv::outerF32WorkspaceBytes(m, n, batch ? batch : 1, cus);
    *outBytes = std::max(fast, std::max(scalar, f32));      // whichever kernel the element types select
    return CV_OK;
}

CV_API CvResult cvOuterProductAccumulate(void* stream, const void* a, size_t aStride, int32_t m,
                                         const void* b, size_t bStride, int32_t n, int32_t elementType,
                                         uint32_t batch, void* matrix, size_t matrixOffset, uint32_t matrixStride,
                                         int32_t layout, int32_t matrixInterpretation, void* workspace,
                                         size_t workspaceBytes)
{
    if (m <= 0 || n <= 0) return fail(CV_E_INVALID_ARG, "cvOuterProductAccumulate: m=%d n=%d", m, n);
    if (cvComponentPackingFactor(matrixInterpretation) != 1)   // static_assert hlsl.meta.slang:33237
        return fail(CV_E_INVALID_ARG, "cvOuterProductAccumulate: can't use packed component type in matrixInterpretation");
    if (layout < 0 || layout > 3) return fail(CV_E_INVALID_ARG, "cvOuterProductAccumulate: unknown layout %d", layout);
    const bool onMatrixCores = elementType == CV_FLOAT16 && (matrixInterpretation == CV_FLOAT16 || matrixInterpretation == CV_FLOAT32);
    if (!onMatrixCores) {
        // every other pair of the fallback's types (hlsl.meta.slang:33261-33315): the scalar definition
        if (!cv::isPlainComponent(elementType) || !cv::isPlainComponent(matrixInterpretation))
            return fail(CV_E_NOT_AVAILABLE, "cvOuterProductAccumulate: vectors of type %d into a matrix of type %d (supported: FLOAT16/32/64 "
                        "and the 8/16/32/64-bit integers on either side)", elementType, matrixInterpretation);
        if (!cv::layoutSupports(matrixInterpretation, layout))
            return fail(CV_E_NOT_AVAILABLE, "cvOuterProductAccumulate: component type %d has no layout %d", matrixInterpretation, layout);
        if (batch == 0) return CV_OK;
        if (!a || !b || !matrix || !workspace) return fail(CV_E_INVALID_ARG, "cvOuterProductAccumulate: null argument");
        const uint32_t tsz = cv::elemSize(elementType), msz = cv::elemSize(matrixInterpretation);
        if ((uintptr_t)a % tsz || aStride % tsz || (uintptr_t)b % tsz || bStride % tsz || (uintptr_t)workspace % 8)
            return fail(CV_E_INVALID_ARG, "cvOuterProductAccumulate: misaligned vectors/workspace");
        if (batch > 1 && (aStride < (size_t)m * tsz || bStride < (size_t)n * tsz))
            return fail(CV_E_INVALID_ARG, "cvOuterProductAccumulate: vector stride smaller than the vector");
        const cv::MatrixShape shape{(uint32_t)m, (uint32_t)n, matrixInterpretation, layout, isOptimal(layout) ? 0 : (size_t)matrixStride};
        if (cv::matrixSize(shape) == 0) return fail(CV_E_INVALID_ARG, "cvOuterProductAccumulate: matrixStride %u smaller than a row/column", matrixStride);
        uint8_t* dst = (uint8_t*)matrix + matrixOffset;
        if ((uintptr_t)dst % msz || (!isOptimal(layout) && matrixStride % msz)) return fail(CV_E_INVALID_ARG, "cvOuterProductAccumulate: matrix misaligned");
        if (elementType == CV_FLOAT32 && matrixInterpretation == CV_FLOAT32) {      // the matrix pipeline's fp32 instruction
            CvResult rc;
            const int cus = currentDeviceCUs(&rc);
            if (CV_FAILED(rc)) return rc;
            const size_t need = cv::outerF32WorkspaceBytes(m, n, batch, cus);
            if (workspaceBytes < need) return fail(CV_E_BUFFER_TOO_SMALL, "cvOuterProductAccumulate: workspace of %zu bytes, %zu needed", workspaceBytes, need);
            return fromHip(cv::launchOuterProductF32((hipStream_t)stream, (const uint8_t*)a, aStride, m, (const uint8_t*)b, bStride, n, batch, dst,
                                                     shape, workspace, cus), "cvOuterProductAccumulate launch");
        }
        const size_t need = cv::accumScalarWorkspaceBytes(m, n, batch);
        if (workspaceBytes < need) return fail(CV_E_BUFFER_TOO_SMALL, "cvOuterProductAccumulate: workspace of %zu bytes, %zu needed", workspaceBytes, need);
        return fromHip(cv::launchAccumScalar((hipStream_t)stream, (const uint8_t*)a, aStride, m, (const uint8_t*)b, bStride, n, elementType, batch,
                                             dst, shape, workspace), "cvOuterProductAccumulate launch");
    }
    if (batch == 0) return CV_OK;
    if (!a || !b || !matrix || !workspace) return fail(CV_E_INVALID_ARG, "cvOuterProductAccumulate: null argument");
    if ((uintptr_t)a % 2 || aStride % 2 || (uintptr_t)b % 2 || bStride % 2 || (uintptr_t)workspace % 16)
        return fail(CV_E_INVALID_ARG, "cvOuterProductAccumulate: misaligned vectors/workspace");
    if (batch > 1 && (aStride < (size_t)m * 2 || bStride < (size_t)n * 2))
        return fail(CV_E_INVALID_ARG, "cvOuterProductAccumulate: vector stride smaller than the vector");
    cv::OuterArgs o;
    memset(&o, 0, sizeof(o));
    o.a = (const uint8_t*)a; o.b = (const uint8_t*)b; o.aStride = aStride; o.bStride = bStride;
    o.aAlign = alignOf(a, aStride); o.bAlign = alignOf(b, bStride);
    o.m = m; o.n = n; o.batch = batch;
    o.mat = (uint8_t*)matrix + matrixOffset;
    o.shape = cv::MatrixShape{(uint32_t)m, (uint32_t)n, matrixInterpretation, layout, isOptimal(layout) ? 0 : (size_t)matrixStride};
    if (cv::matrixSize(o.shape) == 0) return fail(CV_E_INVALID_ARG, "cvOuterProductAccumulate: matrixStride %u smaller than a row/column", matrixStride);
    const uint32_t esz = cv::elemSize(matrixInterpretation);
    if ((uintptr_t)o.mat % esz || (!isOptimal(layout) && matrixStride % esz)) return fail(CV_E_INVALID_ARG, "cvOuterProductAccumulate: matrix misaligned");
    o.partials = (float*)workspace;
    CvResult rc;
    const int cus = currentDeviceCUs(&rc);
    if (CV_FAILED(rc)) return rc;
    const size_t need = cv::outerWorkspaceBytes(m, n, batch, cus);
    if (workspaceBytes < need) return fail(CV_E_BUFFER_TOO_SMALL, "cvOuterProductAccumulate: workspace of %zu bytes, %zu needed", workspaceBytes, need);
    return fromHip(cv::launchOuterProduct((hipStream_t)stream, o, cus), "cvOuterProductAccumulate launch");
}

CV_API CvResult cvReduceSumAccumulateWorkspaceSize(int32_t n, uint32_t batch, size_t* outBytes)
{
    if (!outBytes) return fail(CV_E_INVALID_ARG, "cvReduceSumAccumulateWorkspaceSize: outBytes is null");
    *outBytes = 0;
    if (n <= 0) return fail(CV_E_INVALID_ARG, "cvReduceSumAccumulateWorkspaceSize: n=%d", n);
    CvResult rc;
    const int cus = currentDeviceCUs(&rc);
    if (CV_FAILED(rc)) return rc;
    const size_t fast = cv::reduceSumWorkspaceBytes(batch ? batch : 1, cus), scalar = cv::accumScalarWorkspaceBytes(n, 1, batch ? batch : 1);
    const size_t f32 = cv::outerF32WorkspaceBytes(n, 1, batch ? batch : 1, cus);
    *outBytes = std::max(fast, std::max(scalar, f32));
    return CV_OK;
}

CV_API CvResult cvReduceSumAccumulate(void* stream, const void* v, size_t vStride, int32_t n, int32_t elementType,
                                      uint32_t batch, void* buffer, size_t offset, int32_t bufferType,
                                      void* workspace, size_t workspaceBytes)
{
    if (n <= 0) return fail(CV_E_INVALID_ARG, "cvReduceSumAccumulate: n=%d", n);
    if (elementType != CV_FLOAT16) {
        // the destination has the vectors' type (hlsl.meta.slang:33344-33352): the scalar definition for every plain type
        if (!cv::isPlainComponent(elementType) || bufferType != elementType)
            return fail(CV_E_NOT_AVAILABLE, "cvReduceSumAccumulate: vectors of type %d into a buffer of type %d (the buffer has the vectors' "
                        "type; FLOAT16 vectors also go into FLOAT32)", elementType, bufferType);
        if (batch == 0) return CV_OK;
        if (!v || !buffer || !workspace) return fail(CV_E_INVALID_ARG, "cvReduceSumAccumulate: null argument");
        const uint32_t tsz = cv::elemSize(elementType);
        if ((uintptr_t)v % tsz || vStride % tsz || ((uintptr_t)buffer + offset) % tsz || (uintptr_t)workspace % 8)
            return fail(CV_E_INVALID_ARG, "cvReduceSumAccumulate: misaligned argument");
        if (batch > 1 && vStride < (size_t)n * tsz) return fail(CV_E_INVALID_ARG, "cvReduceSumAccumulate: vector stride smaller than the vector");
        const cv::MatrixShape shape{(uint32_t)n, 1u, elementType, CV_LAYOUT_ROW_MAJOR, (size_t)tsz};
        if (elementType == CV_FLOAT32) {      // the matrix pipeline's fp32 instruction
            CvResult rc;
            const int cus = currentDeviceCUs(&rc);
            if (CV_FAILED(rc)) return rc;
            const size_t need = cv::outerF32WorkspaceBytes(n, 1, batch, cus);
            if (workspaceBytes < need) return fail(CV_E_BUFFER_TOO_SMALL, "cvReduceSumAccumulate: workspace of %zu bytes, %zu needed", workspaceBytes, need);
            return fromHip(cv::launchOuterProductF32((hipStream_t)stream, (const uint8_t*)v, vStride, n, nullptr, 0, 1, batch,
                                                     (uint8_t*)buffer + offset, shape, workspace, cus), "cvReduceSumAccumulate launch");
        }
        const size_t need = cv::accumScalarWorkspaceBytes(n, 1, batch);
        if (workspaceBytes < need) return fail(CV_E_BUFFER_TOO_SMALL, "cvReduceSumAccumulate: workspace of %zu bytes, %zu needed", workspaceBytes, need);
        return fromHip(cv::launchAccumScalar((hipStream_t)stream, (const uint8_t*)v, vStride, n, nullptr, 0, 1, elementType, batch,
                                             (uint8_t*)buffer + offset, shape, workspace), "cvReduceSumAccumulate launch");
    }
    if (n > 256) return fail(CV_E_NOT_AVAILABLE, "cvReduceSumAccumulate: n=%d (limit 256)", n);
    if (bufferType != CV_FLOAT16 && bufferType != CV_FLOAT32)
        return fail(CV_E_NOT_AVAILABLE, "cvReduceSumAccumulate: bufferType %d (supported: FLOAT16, FLOAT32)", bufferType);
    if (batch == 0) return CV_OK;
    if (!v || !buffer || !workspace) return fail(CV_E_INVALID_ARG, "cvReduceSumAccumulate: null argument");
    const uint32_t esz = cv::elemSize(bufferType);
    if ((uintptr_t)v % 2 || vStride % 2 || ((uintptr_t)buffer + offset) % esz || (uintptr_t)workspace % 4)
        return fail(CV_E_INVALID_ARG, "cvReduceSumAccumulate: misaligned argument");
    if (batch > 1 && vStride < (size_t)n * 2) return fail(CV_E_INVALID_ARG, "cvReduceSumAccumulate: vector stride smaller than the vector");
    cv::ReduceSumArgs r;
    memset(&r, 0, sizeof(r));
    r.v = (const uint8_t*)v; r.vStride = vStride; r.n = n;
    r.colsPerGroup = (((n + 3) / 4) + 1) / 2 * 2;
    r.batch = batch; r.buf = (uint8_t*)buffer + offset; r.bufCt = bufferType; r.partials = (float*)workspace;
    CvResult rc;
    const int cus = currentDeviceCUs(&rc);
    if (CV_FAILED(rc)) return rc;
    const size_t need = cv::reduceSumWorkspaceBytes(batch, cus);
    if (workspaceBytes < need) return fail(CV_E_BUFFER_TOO_SMALL, "cvReduceSumAccumulate: workspace of %zu bytes, %zu needed", workspaceBytes, need);
    return fromHip(cv::launchReduceSum((hipStream_t)stream, r, cus), "cvReduceSumAccumulate launch");
}

// Validates the parts of a CvMlpDesc that forward and training share and fills the per-layer
// kernel arguments.
static CvResult fillMlpLayers(const char* who, const CvMlpDesc* mlp, cv::MlpLayerArgs* out)
{
    if (!mlp || !mlp->layers) return fail(CV_E_INVALID_ARG, "%s: mlp/layers is null", who);
    if (mlp->numLayers < 1 || mlp->numLayers > cv::kMaxMlpLayers)
        return fail(CV_E_INVALID_ARG, "%s: numLayers=%d (supported: 1..%d)", who, mlp->numLayers, cv::kMaxMlpLayers);
    const bool uniformT = mlp->weightType == CV_FLOAT32 || mlp->weightType == CV_BFLOAT16;   // T = float / bfloat16 throughout
    if (mlp->weightType != CV_FLOAT16 && mlp->weightType != CV_FLOAT_E4M3 && !uniformT)
        return fail(CV_E_NOT_AVAILABLE, "%s: weightType %d (supported: FLOAT16, FLOAT_E4M3, and FLOAT32 / BFLOAT16 networks of one type)",
                    who, mlp->weightType);
    if (uniformT) {
        if (mlp->inputType != mlp->weightType || mlp->biasType != mlp->weightType || mlp->outputType != mlp->weightType ||
            mlp->inputEncoding != CV_ENCODE_NONE)
            return fail(CV_E_NOT_AVAILABLE, "%s: a network with weightType %d takes vectors, biases and results of that type and no "
                        "input encoding", who, mlp->weightType);
    } else if (mlp->biasType != CV_FLOAT16 || mlp->outputType != CV_FLOAT16)
        return fail(CV_E_NOT_AVAILABLE, "%s: biasType/outputType must be FLOAT16", who);
    if (mlp->inputEncoding == CV_ENCODE_XY_SQUARES) {
        if (mlp->inputType != CV_FLOAT32 || mlp->weightType != CV_FLOAT16 || mlp->layers[0].inputSize != 4 || mlp->numLayers < 2)
            return fail(CV_E_NOT_AVAILABLE, "%s: CV_ENCODE_XY_SQUARES needs FLOAT32 (x, y) samples, FLOAT16 weights, a first "
                        "layer of 4 inputs and at least two layers", who);
    } else if (mlp->inputEncoding != CV_ENCODE_NONE) {
        return fail(CV_E_INVALID_ARG, "%s: unknown inputEncoding %d", who, mlp->inputEncoding);
    } else if (mlp->inputType != mlp->weightType &&
               !(mlp->inputType == CV_FLOAT16 && mlp->weightType == CV_FLOAT_E4M3)) {
        // besides vectors stored like the weights: CoopVec<half> with inputInterpretation FloatE4M3,
        // the form the operator takes on the Slang API (hlsl.meta.slang:32954-32963)
        return fail(CV_E_NOT_AVAILABLE, "%s: inputType %d must equal weightType %d (or be FLOAT16 for FLOAT_E4M3 weights)",
                    who, mlp->inputType, mlp->weightType);
    }
    const uint32_t wEsz = cv::elemSize(mlp->weightType);
    for (int l = 0; l < mlp->numLayers; ++l) {
        const CvMlpLayer& L = mlp->layers[l];
        if (!L.weights) return fail(CV_E_INVALID_ARG, "%s: layer %d has no weights", who, l);
        if (L.inputSize <= 0 || L.outputSize <= 0) return fail(CV_E_INVALID_ARG, "%s: layer %d is %dx%d", who, l, L.outputSize, L.inputSize);
        if (l > 0 && L.inputSize != mlp->layers[l - 1].outputSize)
            return fail(CV_E_INVALID_ARG, "%s: layer %d takes %d inputs but layer %d produces %d", who, l, L.inputSize, l - 1, mlp->layers[l - 1].outputSize);
        if (L.weightLayout < 0 || L.weightLayout > 3 || !cv::layoutSupports(mlp->weightType, L.weightLayout))
            return fail(CV_E_NOT_AVAILABLE, "%s: layer %d: component type %d has no layout %d", who, l, mlp->weightType, L.weightLayout);
        if (L.activation < CV_ACT_NONE || L.activation > CV_ACT_QUICK_GELU)
            return fail(CV_E_INVALID_ARG, "%s: layer %d: unknown activation %d", who, l, L.activation);
        cv::MlpLayerArgs& o = out[l];
        o.w = (const uint8_t*)L.weights;
        o.bias = (const uint8_t*)L.biases;
        o.shape = cv::MatrixShape{(uint32_t)L.outputSize, (uint32_t)L.inputSize, mlp->weightType, L.weightLayout,
                                  isOptimal(L.weightLayout) ? 0 : (size_t)L.weightStride};
        if (cv::matrixSize(o.shape) == 0) return fail(CV_E_INVALID_ARG, "%s: layer %d: weightStride %u smaller than a row/column", who, l, L.weightStride);
        if ((uintptr_t)o.w % (isOptimal(L.weightLayout) ? 16u : wEsz) || (!isOptimal(L.weightLayout) && L.weightStride % wEsz) ||
            (uintptr_t)o.bias % cv::elemSize(mlp->biasType))
            return fail(CV_E_INVALID_ARG, "%s: layer %d: weights/bias misaligned", who, l);
        // the slope of a network of half vectors is a half value (fflayer.slang:64: CoopVec<NFloat, OutputSize>(0.001h))
        o.in = L.inputSize; o.out = L.outputSize; o.act = L.activation;
        o.slope = uniformT ? L.leakySlope : (float)(_Float16)L.leakySlope;
    }
    return CV_OK;
}

CV_API CvResult cvMlpForward(void* stream, const CvMlpDesc* mlp, const void* input, size_t inputStride,
                             void* output, size_t outputStride, uint32_t batch)
{
    cv::MlpArgs a;
    memset(&a, 0, sizeof(a));
    CvResult rc = fillMlpLayers("cvMlpForward", mlp, a.layers);
    if (CV_FAILED(rc)) return rc;
    if (batch == 0) return CV_OK;
    if (!input || !output) return fail(CV_E_INVALID_ARG, "cvMlpForward: null input/output");
    const uint32_t inEsz = cv::elemSize(mlp->inputType);
    const int L = mlp->numLayers;
    const bool encoded = mlp->inputEncoding == CV_ENCODE_XY_SQUARES;
    const size_t sampleBytes = encoded ? 2 * sizeof(float) : (size_t)mlp->layers[0].inputSize * inEsz;
    const uint32_t outEsz = cv::elemSize(mlp->outputType);
    if ((uintptr_t)input % inEsz || inputStride % inEsz || (uintptr_t)output % outEsz || outputStride % outEsz)
        return fail(CV_E_INVALID_ARG, "cvMlpForward: vector address/stride not aligned to the element size");
    if (batch > 1 && (inputStride < sampleBytes || outputStride < (size_t)mlp->layers[L - 1].outputSize * outEsz))
        return fail(CV_E_INVALID_ARG, "cvMlpForward: vector stride smaller than the vector");
    if (L == 1) {   // a single layer is the plain operator
        const CvMlpLayer& l0 = mlp->layers[0];
        CvMatMulDesc d;
        memset(&d, 0, sizeof(d));
        d.input = input; d.inputStride = inputStride; d.inputType = mlp->inputType; d.inputInterpretation = mlp->weightType;
        d.k = l0.inputSize; d.output = output; d.outputStride = outputStride; d.resultType = mlp->outputType; d.m = l0.outputSize;
        d.matrix = l0.weights; d.matrixInterpretation = mlp->weightType; d.layout = l0.weightLayout; d.matrixStride = l0.weightStride;
        d.bias = l0.biases; d.biasInterpretation = mlp->biasType; d.activation = l0.activation; d.leakySlope = l0.leakySlope;
        d.batch = batch; d.flags = mlp->flags;
        return cvMatMul(stream, &d);
    }
    a.numLayers = L;
    a.in = (const uint8_t*)input; a.out = (uint8_t*)output;
    a.inStride = inputStride; a.outStride = outputStride; a.batch = batch;
    a.inAlign = alignOf(input, inputStride); a.outAlign = alignOf(output, outputStride);
    a.inEncoding = encoded ? cv::kEncodeXYSquares : cv::kEncodeNone;
    a.inHalfAsE4M3 = (mlp->inputType == CV_FLOAT16 && mlp->weightType == CV_FLOAT_E4M3) ? 1 : 0;
    a.noWideTiles = (mlp->flags & CV_FLAG_FORWARD_TILE16) ? 1 : 0;
    const int cus = currentDeviceCUs(&rc);
    if (CV_FAILED(rc)) return rc;
    hipError_t e;
    if (mlp->weightType == CV_FLOAT32 || mlp->weightType == CV_BFLOAT16) {
        e = cv::launchMlpFloat((hipStream_t)stream, mlp->weightType == CV_FLOAT32 ? cv::MmaKind::F32 : cv::MmaKind::Bf16, a, cus);
    } else {
        cv::MmaKind kind = mlp->weightType == CV_FLOAT16 ? cv::MmaKind::F16
                         : (mlp->flags & CV_FLAG_FP8_MATRIX_PIPELINE) ? cv::MmaKind::Fp8Native : cv::MmaKind::Fp8AsF16;
        e = cv::launchMlpForward((hipStream_t)stream, kind, a, cus);
        if (e == hipErrorInvalidValue) e = cv::launchMlpGeneric((hipStream_t)stream, kind, a, cus);   // no built-in shape: general kernel
    }
    if (e == hipErrorInvalidValue)
        return fail(CV_E_NOT_AVAILABLE, "cvMlpForward: layer sizes beyond the fused kernels (every dimension must be <= 128 "
                    "and all weights must fit 144 KB of LDS); chain cvMatMul calls instead");
    return fromHip(e, "cvMlpForward launch");
}

CV_API CvResult cvPermutoMlpForward(void* stream, const CvPermutoDesc* desc, const void* positions, size_t positionStride,
                                    const void* featureTable, const CvMlpDesc* mlp, void* output, size_t outputStride, uint32_t batch)
{
    const char* who = "cvPermutoMlpForward";
    CvResult rc = cv::checkPermutoDesc(who, desc);
    if (CV_FAILED(rc)) return rc;
    cv::MlpArgs a;
    memset(&a, 0, sizeof(a));
    rc = fillMlpLayers(who, mlp, a.layers);
    if (CV_FAILED(rc)) return rc;
    const int F = desc->featureDimensionPerEntry, L = mlp->numLayers;
    if (desc->elementType != CV_FLOAT16 || mlp->weightType != CV_FLOAT16 || mlp->inputType != CV_FLOAT16 ||
        mlp->inputEncoding != CV_ENCODE_NONE || L < 2)
        return fail(CV_E_NOT_AVAILABLE, "%s: a FLOAT16 encoder in front of a FLOAT16 network of at least two layers without another "
                    "input encoding; otherwise call cvPermutoEncode and cvMlpForward", who);
    if (desc->dimensions > 4 || (F != 1 && F != 2 && F != 4))
        return fail(CV_E_NOT_AVAILABLE, "%s: dimensions=%d (1..4), featureDimensionPerEntry=%d (1, 2 or 4); otherwise call "
                    "cvPermutoEncode and cvMlpForward", who, desc->dimensions, F);
    if ((uint32_t)mlp->layers[0].inputSize != desc->maxLevels * (uint32_t)F)
        return fail(CV_E_INVALID_ARG, "%s: the first layer takes %d inputs, the encoder produces %u", who, mlp->layers[0].inputSize,
                    desc->maxLevels * (uint32_t)F);
    for (uint32_t l = 0; l < desc->maxLevels; ++l)
        if (desc->levelInfo[l].currentLevelIndex != l)
            return fail(CV_E_NOT_AVAILABLE, "%s: level record %u writes level %u (records in level order only)", who, l,
                        desc->levelInfo[l].currentLevelIndex);
    if (batch == 0) return CV_OK;
    if (!positions || !featureTable || !output) return fail(CV_E_INVALID_ARG, "%s: null argument", who);
    if ((uintptr_t)positions % 2 || positionStride % 2 || (uintptr_t)featureTable % (2u * (uint32_t)F) || (uintptr_t)output % 2 || outputStride % 2)
        return fail(CV_E_INVALID_ARG, "%s: misaligned argument (positions and output to 2 bytes, the feature table to one entry)", who);
    if (batch > 1 && (positionStride < (size_t)desc->dimensions * 2 || outputStride < (size_t)mlp->layers[L - 1].outputSize * 2))
        return fail(CV_E_INVALID_ARG, "%s: vector stride smaller than the vector", who);
    a.numLayers = L;
    a.out = (uint8_t*)output; a.outStride = outputStride; a.batch = batch;
    a.outAlign = alignOf(output, outputStride);
    a.noWideTiles = (mlp->flags & CV_FLAG_FORWARD_TILE16) ? 1 : 0;
    const int cus = currentDeviceCUs(&rc);
    if (CV_FAILED(rc)) return rc;
    const hipError_t e = cv::launchPermutoMlp((hipStream_t)stream, *desc, positions, positionStride, featureTable, a, cus);
    if (e == hipErrorInvalidValue)
        return fail(CV_E_NOT_AVAILABLE, "%s: every dimension of the network must be <= 128, its weights must fit in LDS beside the level "
                    "records and its activations must be NONE, RELU or LEAKY_RELU; otherwise call cvPermutoEncode and cvMlpForward", who);
    return fromHip(e, "cvPermutoMlpForward launch");
}

CV_API CvResult cvMlpTrainStepWorkspaceSize(const CvMlpDesc* mlp, uint32_t batch, size_t* outBytes)
{
    if (!outBytes) return fail(CV_E_INVALID_ARG, "cvMlpTrainStepWorkspaceSize: outBytes is null");
    *outBytes = 0;
    cv::MlpArgs a;
    memset(&a, 0, sizeof(a));
    CvResult rc = fillMlpLayers("cvMlpTrainStepWorkspaceSize", mlp, a.layers);
    if (CV_FAILED(rc)) return rc;
    const bool f32net = mlp->weightType == CV_FLOAT32;      // a network of float: layer by layer
    if (mlp->weightType != CV_FLOAT16 && !f32net)
        return fail(CV_E_NOT_AVAILABLE, "cvMlpTrainStep: training needs FLOAT16 weights (or a FLOAT32 network)");
    if (mlp->numLayers < 2) return fail(CV_E_NOT_AVAILABLE, "cvMlpTrainStep: needs at least two layers");
    a.numLayers = mlp->numLayers;
    a.batch = batch;
    a.inEncoding = mlp->inputEncoding == CV_ENCODE_XY_SQUARES ? cv::kEncodeXYSquares : cv::kEncodeNone;
    const int cus = currentDeviceCUs(&rc);
    if (CV_FAILED(rc)) return rc;
    size_t n = ((mlp->flags & CV_FLAG_LAYERWISE_TRAINING) || f32net) ? 0 : cv::trainWorkspaceBytes(a, cus);
    if (!n) n = cv::trainGeneralWorkspaceBytes(a, cus, f32net ? CV_FLOAT32 : CV_FLOAT16);   // no fused shape: the layer-by-layer step
    *outBytes = n;
    return CV_OK;
}

// Shared body of cvMlpTrainStep and cvMlpTrainStepNoAlloc; `ownScratch` marks the library's own
// scratch array, whose fixed size is a limit of the entry point rather than a caller's mistake.
static CvResult trainStep(const char* who, void* stream, const CvMlpDesc* mlp, const void* input, size_t inputStride,
                          const void* targets, size_t targetStride, float lossScale, uint32_t batch,
                          float* lossSum, void* workspace, size_t workspaceBytes, bool ownScratch)
{
    cv::TrainLaunch t;
    memset(&t, 0, sizeof(t));
    CvResult rc = fillMlpLayers(who, mlp, t.mlp.layers);
    if (CV_FAILED(rc)) return rc;
    const bool f32net = mlp->weightType == CV_FLOAT32;      // a network of float: layer by layer, fp32 gradients
    if (mlp->weightType != CV_FLOAT16 && !f32net)
        return fail(CV_E_NOT_AVAILABLE, "%s: training needs FLOAT16 weights (or a FLOAT32 network)", who);
    if (mlp->gradType != CV_FLOAT16 && mlp->gradType != CV_FLOAT32)
        return fail(CV_E_NOT_AVAILABLE, "%s: gradType %d (supported: FLOAT16, FLOAT32)", who, mlp->gradType);
    if (f32net && mlp->gradType != CV_FLOAT32)
        return fail(CV_E_NOT_AVAILABLE, "%s: a FLOAT32 network accumulates FLOAT32 gradients", who);
    const size_t vEsz = f32net ? 4 : 2;                     // element size of vectors and targets
    const int L = mlp->numLayers;
    if (L < 2) return fail(CV_E_NOT_AVAILABLE, "%s: needs at least two layers", who);
    if (batch == 0) return CV_OK;
    if (!input || !workspace) return fail(CV_E_INVALID_ARG, "%s: null input/workspace", who);
    const bool encoded = mlp->inputEncoding == CV_ENCODE_XY_SQUARES;
    const size_t inAlignTo = encoded ? 4 : vEsz, sampleBytes = encoded ? 2 * sizeof(float) : (size_t)mlp->layers[0].inputSize * vEsz;
    if ((uintptr_t)input % inAlignTo || inputStride % inAlignTo || (uintptr_t)targets % vEsz || targetStride % vEsz ||
        (uintptr_t)workspace % 16 || (uintptr_t)lossSum % 4 || (uintptr_t)mlp->lossMax % 4)
        return fail(CV_E_INVALID_ARG, "%s: misaligned input/targets/workspace/lossSum/lossMax", who);
    if (encoded && !targets && mlp->layers[L - 1].outputSize != 4)
        return fail(CV_E_INVALID_ARG, "%s: the example's loss (targets == NULL with CV_ENCODE_XY_SQUARES) needs 4 outputs", who);
    if (batch > 1 && (inputStride < sampleBytes ||
                      (targets && targetStride < (size_t)mlp->layers[L - 1].outputSize * vEsz)))
        return fail(CV_E_INVALID_ARG, "%s: vector stride smaller than the vector", who);
    const uint32_t gEsz = cv::elemSize(mlp->gradType);
    for (int l = 0; l < L; ++l) {
        const CvMlpLayer& ly = mlp->layers[l];
        if (ly.activation > CV_ACT_LEAKY_RELU)
            return fail(CV_E_NOT_AVAILABLE, "%s: layer %d: the fused training step differentiates NONE, RELU and LEAKY_RELU only", who, l);
        // with 0 <= slope <= 0.5 the outcome of max(z, z*slope) is the sign of z for every fp16 z
        if (ly.activation == CV_ACT_LEAKY_RELU && !(ly.leakySlope >= 0.f && ly.leakySlope <= 0.5f))
            return fail(CV_E_INVALID_ARG, "%s: layer %d: leakySlope must be in [0, 0.5]", who, l);
        t.wGrad[l] = (uint8_t*)ly.weightsGrad;
        t.bGrad[l] = (uint8_t*)ly.biasesGrad;
        if (ly.weightsGrad) {
            if (ly.gradLayout < 0 || ly.gradLayout > 3 || !cv::layoutSupports(mlp->gradType, ly.gradLayout))
                return fail(CV_E_NOT_AVAILABLE, "%s: layer %d: component type %d has no layout %d", who, l, mlp->gradType, ly.gradLayout);
            t.gradShape[l] = cv::MatrixShape{(uint32_t)ly.outputSize, (uint32_t)ly.inputSize, mlp->gradType, ly.gradLayout,
                                             isOptimal(ly.gradLayout) ? 0 : (size_t)ly.gradStride};
            if (cv::matrixSize(t.gradShape[l]) == 0) return fail(CV_E_INVALID_ARG, "%s: layer %d: gradStride %u smaller than a row/column", who, l, ly.gradStride);
            if ((uintptr_t)ly.weightsGrad % gEsz || ly.gradStride % gEsz) return fail(CV_E_INVALID_ARG, "%s: layer %d: weightsGrad misaligned", who, l);
        }
        if ((uintptr_t)ly.biasesGrad % gEsz) return fail(CV_E_INVALID_ARG, "%s: layer %d: biasesGrad misaligned", who, l);
    }
    t.mlp.numLayers = L;
    t.mlp.in = (const uint8_t*)input;
    t.mlp.inStride = inputStride;
    t.mlp.batch = batch;
    t.mlp.inAlign = alignOf(input, inputStride);
    t.mlp.inEncoding = encoded ? cv::kEncodeXYSquares : cv::kEncodeNone;
    t.splitByRole = (mlp->flags & CV_FLAG_TRAIN_SPLIT_BY_ROLE) ? 1 : 0;
    t.targets = (const uint8_t*)targets;
    t.targetStride = targetStride;
    t.lossScale = lossScale;
    t.gradCt = mlp->gradType;
    t.carrierCt = f32net ? CV_FLOAT32 : CV_FLOAT16;
    t.lossSum = lossSum;
    t.lossMax = mlp->lossMax;
    t.workspace = (float*)workspace;
    const int cus = currentDeviceCUs(&rc);
    if (CV_FAILED(rc)) return rc;
    size_t need = ((mlp->flags & CV_FLAG_LAYERWISE_TRAINING) || f32net) ? 0 : cv::trainWorkspaceBytes(t.mlp, cus);
    const bool fused = need != 0;
    if (!fused) need = cv::trainGeneralWorkspaceBytes(t.mlp, cus, t.carrierCt);   // layer by layer, any layer sizes
    if (workspaceBytes < need) {
        if (ownScratch)
            return fail(CV_E_NOT_AVAILABLE, "%s: this network needs %zu bytes of scratch, the built-in array holds %zu; "
                        "use cvMlpTrainStep with a caller-provided workspace", who, need, workspaceBytes);
        return fail(CV_E_BUFFER_TOO_SMALL, "%s: workspace of %zu bytes, %zu needed", who, workspaceBytes, need);
    }
    if (fused) return fromHip(cv::launchMlpTrain((hipStream_t)stream, t, cus), who);
    const hipError_t e = cv::launchMlpTrainGeneral((hipStream_t)stream, t, cus);
    if (e == hipErrorInvalidValue)
        return fail(CV_E_NOT_AVAILABLE, "%s: a layer is wider than the matMul kernels serve (k beyond 4096)", who);
    return fromHip(e, who);
}

CV_API CvResult cvMlpTrainStep(void* stream, const CvMlpDesc* mlp, const void* input, size_t inputStride,
                               const void* targets, size_t targetStride, float lossScale, uint32_t batch,
                               float* lossSum, void* workspace, size_t workspaceBytes)
{
    return trainStep("cvMlpTrainStep", stream, mlp, input, inputStride, targets, targetStride, lossScale, batch,
                     lossSum, workspace, workspaceBytes, false);
}

CV_API CvResult cvMlpTrainStepNoAlloc(void* stream, const CvMlpDesc* mlp, const void* input, size_t inputStride,
                                      const void* targets, size_t targetStride, float lossScale, uint32_t batch,
                                      float* lossSum)
{
    CvResult rc;
    void* ws = scratchOfCurrentDevice(&rc);
    if (CV_FAILED(rc)) return rc;
    return trainStep("cvMlpTrainStepNoAlloc", stream, mlp, input, inputStride, targets, targetStride, lossScale,
                     batch, lossSum, ws, CV_NOALLOC_SCRATCH_BYTES, true);
}

} // extern "C"
