// cv_elementwise.hip -- the per-component surface of CoopVec<T,N> over a batch, forward and reverse.
//
// Replaces, for a whole dispatch of shader threads at once, the element-wise operators and math
// functions Slang declares on CoopVec<T,N> -- arithmetic expanded per element by
// source/slang/slang-ir-lower-coopvec.cpp:113-166; min/max/clamp/step
// source/slang/hlsl.meta.slang:32043-32229; sin, cos, exp, log, log2, exp2, tanh, atan, fma
// :32231-32421 -- the activations of the neural module
// (source/standard-modules/neural/activations.slang), and their reverse-mode derivative rules
// (source/slang/diff.meta.slang:1948-2470).  Pure streaming: HBM-bound.
#include <hip/hip_runtime.h>

#include <cstring>
#include <type_traits>

#include "cv_device.h"
#include "cv_error.h"

namespace cv {
namespace {

struct EwArgs {
    const uint8_t* a; const uint8_t* b; const uint8_t* c; const uint8_t* dOut;
    uint8_t* out; uint8_t* dA; uint8_t* dB; uint8_t* dC;
    uint64_t aStride, bStride, cStride, dOutStride, outStride, dAStride, dBStride, dCStride;
    int32_t op, n;
    uint32_t batch;
    float param;
};

enum : int {
    kOpAdd = 0, kOpSub, kOpMul, kOpDiv, kOpNeg, kOpMin, kOpMax, kOpClamp, kOpStep, kOpSin, kOpCos, kOpExp, kOpLog,
    kOpLog2, kOpExp2, kOpTanh, kOpAtan, kOpFma, kOpRelu, kOpLeakyRelu, kOpSigmoid, kOpSilu, kOpQuickGelu, kOpScale, kOpCount
};

__host__ __device__ constexpr int operandCount(int op)
{
    switch (op) {
    case kOpAdd: case kOpSub: case kOpMul: case kOpDiv: case kOpMin: case kOpMax: case kOpStep: return 2;
    case kOpClamp: case kOpFma: return 3;
    }
    return 1;
}

// double -> half in one rounding: through a float that keeps a sticky last bit (round to odd)
__device__ __forceinline__ half_t halfOfDouble(double d)
{
    float f = (float)d;
    const double back = (double)f;
    if (back != d) {
        uint32_t u = __builtin_bit_cast(uint32_t, f);
        if (__builtin_fabs(back) > __builtin_fabs(d)) u -= 1u;      // towards zero
        f = __builtin_bit_cast(float, u | 1u);
    }
    return (half_t)f;
}

__device__ __forceinline__ float evalOp(int op, float a, float b, float c, float param)
{
    switch (op) {
    case kOpAdd: return a + b;
    case kOpSub: return a - b;
    case kOpMul: return a * b;
    case kOpDiv: return a / b;
    case kOpNeg: return -a;
    case kOpMin: return fminf(a, b);
    case kOpMax: return fmaxf(a, b);
    case kOpClamp: return fminf(fmaxf(a, b), c);
    case kOpStep: return b >= a ? 1.f : 0.f;            // step(edge, x) = x >= edge
    case kOpSin: return sinf(a);
    case kOpCos: return cosf(a);
    case kOpExp: return expf(a);
    case kOpLog: return logf(a);
    case kOpLog2: return log2f(a);
    case kOpExp2: return exp2f(a);
    case kOpTanh: return tanhf(a);
    case kOpAtan: return atanf(a);
    case kOpFma: return __builtin_fmaf(a, b, c);
    case kOpRelu: return fmaxf(a, 0.f);
    case kOpLeakyRelu: return a < 0.f ? param * a : a;  // activations.slang:69-74
    case kOpSigmoid: return smoothActivation(a, kActSigmoid);
    case kOpSilu: return smoothActivation(a, kActSilu);
    case kOpQuickGelu: return smoothActivation(a, kActQuickGelu);
    case kOpScale: return a * param;                    // vector * scalar, hlsl.meta.slang:32004 (param already of type T)
    }
    return a;
}

// The result as an element of type T.  A half vector is evaluated in float and rounded once, which is the correctly
// rounded half result for + - * / (a float holds more than twice the bits of a half plus two); fma is not of that kind
// (a float result can land on a half tie that the exact value misses), so it is summed exactly in double (exact for
// half operands whenever the result is finite) and rounded to half once.
// tanh for a result that is rounded to half: 1 - 2 / (1 + exp(2|x|)) from the hardware's exp2 and reciprocal (1 ulp of a
// float each; an overflowing exponential ends at exactly 1), and below |x| = 1/16, where that difference cancels, x - x^3/3
// (the next term is 2 x^5/15, under 2 * 10^-6 of x there): errors of 10^-7 absolute above and 2 * 10^-6 relative below, far
// inside a half's spacing of 5 * 10^-4.  Half the instructions of the float routine.
__device__ __forceinline__ float tanhForHalf(float x)
{
    const float ax = __builtin_fabsf(x);
    const float t = __builtin_amdgcn_exp2f(ax * 2.885390082f);             // exp(2|x|), 2 / ln 2 = 2.88539...
    const float big = __builtin_fmaf(-2.f, __builtin_amdgcn_rcpf(1.f + t), 1.f);
    const float small = ax * __builtin_fmaf(x * x, -1.f / 3.f, 1.f);
    return __builtin_copysignf(ax < 0.0625f ? small : big, x);
}

template <typename T>
__device__ __forceinline__ T evalOpAs(int op, float a, float b, float c, float param)
{
    if constexpr (std::is_same<T, half_t>::value) {
        if (op == kOpFma) return halfOfDouble((double)a * (double)b + (double)c);
        if (op == kOpTanh) return (half_t)tanhForHalf(a);
    }
    return (T)evalOp(op, a, b, c, param);
}

// d(sigmoid(k x) * x)/dx for k = 1 (SiLU) or 1.702 (QuickGELU): s + k x s (1 - s)
__device__ __forceinline__ float gatedSigmoidGrad(float x, float k)
{
    const float s = smoothActivation(k * x, kActSigmoid);
    return s + k * x * s * (1.f - s);
}

// partial derivatives times dOut, by the rules of diff.meta.slang
__device__ __forceinline__ void gradOp(int op, float a, float b, float c, float g, float param, float& da, float& db, float& dc)
{
    da = db = dc = 0.f;
    switch (op) {
    case kOpAdd: da = g; db = g; break;
    case kOpSub: da = g; db = -g; break;
    case kOpMul: da = b * g; db = a * g; break;
    case kOpDiv: da = g / b; db = -a * g / (b * b); break;
    case kOpNeg: da = -g; break;
    case kOpMin:    // :2293-2300: the smaller operand takes dOut, a tie splits it
        da = a < b ? g : (a > b ? 0.f : 0.5f * g);
        db = b < a ? g : (b > a ? 0.f : 0.5f * g);
        break;
    case kOpMax:    // :2266-2273
        da = a > b ? g : (a < b ? 0.f : 0.5f * g);
        db = b > a ? g : (b < a ? 0.f : 0.5f * g);
        break;
    case kOpClamp:  // :2413-2421: x inside [min, max] (bounds included) keeps dOut, otherwise the bound it hit
        da = (a >= b && a <= c) ? g : 0.f;
        db = a < b ? g : 0.f;
        dc = a > c ? g : 0.f;
        break;
    case kOpStep: break;
    case kOpSin: da = cosf(a) * g; break;
    case kOpCos: da = -(sinf(a) * g); break;
    case kOpExp: da = expf(a) * g; break;
    case kOpLog: da = g / a; break;
    case kOpLog2: da = g / (a * 0.69314718055994530941723212145818f); break;
    case kOpExp2: da = exp2f(a) * 0.69314718055994530941723212145818f * g; break;
    case kOpTanh: { const float t = tanhf(a); da = g - t * t * g; break; }     // :2116-2124
    case kOpAtan: da = g / (a * a + 1.f); break;
    case kOpFma: da = b * g; db = a * g; dc = g; break;
    case kOpRelu: da = a > 0.f ? g : (a < 0.f ? 0.f : 0.5f * g); break;       // max(x, 0) by the max rule
    case kOpLeakyRelu: da = a < 0.f ? param * g : g; break;
    case kOpSigmoid: { const float s = smoothActivation(a, kActSigmoid); da = s * (1.f - s) * g; break; }
    case kOpSilu: da = gatedSigmoidGrad(a, 1.f) * g; break;
    case kOpQuickGelu: da = gatedSigmoidGrad(a, 1.702f) * g; break;
    case kOpScale: da = param * g; break;
    }
}

template <typename T> __device__ __forceinline__ float ld(const uint8_t* p) { return (float)*(const T*)p; }
template <typename T> __device__ __forceinline__ void st(uint8_t* p, float v) { *(T*)p = (T)v; }

// one thread per element; rows are contiguous, so consecutive lanes touch consecutive addresses
template <typename T, bool BACKWARD>
__global__ __launch_bounds__(256) void elementwiseKernel(const EwArgs e)
{
    const uint64_t total = (uint64_t)e.batch * (uint32_t)e.n;
    const int nOps = operandCount(e.op);
    for (uint64_t idx = (uint64_t)blockIdx.x * 256u + threadIdx.x; idx < total; idx += (uint64_t)gridDim.x * 256u) {
        const uint64_t s = idx / (uint32_t)e.n;
        const uint64_t off = (idx - s * (uint32_t)e.n) * sizeof(T);
        const float a = ld<T>(e.a + s * e.aStride + off);
        const float b = nOps >= 2 ? ld<T>(e.b + s * e.bStride + off) : 0.f;
        const float c = nOps >= 3 ? ld<T>(e.c + s * e.cStride + off) : 0.f;
        if constexpr (!BACKWARD) {
            *(T*)(e.out + s * e.outStride + off) = evalOpAs<T>(e.op, a, b, c, e.param);
        } else {
            const float g = ld<T>(e.dOut + s * e.dOutStride + off);
            float da, db, dc;
            gradOp(e.op, a, b, c, g, e.param, da, db, dc);
            if (e.dA) st<T>(e.dA + s * e.dAStride + off, da);
            if (e.dB && nOps >= 2) st<T>(e.dB + s * e.dBStride + off, db);
            if (e.dC && nOps >= 3) st<T>(e.dC + s * e.dCStride + off, dc);
        }
    }
}

// dense rows (stride = n elements) of a unary / binary operator on 16-byte pieces: the whole batch is
// one flat array
// (the operator is a template parameter of the loop: chosen once per thread, not once per element)
template <typename T, int OP>
__device__ __forceinline__ void elementwiseDenseLoop(const EwArgs& e, uint64_t pieces)
{
    constexpr int PER = 16 / sizeof(T);
    constexpr int nOps = operandCount(OP);
    for (uint64_t p = (uint64_t)blockIdx.x * 256u + threadIdx.x; p < pieces; p += (uint64_t)gridDim.x * 256u) {
        T va[PER], vb[PER], vc[PER], vo[PER];
        // (streaming accesses: every byte is touched once)
        *(u32x4*)va = __builtin_nontemporal_load((const u32x4*)(e.a + p * 16u));
        if constexpr (nOps >= 2) *(u32x4*)vb = __builtin_nontemporal_load((const u32x4*)(e.b + p * 16u));
        if constexpr (nOps >= 3) *(u32x4*)vc = __builtin_nontemporal_load((const u32x4*)(e.c + p * 16u));
#pragma unroll
        for (int i = 0; i < PER; ++i)
            vo[i] = evalOpAs<T>(OP, (float)va[i], nOps >= 2 ? (float)vb[i] : 0.f, nOps >= 3 ? (float)vc[i] : 0.f, e.param);
        __builtin_nontemporal_store(*(const u32x4*)vo, (u32x4*)(e.out + p * 16u));
    }
}

template <typename T, int OP = 0>
__device__ __forceinline__ void elementwiseDenseDispatch(const EwArgs& e, uint64_t pieces)
{
    if constexpr (OP < kOpCount) {
        if (e.op == OP) elementwiseDenseLoop<T, OP>(e, pieces);
        else elementwiseDenseDispatch<T, OP + 1>(e, pieces);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void elementwiseDenseKernel(const EwArgs e, uint64_t pieces)
{
    elementwiseDenseDispatch<T>(e, pieces);
}

// The operators Slang declares on integer vectors (arithmetic, min / max / clamp: hlsl.meta.slang:32115-32229) and,
// for double, those and step / fma, evaluated in the element type itself.  Integers wrap in two's complement like
// the reference's scalar code; the quotients C leaves undefined are given values here: x / 0 = 0, MIN / -1 = MIN.
template <typename T>
__device__ __forceinline__ T evalArith(int op, T a, T b, T c)
{
    if constexpr (std::is_integral<T>::value) {
        typedef typename std::make_unsigned<T>::type U;
        switch (op) {
        case kOpAdd: return (T)((U)a + (U)b);
        case kOpSub: return (T)((U)a - (U)b);
        case kOpMul: return (T)((U)a * (U)b);
        case kOpDiv:
            if (b == 0) return 0;
            if (std::is_signed<T>::value && b == (T)-1) return (T)((U)0 - (U)a);
            return (T)(a / b);
        case kOpNeg: return (T)((U)0 - (U)a);
        case kOpMin: return a < b ? a : b;
        case kOpMax: return a > b ? a : b;
        case kOpClamp: { const T lo = a > b ? a : b; return lo < c ? lo : c; }
        }
        return a;
    } else {
        switch (op) {
        case kOpAdd: return a + b;
        case kOpSub: return a - b;
        case kOpMul: return a * b;
        case kOpDiv: return a / b;
        case kOpNeg: return -a;
        case kOpMin: return fmin(a, b);
        case kOpMax: return fmax(a, b);
        case kOpClamp: return fmin(fmax(a, b), c);
        case kOpStep: return b >= a ? (T)1 : (T)0;
        case kOpFma: return __builtin_fma(a, b, c);
        }
        return a;
    }
}

bool arithOpFor(int32_t ct, int op)
{
    const bool common = op == kOpAdd || op == kOpSub || op == kOpMul || op == kOpDiv || op == kOpNeg || op == kOpMin ||
                        op == kOpMax || op == kOpClamp;
    return common || (ct == kF64 && (op == kOpStep || op == kOpFma));
}

template <typename T>
__global__ __launch_bounds__(256) void elementwiseArithKernel(const EwArgs e)
{
    const uint64_t total = (uint64_t)e.batch * (uint32_t)e.n;
    const int nOps = operandCount(e.op);
    for (uint64_t idx = (uint64_t)blockIdx.x * 256u + threadIdx.x; idx < total; idx += (uint64_t)gridDim.x * 256u) {
        const uint64_t s = idx / (uint32_t)e.n;
        const uint64_t off = (idx - s * (uint32_t)e.n) * sizeof(T);
        const T a = *(const T*)(e.a + s * e.aStride + off);
        const T b = nOps >= 2 ? *(const T*)(e.b + s * e.bStride + off) : (T)0;
        const T c = nOps >= 3 ? *(const T*)(e.c + s * e.cStride + off) : (T)0;
        *(T*)(e.out + s * e.outStride + off) = evalArith<T>(e.op, a, b, c);
    }
}

// CoopVec<T,N>(CoopVec<U,N>) / copyFrom (hlsl.meta.slang:30683-30730): element-wise conversion between any two of the
// plain types.  integer -> integer keeps the low bits (sign- or zero-extended from the source); integer -> float and
// float -> float round to nearest even, in one rounding; float -> integer truncates towards zero, with the values C
// leaves undefined fixed as: NaN -> 0, out of range -> saturated to 32 bits (64 for 64-bit targets), then the low
// bits for narrower targets.
struct CastArgs {
    const uint8_t* src; uint8_t* dst;
    uint64_t srcStride, dstStride;
    int32_t srcCt, dstCt, n;
    uint32_t batch;
};

// A 64-bit integer as a double that rounds like the integer itself in any later rounding to fewer bits: exact up to
// 2^53, beyond that the top 53 bits with the last one set if anything was cut off (sticky).
__device__ __forceinline__ double stickyDoubleOfInt(uint64_t bits, bool isUnsigned)
{
    const bool neg = !isUnsigned && (int64_t)bits < 0;
    const uint64_t mag = neg ? (uint64_t)0 - bits : bits;
    double d;
    if (mag < (1ull << 53)) {
        d = (double)mag;
    } else {
        const int sh = 64 - __builtin_clzll(mag) - 53;
        const uint64_t top = (mag >> sh) | ((mag & ((1ull << sh) - 1ull)) ? 1ull : 0ull);
        d = __builtin_ldexp((double)top, sh);
    }
    return neg ? -d : d;
}

__global__ __launch_bounds__(256) void vectorCastKernel(const CastArgs e)
{
    const uint64_t total = (uint64_t)e.batch * (uint32_t)e.n;
    const uint32_t sEsz = elemSize(e.srcCt), dEsz = elemSize(e.dstCt);
    const bool srcFloat = e.srcCt == kF16 || e.srcCt == kF32 || e.srcCt == kF64 || e.srcCt == kBF16;
    const bool srcUnsigned = e.srcCt == kU8 || e.srcCt == kU16 || e.srcCt == kU32 || e.srcCt == kU64;
    for (uint64_t idx = (uint64_t)blockIdx.x * 256u + threadIdx.x; idx < total; idx += (uint64_t)gridDim.x * 256u) {
        const uint64_t s = idx / (uint32_t)e.n, i = idx - s * (uint32_t)e.n;
        const uint8_t* p = e.src + s * e.srcStride + i * sEsz;
        uint8_t* q = e.dst + s * e.dstStride + i * dEsz;
        double f = 0.0;          // a float source, exactly
        uint64_t bits = 0;       // an integer source, extended to 64 bits
        switch (e.srcCt) {
        case kF16: f = (double)(float)*(const half_t*)p; break;
        case kBF16: f = (double)__builtin_bit_cast(float, (uint32_t)*(const uint16_t*)p << 16); break;
        case kF32: f = (double)*(const float*)p; break;
        case kF64: f = *(const double*)p; break;
        case kS8: bits = (uint64_t)(int64_t) * (const int8_t*)p; break;
        case kU8: bits = *p; break;
        case kS16: bits = (uint64_t)(int64_t) * (const int16_t*)p; break;
        case kU16: bits = *(const uint16_t*)p; break;
        case kS32: bits = (uint64_t)(int64_t) * (const int32_t*)p; break;
        case kU32: bits = *(const uint32_t*)p; break;
        default: bits = *(const uint64_t*)p; break;
        }
        switch (e.dstCt) {
        case kF16:
            *(half_t*)q = srcFloat ? (e.srcCt == kF64 ? halfOfDouble(f) : (half_t)(float)f)
                                   : halfOfDouble(stickyDoubleOfInt(bits, srcUnsigned));
            break;
        case kF32:
            *(float*)q = srcFloat ? (float)f : (srcUnsigned ? (float)bits : (float)(int64_t)bits);
            break;
        case kBF16: {
            // one rounding to the 8 significant bits of bfloat16: through a float with a sticky last bit where the
            // source holds more than a float does (fp64, integers beyond 2^24)
            const double d = srcFloat ? f : stickyDoubleOfInt(bits, srcUnsigned);
            float x = (float)d;
            const double back = (double)x;
            if (back != d) {
                uint32_t u = __builtin_bit_cast(uint32_t, x);
                if (__builtin_fabs(back) > __builtin_fabs(d)) u -= 1u;
                x = __builtin_bit_cast(float, u | 1u);
            }
            *(bf16_t*)q = (bf16_t)x;
            break; }
        case kF64:
            *(double*)q = srcFloat ? f : (srcUnsigned ? (double)bits : (double)(int64_t)bits);
            break;
        case kS64:
            *(int64_t*)q = srcFloat ? (f != f ? 0 : (f >= 9223372036854775808.0 ? INT64_MAX : (f <= -9223372036854775808.0 ? INT64_MIN : (int64_t)f)))
                                    : (int64_t)bits;
            break;
        case kU64:
            *(uint64_t*)q = srcFloat ? (f != f || f <= 0.0 ? 0u : (f >= 18446744073709551616.0 ? UINT64_MAX : (uint64_t)f)) : bits;
            break;
        default: {
            const bool dstUnsigned = e.dstCt == kU8 || e.dstCt == kU16 || e.dstCt == kU32;
            uint32_t v;
            if (!srcFloat) v = (uint32_t)bits;
            else if (f != f) v = 0u;
            else if (dstUnsigned) v = f <= 0.0 ? 0u : (f >= 4294967296.0 ? UINT32_MAX : (uint32_t)f);
            else v = (uint32_t)(f >= 2147483648.0 ? INT32_MAX : (f <= -2147483648.0 ? INT32_MIN : (int32_t)f));
            if (dEsz == 1) *q = (uint8_t)v;
            else if (dEsz == 2) *(uint16_t*)q = (uint16_t)v;
            else *(uint32_t*)q = v;
            break;
        }
        }
    }
}

bool isCastType(int32_t ct);
bool isPlainType(int32_t ct)
{
    return ct == kF16 || ct == kF32 || ct == kF64 || ct == kS8 || ct == kU8 || ct == kS16 || ct == kU16 || ct == kS32 ||
           ct == kU32 || ct == kS64 || ct == kU64;
}

bool isCastType(int32_t ct) { return isPlainType(ct) || ct == kBF16; }      // conversions also serve bfloat16

bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

int currentCUs()
{
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
        n = 256;
    return n;
}

CvResult checkCommon(const char* who, int32_t op, int32_t elementType, int32_t n, uint32_t esz)
{
    if (op < 0 || op >= kOpCount) return failWith(CV_E_INVALID_ARG, "%s: unknown operator %d", who, op);
    if (elementType != CV_FLOAT16 && elementType != CV_FLOAT32)
        return failWith(CV_E_NOT_AVAILABLE, "%s: elementType %d with operator %d (every operator: FLOAT16, FLOAT32; arithmetic, min, max, "
                        "clamp: the integer types and FLOAT64, which also takes step and fma)", who, elementType, op);
    if (n <= 0) return failWith(CV_E_INVALID_ARG, "%s: n=%d", who, n);
    (void)esz;
    return CV_OK;
}

bool badOperand(const void* p, size_t stride, int32_t n, uint32_t batch, uint32_t esz)
{
    return !p || (uintptr_t)p % esz || stride % esz || (batch > 1 && stride < (size_t)n * esz);
}

} // namespace
} // namespace cv

extern "C" {

CV_API CvResult cvElementwise(void* stream, int32_t op, int32_t elementType, int32_t n, uint32_t batch,
                              const void* a, size_t aStride, const void* b, size_t bStride,
                              const void* c, size_t cStride, void* out, size_t outStride, float param)
{
    using namespace cv;
    const bool arith = isPlainType(elementType) && elementType != CV_FLOAT16 && elementType != CV_FLOAT32 && op >= 0 &&
                       op < kOpCount && arithOpFor(elementType, op);
    const uint32_t esz = arith ? elemSize(elementType) : elementType == CV_FLOAT32 ? 4u : 2u;
    CvResult rc = arith ? (n <= 0 ? failWith(CV_E_INVALID_ARG, "cvElementwise: n=%d", n) : CV_OK)
                        : checkCommon("cvElementwise", op, elementType, n, esz);
    if (CV_FAILED(rc)) return rc;
    if (batch == 0) return CV_OK;
    const int nOps = operandCount(op);
    if (badOperand(a, aStride, n, batch, esz) || badOperand(out, outStride, n, batch, esz) ||
        (nOps >= 2 && badOperand(b, bStride, n, batch, esz)) || (nOps >= 3 && badOperand(c, cStride, n, batch, esz)))
        return failWith(CV_E_INVALID_ARG, "cvElementwise: null, misaligned or overlapping-row operand (operator %d takes %d)", op, nOps);
    EwArgs e;
    memset(&e, 0, sizeof(e));
    e.a = (const uint8_t*)a; e.b = (const uint8_t*)b; e.c = (const uint8_t*)c; e.out = (uint8_t*)out;
    e.aStride = aStride; e.bStride = bStride; e.cStride = cStride; e.outStride = outStride;
    e.op = op; e.n = n; e.batch = batch;
    e.param = (op == kOpScale && elementType == CV_FLOAT16) ? (float)(_Float16)param : param;      // the scalar is of the element type
    const uint64_t total = (uint64_t)batch * (uint32_t)n;
    const size_t row = (size_t)n * esz;
    const bool dense = aStride == row && outStride == row && (nOps < 2 || bStride == row) && (nOps < 3 || cStride == row) &&
                       aligned16(a) && aligned16(out) && (nOps < 2 || aligned16(b)) && (nOps < 3 || aligned16(c)) &&
                       (total * esz) % 16 == 0;
    const uint32_t cap = (uint32_t)currentCUs() * 8u;
    if (arith) {
        const uint32_t blocks = (uint32_t)((total + 255) / 256 < cap ? (total + 255) / 256 : cap);
        noteKernel(false, "elementwiseArithKernel<type %d>", elementType);
        const dim3 g(blocks), t(256);
        hipStream_t st = (hipStream_t)stream;
        switch (elementType) {
        case CV_SINT8: hipLaunchKernelGGL(elementwiseArithKernel<int8_t>, g, t, 0, st, e); break;
        case CV_UINT8: hipLaunchKernelGGL(elementwiseArithKernel<uint8_t>, g, t, 0, st, e); break;
        case CV_SINT16: hipLaunchKernelGGL(elementwiseArithKernel<int16_t>, g, t, 0, st, e); break;
        case CV_UINT16: hipLaunchKernelGGL(elementwiseArithKernel<uint16_t>, g, t, 0, st, e); break;
        case CV_SINT32: hipLaunchKernelGGL(elementwiseArithKernel<int32_t>, g, t, 0, st, e); break;
        case CV_UINT32: hipLaunchKernelGGL(elementwiseArithKernel<uint32_t>, g, t, 0, st, e); break;
        case CV_SINT64: hipLaunchKernelGGL(elementwiseArithKernel<int64_t>, g, t, 0, st, e); break;
        case CV_UINT64: hipLaunchKernelGGL(elementwiseArithKernel<uint64_t>, g, t, 0, st, e); break;
        default: hipLaunchKernelGGL(elementwiseArithKernel<double>, g, t, 0, st, e); break;
        }
    } else if (dense) {
        const uint64_t pieces = total * esz / 16u;
        const uint32_t blocks = (uint32_t)((pieces + 255) / 256 < cap ? (pieces + 255) / 256 : cap);
        noteKernel(false, "elementwiseDenseKernel<%s>", esz == 2 ? "f16" : "f32");
        if (esz == 2) hipLaunchKernelGGL(elementwiseDenseKernel<half_t>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, e, pieces);
        else          hipLaunchKernelGGL(elementwiseDenseKernel<float>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, e, pieces);
    } else {
        const uint32_t blocks = (uint32_t)((total + 255) / 256 < cap ? (total + 255) / 256 : cap);
        noteKernel(false, "elementwiseKernel<%s>", esz == 2 ? "f16" : "f32");
        if (esz == 2) hipLaunchKernelGGL((elementwiseKernel<half_t, false>), dim3(blocks), dim3(256), 0, (hipStream_t)stream, e);
        else          hipLaunchKernelGGL((elementwiseKernel<float, false>), dim3(blocks), dim3(256), 0, (hipStream_t)stream, e);
    }
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess) return failWith(CV_E_INTERNAL_FAIL, "cvElementwise launch: %s", hipGetErrorString(err));
    return CV_OK;
}

CV_API CvResult cvVectorCast(void* stream, int32_t n, uint32_t batch, const void* src, size_t srcStride, int32_t srcType,
                             void* dst, size_t dstStride, int32_t dstType)
{
    using namespace cv;
    if (n <= 0) return failWith(CV_E_INVALID_ARG, "cvVectorCast: n=%d", n);
    if (!isCastType(srcType) || !isCastType(dstType))
        return failWith(CV_E_NOT_AVAILABLE, "cvVectorCast: from type %d to type %d (supported: FLOAT16/32/64, BFLOAT16 and the 8/16/32/64-bit integers)",
                        srcType, dstType);
    if (batch == 0) return CV_OK;
    if (badOperand(src, srcStride, n, batch, elemSize(srcType)) || badOperand(dst, dstStride, n, batch, elemSize(dstType)))
        return failWith(CV_E_INVALID_ARG, "cvVectorCast: null, misaligned or overlapping-row operand");
    CastArgs e;
    memset(&e, 0, sizeof(e));
    e.src = (const uint8_t*)src; e.dst = (uint8_t*)dst; e.srcStride = srcStride; e.dstStride = dstStride;
    e.srcCt = srcType; e.dstCt = dstType; e.n = n; e.batch = batch;
    const uint64_t total = (uint64_t)batch * (uint32_t)n;
    const uint32_t cap = (uint32_t)currentCUs() * 8u;
    const uint32_t blocks = (uint32_t)((total + 255) / 256 < cap ? (total + 255) / 256 : cap);
    noteKernel(false, "vectorCastKernel<%d -> %d>", srcType, dstType);
    hipLaunchKernelGGL(vectorCastKernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, e);
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess) return failWith(CV_E_INTERNAL_FAIL, "cvVectorCast launch: %s", hipGetErrorString(err));
    return CV_OK;
}

CV_API CvResult cvElementwiseBackward(void* stream, int32_t op, int32_t elementType, int32_t n, uint32_t batch,
                                      const void* a, size_t aStride, const void* b, size_t bStride,
                                      const void* c, size_t cStride, const void* dOut, size_t dOutStride,
                                      void* dA, size_t dAStride, void* dB, size_t dBStride,
                                      void* dC, size_t dCStride, float param)
{
    using namespace cv;
    const uint32_t esz = elementType == CV_FLOAT32 ? 4u : 2u;
    CvResult rc = checkCommon("cvElementwiseBackward", op, elementType, n, esz);
    if (CV_FAILED(rc)) return rc;
    if (batch == 0) return CV_OK;
    const int nOps = operandCount(op);
    if (badOperand(a, aStride, n, batch, esz) || badOperand(dOut, dOutStride, n, batch, esz) ||
        (nOps >= 2 && badOperand(b, bStride, n, batch, esz)) || (nOps >= 3 && badOperand(c, cStride, n, batch, esz)) ||
        (dA && badOperand(dA, dAStride, n, batch, esz)) || (dB && nOps >= 2 && badOperand(dB, dBStride, n, batch, esz)) ||
        (dC && nOps >= 3 && badOperand(dC, dCStride, n, batch, esz)))
        return failWith(CV_E_INVALID_ARG, "cvElementwiseBackward: null, misaligned or overlapping-row operand (operator %d takes %d)", op, nOps);
    EwArgs e;
    memset(&e, 0, sizeof(e));
    e.a = (const uint8_t*)a; e.b = (const uint8_t*)b; e.c = (const uint8_t*)c; e.dOut = (const uint8_t*)dOut;
    e.dA = (uint8_t*)dA; e.dB = (uint8_t*)dB; e.dC = (uint8_t*)dC;
    e.aStride = aStride; e.bStride = bStride; e.cStride = cStride; e.dOutStride = dOutStride;
    e.dAStride = dAStride; e.dBStride = dBStride; e.dCStride = dCStride;
    e.op = op; e.n = n; e.batch = batch;
    e.param = (op == kOpScale && elementType == CV_FLOAT16) ? (float)(_Float16)param : param;      // the scalar is of the element type
    const uint64_t total = (uint64_t)batch * (uint32_t)n;
    const uint32_t cap = (uint32_t)currentCUs() * 8u;
    const uint32_t blocks = (uint32_t)((total + 255) / 256 < cap ? (total + 255) / 256 : cap);
    noteKernel(false, "elementwiseKernel<%s,backward>", esz == 2 ? "f16" : "f32");
    if (esz == 2) hipLaunchKernelGGL((elementwiseKernel<half_t, true>), dim3(blocks), dim3(256), 0, (hipStream_t)stream, e);
    else          hipLaunchKernelGGL((elementwiseKernel<float, true>), dim3(blocks), dim3(256), 0, (hipStream_t)stream, e);
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess) return failWith(CV_E_INTERNAL_FAIL, "cvElementwiseBackward launch: %s", hipGetErrorString(err));
    return CV_OK;
}

} // extern "C"
