// cv_matmul_scalar.hip -- coopVecMatMul[Add] for the type combinations that have no matrix instruction:
// 16- and 32-bit integer matrices or vectors, and mixed forms such as fp32 vectors against an int8
// matrix or fp16 vectors against an fp32 matrix.  The scalar definition (source/slang/hlsl.meta.slang:
// 32835-32912, bias :33043-33103) is evaluated as it is written, one thread per sample (also for the 64-bit types):
//     v[j] = cast<T>(input[j]);   r[i] = sum_j cast<T>(W[i][j]) * v[j]   (j ascending);   r[i] += cast<T>(bias[i])
// with T = int32/uint32/int64/uint64 in two's complement (exact, wraps like the reference), or T = float / double
// with every product and sum rounded to T in that order (no fused multiply-add), or T = half with the operands
// cast to half, products and sums in fp32 and one rounding of the result (the rule of the matrix-pipeline
// kernels).  The matrix block lives in LDS already cast to the accumulation type and is read as a broadcast.
#include "cv_device.h"
#include "cv_error.h"
#include "cv_kernels.h"
#include "cv_launch.h"

#include <type_traits>

namespace cv {
namespace {

// The accumulation type per result type T: two's-complement integers of T's width (signed and unsigned share
// their bits), float for half / float results, double for double.
enum : int { kAccI32 = 0, kAccF32 = 1, kAccI64 = 2, kAccF64 = 3 };
template <int ACC> struct AccOf;
template <> struct AccOf<kAccI32> { typedef uint32_t type; };
template <> struct AccOf<kAccF32> { typedef float type; };
template <> struct AccOf<kAccI64> { typedef uint64_t type; };
template <> struct AccOf<kAccF64> { typedef double type; };

// load<ct>(p) followed by __arithmetic_cast to the accumulation type.  Integer targets: sign or zero extension /
// truncation to the low bits, floats towards zero; `dstUnsigned` picks the unsigned float->integer conversion.
// Float targets: nearest even; `viaHalf` (T = half) rounds the operand to half first.
template <int ACC>
__device__ __forceinline__ typename AccOf<ACC>::type loadCast(const uint8_t* p, int ct, bool dstUnsigned, bool viaHalf)
{
    typedef typename AccOf<ACC>::type A;
    if constexpr (ACC == kAccI32 || ACC == kAccI64) {
        typedef typename std::conditional<ACC == kAccI32, int32_t, int64_t>::type S;
        switch (ct) {
        case kS8: return (A)(S) * (const int8_t*)p;
        case kU8: return (A) * p;
        case kS16: return (A)(S) * (const int16_t*)p;
        case kU16: return (A) * (const uint16_t*)p;
        case kS32: return (A)(S) * (const int32_t*)p;
        case kU32: return (A) * (const uint32_t*)p;
        case kS64: case kU64: return (A) * (const uint64_t*)p;
        case kF16: { const float f = (float)*(const half_t*)p; return dstUnsigned ? (A)f : (A)(S)f; }
        case kF32: { const float f = *(const float*)p; return dstUnsigned ? (A)f : (A)(S)f; }
        case kF64: { const double f = *(const double*)p; return dstUnsigned ? (A)f : (A)(S)f; }
        }
        return 0;
    } else {
        A f = 0;
        switch (ct) {
        case kF16: return (A)(float)*(const half_t*)p;
        case kF32: f = (A) * (const float*)p; break;
        case kF64: f = (A) * (const double*)p; break;
        case kS8: f = (A) * (const int8_t*)p; break;
        case kU8: f = (A) * p; break;
        case kS16: f = (A) * (const int16_t*)p; break;
        case kU16: f = (A) * (const uint16_t*)p; break;
        case kS32: f = (A) * (const int32_t*)p; break;
        case kU32: f = (A) * (const uint32_t*)p; break;
        case kS64: f = (A) * (const int64_t*)p; break;
        case kU64: f = (A) * (const uint64_t*)p; break;
        }
        if constexpr (ACC == kAccF32) return viaHalf ? (float)(half_t)f : f;       // T = half: cast<half>(x), nearest even
        else return f;
    }
}

struct ScalarArgs {
    MatMulArgs mm;
    uint32_t rowsPerBlock;      // matrix rows kept in LDS at once
};

constexpr int kScalarLdsBytes = 49152;      // of LDS for the matrix block
constexpr int kRowChunk = 8;                // output rows accumulated in registers at once

template <int ACC>
__global__ __launch_bounds__(256) void matmulScalarKernel(const ScalarArgs sa)
{
    typedef typename AccOf<ACC>::type A;
    constexpr bool IS_FLOAT = ACC == kAccF32 || ACC == kAccF64;
    const MatMulArgs& a = sa.mm;
    __shared__ __attribute__((aligned(8))) uint8_t ldsRaw[kScalarLdsBytes];
    A* ldsW = (A*)ldsRaw;
    const int m = a.m, k = a.k;
    const bool resHalf = a.outCt == kF16, resUnsigned = a.outCt == kU32 || a.outCt == kU64;
    const uint32_t inEsz = elemSize(a.inCt), outEsz = elemSize(a.outCt);
    const uint32_t biasEsz = a.bias ? elemSize(a.biasCt) : 0;

    for (int r0 = 0; r0 < m; r0 += (int)sa.rowsPerBlock) {
        const int rows = m - r0 < (int)sa.rowsPerBlock ? m - r0 : (int)sa.rowsPerBlock;
        __syncthreads();
        for (int e = threadIdx.x; e < rows * k; e += 256) {
            const int i = e / k, j = e % k;
            const uint8_t* p = a.mat + (a.transpose ? elemOffset(a.shape, (uint32_t)j, (uint32_t)(r0 + i))
                                                    : elemOffset(a.shape, (uint32_t)(r0 + i), (uint32_t)j));
            ldsW[e] = loadCast<ACC>(p, a.shape.ct, resUnsigned, resHalf);
        }
        __syncthreads();
        for (uint32_t s = blockIdx.x * 256u + threadIdx.x; s < a.batch; s += gridDim.x * 256u) {
            const uint8_t* x = a.in + (size_t)s * a.inStride;
            uint8_t* y = a.out + (size_t)s * a.outStride;
            for (int c0 = 0; c0 < rows; c0 += kRowChunk) {
                A acc[kRowChunk];
#pragma unroll
                for (int r = 0; r < kRowChunk; ++r) acc[r] = 0;
                for (int j = 0; j < k; ++j) {
                    const A v = loadCast<ACC>(x + (size_t)j * inEsz, a.inCt, resUnsigned, resHalf);
#pragma unroll
                    for (int r = 0; r < kRowChunk; ++r) {
                        const int row = c0 + r < rows ? c0 + r : rows - 1;
                        const A p = ldsW[row * k + j] * v;      // floats: a rounded product ...
                        acc[r] = acc[r] + p;                    // ... then a rounded sum (no contraction: -ffp-contract=off)
                    }
                }
#pragma unroll
                for (int r = 0; r < kRowChunk; ++r) {
                    const int i = r0 + c0 + r;
                    if (c0 + r >= rows) break;
                    uint8_t* o = y + (size_t)i * outEsz;
                    A z = acc[r];
                    if (a.bias) z = z + loadCast<ACC>(a.bias + (size_t)i * biasEsz, a.biasCt, resUnsigned, resHalf);
                    if constexpr (ACC == kAccF32) {
                        if (resHalf) {
                            half_t hz = (half_t)z;
                            if (a.act == kActRelu) hz = hz > (half_t)0.f ? hz : (half_t)0.f;
                            else if (a.act == kActLeakyRelu) { const half_t t = (half_t)(hz * (half_t)a.slope); hz = hz > t ? hz : t; }
                            if (a.accumulate) hz = (half_t)((float)*(const half_t*)o + (float)hz);
                            *(half_t*)o = hz;
                            continue;
                        }
                    }
                    if constexpr (IS_FLOAT) {
                        if (a.act == kActRelu) z = z > (A)0 ? z : (A)0;
                        else if (a.act == kActLeakyRelu) { const A t = z * (A)a.slope; z = z > t ? z : t; }
                    } else {
                        typedef typename std::conditional<ACC == kAccI32, int32_t, int64_t>::type S;
                        if (a.act == kActRelu && !resUnsigned) z = (S)z > 0 ? z : (A)0;
                    }
                    if (a.accumulate) z = *(const A*)o + z;
                    *(A*)o = z;
                }
            }
        }
    }
}

} // namespace

// hipErrorInvalidValue when k is beyond what LDS holds of one row
hipError_t launchMatMulScalar(hipStream_t stream, const MatMulArgs& a, int numCUs)
{
    if (a.batch == 0) return hipSuccess;
    const int acc = a.outCt == kF16 || a.outCt == kF32 ? kAccF32 : a.outCt == kF64 ? kAccF64
                  : (a.outCt == kS64 || a.outCt == kU64) ? kAccI64 : kAccI32;
    const int capacity = kScalarLdsBytes / ((acc == kAccI64 || acc == kAccF64) ? 8 : 4);
    if (a.k > capacity) return hipErrorInvalidValue;
    ScalarArgs sa;
    sa.mm = a;
    uint32_t rpb = (uint32_t)(capacity / a.k);
    if (rpb > (uint32_t)a.m) rpb = (uint32_t)a.m;
    if (rpb > kRowChunk) rpb = rpb / kRowChunk * kRowChunk;
    sa.rowsPerBlock = rpb;
    const uint32_t needed = (a.batch + 255u) / 256u;
    const uint32_t maxBlocks = (uint32_t)numCUs * 8u;
    const uint32_t blocks = needed < maxBlocks ? needed : maxBlocks;
    static const char* const names[4] = {"int32", "fp32-accumulate", "int64", "fp64"};
    noteKernel(false, "matmulScalarKernel<%s,in=%d,matrix=%d,out=%d,rows/block=%u>", names[acc], a.inCt, a.shape.ct, a.outCt, rpb);
    switch (acc) {
    case kAccI32: hipLaunchKernelGGL(matmulScalarKernel<kAccI32>, dim3(blocks), dim3(256), 0, stream, sa); break;
    case kAccF32: hipLaunchKernelGGL(matmulScalarKernel<kAccF32>, dim3(blocks), dim3(256), 0, stream, sa); break;
    case kAccI64: hipLaunchKernelGGL(matmulScalarKernel<kAccI64>, dim3(blocks), dim3(256), 0, stream, sa); break;
    default:      hipLaunchKernelGGL(matmulScalarKernel<kAccF64>, dim3(blocks), dim3(256), 0, stream, sa); break;
    }
    return hipGetLastError();
}

} // namespace cv
