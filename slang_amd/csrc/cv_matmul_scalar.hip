// cv_matmul_scalar.hip -- coopVecMatMul[Add] for the type combinations that have no matrix instruction:
// 16- and 32-bit integer matrices or vectors, and mixed forms such as fp32 vectors against an int8
// matrix or fp16 vectors against an fp32 matrix.  The scalar definition (source/slang/hlsl.meta.slang:
// 32835-32912, bias :33043-33103) is evaluated as it is written, one thread per sample:
//     v[j] = cast<T>(input[j]);   r[i] = sum_j cast<T>(W[i][j]) * v[j]   (j ascending);   r[i] += cast<T>(bias[i])
// with T = int32/uint32 in two's complement (exact, wraps like the reference), or T = float with every
// product and sum rounded to fp32 in that order (no fused multiply-add), or T = half with the operands
// cast to half, products and sums in fp32 and one rounding of the result (the rule of the matrix-pipeline
// kernels).  The matrix block lives in LDS already cast to the accumulation type and is read as a broadcast.
#include "cv_device.h"
#include "cv_error.h"
#include "cv_kernels.h"
#include "cv_launch.h"

namespace cv {
namespace {

// load<ct>(p) as an int32 bit pattern (8/16-bit sources sign- or zero-extended) or as a float
__device__ __forceinline__ int32_t loadAsInt(const uint8_t* p, int ct)
{
    switch (ct) {
    case kS8: return (int32_t) * (const int8_t*)p;
    case kU8: return (int32_t) * p;
    case kS16: return (int32_t) * (const int16_t*)p;
    case kU16: return (int32_t) * (const uint16_t*)p;
    case kS32: case kU32: return *(const int32_t*)p;
    case kF16: return (int32_t)(float)*(const half_t*)p;      // __arithmetic_cast<int>(half): towards zero
    case kF32: return (int32_t) * (const float*)p;
    }
    return 0;
}
__device__ __forceinline__ uint32_t loadAsUint(const uint8_t* p, int ct)
{
    switch (ct) {
    case kF16: return (uint32_t)(float)*(const half_t*)p;
    case kF32: return (uint32_t) * (const float*)p;
    }
    return (uint32_t)loadAsInt(p, ct);       // integers: the same bits modulo 2^32
}
__device__ __forceinline__ float loadAsFloat(const uint8_t* p, int ct, bool viaHalf)
{
    float f;
    switch (ct) {
    case kF16: return (float)*(const half_t*)p;
    case kF32: f = *(const float*)p; break;
    case kU32: f = (float)*(const uint32_t*)p; break;
    default: f = (float)loadAsInt(p, ct); break;
    }
    return viaHalf ? (float)(half_t)f : f;       // T = half: cast<half>(x), nearest even
}

struct ScalarArgs {
    MatMulArgs mm;
    uint32_t rowsPerBlock;      // matrix rows kept in LDS at once
};

constexpr int kScalarLdsElems = 12288;      // 48 KB of 4-byte elements
constexpr int kRowChunk = 8;                // output rows accumulated in registers at once

template <bool IS_FLOAT>
__global__ __launch_bounds__(256) void matmulScalarKernel(const ScalarArgs sa)
{
    const MatMulArgs& a = sa.mm;
    __shared__ uint32_t ldsW[kScalarLdsElems];
    const int m = a.m, k = a.k;
    const bool resHalf = a.outCt == kF16, resUnsigned = a.outCt == kU32;
    const uint32_t inEsz = elemSize(a.inCt), outEsz = elemSize(a.outCt);
    const uint32_t biasEsz = a.bias ? elemSize(a.biasCt) : 0;

    for (int r0 = 0; r0 < m; r0 += (int)sa.rowsPerBlock) {
        const int rows = m - r0 < (int)sa.rowsPerBlock ? m - r0 : (int)sa.rowsPerBlock;
        __syncthreads();
        for (int e = threadIdx.x; e < rows * k; e += 256) {
            const int i = e / k, j = e % k;
            const uint8_t* p = a.mat + (a.transpose ? elemOffset(a.shape, (uint32_t)j, (uint32_t)(r0 + i))
                                                    : elemOffset(a.shape, (uint32_t)(r0 + i), (uint32_t)j));
            if constexpr (IS_FLOAT) ldsW[e] = __builtin_bit_cast(uint32_t, loadAsFloat(p, a.shape.ct, resHalf));
            else ldsW[e] = resUnsigned ? loadAsUint(p, a.shape.ct) : (uint32_t)loadAsInt(p, a.shape.ct);
        }
        __syncthreads();
        for (uint32_t s = blockIdx.x * 256u + threadIdx.x; s < a.batch; s += gridDim.x * 256u) {
            const uint8_t* x = a.in + (size_t)s * a.inStride;
            uint8_t* y = a.out + (size_t)s * a.outStride;
            for (int c0 = 0; c0 < rows; c0 += kRowChunk) {
                float accF[kRowChunk];
                uint32_t accI[kRowChunk];
#pragma unroll
                for (int r = 0; r < kRowChunk; ++r) { accF[r] = 0.f; accI[r] = 0u; }
                for (int j = 0; j < k; ++j) {
                    const uint8_t* xp = x + (size_t)j * inEsz;
                    if constexpr (IS_FLOAT) {
                        const float v = loadAsFloat(xp, a.inCt, resHalf);
#pragma unroll
                        for (int r = 0; r < kRowChunk; ++r) {
                            const int row = c0 + r < rows ? c0 + r : rows - 1;
                            const float p = __builtin_bit_cast(float, ldsW[row * k + j]) * v;     // rounded product ...
                            accF[r] = accF[r] + p;                                                 // ... then rounded sum
                        }
                    } else {
                        const uint32_t v = resUnsigned ? loadAsUint(xp, a.inCt) : (uint32_t)loadAsInt(xp, a.inCt);
#pragma unroll
                        for (int r = 0; r < kRowChunk; ++r) {
                            const int row = c0 + r < rows ? c0 + r : rows - 1;
                            accI[r] += ldsW[row * k + j] * v;
                        }
                    }
                }
#pragma unroll
                for (int r = 0; r < kRowChunk; ++r) {
                    const int i = r0 + c0 + r;
                    if (c0 + r >= rows) break;
                    uint8_t* o = y + (size_t)i * outEsz;
                    if constexpr (IS_FLOAT) {
                        float z = accF[r];
                        if (a.bias) z = z + loadAsFloat(a.bias + (size_t)i * biasEsz, a.biasCt, resHalf);
                        if (resHalf) {
                            half_t hz = (half_t)z;
                            if (a.act == kActRelu) hz = hz > (half_t)0.f ? hz : (half_t)0.f;
                            else if (a.act == kActLeakyRelu) { const half_t t = (half_t)(hz * (half_t)a.slope); hz = hz > t ? hz : t; }
                            if (a.accumulate) hz = (half_t)((float)*(const half_t*)o + (float)hz);
                            *(half_t*)o = hz;
                        } else {
                            if (a.act == kActRelu) z = z > 0.f ? z : 0.f;
                            else if (a.act == kActLeakyRelu) { const float t = z * a.slope; z = z > t ? z : t; }
                            if (a.accumulate) z = *(const float*)o + z;
                            *(float*)o = z;
                        }
                    } else {
                        uint32_t z = accI[r];
                        if (a.bias) z += resUnsigned ? loadAsUint(a.bias + (size_t)i * biasEsz, a.biasCt)
                                                     : (uint32_t)loadAsInt(a.bias + (size_t)i * biasEsz, a.biasCt);
                        if (a.act == kActRelu && !resUnsigned) z = (int32_t)z > 0 ? z : 0u;
                        if (a.accumulate) z += *(const uint32_t*)o;
                        *(uint32_t*)o = z;
                    }
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
    if (a.k > kScalarLdsElems) return hipErrorInvalidValue;
    ScalarArgs sa;
    sa.mm = a;
    uint32_t rpb = (uint32_t)(kScalarLdsElems / a.k);
    if (rpb > (uint32_t)a.m) rpb = (uint32_t)a.m;
    if (rpb > kRowChunk) rpb = rpb / kRowChunk * kRowChunk;
    sa.rowsPerBlock = rpb;
    const bool isFloat = a.outCt == kF16 || a.outCt == kF32;
    const uint32_t needed = (a.batch + 255u) / 256u;
    const uint32_t maxBlocks = (uint32_t)numCUs * 8u;
    const uint32_t blocks = needed < maxBlocks ? needed : maxBlocks;
    noteKernel(false, "matmulScalarKernel<%s,in=%d,matrix=%d,out=%d,rows/block=%u>", isFloat ? "fp32-accumulate" : "int32", a.inCt,
               a.shape.ct, a.outCt, rpb);
    if (isFloat) hipLaunchKernelGGL(matmulScalarKernel<true>, dim3(blocks), dim3(256), 0, stream, sa);
    else hipLaunchKernelGGL(matmulScalarKernel<false>, dim3(blocks), dim3(256), 0, stream, sa);
    return hipGetLastError();
}

} // namespace cv
