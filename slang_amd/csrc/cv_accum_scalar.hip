// cv_accum_scalar.hip -- coopVecOuterProductAccumulate / coopVecReduceSumAccumulate for the element types that
// have no matrix-instruction kernel: the scalar definition (source/slang/hlsl.meta.slang:33261-33315 and
// :33344-33352) over a batch, for every plain vector type T and every plain matrix interpretation:
//     product = a[i] * b[j]                      in T (integers wrap to T's width, floats round to T)
//     matrix[i][j] += cast<MatT>(product)        for every sample of the batch
//     buffer[i]    += v[i]                       in T (the reduce-sum form: b == 1, MatT == T)
// Integer destinations are exact modulo 2^width, so the batched sum equals the reference's sample-by-sample
// accumulation bit for bit.  Float destinations sum the cast products in fp32 (fp64 for Float64) in a fixed order
// and add the sum to the destination with one rounding, as the matrix-pipeline kernels do: deterministic, and within
// the float bar of the reference's own sample-by-sample order.  Not a tuned path.
#include "cv_device.h"
#include "cv_error.h"
#include "cv_kernels.h"
#include "cv_launch.h"

#include <type_traits>

namespace cv {
namespace {

enum : int { kSumU32 = 0, kSumF32 = 1, kSumU64 = 2, kSumF64 = 3 };
template <int ACC> struct SumOf;
template <> struct SumOf<kSumU32> { typedef uint32_t type; };
template <> struct SumOf<kSumF32> { typedef float type; };
template <> struct SumOf<kSumU64> { typedef uint64_t type; };
template <> struct SumOf<kSumF64> { typedef double type; };

__host__ __device__ inline int sumKindOf(int matCt)
{
    return matCt == kF16 || matCt == kF32 ? kSumF32 : matCt == kF64 ? kSumF64 : (matCt == kS64 || matCt == kU64) ? kSumU64 : kSumU32;
}
__host__ __device__ inline bool isUnsignedCt(int ct) { return ct == kU8 || ct == kU16 || ct == kU32 || ct == kU64; }
__host__ __device__ inline bool isFloatCt(int ct) { return ct == kF16 || ct == kF32 || ct == kF64; }

// a[i] * b[j] in T, then cast<MatT> of the product, delivered in the summation type of MatT.
// Integer T: the product wraps to T's width and is sign- or zero-extended from there; integer MatT narrower than the
// summation type is cut to its width when the sum is stored.  Float -> integer truncates towards zero.
template <int ACC, typename T>
__device__ __forceinline__ typename SumOf<ACC>::type productAs(const uint8_t* pa, const uint8_t* pb, bool matUnsigned)
{
    typedef typename SumOf<ACC>::type A;
    const T x = *(const T*)pa;
    const T y = pb ? *(const T*)pb : (T)1;
    if constexpr (std::is_integral<T>::value) {
        typedef typename std::make_unsigned<T>::type U;
        const T p = (T)(U)((U)x * (U)y);
        if constexpr (ACC == kSumU32 || ACC == kSumU64) {
            typedef typename std::conditional<ACC == kSumU32, int32_t, int64_t>::type S;
            return std::is_signed<T>::value ? (A)(S)p : (A)p;
        } else {
            return (A)p;
        }
    } else {
        T p;
        if constexpr (std::is_same<T, half_t>::value) p = (half_t)((float)x * (float)y);      // the exact product, rounded to half
        else p = x * y;
        if constexpr (ACC == kSumU32) return matUnsigned ? (A)(uint32_t)(float)p : (A)(int32_t)(float)p;
        else if constexpr (ACC == kSumU64) return matUnsigned ? (A)(uint64_t)(double)p : (A)(int64_t)(double)p;
        else return (A)p;
    }
}

struct OuterScalarArgs {
    const uint8_t* a; const uint8_t* b;          // b == nullptr: every b[j] is 1 (the reduce-sum form, n == 1)
    uint64_t aStride, bStride;
    int32_t m, n, tCt;
    uint32_t batch, chunks;
    uint8_t* mat;
    MatrixShape shape;
    uint64_t* partials;                          // [chunks][m * n] slots of 8 bytes
};

// grid (ceil(m*n / 256), chunks): a thread owns one element of the matrix and sums over its chunk of the batch
template <int ACC, typename T>
__global__ __launch_bounds__(256) void outerScalarKernel(const OuterScalarArgs o)
{
    typedef typename SumOf<ACC>::type A;
    const uint32_t e = blockIdx.x * 256u + threadIdx.x;
    if (e >= (uint32_t)(o.m * o.n)) return;
    const uint32_t i = e / (uint32_t)o.n, j = e % (uint32_t)o.n;
    const uint32_t per = (o.batch + o.chunks - 1) / o.chunks;
    const uint32_t s0 = blockIdx.y * per, s1 = s0 + per < o.batch ? s0 + per : o.batch;
    const bool matUnsigned = isUnsignedCt(o.shape.ct);
    A sum = 0;
    for (uint32_t s = s0; s < s1; ++s) {
        const uint8_t* pa = o.a + (size_t)s * o.aStride + (size_t)i * sizeof(T);
        const uint8_t* pb = o.b ? o.b + (size_t)s * o.bStride + (size_t)j * sizeof(T) : nullptr;
        sum = sum + productAs<ACC, T>(pa, pb, matUnsigned);
    }
    A* slot = (A*)(o.partials + (size_t)blockIdx.y * (size_t)(o.m * o.n) + e);
    *slot = sum;
}

// the chunks in ascending order, then destination += sum in the matrix type
template <int ACC>
__global__ __launch_bounds__(256) void outerScalarFinalKernel(const OuterScalarArgs o)
{
    typedef typename SumOf<ACC>::type A;
    const uint32_t e = blockIdx.x * 256u + threadIdx.x;
    if (e >= (uint32_t)(o.m * o.n)) return;
    A sum = 0;
    for (uint32_t c = 0; c < o.chunks; ++c) sum = sum + *(const A*)(o.partials + (size_t)c * (size_t)(o.m * o.n) + e);
    uint8_t* d = o.mat + elemOffset(o.shape, e / (uint32_t)o.n, e % (uint32_t)o.n);
    switch (o.shape.ct) {
    case kF16: *(half_t*)d = (half_t)((float)*(const half_t*)d + (float)sum); break;
    case kF32: *(float*)d = *(const float*)d + (float)sum; break;
    case kF64: *(double*)d = *(const double*)d + (double)sum; break;
    case kS8: case kU8: *d = (uint8_t)(*d + (uint8_t)sum); break;
    case kS16: case kU16: *(uint16_t*)d = (uint16_t)(*(const uint16_t*)d + (uint16_t)sum); break;
    case kS32: case kU32: *(uint32_t*)d = *(const uint32_t*)d + (uint32_t)sum; break;
    default: *(uint64_t*)d = *(const uint64_t*)d + (uint64_t)sum; break;
    }
}

template <int ACC>
void launchFirst(hipStream_t stream, const OuterScalarArgs& o, dim3 grid)
{
    const dim3 t(256);
    switch (o.tCt) {
    case kF16: hipLaunchKernelGGL((outerScalarKernel<ACC, half_t>), grid, t, 0, stream, o); break;
    case kF32: hipLaunchKernelGGL((outerScalarKernel<ACC, float>), grid, t, 0, stream, o); break;
    case kF64: hipLaunchKernelGGL((outerScalarKernel<ACC, double>), grid, t, 0, stream, o); break;
    case kS8: hipLaunchKernelGGL((outerScalarKernel<ACC, int8_t>), grid, t, 0, stream, o); break;
    case kU8: hipLaunchKernelGGL((outerScalarKernel<ACC, uint8_t>), grid, t, 0, stream, o); break;
    case kS16: hipLaunchKernelGGL((outerScalarKernel<ACC, int16_t>), grid, t, 0, stream, o); break;
    case kU16: hipLaunchKernelGGL((outerScalarKernel<ACC, uint16_t>), grid, t, 0, stream, o); break;
    case kS32: hipLaunchKernelGGL((outerScalarKernel<ACC, int32_t>), grid, t, 0, stream, o); break;
    case kU32: hipLaunchKernelGGL((outerScalarKernel<ACC, uint32_t>), grid, t, 0, stream, o); break;
    case kS64: hipLaunchKernelGGL((outerScalarKernel<ACC, int64_t>), grid, t, 0, stream, o); break;
    default: hipLaunchKernelGGL((outerScalarKernel<ACC, uint64_t>), grid, t, 0, stream, o); break;
    }
}

constexpr uint32_t kMaxChunks = 64;
constexpr uint32_t kSamplesPerChunk = 128;

uint32_t chunksFor(uint32_t batch)
{
    const uint32_t c = (batch + kSamplesPerChunk - 1) / kSamplesPerChunk;
    return c < 1 ? 1 : (c > kMaxChunks ? kMaxChunks : c);
}

} // namespace

bool isPlainComponent(int ct)
{
    return ct == kF16 || ct == kF32 || ct == kF64 || ct == kS8 || ct == kU8 || ct == kS16 || ct == kU16 || ct == kS32 ||
           ct == kU32 || ct == kS64 || ct == kU64;
}

size_t accumScalarWorkspaceBytes(int m, int n, uint32_t batch)
{
    return (size_t)chunksFor(batch) * (size_t)m * (size_t)n * sizeof(uint64_t);
}

// b == nullptr with n == 1: the reduce-sum form
hipError_t launchAccumScalar(hipStream_t stream, const uint8_t* a, uint64_t aStride, int m, const uint8_t* b, uint64_t bStride,
                             int n, int tCt, uint32_t batch, uint8_t* mat, const MatrixShape& shape, void* workspace)
{
    if (batch == 0) return hipSuccess;
    OuterScalarArgs o;
    o.a = a; o.b = b; o.aStride = aStride; o.bStride = bStride; o.m = m; o.n = n; o.tCt = tCt; o.batch = batch;
    o.chunks = chunksFor(batch); o.mat = mat; o.shape = shape; o.partials = (uint64_t*)workspace;
    const uint32_t blocks = ((uint32_t)(m * n) + 255u) / 256u;
    const int acc = sumKindOf(shape.ct);
    noteKernel(false, "outerScalarKernel<vectors %d, matrix %d, chunks=%u>", tCt, shape.ct, o.chunks);
    const dim3 g1(blocks, o.chunks), g2(blocks);
    switch (acc) {
    case kSumU32:
        launchFirst<kSumU32>(stream, o, g1);
        hipLaunchKernelGGL(outerScalarFinalKernel<kSumU32>, g2, dim3(256), 0, stream, o); break;
    case kSumF32:
        launchFirst<kSumF32>(stream, o, g1);
        hipLaunchKernelGGL(outerScalarFinalKernel<kSumF32>, g2, dim3(256), 0, stream, o); break;
    case kSumU64:
        launchFirst<kSumU64>(stream, o, g1);
        hipLaunchKernelGGL(outerScalarFinalKernel<kSumU64>, g2, dim3(256), 0, stream, o); break;
    default:
        launchFirst<kSumF64>(stream, o, g1);
        hipLaunchKernelGGL(outerScalarFinalKernel<kSumF64>, g2, dim3(256), 0, stream, o); break;
    }
    return hipGetLastError();
}

} // namespace cv
