// cv_permuto_wide.h -- permutohedral encoding in front of the 32-sample-tile forward kernel.
//
// The decoder networks of hash-grid encoders (hidden layers of 32 or 64 ReLU units, up to 32 outputs) are what
// mlpWide16Body (cv_mlp_wide16.h) runs on v_mfma_f32_32x32x16_f16 with the weights in registers.  Here its first-layer
// operands do not come from memory: lane (n, h) of a tile evaluates PermutoEncoder::encode
// (source/standard-modules/neural/permuto-encoder.slang:240-337) for the levels whose features its k-slots hold --
// features 2*CE*s + CE*h .. + CE-1 of k-step s, CE = 4 (8 or 16 inputs) or 8 (32 inputs), the chunks the single-layer
// operator deals out -- from level records and a feature table held in LDS.  Per level the arithmetic is that of
// cvPermutoEncode, per layer that of cvMlpForward: same bits as the two calls.  While one wave of a SIMD encodes
// (vector ALU), the other one runs its layers (matrix pipeline).
#pragma once
#include "cv_mlp_wide16.h"
#include "cv_permuto_impl.h"

namespace cv {
namespace {

template <int K0, int D, int F>
struct Wide16PermutoFront {
    struct Input { half_t pos[2][D]; };
    const uint8_t* pos; uint64_t posStride;
    const CvPermutoLevelInfo* levels;      // in LDS
    const half_t* table;                   // in LDS
    float maxLevel;
    __device__ __forceinline__ Input load(uint32_t p, int n, int, uint32_t lastSample) const
    {
        Input x;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            uint32_t s = (2u * p + (uint32_t)j) * 32u + (uint32_t)n;
            s = s < lastSample ? s : lastSample;
#pragma unroll
            for (int d = 0; d < D; ++d) x.pos[j][d] = ((const half_t*)(pos + (uint64_t)s * posStride))[d];
        }
        return x;
    }
    template <int NS>
    __device__ __forceinline__ void operands(const Input& x, uint32_t (&B)[2][NS][4], int, int h) const
    {
        constexpr int S0 = K0 == 8 ? 1 : 2, CE = K0 == 32 ? 8 : 4, PER = CE / F;      // k-steps; features and levels per chunk
        static_assert(CE % F == 0, "a lane's chunk holds whole table entries");
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            float p[D];
#pragma unroll
            for (int d = 0; d < D; ++d) p[d] = (float)x.pos[j][d];
#pragma unroll
            for (int s = 0; s < S0; ++s) {
                uint32_t v[4] = {0u, 0u, 0u, 0u};
#pragma unroll
                for (int c = 0; c < PER; ++c) {
                    const int level = (2 * s + h) * PER + c;
                    const auto e = permutoEncodeEntry<half_t, D, F>(p, levels[level], table, maxLevel);
#pragma unroll
                    for (int f = 0; f < F; ++f) {
                        const int q = c * F + f;
                        v[q / 2] |= (uint32_t)__builtin_bit_cast(uint16_t, (half_t)e[f]) << (16 * (q & 1));
                    }
                }
#pragma unroll
                for (int d = 0; d < 4; ++d) B[j][s][d] = v[d];
            }
        }
    }
};

struct PermutoWideArgs {
    MlpArgs mlp;
    CvPermutoDesc desc;
    const uint8_t* pos; uint64_t posStride;
    const uint8_t* table;
    uint32_t tableElems;
};

constexpr uint32_t kWideLevelBytes = CV_PERMUTO_MAX_LEVELS * sizeof(CvPermutoLevelInfo);

template <int H, int NH, int K0, int WAVES, int D, int F>
__global__ __launch_bounds__(64 * WAVES) void permutoWide16Kernel(const PermutoWideArgs pa)
{
    typedef typename PermutoEntry<half_t, F>::type Entry;
    extern __shared__ __attribute__((aligned(16))) uint8_t dyn[];
    {
        const uint32_t* src = (const uint32_t*)pa.desc.levelInfo;
        for (uint32_t i = threadIdx.x; i < pa.desc.maxLevels * (uint32_t)(sizeof(CvPermutoLevelInfo) / 4); i += blockDim.x) ((uint32_t*)dyn)[i] = src[i];
        const Entry* t = (const Entry*)pa.table;
        Entry* dst = (Entry*)(dyn + kWideLevelBytes);
        for (uint32_t i = threadIdx.x; i < pa.tableElems / (uint32_t)F; i += blockDim.x) dst[i] = t[i];
    }
    // (the body synchronises the workgroup after it has staged the weights, before any wave encodes)
    const Wide16PermutoFront<K0, D, F> front{pa.pos, pa.posStride, (const CvPermutoLevelInfo*)dyn, (const half_t*)(dyn + kWideLevelBytes), pa.desc.maxLevel};
    mlpWide16Body<H, NH, K0, WAVES, true>(pa.mlp, front);
}

template <int H, int NH, int K0, int D, int F>
hipError_t launchPermutoWide16Shape(hipStream_t stream, const PermutoWideArgs& pa, int numCUs)
{
    // waves per workgroup (= per compute unit) as the registers allow; with two or more per SIMD one encodes while another
    // is in the matrix pipeline.  The build fails if an instantiation spills.
    constexpr int WAVES = H == 1 ? 16 : (NH == 1 ? 12 : 8);
    auto kernel = permutoWide16Kernel<H, NH, K0, WAVES, D, F>;
    // LDS the kernel declares itself (weights in operand order, biases): a property of the instantiation, asked once
    static const size_t staticLds = [&]() -> size_t {
        hipFuncAttributes attr;
        return hipFuncGetAttributes(&attr, (const void*)kernel) == hipSuccess ? attr.sharedSizeBytes : (size_t)160 * 1024;
    }();
    const size_t dynBytes = kWideLevelBytes + (size_t)pa.tableElems * 2;
    if (staticLds + dynBytes > 160 * 1024) return hipErrorInvalidValue;      // the table does not fit beside the weights
    hipError_t e = allowDynamicLds<permutoWide16Kernel<H, NH, K0, WAVES, D, F>>((int)dynBytes);
    if (e != hipSuccess) return e;
    const uint32_t numPairs = ((pa.mlp.batch + 31u) / 32u + 1u) / 2u;
    const uint32_t blocks = numPairs < (uint32_t)numCUs ? numPairs : (uint32_t)numCUs;
    noteKernel(false, "permutoWide16Kernel<D=%d,F=%d,32x32x16,inputs=%d,hidden=%dx%d,waves=%d>", D, F, K0, NH, 32 * H, WAVES);
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(64 * WAVES), dynBytes, stream, pa);
    return hipGetLastError();
}

// all shapes of one input width (one translation unit each); hipErrorInvalidValue for the others
template <int K0>
hipError_t launchPermutoWide16K(hipStream_t stream, const PermutoWideArgs& pa, int numCUs, int H, int NH)
{
    const int D = pa.desc.dimensions, F = pa.desc.featureDimensionPerEntry;
#define CV_PW(h_, nh_, d_, f_) if (H == h_ && NH == nh_ && D == d_ && F == f_) return launchPermutoWide16Shape<h_, nh_, K0, d_, f_>(stream, pa, numCUs);
#define CV_PW_D(h_, nh_) CV_PW(h_, nh_, 2, 2) CV_PW(h_, nh_, 3, 2) CV_PW(h_, nh_, 4, 2)
    CV_PW_D(1, 1) CV_PW_D(1, 2) CV_PW_D(2, 1) CV_PW_D(2, 2)
#undef CV_PW_D
#undef CV_PW
    return hipErrorInvalidValue;
}

} // namespace
} // namespace cv
