// cv_accum_f32.hip -- batched coopVecOuterProductAccumulate and coopVecReduceSumAccumulate of fp32 vectors into an fp32
// destination, on the matrix pipeline of gfx950.
//
// The operators add a[i] * b[j] (reduce-sum: v[i]) of one thread to memory
// (source/slang/hlsl.meta.slang:33261-33315, :33344-33352); over a batch that is Mat[i][j] += sum_s a[s][i] * b[s][j].
// v_mfma_f32_16x16x4_f32 takes its operands the way the vectors lie in memory: lane 16*k + i supplies element i of sample
// k of a group of four samples (A: a row of the block, B: a column), so a fragment is one 4-byte load per lane with no
// transposition, and the batch is the instruction's k axis.  A workgroup of four waves keeps a block of up to 64 x 64
// fp32 sums in accumulators over its share of the batch; the waves are summed in LDS in a fixed order into one partial
// per workgroup, and a second kernel adds the partials in a fixed order to the destination ("+=", any layout): no atomics,
// bitwise reproducible.  Each product enters its sum through the instruction's fused multiply-add (the scalar definition
// rounds the product first: one sample gives the same bits, more samples differ within the float bar of the reference's own
// order-dependent sum).  The reduce-sum form is the outer product with b == 1 and one column.
#include "cv_device.h"
#include "cv_kernels.h"
#include "cv_error.h"

namespace cv {

namespace {

constexpr int kBlk = 64;                    // an output block is up to 64 x 64: TM x TN accumulator tiles of 16 x 16
constexpr int kPartialFloats = 16 * 256;
constexpr int kSteps = 4;                   // groups of four samples a wave has in flight: 16 samples per iteration

struct OuterF32Args {
    const uint8_t* a; const uint8_t* b;     // fp32 [batch][m], [batch][n]; b == nullptr: every b[j] is 1 (n == 1)
    uint64_t aStride, bStride;
    int32_t m, n;
    uint32_t batch;
    uint8_t* mat;
    MatrixShape shape;                      // m x n, FLOAT32, any layout
    float* partials;
};

// grid: x = persistent workgroups over the batch, y = output block (by * nbx + bx)
// ONES: the reduce-sum form (no b; a branch on the pointer inside the loop would make the waits for the loads conservative)
template <int TM, int TN, bool ONES>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void outerProductF32Kernel(const OuterF32Args o)
{
    __shared__ __attribute__((aligned(16))) float ldsRed[4 * 256];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, n = lane & 15;
    const int nbx = (o.n + kBlk - 1) / kBlk;
    const int by = blockIdx.y / nbx, bx = blockIdx.y % nbx;
    const int m0 = by * kBlk, n0 = bx * kBlk;

    floatx4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    // element of the vectors this lane supplies per tile (clamped to the vector: loads are unconditional, masked at use)
    uint32_t colA[TM], colB[TN];
    bool haveA[TM], haveB[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) { const int c = m0 + 16 * i + n; haveA[i] = c < o.m; colA[i] = (uint32_t)(haveA[i] ? c : o.m - 1) * 4u; }
#pragma unroll
    for (int j = 0; j < TN; ++j) { const int c = n0 + 16 * j + n; haveB[j] = c < o.n; colB[j] = (uint32_t)(haveB[j] ? c : o.n - 1) * 4u; }

    const uint32_t lastSample = o.batch - 1;
    const uint32_t numIters = (o.batch + 4 * kSteps - 1) / (4 * kSteps);
    const uint32_t iterStride = gridDim.x * 4;
    auto load = [&](float (&av)[kSteps][TM], float (&bv)[kSteps][TN], uint32_t it) {
#pragma unroll
        for (int u = 0; u < kSteps; ++u) {
            const uint32_t s = min(it * (4 * kSteps) + 4 * u + g, lastSample);
            const uint8_t* pa = o.a + (size_t)s * o.aStride;
#pragma unroll
            for (int i = 0; i < TM; ++i) av[u][i] = *(const float*)(pa + colA[i]);
            if constexpr (!ONES) {
                const uint8_t* pb = o.b + (size_t)s * o.bStride;
#pragma unroll
                for (int j = 0; j < TN; ++j) bv[u][j] = *(const float*)(pb + colB[j]);
            } else {
#pragma unroll
                for (int j = 0; j < TN; ++j) bv[u][j] = 1.f;
            }
        }
    };
    auto contract = [&](const float (&av)[kSteps][TM], const float (&bv)[kSteps][TN], uint32_t it) {
#pragma unroll
        for (int u = 0; u < kSteps; ++u) {
            const bool live = it * (4 * kSteps) + 4 * u + g <= lastSample;      // samples past the end contribute nothing
            float bq[TN];
#pragma unroll
            for (int j = 0; j < TN; ++j) bq[j] = (live && haveB[j]) ? bv[u][j] : 0.f;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const float aq = (live && haveA[i]) ? av[u][i] : 0.f;
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(aq, bq[j], acc[i][j], 0, 0, 0);
            }
        }
    };
    // the next iteration's loads are in flight while the current one is contracted
    {
        uint32_t it = blockIdx.x * 4 + wave;
        if (it < numIters) {
            float aCur[kSteps][TM], bCur[kSteps][TN], aNxt[kSteps][TM], bNxt[kSteps][TN];
            load(aCur, bCur, it);
            for (; it < numIters; it += iterStride) {
                const uint32_t i1 = it + iterStride;
                load(aNxt, bNxt, i1 < numIters ? i1 : it);
                contract(aCur, bCur, it);
#pragma unroll
                for (int u = 0; u < kSteps; ++u) {
#pragma unroll
                    for (int i = 0; i < TM; ++i) aCur[u][i] = aNxt[u][i];
#pragma unroll
                    for (int j = 0; j < TN; ++j) bCur[u][j] = bNxt[u][j];
                }
            }
        }
    }

    float* part = o.partials + ((size_t)blockIdx.y * gridDim.x + blockIdx.x) * kPartialFloats;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            *(floatx4*)&ldsRed[wave * 256 + lane * 4] = acc[i][j];
            __syncthreads();
            part[(i * TN + j) * 256 + threadIdx.x] =
                ((ldsRed[threadIdx.x] + ldsRed[256 + threadIdx.x]) + ldsRed[512 + threadIdx.x]) + ldsRed[768 + threadIdx.x];
            __syncthreads();
        }
}

// A workgroup owns 64 consecutive values of one block's partial (see sumPartials).  Value (tile, lane, r) of a partial is
// element (16 * (tile / tn) + 4 * (lane / 16) + r, 16 * (tile % tn) + lane % 16) of the block.
__global__ __launch_bounds__(64 * kReduceWaves) void outerF32ReduceKernel(const OuterF32Args o, uint32_t numPartials, uint32_t tn)
{
    __shared__ float red[kReduceWaves * 64];
    const uint32_t p = blockIdx.x * 64u + (threadIdx.x & 63u);
    float s;
    if (!sumPartials(o.partials + (size_t)blockIdx.y * numPartials * kPartialFloats + p, kPartialFloats, numPartials, true, red, s))
        return;
    const int nbx = (o.n + kBlk - 1) / kBlk;
    const int by = blockIdx.y / nbx, bx = blockIdx.y % nbx;
    const uint32_t tile = p >> 8, ln = (p >> 2) & 63u, r = p & 3u;
    const uint32_t row = (uint32_t)by * kBlk + 16u * (tile / tn) + 4u * (ln >> 4) + r;
    const uint32_t col = (uint32_t)bx * kBlk + 16u * (tile % tn) + (ln & 15u);
    if (row >= (uint32_t)o.m || col >= (uint32_t)o.n) return;
    float* d = (float*)(o.mat + elemOffset(o.shape, row, col));
    *d += s;
}

uint32_t gridX(uint32_t batch, int numCUs)
{
    // two workgroups per compute unit: eight waves whose loads overlap each other's matrix instructions
    const uint32_t iters = (batch + 4 * kSteps - 1) / (4 * kSteps), need = (iters + 3) / 4;
    const uint32_t cap = 2u * (uint32_t)numCUs;
    return need < cap ? (need ? need : 1) : cap;
}

} // namespace

size_t outerF32WorkspaceBytes(int m, int n, uint32_t batch, int numCUs)
{
    const size_t blocks = (size_t)((m + kBlk - 1) / kBlk) * ((n + kBlk - 1) / kBlk);
    return blocks * gridX(batch, numCUs) * kPartialFloats * sizeof(float);
}

// b == nullptr with n == 1: the reduce-sum form
hipError_t launchOuterProductF32(hipStream_t stream, const uint8_t* a, uint64_t aStride, int m, const uint8_t* b, uint64_t bStride,
                                 int n, uint32_t batch, uint8_t* mat, const MatrixShape& shape, void* workspace, int numCUs)
{
    if (batch == 0) return hipSuccess;
    if (shape.ct != kF32 || (!b && n != 1)) return hipErrorInvalidValue;
    OuterF32Args o;
    o.a = a; o.b = b; o.aStride = aStride; o.bStride = bStride; o.m = m; o.n = n; o.batch = batch;
    o.mat = mat; o.shape = shape; o.partials = (float*)workspace;
    const uint32_t gx = gridX(batch, numCUs);
    const uint32_t blocks = (uint32_t)((m + kBlk - 1) / kBlk) * (uint32_t)((n + kBlk - 1) / kBlk);
    // (a block of at most 16 rows or columns keeps one tile on that side)
    const int tm = m <= 16 ? 1 : 4, tn = n <= 16 ? 1 : 4;
    noteKernel(false, "outerProductF32Kernel<%dx%d tiles> + outerF32ReduceKernel", tm, tn);
    const dim3 grid(gx, blocks), block(256);
    if (!b)                      { if (tm == 4) hipLaunchKernelGGL((outerProductF32Kernel<4, 1, true>), grid, block, 0, stream, o);
                                   else         hipLaunchKernelGGL((outerProductF32Kernel<1, 1, true>), grid, block, 0, stream, o); }
    else if (tm == 4 && tn == 4) hipLaunchKernelGGL((outerProductF32Kernel<4, 4, false>), grid, block, 0, stream, o);
    else if (tm == 4)            hipLaunchKernelGGL((outerProductF32Kernel<4, 1, false>), grid, block, 0, stream, o);
    else if (tn == 4)            hipLaunchKernelGGL((outerProductF32Kernel<1, 4, false>), grid, block, 0, stream, o);
    else                         hipLaunchKernelGGL((outerProductF32Kernel<1, 1, false>), grid, block, 0, stream, o);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(outerF32ReduceKernel, dim3((uint32_t)(tm * tn * 256 / 64), blocks), dim3(64 * kReduceWaves), 0, stream, o, gx,
                       (uint32_t)tn);
    return hipGetLastError();
}

} // namespace cv
