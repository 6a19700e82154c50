// cv_accum.hip -- batched coopVecOuterProductAccumulate and coopVecReduceSumAccumulate for gfx950.
//
// The reference operators add one thread's contribution to memory atomically
// (source/slang/hlsl.meta.slang:33200-33224 `atomicAdd(matrix[i][j], a[i]*b[j])`, :33318-33326
// `atomicAdd(dest[i], v[i])`; CPU fallback :33261-33315, :33344-33352).  Over a batch that is
//     Mat[i][j] += sum_s a[s][i] * b[s][j]          buf[i] += sum_s v[s][i]
// which is computed here without atomics:
//   - outer product: both operands are loaded as "S" fragments (lane%16 = sample), turned exactly
//     into "F" fragments (lane%16 = feature, samples on the MFMA k axis) by an MFMA against a 0/1
//     selection matrix, and contracted over the batch with v_mfma_f32_16x16x32_f16 into fp32
//     accumulators held for the lifetime of the wave;
//   - reduce-sum: per-lane fp32 running sums;
//   - the four waves of a workgroup are summed in LDS in a fixed order into one partial per
//     workgroup (in the caller's workspace), and a second kernel adds the partials in a fixed
//     order to the destination ("+=", any matrix layout, fp16 or fp32): bitwise reproducible.
#include "cv_device.h"
#include "cv_kernels.h"
#include "cv_error.h"

namespace cv {

namespace {

constexpr int kBlk = 64;                 // an output block is 64 x 64 (4 x 4 accumulator tiles)
constexpr int kOuterPartialFloats = 16 * 256;

__device__ __forceinline__ void loadQuarter(uint32_t (&dst)[8], const uint8_t* row, int colBase, int cols, bool aligned16)
{
    // 16 halfs starting at column colBase (clipped to `cols`), zero padded
    const int valid = min(16, max(cols - colBase, 0));
    const uint8_t* p = row + (size_t)colBase * 2;
    if (valid == 16 && aligned16) {
        const u32x4 v0 = *(const u32x4*)p, v1 = *(const u32x4*)(p + 16);
        dst[0] = v0.x; dst[1] = v0.y; dst[2] = v0.z; dst[3] = v0.w;
        dst[4] = v1.x; dst[5] = v1.y; dst[6] = v1.z; dst[7] = v1.w;
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            uint32_t v = 0;
            if (2 * i < valid) v = *(const uint16_t*)(p + 4 * i);
            if (2 * i + 1 < valid) v |= (uint32_t)*(const uint16_t*)(p + 4 * i + 2) << 16;
            dst[i] = v;
        }
    }
}

// grid: x = persistent workgroups over the batch, y = output block (by * nbx + bx)
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void outerProductKernel(const OuterArgs a)
{
    typedef F16Mma Mma;
    __shared__ __attribute__((aligned(16))) float ldsRed[4 * 256];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, n = lane & 15;
    const int nbx = (a.n + kBlk - 1) / kBlk;
    const int by = blockIdx.y / nbx, bx = blockIdx.y % nbx;
    const int m0 = by * kBlk, n0 = bx * kBlk;            // first row / column of this block

    uint32_t Isel[2][4];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const int s0 = 4 * h + (lane & 3);
            const bool mine = g == (n >> 2);
            Isel[h][d] = ((mine && s0 == 2 * d) ? 0x3C00u : 0u) | (((mine && s0 == 2 * d + 1) ? 0x3C00u : 0u) << 16);
        }
    auto toF = [&](const uint32_t* s0, const uint32_t* s1, int h, uint32_t* frag) {
        typedef float floatx2 __attribute__((ext_vector_type(2)));
        const floatx4 z = {0.f, 0.f, 0.f, 0.f};
        const floatx4 t0 = Mma::mma(s0, Isel[h], z), t1 = Mma::mma(s1, Isel[h], z);
        frag[0] = __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{t0[0], t0[1]}, halfx2));
        frag[1] = __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{t0[2], t0[3]}, halfx2));
        frag[2] = __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{t1[0], t1[1]}, halfx2));
        frag[3] = __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{t1[2], t1[3]}, halfx2));
    };

    floatx4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    const uint32_t numTiles = (a.batch + 31) / 32;
    const uint32_t lastSample = a.batch - 1;
    const uint32_t tileStride = gridDim.x * 4;
    // S fragments of a tile of 32 samples: lane group g owns columns [16g, 16g+16) of the block, as
    // two 8-slot fragments per 16-sample half
    auto loadTile = [&](uint32_t (&aS)[2][8], uint32_t (&bS)[2][8], uint32_t tile) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t sc = min(tile * 32 + 16 * j + n, lastSample);
            loadQuarter(aS[j], a.a + (size_t)sc * a.aStride, m0 + 16 * g, a.m, a.aAlign >= 16u);
            loadQuarter(bS[j], a.b + (size_t)sc * a.bStride, n0 + 16 * g, a.n, a.bAlign >= 16u);
        }
    };
    auto compute = [&](uint32_t (&aS)[2][8], const uint32_t (&bS)[2][8], uint32_t tile) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
            if (tile * 32 + 16 * j + n > lastSample) {      // samples past the end contribute nothing
#pragma unroll
                for (int i = 0; i < 8; ++i) aS[j][i] = 0u;
            }
        uint32_t bF[4][4];
#pragma unroll
        for (int e = 0; e < 4; ++e) toF(&bS[0][4 * (e / 2)], &bS[1][4 * (e / 2)], e & 1, bF[e]);
#pragma unroll
        for (int eo = 0; eo < 4; ++eo) {
            uint32_t aF[4];
            toF(&aS[0][4 * (eo / 2)], &aS[1][4 * (eo / 2)], eo & 1, aF);
#pragma unroll
            for (int ei = 0; ei < 4; ++ei) acc[eo][ei] = Mma::mma(aF, bF[ei], acc[eo][ei]);
        }
    };
    // the next tile's loads are in flight while the current one is contracted
    {
        uint32_t tile = blockIdx.x * 4 + wave;
        if (tile < numTiles) {
            uint32_t aCur[2][8], bCur[2][8], aNxt[2][8], bNxt[2][8];
            loadTile(aCur, bCur, tile);
            for (; tile < numTiles; tile += tileStride) {
                const uint32_t t1 = tile + tileStride;
                loadTile(aNxt, bNxt, t1 < numTiles ? t1 : tile);
                compute(aCur, bCur, tile);
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int i = 0; i < 8; ++i) { aCur[j][i] = aNxt[j][i]; bCur[j][i] = bNxt[j][i]; }
            }
        }
    }

    float* part = a.partials + ((size_t)blockIdx.y * gridDim.x + blockIdx.x) * kOuterPartialFloats;
#pragma unroll
    for (int eo = 0; eo < 4; ++eo)
#pragma unroll
        for (int ei = 0; ei < 4; ++ei) {
            *(floatx4*)&ldsRed[wave * 256 + lane * 4] = acc[eo][ei];
            __syncthreads();
            part[(eo * 4 + ei) * 256 + threadIdx.x] =
                ((ldsRed[threadIdx.x] + ldsRed[256 + threadIdx.x]) + ldsRed[512 + threadIdx.x]) + ldsRed[768 + threadIdx.x];
            __syncthreads();
        }
}

// A workgroup owns 64 consecutive values of one block's partial (see sumPartials).
__global__ __launch_bounds__(64 * kReduceWaves) void outerReduceKernel(const OuterArgs a, uint32_t numPartials)
{
    __shared__ float red[kReduceWaves * 64];
    const uint32_t p = blockIdx.x * 64u + (threadIdx.x & 63u);   // index inside one block's partial
    float s;
    if (!sumPartials(a.partials + (size_t)blockIdx.y * numPartials * kOuterPartialFloats + p, kOuterPartialFloats,
                     numPartials, true, red, s)) return;
    const int nbx = (a.n + kBlk - 1) / kBlk;
    const int by = blockIdx.y / nbx, bx = blockIdx.y % nbx;
    const uint32_t tile = p >> 8, ln = (p >> 2) & 63u, r = p & 3u;
    const uint32_t eo = tile >> 2, ei = tile & 3u, gq = ln >> 4, qi = ln & 15u;
    // F tile e, column q  <->  feature (q/4)*16 + 4e + q%4 of the block (see cv_train_impl.h)
    const uint32_t row = (uint32_t)by * kBlk + gq * 16u + 4u * eo + r;
    const uint32_t col = (uint32_t)bx * kBlk + (qi >> 2) * 16u + 4u * ei + (qi & 3u);
    if (row >= (uint32_t)a.m || col >= (uint32_t)a.n) return;
    uint8_t* d = a.mat + elemOffset(a.shape, row, col);
    if (a.shape.ct == kF32) *(float*)d += s;
    else *(half_t*)d = (half_t)((float)*(half_t*)d + s);
}

// ---- reduce-sum -----------------------------------------------------------------------------
// lane (g,n) sums columns [g*CPL, (g+1)*CPL) of samples n, n+16, ...; CPL = ceil(N/4) rounded to 2
constexpr int kMaxReduceCols = 256;           // 64 per lane group

__global__ __launch_bounds__(256) void reduceSumKernel(const ReduceSumArgs a)
{
    __shared__ float ldsRed[4 * 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, n = lane & 15;
    const int cpl = a.colsPerGroup;           // multiple of 2, <= 64
    float acc[64];
#pragma unroll
    for (int i = 0; i < 64; ++i) acc[i] = 0.f;
    const int colBase = g * cpl;
    const int valid = min(cpl, max(a.n - colBase, 0));
    const uint32_t numTiles = (a.batch + 15) / 16;
    for (uint32_t tile = blockIdx.x * 4 + wave; tile < numTiles; tile += gridDim.x * 4) {
        const uint32_t s = tile * 16 + n;
        if (s >= a.batch) continue;
        const uint8_t* p = a.v + (size_t)s * a.vStride + (size_t)colBase * 2;
#pragma unroll
        for (int i = 0; i < 64; ++i)
            if (i < valid) acc[i] += (float)*(const half_t*)(p + 2 * i);
    }
    // sum over the 16 sample lanes and the 4 waves, column by column, in a fixed order
    float* part = a.partials + (size_t)blockIdx.x * kMaxReduceCols;
#pragma unroll
    for (int i = 0; i < 64; ++i) {
        if (i < cpl) {      // uniform; every acc[] index stays a compile-time constant
            ldsRed[wave * 64 + lane] = acc[i];
            __syncthreads();
            if (threadIdx.x < 4) {
                float s = 0.f;
                for (int w = 0; w < 4; ++w)
                    for (int k = 0; k < 16; ++k) s += ldsRed[w * 64 + threadIdx.x * 16 + k];
                const int col = threadIdx.x * cpl + i;
                if (col < a.n) part[col] = s;
            }
            __syncthreads();
        }
    }
}

// Streaming form for rows of whole 16-byte chunks (n % 8 == 0, 16-byte aligned base and stride): a row
// is C = n/8 chunks; LP = C rounded up to a power of two lanes share a row, a wave covers 64/LP rows
// per load, and every lane keeps eight fp32 sums for the eight columns of its chunk.  With a dense
// batch (stride = 2n) consecutive lanes read consecutive 16-byte pieces of memory.
constexpr int kRsUnroll = 8;
__global__ __launch_bounds__(256) void reduceSumStreamKernel(const ReduceSumArgs a, uint32_t lanesPerRow)
{
    __shared__ __attribute__((aligned(16))) float ldsRed[4 * 64 * 8];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t chunks = (uint32_t)a.n / 8u;
    const uint32_t rowsPerLoad = 64u / lanesPerRow;
    const uint32_t r = lane / lanesPerRow, c = lane % lanesPerRow;
    const bool active = c < chunks;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
    const uint32_t span = rowsPerLoad * kRsUnroll;                 // rows a wave takes per iteration
    const uint8_t* base = a.v + (size_t)c * 16u;
    for (uint64_t row0 = (uint64_t)(blockIdx.x * 4u + wave) * span; row0 < a.batch; row0 += (uint64_t)gridDim.x * 4u * span) {
        u32x4 v[kRsUnroll];
#pragma unroll
        for (int u = 0; u < kRsUnroll; ++u) {
            const uint64_t s = row0 + (uint64_t)u * rowsPerLoad + r;
            v[u] = u32x4{0u, 0u, 0u, 0u};
            if (active && s < a.batch) v[u] = loadStream16(base + s * a.vStride);
        }
#pragma unroll
        for (int u = 0; u < kRsUnroll; ++u) {
            const uint32_t dw[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const halfx2 h = __builtin_bit_cast(halfx2, dw[d]);
                acc[2 * d] += (float)h.x;
                acc[2 * d + 1] += (float)h.y;
            }
        }
    }
    // workgroup partial per column: rows of the wave, then the four waves, in a fixed order
#pragma unroll
    for (int i = 0; i < 8; ++i) ldsRed[(wave * 64 + lane) * 8 + i] = acc[i];
    __syncthreads();
    const uint32_t col = threadIdx.x;
    if (col < (uint32_t)a.n) {
        float s = 0.f;
        for (uint32_t w = 0; w < 4; ++w)
            for (uint32_t rr = 0; rr < rowsPerLoad; ++rr) s += ldsRed[(w * 64 + rr * lanesPerRow + col / 8u) * 8 + (col & 7u)];
        a.partials[(size_t)blockIdx.x * kMaxReduceCols + col] = s;
    }
}

// 64 columns per workgroup (see sumPartials).
__global__ __launch_bounds__(64 * kReduceWaves) void reduceSumFinalKernel(const ReduceSumArgs a, uint32_t numPartials)
{
    __shared__ float red[kReduceWaves * 64];
    const uint32_t col = blockIdx.x * 64u + (threadIdx.x & 63u);
    const bool inRange = col < (uint32_t)a.n;
    float s;
    if (!sumPartials(a.partials + col, kMaxReduceCols, numPartials, inRange, red, s) || !inRange) return;
    if (a.bufCt == kF32) ((float*)a.buf)[col] += s;
    else ((half_t*)a.buf)[col] = (half_t)((float)((half_t*)a.buf)[col] + s);
}

// persistent workgroups of the streaming reduce-sum kernel: eight per compute unit
uint32_t reduceStreamGridX(uint32_t batch, int numCUs)
{
    const uint32_t need = (batch + 4u * kRsUnroll - 1u) / (4u * kRsUnroll);      // at least one row per wave-iteration
    const uint32_t cap = 8u * (uint32_t)numCUs;
    return need < cap ? (need ? need : 1) : cap;
}

uint32_t outerGridX(uint32_t batch, int numCUs)
{
    // two workgroups per compute unit: eight waves whose loads overlap each other's MFMAs
    const uint32_t rounds = (batch + 31) / 32, need = (rounds + 3) / 4;
    const uint32_t cap = 2u * (uint32_t)numCUs;
    return need < cap ? (need ? need : 1) : cap;
}

} // namespace

size_t outerWorkspaceBytes(int m, int n, uint32_t batch, int numCUs)
{
    const size_t blocks = (size_t)((m + kBlk - 1) / kBlk) * ((n + kBlk - 1) / kBlk);
    return blocks * outerGridX(batch, numCUs) * kOuterPartialFloats * sizeof(float);
}

hipError_t launchOuterProduct(hipStream_t stream, const OuterArgs& a, int numCUs)
{
    if (a.batch == 0) return hipSuccess;
    const uint32_t gx = outerGridX(a.batch, numCUs);
    const uint32_t blocks = (uint32_t)((a.m + kBlk - 1) / kBlk) * (uint32_t)((a.n + kBlk - 1) / kBlk);
    noteKernel(false, "outerProductKernel + outerReduceKernel");
    hipLaunchKernelGGL(outerProductKernel, dim3(gx, blocks), dim3(256), 0, stream, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(outerReduceKernel, dim3(kOuterPartialFloats / 64, blocks), dim3(64 * kReduceWaves), 0, stream, a, gx);
    return hipGetLastError();
}

size_t reduceSumWorkspaceBytes(uint32_t batch, int numCUs)
{
    const uint32_t gx = max(outerGridX(batch * 2, numCUs), reduceStreamGridX(batch, numCUs));
    return (size_t)gx * kMaxReduceCols * sizeof(float);
}

hipError_t launchReduceSum(hipStream_t stream, const ReduceSumArgs& a, int numCUs)
{
    if (a.batch == 0) return hipSuccess;
    if (a.n > kMaxReduceCols) return hipErrorInvalidValue;
    uint32_t gx;
    if (a.n % 8 == 0 && ((uintptr_t)a.v & 15u) == 0 && (a.vStride & 15u) == 0) {
        uint32_t lanesPerRow = 1;
        while (lanesPerRow < (uint32_t)a.n / 8u) lanesPerRow *= 2;
        gx = reduceStreamGridX(a.batch, numCUs);
        noteKernel(false, "reduceSumStreamKernel + reduceSumFinalKernel");
        hipLaunchKernelGGL(reduceSumStreamKernel, dim3(gx), dim3(256), 0, stream, a, lanesPerRow);
    } else {
        gx = outerGridX(a.batch * 2, numCUs);
        noteKernel(false, "reduceSumKernel + reduceSumFinalKernel");
        hipLaunchKernelGGL(reduceSumKernel, dim3(gx), dim3(256), 0, stream, a);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(reduceSumFinalKernel, dim3((a.n + 63) / 64), dim3(64 * kReduceWaves), 0, stream, a, gx);
    return hipGetLastError();
}

} // namespace cv
