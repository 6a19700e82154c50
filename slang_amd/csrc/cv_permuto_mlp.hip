// cv_permuto_mlp.hip -- permutohedral encoding and the decoder network in one kernel, for gfx950.
//
// In Slang a thread calls PermutoEncoder::encode (source/standard-modules/neural/permuto-encoder.slang:240-337) and
// hands the encoded vector straight to the first FFLayer / FeedForwardLayer of its network
// (source/standard-modules/neural/layers.slang:34-110, examples/mlp-training-coopvec/network.slang:41-47): the
// features never exist in memory.  Batched, the two-call form (cvPermutoEncode, cvMlpForward) writes and re-reads
// levels x features elements per position; here a wave encodes 16 positions directly into the B operand of the first
// layer -- lane 16g+n computes the levels whose features make up lane group g's share of sample n's vector -- and
// pushes the tile through the layers with the weights of the whole network, the level records and (when it fits) the
// feature table in LDS.  Arithmetic per level and per layer is that of the two separate kernels, so the results are
// the same bits.
#include <string.h>

#include "cv_kernels.h"
#include "cv_launch.h"
#include "cv_mlp_generic_impl.h"
#include "cv_permuto_impl.h"

namespace cv {

namespace {

struct PermutoMlpArgs {
    GenArgs net;
    CvPermutoDesc desc;
    const uint8_t* pos; uint64_t posStride;
    const uint8_t* table;
    uint32_t tableElems;
    uint32_t levelDword;     // where the level records start in LDS (dwords)
    uint32_t tableDword;     // where the feature table starts in LDS (dwords); unused when it stays in memory
};

constexpr uint32_t kLevelDwords = CV_PERMUTO_MAX_LEVELS * sizeof(CvPermutoLevelInfo) / 4;
constexpr uint32_t kLdsLimitDwords = 160 * 1024 / 4;

template <int D, int F, int MAXT, bool LDS_TABLE>
__global__ __launch_bounds__(1024) void permutoMlpKernel(const PermutoMlpArgs pa)
{
    using Mma = F16Mma;
    typedef typename PermutoEntry<half_t, F>::type Entry;
    constexpr int KT = MAXT / 2, FD = Mma::kFD, EPL = Mma::kEpl;
    static_assert(Mma::kRawDW == FD && EPL == 8, "fp16 fragments are used as they lie");
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    const GenArgs& ga = pa.net;
    const MlpArgs& a = ga.mlp;
    genericStage<Mma>(ga, lds);
    CvPermutoLevelInfo* levels = (CvPermutoLevelInfo*)(lds + pa.levelDword);
    {
        const uint32_t L = pa.desc.maxLevels;
        const uint32_t* src = (const uint32_t*)pa.desc.levelInfo;
        for (uint32_t i = threadIdx.x; i < L * (uint32_t)(sizeof(CvPermutoLevelInfo) / 4); i += blockDim.x) ((uint32_t*)levels)[i] = src[i];
        if constexpr (LDS_TABLE) {
            const Entry* t = (const Entry*)pa.table;
            Entry* dst = (Entry*)(lds + pa.tableDword);
            for (uint32_t i = threadIdx.x; i < pa.tableElems / (uint32_t)F; i += blockDim.x) dst[i] = t[i];
        }
    }
    __syncthreads();
    const half_t* table = LDS_TABLE ? (const half_t*)(lds + pa.tableDword) : (const half_t*)pa.table;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const int g = lane >> 4, n = lane & 15;
    const uint32_t in0 = (uint32_t)a.layers[0].in;            // = maxLevels * F
    const uint32_t gs0 = optGS(in0);                           // features per lane group: a multiple of 4, hence of F
    const uint32_t perLane = gs0 / (uint32_t)F;                // levels whose features this lane supplies
    const uint32_t numTiles = (a.batch + 15) / 16;
    // a tile's position is requested one tile ahead: a wave's load -> encode -> layers -> store chain would otherwise
    // wait out a memory round trip per tile, and the next load would queue behind the tile's stores
    auto loadPosition = [&](uint32_t tile, half_t* p) {
        const uint32_t sc = min(min(tile, numTiles - 1) * 16 + (uint32_t)n, a.batch - 1);
#pragma unroll
        for (int d = 0; d < D; ++d) p[d] = ((const half_t*)(pa.pos + (size_t)sc * pa.posStride))[d];
    };
    const uint32_t tileStep = gridDim.x * waves;
    half_t ahead[D];
    loadPosition(blockIdx.x * waves + wave, ahead);
    for (uint32_t tile = blockIdx.x * waves + wave; tile < numTiles; tile += tileStep) {
        const uint32_t sample = tile * 16 + n;
        float pos[D];
#pragma unroll
        for (int d = 0; d < D; ++d) pos[d] = (float)ahead[d];
        loadPosition(tile + tileStep, ahead);
        uint32_t act[KT][FD];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int d = 0; d < FD; ++d) act[kt][d] = 0u;
        // element q of the lane's share is feature (q % F) of level g * perLane + q / F; shares are whole entries
#pragma unroll
        for (int e = 0; e < KT * EPL / F; ++e) {
            if ((uint32_t)e < perLane) {                                       // uniform over the wave
                const uint32_t level = (uint32_t)g * perLane + (uint32_t)e;
                Entry v;
#pragma unroll
                for (int f = 0; f < F; ++f) v[f] = (half_t)0.f;
#ifndef PM_NO_ENCODE
                if (level < pa.desc.maxLevels) v = permutoEncodeEntry<half_t, D, F>(pos, levels[level], table, pa.desc.maxLevel);
#else
                v[0] = (half_t)pos[0];
#endif
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    const int q = e * F + f;
                    const uint32_t bits = (uint32_t)__builtin_bit_cast(uint16_t, (half_t)v[f]);
                    act[q / EPL][(q % EPL) / 2] |= bits << (16 * (q & 1));
                }
            }
        }
#ifndef PM_NO_MLP
        genericRunLayers<Mma, MAXT, false>(ga, lds, lane, sample, act);      // plain, ReLU and leaky ReLU layers
#else
        if (sample < a.batch && g == 0) *(uint16_t*)(a.out + (size_t)sample * a.outStride) = (uint16_t)(act[0][0] ^ act[0][1]);
#endif
    }
}

template <int D, int F, int MAXT>
hipError_t launchShape(hipStream_t stream, PermutoMlpArgs& pa, uint32_t netDwords, int numCUs)
{
    pa.levelDword = (netDwords + 3u) & ~3u;
    pa.tableDword = pa.levelDword + kLevelDwords;
    const uint32_t tableDwords = (pa.tableElems + 1u) / 2u;
    const bool inLds = (uint64_t)pa.tableDword + tableDwords <= kLdsLimitDwords;
    const size_t ldsBytes = ((size_t)pa.tableDword + (inLds ? tableDwords : 0u)) * 4;
    const uint32_t numTiles = (pa.net.mlp.batch + 15) / 16, need = (numTiles + 15) / 16;
    noteKernel(false, "permutoMlpKernel<D=%d,F=%d,up to %d rows,table in %s>", D, F, 16 * MAXT, inLds ? "LDS" : "memory");
    auto launch = [&](auto kernel) -> hipError_t {
        int perCU = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&perCU, kernel, 1024, ldsBytes) != hipSuccess || perCU < 1) perCU = 1;
        const uint32_t cap = (uint32_t)numCUs * (uint32_t)perCU;
        hipLaunchKernelGGL(kernel, dim3(need < cap ? need : cap), dim3(1024), ldsBytes, stream, pa);
        return hipGetLastError();
    };
    if (inLds) {
        const hipError_t e = allowDynamicLds<permutoMlpKernel<D, F, MAXT, true>>((int)(kLdsLimitDwords * 4));
        return e != hipSuccess ? e : launch(permutoMlpKernel<D, F, MAXT, true>);
    }
    const hipError_t e = allowDynamicLds<permutoMlpKernel<D, F, MAXT, false>>((int)(kLdsLimitDwords * 4));
    return e != hipSuccess ? e : launch(permutoMlpKernel<D, F, MAXT, false>);
}

} // namespace

hipError_t launchPermutoWide16In16(hipStream_t stream, const CvPermutoDesc& desc, const void* positions, uint64_t positionStride,
                                   const void* featureTable, uint32_t tableElems, const MlpArgs& mlp, int numCUs, int H, int NH);
hipError_t launchPermutoWide16In32(hipStream_t stream, const CvPermutoDesc& desc, const void* positions, uint64_t positionStride,
                                   const void* featureTable, uint32_t tableElems, const MlpArgs& mlp, int numCUs, int H, int NH);

// the networks mlpWide16Body takes: ReLU hidden layers of one width, 32 or 64, at most 32 outputs without or with ReLU
static bool wideDecoder(const MlpArgs& a, int& H, int& NH)
{
    const int L = a.numLayers, width = a.layers[0].out;
    if (L < 2 || L > 3 || (width != 32 && width != 64) || a.noWideTiles || a.batch > (1u << 31)) return false;
    for (int l = 0; l < L; ++l) {
        if (l + 1 < L && (a.layers[l].out != width || a.layers[l].act != kActRelu)) return false;
        if (l > 0 && a.layers[l].in != width) return false;
    }
    if ((a.layers[L - 1].act != kActNone && a.layers[L - 1].act != kActRelu) || a.layers[L - 1].out > 32) return false;
    H = width / 32; NH = L - 1;
    return true;
}

hipError_t launchPermutoMlp(hipStream_t stream, const CvPermutoDesc& desc, const void* positions, uint64_t positionStride,
                            const void* featureTable, const MlpArgs& mlp, int numCUs)
{
    if (mlp.batch == 0) return hipSuccess;
    const int D = desc.dimensions, F = desc.featureDimensionPerEntry;
    if (D < 1 || D > 4 || (F != 1 && F != 2 && F != 4)) return hipErrorInvalidValue;
    if ((uint32_t)mlp.layers[0].in != desc.maxLevels * (uint32_t)F) return hipErrorInvalidValue;
    PermutoMlpArgs pa;
    memset(&pa, 0, sizeof(pa));
    uint32_t widest = 0;
    // the network's fragments must leave room for the level records
    const uint32_t netDwords = planGeneric<F16Mma>(mlp, pa.net, kLdsLimitDwords - kLevelDwords - 4u, &widest);
    if (!netDwords) return hipErrorInvalidValue;
    pa.desc = desc;
    pa.pos = (const uint8_t*)positions; pa.posStride = positionStride; pa.table = (const uint8_t*)featureTable;
    uint64_t tableElems = 0;
    for (uint32_t l = 0; l < desc.maxLevels; ++l) {
        const uint64_t e = ((uint64_t)desc.levelInfo[l].offsetOfFeatureTable + desc.levelInfo[l].featureTableSize) * (uint64_t)F;
        tableElems = e > tableElems ? e : tableElems;
    }
    if (tableElems > 0xffffffffull) return hipErrorInvalidValue;
    pa.tableElems = (uint32_t)tableElems;
    int H = 0, NH = 0;
    if ((mlp.layers[0].in == 16 || mlp.layers[0].in == 32) && wideDecoder(mlp, H, NH)) {      // 32-sample tiles where the network allows them
        const hipError_t e = mlp.layers[0].in == 16
            ? launchPermutoWide16In16(stream, desc, positions, positionStride, featureTable, pa.tableElems, mlp, numCUs, H, NH)
            : launchPermutoWide16In32(stream, desc, positions, positionStride, featureTable, pa.tableElems, mlp, numCUs, H, NH);
        if (e != hipErrorInvalidValue) return e;
    }
    const bool small = widest <= 4;
    if (hasSmoothActivation(mlp)) return hipErrorInvalidValue;      // plain, ReLU and leaky ReLU layers only
    switch (D * 16 + F) {
#define CV_DF(N, G) case N * 16 + G: return small ? launchShape<N, G, 4>(stream, pa, netDwords, numCUs) : launchShape<N, G, 8>(stream, pa, netDwords, numCUs);
    CV_DF(1, 1) CV_DF(1, 2) CV_DF(1, 4) CV_DF(2, 1) CV_DF(2, 2) CV_DF(2, 4) CV_DF(3, 1) CV_DF(3, 2) CV_DF(3, 4) CV_DF(4, 1) CV_DF(4, 2) CV_DF(4, 4)
#undef CV_DF
    }
    return hipErrorInvalidValue;
}

} // namespace cv
