// cv_mlp_float.hip -- fused forward MLP whose carrier is not half: T = float or bfloat16 throughout
// (vectors, weights, biases, results), the form the neural module's FFLayer<T, ...> chain takes for T = float
// (source/standard-modules/neural/layers.slang:34-110) and this library's bfloat16 extension.
//
// Every layer is coopVecMatMulAdd + activation in T, exactly as the single-layer kernels of
// cv_matmul_impl.h evaluate it (fp32 accumulation seeded with the bias, k ascending; T = bfloat16 rounds
// the sum to bfloat16 before the activation, T = float applies the activation to the sum itself), so the
// fused network equals the chain of single-layer operators bit for bit.  Layer sizes are run-time values up
// to 128; the A fragments of all layers live in LDS.  Activations stay in registers between layers: a
// layer's accumulators (lane%16 = sample, rows 4t..4t+3 of lane group g) are the next layer's B operand.
#include <type_traits>

#include "cv_matmul_impl.h"
#include "cv_mlp_impl.h"

namespace cv {

namespace {

constexpr int kFltTileLimit = 8;                    // 128 rows / columns
constexpr uint32_t kFltLdsDwords = 36 * 1024;       // 144 KB for all layers' fragments and biases

struct FltLayer {
    int32_t mt, kt;
    uint32_t fragBase, biasBase;
};
struct FltArgs {
    MlpArgs mlp;
    FltLayer gl[kMaxMlpLayers];
    uint32_t biasDwordBase;
    int32_t ct;              // kF32 or kBF16
};

__device__ __forceinline__ float activateFloat(float x, int act, float slope)
{
    if (act == kActRelu) return x > 0.f ? x : 0.f;
    if (act == kActLeakyRelu) return fmaxf(x, x * slope);
    if (act >= kActSigmoid) return smoothActivation(x, act);
    return x;
}

// MAXT: the unrolled bound on a layer's 16-row tiles (4 for networks up to 64 wide, which then need half the
// registers and run more waves per SIMD; 8 up to 128)
template <class Mma, int MAXT>
__global__ __launch_bounds__(256) void mlpFloatKernel(const FltArgs ga)
{
    constexpr int kFltMaxTiles = MAXT, kFltMaxKT = MAXT / 2;
    constexpr int EPL = Mma::kEpl, FD = Mma::kFD, ESZ = Mma::kEsz, RAW = Mma::kRawDW;
    constexpr bool F32 = ESZ == 4;
    static_assert(EPL == 8, "the layer chain needs 8 k-slots per lane per fragment");
    const MlpArgs& a = ga.mlp;
    const int L = a.numLayers;
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    float* ldsB = (float*)(lds + ga.biasDwordBase);

    for (int l = 0; l < L; ++l) {
        const MlpLayerArgs& ly = a.layers[l];
        const int MT = ga.gl[l].mt, KT = ga.gl[l].kt, ROWS = 4 * MT;
        stageFragments<ESZ, EPL>(lds + ga.gl[l].fragBase * 64 * RAW, ly.w, ly.shape, false, MT, KT, optGS((uint32_t)ly.in),
                                 (uint32_t)ly.out, (uint32_t)ly.in);
        for (int e = threadIdx.x; e < MT * 16; e += 256) {
            const int t = e >> 4, g = (e >> 2) & 3, r = e & 3;
            const int row = g * ROWS + 4 * t + r;
            ldsB[ga.gl[l].biasBase + e] = (ly.bias && row < ly.out) ? loadAsFloat(ly.bias + (size_t)row * ESZ, ga.ct) : 0.f;
        }
    }
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, n = lane & 15;
    const int in0 = a.layers[0].in;
    const uint32_t gs0 = optGS((uint32_t)in0);
    const int kt0 = ga.gl[0].kt;
    const int outDim = a.layers[L - 1].out;
    const int orows = 4 * ga.gl[L - 1].mt;

    const uint32_t numTiles = (a.batch + 15) / 16;
    for (uint32_t tile = blockIdx.x * 4 + wave; tile < numTiles; tile += gridDim.x * 4) {
        const uint32_t sample = tile * 16 + n;
        const uint32_t sc = min(sample, a.batch - 1);
        uint32_t act[kFltMaxKT][FD];
        {
            const uint8_t* p = a.in + (size_t)sc * a.inStride;
#pragma unroll
            for (int kt = 0; kt < kFltMaxKT; ++kt) {
#pragma unroll
                for (int d = 0; d < FD; ++d) act[kt][d] = 0u;
                if (kt < kt0) {
#pragma unroll
                    for (int s = 0; s < EPL; ++s) {
                        const uint32_t q = (uint32_t)(kt * EPL + s);
                        const uint32_t col = g * gs0 + q;
                        if (q < gs0 && col < (uint32_t)in0) {
                            if constexpr (F32) act[kt][s] = *(const uint32_t*)(p + 4 * col);
                            else act[kt][s / 2] |= (uint32_t)*(const uint16_t*)(p + 2 * col) << (16 * (s & 1));
                        }
                    }
                }
            }
        }

        for (int l = 0; l < L; ++l) {
            const int MT = ga.gl[l].mt, KT = ga.gl[l].kt;
            const uint32_t* wbase = lds + ((size_t)ga.gl[l].fragBase * 64 + lane) * RAW;
            const float* bbase = ldsB + ga.gl[l].biasBase + 4 * g;
            const int actKind = a.layers[l].act;
            const float slope = a.layers[l].slope;
            floatx4 acc[kFltMaxTiles];
#pragma unroll
            for (int t = 0; t < kFltMaxTiles; ++t)
                if (t < MT) acc[t] = *(const floatx4*)(bbase + 16 * t);
#pragma unroll
            for (int kt = 0; kt < kFltMaxKT; ++kt) {
                if (kt < KT) {
#pragma unroll
                    for (int t = 0; t < kFltMaxTiles; ++t) {
                        if (t < MT) {
                            uint32_t w[FD];
                            Mma::decode(wbase + (size_t)(t * KT + kt) * 64 * RAW, w);
                            acc[t] = Mma::mma(w, act[kt], acc[t]);
                        }
                    }
                }
            }
            // the layer's result in T, activated: what coopVecMatMulAdd + activation returns
            float z[kFltMaxTiles][4];
#pragma unroll
            for (int t = 0; t < kFltMaxTiles; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (t < MT) z[t][r] = F32 ? activateFloat(acc[t][r], actKind, slope) : activate16<bf16_t>(acc[t][r], actKind, slope);
                    else z[t][r] = 0.f;
                }
            if (l + 1 < L) {
#pragma unroll
                for (int kt = 0; kt < kFltMaxKT; ++kt) {
                    if constexpr (F32) {
#pragma unroll
                        for (int s = 0; s < 8; ++s) act[kt][s] = __builtin_bit_cast(uint32_t, z[2 * kt + s / 4][s % 4]);
                    } else {
                        act[kt][0] = pack16<bf16_t>(z[2 * kt][0], z[2 * kt][1]);
                        act[kt][1] = pack16<bf16_t>(z[2 * kt][2], z[2 * kt][3]);
                        act[kt][2] = pack16<bf16_t>(z[2 * kt + 1][0], z[2 * kt + 1][1]);
                        act[kt][3] = pack16<bf16_t>(z[2 * kt + 1][2], z[2 * kt + 1][3]);
                    }
                }
            } else if (sample < a.batch) {
                uint8_t* o = a.out + (size_t)sample * a.outStride + (size_t)g * orows * ESZ;
#pragma unroll
                for (int t = 0; t < kFltMaxTiles; ++t) {
                    if (t < MT) {
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            if (g * orows + 4 * t + r < outDim) {
                                if constexpr (F32) ((float*)o)[4 * t + r] = z[t][r];
                                else ((bf16_t*)o)[4 * t + r] = (bf16_t)z[t][r];
                            }
                        }
                    }
                }
            }
        }
    }
}

template <class Mma, int MAXT>
hipError_t launchFloatSized(hipStream_t stream, const FltArgs& ga, size_t ldsBytes, int numCUs)
{
    const hipError_t ea = allowDynamicLds<mlpFloatKernel<Mma, MAXT>>((int)(kFltLdsDwords * 4));
    if (ea != hipSuccess) return ea;
    int perCU = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&perCU, mlpFloatKernel<Mma, MAXT>, 256, ldsBytes) != hipSuccess || perCU < 1) perCU = 1;
    const uint32_t numTiles = (ga.mlp.batch + 15) / 16, need = (numTiles + 3) / 4;
    const uint32_t cap = (uint32_t)numCUs * (uint32_t)perCU;
    noteKernel(false, "mlpFloatKernel<%s,up to %d rows>", Mma::kName, 16 * MAXT);
    hipLaunchKernelGGL((mlpFloatKernel<Mma, MAXT>), dim3(need < cap ? need : cap), dim3(256), ldsBytes, stream, ga);
    return hipGetLastError();
}

template <class Mma>
hipError_t launchFloat(hipStream_t stream, const MlpArgs& a, int ct, int numCUs)
{
    FltArgs ga;
    ga.mlp = a;
    ga.ct = ct;
    uint32_t frag = 0, bias = 0, widest = 0;
    for (int l = 0; l < a.numLayers; ++l) {
        const uint32_t mt = optMT((uint32_t)a.layers[l].out), kt = optKT((uint32_t)a.layers[l].in, Mma::kEpl);
        if (mt > (uint32_t)kFltTileLimit || kt > (uint32_t)kFltTileLimit / 2) return hipErrorInvalidValue;
        ga.gl[l].mt = (int32_t)mt; ga.gl[l].kt = (int32_t)kt;
        ga.gl[l].fragBase = frag; ga.gl[l].biasBase = bias;
        frag += mt * kt; bias += mt * 16;
        if (mt > widest) widest = mt;
        if (2 * kt > widest) widest = 2 * kt;
    }
    ga.biasDwordBase = frag * 64 * Mma::kRawDW;
    const uint32_t dwords = ga.biasDwordBase + bias;
    if (dwords > kFltLdsDwords) return hipErrorInvalidValue;
    const size_t ldsBytes = (size_t)dwords * 4;
    return widest <= 4 ? launchFloatSized<Mma, 4>(stream, ga, ldsBytes, numCUs) : launchFloatSized<Mma, 8>(stream, ga, ldsBytes, numCUs);
}

} // namespace

// T = float (MmaKind::F32) or bfloat16 (MmaKind::Bf16) for vectors, weights, biases and results;
// hipErrorInvalidValue for layers beyond 128 or weights beyond 144 KB of LDS
hipError_t launchMlpFloat(hipStream_t stream, MmaKind kind, const MlpArgs& a, int numCUs)
{
    if (a.batch == 0) return hipSuccess;
    if (kind == MmaKind::F32) return launchFloat<F32Mma>(stream, a, kF32, numCUs);
    if (kind == MmaKind::Bf16) return launchFloat<Bf16Mma>(stream, a, kBF16, numCUs);
    return hipErrorInvalidValue;
}

} // namespace cv
