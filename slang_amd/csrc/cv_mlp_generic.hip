// cv_mlp_generic.hip -- fused forward MLP for arbitrary layer sizes (up to 128 wide) on gfx950.
//
// The specialised kernels of cv_mlp_impl.h / cv_mlp_stream.h cover networks whose hidden layers
// share one width and whose tile counts are built in.  This kernel takes any chain of
// FeedForwardLayer (examples/mlp-training-coopvec/fflayer.slang:7-67) with every dimension <= 128:
// layer sizes are run-time values, the loops over 16-row tiles are unrolled to the maximum and
// predicated with wave-uniform branches, and the A fragments of all layers live in LDS (read per
// use) instead of registers.  Same arithmetic, same register hand-over from one layer's
// accumulators to the next layer's B operand, same rounding points as the specialised kernels.
#include <type_traits>

#include "cv_mlp_impl.h"

namespace cv {

namespace {

constexpr int kGenTileLimit = 8;                    // 128 rows / columns
constexpr uint32_t kGenLdsDwords = 36 * 1024;       // 144 KB for all layers' fragments

struct GenLayer {
    int32_t mt, kt;          // tiles of this layer
    uint32_t fragBase;       // first fragment in LDS
    uint32_t biasBase;       // first bias value in LDS (floats)
};
struct GenArgs {
    MlpArgs mlp;
    GenLayer gl[kMaxMlpLayers];
    uint32_t biasDwordBase;  // biases follow the fragments in LDS
};

// MAXT: the unrolled bound on a layer's 16-row tiles (4 for networks up to 64 wide, which then need half the
// registers and run more waves per SIMD; 8 up to 128)
template <class Mma, int MAXT>
__global__ __launch_bounds__(256) void mlpGenericKernel(const GenArgs ga)
{
    constexpr int kGenMaxTiles = MAXT, kGenMaxKT = MAXT / 2;
    constexpr int EPL = Mma::kEpl, FD = Mma::kFD, ESZ = Mma::kEsz, RAW = Mma::kRawDW;
    const MlpArgs& a = ga.mlp;
    const int L = a.numLayers;
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    float* ldsB = (float*)(lds + ga.biasDwordBase);

    // ---- stage every layer's fragments (any source layout) and biases ------------------------
    for (int l = 0; l < L; ++l) {
        const MlpLayerArgs& ly = a.layers[l];
        const int MT = ga.gl[l].mt, KT = ga.gl[l].kt, ROWS = 4 * MT;
        const uint32_t gs = optGS((uint32_t)ly.in);
        stageFragments<ESZ, EPL>(lds + ga.gl[l].fragBase * 64 * RAW, ly.w, ly.shape, false, MT, KT, gs,
                                 (uint32_t)ly.out, (uint32_t)ly.in);
        for (int e = threadIdx.x; e < MT * 16; e += 256) {
            const int t = e >> 4, g = (e >> 2) & 3, r = e & 3;
            const int row = g * ROWS + 4 * t + r;
            ldsB[ga.gl[l].biasBase + e] = (ly.bias && row < ly.out) ? (float)((const half_t*)ly.bias)[row] : 0.f;
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
        // ---- this lane's quarter of the input vector, element by element (any size, any alignment)
        uint32_t act[kGenMaxKT][FD];
        {
            const uint8_t* p = a.in + (size_t)sc * a.inStride;
#pragma unroll
            for (int kt = 0; kt < kGenMaxKT; ++kt) {
                uint32_t raw[RAW];
#pragma unroll
                for (int d = 0; d < RAW; ++d) raw[d] = 0u;
                if (a.inEncoding == kEncodeXYSquares) {
                    if constexpr (RAW >= 2) {
                        if (kt == 0 && g == 0) encodeXYSquares(p, raw[0], raw[1]);     // a float2 sample -> (x, y, x*x, y*y)
                    }
                } else if (kt < kt0) {
#pragma unroll
                    for (int s = 0; s < EPL; ++s) {
                        const uint32_t q = (uint32_t)(kt * EPL + s);
                        const uint32_t col = g * gs0 + q;
                        if (q < gs0 && col < (uint32_t)in0) {
                            if constexpr (ESZ == 2) {
                                raw[s / 2] |= (uint32_t)*(const uint16_t*)(p + 2 * col) << (16 * (s & 1));
                            } else if (a.inHalfAsE4M3) {   // an fp16 element, quantised to e4m3 (saturating) on the way
                                const float v = (float)*(const half_t*)(p + 2 * col);
                                raw[s / 4] |= (packE4M3Sat(v, 0.f) & 0xffu) << (8 * (s & 3));
                            } else {
                                raw[s / 4] |= (uint32_t)p[col] << (8 * (s & 3));
                            }
                        }
                    }
                }
                Mma::decode(raw, act[kt]);
            }
        }

        for (int l = 0; l < L; ++l) {
            const int MT = ga.gl[l].mt, KT = ga.gl[l].kt;
            const uint32_t* wbase = lds + ((size_t)ga.gl[l].fragBase * 64 + lane) * RAW;
            const float* bbase = ldsB + ga.gl[l].biasBase + 4 * g;
            floatx4 acc[kGenMaxTiles];
#pragma unroll
            for (int t = 0; t < kGenMaxTiles; ++t)
                if (t < MT) acc[t] = *(const floatx4*)(bbase + 16 * t);
#pragma unroll
            for (int kt = 0; kt < kGenMaxKT; ++kt) {
                if (kt < KT) {
#pragma unroll
                    for (int t = 0; t < kGenMaxTiles; ++t) {
                        if (t < MT) {
                            uint32_t w[FD];
                            Mma::decode(wbase + (size_t)(t * KT + kt) * 64 * RAW, w);
                            acc[t] = Mma::mma(w, act[kt], acc[t]);
                        }
                    }
                }
            }
            CarrierCfg cc = makeCarrierCfg<Mma>(a.layers[l].act, a.layers[l].slope);
            if (l + 1 < L) {
                // this layer's accumulators become the next layer's B operand
#pragma unroll
                for (int kt = 0; kt < kGenMaxKT; ++kt) {
                    halfx2 lo01 = {(half_t)0, (half_t)0}, lo23 = lo01, hi01 = lo01, hi23 = lo01;
                    if (2 * kt < MT) carrierFromAcc<true>(acc[2 * kt], cc, lo01, lo23);
                    if (2 * kt + 1 < MT) carrierFromAcc<true>(acc[2 * kt + 1], cc, hi01, hi23);
                    fragFromCarrier<Mma>(lo01, lo23, hi01, hi23, cc, act[kt]);
                }
            } else {
                const half_t lo = a.layers[l].act == kActRelu ? (half_t)0.f : (half_t)-__builtin_inff();
                cc.floor2 = halfx2{lo, lo};       // the last layer's output is not re-quantised
                half_t* o = (half_t*)(a.out + (size_t)sample * a.outStride) + g * orows;
#pragma unroll
                for (int t = 0; t < kGenMaxTiles; ++t) {
                    if (t < MT && sample < a.batch) {
                        halfx2 p0, p1;
                        carrierFromAcc<true>(acc[t], cc, p0, p1);
                        const half_t v[4] = {p0.x, p0.y, p1.x, p1.y};
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (g * orows + 4 * t + r < outDim) o[4 * t + r] = v[r];
                    }
                }
            }
        }
    }
}

template <class Mma, int MAXT>
hipError_t launchGenericSized(hipStream_t stream, const GenArgs& ga, size_t ldsBytes, int numCUs)
{
    const hipError_t ea = allowDynamicLds<mlpGenericKernel<Mma, MAXT>>((int)(kGenLdsDwords * 4));
    if (ea != hipSuccess) return ea;
    int perCU = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&perCU, mlpGenericKernel<Mma, MAXT>, 256, ldsBytes) != hipSuccess || perCU < 1) perCU = 1;
    const uint32_t numTiles = (ga.mlp.batch + 15) / 16, need = (numTiles + 3) / 4;
    const uint32_t cap = (uint32_t)numCUs * (uint32_t)perCU;
    noteKernel(false, "mlpGenericKernel<%s,up to %d rows>", Mma::kName, 16 * MAXT);
    hipLaunchKernelGGL((mlpGenericKernel<Mma, MAXT>), dim3(need < cap ? need : cap), dim3(256), ldsBytes, stream, ga);
    return hipGetLastError();
}

template <class Mma>
hipError_t launchGeneric(hipStream_t stream, const MlpArgs& a, int numCUs)
{
    GenArgs ga;
    ga.mlp = a;
    uint32_t frag = 0, bias = 0, widest = 0;
    for (int l = 0; l < a.numLayers; ++l) {
        const uint32_t mt = optMT((uint32_t)a.layers[l].out), kt = optKT((uint32_t)a.layers[l].in, Mma::kEpl);
        if (mt > (uint32_t)kGenTileLimit || kt > (uint32_t)kGenTileLimit / 2) return hipErrorInvalidValue;
        ga.gl[l].mt = (int32_t)mt; ga.gl[l].kt = (int32_t)kt;
        ga.gl[l].fragBase = frag; ga.gl[l].biasBase = bias;
        frag += mt * kt; bias += mt * 16;
        if (mt > widest) widest = mt;
        if (2 * kt > widest) widest = 2 * kt;
    }
    ga.biasDwordBase = frag * 64 * Mma::kRawDW;
    const uint32_t dwords = ga.biasDwordBase + bias;
    if (dwords > kGenLdsDwords) return hipErrorInvalidValue;
    const size_t ldsBytes = (size_t)dwords * 4;
    return widest <= 4 ? launchGenericSized<Mma, 4>(stream, ga, ldsBytes, numCUs) : launchGenericSized<Mma, 8>(stream, ga, ldsBytes, numCUs);
}

} // namespace

hipError_t launchMlpGeneric(hipStream_t stream, MmaKind kind, const MlpArgs& a, int numCUs)
{
    if (a.batch == 0) return hipSuccess;
    switch (kind) {
    case MmaKind::F16: return launchGeneric<F16Mma>(stream, a, numCUs);
    case MmaKind::Fp8AsF16: return launchGeneric<Fp8AsF16Mma>(stream, a, numCUs);
    case MmaKind::Fp8Native: return launchGeneric<Fp8NativeMma>(stream, a, numCUs);
    default: break;
    }
    return hipErrorInvalidValue;
}

} // namespace cv
