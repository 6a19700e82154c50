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

#include "cv_mlp_generic_impl.h"

namespace cv {

namespace {

template <class Mma, int MAXT, bool SMOOTH, bool TAPS = false>
__global__ __launch_bounds__(256) void mlpGenericKernel(const GenArgs ga)
{
    constexpr int kGenMaxKT = MAXT / 2;
    constexpr int EPL = Mma::kEpl, FD = Mma::kFD, ESZ = Mma::kEsz, RAW = Mma::kRawDW;
    const MlpArgs& a = ga.mlp;
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    genericStage<Mma>(ga, lds);
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, n = lane & 15;
    const int in0 = a.layers[0].in;
    const uint32_t gs0 = optGS((uint32_t)in0);
    const int kt0 = ga.gl[0].kt;

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
                    // every element is loaded from an address inside the vector and masked afterwards: loads under a
                    // per-element condition wait for one another, a memory round trip each
#pragma unroll
                    for (int s = 0; s < EPL; ++s) {
                        const uint32_t q = (uint32_t)(kt * EPL + s);
                        const uint32_t col = g * gs0 + q;
                        const bool on = q < gs0 && col < (uint32_t)in0;
                        const uint32_t cc = on ? col : 0u;
                        if constexpr (ESZ == 2) {
                            const uint32_t v = *(const uint16_t*)(p + 2 * cc);
                            raw[s / 2] |= (on ? v : 0u) << (16 * (s & 1));
                        } else if (a.inHalfAsE4M3) {   // an fp16 element, quantised to e4m3 (saturating) on the way
                            const float v = (float)*(const half_t*)(p + 2 * cc);
                            raw[s / 4] |= (on ? packE4M3Sat(v, 0.f) & 0xffu : 0u) << (8 * (s & 3));
                        } else {
                            const uint32_t v = p[cc];
                            raw[s / 4] |= (on ? v : 0u) << (8 * (s & 3));
                        }
                    }
                }
                Mma::decode(raw, act[kt]);
            }
        }

        genericRunLayers<Mma, MAXT, SMOOTH, TAPS>(ga, lds, lane, sample, act);
    }
}

template <class Mma, int MAXT, bool SMOOTH, bool TAPS = false>
hipError_t launchGenericSized(hipStream_t stream, const GenArgs& ga, size_t ldsBytes, int numCUs)
{
    const hipError_t ea = allowDynamicLds<mlpGenericKernel<Mma, MAXT, SMOOTH, TAPS>>((int)(kGenLdsDwords * 4));
    if (ea != hipSuccess) return ea;
    int perCU = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&perCU, mlpGenericKernel<Mma, MAXT, SMOOTH, TAPS>, 256, ldsBytes) != hipSuccess || perCU < 1) perCU = 1;
    const uint32_t numTiles = (ga.mlp.batch + 15) / 16, need = (numTiles + 3) / 4;
    const uint32_t cap = (uint32_t)numCUs * (uint32_t)perCU;
    noteKernel(false, "mlpGenericKernel<%s,up to %d rows%s%s>", Mma::kName, 16 * MAXT, SMOOTH ? ",smooth activations" : "",
               TAPS ? ",every layer's vectors stored" : "");
    hipLaunchKernelGGL((mlpGenericKernel<Mma, MAXT, SMOOTH, TAPS>), dim3(need < cap ? need : cap), dim3(256), ldsBytes, stream, ga);
    return hipGetLastError();
}

template <class Mma>
hipError_t launchGeneric(hipStream_t stream, const MlpArgs& a, int numCUs)
{
    GenArgs ga;
    uint32_t widest = 0;
    const uint32_t dwords = planGeneric<Mma>(a, ga, kGenLdsDwords, &widest);
    if (!dwords) return hipErrorInvalidValue;
    const size_t ldsBytes = (size_t)dwords * 4;
    if (hasSmoothActivation(a))
        return widest <= 4 ? launchGenericSized<Mma, 4, true>(stream, ga, ldsBytes, numCUs) : launchGenericSized<Mma, 8, true>(stream, ga, ldsBytes, numCUs);
    return widest <= 4 ? launchGenericSized<Mma, 4, false>(stream, ga, ldsBytes, numCUs) : launchGenericSized<Mma, 8, false>(stream, ga, ldsBytes, numCUs);
}

} // namespace

hipError_t launchMlpGenericTaps(hipStream_t stream, const MlpArgs& a, uint8_t* const* tapZ, uint8_t* const* tapX, int numCUs)
{
    if (a.batch == 0) return hipSuccess;
    if (hasSmoothActivation(a)) return hipErrorInvalidValue;
    GenArgs ga;
    uint32_t widest = 0;
    const uint32_t dwords = planGeneric<F16Mma>(a, ga, kGenLdsDwords, &widest);
    if (!dwords) return hipErrorInvalidValue;
    for (int l = 0; l < kMaxMlpLayers; ++l) {
        ga.tapZ[l] = l < a.numLayers ? tapZ[l] : nullptr;
        ga.tapX[l] = l < a.numLayers ? tapX[l] : nullptr;
    }
    const size_t ldsBytes = (size_t)dwords * 4;
    return widest <= 4 ? launchGenericSized<F16Mma, 4, false, true>(stream, ga, ldsBytes, numCUs)
                       : launchGenericSized<F16Mma, 8, false, true>(stream, ga, ldsBytes, numCUs);
}

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
