// cv_mlp_generic_impl.h -- the run-time-size fused forward pass shared by the kernels that keep a whole network's
// weights in LDS: staging, and one 16-sample tile pushed through every FeedForwardLayer
// (examples/mlp-training-coopvec/fflayer.slang:7-67; network.slang:41-47) from a first-layer B operand that the caller
// has in registers.  Layer sizes are run-time values, the loops over 16-row tiles are unrolled to a bound and predicated
// with wave-uniform branches, the A fragments of all layers are read from LDS per use.
#pragma once
#include "cv_mlp_impl.h"

namespace cv {

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
    // (TAPS instantiations only) where to leave every layer's pre-activation / activation vectors, [batch][out_l] halfs in
    // contiguous rows, or null: what the backward pass of the layer-by-layer training step reads
    uint8_t* tapZ[kMaxMlpLayers];
    uint8_t* tapX[kMaxMlpLayers];
};

// Tile counts and LDS placement of every layer; the dwords of LDS taken (fragments, then biases), or 0 when a layer is
// wider than 128 or the network does not fit `limitDwords`.  `widest` receives the largest tile count of any layer.
template <class Mma>
inline uint32_t planGeneric(const MlpArgs& a, GenArgs& ga, uint32_t limitDwords, uint32_t* widest)
{
    ga.mlp = a;
    uint32_t frag = 0, bias = 0, w = 0;
    for (int l = 0; l < a.numLayers; ++l) {
        const uint32_t mt = optMT((uint32_t)a.layers[l].out), kt = optKT((uint32_t)a.layers[l].in, Mma::kEpl);
        if (mt > (uint32_t)kGenTileLimit || kt > (uint32_t)kGenTileLimit / 2) return 0;
        ga.gl[l].mt = (int32_t)mt; ga.gl[l].kt = (int32_t)kt;
        ga.gl[l].fragBase = frag; ga.gl[l].biasBase = bias;
        frag += mt * kt; bias += mt * 16;
        if (mt > w) w = mt;
        if (2 * kt > w) w = 2 * kt;
    }
    ga.biasDwordBase = frag * 64 * Mma::kRawDW;
    const uint32_t dwords = ga.biasDwordBase + bias;
    if (dwords > limitDwords) return 0;
    *widest = w;
    return dwords;
}

inline bool hasSmoothActivation(const MlpArgs& a)
{
    for (int l = 0; l < a.numLayers; ++l)
        if (a.layers[l].act >= kActSigmoid) return true;
    return false;
}

// stage every layer's fragments (any source layout) and biases; the caller synchronises the workgroup afterwards
template <class Mma>
__device__ __forceinline__ void genericStage(const GenArgs& ga, uint32_t* lds)
{
    constexpr int EPL = Mma::kEpl, ESZ = Mma::kEsz, RAW = Mma::kRawDW;
    const MlpArgs& a = ga.mlp;
    float* ldsB = (float*)(lds + ga.biasDwordBase);
    for (int l = 0; l < a.numLayers; ++l) {
        const MlpLayerArgs& ly = a.layers[l];
        const int MT = ga.gl[l].mt, KT = ga.gl[l].kt, ROWS = 4 * MT;
        const uint32_t gs = optGS((uint32_t)ly.in);
        stageFragments<ESZ, EPL>(lds + ga.gl[l].fragBase * 64 * RAW, ly.w, ly.shape, false, MT, KT, gs,
                                 (uint32_t)ly.out, (uint32_t)ly.in);
        for (int e = threadIdx.x; e < MT * 16; e += blockDim.x) {
            const int t = e >> 4, g = (e >> 2) & 3, r = e & 3;
            const int row = g * ROWS + 4 * t + r;
            ldsB[ga.gl[l].biasBase + e] = (ly.bias && row < ly.out) ? (float)((const half_t*)ly.bias)[row] : 0.f;
        }
    }
}

// One tile of 16 samples (lane 16g+n: sample `sample`, lane group g) through all layers; `act` holds the first layer's
// B operand and is overwritten; the last layer's outputs are stored for samples inside the batch.
// MAXT: the unrolled bound on a layer's 16-row tiles (4 for networks up to 64 wide, which then need half the
// registers and run more waves per SIMD; 8 up to 128).  SMOOTH: some layer has one of the neural module's smooth
// activations (their exp / division code, inlined per element, is four fifths of the kernel: networks of plain, ReLU and
// leaky ReLU layers run an instantiation without it)
template <class Mma, int MAXT, bool SMOOTH, bool TAPS = false>
__device__ __forceinline__ void genericRunLayers(const GenArgs& ga, const uint32_t* lds, int lane, uint32_t sample,
                                                 uint32_t (&act)[MAXT / 2][Mma::kFD])
{
    constexpr int kGenMaxTiles = MAXT, kGenMaxKT = MAXT / 2;
    constexpr int RAW = Mma::kRawDW, FD = Mma::kFD;
    const MlpArgs& a = ga.mlp;
    const int L = a.numLayers, g = lane >> 4;
    const float* ldsB = (const float*)(lds + ga.biasDwordBase);
    const int outDim = a.layers[L - 1].out;
    const int orows = 4 * ga.gl[L - 1].mt;
    for (int l = 0; l < L; ++l) {
        const int MT = ga.gl[l].mt, KT = ga.gl[l].kt;
        const uint32_t* wbase = lds + ((size_t)ga.gl[l].fragBase * 64 + lane) * RAW;
        const float* bbase = ldsB + ga.gl[l].biasBase + 4 * g;
        // Every one of the MAXT accumulator tiles is computed, those beyond the layer's MT from the fragments of its
        // last tile (results unused): updates of single tiles under `if (t < MT)` made the compiler copy the whole
        // accumulator array at every branch, some 700 moves per 16 samples, five times the useful instructions.
        floatx4 acc[kGenMaxTiles];
#pragma unroll
        for (int t = 0; t < kGenMaxTiles; ++t) acc[t] = *(const floatx4*)(bbase + 16 * (t < MT ? t : MT - 1));
#pragma unroll
        for (int kt = 0; kt < kGenMaxKT; ++kt) {
            if (kt == 0 || kt < KT) {
#pragma unroll
                for (int t = 0; t < kGenMaxTiles; ++t) {
                    uint32_t w[FD];
                    Mma::decode(wbase + (size_t)((t < MT ? t : MT - 1) * KT + kt) * 64 * RAW, w);
                    acc[t] = Mma::mma(w, act[kt], acc[t]);
                }
            }
        }
        CarrierCfg cc = makeCarrierCfg<Mma>(a.layers[l].act, a.layers[l].slope);
        if constexpr (TAPS) {
            // rows 4t .. 4t+3 of the lane group, as halfs before and after the activation (the roundings of the carrier)
            uint8_t* tz = ga.tapZ[l];
            uint8_t* tx = ga.tapX[l];
            const int outL = a.layers[l].out, rowsL = 4 * MT;
            const bool quads = outL % 4 == 0;
            if ((tz || tx) && sample < a.batch) {
                const size_t row = (size_t)sample * (size_t)outL * 2u;
#pragma unroll
                for (int t = 0; t < kGenMaxTiles; ++t) {
                    const int r0 = g * rowsL + 4 * t;
                    if (t < MT && r0 < outL) {
                        typedef float floatx2 __attribute__((ext_vector_type(2)));
                        const halfx2 z01 = __builtin_convertvector(floatx2{acc[t][0], acc[t][1]}, halfx2);
                        const halfx2 z23 = __builtin_convertvector(floatx2{acc[t][2], acc[t][3]}, halfx2);
                        halfx2 x01, x23;
                        carrierFromAcc<SMOOTH>(acc[t], cc, x01, x23);
                        if (l + 1 == L) {       // the last layer's result is not clamped for a carrier
                            const half_t lo = a.layers[l].act == kActRelu ? (half_t)0.f : (half_t)-__builtin_inff();
                            CarrierCfg last = cc;
                            last.floor2 = halfx2{lo, lo};
                            carrierFromAcc<SMOOTH>(acc[t], last, x01, x23);
                        }
                        const uint32_t zb[2] = {__builtin_bit_cast(uint32_t, z01), __builtin_bit_cast(uint32_t, z23)};
                        const uint32_t xb[2] = {__builtin_bit_cast(uint32_t, x01), __builtin_bit_cast(uint32_t, x23)};
                        if (quads) {
                            if (tz) *(u32x2*)(tz + row + 2 * r0) = u32x2{zb[0], zb[1]};
                            if (tx) *(u32x2*)(tx + row + 2 * r0) = u32x2{xb[0], xb[1]};
                        } else {
#pragma unroll
                            for (int r = 0; r < 4; ++r) {
                                if (r0 + r < outL) {
                                    if (tz) *(uint16_t*)(tz + row + 2 * (r0 + r)) = (uint16_t)(zb[r / 2] >> (16 * (r & 1)));
                                    if (tx) *(uint16_t*)(tx + row + 2 * (r0 + r)) = (uint16_t)(xb[r / 2] >> (16 * (r & 1)));
                                }
                            }
                        }
                    }
                }
            }
        }
        if (l + 1 < L) {
            // this layer's accumulators become the next layer's B operand
#pragma unroll
            for (int kt = 0; kt < kGenMaxKT; ++kt) {
                halfx2 lo01 = {(half_t)0, (half_t)0}, lo23 = lo01, hi01 = lo01, hi23 = lo01;
                if constexpr (SMOOTH) {      // transcendental code per element: only for the tiles that exist
                    if (2 * kt < MT) carrierFromAcc<SMOOTH>(acc[2 * kt], cc, lo01, lo23);
                    if (2 * kt + 1 < MT) carrierFromAcc<SMOOTH>(acc[2 * kt + 1], cc, hi01, hi23);
                } else {                     // a few instructions: converted always, kept by a wave-uniform mask
                    carrierFromAcc<SMOOTH>(acc[2 * kt], cc, lo01, lo23);
                    carrierFromAcc<SMOOTH>(acc[2 * kt + 1], cc, hi01, hi23);
                    const uint32_t keepLo = 2 * kt < MT ? 0xffffffffu : 0u, keepHi = 2 * kt + 1 < MT ? 0xffffffffu : 0u;
                    lo01 = __builtin_bit_cast(halfx2, __builtin_bit_cast(uint32_t, lo01) & keepLo);
                    lo23 = __builtin_bit_cast(halfx2, __builtin_bit_cast(uint32_t, lo23) & keepLo);
                    hi01 = __builtin_bit_cast(halfx2, __builtin_bit_cast(uint32_t, hi01) & keepHi);
                    hi23 = __builtin_bit_cast(halfx2, __builtin_bit_cast(uint32_t, hi23) & keepHi);
                }
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
                    carrierFromAcc<SMOOTH>(acc[t], cc, p0, p1);
                    const half_t v[4] = {p0.x, p0.y, p1.x, p1.y};
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (g * orows + 4 * t + r < outDim) o[4 * t + r] = v[r];
                }
            }
        }
    }
}

} // namespace cv
