// cv_mlp_impl.h -- fused forward MLP kernel template for gfx950.
//
// Runs the chain the example builds from FeedForwardLayer.eval
// (examples/mlp-training-coopvec/fflayer.slang:60-66: coopVecMatMulAdd + activation, with
// CoopVec<half> as the carrier between layers; network.slang:41-47) for a whole batch:
//
//   - every layer is D = W . X^T on the matrix cores with the 16 samples of a tile as N;
//   - under the row order of cv_layout.h the fp32 accumulators of layer l are, register for
//     register, the B operand of layer l+1 once rounded to fp16 (and, for e4m3 networks,
//     re-quantised): activations never leave the VGPRs and never cross lanes;
//   - the workgroup stages all weights into LDS once (any source layout), then every wave
//     keeps all A fragments and the biases (packed fp16) in VGPRs while it strides over
//     tiles of NT*16 samples with the next tile's inputs prefetched.
//
// The kernel is specialised on tile counts (input k-tiles, hidden width in 16-row tiles,
// number of hidden layers, output tiles); actual dimensions are runtime values padded with
// zero weights.
#pragma once
#include <type_traits>

#include "cv_device.h"
#include "cv_kernels.h"
#include "cv_launch.h"
#include "cv_error.h"
#include "cv_stage.h"

namespace cv {
namespace {

template <int B, int E, class F>
__device__ __forceinline__ void staticFor(F&& f)
{
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        staticFor<B + 1, E>(f);
    }
}

// hidden layers all 16*HT wide: layer 0 is in->hidden, layers 1..NHID-1 hidden->hidden,
// layer NHID hidden->out
template <int KT0_, int HT_, int NHID_, int MTL_>
struct UniformNet {
    static constexpr int KT0 = KT0_, HT = HT_, NHID = NHID_, MTL = MTL_;
    static constexpr int L = NHID_ + 1;
    static constexpr int KTH = (HT_ + 1) / 2;
    static constexpr int MTMAX = HT_ > MTL_ ? HT_ : MTL_;
    static constexpr int KTMAX = KT0_ > KTH ? KT0_ : KTH;
    static constexpr int mt(int l) { return l < NHID_ ? HT_ : MTL_; }
    static constexpr int kt(int l) { return l == 0 ? KT0_ : KTH; }
    static constexpr int fragBase(int l)   // index of layer l's first fragment in LDS
    {
        int b = 0;
        for (int i = 0; i < l; ++i) b += mt(i) * kt(i);
        return b;
    }
    static constexpr int totalFrags = fragBase(L);
    static constexpr int biasBase(int l)   // in 16-row tiles
    {
        int b = 0;
        for (int i = 0; i < l; ++i) b += mt(i);
        return b;
    }
    static constexpr int totalBiasTiles = biasBase(L);
};

// Per-layer constants of the carrier conversion.  ReLU is a lower bound on the packed fp16
// pair (max(z, 0), or max(z, -inf) = z when off); e4m3 networks also clamp to +-448 so that
// the conversion saturates (the instruction itself yields NaN beyond the finite range).
struct CarrierCfg {
    halfx2 floor2, ceil2;
    int act;
    float slope;
};

template <class Mma>
__device__ __forceinline__ CarrierCfg makeCarrierCfg(int act, float slope)
{
    constexpr bool quant = !std::is_same<Mma, F16Mma>::value;
    const half_t lo = act == kActRelu ? (half_t)0.f : (quant ? (half_t)-448.f : (half_t)-__builtin_inff());
    CarrierCfg c;
    c.floor2 = halfx2{lo, lo};
    c.ceil2 = halfx2{(half_t)448.f, (half_t)448.f};
    c.act = act; c.slope = slope;
    return c;
}

// accumulators (one 16-row tile, 4 values per lane) -> the carrier CoopVec<half>: round to
// fp16 (v_cvt_pk_f16_f32, nearest even), then the activation, on packed pairs
// SMOOTH: the kernel also serves the neural module's smooth activations (only the general kernel
// does; the specialised ones would carry the transcendental code in every instantiation)
template <bool SMOOTH = false>
__device__ __forceinline__ void carrierFromAcc(const floatx4& acc, const CarrierCfg& c, halfx2& h01, halfx2& h23)
{
    typedef float floatx2 __attribute__((ext_vector_type(2)));
    const floatx2 a01 = {acc[0], acc[1]}, a23 = {acc[2], acc[3]};
    h01 = __builtin_convertvector(a01, halfx2);
    h23 = __builtin_convertvector(a23, halfx2);
    if (c.act == kActLeakyRelu || (SMOOTH && c.act >= kActSigmoid)) {   // leaky: max(z, z*slope) in half, fflayer.slang:64-65
        const int act = SMOOTH ? c.act : (int)kActLeakyRelu;      // without SMOOTH the transcendental code is not even compiled
        h01 = halfx2{activateHalf(h01.x, act, c.slope), activateHalf(h01.y, act, c.slope)};
        h23 = halfx2{activateHalf(h23.x, act, c.slope), activateHalf(h23.y, act, c.slope)};
    }
    h01 = __builtin_elementwise_max(h01, c.floor2);
    h23 = __builtin_elementwise_max(h23, c.floor2);
}

// fp16 pair x2 -> one dword of four e4m3 bytes (saturating, nearest even: v_cvt_scalef32_pk_fp8_f16
// rounds like the fp32 route for every fp16 input within +-448).  MODE_CLAMPS: the caller runs
// with MODE.FP16_OVFL set, under which the instruction saturates by itself.
template <bool MODE_CLAMPS = false>
__device__ __forceinline__ uint32_t quantE4M3x4(halfx2 h01, halfx2 h23, const CarrierCfg& c)
{
    typedef short shortx2 __attribute__((ext_vector_type(2)));
    if constexpr (!MODE_CLAMPS) {
        h01 = __builtin_elementwise_min(h01, c.ceil2);
        h23 = __builtin_elementwise_min(h23, c.ceil2);
    }
    // both halves of r are overwritten; starting from a value that is live anyway saves a move
    shortx2 r = __builtin_bit_cast(shortx2, h01);
    r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r, h01, 1.0f, false);
    r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r, h23, 1.0f, true);
    return __builtin_bit_cast(uint32_t, r);
}

// Two accumulator tiles (already carriers) -> one B fragment of the next layer (8 k-slots per lane).
template <class Mma, bool MODE_CLAMPS = false>
__device__ __forceinline__ void fragFromCarrier(halfx2 lo01, halfx2 lo23, halfx2 hi01, halfx2 hi23,
                                                const CarrierCfg& c, uint32_t* frag)
{
    if constexpr (std::is_same<Mma, F16Mma>::value) {
        frag[0] = __builtin_bit_cast(uint32_t, lo01); frag[1] = __builtin_bit_cast(uint32_t, lo23);
        frag[2] = __builtin_bit_cast(uint32_t, hi01); frag[3] = __builtin_bit_cast(uint32_t, hi23);
    } else {
        // re-quantise the fp16 carrier to OCP e4m3
        const uint32_t raw[2] = {quantE4M3x4<MODE_CLAMPS>(lo01, lo23, c), quantE4M3x4<MODE_CLAMPS>(hi01, hi23, c)};
        Mma::decode(raw, frag);      // e4m3 bytes as they are, or decoded back to fp16 operands
    }
}

// LEAN (kChunkRowDwords or kChunkDirect, the kind of all weight matrices; kChunkNone: the general instantiation): for
// calls bound by launch latency.  Every lane's slice of an input vector is whole, 4-byte aligned dwords and every weight
// matrix is one that ChunkInFlight takes.  Input loads then are straight-line code (a
// dword outside the slice is fetched from the start of the row, which always exists, and masked when the tile is used)
// and the weights are requested before anything waits: no wait for one load stands between two others, and a batch of
// one super-tile per wave costs one round trip to memory for inputs, weights and biases together.
template <class Mma, class Net, int NT, int S, int LEAN>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 2))) void mlpForwardKernel(const MlpArgs a)
{
    constexpr int EPL = Mma::kEpl, FD = Mma::kFD, ESZ = Mma::kEsz, RAW = Mma::kRawDW;
    constexpr int L = Net::L;
    constexpr int IN_DW = RAW * Net::KT0;
    static_assert(EPL == 8, "the layer chain needs 8 k-slots per lane per fragment");

    __shared__ __attribute__((aligned(16))) uint32_t ldsW[Net::totalFrags * 64 * RAW];
    __shared__ __attribute__((aligned(16))) uint16_t ldsB[Net::totalBiasTiles * 16];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, n = lane & 15;

    // ---- per-lane constants ----------------------------------------------------------------
    const uint32_t gs0 = optGS((uint32_t)a.layers[0].in);
    const int colBase = (int)(g * gs0);
    const int validBytes = min((int)gs0, max(a.layers[0].in - colBase, 0)) * ESZ;
    const int loadMode = a.inEncoding == kEncodeXYSquares ? 3 : a.inHalfAsE4M3 ? 4
                       : (validBytes == IN_DW * 4 && a.inAlign >= (IN_DW % 4 == 0 ? 16u : 8u)) ? 0
                       : ((validBytes & 3) == 0 && a.inAlign >= 4u) ? 1 : 2;
    constexpr int OROWS = 4 * Net::MTL;
    const int outDim = a.layers[L - 1].out;
    const int rowBase = g * OROWS;
    const int validRows = min(max(outDim - rowBase, 0), OROWS);
    const bool vecStore = validRows == OROWS && a.outAlign >= 8u;

    // One wave-iteration covers a super-tile of S tiles (16*S samples): all of its inputs are
    // loaded at once, a whole iteration ahead (narrow inputs need many samples in flight to keep
    // HBM busy), and then pushed through the layers NT tiles at a time.
    constexpr uint32_t TILE = 16 * S;
    const uint32_t numTiles = (a.batch + TILE - 1) / TILE;
    const uint32_t tileStride = gridDim.x * 4;
    uint32_t tile = blockIdx.x * 4 + wave;
    const uint8_t* inLane = a.in + (size_t)colBase * (a.inHalfAsE4M3 ? 2 : ESZ);
    uint8_t* outLane = a.out + (size_t)rowBase * 2;
    const uint32_t lastSample = a.batch - 1;

    auto loadTile = [&](uint32_t (&buf)[S][IN_DW], uint32_t t) {
#pragma unroll
        for (int j = 0; j < S; ++j) {
            const uint32_t s = min(t * TILE + 16 * j + n, lastSample);
            const uint8_t* p = inLane + (size_t)s * a.inStride;
            if constexpr (LEAN != kChunkNone) {
                const uint8_t* row = a.in + (size_t)s * a.inStride;
#pragma unroll
                for (int i = 0; i < IN_DW; ++i) buf[j][i] = *(const uint32_t*)(4 * i < validBytes ? p + 4 * i : row);
            } else if (loadMode == 3) {
                // a float2 sample; lane group 0 owns all four encoded inputs
#pragma unroll
                for (int i = 0; i < IN_DW; ++i) buf[j][i] = 0u;
                if constexpr (IN_DW >= 2) {
                    if (g == 0) encodeXYSquares(a.in + (size_t)s * a.inStride, buf[j][0], buf[j][1]);
                }
            } else if (loadMode == 4) {
                // fp16 vectors of an e4m3 network (CoopVec<half> with inputInterpretation FloatE4M3):
                // eight halves become the eight e4m3 bytes of one k-tile
                if constexpr (ESZ == 1) {
                    const int validElems = validBytes;
                    const bool whole = validElems == 8 * Net::KT0 && a.inAlign >= 16u;
#pragma unroll
                    for (int kt = 0; kt < Net::KT0; ++kt) {
                        uint32_t h[4];
                        if (whole) {
                            const u32x4 v = *(const u32x4*)(p + 16 * kt);
                            h[0] = v.x; h[1] = v.y; h[2] = v.z; h[3] = v.w;
                        } else {
#pragma unroll
                            for (int d = 0; d < 4; ++d) {
                                const int e0 = 8 * kt + 2 * d;
                                const uint32_t lo = e0 < validElems ? ((const uint16_t*)p)[e0] : 0u;
                                const uint32_t hi = e0 + 1 < validElems ? ((const uint16_t*)p)[e0 + 1] : 0u;
                                h[d] = lo | (hi << 16);
                            }
                        }
                        buf[j][2 * kt] = quantE4M3x4Sat(h[0], h[1]);
                        buf[j][2 * kt + 1] = quantE4M3x4Sat(h[2], h[3]);
                    }
                }
            } else if (loadMode == 0) {
                if constexpr (IN_DW % 4 == 0) {
#pragma unroll
                    for (int i = 0; i < IN_DW / 4; ++i) {
                        const u32x4 v = *(const u32x4*)(p + 16 * i);
                        buf[j][4 * i] = v.x; buf[j][4 * i + 1] = v.y; buf[j][4 * i + 2] = v.z; buf[j][4 * i + 3] = v.w;
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < IN_DW / 2; ++i) {
                        const u32x2 v = *(const u32x2*)(p + 8 * i);
                        buf[j][2 * i] = v.x; buf[j][2 * i + 1] = v.y;
                    }
                }
            } else if (loadMode == 1) {
#pragma unroll
                for (int i = 0; i < IN_DW; ++i) buf[j][i] = (4 * i < validBytes) ? *(const uint32_t*)(p + 4 * i) : 0u;
            } else {
#pragma unroll
                for (int i = 0; i < IN_DW; ++i) {
                    uint32_t v = 0;
#pragma unroll
                    for (int b = 0; b < 4; ++b)
                        if (4 * i + b < validBytes) v |= (uint32_t)p[4 * i + b] << (8 * b);
                    buf[j][i] = v;
                }
            }
        }
    };

    // the first super-tile's inputs are requested with the weights: the round trips to memory overlap (a wave without a
    // tile loads the batch's last sample and leaves after the barrier)
    uint32_t bufA[S][IN_DW], bufB[S][IN_DW];
    if constexpr (LEAN == kChunkNone) loadTile(bufA, tile);
    // (the wave's number as the scalar it is: the lean instantiation branches around the layers of other waves)
    const int waveS = __builtin_amdgcn_readfirstlane(wave);

    // ---- stage weights (fragment order) and biases (fp16, kernel row order) into LDS -------
    // (each layer from another wave of the workgroup: the loads of the layers overlap.  The lean instantiations request
    // weights, biases and the first inputs and then wait once; the general one requests a thread's bias element, from an
    // address that always exists, before its weights, so that the first wait of the staging covers it)
    uint32_t chunk[L][RAW];     // (lean instantiations) a thread's chunk of every layer while its loads are in flight
    int chunkValid[L];
    if constexpr (LEAN != kChunkNone) {
        staticFor<0, L>([&](auto lc) {
            constexpr int l = decltype(lc)::value;
            constexpr int MT = Net::mt(l), KT = Net::kt(l), CHUNKS = MT * KT * 64;
            static_assert(CHUNKS <= 256, "one chunk per thread and layer");
            const MlpLayerArgs& ly = a.layers[l];
            const int c = (int)((threadIdx.x + 256u - (uint32_t)(Net::fragBase(l) * 64) % 256u) % 256u);
#pragma unroll
            for (int d = 0; d < RAW; ++d) chunk[l][d] = 0u;
            chunkValid[l] = 0;
            if (((waveS + 4 - Net::fragBase(l) % 4) & 3) * 64 < CHUNKS)        // (a wave skips the layers that are other waves')
                ChunkInFlight<ESZ, EPL, LEAN>::request(chunk[l], chunkValid[l], ly.w, ly.shape, MT, KT, optGS((uint32_t)ly.in),
                                                        (uint32_t)ly.out, (uint32_t)ly.in, c);
        });
    }
    uint16_t biasElem[L];
    staticFor<0, L>([&](auto lc) {
        constexpr int l = decltype(lc)::value;
        constexpr int MT = Net::mt(l), ROWS = 4 * MT;
        static_assert(MT * 16 <= 256, "one bias element per thread");
        const MlpLayerArgs& ly = a.layers[l];
        const int e = (int)((threadIdx.x + 256u - 64u * (l % 4)) % 256u);
        const int row = ((e >> 2) & 3) * ROWS + 4 * (e >> 4) + (e & 3);
        const bool have = e < MT * 16 && ly.bias && row < ly.out;
        if constexpr (LEAN != kChunkNone) {
            // (at its start the kernel waits once, for everything: a thread without an element skips the request)
            biasElem[l] = 0;
            if (((waveS + 4 - l % 4) & 3) * 64 < MT * 16) {
                if (have) biasElem[l] = ((const uint16_t*)ly.bias)[row];
            }
        } else {
            biasElem[l] = *(have ? (const uint16_t*)ly.bias + row : (const uint16_t*)a.out);   // (the output holds a half at least)
        }
    });
    if constexpr (LEAN != kChunkNone) {
        loadTile(bufA, tile);
        // (every request stands before this point and every use after it: left alone, the compiler moves a layer's
        // packing up into its request, and with it the wait for its loads)
#pragma unroll
        for (int l = 0; l < L; ++l)
#pragma unroll
            for (int d = 0; d < RAW; ++d) asm volatile("" : "+v"(chunk[l][d]) : : "memory");
        staticFor<0, L>([&](auto lc) {
            constexpr int l = decltype(lc)::value;
            constexpr int CHUNKS = Net::mt(l) * Net::kt(l) * 64;
            const int c = (int)((threadIdx.x + 256u - (uint32_t)(Net::fragBase(l) * 64) % 256u) % 256u);
            if (c < CHUNKS) ChunkInFlight<ESZ, EPL, LEAN>::finish(chunk[l], chunkValid[l], ldsW + (Net::fragBase(l) * 64 + c) * RAW);
        });
    } else {
        staticFor<0, L>([&](auto lc) {
            constexpr int l = decltype(lc)::value;
            constexpr int MT = Net::mt(l), KT = Net::kt(l);
            const MlpLayerArgs& ly = a.layers[l];
            const uint32_t gs = optGS((uint32_t)ly.in);
            uint32_t* base = ldsW + Net::fragBase(l) * 64 * RAW;
            stageFragments<ESZ, EPL>(base, ly.w, ly.shape, false, MT, KT, gs, (uint32_t)ly.out, (uint32_t)ly.in, 0, 0,
                                     (uint32_t)(Net::fragBase(l) * 64) % 256u);
        });
    }
    staticFor<0, L>([&](auto lc) {
        constexpr int l = decltype(lc)::value;
        constexpr int MT = Net::mt(l), ROWS = 4 * MT;
        const MlpLayerArgs& ly = a.layers[l];
        // bias of tile t, lane group g, r: row g*ROWS + 4t + r  ->  ldsB[(biasBase + t)*16 + 4g + r]
        const int e = (int)((threadIdx.x + 256u - 64u * (l % 4)) % 256u);
        const int t = e >> 4, g = (e >> 2) & 3, r = e & 3;
        const int row = g * ROWS + 4 * t + r;
        if (e < MT * 16) ldsB[(Net::biasBase(l) + t) * 16 + 4 * g + r] = (ly.bias && row < ly.out) ? biasElem[l] : (uint16_t)0;
    });
    __syncthreads();

    if (tile >= numTiles) return;

    // ---- weights and biases to registers ---------------------------------------------------
    uint32_t W[L][Net::MTMAX][Net::KTMAX][FD];
    uint32_t Bs[L][Net::MTMAX][2];          // 4 fp16 biases per tile, packed
    staticFor<0, L>([&](auto lc) {
        constexpr int l = decltype(lc)::value;
#pragma unroll
        for (int t = 0; t < Net::mt(l); ++t) {
#pragma unroll
            for (int kt = 0; kt < Net::kt(l); ++kt)
                Mma::decode(&ldsW[((Net::fragBase(l) + t * Net::kt(l) + kt) * 64 + lane) * RAW], W[l][t][kt]);
            const uint16_t* bp = &ldsB[(Net::biasBase(l) + t) * 16 + 4 * g];
            Bs[l][t][0] = (uint32_t)bp[0] | ((uint32_t)bp[1] << 16);
            Bs[l][t][1] = (uint32_t)bp[2] | ((uint32_t)bp[3] << 16);
        }
    });

    CarrierCfg cc[L];
    staticFor<0, L>([&](auto lc) {
        constexpr int l = decltype(lc)::value;
        cc[l] = makeCarrierCfg<Mma>(a.layers[l].act, a.layers[l].slope);
        if constexpr (l + 1 == L) {   // the last layer's output is not re-quantised: plain ReLU floor
            const half_t lo = a.layers[l].act == kActRelu ? (half_t)0.f : (half_t)-__builtin_inff();
            cc[l].floor2 = halfx2{lo, lo};
        }
    });

    auto computeStore = [&](const uint32_t (&buf)[S][IN_DW], uint32_t t0) {
#pragma unroll
        for (int r0 = 0; r0 < S; r0 += NT) {
            uint32_t act[NT][Net::KTMAX][FD];    // B fragments of the current layer's input
#pragma unroll
            for (int j = 0; j < NT; ++j)
#pragma unroll
                for (int kt = 0; kt < Net::KT0; ++kt) {
                    if constexpr (LEAN != kChunkNone) {
                        uint32_t own[RAW];
#pragma unroll
                        for (int d = 0; d < RAW; ++d) own[d] = 4 * (kt * RAW + d) < validBytes ? buf[r0 + j][kt * RAW + d] : 0u;
                        Mma::decode(own, act[j][kt]);
                    } else {
                        Mma::decode(&buf[r0 + j][kt * RAW], act[j][kt]);
                    }
                }

            staticFor<0, L>([&](auto lc) {
                constexpr int l = decltype(lc)::value;
                constexpr int MT = Net::mt(l), KT = Net::kt(l);
                floatx4 acc[NT][MT];
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    const halfx2 b01 = __builtin_bit_cast(halfx2, Bs[l][t][0]);
                    const halfx2 b23 = __builtin_bit_cast(halfx2, Bs[l][t][1]);
                    const floatx4 bv = {(float)b01.x, (float)b01.y, (float)b23.x, (float)b23.y};
#pragma unroll
                    for (int j = 0; j < NT; ++j) acc[j][t] = bv;
                }
#pragma unroll
                for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                    for (int t = 0; t < MT; ++t)
#pragma unroll
                        for (int j = 0; j < NT; ++j) acc[j][t] = Mma::mma(W[l][t][kt], act[j][kt], acc[j][t]);

                if constexpr (l + 1 < L) {
                    // this layer's output becomes the next layer's B operand, in place
                    constexpr int KTN = Net::kt(l + 1);
#pragma unroll
                    for (int j = 0; j < NT; ++j)
#pragma unroll
                        for (int kt = 0; kt < KTN; ++kt) {
                            halfx2 lo01, lo23, hi01 = {(half_t)0, (half_t)0}, hi23 = {(half_t)0, (half_t)0};
                            carrierFromAcc(acc[j][2 * kt], cc[l], lo01, lo23);
                            if (2 * kt + 1 < MT) carrierFromAcc(acc[j][2 * kt + 1 < MT ? 2 * kt + 1 : 0], cc[l], hi01, hi23);
                            fragFromCarrier<Mma>(lo01, lo23, hi01, hi23, cc[l], act[j][kt]);
                        }
                } else {
#pragma unroll
                    for (int j = 0; j < NT; ++j) {
                        const uint32_t sample = t0 * TILE + 16 * (r0 + j) + n;
                        if (sample >= a.batch || validRows <= 0) continue;
                        half_t* o = (half_t*)(outLane + (size_t)sample * a.outStride);
                        uint32_t pk[2 * MT];
#pragma unroll
                        for (int t = 0; t < MT; ++t) {
                            halfx2 p0, p1;
                            carrierFromAcc(acc[j][t], cc[l], p0, p1);
                            pk[2 * t] = __builtin_bit_cast(uint32_t, p0);
                            pk[2 * t + 1] = __builtin_bit_cast(uint32_t, p1);
                        }
                        if (vecStore) {
#pragma unroll
                            for (int t = 0; t < MT; ++t) {
                                const u32x2 v = {pk[2 * t], pk[2 * t + 1]};
                                ((u32x2*)o)[t] = v;
                            }
                        } else {
#pragma unroll
                            for (int e = 0; e < OROWS; ++e)
                                if (e < validRows) {
                                    const uint16_t bits = (uint16_t)(pk[e / 2] >> (16 * (e & 1)));
                                    o[e] = __builtin_bit_cast(half_t, bits);
                                }
                        }
                    }
                }
            });
        }
    };

    if constexpr (LEAN != kChunkNone) {
        // a wave with one super-tile, the launch-latency case, requests nothing more
        if (tile + tileStride >= numTiles) {
            computeStore(bufA, tile);
            return;
        }
    }
    while (true) {
        const uint32_t t1 = tile + tileStride;
        loadTile(bufB, t1 < numTiles ? t1 : tile);
        computeStore(bufA, tile);
        if (t1 >= numTiles) break;
        const uint32_t t2 = t1 + tileStride;
        loadTile(bufA, t2 < numTiles ? t2 : t1);
        computeStore(bufB, t1);
        if (t2 >= numTiles) break;
        tile = t2;
    }
}

#ifndef CV_MLP_PREFETCH_DW
#define CV_MLP_PREFETCH_DW 8      // input dwords per lane held in flight per buffer
#endif

// true when no layer of the network has more lane-chunks than a workgroup has threads (what the lean instantiations of
// mlpForwardKernel assume)
template <class Net>
constexpr bool oneChunkPerThread()
{
    for (int l = 0; l < Net::L; ++l)
        if (Net::mt(l) * Net::kt(l) * 64 > 256) return false;
    return true;
}

template <class Mma, class Net>
hipError_t launchMlpNet(hipStream_t stream, const MlpArgs& a, int numCUs)
{
    // tiles pushed through the layers together (independent MFMA chains), limited by registers
    // (with all weights in registers, wide networks run faster with one tile per round and a
    // second wave on the SIMD than with two tiles and a single wave: 63 us vs 79 us for 8-64x4-1)
    constexpr int NT = (Net::totalFrags * Mma::kFD <= 32) ? 4 : (Net::totalFrags * Mma::kFD <= 64 ? 2 : 1);
    constexpr int IN_DW = Mma::kRawDW * Net::KT0;
    constexpr int S0 = CV_MLP_PREFETCH_DW / IN_DW;
    constexpr int S = S0 < NT ? NT : (S0 > 16 ? 16 : S0 / NT * NT);
    // the small networks, whose calls are the ones bound by launch latency, have the lean instantiations
    int lean = kChunkNone;
    constexpr bool kLean = NT == 4 && oneChunkPerThread<Net>();
    if (kLean && a.inEncoding == kEncodeNone && !a.inHalfAsE4M3 && a.inAlign >= 4u && (a.layers[0].in * Mma::kEsz) % 4 == 0) {
        for (int l = 0; l < Net::L; ++l) {
            const MlpLayerArgs& ly = a.layers[l];
            const int kind = chunkInFlightKind<Mma::kEsz, Mma::kEpl>(ly.w, ly.shape, Net::mt(l), Net::kt(l), optGS((uint32_t)ly.in),
                                                                      (uint32_t)ly.out, (uint32_t)ly.in);
            lean = l == 0 || kind == lean ? kind : kChunkNone;
            if (lean == kChunkNone) break;
        }
    }
    const int blocksPerCU = residentBlocksPerCU<mlpForwardKernel<Mma, Net, NT, S, kChunkNone>>(256);
    const uint32_t tile = 16 * S;
    const uint32_t numTiles = (a.batch + tile - 1) / tile;
    const uint32_t blocksNeeded = (numTiles + 3) / 4;
    const uint32_t blocksMax = (uint32_t)numCUs * (uint32_t)blocksPerCU;
    const uint32_t blocks = blocksNeeded < blocksMax ? blocksNeeded : blocksMax;
    noteKernel(false, "mlpForwardKernel<%s,KT0=%d,HT=%d,hidden=%d,MTL=%d,NT=%d,S=%d%s>", Mma::kName, Net::KT0, Net::HT,
               Net::L - 1, Net::MTL, NT, S, lean == kChunkRowDwords ? ",lean,RowMajor" : lean == kChunkDirect ? ",lean,InferencingOptimal" : "");
    if constexpr (kLean) {
        if (lean == kChunkRowDwords) {
            hipLaunchKernelGGL((mlpForwardKernel<Mma, Net, NT, S, kChunkRowDwords>), dim3(blocks), dim3(256), 0, stream, a);
            return hipGetLastError();
        }
        if (lean == kChunkDirect) {
            hipLaunchKernelGGL((mlpForwardKernel<Mma, Net, NT, S, kChunkDirect>), dim3(blocks), dim3(256), 0, stream, a);
            return hipGetLastError();
        }
    }
    hipLaunchKernelGGL((mlpForwardKernel<Mma, Net, NT, S, kChunkNone>), dim3(blocks), dim3(256), 0, stream, a);
    return hipGetLastError();
}

// streaming instantiation for full-width contiguous inputs (cv_mlp_stream.h)
template <class Mma, class Net> bool mlpStreamEligible(const MlpArgs& a);
template <class Mma, class Net> hipError_t launchMlpStream(hipStream_t stream, const MlpArgs& a, int numCUs);

// The specialisations built into the library: (input k-tiles, hidden tiles, hidden layers,
// output tiles).  Dimensions smaller than a tile are padded with zeros at run time.
#ifndef CV_MLP_SHAPES
#define CV_MLP_SHAPES(X) \
    X(1, 1, 1, 1) X(1, 1, 2, 1) X(1, 1, 3, 1) \
    X(1, 2, 1, 1) X(1, 2, 2, 1) X(1, 2, 3, 1) X(1, 2, 1, 2) X(1, 2, 2, 2) X(1, 2, 3, 2) \
    X(1, 4, 1, 1) X(1, 4, 2, 1) X(1, 4, 3, 1) X(1, 4, 4, 1) X(1, 4, 2, 4) X(1, 4, 3, 4) \
    X(2, 4, 1, 4) X(2, 4, 2, 4) X(2, 4, 3, 4) X(2, 4, 2, 1)
#endif

template <class Mma>
hipError_t dispatchMlp(hipStream_t stream, const MlpArgs& a, int numCUs)
{
    const int L = a.numLayers;
    if (L < 2) return hipErrorInvalidValue;
    for (int l = 0; l < L; ++l)
        if (a.layers[l].act >= kActSigmoid) return hipErrorInvalidValue;     // smooth activations: general kernel
    const int kt0 = (int)optKT((uint32_t)a.layers[0].in, Mma::kEpl);
    const int ht = (int)optMT((uint32_t)a.layers[0].out);
    for (int l = 1; l + 1 < L; ++l)
        if ((int)optMT((uint32_t)a.layers[l].out) != ht) return hipErrorInvalidValue;
    const int mtl = (int)optMT((uint32_t)a.layers[L - 1].out);
#define CV_X(K0, HT, NH, ML) \
    if (kt0 <= K0 && (K0 == 1 || kt0 == K0) && ht == HT && L - 1 == NH && mtl == ML) { \
        typedef UniformNet<K0, HT, NH, ML> N_; \
        return mlpStreamEligible<Mma, N_>(a) ? launchMlpStream<Mma, N_>(stream, a, numCUs) \
                                             : launchMlpNet<Mma, N_>(stream, a, numCUs); \
    }
    CV_MLP_SHAPES(CV_X)
#undef CV_X
    return hipErrorInvalidValue;
}

} // namespace
} // namespace cv
