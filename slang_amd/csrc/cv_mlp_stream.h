// cv_mlp_stream.h -- streaming instantiation of the fused forward MLP for gfx950.
//
// Same arithmetic as mlpForwardKernel (cv_mlp_impl.h), different data movement, for the case
// that dominates inference: full-width, contiguous, 16-byte aligned input rows.  Narrow rows
// (e.g. 32 e4m3 bytes per sample) need many samples in flight to keep HBM busy and many waves
// per SIMD to keep the VALU/MFMA pipes busy, so here
//   - a wave fetches a slot of S*16 samples with fully coalesced 16-byte loads (lane l reads
//     bytes [16l, 16l+16) of every 1 KB chunk) into a handful of staging registers, a whole
//     slot ahead of the arithmetic;
//   - the slot is dropped into a per-wave LDS buffer and read back in MFMA operand order
//     (lane (g,n): its quarter of sample n), NT tiles at a time, in a rolled loop: small code,
//     few live registers, 2-4 waves per SIMD;
//   - biases are compiled out when no layer has one;
//   - IN_HALF (e4m3 networks): the rows in memory are fp16 vectors (CoopVec<half> with
//     inputInterpretation FloatE4M3) and are quantised to e4m3 as they are read back from LDS.
#pragma once
#include "cv_mlp_impl.h"

namespace cv {
namespace {

// carrier for ReLU / no activation only (the launcher sends leaky-ReLU networks to the general
// kernel): no per-tile branch in the round loop
__device__ __forceinline__ void carrierNoLeaky(const floatx4& acc, const CarrierCfg& c, halfx2& h01, halfx2& h23)
{
    typedef float floatx2 __attribute__((ext_vector_type(2)));
    h01 = __builtin_elementwise_max(__builtin_convertvector(floatx2{acc[0], acc[1]}, halfx2), c.floor2);
    h23 = __builtin_elementwise_max(__builtin_convertvector(floatx2{acc[2], acc[3]}, halfx2), c.floor2);
}

#ifndef CV_MLP_STREAM_MINWAVES
#define CV_MLP_STREAM_MINWAVES 1
#endif
template <class Mma, class Net, int NT, int S, bool HAS_BIAS, bool IN_HALF = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(CV_MLP_STREAM_MINWAVES))) void mlpStreamKernel(const MlpArgs a)
{
    constexpr int EPL = Mma::kEpl, FD = Mma::kFD, ESZ = Mma::kEsz, RAW = Mma::kRawDW;
    constexpr int L = Net::L;
    constexpr bool QUANT = !std::is_same<Mma, F16Mma>::value;   // e4m3 carrier between layers
    constexpr int IN_DW = RAW * Net::KT0;          // dwords one lane contributes per sample tile
    constexpr int LANE_DW = IN_HALF ? 2 * IN_DW : IN_DW;   // dwords of a lane's quarter of a row as it lies in memory
    constexpr int ROW_DW = 4 * LANE_DW;            // dwords of one sample's input row
    constexpr int SLOT_DW = S * 16 * ROW_DW;       // dwords of one slot
    static_assert(!IN_HALF || (!std::is_same<Mma, F16Mma>::value && Mma::kEsz == 1), "fp16 rows are quantised for e4m3 networks only");
    constexpr int CH = SLOT_DW / 256;              // 1 KB chunks per slot
    static_assert(SLOT_DW % 256 == 0 && S % NT == 0, "slot must be whole 1 KB chunks and whole rounds");

    __shared__ __attribute__((aligned(16))) uint32_t ldsW[Net::totalFrags * 64 * RAW];
    __shared__ __attribute__((aligned(16))) uint16_t ldsB[Net::totalBiasTiles * 16];
    __shared__ __attribute__((aligned(16))) uint32_t ldsIn[4 * SLOT_DW];

    // ---- stage weights (fragment order) and biases into LDS (as in mlpForwardKernel) ---------
    staticFor<0, L>([&](auto lc) {
        constexpr int l = decltype(lc)::value;
        constexpr int MT = Net::mt(l), KT = Net::kt(l), ROWS = 4 * MT;
        const MlpLayerArgs& ly = a.layers[l];
        const uint32_t gs = optGS((uint32_t)ly.in);
        uint32_t* base = ldsW + Net::fragBase(l) * 64 * RAW;
        stageFragments<ESZ, EPL>(base, ly.w, ly.shape, false, MT, KT, gs, (uint32_t)ly.out, (uint32_t)ly.in);
        if constexpr (HAS_BIAS) {
            for (int e = threadIdx.x; e < MT * 16; e += 256) {
                const int t = e >> 4, g = (e >> 2) & 3, r = e & 3;
                const int row = g * ROWS + 4 * t + r;
                uint16_t v = 0;
                if (ly.bias && row < ly.out) v = ((const uint16_t*)ly.bias)[row];
                ldsB[(Net::biasBase(l) + t) * 16 + 4 * g + r] = v;
            }
        }
    });
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, n = lane & 15;

    uint32_t W[L][Net::MTMAX][Net::KTMAX][FD];
    uint32_t Bs[L][Net::MTMAX][2];
    CarrierCfg cc[L];
    staticFor<0, L>([&](auto lc) {
        constexpr int l = decltype(lc)::value;
#pragma unroll
        for (int t = 0; t < Net::mt(l); ++t) {
#pragma unroll
            for (int kt = 0; kt < Net::kt(l); ++kt)
                Mma::decode(&ldsW[((Net::fragBase(l) + t * Net::kt(l) + kt) * 64 + lane) * RAW], W[l][t][kt]);
            if constexpr (HAS_BIAS) {
                const uint16_t* bp = &ldsB[(Net::biasBase(l) + t) * 16 + 4 * g];
                Bs[l][t][0] = (uint32_t)bp[0] | ((uint32_t)bp[1] << 16);
                Bs[l][t][1] = (uint32_t)bp[2] | ((uint32_t)bp[3] << 16);
            }
        }
        cc[l] = makeCarrierCfg<Mma>(a.layers[l].act, a.layers[l].slope);
        if constexpr (l + 1 == L) {   // the last layer's output is not re-quantised: plain ReLU floor
            const half_t lo = a.layers[l].act == kActRelu ? (half_t)0.f : (half_t)-__builtin_inff();
            cc[l].floor2 = halfx2{lo, lo};
        }
    });

    constexpr int OROWS = 4 * Net::MTL;
    const int outDim = a.layers[L - 1].out;
    const bool hasRows = g * OROWS < outDim;       // the launcher guarantees outDim % OROWS == 0
    uint8_t* outLane = a.out + (size_t)(g * OROWS) * 2;

    constexpr uint32_t SLOT = 16 * S;              // samples per slot
    const uint32_t numSlots = (a.batch + SLOT - 1) / SLOT;
    const uint32_t slotStride = gridDim.x * 4;
    uint32_t slot = blockIdx.x * 4 + wave;
    if (slot >= numSlots) return;
    const uint64_t totalBytes = (uint64_t)a.batch * (ROW_DW * 4);
    uint32_t* myIn = ldsIn + wave * SLOT_DW;

    uint32_t stg[CH][4];
    auto fetch = [&](uint32_t sl) {
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            // clamp the last, partial slot to the end of the input (those samples are not stored)
            uint64_t off = (uint64_t)sl * (SLOT_DW * 4) + (uint64_t)c * 1024 + (uint64_t)lane * 16;
            off = off + 16 <= totalBytes ? off : totalBytes - 16;
            const u32x4 v = loadStream16(a.in + off);
            stg[c][0] = v.x; stg[c][1] = v.y; stg[c][2] = v.z; stg[c][3] = v.w;
        }
    };

    fetch(slot);
    for (; slot < numSlots; slot += slotStride) {
        // staging registers -> LDS; then the registers take the next slot
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const u32x4 v = {stg[c][0], stg[c][1], stg[c][2], stg[c][3]};
            *(u32x4*)(myIn + c * 256 + lane * 4) = v;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        {
            const uint32_t nextSlot = slot + slotStride;
            fetch(nextSlot < numSlots ? nextSlot : slot);
        }

#pragma unroll 1
        for (int r0 = 0; r0 < S; r0 += NT) {
            uint32_t act[NT][Net::KTMAX][FD];
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                const uint32_t* src = myIn + ((r0 + j) * 16 + n) * ROW_DW + g * LANE_DW;
                uint32_t mem[LANE_DW];
                if constexpr (LANE_DW % 4 == 0) {
#pragma unroll
                    for (int i = 0; i < LANE_DW / 4; ++i) {
                        const u32x4 v = *(const u32x4*)(src + 4 * i);
                        mem[4 * i] = v.x; mem[4 * i + 1] = v.y; mem[4 * i + 2] = v.z; mem[4 * i + 3] = v.w;
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < LANE_DW / 2; ++i) {
                        const u32x2 v = *(const u32x2*)(src + 2 * i);
                        mem[2 * i] = v.x; mem[2 * i + 1] = v.y;
                    }
                }
                uint32_t raw[IN_DW];
                if constexpr (!IN_HALF) {
#pragma unroll
                    for (int i = 0; i < IN_DW; ++i) raw[i] = mem[i];
                }
                if constexpr (QUANT) {
                    // from here to the last layer's accumulators the conversions saturate by mode
                    if (j == 0) {
#pragma unroll
                        for (int i = 0; i < LANE_DW; ++i) pinHere(mem[i]);
                        setFp16OverflowClamp<true>();
                    }
#pragma unroll
                    for (int i = 0; i < LANE_DW; ++i) pinHere(mem[i]);
                    if constexpr (IN_HALF) {
                        // four halves -> four e4m3 bytes (saturating by mode, nearest even)
#pragma unroll
                        for (int i = 0; i < IN_DW; ++i)
                            raw[i] = quantE4M3x4<true>(__builtin_bit_cast(halfx2, mem[2 * i]), __builtin_bit_cast(halfx2, mem[2 * i + 1]), cc[0]);
                    } else {
#pragma unroll
                        for (int i = 0; i < IN_DW; ++i) raw[i] = mem[i];
                    }
                }
#pragma unroll
                for (int kt = 0; kt < Net::KT0; ++kt) Mma::decode(&raw[kt * RAW], act[j][kt]);
            }

            staticFor<0, L>([&](auto lc) {
                constexpr int l = decltype(lc)::value;
                constexpr int MT = Net::mt(l), KT = Net::kt(l);
                floatx4 acc[NT][MT];
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    floatx4 bv = {0.f, 0.f, 0.f, 0.f};
                    if constexpr (HAS_BIAS) {
                        const halfx2 b01 = __builtin_bit_cast(halfx2, Bs[l][t][0]);
                        const halfx2 b23 = __builtin_bit_cast(halfx2, Bs[l][t][1]);
                        bv = floatx4{(float)b01.x, (float)b01.y, (float)b23.x, (float)b23.y};
                    }
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
                    constexpr int KTN = Net::kt(l + 1);
#pragma unroll
                    for (int j = 0; j < NT; ++j)
#pragma unroll
                        for (int kt = 0; kt < KTN; ++kt) {
                            halfx2 lo01, lo23, hi01 = {(half_t)0, (half_t)0}, hi23 = {(half_t)0, (half_t)0};
                            carrierNoLeaky(acc[j][2 * kt], cc[l], lo01, lo23);
                            if (2 * kt + 1 < MT) carrierNoLeaky(acc[j][2 * kt + 1 < MT ? 2 * kt + 1 : 0], cc[l], hi01, hi23);
                            fragFromCarrier<Mma, QUANT>(lo01, lo23, hi01, hi23, cc[l], act[j][kt]);
                        }
                } else {
                    if constexpr (QUANT) {
                        // the network's fp16 output keeps inf for an overflow: mode off before it is formed
#pragma unroll
                        for (int j = 0; j < NT; ++j)
#pragma unroll
                            for (int t = 0; t < MT; ++t) pinHere(acc[j][t]);
                        setFp16OverflowClamp<false>();
#pragma unroll
                        for (int j = 0; j < NT; ++j)
#pragma unroll
                            for (int t = 0; t < MT; ++t) pinHere(acc[j][t]);
                    }
#pragma unroll
                    for (int j = 0; j < NT; ++j) {
                        const uint32_t sample = slot * SLOT + 16 * (r0 + j) + n;
                        if (sample < a.batch && hasRows) {
                            u32x2* o = (u32x2*)(outLane + (size_t)sample * a.outStride);
#pragma unroll
                            for (int t = 0; t < MT; ++t) {
                                halfx2 p0, p1;
                                carrierNoLeaky(acc[j][t], cc[l], p0, p1);
                                const u32x2 v = {__builtin_bit_cast(uint32_t, p0), __builtin_bit_cast(uint32_t, p1)};
                                storeStream8(&o[t], v);      // (written once, read by nobody here)
                            }
                        }
                    }
                }
            });
        }
        // the next iteration overwrites the LDS slot: every lane must be done reading it
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

#ifndef CV_MLP_STREAM_SLOT_DW
#define CV_MLP_STREAM_SLOT_DW 1024    // dwords of input per slot and wave (4 KB)
#endif

// true when the streaming kernel can take this call
template <class Mma, class Net>
bool mlpStreamEligible(const MlpArgs& a)
{
    const bool inHalf = a.inHalfAsE4M3 != 0;
    if (inHalf && (std::is_same<Mma, F16Mma>::value || Mma::kEsz != 1)) return false;
    const int rowBytes = 16 * Mma::kRawDW * Net::KT0 * (inHalf ? 2 : 1);
    const int outDim = a.layers[Net::L - 1].out;
    if (a.inEncoding != kEncodeNone) return false;
    for (int l = 0; l < Net::L; ++l)
        if (a.layers[l].act == kActLeakyRelu) return false;
    return a.layers[0].in * (inHalf ? 2 : Mma::kEsz) == rowBytes && a.inStride == (uint64_t)rowBytes &&
           ((uintptr_t)a.in & 15u) == 0 && outDim % (4 * Net::MTL) == 0 && a.outAlign >= 8u &&
           (uint64_t)a.batch * rowBytes >= 16;
}

template <class Mma, class Net, bool HAS_BIAS, bool IN_HALF>
hipError_t launchMlpStreamB(hipStream_t stream, const MlpArgs& a, int numCUs)
{
#ifdef CV_MLP_STREAM_NT
    constexpr int NT = CV_MLP_STREAM_NT;
#else
    constexpr int NT = (Net::totalFrags * Mma::kFD <= 32) ? 4 : 2;
#endif
    constexpr int ROW_DW = 4 * Mma::kRawDW * Net::KT0 * (IN_HALF ? 2 : 1);
    constexpr int S0 = CV_MLP_STREAM_SLOT_DW / (16 * ROW_DW);
    constexpr int S = S0 < NT ? NT : S0 / NT * NT;
    const int blocksPerCU = residentBlocksPerCU<mlpStreamKernel<Mma, Net, NT, S, HAS_BIAS, IN_HALF>>(256);
    const uint32_t slot = 16 * S;
    const uint32_t numSlots = (a.batch + slot - 1) / slot;
    const uint32_t blocksNeeded = (numSlots + 3) / 4;
    const uint32_t blocksMax = (uint32_t)numCUs * (uint32_t)blocksPerCU;
    const uint32_t blocks = blocksNeeded < blocksMax ? blocksNeeded : blocksMax;
    noteKernel(false, "mlpStreamKernel<%s,KT0=%d,HT=%d,hidden=%d,MTL=%d,NT=%d,S=%d,%s%s>", Mma::kName, Net::KT0, Net::HT,
               Net::L - 1, Net::MTL, NT, S, HAS_BIAS ? "bias" : "nobias", IN_HALF ? ",fp16-vectors" : "");
    hipLaunchKernelGGL((mlpStreamKernel<Mma, Net, NT, S, HAS_BIAS, IN_HALF>), dim3(blocks), dim3(256), 0, stream, a);
    return hipGetLastError();
}

template <class Mma, class Net>
hipError_t launchMlpStream(hipStream_t stream, const MlpArgs& a, int numCUs)
{
    bool hasBias = false;
    for (int l = 0; l < Net::L; ++l) hasBias = hasBias || a.layers[l].bias != nullptr;
    if constexpr (!std::is_same<Mma, F16Mma>::value && Mma::kEsz == 1) {
        if (a.inHalfAsE4M3)
            return hasBias ? launchMlpStreamB<Mma, Net, true, true>(stream, a, numCUs)
                           : launchMlpStreamB<Mma, Net, false, true>(stream, a, numCUs);
    }
    return hasBias ? launchMlpStreamB<Mma, Net, true, false>(stream, a, numCUs)
                   : launchMlpStreamB<Mma, Net, false, false>(stream, a, numCUs);
}

} // namespace
} // namespace cv
