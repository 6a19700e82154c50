// cv_train_pair.h -- the fused training step with two waves per SIMD.
//
// Same computation and rounding points as mlpTrainKernel (cv_train_impl.h), reorganised so that
// the dW accumulators of the network are shared by a pair of waves instead of living in one:
//
//   - a workgroup is four pairs of waves; a pair takes rounds of 32 samples, wave 0 of the pair
//     the first 16, wave 1 the other 16.  Forward, loss and dX = W^T dY run per wave on its 16
//     samples exactly as in the one-wave kernel ("S" orientation: lane%16 = sample);
//   - every layer input X_l and every dZ_l is also written to LDS as it is produced, as
//     [32 samples][16 features] tiles of fp16.  The weight gradient dW_l = sum_s dZ_l (x) X_l
//     needs both with the sample index on the MFMA k axis ("F" orientation: lane%16 = feature):
//     ds_read_b64_tr_b16 delivers that transposition directly from those tiles (no
//     selection-matrix MFMAs, no conversions);
//   - each wave of the pair accumulates half of the dW tiles of every layer over all 32 samples
//     of the round (its own 16 and its partner's), so a wave holds half of the accumulators
//     (112 instead of 224 registers for 8-64-64-64-64-1) and two waves fit on a SIMD: the one
//     covers the other's LDS and MFMA latencies.  The accumulators are ordinary VGPRs here: a
//     kernel that names no AGPR may use all 256 registers of its share as VGPRs, while one that
//     does gets them split evenly, which is too few VGPRs for the rest of the round.
//
// The two waves of a pair meet once per layer in the backward pass (dZ_l of both halves must be in
// LDS before either wave contracts over it) and once per round.  Only the pair meets, through a
// sequence number each wave publishes in LDS (pairPublish, pairAwait), not the workgroup at s_barrier: the four
// pairs of a workgroup drift apart, so that the two waves of a SIMD, which belong to different
// pairs, are in different phases of the round and want different units.  The two waves of a pair run
// the same rounds (a round past the end of the batch is run with all samples masked), so their
// sequence numbers always match; the pairs of a workgroup take different numbers of rounds (below).  Partials and their second-stage reduction are those of the
// one-wave kernel (mlpTrainReduceKernel): same layout, fixed order, no atomics.
#pragma once
#include "cv_train_impl.h"

namespace cv {
namespace {

// which dW tiles of layer l a wave of parity `par` accumulates
template <class Net>
struct PairSplit {
    static constexpr int L = Net::L;
    static constexpr bool byOut(int l) { return Net::mt(l) >= 2; }                       // split the out tiles
    static constexpr bool byIn(int l) { return Net::mt(l) < 2 && Net::nIt(l) >= 2; }      // else split the in tiles
    static constexpr bool single(int l) { return Net::mt(l) < 2 && Net::nIt(l) < 2; }     // else wave 0 alone
    static constexpr int ownedOut(int l) { return byOut(l) ? Net::mt(l) / 2 : 1; }
    static constexpr int ownedIn(int l) { return byIn(l) ? Net::nIt(l) / 2 : Net::nIt(l); }
    static constexpr int locTiles(int l) { return ownedOut(l) * ownedIn(l); }
    static constexpr int locBase(int l)
    {
        int b = 0;
        for (int i = 0; i < l; ++i) b += locTiles(i);
        return b;
    }
    static constexpr int totalLoc = locBase(L);
    static constexpr int locDbBase(int l)
    {
        int b = 0;
        for (int i = 0; i < l; ++i) b += ownedOut(i);
        return b;
    }
    static constexpr int totalLocDb = locDbBase(L);
    static constexpr int layerOfLoc(int q)          // the layer a wave's q-th dW tile belongs to
    {
        int l = 0;
        while (l + 1 < L && locBase(l + 1) <= q) ++l;
        return l;
    }
    static constexpr int layerOfLocDb(int q)
    {
        int l = 0;
        while (l + 1 < L && locDbBase(l + 1) <= q) ++l;
        return l;
    }
};

// LDS tile of one 16-feature group over the 32 samples of a round, 1 KB, in 8-byte chunks of four
// features: chunk c (features 4c..4c+3) of sample s sits at chunk index 32c + (s ^ k_c), k = {0, 24, 12, 20}.
// With that swizzle both access patterns are free of bank conflicts whether the LDS serves 16 or 32
// lanes of an 8-byte access per pass: a 16-lane group writes one chunk column of 16 consecutive
// samples (a permutation of 16 consecutive slots; the columns c and c+1 of the neighbouring group
// land in the other half of the 32 slots), and reads, transposed, the four chunks of four
// consecutive samples (four different 4-slot blocks modulo 16, and for two neighbouring groups
// eight different ones modulo 32).
constexpr int kPairTileDW = 256;
__device__ __forceinline__ int pairChunkDW(int sample, int c)
{
    const int k = (0x14 << 24 | 0x0c << 16 | 0x18 << 8 | 0x00) >> (8 * c) & 0xff;
    return (c * 32 + (sample ^ k)) * 2;
}

// Transposed read of one F fragment (feature = lane%16, k-slots = 8 samples) from such a tile.
// Lane 16g+i receives feature i of samples 4g..4g+3 (first instruction) and 16+4g..16+4g+3 (second):
// within a 16-lane group, lane q hands in the address of the 8-byte chunk (sample 4g + q/4, features
// 4(q%4)..), and the instruction returns to lane i element r = half i%4 of the chunk of lane 4r + i/4.
__device__ __forceinline__ void readF(const uint32_t* tile, int g, int n, uint32_t* frag)
{
    typedef short shortx4 __attribute__((ext_vector_type(4)));
    typedef shortx4 __attribute__((address_space(3))) * LdsPtr;
    const shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsPtr)(tile + pairChunkDW(4 * g + (n >> 2), n & 3)));
    const shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsPtr)(tile + pairChunkDW(16 + 4 * g + (n >> 2), n & 3)));
    const u32x2 a = __builtin_bit_cast(u32x2, lo), b = __builtin_bit_cast(u32x2, hi);
    frag[0] = a.x; frag[1] = a.y; frag[2] = b.x; frag[3] = b.y;
}

// Meeting of the two waves of a pair, in two halves.  `mine` and `theirs` are the LDS words of this
// wave and of its partner; `seq` counts the meetings and is the same in both waves.  A wave
// publishes the number as soon as its part is done and awaits the partner's as late as it can, with
// work that needs nothing from the partner in between, so that the number has usually arrived.
// LDS executes the instructions of one wave in the order they were issued: the tile accesses above
// pairPublish are complete when the partner sees the number; the compiler is kept from moving LDS
// accesses across either call.  The wait is bounded: a partner that never arrives (which would be a defect of the kernel)
// costs a wrong result (the return value says so), not a hung GPU.
constexpr uint32_t kPairSpinLimit = 1u << 20;
typedef uint32_t __attribute__((address_space(3))) LdsWord;
__device__ __forceinline__ void pairPublish(volatile LdsWord* mine, uint32_t seq)
{
    asm volatile("" ::: "memory");
    *mine = seq;
}
__device__ __forceinline__ uint32_t pairAwait(const volatile LdsWord* theirs, uint32_t seq)
{
    uint32_t spins = 0;
#pragma nounroll
    while ((uint32_t)__builtin_amdgcn_readfirstlane((int)*theirs) < seq && spins < kPairSpinLimit) ++spins;
    asm volatile("" ::: "memory");
    return spins / kPairSpinLimit;      // 1 after a time-out
}

// ReLU on the hidden layers, none on the last one (the launcher sends everything else to the
// one-wave kernel); LOADS as in mlpTrainKernel.
// LEAKY: each hidden layer ReLU or leaky ReLU and the last layer none, ReLU or leaky ReLU, as the arguments say
// (max(z, z * slope) with the slope as a half, the multiplier of applyActGrad on the way back: fflayer.slang:60-66);
// without it every hidden layer is ReLU and the last layer has no activation.
template <class Net, int LOADS, bool LEAKY = false>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void mlpTrainPairKernel(const TrainArgs ta)
{
    typedef F16Mma Mma;
    typedef PairSplit<Net> Split;
    constexpr int L = Net::L;
    constexpr int FD = 4, RAW = 4, EPL = 8;
    constexpr int IN_DW = RAW * Net::KT0;
    const MlpArgs& a = ta.mlp;

    // One LDS array, carved by hand: the weights and biases come first so that every read of them is
    // the lane's base address plus an immediate offset (the 16-bit offset field reaches 64 KB; arrays
    // placed beyond that by the compiler cost an address register per fragment).
    constexpr int W_DW = Net::totalFrags * 64 * RAW;
    constexpr int WT_DW = (Net::totalTFrags > 0 ? Net::totalTFrags : 1) * 64 * RAW;
    constexpr int B_DW = Net::totalBiasTiles * 16;
    constexpr int X_DW = 4 * Net::totalXTiles * kPairTileDW;          // per pair: every layer's input of the round
    constexpr int DZ_DW = 4 * 2 * Net::MTMAX * kPairTileDW;           // per pair: two alternating slots for dZ
    constexpr int FLAG_DW = 8;                                        // per wave: the number of its last meeting
    constexpr int MAX_DW = 4;                                         // the workgroup's largest per-sample loss (one word used)
    static_assert((W_DW + WT_DW + B_DW + X_DW + DZ_DW + FLAG_DW + MAX_DW) * 4 <= 160 * 1024, "LDS of one compute unit");
    __shared__ __attribute__((aligned(16))) uint32_t lds[W_DW + WT_DW + B_DW + X_DW + DZ_DW + FLAG_DW + MAX_DW];
    uint32_t* const ldsW = lds;
    uint32_t* const ldsWT = lds + W_DW;
    float* const ldsB = (float*)(lds + W_DW + WT_DW);
    uint32_t* const ldsX = lds + W_DW + WT_DW + B_DW;
    uint32_t* const ldsDZ = ldsX + X_DW;
    uint32_t* const ldsFlag = ldsDZ + DZ_DW;
    uint32_t* const ldsLossMax = ldsFlag + FLAG_DW;
    if (threadIdx.x < FLAG_DW + MAX_DW) ldsFlag[threadIdx.x] = 0u;

    stageTrainingWeights<Net, 512>(a, ldsW, ldsWT, ldsB);

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int pair = wave >> 1, par = wave & 1;      // partners sit on neighbouring SIMDs
    const int g = lane >> 4, n = lane & 15;
    const halfx2 ones2 = {(half_t)1.f, (half_t)1.f};

    floatx4 accW[Split::totalLoc];
    float accB[Split::totalLocDb];
#pragma unroll
    for (int i = 0; i < Split::totalLoc; ++i) accW[i] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < Split::totalLocDb; ++i) accB[i] = 0.f;
    float lossAcc = 0.f, lossMaxAcc = 0.f;

    // ---- per-lane constants ----------------------------------------------------------------------
    const int in0 = a.layers[0].in;
    const uint32_t gs0 = optGS((uint32_t)in0);
    const int colBase = (int)(g * gs0);
    const int validBytes = min((int)gs0, max(in0 - colBase, 0)) * 2;
    const int outDim = a.layers[L - 1].out;
    constexpr int OROWS = 4 * Net::MTL;

    // Rounds blockIdx.x + j * gridDim.x belong to this workgroup; its four pairs share them unevenly.  A SIMD
    // favours its older wave, and the waves of pairs 0 and 1 are the older ones on all four SIMDs: with equal
    // shares they were done after 105 us and left pairs 2 and 3 to run alone, one wave per SIMD, for another
    // 30 us.  With 37 : 27 the four pairs end together (146 -> 138 us for 8-64x4-1 at batch 2^20; 36 and 38 are
    // within 1 %).  The split is a function of the pair's index, so results stay bitwise reproducible.
#ifndef CV_TRAIN_PAIR_OLD_SHARE
#define CV_TRAIN_PAIR_OLD_SHARE 37      // of 128: the share of each of the pairs 0 and 1 (pairs 2 and 3 get 64 minus that)
#endif
    const uint32_t numRounds = (a.batch + 31u) / 32u;
    const uint32_t blockRounds = blockIdx.x < numRounds ? (numRounds - blockIdx.x + gridDim.x - 1u) / gridDim.x : 0u;
    constexpr uint32_t kOld = CV_TRAIN_PAIR_OLD_SHARE, kYoung = 64u - kOld;
    const uint32_t cumLo = pair == 0 ? 0u : pair == 1 ? kOld : pair == 2 ? 2u * kOld : 2u * kOld + kYoung;
    const uint32_t cumHi = pair == 0 ? kOld : pair == 1 ? 2u * kOld : pair == 2 ? 2u * kOld + kYoung : 128u;
    const uint32_t firstRound = blockRounds * cumLo / 128u, endRound = blockRounds * cumHi / 128u;
    const uint32_t roundsPerPair = endRound - firstRound;     // the same for both waves of a pair
    const uint32_t lastSample = a.batch - 1;
    uint32_t* myX = ldsX + pair * (Net::totalXTiles * kPairTileDW);
    uint32_t* myDZ = ldsDZ + pair * (2 * Net::MTMAX * kPairTileDW);
    // where this lane puts its four halves of a tile (S fragment half: sample 16*par+n, rows 4g..4g+3) ...
    const int putDW = pairChunkDW(16 * par + n, g);
    volatile LdsWord* const myFlag = (LdsWord*)(ldsFlag + wave);
    const volatile LdsWord* const partnerFlag = (LdsWord*)(ldsFlag + (wave ^ 1));
    uint32_t meetings = 0, timeouts = 0;

    auto loadTile = [&](uint32_t (&raw)[IN_DW], uint32_t r) {
        const uint32_t s = min(r * 32u + 16u * par + n, lastSample);
        const uint8_t* row = a.in + (size_t)s * a.inStride;
        const uint8_t* p = row + (size_t)colBase * 2;
        if constexpr (LOADS == kLoadXY) {
#pragma unroll
            for (int i = 0; i < IN_DW; ++i) raw[i] = i < 2 ? ((const uint32_t*)row)[i] : 0u;
        } else {
#pragma unroll
            for (int i = 0; i < IN_DW; ++i) raw[i] = *(const uint32_t*)(4 * i < validBytes ? p + 4 * i : row);
        }
    };

    // one S fragment (8 k-slots) -> the two tiles it belongs to
    auto putS = [&](uint32_t* tiles, int e0, int tilesInLayer, const uint32_t* frag) {
        *(u32x2*)(tiles + e0 * kPairTileDW + putDW) = u32x2{frag[0], frag[1]};
        if (e0 + 1 < tilesInLayer) *(u32x2*)(tiles + (e0 + 1) * kPairTileDW + putDW) = u32x2{frag[2], frag[3]};
    };

    auto round = [&](const uint32_t (&raw)[IN_DW], uint32_t r) {
        const uint32_t sample = r * 32u + 16u * par + n;
        const bool live = sample < a.batch;
        uint32_t buf[IN_DW];
#pragma unroll
        for (int d = 0; d < IN_DW; ++d) {
            if constexpr (LOADS == kLoadDwords) buf[d] = 4 * d < validBytes ? raw[d] : 0u;
            else buf[d] = 0u;
        }
        if constexpr (LOADS == kLoadXY) {
            if (g == 0) encodeXYSquares(__builtin_bit_cast(float, raw[0]), __builtin_bit_cast(float, raw[1]), buf[0], buf[1]);
        }
        // The target of the round's sample when the caller passes none: it depends on the input alone, and
        // computed here its long dependent chain runs in the shadow of the forward pass.
        float tgtAll = 0.f;
        half_t gt[4] = {(half_t)0, (half_t)0, (half_t)0, (half_t)0};
        const bool exampleLoss = !ta.targets && LOADS == kLoadXY;
        if constexpr (LOADS == kLoadXY) {
            const halfx2 xy = __builtin_bit_cast(halfx2, buf[0]);
            exampleGroundTruth(xy.x, xy.y, gt);
        } else if (!ta.targets) {
            float part = 0.f;
#pragma unroll
            for (int d = 0; d < IN_DW; ++d) {
                const halfx2 v = __builtin_bit_cast(halfx2, buf[d]);
                part += (float)v.x; part += (float)v.y;
            }
            tgtAll = (float)(half_t)sinf(sumOverGroups(part));
        }
        uint32_t actS[Net::KTMAX][FD];
        halfx2 zs[L][Net::MTMAX][2];              // pre-activations of the hidden layers: the backward pass derives
                                                  // the gradient multiplier of max() from them
        halfx2 yS[Net::MTL][2];
#pragma unroll
        for (int kt = 0; kt < Net::KT0; ++kt)
#pragma unroll
            for (int d = 0; d < FD; ++d) actS[kt][d] = buf[kt * RAW + d];

        // the partner has left the previous round (published at its end): the round's tiles may be overwritten
        timeouts |= pairAwait(partnerFlag, meetings);

        // ---------------- forward ----------------
        staticFor<0, L>([&](auto lc) {
            constexpr int l = decltype(lc)::value;
            constexpr int MT = Net::mt(l), KT = Net::kt(l);
            constexpr bool relu = l + 1 < L;
            // this layer's input, for the dW contraction of the backward pass
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
                if (2 * kt < Net::nIt(l)) putS(myX + Net::xTileBase(l) * kPairTileDW, 2 * kt, Net::nIt(l), actS[kt]);

            // all of the layer's fragments are requested before the first MFMA: a wave has one partner on
            // its SIMD to cover an LDS round trip, not enough to wait for every fragment on its own
            floatx4 acc[MT];
            uint32_t wf[KT][MT][4];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    const u32x4 v = *(const u32x4*)&ldsW[((Net::fragBase(l) + t * KT + kt) * 64 + lane) * RAW];
                    wf[kt][t][0] = v.x; wf[kt][t][1] = v.y; wf[kt][t][2] = v.z; wf[kt][t][3] = v.w;
                }
#pragma unroll
            for (int t = 0; t < MT; ++t) acc[t] = *(const floatx4*)&ldsB[(Net::biasBase(l) + t) * 16 + 4 * g];
            __builtin_amdgcn_sched_group_barrier(0x100, KT * MT + MT, 0);     // the LDS reads ...
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int t = 0; t < MT; ++t) acc[t] = Mma::mma(wf[kt][t], actS[kt], acc[t]);
            __builtin_amdgcn_sched_group_barrier(0x008, KT * MT, 0);          // ... then the MFMAs
            halfx2 car[MT][2];
            const halfx2 zero2 = {(half_t)0, (half_t)0};
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                typedef float floatx2 __attribute__((ext_vector_type(2)));
                halfx2 z01 = __builtin_convertvector(floatx2{acc[t][0], acc[t][1]}, halfx2);
                halfx2 z23 = __builtin_convertvector(floatx2{acc[t][2], acc[t][3]}, halfx2);
                if constexpr (relu) {
                    zs[l][t][0] = z01; zs[l][t][1] = z23;
                    halfx2 s01 = zero2, s23 = zero2;
                    if constexpr (LEAKY) {
                        if (a.layers[l].act != kActRelu) {
                            const half_t sl = (half_t)a.layers[l].slope;
                            s01 = z01 * halfx2{sl, sl}; s23 = z23 * halfx2{sl, sl};
                        }
                    }
                    z01 = __builtin_elementwise_max(z01, s01);
                    z23 = __builtin_elementwise_max(z23, s23);
                } else if constexpr (LEAKY) {
                    // the last layer's own activation (the example's layers all have one, fflayer.slang:60-66)
                    zs[l][t][0] = z01; zs[l][t][1] = z23;
                    if (a.layers[l].act != kActNone) {
                        halfx2 s01 = zero2, s23 = zero2;
                        if (a.layers[l].act != kActRelu) {
                            const half_t sl = (half_t)a.layers[l].slope;
                            s01 = z01 * halfx2{sl, sl}; s23 = z23 * halfx2{sl, sl};
                        }
                        z01 = __builtin_elementwise_max(z01, s01);
                        z23 = __builtin_elementwise_max(z23, s23);
                    }
                }
                car[t][0] = z01; car[t][1] = z23;
            }
            if constexpr (l + 1 < L) {
                constexpr int KTN = Net::kt(l + 1);
#pragma unroll
                for (int kt = 0; kt < KTN; ++kt) {
                    actS[kt][0] = __builtin_bit_cast(uint32_t, car[2 * kt][0]);
                    actS[kt][1] = __builtin_bit_cast(uint32_t, car[2 * kt][1]);
                    actS[kt][2] = (2 * kt + 1 < MT) ? __builtin_bit_cast(uint32_t, car[2 * kt + 1 < MT ? 2 * kt + 1 : 0][0]) : 0u;
                    actS[kt][3] = (2 * kt + 1 < MT) ? __builtin_bit_cast(uint32_t, car[2 * kt + 1 < MT ? 2 * kt + 1 : 0][1]) : 0u;
                }
            } else {
#pragma unroll
                for (int t = 0; t < MT; ++t) { yS[t][0] = car[t][0]; yS[t][1] = car[t][1]; }
            }
        });
        auto packS = [&](halfx2 (*dz)[2], int MT, int KT, uint32_t (*out)[FD]) {
#pragma unroll
            for (int kt = 0; kt < Net::KOMAX; ++kt) {
                if (kt < KT) {
                    out[kt][0] = __builtin_bit_cast(uint32_t, dz[2 * kt][0]);
                    out[kt][1] = __builtin_bit_cast(uint32_t, dz[2 * kt][1]);
                    out[kt][2] = (2 * kt + 1 < MT) ? __builtin_bit_cast(uint32_t, dz[2 * kt + 1 < MT ? 2 * kt + 1 : 0][0]) : 0u;
                    out[kt][3] = (2 * kt + 1 < MT) ? __builtin_bit_cast(uint32_t, dz[2 * kt + 1 < MT ? 2 * kt + 1 : 0][1]) : 0u;
                }
            }
        };

        // ---------------- loss and its gradient (S orientation) ----------------
        uint32_t bS[Net::KOMAX][FD];                // S fragments of dZ of the current layer
        {
            halfx2 dz[Net::MTL][2];
            float sampleLoss = 0.f;             // this lane's rows of the sample's loss
#pragma unroll
            for (int t = 0; t < Net::MTL; ++t) {
                const half_t yv[4] = {yS[t][0].x, yS[t][0].y, yS[t][1].x, yS[t][1].y};
                half_t gv[4];
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    gv[rr] = (half_t)0;
                    // rows 4t+rr and beyond of every lane group lie past the output (a one-output network uses one
                    // of these four steps): a wave-uniform skip
                    if (4 * t + rr >= outDim) continue;
                    const int row = g * OROWS + 4 * t + rr;
                    const bool on = live && row < outDim;
                    float tv = exampleLoss ? (float)gt[rr] : tgtAll;
                    if (ta.targets)
                        tv = (float)*(const half_t*)(ta.targets + (size_t)min(sample, lastSample) * ta.targetStride + 2 * (on ? row : 0));
                    // straight-line: rows past the output and samples past the batch compute, then count for nothing
                    const half_t diff = (half_t)((float)yv[rr] - tv);
                    lossAcc += on ? (float)diff * (float)diff : 0.f;
                    sampleLoss += on ? (float)diff * (float)diff : 0.f;
                    gv[rr] = on ? (half_t)(2.0f * (float)diff * ta.lossScale) : (half_t)0;
                }
                dz[t][0] = halfx2{gv[0], gv[1]};       // (without LEAKY the last layer has no activation)
                dz[t][1] = halfx2{gv[2], gv[3]};
                if constexpr (LEAKY) {
                    const half_t sl = (half_t)a.layers[L - 1].slope;
                    dz[t][0] = applyActGrad<true>(dz[t][0], maxGradMultiplier(zs[L - 1][t][0]), a.layers[L - 1].act, halfx2{sl, sl});
                    dz[t][1] = applyActGrad<true>(dz[t][1], maxGradMultiplier(zs[L - 1][t][1]), a.layers[L - 1].act, halfx2{sl, sl});
                }
            }
            if (ta.wantLossMax) {       // the sample's rows lie in the four lane groups
                const float whole = sumOverGroups(sampleLoss);
                lossMaxAcc = (whole > lossMaxAcc || whole != whole) ? whole : lossMaxAcc;
            }
            packS(dz, Net::MTL, Net::ktOut(L - 1), bS);
        }
        // ---------------- backward ----------------
        // The dW contraction of a layer is not on the round's chain of dependences (it only feeds the
        // accumulators), so its operands are requested as soon as both halves of dZ_l are in LDS and its
        // MFMAs are issued one layer later, behind the dX MFMAs of the layer below: by then the
        // transposed reads have long arrived, and the MFMAs fill the time in which the partner's half of
        // the next dZ is awaited.
        uint32_t xFp[Net::ITMAX][FD], dzFp[Net::MTMAX][FD];      // pending operands: F fragments of X_l and dZ_l
        auto contract = [&](auto lc) {
            constexpr int l = decltype(lc)::value;
            constexpr int OO = Split::ownedOut(l), OI = Split::ownedIn(l);
            if (!Split::single(l) || par == 0) {
#pragma unroll
                for (int eo = 0; eo < OO; ++eo) {
                    if (Split::byOut(l) || par == 0) {
                        float s = accB[Split::locDbBase(l) + eo];
#pragma unroll
                        for (int d = 0; d < FD; ++d) s = __builtin_amdgcn_fdot2(__builtin_bit_cast(halfx2, dzFp[eo][d]), ones2, s, false);
                        accB[Split::locDbBase(l) + eo] = s;
                    }
#pragma unroll
                    for (int ei = 0; ei < OI; ++ei) {
                        floatx4& w = accW[Split::locBase(l) + eo * OI + ei];
                        w = Mma::mma(dzFp[eo], xFp[ei], w);
                    }
                }
            }
        };
        staticFor<0, L>([&](auto lc) {
            constexpr int l = L - 1 - decltype(lc)::value;
            constexpr int MT = Net::mt(l), NI = Net::nIt(l), KO = Net::ktOut(l);
            uint32_t* slot = myDZ + (l & 1) * (Net::MTMAX * kPairTileDW);
#pragma unroll
            for (int kt = 0; kt < KO; ++kt) putS(slot, 2 * kt, MT, bS[kt]);
            pairPublish(myFlag, ++meetings);          // this wave's half of dZ_l is in LDS

            // dX = W^T dZ needs only this wave's own dZ: it runs between the two halves of the meeting
            floatx4 gacc[l > 0 ? Net::mt(l > 0 ? l - 1 : 0) : 1];
            if constexpr (l > 0) {
                constexpr int MTI = Net::mt(l - 1);
#pragma unroll
                for (int t = 0; t < MTI; ++t) gacc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
                uint32_t wf[KO][MTI][4];
#pragma unroll
                for (int kt = 0; kt < KO; ++kt)
#pragma unroll
                    for (int t = 0; t < MTI; ++t) {
                        const u32x4 v = *(const u32x4*)&ldsWT[((Net::tFragBase(l) + t * KO + kt) * 64 + lane) * RAW];
                        wf[kt][t][0] = v.x; wf[kt][t][1] = v.y; wf[kt][t][2] = v.z; wf[kt][t][3] = v.w;
                    }
                __builtin_amdgcn_sched_group_barrier(0x100, KO * MTI, 1);
#pragma unroll
                for (int kt = 0; kt < KO; ++kt)
#pragma unroll
                    for (int t = 0; t < MTI; ++t) gacc[t] = Mma::mma(wf[kt][t], bS[kt], gacc[t]);
                __builtin_amdgcn_sched_group_barrier(0x008, KO * MTI, 1);
            }
            if constexpr (l < L - 1) contract(std::integral_constant<int, (l < L - 1 ? l + 1 : 0)>{});
            timeouts |= pairAwait(partnerFlag, meetings);     // the partner's half of dZ_l is in LDS

            // operands of dW_l and db_l: this wave's share of the tiles, over all 32 samples of the round
            {
                constexpr int OO = Split::ownedOut(l), OI = Split::ownedIn(l);
                const int eo0 = Split::byOut(l) ? par * OO : 0;
                const int ei0 = Split::byIn(l) ? par * OI : 0;
                if (!Split::single(l) || par == 0) {
#pragma unroll
                    for (int ei = 0; ei < OI; ++ei) readF(myX + (Net::xTileBase(l) + ei0 + ei) * kPairTileDW, g, n, xFp[ei]);
#pragma unroll
                    for (int eo = 0; eo < OO; ++eo) readF(slot + (eo0 + eo) * kPairTileDW, g, n, dzFp[eo]);
                }
            }

            if constexpr (l > 0) {
                // through the previous layer's activation (ReLU on every hidden layer)
                constexpr int MTI = Net::mt(l - 1);
                halfx2 dz[MTI][2];
#pragma unroll
                for (int t = 0; t < MTI; ++t) {
                    typedef float floatx2 __attribute__((ext_vector_type(2)));
                    const halfx2 g01 = __builtin_convertvector(floatx2{gacc[t][0], gacc[t][1]}, halfx2);
                    const halfx2 g23 = __builtin_convertvector(floatx2{gacc[t][2], gacc[t][3]}, halfx2);
                    if constexpr (LEAKY) {
                        const half_t sl = (half_t)a.layers[l - 1].slope;
                        dz[t][0] = applyActGrad<true>(g01, maxGradMultiplier(zs[l - 1][t][0]), a.layers[l - 1].act, halfx2{sl, sl});
                        dz[t][1] = applyActGrad<true>(g23, maxGradMultiplier(zs[l - 1][t][1]), a.layers[l - 1].act, halfx2{sl, sl});
                    } else {
                        dz[t][0] = g01 * maxGradMultiplier(zs[l - 1][t][0]);
                        dz[t][1] = g23 * maxGradMultiplier(zs[l - 1][t][1]);
                    }
                }
                packS(dz, MTI, Net::ktOut(l - 1), bS);
            }
        });
        contract(std::integral_constant<int, 0>{});
        pairPublish(myFlag, ++meetings);          // this wave reads the round's tiles no more
    };

    // ---- main loop ---------------------------------------------------------------------------------
    {
        uint32_t cur[IN_DW], nxt[IN_DW];
        uint32_t r = blockIdx.x + firstRound * gridDim.x;
        loadTile(cur, r);
        for (uint32_t k = 0; k < roundsPerPair; ++k, r += gridDim.x) {
            loadTile(nxt, r + gridDim.x);
            asm volatile("" ::: "memory");        // the requests stay above the round ...
            round(cur, r);
#pragma unroll
            for (int d = 0; d < IN_DW; ++d) { pinHere(nxt[d]); cur[d] = nxt[d]; }   // ... their results are first touched below it
        }
    }

    // ---- workgroup partial: the four waves of each parity hold the same tiles; summed in a fixed order
    // a meeting timed out: the step's result is void; the NaN in the workgroup's loss partial makes the reduction
    // kernel turn the loss and every gradient sum of the step into NaN
    if (timeouts) lossAcc = __builtin_nanf("");
    if (ta.wantLossMax) noteLossMax(ldsLossMax, lossMaxAcc);
    __syncthreads();                              // every pair has left its last round: the X and dZ tiles are free
    // The eight waves put up to ten of their dW tiles at a time into the tile area (X and dZ tiles lie back to back), and all
    // 512 threads sum them: a few rounds of two barriers instead of two barriers per tile (which took 15 us of a 135 us
    // step).  The order of every sum is what it was: waves 0, 2, 4, 6 of a parity, left to right.
    constexpr int kRoomForTiles = (X_DW + DZ_DW - 8 * Split::totalLocDb * 64 - 512) / (8 * 256);
    constexpr int kTilesPerPhase = kRoomForTiles < 10 ? kRoomForTiles : 10;
    constexpr int kRedTileFloats = 8 * kTilesPerPhase * 256;
    static_assert(kTilesPerPhase >= 1, "the final reduction reuses the tile area");
    float* ldsRed = (float*)ldsX;                 // [8 waves][kTilesPerPhase][256], then [8 waves][totalLocDb][64], then 512 for the loss
    float* ldsRedB = ldsRed + kRedTileFloats;
    float* ldsLoss = ldsRedB + 8 * Split::totalLocDb * 64;      // one value per thread, behind the bias values
    float* part = ta.partials + (size_t)blockIdx.x * Net::partialFloats;
    const int rpar = threadIdx.x >> 8, ridx = threadIdx.x & 255;      // the parity / element this thread sums
    constexpr int kPhases = (Split::totalLoc + kTilesPerPhase - 1) / kTilesPerPhase;
    staticFor<0, kPhases>([&](auto pc) {
        constexpr int q0 = decltype(pc)::value * kTilesPerPhase;
        constexpr int q1 = q0 + kTilesPerPhase < Split::totalLoc ? q0 + kTilesPerPhase : Split::totalLoc;
        if constexpr (q0 > 0) __syncthreads();    // the sums of the phase before have been read
        staticFor<q0, q1>([&](auto qc) {
            constexpr int q = decltype(qc)::value;
            *(floatx4*)&ldsRed[(wave * kTilesPerPhase + (q - q0)) * 256 + lane * 4] = accW[q];
        });
        if constexpr (q0 == 0) {
#pragma unroll
            for (int j = 0; j < Split::totalLocDb; ++j) ldsRedB[(wave * Split::totalLocDb + j) * 64 + lane] = accB[j];
            ldsLoss[threadIdx.x] = lossAcc;
        }
        __syncthreads();
        staticFor<q0, q1>([&](auto qc) {
            constexpr int q = decltype(qc)::value;
            constexpr int l = Split::layerOfLoc(q), j = q - Split::locBase(l);
            constexpr int OO = Split::ownedOut(l), OI = Split::ownedIn(l), NI = Net::nIt(l);
            const float* r = ldsRed + (q - q0) * 256 + ridx;
            constexpr int W = kTilesPerPhase * 256;      // floats from one wave's tiles to the next wave's
            const float sum = ((r[(0 + rpar) * W] + r[(2 + rpar) * W]) + r[(4 + rpar) * W]) + r[(6 + rpar) * W];
            const int eo = (Split::byOut(l) ? rpar * OO : 0) + j / OI, ei = (Split::byIn(l) ? rpar * OI : 0) + j % OI;
            // (a streaming store: nobody on this die reads the partial, and it need not wait in the die's L2 for the write-back at
            // the kernel's end; 2.2 us of the step)
            if (!Split::single(l) || rpar == 0) __builtin_nontemporal_store(sum, &part[(Net::gradTileBase(l) + eo * NI + ei) * 256 + ridx]);
        });
        if constexpr (q0 == 0) {
            // bias gradients: 16 values per output row (four waves of a parity x four lane groups), summed by one thread
            if (threadIdx.x < 32 * Split::totalLocDb) {
                const int j = threadIdx.x >> 5, p2 = (threadIdx.x >> 4) & 1, q = threadIdx.x & 15;
                float sum = 0.f;
                for (int w = 0; w < 4; ++w)
                    for (int gg = 0; gg < 4; ++gg) sum += ldsRedB[((2 * w + p2) * Split::totalLocDb + j) * 64 + gg * 16 + q];
                staticFor<0, Split::totalLocDb>([&](auto jc) {
                    constexpr int jj = decltype(jc)::value;
                    constexpr int l = Split::layerOfLocDb(jj), jl = jj - Split::locDbBase(l), OO = Split::ownedOut(l);
                    if (j == jj) {
                        const int eo = (Split::byOut(l) ? p2 * OO : 0) + jl;
                        if (Split::byOut(l) || p2 == 0) part[Net::totalGradTiles * 256 + (Net::dbTileBase(l) + eo) * 16 + q] = sum;
                    }
                });
            }
        }
    });
    // The loss (its 512 values were put up with the bias values): the last wave sums them in a fixed order, eight
    // neighbours per lane, then lanes 32, 16, 8, 4, 2, 1 places apart.
    if (threadIdx.x >= 448) {
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) s += ldsLoss[lane * 8 + i];
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) s += __shfl_xor(s, d, 64);
        if (lane == 0) {
            part[Net::totalGradTiles * 256 + Net::totalDbTiles * 16] = s;
            part[Net::totalGradTiles * 256 + Net::totalDbTiles * 16 + 1] = __builtin_bit_cast(float, *ldsLossMax);
        }
    }
}

} // namespace
} // namespace cv
