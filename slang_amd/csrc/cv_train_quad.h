// cv_train_quad.h -- the fused training step for 128-wide hidden layers: four waves share the dW accumulators.
//
// The organisation of mlpTrainPairKernel (cv_train_pair.h) with a group of four waves in the place of a pair: a
// workgroup is one group, one wave per SIMD (the weight fragments of a 128x128 layer alone are 128 registers of a wave, its
// accumulators 32, the wave's share of the dW accumulators 80: two waves per SIMD do not fit).  The group takes rounds of
// 64 samples, 16 per wave; forward, loss and dX = W^T dY run per wave on its 16 samples; every layer input X_l and every
// dZ_l is also written to LDS ([32 samples][16 features] tiles as in the paired kernel, two of them per 16 features: waves
// 0 and 1 fill the first, waves 2 and 3 the second) and read back transposed with ds_read_b64_tr_b16; each wave
// accumulates a quarter of the dW tiles of every layer over all 64 samples of the round.  The four waves meet once per
// layer in the backward pass and once per round through sequence numbers in LDS (pairPublish / pairAwait, bounded).
// Every dW tile lives in exactly one wave, so the workgroup's partial is written without a reduction across waves;
// partials and second stage are those of the other fused kernels (fixed order, no atomics, bitwise reproducible).
//
// LDS: W and W^T of 16-128-128-8 are 84 KB, the tiles of a round 36 + 32 KB: 153 KB; a third 128-wide hidden layer does not
// fit (148 KB of weights), such networks train layer by layer.
#pragma once
#include "cv_train_pair.h"

namespace cv {
namespace {

// which dW tiles of layer l wave p of the group accumulates
template <class Net>
struct QuadSplit {
    static constexpr int L = Net::L, G = 4;
    static constexpr bool byOut(int l) { return Net::mt(l) >= G; }                        // split the out tiles
    static constexpr bool byIn(int l) { return Net::mt(l) < G && Net::nIt(l) >= G; }      // else split the in tiles
    static constexpr bool single(int l) { return !byOut(l) && !byIn(l); }                 // else wave 0 alone
    static constexpr int ownedOut(int l) { return byOut(l) ? Net::mt(l) / G : Net::mt(l); }
    static constexpr int ownedIn(int l) { return byIn(l) ? Net::nIt(l) / G : Net::nIt(l); }
    static constexpr bool divides(int l) { return (!byOut(l) || Net::mt(l) % G == 0) && (!byIn(l) || Net::nIt(l) % G == 0); }
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
    static constexpr int maxOwnedOut()
    {
        int m = 1;
        for (int i = 0; i < L; ++i) m = ownedOut(i) > m ? ownedOut(i) : m;
        return m;
    }
    static constexpr int maxOwnedIn()
    {
        int m = 1;
        for (int i = 0; i < L; ++i) m = ownedIn(i) > m ? ownedIn(i) : m;
        return m;
    }
};

// ReLU on the hidden layers (LEAKY: each hidden layer ReLU or leaky ReLU, as the arguments say: max(z, z*slope) with the
// product rounded to fp16, fflayer.slang:64-65), none on the last one (the launcher sends everything else to the
// layer-by-layer step).
template <class Net, bool LEAKY>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void mlpTrainQuadKernel(const TrainArgs ta)
{
    typedef F16Mma Mma;
    typedef QuadSplit<Net> Split;
    constexpr int L = Net::L;
    constexpr int FD = 4, RAW = 4, EPL = 8;
    constexpr int IN_DW = RAW * Net::KT0;
    constexpr int kTileDW = 2 * kPairTileDW;              // 16 features of the round's 64 samples
    const MlpArgs& a = ta.mlp;

    constexpr int W_DW = Net::totalFrags * 64 * RAW;
    constexpr int WT_DW = (Net::totalTFrags > 0 ? Net::totalTFrags : 1) * 64 * RAW;
    constexpr int B_DW = Net::totalBiasTiles * 16;
    constexpr int X_DW = Net::totalXTiles * kTileDW;                  // every layer's input of the round
    constexpr int DZ_DW = 2 * Net::MTMAX * kTileDW;                   // two alternating slots for dZ
    constexpr int FLAG_DW = 8;
    static_assert((W_DW + WT_DW + B_DW + X_DW + DZ_DW + FLAG_DW) * 4 <= 160 * 1024, "LDS of one compute unit");
    __shared__ __attribute__((aligned(16))) uint32_t lds[W_DW + WT_DW + B_DW + X_DW + DZ_DW + FLAG_DW];
    uint32_t* const ldsW = lds;
    uint32_t* const ldsWT = lds + W_DW;
    float* const ldsB = (float*)(lds + W_DW + WT_DW);
    uint32_t* const ldsX = lds + W_DW + WT_DW + B_DW;
    uint32_t* const ldsDZ = ldsX + X_DW;
    uint32_t* const ldsFlag = ldsDZ + DZ_DW;              // words 0..3: the waves' meeting numbers; 4: largest loss; 5: time-outs
    if (threadIdx.x < FLAG_DW) ldsFlag[threadIdx.x] = 0u;

    // ---- stage W and biases from memory, W^T from the W fragments in LDS (as in the paired kernel) -----------------
    staticFor<0, L>([&](auto lc) {
        constexpr int l = decltype(lc)::value;
        constexpr int MT = Net::mt(l), KT = Net::kt(l), ROWS = 4 * MT;
        static_assert(Split::divides(l), "the tiles of a layer divide among the four waves");
        const MlpLayerArgs& ly = a.layers[l];
        stageFragments<2, EPL>(ldsW + Net::fragBase(l) * 64 * RAW, ly.w, ly.shape, false, MT, KT,
                               l == 0 ? optGS((uint32_t)ly.in) : 4u * (uint32_t)Net::mt(l > 0 ? l - 1 : 0),
                               (uint32_t)ly.out, (uint32_t)ly.in);
        for (int e = threadIdx.x; e < MT * 16; e += 256) {
            const int t = e >> 4, gg = (e >> 2) & 3, r = e & 3, row = gg * ROWS + 4 * t + r;
            ldsB[Net::biasBase(l) * 16 + e] = (ly.bias && row < ly.out) ? (float)((const half_t*)ly.bias)[row] : 0.f;
        }
    });
    __syncthreads();
    staticFor<1, L>([&](auto lc) {
        constexpr int l = decltype(lc)::value;
        constexpr int MT = Net::mt(l), KT = Net::kt(l), MTI = Net::mt(l - 1), KTO = Net::ktOut(l);
        constexpr int gsOut = 4 * MT, gsIn = 4 * MTI, chunks = MTI * KTO * 64;
        const uint16_t* src = (const uint16_t*)(ldsW + Net::fragBase(l) * 64 * RAW);
        for (int c = threadIdx.x; c < chunks; c += 256) {
            const int ln = c & 63, f = c >> 6, kt = f % KTO, t = f / KTO, g = ln >> 4, i = ln & 15;
            const int col = (i >> 2) * 4 * MTI + 4 * t + (i & 3);         // the input unit
            const int gW = col / gsIn, ktW = (col % gsIn) / EPL, sW = (col % gsIn) % EPL;
            uint32_t v[EPL];
#pragma unroll
            for (int s2 = 0; s2 < EPL; ++s2) {
                const int q = kt * EPL + s2, o = g * gsOut + q;          // the output unit
                const int tW = (o % (4 * MT)) / 4, iW = 4 * (o / (4 * MT)) + o % 4;
                const int idx = (((q < gsOut ? tW : 0) * KT + ktW) * 64 + 16 * gW + (q < gsOut ? iW : 0)) * EPL + sW;
                const uint32_t x = src[idx];
                v[s2] = q < gsOut ? x : 0u;
            }
            *(u32x4*)&ldsWT[(Net::tFragBase(l) * 64 + c) * RAW] = u32x4{v[0] | v[1] << 16, v[2] | v[3] << 16, v[4] | v[5] << 16, v[6] | v[7] << 16};
        }
    });
    __syncthreads();

    const int lane = threadIdx.x & 63, p = threadIdx.x >> 6;          // p: the wave's place in the group
    const int g = lane >> 4, n = lane & 15;
    const halfx2 ones2 = {(half_t)1.f, (half_t)1.f};

    floatx4 accW[Split::totalLoc];
    float accB[Split::totalLocDb];
#pragma unroll
    for (int i = 0; i < Split::totalLoc; ++i) accW[i] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < Split::totalLocDb; ++i) accB[i] = 0.f;
    float lossAcc = 0.f, lossMaxAcc = 0.f;

    const int in0 = a.layers[0].in;
    const uint32_t gs0 = optGS((uint32_t)in0);
    const int colBase = (int)(g * gs0);
    const int validBytes = min((int)gs0, max(in0 - colBase, 0)) * 2;
    const int outDim = a.layers[L - 1].out;
    constexpr int OROWS = 4 * Net::MTL;

    const uint32_t numRounds = (a.batch + 63u) / 64u;
    const uint32_t myRounds = blockIdx.x < numRounds ? (numRounds - blockIdx.x + gridDim.x - 1u) / gridDim.x : 0u;
    const uint32_t lastSample = a.batch - 1;
    // where this lane puts its four halves of a tile (S fragment half: sample 16*p + n of the round, rows 4g..4g+3)
    const int putDW = (p >> 1) * kPairTileDW + pairChunkDW(16 * (p & 1) + n, g);
    volatile LdsWord* const myFlag = (LdsWord*)(ldsFlag + p);
    uint32_t meetings = 0, timeouts = 0;
    auto awaitOthers = [&]() {
#pragma unroll
        for (int o = 1; o < 4; ++o) timeouts |= pairAwait((LdsWord*)(ldsFlag + ((p + o) & 3)), meetings);
    };

    // (element by element: rows of any length at any 2-byte aligned address; the loads are in flight for a whole round)
    auto loadTile = [&](uint32_t (&raw)[IN_DW], uint32_t r) {
        const uint32_t s = min(r * 64u + 16u * p + n, lastSample);
        const uint8_t* row = a.in + (size_t)s * a.inStride;
        const uint8_t* q = row + (size_t)colBase * 2;
        uint32_t hv[2 * IN_DW];
#pragma unroll
        for (int i = 0; i < 2 * IN_DW; ++i) hv[i] = *(const uint16_t*)(2 * i < validBytes ? q + 2 * i : row);
#pragma unroll
        for (int i = 0; i < IN_DW; ++i) raw[i] = hv[2 * i] | hv[2 * i + 1] << 16;
    };
    // one S fragment (8 k-slots) -> the two tiles it belongs to
    auto putS = [&](uint32_t* tiles, int e0, int tilesInLayer, const uint32_t* frag) {
        *(u32x2*)(tiles + e0 * kTileDW + putDW) = u32x2{frag[0], frag[1]};
        if (e0 + 1 < tilesInLayer) *(u32x2*)(tiles + (e0 + 1) * kTileDW + putDW) = u32x2{frag[2], frag[3]};
    };

    auto round = [&](const uint32_t (&raw)[IN_DW], uint32_t r) {
        const uint32_t sample = r * 64u + 16u * p + n;
        const bool live = sample < a.batch;
        uint32_t buf[IN_DW];
#pragma unroll
        for (int d = 0; d < IN_DW; ++d)
            buf[d] = (4 * d < validBytes ? raw[d] & 0xffffu : 0u) | (4 * d + 2 < validBytes ? raw[d] & 0xffff0000u : 0u);
        float tgtAll = 0.f;
        if (!ta.targets) {
            float part = 0.f;
#pragma unroll
            for (int d = 0; d < IN_DW; ++d) {
                const halfx2 v = __builtin_bit_cast(halfx2, buf[d]);
                part += (float)v.x; part += (float)v.y;
            }
            tgtAll = (float)(half_t)sinf(sumOverGroups(part));
        }
        uint32_t actS[Net::KTMAX][FD];
        halfx2 zs[L][Net::MTMAX][2];              // pre-activations of the hidden layers, for the multiplier of max()
        halfx2 yS[Net::MTL][2];
#pragma unroll
        for (int kt = 0; kt < Net::KT0; ++kt)
#pragma unroll
            for (int d = 0; d < FD; ++d) actS[kt][d] = buf[kt * RAW + d];

        // the others have left the previous round: the round's tiles may be overwritten
        awaitOthers();

        // ---------------- forward ----------------
        staticFor<0, L>([&](auto lc) {
            constexpr int l = decltype(lc)::value;
            constexpr int MT = Net::mt(l), KT = Net::kt(l);
            constexpr bool relu = l + 1 < L;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
                if (2 * kt < Net::nIt(l)) putS(ldsX + Net::xTileBase(l) * kTileDW, 2 * kt, Net::nIt(l), actS[kt]);
            floatx4 acc[MT];
#pragma unroll
            for (int t = 0; t < MT; ++t) acc[t] = *(const floatx4*)&ldsB[(Net::biasBase(l) + t) * 16 + 4 * g];
            // a k-step's fragments are requested together, a k-step ahead of their matrix instructions
            uint32_t wf[2][MT][4];
            auto request = [&](int kt) {
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    const u32x4 v = *(const u32x4*)&ldsW[((Net::fragBase(l) + t * KT + kt) * 64 + lane) * RAW];
                    wf[kt & 1][t][0] = v.x; wf[kt & 1][t][1] = v.y; wf[kt & 1][t][2] = v.z; wf[kt & 1][t][3] = v.w;
                }
            };
            request(0);
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                if (kt + 1 < KT) request(kt + 1);
#pragma unroll
                for (int t = 0; t < MT; ++t) acc[t] = Mma::mma(wf[kt & 1][t], actS[kt], acc[t]);
            }
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
            float sampleLoss = 0.f;
#pragma unroll
            for (int t = 0; t < Net::MTL; ++t) {
                const half_t yv[4] = {yS[t][0].x, yS[t][0].y, yS[t][1].x, yS[t][1].y};
                half_t gv[4];
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    gv[rr] = (half_t)0;
                    if (4 * t + rr >= outDim) continue;       // rows past the output in every lane group: a wave-uniform skip
                    const int row = g * OROWS + 4 * t + rr;
                    const bool on = live && row < outDim;
                    float tv = tgtAll;
                    if (ta.targets)
                        tv = (float)*(const half_t*)(ta.targets + (size_t)min(sample, lastSample) * ta.targetStride + 2 * (on ? row : 0));
                    const half_t diff = (half_t)((float)yv[rr] - tv);
                    lossAcc += on ? (float)diff * (float)diff : 0.f;
                    sampleLoss += on ? (float)diff * (float)diff : 0.f;
                    gv[rr] = on ? (half_t)(2.0f * (float)diff * ta.lossScale) : (half_t)0;
                }
                dz[t][0] = halfx2{gv[0], gv[1]};
                dz[t][1] = halfx2{gv[2], gv[3]};
                if constexpr (LEAKY) {      // (without LEAKY the last layer has no activation)
                    const half_t sl = (half_t)a.layers[L - 1].slope;
                    dz[t][0] = applyActGrad<true>(dz[t][0], maxGradMultiplier(zs[L - 1][t][0]), a.layers[L - 1].act, halfx2{sl, sl});
                    dz[t][1] = applyActGrad<true>(dz[t][1], maxGradMultiplier(zs[L - 1][t][1]), a.layers[L - 1].act, halfx2{sl, sl});
                }
            }
            if (ta.wantLossMax) {
                const float whole = sumOverGroups(sampleLoss);
                lossMaxAcc = (whole > lossMaxAcc || whole != whole) ? whole : lossMaxAcc;
            }
            packS(dz, Net::MTL, Net::ktOut(L - 1), bS);
        }
        // ---------------- backward ----------------
        // The dW contraction of a layer is issued one layer late, behind the dX matrix instructions of the layer below
        // (its operands were requested as soon as all four quarters of dZ_l were in LDS).
        uint32_t xFp[Split::maxOwnedIn()][2][FD], dzFp[Split::maxOwnedOut()][2][FD];      // F fragments of X_l and dZ_l, both halves of the round
        auto contract = [&](auto lc) {
            constexpr int l = decltype(lc)::value;
            constexpr int OO = Split::ownedOut(l), OI = Split::ownedIn(l);
            if (!Split::single(l) || p == 0) {
#pragma unroll
                for (int eo = 0; eo < OO; ++eo) {
                    if (Split::byOut(l) || p == 0) {
                        float s = accB[Split::locDbBase(l) + eo];
#pragma unroll
                        for (int hf = 0; hf < 2; ++hf)
#pragma unroll
                            for (int d = 0; d < FD; ++d) s = __builtin_amdgcn_fdot2(__builtin_bit_cast(halfx2, dzFp[eo][hf][d]), ones2, s, false);
                        accB[Split::locDbBase(l) + eo] = s;
                    }
#pragma unroll
                    for (int ei = 0; ei < OI; ++ei) {
                        floatx4& w = accW[Split::locBase(l) + eo * OI + ei];
#pragma unroll
                        for (int hf = 0; hf < 2; ++hf) w = Mma::mma(dzFp[eo][hf], xFp[ei][hf], w);
                    }
                }
            }
        };
        staticFor<0, L>([&](auto lc) {
            constexpr int l = L - 1 - decltype(lc)::value;
            constexpr int MT = Net::mt(l), KO = Net::ktOut(l);
            uint32_t* slot = ldsDZ + (l & 1) * (Net::MTMAX * kTileDW);
#pragma unroll
            for (int kt = 0; kt < KO; ++kt) putS(slot, 2 * kt, MT, bS[kt]);
            pairPublish(myFlag, ++meetings);          // this wave's quarter of dZ_l is in LDS

            // dX = W^T dZ needs only this wave's own dZ: it runs between the two halves of the meeting
            floatx4 gacc[l > 0 ? Net::mt(l > 0 ? l - 1 : 0) : 1];
            if constexpr (l > 0) {
                constexpr int MTI = Net::mt(l - 1);
#pragma unroll
                for (int t = 0; t < MTI; ++t) gacc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
                uint32_t wf[2][MTI][4];
                auto request = [&](int kt) {
#pragma unroll
                    for (int t = 0; t < MTI; ++t) {
                        const u32x4 v = *(const u32x4*)&ldsWT[((Net::tFragBase(l) + t * KO + kt) * 64 + lane) * RAW];
                        wf[kt & 1][t][0] = v.x; wf[kt & 1][t][1] = v.y; wf[kt & 1][t][2] = v.z; wf[kt & 1][t][3] = v.w;
                    }
                };
                request(0);
#pragma unroll
                for (int kt = 0; kt < KO; ++kt) {
                    if (kt + 1 < KO) request(kt + 1);
#pragma unroll
                    for (int t = 0; t < MTI; ++t) gacc[t] = Mma::mma(wf[kt & 1][t], bS[kt], gacc[t]);
                }
            }
            if constexpr (l < L - 1) contract(std::integral_constant<int, (l < L - 1 ? l + 1 : 0)>{});
            awaitOthers();                            // everybody's quarter of dZ_l is in LDS

            // operands of dW_l and db_l: this wave's share of the tiles, over all 64 samples of the round
            {
                constexpr int OO = Split::ownedOut(l), OI = Split::ownedIn(l);
                const int eo0 = Split::byOut(l) ? p * OO : 0;
                const int ei0 = Split::byIn(l) ? p * OI : 0;
                if (!Split::single(l) || p == 0) {
#pragma unroll
                    for (int ei = 0; ei < OI; ++ei)
#pragma unroll
                        for (int hf = 0; hf < 2; ++hf) readF(ldsX + (Net::xTileBase(l) + ei0 + ei) * kTileDW + hf * kPairTileDW, g, n, xFp[ei][hf]);
#pragma unroll
                    for (int eo = 0; eo < OO; ++eo)
#pragma unroll
                        for (int hf = 0; hf < 2; ++hf) readF(slot + (eo0 + eo) * kTileDW + hf * kPairTileDW, g, n, dzFp[eo][hf]);
                }
            }

            if constexpr (l > 0) {
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
        uint32_t r = blockIdx.x;
        loadTile(cur, r);
        for (uint32_t k = 0; k < myRounds; ++k, r += gridDim.x) {
            loadTile(nxt, r + gridDim.x);
            asm volatile("" ::: "memory");        // the requests stay above the round ...
            round(cur, r);
#pragma unroll
            for (int d = 0; d < IN_DW; ++d) { pinHere(nxt[d]); cur[d] = nxt[d]; }   // ... their results are first touched below it
        }
    }

    // ---- the workgroup's partial: every dW tile lies in one wave (streaming stores: nobody on this die reads them, and they
    // need not wait in its L2 for the write-back at the kernel's end) -----------------------------------------------------
    if (timeouts && lane == 0) atomicOr(ldsFlag + 5, 1u);
    if (ta.wantLossMax) noteLossMax(ldsFlag + 4, lossMaxAcc);
    float* part = ta.partials + (size_t)blockIdx.x * Net::partialFloats;
    staticFor<0, L>([&](auto lc) {
        constexpr int l = decltype(lc)::value;
        constexpr int OO = Split::ownedOut(l), OI = Split::ownedIn(l), NI = Net::nIt(l);
        const int eo0 = Split::byOut(l) ? p * OO : 0, ei0 = Split::byIn(l) ? p * OI : 0;
        if (!Split::single(l) || p == 0) {
#pragma unroll
            for (int eo = 0; eo < OO; ++eo) {
#pragma unroll
                for (int ei = 0; ei < OI; ++ei)
                    __builtin_nontemporal_store(accW[Split::locBase(l) + eo * OI + ei],
                                                (floatx4*)&part[(Net::gradTileBase(l) + (eo0 + eo) * NI + ei0 + ei) * 256 + lane * 4]);
                if (Split::byOut(l) || p == 0) {
                    // a row's bias gradient lies in the four lane groups (eight samples of the round's 32 + 32 each)
                    float s = accB[Split::locDbBase(l) + eo];
                    s += __shfl_xor(s, 16, 64);
                    s += __shfl_xor(s, 32, 64);
                    if (g == 0) part[Net::totalGradTiles * 256 + (Net::dbTileBase(l) + eo0 + eo) * 16 + n] = s;
                }
            }
        }
    });
    // the loss: the four waves' lanes, summed in a fixed order
    float* const ldsLoss = (float*)ldsX;
    __syncthreads();                              // every wave has left its last round: the tile area is free
    ldsLoss[threadIdx.x] = lossAcc;
    __syncthreads();
    if (p == 0) {
        float s = ((ldsLoss[lane] + ldsLoss[64 + lane]) + ldsLoss[128 + lane]) + ldsLoss[192 + lane];
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) s += __shfl_xor(s, d, 64);
        if (ldsFlag[5]) s = __builtin_nanf("");
        if (lane == 0) {
            part[Net::totalGradTiles * 256 + Net::totalDbTiles * 16] = s;
            part[Net::totalGradTiles * 256 + Net::totalDbTiles * 16 + 1] = __builtin_bit_cast(float, ldsFlag[4]);
        }
    }
}

} // namespace
} // namespace cv
