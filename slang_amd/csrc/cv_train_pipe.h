// cv_train_pipe.h -- layer-pipelined training step for wide fp16 MLPs on gfx950.
//
// Same arithmetic as mlpTrainKernel (cv_train_impl.h), organised for occupancy.  In that kernel one
// wave runs a whole forward + backward pass and owns all gradient accumulators (224 registers for
// 8-64-64-64-64-1), so a SIMD holds a single wave whose MFMA and VALU phases alternate with nothing
// to overlap them.  Here one workgroup per compute unit is a pipeline of waves, one role each:
//
//     F_l   forward of layer l          X_l -> X_{l+1}          (weights of layer l in registers)
//     BX_l  dX of layer l               D_l -> D_{l-1}          (transposed weights in registers)
//     BW_l  dW/db of layer l            D_l, X_l -> accumulators (layer l's gradients in registers)
//   (the light first and last layers share waves: F_0 with F_{L-1}, BW_0 with BW_{L-1})
//
// X_l (a layer's input) and D_l (the gradient of its output) travel between waves through ring
// buffers in LDS as MFMA "S" fragments; one round of 32 samples enters per step and every wave
// does one unit of work per step, separated by a single workgroup barrier (the only barrier call
// site, executed the same number of times by every wave).  Weights never leave registers, every
// wave needs <= 170 registers, three waves share a SIMD, and roles are placed so that each SIMD gets
// about a quarter of the MFMA and VALU work.
//
// The ReLU derivative (Slang's max rule with the 0.5 tie, diff.meta.slang:2258-2277) needs the
// sign of the pre-activation in the backward pass.  Instead of parking a mask, the forward stores
// max(z, -0.0): a negative z leaves -0.0, an exact zero leaves +0.0.  Both are zero to every MFMA
// that consumes them; the backward reads the sign bit back.
//
// Used for ReLU-hidden / linear-output networks with 64-wide hidden layers; everything else takes
// mlpTrainKernel.  Partials are laid out exactly as mlpTrainKernel's, so mlpTrainReduceKernel
// finishes both.
#pragma once
#include "cv_train_impl.h"

namespace cv {
namespace {

template <class Net>
struct PipeLayout {
    static constexpr int L = Net::L;
    // X_l: input of layer l as S fragments, 2 tiles x kt(l) fragments of 256 dwords
    static constexpr int xSize(int l) { return 2 * Net::kt(l) * 256; }
    // a slot written for round r (by F_{l-1} at step r+l-1, or by F_0 at step r for l = 0) is read
    // last by BW_l at step r + 2L-1-l
    static constexpr int xSlots(int l) { return l == 0 ? 2 * L : 2 * L - 2 * l + 1; }
    static constexpr int xBase(int l)
    {
        int b = 0;
        for (int i = 0; i < l; ++i) b += xSize(i) * xSlots(i);
        return b;
    }
    // D_l: gradient of layer l's output, 2 tiles x ktOut(l) fragments; read in the step after it is written
    static constexpr int dSize(int l) { return 2 * Net::ktOut(l) * 256; }
    static constexpr int dBase(int l)
    {
        int b = xBase(L);
        for (int i = 0; i < l; ++i) b += dSize(i) * 2;
        return b;
    }
    static constexpr int ringDwords = dBase(L);
    // the weights are staged through the same memory before the pipeline starts
    static constexpr int stageDwords = (Net::totalFrags + Net::totalTFrags) * 256;
    static constexpr int ldsDwords = ringDwords > stageDwords ? ringDwords : stageDwords;
    // pipeline step (relative to the round) at which each role works
    static constexpr int stepF(int l) { return l; }
    static constexpr int stepBX(int l) { return L + (L - 1 - l); }
    static constexpr int stepBW(int l) { return 2 * L - 1 - l; }
    static constexpr int depth = 2 * L;           // steps to drain
};

enum : int { kRoleNone = 0, kRoleF = 1, kRoleBX = 2, kRoleBW = 3, kRoleF0FL = 4, kRoleBWEnds = 5 };
constexpr int kPipeWaves = 12;      // three per SIMD: 170 registers each

template <class Net>
__global__ __launch_bounds__(64 * kPipeWaves) void mlpTrainPipeKernel(const TrainArgs ta)
{
    typedef F16Mma Mma;
    typedef PipeLayout<Net> P;
    constexpr int L = Net::L;
    constexpr int FD = 4, RAW = 4, EPL = 8;
    constexpr int IN_DW = RAW * Net::KT0;
    static_assert(L >= 3 && L <= 5, "roles are laid out for three to five layers");
    static_assert(Net::MTL == 1 && Net::mt(0) * Net::kt(0) <= 8 && Net::nOt(0) * Net::nIt(0) <= 8,
                  "the end layers share one wave's registers");
    static_assert(P::ldsDwords * 4 + Net::totalBiasTiles * 64 <= 160 * 1024, "rings must fit the LDS");
    const MlpArgs& a = ta.mlp;

    __shared__ __attribute__((aligned(16))) uint32_t lds[P::ldsDwords];
    __shared__ __attribute__((aligned(16))) float ldsB[Net::totalBiasTiles * 16];

    // ---- stage W, W^T (fragment order) and biases; same maps as mlpTrainKernel -------------------
    uint32_t* ldsW = lds;
    uint32_t* ldsWT = lds + Net::totalFrags * 256;
    staticFor<0, L>([&](auto lc) {
        constexpr int l = decltype(lc)::value;
        constexpr int MT = Net::mt(l), KT = Net::kt(l), ROWS = 4 * MT;
        const MlpLayerArgs& ly = a.layers[l];
        const uint32_t gs = optGS((uint32_t)ly.in);
        uint16_t* dst = (uint16_t*)(ldsW + Net::fragBase(l) * 64 * RAW);
        for (int e = threadIdx.x; e < MT * KT * 64 * EPL; e += 64 * kPipeWaves) {
            const int s = e % EPL, ln = (e / EPL) & 63, f = e / (EPL * 64);
            const int kt = f % KT, t = f / KT, gg = ln >> 4, i = ln & 15;
            const uint32_t row = (uint32_t)((i >> 2) * ROWS + 4 * t + (i & 3));
            const uint32_t q = (uint32_t)(kt * EPL + s), col = gg * gs + q;
            const bool valid = row < (uint32_t)ly.out && q < gs && col < (uint32_t)ly.in;
            dst[e] = valid ? *(const uint16_t*)(ly.w + elemOffset(ly.shape, row, col)) : (uint16_t)0;
        }
        if constexpr (l > 0) {
            constexpr int MTI = Net::mt(l - 1), KTO = Net::ktOut(l), ROWSI = 4 * MTI;
            const uint32_t gso = 4u * MT;
            uint16_t* dt = (uint16_t*)(ldsWT + Net::tFragBase(l) * 64 * RAW);
            for (int e = threadIdx.x; e < MTI * KTO * 64 * EPL; e += 64 * kPipeWaves) {
                const int s = e % EPL, ln = (e / EPL) & 63, f = e / (EPL * 64);
                const int kt = f % KTO, t = f / KTO, gg = ln >> 4, p = ln & 15;
                const uint32_t irow = (uint32_t)((p >> 2) * ROWSI + 4 * t + (p & 3));
                const uint32_t q = (uint32_t)(kt * EPL + s), ocol = gg * gso + q;
                const bool valid = irow < (uint32_t)ly.in && q < gso && ocol < (uint32_t)ly.out;
                dt[e] = valid ? *(const uint16_t*)(ly.w + elemOffset(ly.shape, ocol, irow)) : (uint16_t)0;
            }
        }
        for (int e = threadIdx.x; e < MT * 16; e += 64 * kPipeWaves) {
            const int t = e >> 4, gg = (e >> 2) & 3, r = e & 3;
            const int row = gg * ROWS + 4 * t + r;
            ldsB[(Net::biasBase(l) + t) * 16 + 4 * gg + r] = (ly.bias && row < ly.out) ? (float)((const half_t*)ly.bias)[row] : 0.f;
        }
    });
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, n = lane & 15;

    // ---- role of this wave.  Waves w, w+4, w+8, w+12 share a SIMD (round-robin placement): each of
    //      the first L-2 SIMDs gets the three roles of one hidden layer, the last one the light ends.
    int role = kRoleNone, layer = 0;
    {
        const int s = wave & 3, k = wave >> 2;
        if (s < L - 2 && s < 3) {
            layer = s + 1;
            role = k == 0 ? kRoleBW : k == 1 ? kRoleBX : kRoleF;
        } else if (s == 3) {
            if (k == 0) { role = kRoleF0FL; layer = 0; }
            else if (k == 1) { role = kRoleBX; layer = L - 1; }
            else { role = kRoleBWEnds; layer = L - 1; }
        }
    }

    // ---- per-role registers: weights / biases for F and BX, accumulators for BW -----------------
    floatx4 S[16];                                  // 16 x 4 registers, meaning depends on the role
    float accB[5] = {0.f, 0.f, 0.f, 0.f, 0.f};
    float lossAcc = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) S[i] = floatx4{0.f, 0.f, 0.f, 0.f};
    auto fragOf = [&](int i) -> const uint32_t* { return (const uint32_t*)&S[i]; };
    // forward fragments of layer l at S[WB..], its bias tiles at S[BB..]
    auto loadForward = [&](auto lc, auto wb, auto bb) {
        constexpr int l = decltype(lc)::value, WB = decltype(wb)::value, BB = decltype(bb)::value;
#pragma unroll
        for (int t = 0; t < Net::mt(l); ++t) {
#pragma unroll
            for (int kt = 0; kt < Net::kt(l); ++kt)
                S[WB + t * Net::kt(l) + kt] = *(const floatx4*)&ldsW[((Net::fragBase(l) + t * Net::kt(l) + kt) * 64 + lane) * RAW];
            S[BB + t] = *(const floatx4*)&ldsB[(Net::biasBase(l) + t) * 16 + 4 * g];
        }
    };
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 8> I8;
    typedef std::integral_constant<int, 12> I12;
    typedef std::integral_constant<int, 15> I15;
    if (role == kRoleF0FL) {
        loadForward(std::integral_constant<int, 0>{}, I0{}, I8{});          // layer 0: S[0..], bias S[8..]
        loadForward(std::integral_constant<int, L - 1>{}, I12{}, I15{});    // last layer: S[12..13], bias S[15]
    }
    staticFor<1, L>([&](auto lc) {
        constexpr int l = decltype(lc)::value;
        if constexpr (l < L - 1) {
            if (role == kRoleF && layer == l) loadForward(lc, I0{}, I8{});
        }
        if (role == kRoleBX && layer == l) {
#pragma unroll
            for (int t = 0; t < Net::mt(l - 1); ++t)
#pragma unroll
                for (int kt = 0; kt < Net::ktOut(l); ++kt)
                    S[t * Net::ktOut(l) + kt] = *(const floatx4*)&ldsWT[((Net::tFragBase(l) + t * Net::ktOut(l) + kt) * 64 + lane) * RAW];
        }
    });
    __syncthreads();                                // the staging area becomes the rings

    // 0/1 selection fragments (see mlpTrainKernel)
    uint32_t Isel[2][FD];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int d = 0; d < FD; ++d) {
            const int s0 = 4 * h + (lane & 3);
            const bool mine = g == (n >> 2);
            Isel[h][d] = ((mine && s0 == 2 * d) ? 0x3C00u : 0u) | (((mine && s0 == 2 * d + 1) ? 0x3C00u : 0u) << 16);
        }
    const halfx2 ones2 = {(half_t)1.f, (half_t)1.f};
    const halfx2 negZero2 = __builtin_bit_cast(halfx2, 0x80008000u);

    // ---- rounds of this workgroup ----------------------------------------------------------------
    const uint32_t numRounds = (a.batch + 31) / 32;
    const uint32_t myRounds = blockIdx.x < numRounds ? (numRounds - blockIdx.x + gridDim.x - 1) / gridDim.x : 0;
    const uint32_t totalSteps = myRounds ? myRounds + P::depth : 0;
    auto globalRound = [&](uint32_t r) { return blockIdx.x + r * gridDim.x; };

    const int in0 = a.layers[0].in;
    const uint32_t gs0 = optGS((uint32_t)in0);
    const int colBase = (int)(g * gs0);
    const int validBytes = min((int)gs0, max(in0 - colBase, 0)) * 2;
    const bool vecLoad = validBytes == IN_DW * 4 && a.inAlign >= 16u;
    const uint8_t* inLane = a.in + (size_t)colBase * 2;
    const uint32_t lastSample = a.batch - 1;
    const int outDim = a.layers[L - 1].out;
    constexpr int OROWS = 4 * Net::MTL;

    auto loadInput = [&](uint32_t (&buf)[2][IN_DW], uint32_t r) {
        const uint32_t gr = globalRound(r < myRounds ? r : (myRounds ? myRounds - 1 : 0));
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t s = min(gr * 32 + 16 * j + n, lastSample);
            const uint8_t* p = inLane + (size_t)s * a.inStride;
            if (vecLoad) {
#pragma unroll
                for (int i = 0; i < IN_DW / 4; ++i) {
                    const u32x4 v = *(const u32x4*)(p + 16 * i);
                    buf[j][4 * i] = v.x; buf[j][4 * i + 1] = v.y; buf[j][4 * i + 2] = v.z; buf[j][4 * i + 3] = v.w;
                }
            } else {
#pragma unroll
                for (int i = 0; i < IN_DW; ++i) {
                    uint32_t v = 0;
                    if (4 * i < validBytes) v = *(const uint16_t*)(p + 4 * i);
                    if (4 * i + 2 < validBytes) v |= (uint32_t)*(const uint16_t*)(p + 4 * i + 2) << 16;
                    buf[j][i] = v;
                }
            }
        }
    };

    // S fragment helpers: fragment (j, kt) of a ring slot
    auto ringRead = [&](const uint32_t* slot, int KT, int j, int kt, uint32_t* out) {
        const u32x4 v = *(const u32x4*)(slot + (j * KT + kt) * 256 + lane * 4);
        out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
    };
    auto ringWrite = [&](uint32_t* slot, int KT, int j, int kt, uint32_t d0, uint32_t d1, uint32_t d2, uint32_t d3) {
        const u32x4 v = {d0, d1, d2, d3};
        *(u32x4*)(slot + (j * KT + kt) * 256 + lane * 4) = v;
    };
    auto cvt2 = [&](float x, float y) -> halfx2 {
        typedef float floatx2 __attribute__((ext_vector_type(2)));
        return __builtin_convertvector(floatx2{x, y}, halfx2);
    };
    auto toF = [&](const uint32_t* s0, const uint32_t* s1, int h, uint32_t* frag) {
        const floatx4 z = {0.f, 0.f, 0.f, 0.f};
        const floatx4 t0 = Mma::mma(s0, Isel[h], z), t1 = Mma::mma(s1, Isel[h], z);
        frag[0] = __builtin_bit_cast(uint32_t, cvt2(t0[0], t0[1]));
        frag[1] = __builtin_bit_cast(uint32_t, cvt2(t0[2], t0[3]));
        frag[2] = __builtin_bit_cast(uint32_t, cvt2(t1[0], t1[1]));
        frag[3] = __builtin_bit_cast(uint32_t, cvt2(t1[2], t1[3]));
    };

    // ---- forward of layer l for round r: X_l -> X_{l+1} (or, for the last layer, the loss and D_{L-1})
    auto forward = [&](auto lc, auto wb, auto bb, uint32_t r, const uint32_t (*inReg)[IN_DW]) {
        constexpr int l = decltype(lc)::value, wbase = decltype(wb)::value, bbase = decltype(bb)::value;
        constexpr int MT = Net::mt(l), KT = Net::kt(l);
        uint32_t actS[2][KT][FD];
        if constexpr (l == 0) {
            // the input comes from registers; it is also parked as X_0 for BW_0 and for the loss target
            uint32_t* x0 = lds + P::xBase(0) + (r % P::xSlots(0)) * P::xSize(0);
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
                    for (int d = 0; d < FD; ++d) actS[j][kt][d] = inReg[j][kt * RAW + d];
                    ringWrite(x0, KT, j, kt, actS[j][kt][0], actS[j][kt][1], actS[j][kt][2], actS[j][kt][3]);
                }
        } else {
            const uint32_t* xin = lds + P::xBase(l) + (r % P::xSlots(l)) * P::xSize(l);
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) ringRead(xin, KT, j, kt, actS[j][kt]);
        }
        floatx4 acc[2][MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) { acc[0][t] = S[bbase + t]; acc[1][t] = S[bbase + t]; }
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                acc[0][t] = Mma::mma(fragOf(wbase + t * KT + kt), actS[0][kt], acc[0][t]);
                acc[1][t] = Mma::mma(fragOf(wbase + t * KT + kt), actS[1][kt], acc[1][t]);
            }
        if constexpr (l + 1 < L) {
            // ReLU that keeps the sign of a negative pre-activation as -0.0 (see the header comment)
            constexpr int KTN = Net::kt(l + 1);
            uint32_t* xout = lds + P::xBase(l + 1) + (r % P::xSlots(l + 1)) * P::xSize(l + 1);
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int kt = 0; kt < KTN; ++kt) {
                    uint32_t d[4] = {0u, 0u, 0u, 0u};
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        if (2 * kt + h < MT) {
                            const floatx4& c = acc[j][2 * kt + h < MT ? 2 * kt + h : 0];
                            d[2 * h] = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(cvt2(c[0], c[1]), negZero2));
                            d[2 * h + 1] = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(cvt2(c[2], c[3]), negZero2));
                        }
                    }
                    ringWrite(xout, KTN, j, kt, d[0], d[1], d[2], d[3]);
                }
        } else {
            // loss_s = sum_i (y - t)^2, seed 2 (y - t) lossScale; dead samples contribute nothing
            const uint32_t gr = globalRound(r);
            const uint32_t* x0 = lds + P::xBase(0) + (r % P::xSlots(0)) * P::xSize(0);
            uint32_t* dout = lds + P::dBase(l) + (r & 1u) * P::dSize(l);
            constexpr int KTO = Net::ktOut(l);
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const uint32_t sample = gr * 32 + 16 * j + n;
                const bool live = sample < a.batch;
                float tgtAll = 0.f;
                if (!ta.targets) {
                    float part = 0.f;
#pragma unroll
                    for (int kt = 0; kt < Net::KT0; ++kt) {
                        uint32_t xi[FD];
                        ringRead(x0, Net::KT0, j, kt, xi);
#pragma unroll
                        for (int d = 0; d < FD; ++d) {
                            const halfx2 v = __builtin_bit_cast(halfx2, xi[d]);
                            part += (float)v.x; part += (float)v.y;
                        }
                    }
                    part += __shfl_xor(part, 16);
                    part += __shfl_xor(part, 32);
                    tgtAll = (float)(half_t)sinf(part);
                }
                uint32_t dz[MT][2];
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    const halfx2 y01 = cvt2(acc[j][t][0], acc[j][t][1]), y23 = cvt2(acc[j][t][2], acc[j][t][3]);
                    const half_t yv[4] = {y01.x, y01.y, y23.x, y23.y};
                    half_t gv[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int row = g * OROWS + 4 * t + q;
                        gv[q] = (half_t)0;
                        if (live && row < outDim) {
                            const float tv = ta.targets
                                ? (float)*(const half_t*)(ta.targets + (size_t)sample * ta.targetStride + 2 * row) : tgtAll;
                            const half_t diff = (half_t)((float)yv[q] - tv);
                            lossAcc += (float)diff * (float)diff;
                            gv[q] = (half_t)(2.0f * (float)diff * ta.lossScale);
                        }
                    }
                    dz[t][0] = __builtin_bit_cast(uint32_t, halfx2{gv[0], gv[1]});
                    dz[t][1] = __builtin_bit_cast(uint32_t, halfx2{gv[2], gv[3]});
                }
#pragma unroll
                for (int kt = 0; kt < KTO; ++kt)
                    ringWrite(dout, KTO, j, kt, dz[2 * kt][0], dz[2 * kt][1],
                              2 * kt + 1 < MT ? dz[2 * kt + 1 < MT ? 2 * kt + 1 : 0][0] : 0u,
                              2 * kt + 1 < MT ? dz[2 * kt + 1 < MT ? 2 * kt + 1 : 0][1] : 0u);
            }
        }
    };

    // ---- dX of layer l for round r: D_l -> D_{l-1} through the ReLU of layer l-1 -----------------
    auto backwardX = [&](auto lc, uint32_t r) {
        constexpr int l = decltype(lc)::value;
        if constexpr (l > 0) {
            constexpr int MTI = Net::mt(l - 1), KTO = Net::ktOut(l), KTP = Net::ktOut(l - 1);
            static_assert(KTP == Net::kt(l), "X_l and D_{l-1} share the fragment shape");
            const uint32_t* din = lds + P::dBase(l) + (r & 1u) * P::dSize(l);
            const uint32_t* xin = lds + P::xBase(l) + (r % P::xSlots(l)) * P::xSize(l);
            uint32_t* dout = lds + P::dBase(l - 1) + (r & 1u) * P::dSize(l - 1);
            uint32_t bS[2][KTO][FD];
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int kt = 0; kt < KTO; ++kt) ringRead(din, KTO, j, kt, bS[j][kt]);
            floatx4 gacc[2][MTI];
#pragma unroll
            for (int t = 0; t < MTI; ++t) { gacc[0][t] = floatx4{0.f, 0.f, 0.f, 0.f}; gacc[1][t] = gacc[0][t]; }
#pragma unroll
            for (int kt = 0; kt < KTO; ++kt)
#pragma unroll
                for (int t = 0; t < MTI; ++t) {
                    gacc[0][t] = Mma::mma(fragOf(t * KTO + kt), bS[0][kt], gacc[0][t]);
                    gacc[1][t] = Mma::mma(fragOf(t * KTO + kt), bS[1][kt], gacc[1][t]);
                }
            // multiplier of max(z, 0) from the parked activation a = X_l: a > 0 -> 1, +0 -> 0.5, -0 -> 0:
            // clamp(a*BIG*BIG + copysign(0.5, a), 0, 1)
            const halfx2 big = {(half_t)65504.f, (half_t)65504.f};
            const halfx2 zero2 = {(half_t)0.f, (half_t)0.f}, one2 = {(half_t)1.f, (half_t)1.f};
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int kt = 0; kt < KTP; ++kt) {
                    uint32_t av[FD], d[4] = {0u, 0u, 0u, 0u};
                    ringRead(xin, KTP, j, kt, av);
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        if (2 * kt + h < MTI) {
                            const floatx4& c = gacc[j][2 * kt + h < MTI ? 2 * kt + h : 0];
#pragma unroll
                            for (int q = 0; q < 2; ++q) {
                                const uint32_t ab = av[2 * h + q];
                                const halfx2 av2 = __builtin_bit_cast(halfx2, ab);
                                const halfx2 sgnHalf = __builtin_bit_cast(halfx2, (ab & 0x80008000u) | 0x38003800u);
                                halfx2 m = (av2 * big) * big + sgnHalf;
                                m = __builtin_elementwise_min(__builtin_elementwise_max(m, zero2), one2);
                                d[2 * h + q] = __builtin_bit_cast(uint32_t, cvt2(c[2 * q], c[2 * q + 1]) * m);
                            }
                        }
                    }
                    ringWrite(dout, KTP, j, kt, d[0], d[1], d[2], d[3]);
                }
        }
    };

    // ---- dW / db of layer l for round r ------------------------------------------------------------
    auto backwardW = [&](auto lc, auto sb, auto ab, uint32_t r) {
        constexpr int l = decltype(lc)::value, SB = decltype(sb)::value, AB = decltype(ab)::value;
        constexpr int MT = Net::mt(l), NI = Net::nIt(l), KTO = Net::ktOut(l), KTI = Net::kt(l);
        const uint32_t* din = lds + P::dBase(l) + (r & 1u) * P::dSize(l);
        const uint32_t* xin = lds + P::xBase(l) + (r % P::xSlots(l)) * P::xSize(l);
        uint32_t xF[NI][FD];
#pragma unroll
        for (int e = 0; e < NI; ++e) {
            uint32_t s0[FD], s1[FD];
            ringRead(xin, KTI, 0, e / 2, s0);
            ringRead(xin, KTI, 1, e / 2, s1);
            toF(s0, s1, e & 1, xF[e]);
        }
#pragma unroll
        for (int eo = 0; eo < MT; ++eo) {
            uint32_t s0[FD], s1[FD], dzF[FD];
            ringRead(din, KTO, 0, eo / 2, s0);
            ringRead(din, KTO, 1, eo / 2, s1);
            toF(s0, s1, eo & 1, dzF);
            float sum = accB[AB + eo];
#pragma unroll
            for (int d = 0; d < FD; ++d) sum = __builtin_amdgcn_fdot2(__builtin_bit_cast(halfx2, dzF[d]), ones2, sum, false);
            accB[AB + eo] = sum;
#pragma unroll
            for (int ei = 0; ei < NI; ++ei) S[SB + eo * NI + ei] = Mma::mma(dzF, xF[ei], S[SB + eo * NI + ei]);
        }
    };

    // ---- the pipeline -------------------------------------------------------------------------------
    uint32_t inBuf[2][IN_DW];
    constexpr int kEndsBase = Net::nOt(L - 1) * Net::nIt(L - 1);     // BW_0's tiles follow BW_{L-1}'s
    typedef std::integral_constant<int, kEndsBase> IEndsS;
    typedef std::integral_constant<int, Net::nOt(L - 1)> IEndsB;
    if (role == kRoleF0FL && myRounds) loadInput(inBuf, 0);
    for (uint32_t step = 0; step < totalSteps; ++step) {
        if (role == kRoleF0FL) {
            const uint32_t r0 = step;                              // F_0 works on round `step`
            if (r0 < myRounds) {
                forward(std::integral_constant<int, 0>{}, I0{}, I8{}, r0, inBuf);
                loadInput(inBuf, r0 + 1);                          // next round's input, a step ahead
            }
            const uint32_t rl = step - (uint32_t)P::stepF(L - 1);  // F_{L-1} lags by L-1 steps
            if (step >= (uint32_t)P::stepF(L - 1) && rl < myRounds)
                forward(std::integral_constant<int, L - 1>{}, I12{}, I15{}, rl, inBuf);
        } else if (role == kRoleBWEnds) {
            const uint32_t ra = step - (uint32_t)P::stepBW(L - 1);
            if (step >= (uint32_t)P::stepBW(L - 1) && ra < myRounds) backwardW(std::integral_constant<int, L - 1>{}, I0{}, I0{}, ra);
            const uint32_t rb = step - (uint32_t)P::stepBW(0);
            if (step >= (uint32_t)P::stepBW(0) && rb < myRounds) backwardW(std::integral_constant<int, 0>{}, IEndsS{}, IEndsB{}, rb);
        } else {
            staticFor<1, L>([&](auto lc) {
                constexpr int l = decltype(lc)::value;
                if (layer == l) {
                    if constexpr (l < L - 1) {
                        if (role == kRoleF) {
                            const uint32_t r = step - (uint32_t)P::stepF(l);
                            if (step >= (uint32_t)P::stepF(l) && r < myRounds) forward(lc, I0{}, I8{}, r, inBuf);
                        }
                        if (role == kRoleBW) {
                            const uint32_t r = step - (uint32_t)P::stepBW(l);
                            if (step >= (uint32_t)P::stepBW(l) && r < myRounds) backwardW(lc, I0{}, I0{}, r);
                        }
                    }
                    if (role == kRoleBX) {
                        const uint32_t r = step - (uint32_t)P::stepBX(l);
                        if (step >= (uint32_t)P::stepBX(l) && r < myRounds) backwardX(lc, r);
                    }
                }
            });
        }
        __syncthreads();        // the only barrier of the loop: every wave passes it once per step
    }

    // ---- partials: each BW wave owns its layer's gradients for all samples of this workgroup ------
    float* part = ta.partials + (size_t)blockIdx.x * Net::partialFloats;
    auto writeLayer = [&](auto lc, auto sb, auto ab) {
        constexpr int l = decltype(lc)::value, SB = decltype(sb)::value, AB = decltype(ab)::value;
#pragma unroll
        for (int i = 0; i < Net::nOt(l) * Net::nIt(l); ++i)
            *(floatx4*)&part[(Net::gradTileBase(l) + i) * 256 + lane * 4] = S[SB + i];
#pragma unroll
        for (int eo = 0; eo < Net::nOt(l); ++eo) {
            const float v = accB[AB + eo];          // lane (g,q): sum the four lane groups in a fixed order
            const float s0 = __shfl(v, n), s1 = __shfl(v, n + 16), s2 = __shfl(v, n + 32), s3 = __shfl(v, n + 48);
            if (g == 0) part[Net::totalGradTiles * 256 + (Net::dbTileBase(l) + eo) * 16 + n] = ((s0 + s1) + s2) + s3;
        }
    };
    if (role == kRoleBWEnds) {
        writeLayer(std::integral_constant<int, L - 1>{}, I0{}, I0{});
        writeLayer(std::integral_constant<int, 0>{}, IEndsS{}, IEndsB{});
    }
    staticFor<1, L - 1>([&](auto lc) {
        constexpr int l = decltype(lc)::value;
        if (role == kRoleBW && layer == l) writeLayer(lc, I0{}, I0{});
    });
    if (role == kRoleF0FL) {
        float s = lossAcc;                          // fixed-order butterfly over the wave
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
        if (lane == 0) part[Net::totalGradTiles * 256 + Net::totalDbTiles * 16] = s;
    }
}

} // namespace
} // namespace cv
