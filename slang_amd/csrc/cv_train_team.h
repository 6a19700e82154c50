// cv_train_team.h -- the fused training step with the weights in registers: waves with different jobs.
//
// Same computation and rounding points as mlpTrainKernel (cv_train_impl.h: what the example's
// learnGradient does per shader thread, examples/mlp-training-coopvec/kernels.slang:9-27,
// fflayer.slang:29-58), for networks with up to 16 inputs, one to four ReLU hidden layers of 64 units and up to 16
// outputs.  In the kernels that give every wave whole samples to take through forward pass, backward pass and weight
// gradients, a wave has no registers left for the weights and reads every W and W^T fragment from LDS again for each
// 16 samples.  Here a team of four waves shares the work on a tile of 32 samples by kind:
//
//   forward wave    W of all layers in registers (A operands of v_mfma_f32_32x32x16_f16), takes the tile through the
//                   layers, leaves the input and every hidden layer's pre-activations in LDS, forms the loss and its
//                   gradient dZ of the last layer;
//   backward wave   W^T of layers 1.. in registers: dZ_l = (W^T_(l+1) dZ_(l+1)) * max'(z_l), left in LDS layer by layer;
//   two dW waves    each holds half of the dW / db accumulators of every layer (112 registers for 8-64x4-1) and
//                   contracts dZ_l with X_l = max(z_(l-1), 0) over the 32 samples, both read from LDS transposed
//                   (ds_read_b64_tr_b16: the sample index moves to the k axis of the matrix instruction).
//
// A workgroup is two teams; each SIMD runs one forward or backward wave of one team and one dW wave of the other.  The
// waves of a team hand tiles on through sequence numbers in LDS (teamPublish / teamAwait, bounded waits), two tiles
// in flight per team: the forward wave works on tile k+1 while the backward and dW waves work on tile k.
//
// Hidden units keep their order in memory; matrix row rho of a 32-row tile computes unit 32*T + swap23(rho) (bits 2 and 3
// of rho exchanged), so that the sixteen accumulator registers of a lane are, converted to fp16, the lane's k-slots of the
// next layer's B operand: register r of tile T in lane half h is unit 32*T + 16*(r/8) + 8*h + r%8, k-slot r%8 of half h
// in k-step 2*T + r/8.
//
// Partials and their second-stage reduction are those of the other fused kernels (mlpTrainReduceKernel): same layout,
// fixed order, no atomics, bitwise reproducible.
#pragma once
#include "cv_train_impl.h"
#include "cv_wide_tiles.h"

namespace cv {
namespace {

// One LDS tile = 16 units of 32 samples, fp16: sample n at byte 32*n, the lane half h at 16*h behind it; 128 bytes of
// padding so that the tiles 2*T and 2*T + 1, which the two 16-lane groups of a transposed read touch together, start 32
// banks apart.
constexpr int kTeamTileDW = 288;
constexpr uint32_t kTeamSpinLimit = 1u << 17;

__host__ __device__ constexpr int teamSwap23(int rho) { return (rho & ~12) | ((rho & 4) << 1) | ((rho & 8) >> 1); }

template <int NH>
struct TeamGeom {
    // a slot = what the forward wave leaves of one tile: the input, every hidden layer's pre-activations, dZ of the last layer
    static constexpr int tileX0 = 0;
    static constexpr int tileZ(int l) { return 1 + 4 * l; }                  // pre-activations of hidden layer l < NH
    static constexpr int tileDZLast = 1 + 4 * NH;
    static constexpr int slotTiles = 2 + 4 * NH;
    static constexpr int kSlots = 3;            // tiles in flight per team
    // dZ of the hidden layers goes from the backward wave to the dW waves through a ring of kRing buffers of four tiles;
    // the q-th dZ of a team (q = k * NH + NH - 1 - l for layer l of the team's k-th tile) lies in buffer q % kRing
    static constexpr int kRing = 3;
    static constexpr int teamTiles = kSlots * slotTiles + kRing * 4;
    // fragments (64 lanes x 16 bytes) of the forward wave: layer 0 (T = 0, 1), layers 1..NH-1 ([T][s]), last layer ([s])
    static constexpr int fHidden(int l, int T, int s) { return 2 + 8 * (l - 1) + 4 * T + s; }
    static constexpr int fLast(int s) { return 2 + 8 * (NH - 1) + s; }
    static constexpr int fFrags = 2 + 8 * (NH - 1) + 4;
    // of the backward wave: W^T of the last layer (T = 0, 1), of layers 1..NH-1 ([T][s])
    static constexpr int bHidden(int l, int T, int s) { return 2 + 8 * (l - 1) + 4 * T + s; }
    static constexpr int bFrags = 2 + 8 * (NH - 1);
};

typedef uint32_t __attribute__((address_space(3))) TeamLdsWord;
__device__ __forceinline__ void teamPublish(volatile TeamLdsWord* mine, uint32_t seq)
{
    asm volatile("" ::: "memory");
    *mine = seq;
}
// waits until *flag >= want; returns 1 after a time-out (which only a defect of the kernel could cause: the step's
// result is then declared void instead of the GPU hanging).  After a first time-out nothing is waited for any more.
__device__ __forceinline__ void teamAwait(const volatile TeamLdsWord* flag, uint32_t want, uint32_t& timeouts)
{
    // (everything here is the same in all lanes; said so explicitly, the loop runs on the scalar unit)
    uint32_t spins = 0;
    const uint32_t limit = __builtin_amdgcn_readfirstlane((int)timeouts) ? 0u : kTeamSpinLimit;
    const uint32_t wanted = (uint32_t)__builtin_amdgcn_readfirstlane((int)want);
#pragma nounroll
    while ((uint32_t)__builtin_amdgcn_readfirstlane((int)*flag) < wanted && spins < limit) {
        __builtin_amdgcn_s_sleep(1);
        ++spins;
    }
    asm volatile("" ::: "memory");
    timeouts |= spins >= kTeamSpinLimit ? 1u : 0u;
}

__device__ __forceinline__ u32x2 teamReadTr(const uint32_t* p)
{
    typedef short shortx4 __attribute__((ext_vector_type(4)));
    typedef shortx4 __attribute__((address_space(3))) * LdsPtr;
    return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsPtr)p));
}

// Where element (o, i) of a layer's weight gradient lies in a workgroup's partial: the inverse of the map in
// addToGradients (16x16 tiles in accumulator order; MTO / NI = 16-row tiles of the layer's outputs / inputs).
template <int MTO, int NI>
__device__ __forceinline__ uint32_t teamGradIndex(uint32_t tileBase, uint32_t o, uint32_t i)
{
    const uint32_t gq = o / (4u * MTO), eo = (o % (4u * MTO)) / 4u, r = o % 4u;
    const uint32_t ei = (i % (4u * NI)) / 4u, qi = 4u * (i / (4u * NI)) + i % 4u;
    return (tileBase + eo * NI + ei) * 256u + (gq * 16u + qi) * 4u + r;
}
template <int MTO>
__device__ __forceinline__ uint32_t teamDbIndex(uint32_t tileBase, uint32_t o)
{
    return (tileBase + (o % (4u * MTO)) / 4u) * 16u + 4u * (o / (4u * MTO)) + o % 4u;
}

template <class Net>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void mlpTrainTeamKernel(const TrainArgs ta)
{
    constexpr int NH = Net::NHID, L = NH + 1;
    static_assert(Net::IT0 == 1 && Net::KT0 == 1 && Net::HT == 4 && Net::MTL == 1, "up to 16 inputs, 64-wide hidden layers, up to 16 outputs");
    typedef TeamGeom<NH> G;
    typedef float floatx2 __attribute__((ext_vector_type(2)));
    const MlpArgs& a = ta.mlp;
    constexpr int SLOT_DW = G::slotTiles * kTeamTileDW;
    constexpr int TEAM_DW = G::teamTiles * kTeamTileDW;
    constexpr int SEED_DW = (2 * NH + 1) * 32;
    constexpr int FLAG_DW = 16;
    static_assert((2 * TEAM_DW + SEED_DW + FLAG_DW) * 4 <= 160 * 1024, "LDS of one compute unit");
    static_assert((G::fFrags + G::bFrags) * 256 <= 2 * TEAM_DW, "the weights are staged in the tile area");
    __shared__ __attribute__((aligned(16))) uint32_t lds[2 * TEAM_DW + SEED_DW + FLAG_DW];
    float* const ldsSeed = (float*)(lds + 2 * TEAM_DW);
    uint32_t* const ldsFlag = lds + 2 * TEAM_DW + SEED_DW;
    if (threadIdx.x < FLAG_DW) ldsFlag[threadIdx.x] = 0u;

    // ---- float(bias) in accumulator order: [2*l + T][h][r] = bias of unit 32*T + 16*(r/8) + 8*h + r%8 -------------
    for (int c = threadIdx.x; c < SEED_DW; c += 512) {
        const int f = c >> 5, hh = (c >> 4) & 1, r = c & 15;
        const int l = f >> 1, T = f & 1, unit = 32 * T + 16 * (r / 8) + 8 * hh + r % 8;
        float v = 0.f;
        if (a.layers[l].bias && unit < a.layers[l].out) v = (float)((const half_t*)a.layers[l].bias)[unit];
        ldsSeed[c] = v;
    }

    // ---- W and W^T into LDS in operand order: all loads first, then all stores (one round trip to memory) ----------
    {
        constexpr int TOTAL = (G::fFrags + G::bFrags) * 64;
        constexpr int NCH = (TOTAL + 511) / 512;
        uint32_t stg[NCH][8];
        uint32_t ok[NCH];
#pragma unroll
        for (int it = 0; it < NCH; ++it) {
            const int c = threadIdx.x + 512 * it;
            int f = c >> 6;
            const int ln = c & 63, rho = ln & 31, hh = ln >> 5;
            const bool back = f >= G::fFrags;
            if (back) f -= G::fFrags;
            // (l, T, s) of the fragment
            int l, T, s;
            if (f < 2) { l = back ? NH : 0; T = f; s = 0; }
            else if (!back && f >= 2 + 8 * (NH - 1)) { l = NH; T = 0; s = f - (2 + 8 * (NH - 1)); }
            else { l = 1 + (f - 2) / 8; T = ((f - 2) >> 2) & 1; s = (f - 2) & 3; }
            const MlpLayerArgs& ly = a.layers[l];
            const int across = 32 * T + teamSwap23(rho);      // the unit of the operand's row
            const int along0 = 16 * s + 8 * hh;               // the first of the lane's eight k-slots
            // Row/ColumnMajor only (the launcher sends other layouts to the other kernels): bytes from row to row, column to column
            const bool rowMajor = ly.shape.layout == kRowMajor;
            const uint32_t line = ly.shape.stride ? (uint32_t)ly.shape.stride : 2u * (rowMajor ? ly.shape.cols : ly.shape.rows);
            const uint32_t sr = rowMajor ? line : 2u, sc = rowMajor ? 2u : line;
            ok[it] = 0u;
            // the lane's eight elements lie side by side in memory (W row-major, W^T column-major) and are all there or all
            // missing: one 16-byte load
            const int alongEnd = back ? ly.out : ly.in;
            const bool fast = back != rowMajor && line % 16u == 0 && ((uintptr_t)ly.w & 15u) == 0 && alongEnd % 8 == 0;
            if (fast) {
                const bool valid = c < TOTAL && across < (back ? ly.in : ly.out) && along0 < alongEnd;
                const u32x4 v = *(const u32x4*)(ly.w + (valid ? (uint32_t)across * line + 2u * (uint32_t)along0 : 0u));
                stg[it][0] = v.x; stg[it][1] = v.y; stg[it][2] = v.z; stg[it][3] = v.w;
                ok[it] = valid ? 0x300u : 0x200u;
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int row = back ? along0 + e : across, col = back ? across : along0 + e;
                    const bool valid = c < TOTAL && row < ly.out && col < ly.in;
                    const uint32_t off = valid ? (uint32_t)row * sr + (uint32_t)col * sc : 0u;
                    stg[it][e] = *(const uint16_t*)(ly.w + off);
                    ok[it] |= valid ? 1u << e : 0u;
                }
            }
        }
#pragma unroll
        for (int it = 0; it < NCH; ++it) {
            const int c = threadIdx.x + 512 * it;
            uint32_t v[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = (ok[it] >> e & 1u) ? stg[it][e] : 0u;
            u32x4 out = {v[0] | v[1] << 16, v[2] | v[3] << 16, v[4] | v[5] << 16, v[6] | v[7] << 16};
            if (ok[it] & 0x200u) {
                const uint32_t m = (ok[it] & 0x100u) ? 0xffffffffu : 0u;
                out = u32x4{stg[it][0] & m, stg[it][1] & m, stg[it][2] & m, stg[it][3] & m};
            }
            if (c < TOTAL) *(u32x4*)&lds[4 * c] = out;
        }
    }
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 31, h = lane >> 5;
    const int team = wave >> 2;
    // 0 forward, 1 backward, 2 and 3 dW.  Waves w and w + 4 share a SIMD: a forward or backward wave of one team with a dW
    // wave of the other (two waves of a kind on one SIMD were slower: 176 against 151 us for 8-64x4-1 at 2^20 samples)
    const int role = team == 0 ? (wave & 3) : ((wave + 2) & 3);
    // the role's weights: the lane's 16 bytes of each fragment
    uint32_t wreg[G::fFrags][4];
    if (role < 2) {
#pragma unroll
        for (int f = 0; f < G::fFrags; ++f) {
            if (role == 0 || f < G::bFrags) {
                const u32x4 v = *(const u32x4*)&lds[(((role == 0 ? 0 : G::fFrags) + f) * 64 + lane) * 4];
                wreg[f][0] = v.x; wreg[f][1] = v.y; wreg[f][2] = v.z; wreg[f][3] = v.w;
            }
        }
    }
    __syncthreads();          // the tile area is free

    const uint32_t numTiles = (a.batch + 31u) / 32u;
    const uint32_t numTeams = 2u * gridDim.x, firstTile = 2u * blockIdx.x + (uint32_t)team;
    const uint32_t myTiles = firstTile < numTiles ? (numTiles - firstTile + numTeams - 1u) / numTeams : 0u;
    const uint32_t lastSample = a.batch - 1u;
    uint32_t* const teamTiles = lds + team * TEAM_DW;
    uint32_t* const teamRing = teamTiles + G::kSlots * SLOT_DW;
    // Progress of the team's waves: tiles the forward wave has left in their slots; dZ buffers the backward wave has
    // filled; dZ buffers each dW wave has read (NH per tile, the last one of a tile after everything else of the tile).
    volatile TeamLdsWord* const fDone = (TeamLdsWord*)(ldsFlag + 4 * team);
    volatile TeamLdsWord* const bProg = (TeamLdsWord*)(ldsFlag + 4 * team + 1);
    volatile TeamLdsWord* const dProg0 = (TeamLdsWord*)(ldsFlag + 4 * team + 2);
    volatile TeamLdsWord* const dProg1 = (TeamLdsWord*)(ldsFlag + 4 * team + 3);
    uint32_t* const ldsLossMax = ldsFlag + 8;
    uint32_t* const ldsTimeouts = ldsFlag + 9;
    uint32_t timeouts = 0;
    const int sOff = n * 8 + 4 * h;                 // dwords: where lane (n, h) keeps its 16 bytes of a tile
    const halfx2 zero2 = {(half_t)0.f, (half_t)0.f};
    const floatx16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    // the dW waves' accumulators (live to the end of the kernel)
    floatx4 acc0[2], accL[2];
    floatx16 accH[NH > 1 ? NH - 1 : 1][2];
    float dbAcc0[2] = {0.f, 0.f}, dbAccH[NH > 1 ? NH - 1 : 1], dbAccL = 0.f;
#pragma unroll
    for (int j = 0; j < 2; ++j) { acc0[j] = floatx4{0.f, 0.f, 0.f, 0.f}; accL[j] = floatx4{0.f, 0.f, 0.f, 0.f}; }
#pragma unroll
    for (int l = 0; l < (NH > 1 ? NH - 1 : 1); ++l) { accH[l][0] = zero16; accH[l][1] = zero16; dbAccH[l] = 0.f; }
    float lossAcc = 0.f, lossMaxAcc = 0.f;

    if (role == 0) {
        // =========================================== forward wave ===========================================
        // A layer's matrix instructions are issued k-steps 0 and 1 first: they need only the first 32 units of the layer
        // before (tile T = 0 of its accumulators), so the conversion of the other 32 runs in their shadow; the two layers'
        // accumulators alternate between two register sets, and a set is filled with the biases of the layer after next as
        // soon as its values have been converted.
        __builtin_amdgcn_s_setprio(2);      // the forward and backward waves are the chain the others wait for
        const int in0 = a.layers[0].in, outDim = a.layers[NH].out;
        const int validBytes = min(8, max(in0 - 8 * h, 0)) * 2;
        auto loadTile = [&](uint32_t (&raw)[4], uint32_t k) {
            const uint32_t s = min((firstTile + k * numTeams) * 32u + (uint32_t)n, lastSample);
            const uint8_t* row = a.in + (size_t)s * a.inStride;
            const uint8_t* p = row + 16 * h;
#pragma unroll
            for (int i = 0; i < 4; ++i) raw[i] = *(const uint32_t*)(4 * i < validBytes ? p + 4 * i : row);
        };
        uint32_t seedOff = (uint32_t)h * 16u;
        auto seed = [&](int l, int T) -> floatx16 {
            const floatx4* p = (const floatx4*)&ldsSeed[(2 * l + T) * 32 + seedOff];
            const floatx4 s0 = p[0], s1 = p[1], s2 = p[2], s3 = p[3];
            return floatx16{s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3], s2[0], s2[1], s2[2], s2[3], s3[0], s3[1], s3[2], s3[3]};
        };
        uint32_t cur[4], nxt[4];
        loadTile(cur, 0);
        floatx16 acc[2][2];
        acc[0][0] = seed(0, 0); acc[0][1] = seed(0, 1);
        for (uint32_t k = 0; k < myTiles; ++k) {
            loadTile(nxt, k + 1 < myTiles ? k + 1 : k);
            asm volatile("" : "+v"(seedOff));       // the bias lines are read again for every tile, not kept in registers
            uint32_t* const slot = teamTiles + (k % (uint32_t)G::kSlots) * SLOT_DW;
            const uint32_t sample = (firstTile + k * numTeams) * 32u + (uint32_t)n;
            const bool live = sample < a.batch;
            uint32_t B[4][4];
#pragma unroll
            for (int i = 0; i < 4; ++i) B[0][i] = 4 * i < validBytes ? cur[i] : 0u;
            float tgtAll = 0.f;
            if (!ta.targets) {
                float part = 0.f;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const halfx2 v = __builtin_bit_cast(halfx2, B[0][i]);
                    part += (float)v.x; part += (float)v.y;
                }
                part += __shfl_xor(part, 32, 64);
                tgtAll = (float)(half_t)sinf(part);
            }
            // the tile that lay in this slot has been contracted by both dW waves
            if (k >= (uint32_t)G::kSlots) {
                teamAwait(dProg0, (k + 1u - (uint32_t)G::kSlots) * (uint32_t)NH, timeouts);
                teamAwait(dProg1, (k + 1u - (uint32_t)G::kSlots) * (uint32_t)NH, timeouts);
            }
            *(u32x4*)(slot + G::tileX0 * kTeamTileDW + sOff) = u32x4{B[0][0], B[0][1], B[0][2], B[0][3]};
            acc[0][0] = mfma32(wreg[0], B[0], acc[0][0]);
            acc[0][1] = mfma32(wreg[1], B[0], acc[0][1]);
            if constexpr (NH >= 2) { acc[1][0] = seed(1, 0); acc[1][1] = seed(1, 1); }
            else acc[1][0] = seed(NH, 0);
            staticFor<0, NH>([&](auto lc) {
                constexpr int l = decltype(lc)::value;       // the hidden layer whose pre-activations are in acc[l & 1]
                constexpr int cs = l & 1, ns = cs ^ 1;
                constexpr bool last = l + 1 == NH;           // the layer computed next is the network's last one
                // fp32 -> fp16 = z_l (to LDS), ReLU = the next layer's operands: units 32*T .. 32*T + 31
                auto carrier = [&](int T) {
#pragma unroll
                    for (int s2 = 0; s2 < 2; ++s2) {
                        const int s = 2 * T + s2, r0 = 8 * s2;
                        uint32_t z[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const halfx2 zz = __builtin_convertvector(floatx2{acc[cs][T][r0 + 2 * i], acc[cs][T][r0 + 2 * i + 1]}, halfx2);
                            z[i] = __builtin_bit_cast(uint32_t, zz);
                            B[s][i] = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(zz, zero2));
                        }
                        *(u32x4*)(slot + (G::tileZ(l) + s) * kTeamTileDW + sOff) = u32x4{z[0], z[1], z[2], z[3]};
                    }
                };
                auto steps = [&](int T, int s0, int s1) {
#pragma unroll
                    for (int s = s0; s < s1; ++s)
                        acc[ns][T] = mfma32(wreg[last ? G::fLast(s) : G::fHidden(l + 1, T, s)], B[s], acc[ns][T]);
                };
                carrier(0);
                steps(0, 0, 1); if constexpr (!last) steps(1, 0, 1);
                steps(0, 1, 2); if constexpr (!last) steps(1, 1, 2);
                carrier(1);
                steps(0, 2, 3); if constexpr (!last) steps(1, 2, 3);
                steps(0, 3, 4); if constexpr (!last) steps(1, 3, 4);
                if constexpr (l + 2 < NH) { acc[cs][0] = seed(l + 2, 0); acc[cs][1] = seed(l + 2, 1); }
                else if constexpr (l + 2 == NH) acc[cs][0] = seed(NH, 0);
            });
            const floatx16 yAcc = acc[NH & 1][0];
            // ---- loss and its gradient: register r < 8 of lane half h is output 8*h + r ----
            {
                half_t gv[8];
                float sampleLoss = 0.f;
#pragma unroll
                for (int r = 0; r < 8; ++r) {
                    gv[r] = (half_t)0;
                    if (r >= outDim) continue;            // wave-uniform: a one-output network takes one of the eight steps
                    const int unit = 8 * h + r;
                    const bool on = live && unit < outDim;
                    float tv = tgtAll;
                    if (ta.targets)
                        tv = (float)*(const half_t*)(ta.targets + (size_t)min(sample, lastSample) * ta.targetStride + 2 * (on ? unit : 0));
                    const half_t y = (half_t)yAcc[r];
                    const half_t diff = (half_t)((float)y - tv);
                    lossAcc += on ? (float)diff * (float)diff : 0.f;
                    sampleLoss += on ? (float)diff * (float)diff : 0.f;
                    gv[r] = on ? (half_t)(2.0f * (float)diff * ta.lossScale) : (half_t)0;
                }
                if (ta.wantLossMax) {
                    const float whole = sampleLoss + __shfl_xor(sampleLoss, 32, 64);
                    lossMaxAcc = (whole > lossMaxAcc || whole != whole) ? whole : lossMaxAcc;
                }
                u32x4 d;
                d.x = __builtin_bit_cast(uint32_t, halfx2{gv[0], gv[1]});
                d.y = __builtin_bit_cast(uint32_t, halfx2{gv[2], gv[3]});
                d.z = __builtin_bit_cast(uint32_t, halfx2{gv[4], gv[5]});
                d.w = __builtin_bit_cast(uint32_t, halfx2{gv[6], gv[7]});
                *(u32x4*)(slot + G::tileDZLast * kTeamTileDW + sOff) = d;
            }
            teamPublish(fDone, k + 1u);
            // the next tile's first layer starts from its biases (the set that holds them is free: layer NH - 1 was converted,
            // the last layer's result has been read)
            acc[0][0] = seed(0, 0); acc[0][1] = seed(0, 1);
#pragma unroll
            for (int i = 0; i < 4; ++i) { pinHere(nxt[i]); cur[i] = nxt[i]; }
        }
    } else if (role == 1) {
        // =========================================== backward wave ==========================================
        // same order as in the forward wave: the k-steps that need only the first half of dZ_l first
        __builtin_amdgcn_s_setprio(2);
        floatx16 g[2][2];
        for (uint32_t k = 0; k < myTiles; ++k) {
            uint32_t* const slot = teamTiles + (k % (uint32_t)G::kSlots) * SLOT_DW;
            teamAwait(fDone, k + 1u, timeouts);
            uint32_t B[4][4], z[2][4][4];
            auto readZ = [&](int l, uint32_t (&dst)[4][4]) {
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const u32x4 v = *(const u32x4*)(slot + (G::tileZ(l) + s) * kTeamTileDW + sOff);
                    dst[s][0] = v.x; dst[s][1] = v.y; dst[s][2] = v.z; dst[s][3] = v.w;
                }
            };
            {
                const u32x4 v = *(const u32x4*)(slot + G::tileDZLast * kTeamTileDW + sOff);
                B[0][0] = v.x; B[0][1] = v.y; B[0][2] = v.z; B[0][3] = v.w;
            }
            readZ(NH - 1, z[0]);
            g[0][0] = mfma32(wreg[0], B[0], zero16);
            g[0][1] = mfma32(wreg[1], B[0], zero16);
            staticFor<0, NH>([&](auto jc) {
                constexpr int j = decltype(jc)::value, l = NH - 1 - j;      // the hidden layer whose dZ is formed from g[j & 1]
                constexpr int cs = j & 1, ns = cs ^ 1;
                if constexpr (l > 0) readZ(l - 1, z[ns]);
                const uint32_t q = k * (uint32_t)NH + (uint32_t)j;       // this dZ's number, and the buffer it goes to
                uint32_t* const buf = teamRing + (q % (uint32_t)G::kRing) * (4 * kTeamTileDW);
                auto carrier = [&](int T) {
#pragma unroll
                    for (int s2 = 0; s2 < 2; ++s2) {
                        const int s = 2 * T + s2, r0 = 8 * s2;
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const halfx2 gg = __builtin_convertvector(floatx2{g[cs][T][r0 + 2 * i], g[cs][T][r0 + 2 * i + 1]}, halfx2);
                            const halfx2 dz = gg * maxGradMultiplier(__builtin_bit_cast(halfx2, z[cs][s][i]));
                            B[s][i] = __builtin_bit_cast(uint32_t, dz);
                        }
                    }
                };
                auto put = [&](int T) {
#pragma unroll
                    for (int s = 2 * T; s < 2 * T + 2; ++s) *(u32x4*)(buf + s * kTeamTileDW + sOff) = u32x4{B[s][0], B[s][1], B[s][2], B[s][3]};
                };
                auto steps = [&](int T, int s0, int s1) {
                    if constexpr (l > 0) {
#pragma unroll
                        for (int s = s0; s < s1; ++s) g[ns][T] = mfma32(wreg[G::bHidden(l, T, s)], B[s], s == 0 ? zero16 : g[ns][T]);
                    }
                };
                carrier(0);
                steps(0, 0, 2);
                // both dW waves have read what lay in the buffer
                if (q >= (uint32_t)G::kRing) {
                    teamAwait(dProg0, q + 1u - (uint32_t)G::kRing, timeouts);
                    teamAwait(dProg1, q + 1u - (uint32_t)G::kRing, timeouts);
                }
                put(0);
                carrier(1);
                put(1);
                teamPublish(bProg, q + 1u);
                steps(1, 0, 1); steps(0, 2, 3); steps(1, 1, 2); steps(0, 3, 4); steps(1, 2, 4);
            });
        }
    } else {
        // ============================================= dW waves =============================================
        const int w = role - 2;
        const halfx2 ones2 = {(half_t)1.f, (half_t)1.f};
        // transposed reads.  Operands of the 32x32x16 instruction: lane (i, hk) = unit i of a 32-unit tile, samples
        // 16*ks + 8*hk .. + 7 in two reads of four; of the 16x16x32 instruction: lane (i, g) = unit i of a 16-unit tile,
        // samples 4*g .. 4*g + 3 and 16 + 4*g .. 16 + 4*g + 3.  Within a 16-lane group, lane q hands in the address of the
        // 8 bytes (sample q/4 of the four, units 4*(q%4) ..).
        const int q = lane & 15;
        const int tr32 = ((lane >> 4) & 1) * kTeamTileDW + (8 * (lane >> 5) + (q >> 2)) * 8 + 2 * (q & 3);
        const int tr16 = (4 * (lane >> 4) + (q >> 2)) * 8 + 2 * (q & 3);
        auto read32 = [&](const uint32_t* tiles, int T, int ks, uint32_t* frag) {      // tiles: the vector's first tile
            const u32x2 lo = teamReadTr(tiles + 2 * T * kTeamTileDW + tr32 + (16 * ks) * 8);
            const u32x2 hi = teamReadTr(tiles + 2 * T * kTeamTileDW + tr32 + (16 * ks + 4) * 8);
            frag[0] = lo.x; frag[1] = lo.y; frag[2] = hi.x; frag[3] = hi.y;
        };
        auto read16 = [&](const uint32_t* tile, uint32_t* frag) {
            const u32x2 lo = teamReadTr(tile + tr16);
            const u32x2 hi = teamReadTr(tile + tr16 + 16 * 8);
            frag[0] = lo.x; frag[1] = lo.y; frag[2] = hi.x; frag[3] = hi.y;
        };
        // max(z, 0) on the bits (as 16-bit integers the negative halves are the negative numbers): one instruction per pair,
        // where the floating-point maximum of a value that was loaded, not computed, costs a second one to quieten NaNs
        auto relu4 = [&](uint32_t* frag) {
            typedef short shortx2 __attribute__((ext_vector_type(2)));
#pragma unroll
            for (int d = 0; d < 4; ++d)
                frag[d] = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(shortx2, frag[d]), shortx2{0, 0}));
        };
        auto dot4 = [&](const uint32_t* frag, float s) {
#pragma unroll
            for (int d = 0; d < 4; ++d) s = __builtin_amdgcn_fdot2(__builtin_bit_cast(halfx2, frag[d]), ones2, s, false);
            return s;
        };
        volatile TeamLdsWord* const myProg = w == 0 ? dProg0 : dProg1;
        // The operands of a step (one layer of one tile) are requested one step ahead, so that their way from LDS is
        // covered by the step before: the last layer's in registers of their own, the hidden layers' alternately in two sets.
        uint32_t dzL[4], xL[2][4];
        uint32_t xs[2][2][2][4], dzs[2][2][4];
        auto requestLast = [&](uint32_t k) {
            const uint32_t* const slot = teamTiles + (k % (uint32_t)G::kSlots) * SLOT_DW;
            teamAwait(fDone, k + 1u, timeouts);
            read16(slot + G::tileDZLast * kTeamTileDW, dzL);
#pragma unroll
            for (int j = 0; j < 2; ++j) read16(slot + (G::tileZ(NH - 1) + 2 * w + j) * kTeamTileDW, xL[j]);
        };
        auto requestHidden = [&](uint32_t k, auto lc) {
            constexpr int l = decltype(lc)::value, b = l & 1;
            const uint32_t* const slot = teamTiles + (k % (uint32_t)G::kSlots) * SLOT_DW;
            const uint32_t q = k * (uint32_t)NH + (uint32_t)(NH - 1 - l);
            const uint32_t* const buf = teamRing + (q % (uint32_t)G::kRing) * (4 * kTeamTileDW);
            // (the number is asked for before anything else of the step: the wait for its way from LDS then covers no
            // other request)
            teamAwait(bProg, q + 1u, timeouts);
            if constexpr (l > 0) {
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) read32(buf, w, ks, dzs[b][ks]);
#pragma unroll
                for (int Tc = 0; Tc < 2; ++Tc)
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks) read32(slot + G::tileZ(l - 1) * kTeamTileDW, Tc, ks, xs[b][Tc][ks]);
            } else {
                read16(slot + G::tileX0 * kTeamTileDW, xs[b][0][0]);
#pragma unroll
                for (int j = 0; j < 2; ++j) read16(buf + (2 * w + j) * kTeamTileDW, dzs[b][j]);
            }
            // LDS serves a wave's requests in order: the reads above come before this number (after layer 0 it also says
            // that the tile's slot is free)
            teamPublish(myProg, q + 1u);
        };
        const uint32_t dTiles = myTiles;
        if (dTiles > 0) requestLast(0);
        for (uint32_t k = 0; k < dTiles; ++k) {
            // ---- last layer: dZ (one tile of outputs) x X = max(z_(NH-1), 0), this wave's two tiles of it ----
            requestHidden(k, std::integral_constant<int, NH - 1>{});
            {
#pragma unroll
                for (int j = 0; j < 2; ++j) relu4(xL[j]);
                if (w == 0) dbAccL = dot4(dzL, dbAccL);
#pragma unroll
                for (int j = 0; j < 2; ++j) accL[j] = F16Mma::mma(dzL, xL[j], accL[j]);
            }
            // ---- hidden layers, from the last one down ----
            staticFor<0, NH>([&](auto lc) {
                constexpr int l = NH - 1 - decltype(lc)::value, b = l & 1;
                if constexpr (l > 0) requestHidden(k, std::integral_constant<int, (l > 0 ? l - 1 : 0)>{});
                else if (k + 1 < dTiles) requestLast(k + 1);
                if constexpr (l > 0) {
#pragma unroll
                    for (int Tc = 0; Tc < 2; ++Tc)
#pragma unroll
                        for (int ks = 0; ks < 2; ++ks) relu4(xs[b][Tc][ks]);
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks) dbAccH[l - 1] = dot4(dzs[b][ks], dbAccH[l - 1]);
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                        for (int Tc = 0; Tc < 2; ++Tc) accH[l - 1][Tc] = mfma32(dzs[b][ks], xs[b][Tc][ks], accH[l - 1][Tc]);
                } else {
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        dbAcc0[j] = dot4(dzs[b][j], dbAcc0[j]);
                        acc0[j] = F16Mma::mma(dzs[b][j], xs[b][0][0], acc0[j]);
                    }
                }
            });
        }
    }

    __builtin_amdgcn_s_setprio(0);
    // ---- the workgroup's partial: team 0 + team 1, value by value ------------------------------------------------------
    if (timeouts && lane == 0) atomicOr(ldsTimeouts, 1u);
    if (role == 0 && ta.wantLossMax) noteLossMax(ldsLossMax, lossMaxAcc);
    __syncthreads();                              // every team has left its last tile: the tile area is free
    float* const ldsPart = (float*)lds;           // the workgroup's partial, in the order in which it goes to memory
    float* part = ta.partials + (size_t)blockIdx.x * Net::partialFloats;
    constexpr uint32_t nW = Net::totalGradTiles * 256, nB = Net::totalDbTiles * 16;
    float* const ldsLoss = ldsPart + nW + nB;     // the two forward waves' losses
    static_assert(nW + nB + 128 <= 4 * SLOT_DW, "the final sums reuse the tile area");
    const int wD = role - 2, g4 = lane >> 4, i16 = lane & 15;
    // every value of a dW wave with the index of the partial it belongs to
    auto forEach = [&](auto&& fn) {
        const int w = wD;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                fn(acc0[j][r], teamGradIndex<4, 1>(Net::gradTileBase(0), 16u * (2 * w + j) + 4u * g4 + r, (uint32_t)i16), true);
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                fn(accL[j][r], teamGradIndex<1, 4>(Net::gradTileBase(NH), 4u * g4 + r, 16u * (2 * w + j) + i16), true);
#pragma unroll
        for (int l = 1; l < NH; ++l)
#pragma unroll
            for (int Tc = 0; Tc < 2; ++Tc)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    fn(accH[l - 1][Tc][r], teamGradIndex<4, 4>(Net::gradTileBase(l), 32u * w + 8u * (r / 4) + 4u * h + r % 4, 32u * Tc + n), true);
#pragma unroll
        for (int j = 0; j < 2; ++j) fn(dbAcc0[j], nW + teamDbIndex<4>(Net::dbTileBase(0), 16u * (2 * w + j) + i16), g4 == 0);
#pragma unroll
        for (int l = 1; l < NH; ++l) fn(dbAccH[l - 1], nW + teamDbIndex<4>(Net::dbTileBase(l), 32u * w + n), h == 0);
        fn(dbAccL, nW + teamDbIndex<1>(Net::dbTileBase(NH), (uint32_t)i16), g4 == 0 && w == 0);
    };
    if (role >= 2) {
        // the bias gradients of a unit lie in the lanes that hold its samples: summed in a fixed order, then in every one of them
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            dbAcc0[j] += __shfl_xor(dbAcc0[j], 16, 64);
            dbAcc0[j] += __shfl_xor(dbAcc0[j], 32, 64);
        }
        dbAccL += __shfl_xor(dbAccL, 16, 64);
        dbAccL += __shfl_xor(dbAccL, 32, 64);
#pragma unroll
        for (int l = 0; l < NH - 1; ++l) dbAccH[l] += __shfl_xor(dbAccH[l], 32, 64);
        if (team == 1) forEach([&](float x, uint32_t p, bool mine) { if (mine) ldsPart[p] = x; });
    } else if (role == 0) {
        ldsLoss[team * 64 + lane] = lossAcc;
    }
    __syncthreads();
    if (role >= 2 && team == 0) forEach([&](float x, uint32_t p, bool mine) { if (mine) ldsPart[p] = x + ldsPart[p]; });
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < (nW + nB) / 4u; i += 512u) __builtin_nontemporal_store(((const floatx4*)ldsPart)[i], (floatx4*)part + i);
    if (wave == 0) {
        float s = ldsLoss[lane] + ldsLoss[64 + lane];
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) s += __shfl_xor(s, d, 64);
        if (*ldsTimeouts) s = __builtin_nanf("");
        if (lane == 0) {
            part[nW + nB] = s;
            part[nW + nB + 1] = __builtin_bit_cast(float, *ldsLossMax);
        }
    }
}

} // namespace
} // namespace cv
