// cv_train_impl.h -- fused forward + backward of the fp16 MLP for gfx950.
//
// Replaces what the example's learnGradient kernel does per shader thread
// (examples/mlp-training-coopvec/kernels.slang:9-27 -> bwd_diff(loss), fflayer.slang:29-58:
// coopVecOuterProductAccumulate + coopVecReduceSumAccumulate + coopVecMatMul with the transposed
// weights; the per-thread atomics of those operators are documented at
// source/slang/hlsl.meta.slang:33200-33224, 33318-33326) by a batch formulation:
//
//   - forward and dX = W^T dY run like the fused forward kernel: 16 samples are the N dimension
//     of an MFMA, the carrier CoopVec<half> stays in VGPRs between layers ("S" orientation:
//     lane%16 = sample, features over lane groups and registers);
//   - the weight gradient dW = sum_s dY_s (x) X_s is an MFMA contraction over the batch.  It
//     needs both operands with the sample index on the k axis ("F" orientation: lane%16 =
//     feature).  An S fragment is turned into F fragments exactly, by an MFMA against a 0/1
//     selection matrix (values are copied, not rounded);
//   - every wave accumulates its share of dW / db in fp32 registers over all of its samples;
//     at the end the four waves of a workgroup are summed in LDS in a fixed order and written
//     as one partial per workgroup; a second kernel sums the partials in a fixed order and
//     adds them to the gradient buffers ("+=", any layout, fp16 or fp32).  No atomics: the
//     result is bitwise reproducible.
//
// Derivative rules follow Slang: max(x,y) sends the whole gradient to the larger operand and
// half to each at a tie (source/slang/diff.meta.slang:2258-2277).
#pragma once
#include <type_traits>

#include "cv_mlp_impl.h"

namespace cv {
namespace {

// tile bookkeeping on top of UniformNet; IT0 = 16-feature tiles of the network input
template <int IT0_, int KT0_, int HT_, int NHID_, int MTL_>
struct TrainNet : UniformNet<KT0_, HT_, NHID_, MTL_> {
    typedef UniformNet<KT0_, HT_, NHID_, MTL_> Base;
    static constexpr int IT0 = IT0_;
    static constexpr int L = Base::L;
    static constexpr int nOt(int l) { return Base::mt(l); }
    static constexpr int nIt(int l) { return l == 0 ? IT0_ : Base::mt(l - 1); }
    static constexpr int ktOut(int l) { return (Base::mt(l) + 1) / 2; }   // S fragments of layer l's output
    static constexpr int ITMAX = IT0_ > HT_ ? IT0_ : HT_;
    static constexpr int KOMAX = (Base::MTMAX + 1) / 2;
    // transposed weights (A operand of dX = W^T dY) exist for layers 1..L-1
    static constexpr int tFragBase(int l)
    {
        int b = 0;
        for (int i = 1; i < l; ++i) b += Base::mt(i - 1) * ktOut(i);
        return b;
    }
    static constexpr int totalTFrags = tFragBase(L);
    static constexpr int gradTileBase(int l)
    {
        int b = 0;
        for (int i = 0; i < l; ++i) b += nOt(i) * nIt(i);
        return b;
    }
    static constexpr int totalGradTiles = gradTileBase(L);
    static constexpr int xTileBase(int l)
    {
        int b = 0;
        for (int i = 0; i < l; ++i) b += nIt(i);
        return b;
    }
    static constexpr int totalXTiles = xTileBase(L);
    static constexpr int dbTileBase(int l) { return Base::biasBase(l); }
    static constexpr int totalDbTiles = Base::totalBiasTiles;
    // floats of one workgroup's partial: dW tiles, db tiles, loss
    static constexpr int partialFloats = totalGradTiles * 256 + totalDbTiles * 16 + 16;
};

struct TrainReduceArgs {
    struct Layer {
        uint8_t* wGrad; uint8_t* bGrad;
        MatrixShape gradShape;   // out x in as the gradient lies in memory
        int32_t in, out;
    } layers[kMaxMlpLayers];
    int32_t numLayers;
    int32_t gradCt;              // kF16 or kF32, also the type of the bias gradients
    const float* partials;
    uint32_t numPartials;
    float* lossSum;              // optional
    float* lossMax;              // optional
};

struct TrainArgs {
    MlpArgs mlp;                 // layers, input, batch (out/outStride unused)
    const uint8_t* targets;      // fp16 [batch][lastOut] or nullptr: sin(sum of the inputs)
    uint64_t targetStride;
    float lossScale;
    float* partials;             // [gridDim.x][partialFloats]
    int32_t wantLossMax;         // also track the largest per-sample loss (slot 1 behind the loss sum of a partial)
    // A launch of a single workgroup (a batch of at most four tiles, such as the example's 16 samples) adds its sums to
    // the gradients itself, from its registers: no partial in memory, no second kernel.  `finish` then holds what that
    // kernel would have been given.
    int32_t finishInKernel;
    TrainReduceArgs finish;
};


// what the second kernel of a step is given: where the sums of `blocks` partials go
template <class Net>
TrainReduceArgs makeTrainReduceArgs(const TrainLaunch& t, uint32_t blocks)
{
    TrainReduceArgs ra;
    for (int l = 0; l < Net::L; ++l) {
        ra.layers[l].wGrad = t.wGrad[l];
        ra.layers[l].bGrad = t.bGrad[l];
        ra.layers[l].gradShape = t.gradShape[l];
        ra.layers[l].in = t.mlp.layers[l].in;
        ra.layers[l].out = t.mlp.layers[l].out;
    }
    ra.numLayers = Net::L;
    ra.gradCt = t.gradCt;
    ra.partials = t.workspace;
    ra.numPartials = blocks;
    ra.lossSum = t.lossSum;
    ra.lossMax = t.lossMax;
    return ra;
}

// The largest per-sample loss of a workgroup, kept as the bits of a non-negative float (whose order is that of the
// integers; a NaN compares above everything, so it wins).  A maximum does not depend on the order of its operands: the
// LDS atomic keeps the result reproducible.
__device__ __forceinline__ void noteLossMax(uint32_t* ldsMaxBits, float waveLaneMax)
{
    float m = waveLaneMax;
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        const float o = __shfl_xor(m, d, 64);
        m = (o > m || o != o) ? o : m;
    }
    if ((threadIdx.x & 63u) == 0) atomicMax(ldsMaxBits, __builtin_bit_cast(uint32_t, m));
}

// Gradient multiplier of max(z, zs) with respect to its first operand, per element of a packed
// fp16 pair: 1 where z wins, 0 where zs wins, 0.5 at a tie (diff.meta.slang:2258-2277).  For the
// two activations here (zs = 0, or zs = z*slope with 0 <= slope <= 0.5) the outcome is the sign
// of z.  clamp(z*BIG*BIG + 0.5, 0, 1): two scalings lift even the smallest subnormal far above
// 1 (or below -1), zero stays at 0.5.
__device__ __forceinline__ halfx2 maxGradMultiplier(halfx2 z)
{
    // two instructions: z * 65504, then * 65504 + 0.5 with the result clamped to [0, 1] by the instruction's own modifier
    // (written as max and min the clamp cost two more, a sixth of a training round's vector instructions; a NaN gives 0
    // either way)
    const halfx2 big = {(half_t)65504.f, (half_t)65504.f}, hlf = {(half_t)0.5f, (half_t)0.5f};
    const halfx2 t = z * big;
    halfx2 m;
    asm("v_pk_fma_f16 %0, %1, %2, %3 clamp" : "=v"(m) : "v"(t), "v"(big), "v"(hlf));
    return m;   // {1, 0.5, 0}
}

// four multipliers in {0, 0.5, 1} <-> four e4m3 bytes (all exactly representable)
__device__ __forceinline__ uint32_t packMultipliers(halfx2 m01, halfx2 m23)
{
    typedef short shortx2 __attribute__((ext_vector_type(2)));
    shortx2 r = {0, 0};
    r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r, m01, 1.0f, false);
    r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r, m23, 1.0f, true);
    return __builtin_bit_cast(uint32_t, r);
}

// dz = g * act'(z) on a packed pair, in half: the scalar statement is cvo_ref_mlp_train's.
//   ReLU  : da = g*m
//   leaky : da = g*m, db = g*(1-m), dz = da + db*slope   (each product and the sum rounded to fp16)
// acc += A . B with the accumulator pinned to AGPRs.  The translation unit is built with VGPR
// destinations for MFMAs (every other MFMA result here is consumed by the VALU at once); the
// gradient accumulators are only ever touched by MFMAs until the end of the kernel, and there
// are too many of them for the 256 architectural VGPRs.  The leading s_nop covers a VALU write
// of an operand immediately before (the compiler does not look inside inline asm).
__device__ __forceinline__ void accumulateInAgpr(floatx4& acc, const uint32_t* a, const uint32_t* b)
{
    const u32x4 av = {a[0], a[1], a[2], a[3]}, bv = {b[0], b[1], b[2], b[3]};
    asm("s_nop 1\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(av), "v"(bv));
}

template <bool LEAKY>
__device__ __forceinline__ halfx2 applyActGrad(halfx2 gv, halfx2 m, int act, halfx2 slope2)
{
    if (act == kActNone) return gv;
    const halfx2 da = gv * m;
    if (!LEAKY || act == kActRelu) return da;
    const halfx2 one = {(half_t)1.f, (half_t)1.f};
    const halfx2 db = gv * (one - m);
    return da + db * slope2;
}

// Where value p of a step's summed partial (dW tiles in accumulator order, then db tiles) belongs in the gradient buffers
// ("+=", any layout, fp16 or fp32): the element's address, or null for a value of the tiling's padding.
template <class Net>
__device__ __forceinline__ uint8_t* gradientSlot(const TrainReduceArgs& ra, uint32_t p)
{
    constexpr int L = Net::L;
    constexpr uint32_t nW = Net::totalGradTiles * 256;
    const uint32_t esz = ra.gradCt == kF32 ? 4u : 2u;
    uint8_t* slot = nullptr;
    staticFor<0, L>([&](auto lc) {
        constexpr int l = decltype(lc)::value;
        constexpr int MTO = Net::nOt(l), NI = Net::nIt(l);
        constexpr uint32_t w0 = Net::gradTileBase(l) * 256, w1 = w0 + MTO * NI * 256;
        constexpr uint32_t b0 = nW + Net::dbTileBase(l) * 16, b1 = b0 + MTO * 16;
        const TrainReduceArgs::Layer& ly = ra.layers[l];
        if (p >= w0 && p < w1) {
            const uint32_t q = p - w0, tile = q >> 8, ln = (q >> 2) & 63u, r = q & 3u;
            const uint32_t eo = tile / NI, ei = tile % NI, gq = ln >> 4, qi = ln & 15u;
            const uint32_t o = gq * (4u * MTO) + 4u * eo + r;
            const uint32_t i = (qi >> 2) * (4u * NI) + 4u * ei + (qi & 3u);
            if (ly.wGrad && o < (uint32_t)ly.out && i < (uint32_t)ly.in) slot = ly.wGrad + elemOffset(ly.gradShape, o, i);
        } else if (p >= b0 && p < b1) {
            const uint32_t q = p - b0, eo = q >> 4, qo = q & 15u;
            const uint32_t o = (qo >> 2) * (4u * MTO) + 4u * eo + (qo & 3u);
            if (ly.bGrad && o < (uint32_t)ly.out) slot = ly.bGrad + (size_t)o * esz;
        }
    });
    return slot;
}
__device__ __forceinline__ float loadGradient(const uint8_t* slot, int gradCt)
{
    return gradCt == kF32 ? *(const float*)slot : (float)*(const half_t*)slot;
}
__device__ __forceinline__ void storeGradient(uint8_t* slot, int gradCt, float v)
{
    if (gradCt == kF32) *(float*)slot = v;
    else *(half_t*)slot = (half_t)v;
}
template <class Net>
__device__ __forceinline__ void addToGradients(const TrainReduceArgs& ra, uint32_t p, float s)
{
    uint8_t* slot = gradientSlot<Net>(ra, p);
    if (slot) storeGradient(slot, ra.gradCt, loadGradient(slot, ra.gradCt) + s);
}

// Stages the weights of every layer as A fragments of the forward pass (ldsW), their transposes as A fragments of the dX
// pass (ldsWT, layers 1 and up) and the biases as fp32 (ldsB); BLOCK threads, ends behind a barrier.
template <class Net, int BLOCK>
__device__ __forceinline__ void stageTrainingWeights(const MlpArgs& a, uint32_t* ldsW, uint32_t* ldsWT, float* ldsB)
{
    constexpr int L = Net::L, EPL = 8, RAW = 4;
    // All loads of all layers first, then all stores: one round trip to memory for the whole staging (layer after
    // layer, each matrix and each bias vector waiting for its own loads, it took 14 us of the paired kernel's 131 us).  W^T is not
    // fetched from memory: used as its transpose, a row-major matrix hands a lane eight elements from eight rows, one
    // 2-byte load each that touches 64 cache lines per instruction (7 us per workgroup, more when all of them do it at
    // once); its fragments are gathered from the W fragments once those lie in LDS.
    constexpr int kStageIters = (Net::MTMAX * Net::KTMAX * 64 + BLOCK - 1) / BLOCK;
    FragmentStage<2, EPL, kStageIters, BLOCK> stW[L];
    float stB[L];
    staticFor<0, L>([&](auto lc) {
        constexpr int l = decltype(lc)::value;
        constexpr int MT = Net::mt(l), KT = Net::kt(l), ROWS = 4 * MT;
        static_assert(MT * 16 <= BLOCK, "one bias value per thread and layer");
        const MlpLayerArgs& ly = a.layers[l];
        // (k-slots per lane group: those of the kernel's tiling; a hidden layer narrower than the widest one is padded to it)
        stW[l].load(ly.w, ly.shape, false, MT, KT, l == 0 ? optGS((uint32_t)ly.in) : 4u * (uint32_t)Net::mt(l > 0 ? l - 1 : 0), (uint32_t)ly.out, (uint32_t)ly.in);
        const int e = threadIdx.x, t = e >> 4, gg = (e >> 2) & 3, r = e & 3;
        const int row = gg * ROWS + 4 * t + r;
        stB[l] = (e < MT * 16 && ly.bias && row < ly.out) ? (float)((const half_t*)ly.bias)[row] : 0.f;
    });
    staticFor<0, L>([&](auto lc) {
        constexpr int l = decltype(lc)::value;
        constexpr int MT = Net::mt(l), KT = Net::kt(l);
        stW[l].store(ldsW + Net::fragBase(l) * 64 * RAW, MT, KT);
        if ((int)threadIdx.x < MT * 16) ldsB[Net::biasBase(l) * 16 + threadIdx.x] = stB[l];
    });
    __syncthreads();
    // Lane 16*g + i of W^T fragment (t, kt) of layer l holds W[g*gsOut + kt*8 + s][(i/4)*4*MTI + 4*t + i%4], s < 8 (output
    // unit on the k axis, input unit as the row); element W[o][c] lies in W fragment ((o % (4*MT)) / 4, (c % gsIn) / 8) at
    // lane 16*(c / gsIn) + 4*(o / (4*MT)) + o%4, slot c % 8 (cv_layout.h).  Rows and columns past the matrix are zero there.
    staticFor<1, L>([&](auto lc) {
        constexpr int l = decltype(lc)::value;
        constexpr int MT = Net::mt(l), KT = Net::kt(l), MTI = Net::mt(l - 1), KTO = Net::ktOut(l);
        constexpr int gsOut = 4 * MT, gsIn = 4 * MTI, chunks = MTI * KTO * 64;
        const uint16_t* src = (const uint16_t*)(ldsW + Net::fragBase(l) * 64 * RAW);
        for (int c = threadIdx.x; c < chunks; c += BLOCK) {
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

}

// LOADS selects how the network input is fetched.  kLoadDwords (every lane's slice is whole, 4-byte
// aligned dwords) and kLoadXY (float2 samples of the example's encoding) are straight-line code: every
// lane loads from an address that is always valid and masks afterwards, so the requests of the next
// round stay in flight during the whole current round.  kLoadAny covers everything else with
// predicated loads, which the round has to wait for.
enum : int { kLoadDwords = 0, kLoadAny = 1, kLoadXY = 2 };

// HACT / LACT fix the activation of the hidden layers / the last layer at compile time (the round
// then is straight-line code the scheduler can interleave); -1 reads them from the arguments and
// keeps the leaky-ReLU arithmetic.
template <class Net, int HACT, int LACT, int LOADS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void mlpTrainKernel(const TrainArgs ta)
{
    typedef F16Mma Mma;
    constexpr int L = Net::L;
    constexpr int FD = 4, RAW = 4, EPL = 8;
    constexpr bool LEAKY = HACT < 0 || LACT < 0;
    auto actOf = [&](int l) -> int {
        const int fixed = (l + 1 < L) ? HACT : LACT;
        return fixed >= 0 ? fixed : ta.mlp.layers[l].act;
    };
    constexpr int IN_DW = RAW * Net::KT0;
    const MlpArgs& a = ta.mlp;

    __shared__ __attribute__((aligned(16))) uint32_t ldsW[Net::totalFrags * 64 * RAW];
    __shared__ __attribute__((aligned(16))) uint32_t ldsWT[(Net::totalTFrags > 0 ? Net::totalTFrags : 1) * 64 * RAW];
    __shared__ __attribute__((aligned(16))) float ldsB[Net::totalBiasTiles * 16];   // biases as fp32
    __shared__ __attribute__((aligned(16))) float ldsRed[4 * 256];
    __shared__ uint32_t ldsLossMax;               // the workgroup's largest per-sample loss, as bits
    if (threadIdx.x == 0) ldsLossMax = 0u;
    // per-wave parking space for the F-orientation copies of every layer's input
    __shared__ __attribute__((aligned(16))) uint32_t ldsXF[4 * Net::totalXTiles * 256];

    // ---- stage W (A operand of the forward pass), W^T (A operand of dX) and biases ----------
    stageTrainingWeights<Net, 256>(a, ldsW, ldsWT, ldsB);

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, n = lane & 15;

    // 0/1 selection fragments: column q of half h picks k-slot (group q/4, slot 4h + q%4)
    uint32_t Isel[2][FD];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int d = 0; d < FD; ++d) {
            const int s0 = 4 * h + (lane & 3);            // the slot this lane may own
            const bool mine = g == (n >> 2);
            const uint32_t lo = (mine && s0 == 2 * d) ? 0x3C00u : 0u;
            const uint32_t hi = (mine && s0 == 2 * d + 1) ? 0x3C00u : 0u;
            Isel[h][d] = lo | (hi << 16);
        }
    const halfx2 ones2 = {(half_t)1.f, (half_t)1.f};

    // gradient accumulators of this wave
    floatx4 accW[Net::totalGradTiles];
    float accB[Net::totalDbTiles];
#pragma unroll
    for (int i = 0; i < Net::totalGradTiles; ++i) accW[i] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < Net::totalDbTiles; ++i) accB[i] = 0.f;
    float lossAcc = 0.f, lossMaxAcc = 0.f;

    // ---- per-lane constants ----------------------------------------------------------------
    const int in0 = a.layers[0].in;
    const uint32_t gs0 = optGS((uint32_t)in0);
    const int colBase = (int)(g * gs0);
    const int validBytes = min((int)gs0, max(in0 - colBase, 0)) * 2;
    const int outDim = a.layers[L - 1].out;
    constexpr int OROWS = 4 * Net::MTL;

    constexpr uint32_t TILE = 32;                 // two 16-sample tiles = one k-tile of dW
    const uint32_t numTiles = (a.batch + TILE - 1) / TILE;
    const uint32_t tileStride = gridDim.x * 4;
    const uint8_t* inLane = a.in + (size_t)colBase * 2;
    const uint32_t lastSample = a.batch - 1;

    // Requests the input registers of one round.  Loads only, no arithmetic on the loaded values: the
    // round that consumes them runs a whole round later (float2 samples of the example's encoding
    // stay raw until then, and slices shorter than IN_DW dwords are masked then).
    auto loadTile = [&](uint32_t (&raw)[2][IN_DW], uint32_t t) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t s = min(t * TILE + 16 * j + n, lastSample);
            const uint8_t* row = a.in + (size_t)s * a.inStride;
            const uint8_t* p = row + (size_t)colBase * 2;
            if constexpr (LOADS == kLoadXY) {
                // a float2 sample (lane group 0 owns all four encoded inputs; the others discard it)
#pragma unroll
                for (int i = 0; i < IN_DW; ++i) raw[j][i] = i < 2 ? ((const uint32_t*)row)[i] : 0u;
            } else if constexpr (LOADS == kLoadDwords) {
                // dwords past the lane's slice are fetched from the start of the row (always valid) and masked later
#pragma unroll
                for (int i = 0; i < IN_DW; ++i) raw[j][i] = *(const uint32_t*)(4 * i < validBytes ? p + 4 * i : row);
            } else if (a.inEncoding == kEncodeXYSquares) {
#pragma unroll
                for (int i = 0; i < IN_DW; ++i) raw[j][i] = (i < 2 && g == 0) ? ((const uint32_t*)row)[i] : 0u;
            } else {
#pragma unroll
                for (int i = 0; i < IN_DW; ++i) {
                    uint32_t v = 0;
                    if (4 * i < validBytes) v = *(const uint16_t*)(p + 4 * i);
                    if (4 * i + 2 < validBytes) v |= (uint32_t)*(const uint16_t*)(p + 4 * i + 2) << 16;
                    raw[j][i] = v;
                }
            }
        }
    };

    // S fragment pair (tiles j = 0,1) -> F fragment of feature tile e = 2*kt + h
    auto toF = [&](const uint32_t* s0, const uint32_t* s1, int h, uint32_t* frag) {
        typedef float floatx2 __attribute__((ext_vector_type(2)));
        const floatx4 z = {0.f, 0.f, 0.f, 0.f};
        const floatx4 t0 = Mma::mma(s0, Isel[h], z), t1 = Mma::mma(s1, Isel[h], z);
        frag[0] = __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{t0[0], t0[1]}, halfx2));
        frag[1] = __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{t0[2], t0[3]}, halfx2));
        frag[2] = __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{t1[0], t1[1]}, halfx2));
        frag[3] = __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{t1[2], t1[3]}, halfx2));
    };

    auto round = [&](const uint32_t (&raw)[2][IN_DW], uint32_t t0) {
        uint32_t buf[2][IN_DW];                     // the network input as layer 0 sees it
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int d = 0; d < IN_DW; ++d) {
                if constexpr (LOADS == kLoadDwords) buf[j][d] = 4 * d < validBytes ? raw[j][d] : 0u;
                else if constexpr (LOADS == kLoadXY) buf[j][d] = 0u;
                else buf[j][d] = raw[j][d];
            }
            if ((LOADS == kLoadXY || a.inEncoding == kEncodeXYSquares) && g == 0)
                encodeXYSquares(__builtin_bit_cast(float, raw[j][0]), __builtin_bit_cast(float, raw[j][1]), buf[j][0], buf[j][1]);
        }
        uint32_t actS[2][Net::KTMAX][FD];           // S fragments of the current layer's input
        uint32_t mst[L][2][Net::MTMAX];             // max() gradient multipliers, four e4m3 bytes per out tile
        halfx2 yS[2][Net::MTL][2];                  // network output (carrier), tile j, out tile t
        uint32_t* myXF = ldsXF + wave * (Net::totalXTiles * 256);
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int kt = 0; kt < Net::KT0; ++kt)
#pragma unroll
                for (int d = 0; d < FD; ++d) actS[j][kt][d] = buf[j][kt * RAW + d];

        // ---------------- forward ----------------
        // The gradient multipliers of layer l are only needed in the backward pass; they are
        // computed from the saved pre-activations while layer l+1's MFMAs execute (left alone,
        // the scheduler sinks all of that VALU work into one serial block after the forward pass).
        halfx2 zprev[2][Net::MTMAX][2];
        uint32_t wbuf[Net::MTMAX][Net::KTMAX > Net::KOMAX ? Net::KTMAX : Net::KOMAX][4];   // A fragments of the layer at hand
        uint32_t xbuf[Net::ITMAX][FD];                                                      // F fragments of its input
        floatx4 bbuf[Net::MTMAX];                                                           // its biases (accumulator seeds)
        auto loadW = [&](auto lc) {           // forward weights of layer l
            constexpr int l = decltype(lc)::value;
#pragma unroll
            for (int t = 0; t < Net::mt(l); ++t)
#pragma unroll
                for (int kt = 0; kt < Net::kt(l); ++kt) {
                    const u32x4 v = *(const u32x4*)&ldsW[((Net::fragBase(l) + t * Net::kt(l) + kt) * 64 + lane) * RAW];
                    wbuf[t][kt][0] = v.x; wbuf[t][kt][1] = v.y; wbuf[t][kt][2] = v.z; wbuf[t][kt][3] = v.w;
                }
#pragma unroll
            for (int t = 0; t < Net::mt(l); ++t) bbuf[t] = *(const floatx4*)&ldsB[(Net::biasBase(l) + t) * 16 + 4 * g];
        };
        auto loadWT = [&](auto lc) {          // transposed weights of layer l (l >= 1)
            constexpr int l = decltype(lc)::value;
            constexpr int MTI = Net::mt(l - 1), KTO = Net::ktOut(l);
#pragma unroll
            for (int t = 0; t < MTI; ++t)
#pragma unroll
                for (int kt = 0; kt < KTO; ++kt) {
                    const u32x4 v = *(const u32x4*)&ldsWT[((Net::tFragBase(l) + t * KTO + kt) * 64 + lane) * RAW];
                    wbuf[t][kt][0] = v.x; wbuf[t][kt][1] = v.y; wbuf[t][kt][2] = v.z; wbuf[t][kt][3] = v.w;
                }
        };
        auto loadXF = [&](auto lc) {          // parked F fragments of layer l's input
            constexpr int l = decltype(lc)::value;
#pragma unroll
            for (int e = 0; e < Net::nIt(l); ++e) {
                const u32x4 v = *(const u32x4*)(myXF + (Net::xTileBase(l) + e) * 256 + lane * 4);
                xbuf[e][0] = v.x; xbuf[e][1] = v.y; xbuf[e][2] = v.z; xbuf[e][3] = v.w;
            }
        };
        loadW(std::integral_constant<int, 0>{});
        auto multipliersOf = [&](int l, int MT) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int t = 0; t < Net::MTMAX; ++t)
                    if (t < MT) mst[l][j][t] = packMultipliers(maxGradMultiplier(zprev[j][t][0]), maxGradMultiplier(zprev[j][t][1]));
        };
        staticFor<0, L>([&](auto lc) {
            constexpr int l = decltype(lc)::value;
            constexpr int MT = Net::mt(l), KT = Net::kt(l);
            const int actv = actOf(l);
            const half_t sl = (half_t)a.layers[l].slope;
            const halfx2 slope2 = {sl, sl};
            const halfx2 zero2 = {(half_t)0, (half_t)0};
            // this layer's input in F orientation, parked in LDS until the backward pass
            {
                // all selection MFMAs first, then the conversions: no stall on each pair's result
                floatx4 tt[Net::nIt(l)][2];
                const floatx4 zf = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int e = 0; e < Net::nIt(l); ++e) {
                    tt[e][0] = Mma::mma(actS[0][e / 2], Isel[e & 1], zf);
                    tt[e][1] = Mma::mma(actS[1][e / 2], Isel[e & 1], zf);
                }
#pragma unroll
                for (int e = 0; e < Net::nIt(l); ++e) {
                    typedef float floatx2 __attribute__((ext_vector_type(2)));
                    u32x4 f;
                    f.x = __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{tt[e][0][0], tt[e][0][1]}, halfx2));
                    f.y = __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{tt[e][0][2], tt[e][0][3]}, halfx2));
                    f.z = __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{tt[e][1][0], tt[e][1][1]}, halfx2));
                    f.w = __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{tt[e][1][2], tt[e][1][3]}, halfx2));
                    *(u32x4*)(myXF + (Net::xTileBase(l) + e) * 256 + lane * 4) = f;
                }
            }

            floatx4 acc[2][MT];
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                acc[0][t] = bbuf[t]; acc[1][t] = bbuf[t];
            }
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    acc[0][t] = Mma::mma(wbuf[t][kt], actS[0][kt], acc[0][t]);
                    acc[1][t] = Mma::mma(wbuf[t][kt], actS[1][kt], acc[1][t]);
                }
            // the MFMAs above have read wbuf: request the next layer's fragments now, so that the
            // LDS latency is covered by this layer's VALU work (one wave per SIMD: nobody else hides it)
            if constexpr (l + 1 < L) loadW(std::integral_constant<int, l + 1>{});
            if constexpr (l > 0) {
                if (actOf(l - 1) != kActNone) multipliersOf(l - 1, Net::mt(l - 1));
            }
            // carrier: round to fp16, remember the gradient multiplier of max(), apply the activation
            halfx2 car[2][MT][2];
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    typedef float floatx2 __attribute__((ext_vector_type(2)));
                    halfx2 z01 = __builtin_convertvector(floatx2{acc[j][t][0], acc[j][t][1]}, halfx2);
                    halfx2 z23 = __builtin_convertvector(floatx2{acc[j][t][2], acc[j][t][3]}, halfx2);
                    if (actv != kActNone) {
                        zprev[j][t][0] = z01; zprev[j][t][1] = z23;
                        const halfx2 s01 = (!LEAKY || actv == kActRelu) ? zero2 : z01 * slope2;
                        const halfx2 s23 = (!LEAKY || actv == kActRelu) ? zero2 : z23 * slope2;
                        z01 = __builtin_elementwise_max(z01, s01);
                        z23 = __builtin_elementwise_max(z23, s23);
                    }
                    car[j][t][0] = z01; car[j][t][1] = z23;
                }
            if constexpr (l + 1 < L) {
                constexpr int KTN = Net::kt(l + 1);
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int kt = 0; kt < KTN; ++kt) {
                        actS[j][kt][0] = __builtin_bit_cast(uint32_t, car[j][2 * kt][0]);
                        actS[j][kt][1] = __builtin_bit_cast(uint32_t, car[j][2 * kt][1]);
                        actS[j][kt][2] = (2 * kt + 1 < MT) ? __builtin_bit_cast(uint32_t, car[j][2 * kt + 1 < MT ? 2 * kt + 1 : 0][0]) : 0u;
                        actS[j][kt][3] = (2 * kt + 1 < MT) ? __builtin_bit_cast(uint32_t, car[j][2 * kt + 1 < MT ? 2 * kt + 1 : 0][1]) : 0u;
                    }
            } else {
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int t = 0; t < MT; ++t) { yS[j][t][0] = car[j][t][0]; yS[j][t][1] = car[j][t][1]; }
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        if (actOf(L - 1) != kActNone) multipliersOf(L - 1, Net::mt(L - 1));

        // decode four multipliers
        auto multipliers = [&](uint32_t raw, halfx2& m01, halfx2& m23) {
            m01 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(raw, 1.0f, false);
            m23 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(raw, 1.0f, true);
        };
        // pack the carrier tiles dz[t] (t < MT) of one sample tile into S fragments
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
        loadXF(std::integral_constant<int, L - 1>{});
        if constexpr (L > 1) loadWT(std::integral_constant<int, L - 1>{});
        uint32_t bS[2][Net::KOMAX][FD];             // S fragments of dY of the current layer
        {
            const int actl = actOf(L - 1);
            const half_t sll = (half_t)a.layers[L - 1].slope;
            const halfx2 slope2 = {sll, sll};
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const uint32_t sample = t0 * TILE + 16 * j + n;
                const bool live = sample < a.batch;
                float tgtAll = 0.f;
                half_t gt[4] = {(half_t)0, (half_t)0, (half_t)0, (half_t)0};
                const bool exampleLoss = !ta.targets && a.inEncoding == kEncodeXYSquares;
                if (exampleLoss) {
                    // the example's loss: groundtruth(x, y); rows 0..3 live in lane group 0, which holds (x, y)
                    const halfx2 xy = __builtin_bit_cast(halfx2, buf[j][0]);
                    exampleGroundTruth(xy.x, xy.y, gt);
                } else if (!ta.targets) {
                    // target = sin(sum of the sample's inputs): every lane group holds a quarter of them
                    float part = 0.f;
#pragma unroll
                    for (int d = 0; d < IN_DW; ++d) {
                        const halfx2 v = __builtin_bit_cast(halfx2, buf[j][d]);
                        part += (float)v.x; part += (float)v.y;
                    }
                    tgtAll = (float)(half_t)sinf(sumOverGroups(part));
                }
                halfx2 dz[Net::MTL][2];
                float sampleLoss = 0.f;         // this lane's rows of the sample's loss
#pragma unroll
                for (int t = 0; t < Net::MTL; ++t) {
                    const half_t yv[4] = {yS[j][t][0].x, yS[j][t][0].y, yS[j][t][1].x, yS[j][t][1].y};
                    half_t gv[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int row = g * OROWS + 4 * t + r;
                        gv[r] = (half_t)0;
                        if (live && row < outDim) {
                            const float tv = ta.targets
                                ? (float)*(const half_t*)(ta.targets + (size_t)sample * ta.targetStride + 2 * row)
                                : (exampleLoss ? (float)gt[row & 3] : tgtAll);
                            const half_t diff = (half_t)((float)yv[r] - tv);
                            lossAcc += (float)diff * (float)diff;
                            sampleLoss += (float)diff * (float)diff;
                            gv[r] = (half_t)(2.0f * (float)diff * ta.lossScale);
                        }
                    }
                    halfx2 m01 = {(half_t)1.f, (half_t)1.f}, m23 = m01;
                    if (actl != kActNone) multipliers(mst[L - 1][j][t], m01, m23);
                    dz[t][0] = applyActGrad<LEAKY>(halfx2{gv[0], gv[1]}, m01, actl, slope2);
                    dz[t][1] = applyActGrad<LEAKY>(halfx2{gv[2], gv[3]}, m23, actl, slope2);
                }
                packS(dz, Net::MTL, Net::ktOut(L - 1), bS[j]);
                if (ta.wantLossMax) {       // the sample's rows lie in the four lane groups
                    const float whole = sumOverGroups(sampleLoss);
                    lossMaxAcc = (whole > lossMaxAcc || whole != whole) ? whole : lossMaxAcc;
                }
            }
        }

        // ---------------- backward ----------------
        staticFor<0, L>([&](auto lc) {
            constexpr int l = L - 1 - decltype(lc)::value;
            constexpr int MT = Net::mt(l), NI = Net::nIt(l);
            // dY in F orientation; bias gradient; weight gradient
#pragma unroll
            for (int eo = 0; eo < MT; ++eo) {
                uint32_t dzF[FD];
                toF(bS[0][eo / 2], bS[1][eo / 2], eo & 1, dzF);
                float s = accB[Net::dbTileBase(l) + eo];
#pragma unroll
                for (int d = 0; d < FD; ++d) s = __builtin_amdgcn_fdot2(__builtin_bit_cast(halfx2, dzF[d]), ones2, s, false);
                accB[Net::dbTileBase(l) + eo] = s;
#pragma unroll
                for (int ei = 0; ei < NI; ++ei) {
                    floatx4& w = accW[Net::gradTileBase(l) + eo * NI + ei];
                    accumulateInAgpr(w, dzF, xbuf[ei]);
                }
            }
            if constexpr (l > 0) {
                // dX = W^T dY, then through the previous layer's activation
                constexpr int MTI = Net::mt(l - 1), KTO = Net::ktOut(l);
                const int actp = actOf(l - 1);
                const half_t slp = (half_t)a.layers[l - 1].slope;
                const halfx2 slope2 = {slp, slp};
                floatx4 gacc[2][MTI];
#pragma unroll
                for (int t = 0; t < MTI; ++t) { gacc[0][t] = floatx4{0.f, 0.f, 0.f, 0.f}; gacc[1][t] = gacc[0][t]; }
#pragma unroll
                for (int kt = 0; kt < KTO; ++kt)
#pragma unroll
                    for (int t = 0; t < MTI; ++t) {
                        gacc[0][t] = Mma::mma(wbuf[t][kt], bS[0][kt], gacc[0][t]);
                        gacc[1][t] = Mma::mma(wbuf[t][kt], bS[1][kt], gacc[1][t]);
                    }
                // next layer down: its parked input and (if it has one) its transposed weights
                loadXF(std::integral_constant<int, l - 1>{});
                if constexpr (l > 1) loadWT(std::integral_constant<int, l - 1>{});
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    halfx2 dz[MTI][2];
#pragma unroll
                    for (int t = 0; t < MTI; ++t) {
                        typedef float floatx2 __attribute__((ext_vector_type(2)));
                        const halfx2 g01 = __builtin_convertvector(floatx2{gacc[j][t][0], gacc[j][t][1]}, halfx2);
                        const halfx2 g23 = __builtin_convertvector(floatx2{gacc[j][t][2], gacc[j][t][3]}, halfx2);
                        halfx2 m01 = {(half_t)1.f, (half_t)1.f}, m23 = m01;
                        if (actp != kActNone) multipliers(mst[l - 1][j][t], m01, m23);
                        dz[t][0] = applyActGrad<LEAKY>(g01, m01, actp, slope2);
                        dz[t][1] = applyActGrad<LEAKY>(g23, m23, actp, slope2);
                    }
                    packS(dz, MTI, Net::ktOut(l - 1), bS[j]);
                }
            }
        });
    };

    // ---- main loop: every wave strides over rounds of 32 samples; the next round's inputs are
    //      requested before the current round and copied over after it ------------------------
    {
        uint32_t tile = blockIdx.x * 4 + wave;
        if (tile < numTiles) {
            uint32_t cur[2][IN_DW], nxt[2][IN_DW];
            loadTile(cur, tile);
            for (; tile < numTiles; tile += tileStride) {
                const uint32_t t1 = tile + tileStride;
                loadTile(nxt, t1 < numTiles ? t1 : tile);
                // the requests stay above the round (a load may not move across this point) ...
                asm volatile("" ::: "memory");
                round(cur, tile);
                // ... and their results are first touched below it
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int d = 0; d < IN_DW; ++d) { pinHere(nxt[j][d]); cur[j][d] = nxt[j][d]; }
            }
        }
    }

    // the last MFMAs into the AGPR accumulators must have retired before they are read
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // ---- workgroup partial: sum the four waves in a fixed order, one tile at a time ----------
    // The only workgroup of a launch (ta.finishInKernel) does with its sums what mlpTrainReduceKernel would do with this one
    // partial: they go from its registers to the gradients.  The gradient elements they are added to are requested ahead,
    // eight tiles at a time, so that a group of tiles costs one round trip to memory, and the loss is summed first: a NaN
    // there makes every sum of the step NaN (see mlpTrainReduceKernel).
    float* part = ta.partials + (size_t)blockIdx.x * Net::partialFloats;
    constexpr uint32_t nValues = Net::totalGradTiles * 256 + Net::totalDbTiles * 16;
    const bool finish = ta.finishInKernel != 0;
    const TrainReduceArgs& ra = ta.finish;
    __shared__ float ldsLossSum;
    ldsRed[threadIdx.x] = lossAcc;
    if (ta.wantLossMax) noteLossMax(&ldsLossMax, lossMaxAcc);
    __syncthreads();
    // the loss: one wave sums the 256 values in a fixed order, four neighbours per lane, then lanes 32 ... 1 places apart
    if (wave == 0) {
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) s += ldsRed[lane * 4 + i];
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) s += __shfl_xor(s, d, 64);
        if (lane == 0) {
            ldsLossSum = s;
            if (!finish) {
                part[nValues] = s;
                part[nValues + 1] = __builtin_bit_cast(float, ldsLossMax);
            }
        }
    }
    // bias gradients' destinations (threads 0 .. 15 hold one element of every tile)
    float oldB[Net::totalDbTiles];
#pragma unroll
    for (int i = 0; i < Net::totalDbTiles; ++i) {
        oldB[i] = 0.f;
        if (finish && threadIdx.x < 16) {
            const uint8_t* slot = gradientSlot<Net>(ra, Net::totalGradTiles * 256 + i * 16 + threadIdx.x);
            if (slot) oldB[i] = loadGradient(slot, ra.gradCt);
        }
    }
    __syncthreads();
    const bool voidStep = finish && ldsLossSum != ldsLossSum;
    constexpr int kAhead = 8;
#pragma unroll
    for (int i0 = 0; i0 < Net::totalGradTiles; i0 += kAhead) {
        float old[kAhead];
#pragma unroll
        for (int k = 0; k < kAhead; ++k) {
            old[k] = 0.f;
            if (finish && i0 + k < Net::totalGradTiles) {
                const uint8_t* slot = gradientSlot<Net>(ra, (i0 + k) * 256 + threadIdx.x);
                if (slot) old[k] = loadGradient(slot, ra.gradCt);
            }
        }
#pragma unroll
        for (int k = 0; k < kAhead; ++k) {
            const int i = i0 + k;
            if (i >= Net::totalGradTiles) break;
            *(floatx4*)&ldsRed[wave * 256 + lane * 4] = accW[i];
            __syncthreads();
            float s = ((ldsRed[threadIdx.x] + ldsRed[256 + threadIdx.x]) + ldsRed[512 + threadIdx.x]) + ldsRed[768 + threadIdx.x];
            if (!finish) {
                part[i * 256 + threadIdx.x] = s;
            } else {
                s = voidStep ? __builtin_nanf("") : 0.f + s;         // (the sum of one partial, as sumPartials forms it)
                uint8_t* slot = gradientSlot<Net>(ra, i * 256 + threadIdx.x);
                if (slot) storeGradient(slot, ra.gradCt, old[k] + s);
            }
            __syncthreads();
        }
    }
    // bias gradients: lane (g,q) holds the sum over its samples; sum the 4 lane groups and 4 waves
#pragma unroll
    for (int i = 0; i < Net::totalDbTiles; ++i) {
        ldsRed[wave * 64 + lane] = accB[i];
        __syncthreads();
        if (threadIdx.x < 16) {
            float s = 0.f;
            for (int w = 0; w < 4; ++w)
                for (int gg = 0; gg < 4; ++gg) s += ldsRed[w * 64 + gg * 16 + threadIdx.x];
            if (!finish) {
                part[Net::totalGradTiles * 256 + i * 16 + threadIdx.x] = s;
            } else {
                s = voidStep ? __builtin_nanf("") : 0.f + s;
                uint8_t* slot = gradientSlot<Net>(ra, Net::totalGradTiles * 256 + i * 16 + threadIdx.x);
                if (slot) storeGradient(slot, ra.gradCt, oldB[i] + s);
            }
        }
        __syncthreads();
    }
    if (finish && threadIdx.x == 0) {
        if (ra.lossSum) *ra.lossSum = voidStep ? __builtin_nanf("") : 0.f + ldsLossSum;
        if (ra.lossMax) *ra.lossMax = voidStep ? __builtin_nanf("") : __builtin_bit_cast(float, ldsLossMax);
    }
}

// Sums the workgroup partials in a fixed order and adds them to the gradient buffers.
template <class Net>
__global__ __launch_bounds__(64 * kReduceWaves) void mlpTrainReduceKernel(const TrainReduceArgs ra)
{
    // a workgroup owns 64 consecutive values of the partial (see sumPartials)
    constexpr int L = Net::L;
    __shared__ float red[kReduceWaves * 64];
    const uint32_t p = blockIdx.x * 64u + (threadIdx.x & 63u);
    constexpr uint32_t nW = Net::totalGradTiles * 256, nB = Net::totalDbTiles * 16;
    const bool inRange = p < nW + nB + 1;
    // A workgroup whose loss partial is NaN declares its whole partial void: a wave of the paired kernel that gave up
    // waiting for its partner has worked on stale tiles and says so there (so does a NaN that came in with the samples).
    // Then every sum of the step is NaN, whether or not the caller reads the loss.
    __shared__ uint32_t maxBits;
    const bool ownsLoss = blockIdx.x == (nW + nB) / 64u;      // the workgroup whose values include the loss
    if (threadIdx.x == 0) maxBits = 0u;
    __syncthreads();
    // (the loss partials are requested here and looked at behind the sums: one round trip to memory for both)
    bool voidStep = false;
    float lp0 = 0.f;
    if (threadIdx.x < ra.numPartials) lp0 = ra.partials[(size_t)threadIdx.x * Net::partialFloats + nW + nB];
    for (uint32_t b = threadIdx.x + 64u * kReduceWaves; b < ra.numPartials; b += 64u * kReduceWaves) {
        const float lp = ra.partials[(size_t)b * Net::partialFloats + nW + nB];
        voidStep = voidStep || lp != lp;
    }
    if (ra.lossMax && ownsLoss)
        for (uint32_t b = threadIdx.x; b < ra.numPartials; b += 64u * kReduceWaves)
            atomicMax(&maxBits, __builtin_bit_cast(uint32_t, ra.partials[(size_t)b * Net::partialFloats + nW + nB + 1]));
    // (so is the gradient element the sum is added to: wave 0, which stores the sums, asks for it before they are formed)
    uint8_t* slot = nullptr;
    float old = 0.f;
    if (threadIdx.x < 64u && inRange && p < nW + nB) {
        slot = gradientSlot<Net>(ra, p);
        if (slot) old = loadGradient(slot, ra.gradCt);
    }
    float s;
    const bool mine = sumPartials(ra.partials + p, Net::partialFloats, ra.numPartials, inRange, red, s);
    voidStep = __syncthreads_or(voidStep || lp0 != lp0) != 0;
    if (ra.lossMax && ownsLoss && threadIdx.x == 0)
        *ra.lossMax = voidStep ? __builtin_nanf("") : __builtin_bit_cast(float, maxBits);
    if (!mine || !inRange) return;
    if (voidStep) s = __builtin_nanf("");
    if (p == nW + nB) {
        if (ra.lossSum) *ra.lossSum = s;
        return;
    }
    if (slot) storeGradient(slot, ra.gradCt, old + s);
}

} // namespace
} // namespace cv
