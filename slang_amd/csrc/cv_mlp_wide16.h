// cv_mlp_wide16.h -- fused forward MLP on 32-sample tiles (v_mfma_f32_32x32x16_f16) for fp16
// networks: the chain FeedForwardLayer.eval builds (examples/mlp-training-coopvec/fflayer.slang:60-66,
// network.slang:41-47) for hidden layers of 32 or 64 units.
//
// An fp16 network has a short carrier chain between layers (fp32 -> fp16, ReLU: one v_cvt_pk_f16_f32
// and one v_pk_max_f16 per pair of hidden values), so what can bind it is the matrix pipeline itself.
// v_mfma_f32_32x32x16_f16 does twice the multiply-adds of v_mfma_f32_16x16x32_f16 for a lower issue
// cost (7.3 against 8.7 cycles of the vector-ALU port), all weights stay in registers as A operands
// (nothing is re-read from LDS per tile), and a tile's input is loaded straight in operand order.
// Geometry, row order of the hidden layers and the order in which the 8-element chunks of k meet the
// accumulator are those of cv_mlp_wide.h: every layer computes bit for bit what the single-layer
// operator computes.
//
// Biases.  The single-layer operator starts its fp32 accumulators from float(bias).  Here the first
// matrix instruction of a layer takes its C operand from sixteen registers that were filled from LDS
// (one 64-byte line per layer, 32-row tile and lane half, read as a broadcast) while the other tile of
// the pair was in the matrix pipeline; a network without biases uses the constant 0 instead.
#pragma once
#include "cv_mlp_impl.h"
#include "cv_wide_tiles.h"

namespace cv {
namespace {

// One fragment = 64 lanes x 8 halves (16 bytes): lane (rho, h) holds W[rowOf(T, rho)][colOf(s, h, 0) + e], e < chunkElems
// (4 or 8), zeros behind them.
template <class RowFn, class ColFn>
__device__ __forceinline__ void stageWideFragments16(uint32_t* dst, const MlpLayerArgs& ly, int tiles, int steps, int chunkElems, RowFn rowOf, ColFn colOf)
{
    const MatrixShape& shape = ly.shape;
    const bool linear = shape.layout == kRowMajor || shape.layout == kColumnMajor;
    const size_t line = shape.stride ? shape.stride : (size_t)(shape.layout == kRowMajor ? shape.cols : shape.rows) * 2u;
    const size_t sr = shape.layout == kRowMajor ? line : (size_t)2, sc = shape.layout == kRowMajor ? (size_t)2 : line;
    for (int c = threadIdx.x; c < tiles * steps * 64; c += blockDim.x) {
        const int lane = c & 63, f = c >> 6, s = f % steps, T = f / steps, rho = lane & 31, h = lane >> 5;
        const int row = rowOf(T, rho), col0 = colOf(s, h, 0);
        int nvalid = row < ly.out ? ly.in - col0 : 0;
        nvalid = nvalid < 0 ? 0 : (nvalid > chunkElems ? chunkElems : nvalid);
        u32x4 out = {0u, 0u, 0u, 0u};
        const uint8_t* p0 = ly.w;
        bool whole = false;
        size_t step = 0;
        if (linear) {
            if (nvalid > 0) p0 = ly.w + (size_t)row * sr + (size_t)col0 * sc;
            step = sc;
            whole = sc == 2 && nvalid == 8;
        } else if (nvalid > 0) {
            // An Optimal layout: eight neighbouring columns that start at a multiple of eight are one lane-chunk of the
            // 16-sample fragments when the two ends of the run say so; anything else goes through the index map.
            const size_t off0 = elemOffset(shape, (uint32_t)row, (uint32_t)col0);
            p0 = ly.w + off0;
            whole = nvalid == 8 && elemOffset(shape, (uint32_t)row, (uint32_t)(col0 + 7)) == off0 + 14;
        }
        if (whole && ((uintptr_t)p0 & 15) == 0) {
            out = *(const u32x4*)p0;
        } else if (whole && ((uintptr_t)p0 & 3) == 0) {
            out = u32x4{((const uint32_t*)p0)[0], ((const uint32_t*)p0)[1], ((const uint32_t*)p0)[2], ((const uint32_t*)p0)[3]};
        } else if (linear) {
            uint32_t v[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = *(const uint16_t*)(e < nvalid ? p0 + (size_t)e * step : ly.w);
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = e < nvalid ? v[e] : 0u;
            out = u32x4{v[0] | (v[1] << 16), v[2] | (v[3] << 16), v[4] | (v[5] << 16), v[6] | (v[7] << 16)};
        } else {
            uint32_t v[4] = {0u, 0u, 0u, 0u};
#pragma nounroll
            for (int e = 0; e < nvalid; ++e) {
                const uint32_t x = *(const uint16_t*)(ly.w + elemOffset(shape, (uint32_t)row, (uint32_t)(col0 + e)));
                v[e >> 1] |= x << (16 * (e & 1));
            }
            out = u32x4{v[0], v[1], v[2], v[3]};
        }
        *(u32x4*)&dst[4 * c] = out;
    }
}

// Order of one scheduling region for the instruction scheduler: NM matrix instructions; the NV vector-ALU instructions
// spread evenly behind all but the last two of them; the NL LDS reads in two halves, each as soon as the vector-ALU
// instructions that free its destination registers are through, so that the second half has two matrix instructions of
// time left before the next phase asks for it.
template <int NM, int NV, int NL>
__device__ __forceinline__ void interleavePhase()
{
    constexpr int NS = NM > 3 ? NM - 2 : NM;      // matrix instructions that have vector-ALU work behind them
    staticFor<0, NM>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                       // one MFMA
        if constexpr (i < NS) {
            constexpr int nv = NV * (i + 1) / NS - NV * i / NS;
            if constexpr (nv > 0) __builtin_amdgcn_sched_group_barrier(0x002, nv, 0);            // VALU
            if constexpr (NL > 0 && i == (NS - 1) / 2) __builtin_amdgcn_sched_group_barrier(0x100, NL / 2, 0);    // DS reads
            if constexpr (NL > 0 && i == NS - 1) __builtin_amdgcn_sched_group_barrier(0x100, NL - NL / 2, 0);
        }
    });
}

// H: hidden width / 32 (1 or 2); NH: hidden layers (1..4); K0: inputs per sample (8, 16 or 32 halves in contiguous
// rows).  Up to 32 outputs.  Hidden layers are ReLU; the last layer's activation (none or ReLU)
// is read from the arguments.  Work distribution as in mlpWideKernel: one workgroup per compute unit, whose waves
// draw pairs of tiles from a counter in LDS.
// Where a pair of tiles gets its first-layer operands from.  This one reads fp16 vectors in contiguous rows:
//   K0 == 8 : 8 bytes per lane: inputs 4h .. 4h+3 of sample n, the lane's operand of the one k-step as they are;
//   K0 == 16: 16 bytes: inputs 8h .. 8h+7;  K0 == 32: 32 bytes: inputs 16h .. 16h+15.
// Rows beyond the end of the batch read the last row instead (their results are not stored).
template <int K0>
struct Wide16MemoryFront {
    static constexpr int NDW = K0 / 4;     // dwords per lane and tile
    struct Input { uint32_t v[2][NDW]; };
    const uint8_t* in;
    __device__ __forceinline__ Input load(uint32_t p, int n, int h, uint32_t lastSample) const
    {
        Input x;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            uint32_t s = (2u * p + (uint32_t)j) * 32u + (uint32_t)n;
            s = s < lastSample ? s : lastSample;
            const uint8_t* row = in + (uint64_t)s * (2u * K0) + (uint32_t)h * (uint32_t)K0;
            if constexpr (K0 == 8) {
                const u32x2 r = *(const u32x2*)row;
                x.v[j][0] = r.x; x.v[j][1] = r.y;
            } else {
#pragma unroll
                for (int i = 0; i < NDW / 4; ++i) {
                    const u32x4 r = *(const u32x4*)(row + 16 * i);
                    x.v[j][4 * i] = r.x; x.v[j][4 * i + 1] = r.y; x.v[j][4 * i + 2] = r.z; x.v[j][4 * i + 3] = r.w;
                }
            }
        }
        return x;
    }
    // v_permlane32_swap exchanges the upper half of its first operand with the lower half of its second
    template <int NS>
    __device__ __forceinline__ void operands(const Input& x, uint32_t (&B)[2][NS][4], int, int) const
    {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            if constexpr (K0 == 8) {
                B[j][0][0] = x.v[j][0]; B[j][0][1] = x.v[j][1]; B[j][0][2] = 0u; B[j][0][3] = 0u;
            } else if constexpr (K0 == 16) {
                // lane (n,0) holds inputs 0..7, lane (n,1) inputs 8..15; k-step s wants 8s + 4h .. 8s + 4h + 3
#pragma unroll
                for (int d = 0; d < 2; ++d) {
                    const u32x2 r = __builtin_amdgcn_permlane32_swap(x.v[j][d], x.v[j][2 + d], false, false);
                    B[j][0][d] = r.x; B[j][1][d] = r.y;
                    B[j][0][2 + d] = 0u; B[j][1][2 + d] = 0u;
                }
            } else {
                // lane (n,0) holds inputs 0..15, lane (n,1) inputs 16..31; k-step s wants 16s + 8h .. 16s + 8h + 7
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    const u32x2 r = __builtin_amdgcn_permlane32_swap(x.v[j][d], x.v[j][4 + d], false, false);
                    B[j][0][d] = r.x; B[j][1][d] = r.y;
                }
            }
        }
    }
};

// LEAKY: every hidden layer is leaky ReLU, max(z, z * slope) on the rounded halfs with the slope as a half (what the
// single-layer operator evaluates, fflayer.slang:60-66): one more packed multiply per pair of values; else every hidden
// layer is ReLU.
template <int H, int NH, int K0, int WAVES, bool HAS_BIAS, bool LEAKY = false, class Front = void>
__device__ __forceinline__ void mlpWide16Body(const MlpArgs& a, const Front& front)
{
    constexpr int KS = 2 * H;                          // k-steps of a hidden vector
    // k-steps of the input vector, and the inputs per lane and k-step.  The result of a matrix instruction depends on
    // which products share a lane's eight k-slots, so the inputs are dealt out as the single-layer operator deals them
    // (cv_layout.h: a lane group owns 4*ceil(K/16) inputs): four per lane for 8 and 16 inputs (the other four k-slots
    // zero), eight per lane for 32.  Same chunks, same bits.
    constexpr int S0 = K0 == 8 ? 1 : 2;
    constexpr int CE0 = K0 == 32 ? 8 : 4;
    constexpr int F0 = H * S0, FH = H * KS, FL = KS;   // fragments of layer 0, of a hidden->hidden layer, of the last layer
    constexpr int TOTAL = F0 + (NH - 1) * FH + FL;
    __shared__ __attribute__((aligned(16))) uint32_t ldsW[TOTAL * 64 * 4];
    // float(bias) in accumulator order: [layer * H + T][h][r] = bias of row 8*(r/4) + 4*h + r%4 of tile T
    constexpr int NSEED = HAS_BIAS ? H * NH + 1 : 1;
    __shared__ __attribute__((aligned(16))) float ldsSeed[NSEED * 32];
    __shared__ uint32_t nextClaim;
    if (threadIdx.x == 0) nextClaim = 0;
    if constexpr (HAS_BIAS) {
        for (int c = threadIdx.x; c < NSEED * 32; c += blockDim.x) {
            const int f = c >> 5, hh = (c >> 4) & 1, r = c & 15, rho = 8 * (r / 4) + 4 * hh + r % 4;
            const int l = f < H * NH ? f / H : NH, T = f < H * NH ? f % H : 0;
            const int unit = l < NH ? wideUnitOfRow(H, T, rho) : rho;
            float v = 0.f;
            if (a.layers[l].bias && unit < a.layers[l].out) v = (float)((const half_t*)a.layers[l].bias)[unit];
            ldsSeed[c] = v;
        }
    }

    // ---- weights into LDS in operand order ---------------------------------------------------
    stageWideFragments16(ldsW, a.layers[0], H, S0, CE0,
                         [](int T, int rho) { return wideUnitOfRow(H, T, rho); },
                         [](int s, int h, int e) { return 2 * CE0 * s + CE0 * h + e; });
#pragma unroll
    for (int l = 1; l < NH; ++l)
        stageWideFragments16(ldsW + (F0 + (l - 1) * FH) * 256, a.layers[l], H, KS, 8,
                             [](int T, int rho) { return wideUnitOfRow(H, T, rho); },
                             [](int s, int h, int e) { return wideUnitOfSlot(H, s, h, e); });
    stageWideFragments16(ldsW + (F0 + (NH - 1) * FH) * 256, a.layers[NH], 1, KS, 8,
                         [](int, int rho) { return rho; },
                         [](int s, int h, int e) { return wideUnitOfSlot(H, s, h, e); });
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const int n = lane & 31, h = lane >> 5;

    uint32_t W0[H][S0][4], WH[NH > 1 ? NH - 1 : 1][H][KS][4], WL[KS][4];
    auto loadFrag = [&](int frag, uint32_t* dst) {
        const u32x4 v = *(const u32x4*)&ldsW[(frag * 64 + lane) * 4];
        dst[0] = v.x; dst[1] = v.y; dst[2] = v.z; dst[3] = v.w;
    };
#pragma unroll
    for (int T = 0; T < H; ++T)
#pragma unroll
        for (int s = 0; s < S0; ++s) loadFrag(T * S0 + s, W0[T][s]);
#pragma unroll
    for (int l = 1; l < NH; ++l)
#pragma unroll
        for (int T = 0; T < H; ++T)
#pragma unroll
            for (int s = 0; s < KS; ++s) loadFrag(F0 + (l - 1) * FH + T * KS + s, WH[l - 1][T][s]);
#pragma unroll
    for (int s = 0; s < KS; ++s) loadFrag(F0 + (NH - 1) * FH + s, WL[s]);

    const uint32_t numTiles = (a.batch + 31u) / 32u;
    const uint32_t numPairs = (numTiles + 1u) / 2u;
    const uint32_t numGroups = (uint32_t)__builtin_amdgcn_readfirstlane((int)gridDim.x);
    // the c-th claim of this workgroup is pair c * numGroups + blockIdx.x (tiles 2*pair, 2*pair + 1)
    auto claim = [&]() -> uint32_t {
        uint32_t c = 0;
        if (lane == 0) c = __hip_atomic_fetch_add(&nextClaim, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        return (uint32_t)__builtin_amdgcn_readfirstlane((int)c) * numGroups + blockIdx.x;
    };
    uint32_t pair = claim();
    if (pair >= numPairs) return;
    const uint32_t lastSample = a.batch - 1u;
    const bool lastRelu = a.layers[NH].act == kActRelu;
    const bool lastLeaky = LEAKY && a.layers[NH].act == kActLeakyRelu;
    const half_t lastSlope = (half_t)a.layers[NH].slope;
    const halfx2 lastSlope2 = {lastSlope, lastSlope};
    const int outDim = a.layers[NH].out;
    const bool storeQuads = outDim % 4 == 0 && a.outAlign >= 8u;
    const halfx2 zero2 = {(half_t)0.f, (half_t)0.f};

    uint32_t B[2][KS > S0 ? KS : S0][4];
    floatx16 acc[2][H];
    const floatx16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // (the lane's offset passes through an empty asm statement once per round of the loop: the lines are the same for
    // every tile, and the optimiser would otherwise keep all of them in registers, which the weights need)
    // (one offset per tile of the pair, or the two tiles would share one read and hold its result in extra registers)
    uint32_t seedOff[2] = {(uint32_t)h * 16u, (uint32_t)h * 16u};
    auto seed = [&](int l, int T, int j) -> floatx16 {       // float(bias) of layer l, tile T, or zeros
        if constexpr (HAS_BIAS) {
            const floatx4* p = (const floatx4*)&ldsSeed[(l * H + T) * 32 + seedOff[j]];
            const floatx4 s0 = p[0], s1 = p[1], s2 = p[2], s3 = p[3];
            return floatx16{s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3], s2[0], s2[1], s2[2], s2[3], s3[0], s3[1], s3[2], s3[3]};
        } else {
            return zero16;
        }
    };
    // the accumulators of tile j start from the biases of layer l
    auto seedLayer = [&](int l, int j) {
#pragma unroll
        for (int T = 0; T < (l < NH ? H : 1); ++T) acc[j][T] = seed(l, T, j);
    };
    // (k-step outer, 32-row tile inner: no two dependent matrix instructions follow one another)
    auto firstLayer = [&](int j) {
#pragma unroll
        for (int s = 0; s < S0; ++s)
#pragma unroll
            for (int T = 0; T < H; ++T) acc[j][T] = mfma32(W0[T][s], B[j][s], acc[j][T]);
    };
    // accumulators -> fp16 -> activation of layer l = operands of the next layer, in place
    halfx2 slope2[NH];
#pragma unroll
    for (int l = 0; l < NH; ++l) { const half_t sl = (half_t)a.layers[l].slope; slope2[l] = halfx2{sl, sl}; }
    auto carrier = [&](int j, int l) {
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const int T = s / 2, r0 = 8 * (s % 2);
            typedef float floatx2 __attribute__((ext_vector_type(2)));
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const halfx2 z = __builtin_convertvector(floatx2{acc[j][T][r0 + 2 * i], acc[j][T][r0 + 2 * i + 1]}, halfx2);
                const halfx2 p = __builtin_elementwise_max(z, LEAKY ? z * slope2[l] : zero2);
                B[j][s][i] = __builtin_bit_cast(uint32_t, p);
            }
        }
    };
    auto hiddenLayer = [&](int l, int j) {
#pragma unroll
        for (int s = 0; s < KS; ++s)
#pragma unroll
            for (int T = 0; T < H; ++T) acc[j][T] = mfma32(WH[l - 1][T][s], B[j][s], acc[j][T]);
    };
    auto lastLayer = [&](int j) {      // result in acc[j][0]
#pragma unroll
        for (int s = 0; s < KS; ++s) acc[j][0] = mfma32(WL[s], B[j][s], acc[j][0]);
    };
    auto storeTile = [&](int j, uint32_t t) {
        const floatx16 o = acc[j][0];
        const uint32_t sample = t * 32u + (uint32_t)n;
        if (sample >= a.batch) return;
        uint8_t* orow = a.out + (uint64_t)sample * a.outStride;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            typedef float floatx2 __attribute__((ext_vector_type(2)));
            const int row0 = 8 * q + 4 * h;
            if (row0 >= outDim) continue;
            halfx2 p0 = __builtin_convertvector(floatx2{o[4 * q], o[4 * q + 1]}, halfx2);
            halfx2 p1 = __builtin_convertvector(floatx2{o[4 * q + 2], o[4 * q + 3]}, halfx2);
            if (lastRelu) {
                p0 = __builtin_elementwise_max(p0, zero2);
                p1 = __builtin_elementwise_max(p1, zero2);
            }
            if constexpr (LEAKY) {      // (the example's layers all have the activation, the last one too)
                if (lastLeaky) {
                    p0 = __builtin_elementwise_max(p0, p0 * lastSlope2);
                    p1 = __builtin_elementwise_max(p1, p1 * lastSlope2);
                }
            }
            if (storeQuads) {
                const u32x2 v = {__builtin_bit_cast(uint32_t, p0), __builtin_bit_cast(uint32_t, p1)};
                storeStream8(orow + 2 * row0, v);      // (written once, read by nobody here)
            } else {
                half_t* o16 = (half_t*)(orow + 2 * row0);
                __builtin_nontemporal_store(p0.x, o16);
                if (row0 + 1 < outDim) __builtin_nontemporal_store(p0.y, o16 + 1);
                if (row0 + 2 < outDim) __builtin_nontemporal_store(p1.x, o16 + 2);
                if (row0 + 3 < outDim) __builtin_nontemporal_store(p1.y, o16 + 3);
            }
        }
    };

    // Two tiles travel through the layers half a layer apart.  A phase = the matrix instructions of one layer for one
    // tile, and between them the vector-ALU work of the other tile: its accumulators of the layer before become operands
    // (two instructions per pair of values), then the biases of its next layer are requested from LDS into the
    // accumulators just freed, a whole phase before the matrix instruction that takes them as C operand.  The order
    // within a phase is given to the scheduler explicitly (left alone it requests the biases right in front of their
    // use and the wave sits out the LDS latency once per layer and tile); nothing moves across a phase boundary.
    constexpr int NV = (LEAKY ? 24 : 16) * H;      // vector-ALU instructions of one tile's carrier
    constexpr int NL = HAS_BIAS ? 4 * H : 0;
    auto endPhase = []() { __builtin_amdgcn_sched_barrier(0); };
    typename Front::Input in = front.load(pair, n, h, lastSample);
    seedLayer(0, 0);
    seedLayer(0, 1);
    while (true) {
        const uint32_t next = claim();
        if constexpr (HAS_BIAS) asm volatile("" : "+v"(seedOff[0]), "+v"(seedOff[1]));
        front.operands(in, B, n, h);
        in = front.load(next < numPairs ? next : numPairs - 1u, n, h, lastSample);      // beyond the end: loaded again, never used
        firstLayer(0);
        endPhase();
        firstLayer(1); carrier(0, 0); seedLayer(1, 0);
        interleavePhase<H * S0, NV, NL>(); endPhase();
#pragma unroll
        for (int l = 1; l < NH; ++l) {
            hiddenLayer(l, 0); carrier(1, l - 1); seedLayer(l, 1);
            interleavePhase<H * KS, NV, NL>(); endPhase();
            hiddenLayer(l, 1); carrier(0, l); seedLayer(l + 1, 0);
            interleavePhase<H * KS, NV, NL>(); endPhase();
        }
        lastLayer(0); carrier(1, NH - 1); seedLayer(NH, 1);
        interleavePhase<KS, NV, HAS_BIAS ? 4 : 0>(); endPhase();
        lastLayer(1); storeTile(0, 2u * pair); seedLayer(0, 0);
        endPhase();
        storeTile(1, 2u * pair + 1u); seedLayer(0, 1);
        if (next >= numPairs) return;
        pair = next;
    }
}

template <int H, int NH, int K0, int WAVES, bool HAS_BIAS, bool LEAKY = false>
__global__ __launch_bounds__(64 * WAVES) void mlpWide16Kernel(const MlpArgs a)
{
    mlpWide16Body<H, NH, K0, WAVES, HAS_BIAS, LEAKY>(a, Wide16MemoryFront<K0>{a.in});
}

// waves per workgroup (one workgroup per compute unit): as many as the weights leave registers for
// (16 waves: 128 registers each, 12: 168, 8: 256); the build fails if an instantiation spills
template <int H, int NH, int K0>
constexpr int wide16Waves()
{
    constexpr int KS = 2 * H, S0 = K0 == 8 ? 1 : 2;
    constexpr int WREGS = 4 * (H * S0 + (NH - 1) * H * KS + KS);
    return (WREGS + 48 * H + 32 <= 128) ? 16 : ((WREGS + 48 * H + 32 <= 168) ? 12 : 8);
}

// Shapes: fp16 vectors of 8, 16 or 32 elements in contiguous rows at a 16-byte aligned address, ReLU hidden layers of
// exactly 32 or 64 units (one to four of them), at most 32 outputs (checked by the dispatcher in cv_mlp_f16.hip).
template <int H, int NH, int K0, bool HAS_BIAS, bool LEAKY = false>
hipError_t launchMlpWide16Shape(hipStream_t stream, const MlpArgs& a, int numCUs)
{
    constexpr int WAVES = wide16Waves<H, NH, K0>();
    const uint32_t numPairs = ((a.batch + 31u) / 32u + 1u) / 2u;
    const uint32_t blocks = numPairs < (uint32_t)numCUs ? numPairs : (uint32_t)numCUs;
    noteKernel(false, "mlpWide16Kernel<f16,32x32x16,inputs=%d,hidden=%dx%d%s,%s,waves=%d>", K0, NH, 32 * H, LEAKY ? ",leaky" : "",
               HAS_BIAS ? "bias" : "nobias", WAVES);
    hipLaunchKernelGGL((mlpWide16Kernel<H, NH, K0, WAVES, HAS_BIAS, LEAKY>), dim3(blocks), dim3(64 * WAVES), 0, stream, a);
    return hipGetLastError();
}

// all shapes of one input width (one translation unit each, compiled in parallel)
template <int K0>
hipError_t launchMlpWide16K(hipStream_t stream, const MlpArgs& a, int numCUs, int H, int NH)
{
    bool hasBias = false;
    for (int l = 0; l < a.numLayers; ++l) hasBias = hasBias || a.layers[l].bias != nullptr;
    // (the dispatcher lets in hidden layers that are all ReLU or all leaky ReLU; the leaky instantiation is the one with
    // biases, which an absent bias vector enters as zeros)
    const bool leaky = a.layers[0].act == kActLeakyRelu;
#define CV_W16(h_, nh_) if (H == h_ && NH == nh_) \
        return leaky ? launchMlpWide16Shape<h_, nh_, K0, true, true>(stream, a, numCUs) \
             : hasBias ? launchMlpWide16Shape<h_, nh_, K0, true>(stream, a, numCUs) : launchMlpWide16Shape<h_, nh_, K0, false>(stream, a, numCUs);
    CV_W16(1, 1) CV_W16(1, 2) CV_W16(1, 3) CV_W16(1, 4) CV_W16(2, 1) CV_W16(2, 2) CV_W16(2, 3) CV_W16(2, 4)
#undef CV_W16
    return hipErrorInvalidValue;
}

} // namespace
} // namespace cv
