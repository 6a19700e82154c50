// cv_mlp_wide.h -- fused forward MLP on 32-sample tiles (v_mfma_f32_32x32x16_f16) for e4m3
// networks whose input rows are 32 contiguous bytes and whose hidden layers are 32 or 64 wide.
//
// Why a second tiling.  Between two layers of an e4m3 network every hidden value passes
// fp32 -> fp16 -> ReLU -> e4m3 -> fp16, one vector-ALU instruction per pair of values and step, and
// that per-element work, not memory or the matrix pipeline, is what bounds the kernel: measured on
// gfx950 a SIMD issues one ordinary VALU instruction per ~4.3 cycles, a conversion *to* fp8 per
// ~8.3 cycles, and an MFMA with 128-bit operands also occupies the VALU port: ~8.7 cycles for
// v_mfma_f32_16x16x32_f16 but only ~7.3 cycles for v_mfma_f32_32x32x16_f16, which does twice the
// multiply-adds.  On 32-sample tiles the matrix instructions of a network therefore cost less than
// half the issue time (16 instead of 28 per 32 samples for 32-64-64-8), and the input can be
// loaded straight in operand order (no staging through LDS):
//
//   lane l = 32*h + n belongs to sample n of the tile and to half h;
//   D = W . X^T per 32-row tile T: register r of lane (n,h) is row 8*(r/4) + 4*h + r%4;
//   as B operand of k-step s, lane (n,h) supplies k-slots 8*h .. 8*h+7 of that step.
//
// The rows of a hidden layer are ordered so that registers 8*(s%2) .. 8*(s%2)+7 of tile s/2 are,
// after conversion to packed fp16, exactly the B operand of k-step s of the next layer (no
// cross-lane movement), and so that the 8-element chunks of k meet the accumulator in the same
// order as in the 16-sample kernels: chunk (kt, g) there is chunk (s, h) = (2*kt + g/2, g%2) here.
#pragma once
#include "cv_mlp_impl.h"
#include "cv_wide_tiles.h"

namespace cv {
namespace {

// One fragment = 64 lanes x 8 e4m3 bytes: lane (rho, h) holds W[rowOf(T, rho)][colOf(s, h, e)], e < 8, where the
// eight columns of a lane are neighbours: colOf(s, h, e) = colOf(s, h, 0) + e.  In a linear layout they lie at a fixed
// step from one another (next to each other in RowMajor: one 8-byte load), and all loads of a chunk are in flight
// together; an InferencingOptimal source has them next to each other as well; only the rest goes element by element
// through the layout's index map.  (The element-by-element
// form, eight dependent round trips per chunk, took 13 us at the head of a 260 us kernel.)
template <class RowFn, class ColFn>
__device__ __forceinline__ void stageWideFragments(uint32_t* dst, const MlpLayerArgs& ly, int tiles, int steps, RowFn rowOf, ColFn colOf)
{
    const MatrixShape& shape = ly.shape;
    const bool linear = shape.layout == kRowMajor || shape.layout == kColumnMajor;
    const size_t line = shape.stride ? shape.stride : (size_t)(shape.layout == kRowMajor ? shape.cols : shape.rows);
    const size_t sr = shape.layout == kRowMajor ? line : (size_t)1, sc = shape.layout == kRowMajor ? (size_t)1 : line;
    for (int c = threadIdx.x; c < tiles * steps * 64; c += blockDim.x) {
        const int lane = c & 63, f = c >> 6, s = f % steps, T = f / steps, rho = lane & 31, h = lane >> 5;
        const int row = rowOf(T, rho), col0 = colOf(s, h, 0);
        int nvalid = row < ly.out ? ly.in - col0 : 0;
        nvalid = nvalid < 0 ? 0 : (nvalid > 8 ? 8 : nvalid);
        uint32_t lo = 0, hi = 0;
        if (linear) {
            const uint8_t* p0 = nvalid > 0 ? ly.w + (size_t)row * sr + (size_t)col0 * sc : ly.w;
            if (sc == 1 && nvalid == 8 && ((uintptr_t)p0 & 7) == 0) {
                const u32x2 x = *(const u32x2*)p0;
                lo = x.x; hi = x.y;
            } else {
                uint32_t v[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = *(e < nvalid ? p0 + (size_t)e * sc : ly.w);
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = e < nvalid ? v[e] : 0u;
                lo = v[0] | (v[1] << 8) | (v[2] << 16) | (v[3] << 24);
                hi = v[4] | (v[5] << 8) | (v[6] << 16) | (v[7] << 24);
            }
        } else {
            // An Optimal layout: in the InferencingOptimal order eight neighbouring columns that start at a multiple of
            // eight are eight neighbouring bytes (one k-chunk of one lane of the 16-sample fragments), which the two
            // ends of the run tell; anything else goes through the index map element by element.
            const size_t off0 = nvalid > 0 ? elemOffset(shape, (uint32_t)row, (uint32_t)col0) : 0;
            const size_t off7 = nvalid == 8 ? elemOffset(shape, (uint32_t)row, (uint32_t)(col0 + 7)) : 0;
            if (nvalid == 8 && off7 == off0 + 7 && (((uintptr_t)ly.w + off0) & 7) == 0) {
                const u32x2 x = *(const u32x2*)(ly.w + off0);
                lo = x.x; hi = x.y;
            } else {
#pragma nounroll
                for (int e = 0; e < nvalid; ++e) {
                    const uint32_t v = ly.w[elemOffset(shape, (uint32_t)row, (uint32_t)(col0 + e))];
                    if (e < 4) lo |= v << (8 * e); else hi |= v << (8 * (e - 4));
                }
            }
        }
        dst[2 * c] = lo; dst[2 * c + 1] = hi;
    }
}

// H: hidden width / 32 (1 or 2); NH: hidden layers; OQ: groups of 8 output rows (1, 2 or 4).
// Hidden layers are ReLU; the last layer's activation (none or ReLU) is read from the arguments.
//
// Work distribution.  A SIMD favours its oldest wave: with a fixed share of tiles per wave the oldest
// wave of every SIMD is done in less than half of the kernel's time and the SIMD limps through the
// rest with fewer and fewer waves (measured: wave 0 alive for 140 us of 311 us).  So one workgroup
// fills a whole compute unit (WAVES waves) and its waves draw pairs of tiles from a counter in LDS;
// all of them stay busy until the compute unit's share is used up.
template <int H, int NH, int OQ, int WAVES, bool IN_HALF, bool HAS_BIAS>
__global__ __launch_bounds__(64 * WAVES) void mlpWideKernel(const MlpArgs a)
{
    constexpr uint32_t ROWB = IN_HALF ? 64u : 32u;       // bytes of an input row in memory
    constexpr uint32_t TILEB = 32u * ROWB;               // bytes of a tile's input
    constexpr int LOADS = IN_HALF ? 2 : 1;               // 16-byte loads per lane and tile
    constexpr int KS = 2 * H;                       // k-steps of a hidden vector
    constexpr int F0 = H * 2, FH = H * KS, FL = KS; // fragments of layer 0, of a hidden->hidden layer, of the last layer
    constexpr int TOTAL = F0 + (NH - 1) * FH + FL;
    __shared__ __attribute__((aligned(16))) uint32_t ldsW[TOTAL * 64 * 2];
    // Biases enter as one more k-step in front of the others: A = the layer's biases in k-slot 0 (zeros
    // elsewhere), B = 1.0 in k-slot 0, C = 0, which leaves exactly float(bias) in the accumulators, the
    // value the 16-sample kernels start from.  One fragment per layer and 32-row tile, read from LDS at use.
    constexpr int NBIAS = HAS_BIAS ? H * NH + 1 : 1;
    __shared__ __attribute__((aligned(16))) uint32_t ldsBias[NBIAS * 64 * 4];
    __shared__ uint32_t nextClaim;
    if (threadIdx.x == 0) nextClaim = 0;
    if constexpr (HAS_BIAS) {
        for (int c = threadIdx.x; c < NBIAS * 64; c += blockDim.x) {
            const int lane = c & 63, f = c >> 6, rho = lane & 31;
            const int l = f < H * NH ? f / H : NH, T = f < H * NH ? f % H : 0;
            const int unit = l < NH ? wideUnitOfRow(H, T, rho) : rho;
            uint32_t v = 0;
            if (lane < 32 && a.layers[l].bias && unit < a.layers[l].out) v = ((const uint16_t*)a.layers[l].bias)[unit];
            ldsBias[4 * c] = v; ldsBias[4 * c + 1] = 0; ldsBias[4 * c + 2] = 0; ldsBias[4 * c + 3] = 0;
        }
    }

    // ---- weights into LDS in operand order ---------------------------------------------------
    stageWideFragments(ldsW, a.layers[0], H, 2,
                       [](int T, int rho) { return wideUnitOfRow(H, T, rho); },
                       [](int s, int h, int e) { return 16 * s + 8 * h + e; });
#pragma unroll
    for (int l = 1; l < NH; ++l)
        stageWideFragments(ldsW + (F0 + (l - 1) * FH) * 128, a.layers[l], H, KS,
                           [](int T, int rho) { return wideUnitOfRow(H, T, rho); },
                           [](int s, int h, int e) { return wideUnitOfSlot(H, s, h, e); });
    stageWideFragments(ldsW + (F0 + (NH - 1) * FH) * 128, a.layers[NH], 1, KS,
                       [](int, int rho) { return rho; },
                       [](int s, int h, int e) { return wideUnitOfSlot(H, s, h, e); });
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const int n = lane & 31, h = lane >> 5;

    uint32_t W0[H][2][4], WH[NH > 1 ? NH - 1 : 1][H][KS][4], WL[KS][4];
    auto loadFrag = [&](int frag, uint32_t* dst) { Fp8AsF16Mma::decode(&ldsW[(frag * 64 + lane) * 2], dst); };
#pragma unroll
    for (int T = 0; T < H; ++T)
#pragma unroll
        for (int s = 0; s < 2; ++s) loadFrag(T * 2 + s, W0[T][s]);
#pragma unroll
    for (int l = 1; l < NH; ++l)
#pragma unroll
        for (int T = 0; T < H; ++T)
#pragma unroll
            for (int s = 0; s < KS; ++s) loadFrag(F0 + (l - 1) * FH + T * KS + s, WH[l - 1][T][s]);
#pragma unroll
    for (int s = 0; s < KS; ++s) loadFrag(F0 + (NH - 1) * FH + s, WL[s]);

    const uint32_t numTiles = (a.batch + 31u) / 32u, fullTiles = a.batch / 32u;
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
    const uint32_t inLane = (uint32_t)n * ROWB + (uint32_t)h * (ROWB / 2u);
    const uint32_t outLane = (uint32_t)n * (uint32_t)a.outStride + (uint32_t)h * 8u;
    const uint64_t totalBytes = (uint64_t)a.batch * ROWB;
    const bool lastRelu = a.layers[NH].act == kActRelu;
    const int outDim = a.layers[NH].out;
    const halfx2 zero2 = {(half_t)0.f, (half_t)0.f};

    // a tile's input, half a row per lane (16 bytes of e4m3, or 32 bytes of fp16 in two instructions), every
    // instruction fully coalesced.  Only the last tile can be partial; its lanes beyond the end of the
    // input read the last bytes instead.
    const uint32_t lastTile = numTiles - 1u;
    uint32_t tailLane = inLane;
    {
        const uint64_t room = totalBytes - ROWB / 2u - (uint64_t)lastTile * TILEB;    // a whole row is there: never negative
        if ((uint64_t)inLane > room) tailLane = (uint32_t)room;
    }
    // The input loads are issued and awaited by hand.  With the loads under its own control the compiler
    // waits for *every* outstanding access at the top of the loop (also for the store it has just
    // issued), which exposes the whole memory latency once per round.  Here a slot's four registers
    // are written by a load that the compiler does not know about.  The statement that consumes a slot
    // first waits until at most one younger access is outstanding (the other slot's load is always
    // younger and loads return in order, so the slot's own load has landed whatever else is pending),
    // takes the rows out, and then refills the same registers for the next pair of tiles.  Between two
    // such statements a slot is only passed along untouched: the kernel must compile without register
    // spills, and nothing may copy a slot while its load is on the way (both hold for every
    // instantiation below; the bit-exact tests at full batch would show a stale register).
    struct Slot { u32x4 v[LOADS]; };
    auto issue = [&](Slot& slot, uint32_t t) {
        t = t < lastTile ? t : lastTile;
        const uint8_t* base = a.in + (uint64_t)t * TILEB;
        const uint32_t voff = t < fullTiles ? inLane : tailLane;
        asm volatile("global_load_dwordx4 %0, %1, %2 nt" : "=v"(slot.v[0]) : "v"(voff), "s"(base) : "memory");
        if constexpr (IN_HALF)
            asm volatile("global_load_dwordx4 %0, %1, %2 offset:16 nt" : "=v"(slot.v[1]) : "v"(voff), "s"(base) : "memory");
    };
    // Half 0 of k-step 0 needs features 0..7 and of k-step 1 features 16..23, half 1 needs 8..15 and
    // 24..31, while lane (n,0) has loaded features 0..15 and lane (n,1) features 16..31:
    // v_permlane32_swap exchanges the upper half of its first operand with the lower half of its second.
    // RAW: per k-step the lane's eight features as they lie in memory (2 dwords of e4m3, 4 of fp16).
    constexpr int RAW = IN_HALF ? 4 : 2;
    auto consume = [&](Slot& slot, uint32_t t, uint32_t (&raw)[2][RAW], uint32_t (&Bj)[KS][4]) {
        if constexpr (IN_HALF) {
            asm volatile("s_waitcnt vmcnt(%2)" : "+v"(slot.v[0]), "+v"(slot.v[1]) : "n"(LOADS) : "memory");
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const u32x2 r = __builtin_amdgcn_permlane32_swap(slot.v[0][d], slot.v[1][d], false, false);
                raw[0][d] = r.x; raw[1][d] = r.y;
            }
        } else {
            asm volatile("s_waitcnt vmcnt(%1)" : "+v"(slot.v[0]) : "n"(LOADS) : "memory");
            const u32x2 r0 = __builtin_amdgcn_permlane32_swap(slot.v[0].x, slot.v[0].z, false, false);
            const u32x2 r1 = __builtin_amdgcn_permlane32_swap(slot.v[0].y, slot.v[0].w, false, false);
            raw[0][0] = r0.x; raw[0][1] = r1.x; raw[1][0] = r0.y; raw[1][1] = r1.y;
        }
        // the slot's registers are free from here on: the refill must not start before the rows are taken out
        // (e4m3 rows are decoded on the spot, which reads the slot's registers in place and saves the copies;
        // fp16 rows must wait for the saturating mode)
        if constexpr (!IN_HALF) {
            Fp8AsF16Mma::decode(raw[0], Bj[0]);
            Fp8AsF16Mma::decode(raw[1], Bj[1]);
#pragma unroll
            for (int i = 0; i < 4; ++i) { pinHere(Bj[0][i]); pinHere(Bj[1][i]); }
        } else {
#pragma unroll
            for (int d = 0; d < RAW; ++d) { pinHere(raw[0][d]); pinHere(raw[1][d]); }
        }
        issue(slot, t);
    };

    // Two tiles travel through the layers half a layer apart: while the vector ALU converts one tile's
    // accumulators into the next layer's operands, the matrix pipeline works on the other tile.
    const floatx16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    uint32_t B[2][KS][4];
    floatx16 acc[2][H];
    const uint32_t onesB[4] = {h == 0 ? 0x3C00u : 0u, 0u, 0u, 0u};       // 1.0 in k-slot 0
    auto seed = [&](int l, int T) -> floatx16 {       // float(bias) of layer l, tile T, or zeros
        if constexpr (HAS_BIAS) {
            const u32x4 bf = *(const u32x4*)&ldsBias[((l * H + T) * 64 + lane) * 4];
            const uint32_t biasA[4] = {bf.x, bf.y, bf.z, bf.w};
            return mfma32(biasA, onesB, zero16);
        } else {
            return zero16;
        }
    };

    auto firstLayer = [&](int j) {
#pragma unroll
        for (int T = 0; T < H; ++T) acc[j][T] = mfma32(W0[T][0], B[j][0], seed(0, T));
#pragma unroll
        for (int T = 0; T < H; ++T) acc[j][T] = mfma32(W0[T][1], B[j][1], acc[j][T]);
    };
    // accumulators -> fp16 -> ReLU -> e4m3 -> fp16 operands of the next layer
    auto carrier = [&](int j) {
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const int T = s / 2, r0 = 8 * (s % 2);
            typedef float floatx2 __attribute__((ext_vector_type(2)));
            typedef short shortx2 __attribute__((ext_vector_type(2)));
            halfx2 p[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                p[i] = __builtin_elementwise_max(__builtin_convertvector(floatx2{acc[j][T][r0 + 2 * i], acc[j][T][r0 + 2 * i + 1]}, halfx2), zero2);
            uint32_t q[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                shortx2 r = __builtin_bit_cast(shortx2, p[2 * i]);
                r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r, p[2 * i], 1.0f, false);
                r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r, p[2 * i + 1], 1.0f, true);
                q[i] = __builtin_bit_cast(uint32_t, r);
            }
            Fp8AsF16Mma::decode(q, B[j][s]);
        }
    };
    auto hiddenLayer = [&](int l, int j) {
#pragma unroll
        for (int T = 0; T < H; ++T) acc[j][T] = mfma32(WH[l - 1][T][0], B[j][0], seed(l, T));
#pragma unroll
        for (int s = 1; s < KS; ++s)
#pragma unroll
            for (int T = 0; T < H; ++T) acc[j][T] = mfma32(WH[l - 1][T][s], B[j][s], acc[j][T]);
    };
    auto lastLayer = [&](int j) {      // result in acc[j][0]
        acc[j][0] = mfma32(WL[0], B[j][0], seed(NH, 0));
#pragma unroll
        for (int s = 1; s < KS; ++s) acc[j][0] = mfma32(WL[s], B[j][s], acc[j][0]);
    };
    auto storeTile = [&](int j, uint32_t t) {
        const floatx16 o = acc[j][0];
        const uint32_t sample = t * 32u + (uint32_t)n;
        uint8_t* obase = a.out + (uint64_t)t * 32u * a.outStride;
#pragma unroll
        for (int q = 0; q < OQ; ++q) {
            typedef float floatx2 __attribute__((ext_vector_type(2)));
            if (sample < a.batch && 8 * q + 4 * h < outDim) {
                halfx2 p0 = __builtin_convertvector(floatx2{o[4 * q], o[4 * q + 1]}, halfx2);
                halfx2 p1 = __builtin_convertvector(floatx2{o[4 * q + 2], o[4 * q + 3]}, halfx2);
                if (lastRelu) {
                    p0 = __builtin_elementwise_max(p0, zero2);
                    p1 = __builtin_elementwise_max(p1, zero2);
                }
                const u32x2 v = {__builtin_bit_cast(uint32_t, p0), __builtin_bit_cast(uint32_t, p1)};
                storeStream8(obase + (outLane + 16u * q), v);      // (written once, read by nobody here)
            }
        }
    };
    uint32_t raw[2][2][RAW];
    auto pinRaw = [&]() {      // whatever the first layer's operands are formed from, on both sides of the mode switch
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            if constexpr (IN_HALF) {
#pragma unroll
                for (int d = 0; d < RAW; ++d) { pinHere(raw[j][0][d]); pinHere(raw[j][1][d]); }
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) { pinHere(B[j][0][i]); pinHere(B[j][1][i]); }
            }
        }
    };
    // the first layer's operands from fp16 vectors: quantised to e4m3 (saturating by mode), decoded again
    // (e4m3 rows were decoded when they were taken out of their slot)
    auto firstOperands = [&](int j) {
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            if constexpr (IN_HALF) {
                typedef short shortx2 __attribute__((ext_vector_type(2)));
                uint32_t q[2];
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const halfx2 p0 = __builtin_bit_cast(halfx2, raw[j][s][2 * i]), p1 = __builtin_bit_cast(halfx2, raw[j][s][2 * i + 1]);
                    shortx2 r = __builtin_bit_cast(shortx2, p0);
                    r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r, p0, 1.0f, false);
                    r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r, p1, 1.0f, true);
                    q[i] = __builtin_bit_cast(uint32_t, r);
                }
                Fp8AsF16Mma::decode(q, B[j][s]);
            }
        }
    };

    Slot pf[2];
    issue(pf[0], 2u * pair);
    issue(pf[1], 2u * pair + 1u);
    while (true) {
        const uint32_t next = claim();      // beyond the end: its loads are redirected to the last tile and never used
        consume(pf[0], 2u * next, raw[0], B[0]);
        consume(pf[1], 2u * next + 1u, raw[1], B[1]);
        // from here to the last layer's accumulators the conversions saturate by mode
        pinRaw();
        setFp16OverflowClamp<true>();
        pinRaw();
        firstOperands(0); firstLayer(0);
        firstOperands(1); firstLayer(1);
#pragma unroll
        for (int l = 1; l < NH; ++l) {
            carrier(0); hiddenLayer(l, 0);
            carrier(1); hiddenLayer(l, 1);
        }
        carrier(0); lastLayer(0);
        carrier(1); lastLayer(1);
        // the network's fp16 output keeps inf for an overflow: mode off before it is formed
        pinHere(acc[0][0]); pinHere(acc[1][0]);
        setFp16OverflowClamp<false>();
        pinHere(acc[0][0]); pinHere(acc[1][0]);
        storeTile(0, 2u * pair);
        storeTile(1, 2u * pair + 1u);
        if (next >= numPairs) return;
        pair = next;
    }
}

// true when mlpWideKernel can take this call: 32 inputs per sample in contiguous rows of e4m3 bytes or
// (to be quantised on the way in) of fp16, ReLU hidden layers of exactly 32 or 64 units, at most 32 outputs in whole
// groups of four with 8-byte aligned rows
inline bool mlpWideEligible(const MlpArgs& a, int& H, int& NH, int& OQ)
{
    const int L = a.numLayers;
    if (L < 2 || L > 4 || a.inEncoding != kEncodeNone || a.noWideTiles) return false;
    const uint64_t rowBytes = a.inHalfAsE4M3 ? 64u : 32u;
    if (a.layers[0].in != 32 || a.inStride != rowBytes || ((uintptr_t)a.in & 15u) != 0 || a.batch == 0 || a.batch > (1u << 31)) return false;
    const int width = a.layers[0].out;
    if (width != 32 && width != 64) return false;
    for (int l = 0; l < L; ++l) {
        if (l + 1 < L && (a.layers[l].out != width || a.layers[l].act != kActRelu)) return false;
        if (l > 0 && a.layers[l].in != width) return false;
    }
    const int outDim = a.layers[L - 1].out;
    if (a.layers[L - 1].act != kActNone && a.layers[L - 1].act != kActRelu) return false;
    if (outDim > 32 || outDim % 4 != 0 || a.outAlign < 8u || a.outStride >= (1u << 26)) return false;
    H = width / 32; NH = L - 1; OQ = outDim <= 8 ? 1 : (outDim <= 16 ? 2 : 4);
    return true;
}

template <int H, int NH, int OQ, bool IN_HALF, bool HAS_BIAS>
hipError_t launchMlpWideShape(hipStream_t stream, const MlpArgs& a, int numCUs)
{
    // one workgroup per compute unit, as many waves as the weights leave registers for
    // (16 waves: 128 registers each, 12: 168, 8: 256); the build fails if an instantiation spills
    constexpr bool twelve = (NH == 1 && !(HAS_BIAS && (IN_HALF || OQ == 4))) || (NH == 2 && !HAS_BIAS && !(IN_HALF && OQ == 4));
    constexpr int WAVES = H == 1 ? 16 : (twelve ? 12 : 8);
    const uint32_t numPairs = ((a.batch + 31u) / 32u + 1u) / 2u;
    const uint32_t blocks = numPairs < (uint32_t)numCUs ? numPairs : (uint32_t)numCUs;
    noteKernel(false, "mlpWideKernel<e4m3-f16pipe,32x32x16,hidden=%dx%d,outputs<=%d,%s%s>", NH, 32 * H, 8 * OQ,
               HAS_BIAS ? "bias" : "nobias", IN_HALF ? ",fp16-vectors" : "");
    hipLaunchKernelGGL((mlpWideKernel<H, NH, OQ, WAVES, IN_HALF, HAS_BIAS>), dim3(blocks), dim3(64 * WAVES), 0, stream, a);
    return hipGetLastError();
}

inline hipError_t launchMlpWide(hipStream_t stream, const MlpArgs& a, int numCUs, int H, int NH, int OQ)
{
    bool hasBias = false;
    for (int l = 0; l < a.numLayers; ++l) hasBias = hasBias || a.layers[l].bias != nullptr;
    const int variant = (a.inHalfAsE4M3 ? 1 : 0) + (hasBias ? 2 : 0);
#define CV_W(h_, nh_, oq_) if (H == h_ && NH == nh_ && OQ == oq_) { \
        switch (variant) { \
        case 0: return launchMlpWideShape<h_, nh_, oq_, false, false>(stream, a, numCUs); \
        case 1: return launchMlpWideShape<h_, nh_, oq_, true, false>(stream, a, numCUs); \
        case 2: return launchMlpWideShape<h_, nh_, oq_, false, true>(stream, a, numCUs); \
        default: return launchMlpWideShape<h_, nh_, oq_, true, true>(stream, a, numCUs); \
        } }
    CV_W(2, 1, 1) CV_W(2, 2, 1) CV_W(2, 3, 1) CV_W(1, 1, 1) CV_W(1, 2, 1) CV_W(1, 3, 1)
    CV_W(2, 1, 2) CV_W(2, 2, 2) CV_W(2, 3, 2) CV_W(2, 1, 4) CV_W(2, 2, 4) CV_W(2, 3, 4)
#undef CV_W
    return hipErrorInvalidValue;
}

} // namespace
} // namespace cv
