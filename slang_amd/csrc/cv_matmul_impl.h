// cv_matmul_impl.h -- batched coopVecMatMul / coopVecMatMulAdd kernel template for gfx950.
//
// Replaces the per-thread operator of source/slang/hlsl.meta.slang:32786-33190 (whose only
// in-tree executable form is the scalar fallback :32835-32912 / :33043-33103) by a dense
// contraction: the 16 samples of a tile are the N dimension of D = W . X^T, computed with
// v_mfma_f32_16x16x32_f16 / v_mfma_f32_16x16x32_fp8_fp8 / v_mfma_i32_16x16x64_i8.  e4m3
// matrices run on the fp16 pipeline by default (exact decode, fp32-grade accumulation) and on
// the fp8 pipeline on request (see cv_device.h for the measured difference).
//
//  - the workgroup stages the matrix once into LDS in fragment order (any source layout is
//    gathered through cv::elemOffset; an InferencingOptimal source of matching shape is a
//    straight 16-byte copy), then every wave keeps its A fragments in VGPRs for its lifetime;
//  - waves are persistent and stride over tiles of NT*16 samples, prefetching the next tile's
//    input registers before the MFMAs of the current one;
//  - lane group g loads the contiguous quarter g of each sample's input vector and stores the
//    contiguous quarter g of its output vector (see cv_device.h), so a K=64 fp16 sample row
//    of 128 B is read by four lanes with two 16-byte loads each and written the same way;
//  - bias seeds the accumulators; activation and the cast to the result type are fused.
//
// Two instantiations per shape: FAST (full-width aligned vectors, m a multiple of 16, no
// leaky ReLU, no accumulate form: a branch-free streaming loop) and the general one (ragged
// shapes, unaligned vectors, `this += ...`, every activation).
//
// Shapes beyond the register-resident ones: more than 128 rows are served in blocks of rows
// (one launch per block, MatMulArgs::rowOff), more than four k-tiles by matmulLargeKernel, which
// keeps its block of the matrix in LDS and walks the k-tiles in a loop.
#pragma once
#include <type_traits>

#include "cv_device.h"
#include "cv_kernels.h"
#include "cv_launch.h"
#include "cv_error.h"
#include "cv_stage.h"

namespace cv {
namespace {

// ---- matMul flavours: a matrix-core flavour plus how the input vectors lie in memory ----------
// kInEsz / kInRawDW / decodeIn describe the vectors the way kEsz / kRawDW / decode describe the
// matrix.  kAnySign: the int8 flavour that also serves unsigned bytes on either side.
template <class Mma>
struct VecAsMatrix : Mma {
    static constexpr int kInEsz = Mma::kEsz, kInRawDW = Mma::kRawDW;
    static constexpr bool kAnySign = false;
    // kStreaming: the flavour also gets the branch-free streaming instantiations (the less common
    // ones run every shape on the general kernel)
    static constexpr bool kStreaming = !std::is_same<Mma, Bf8AsF16Mma>::value;
    // kWideFragments: fp32 fragments are twice as wide; a block of the matrix stays in registers up to 64 rows and two
    // k-tiles (64 columns), everything larger runs on matmulLargeKernel
    static constexpr bool kWideFragments = std::is_same<Mma, F32Mma>::value;
    static __device__ __forceinline__ void decodeIn(const uint32_t* raw, uint32_t* frag) { Mma::decode(raw, frag); }
};

// fp16 vectors with inputInterpretation = FloatE4M3 against an e4m3 matrix: every element is
// quantised to OCP e4m3 (saturating, nearest even) as it is loaded, then runs as the exactly
// equal fp16 value on the fp16 matrix pipeline.
struct F16VecAsE4M3 : Fp8AsF16Mma {
    static constexpr const char* kName = "f16-as-e4m3-f16pipe";
    static constexpr int kInEsz = 2, kInRawDW = 4;
    static constexpr bool kAnySign = false, kStreaming = false, kWideFragments = false;
    static __device__ __forceinline__ uint32_t roundTrip(uint32_t h2)
    {
        typedef short shortx2 __attribute__((ext_vector_type(2)));
        const halfx2 lim = {(half_t)448.f, (half_t)448.f};
        halfx2 h = __builtin_bit_cast(halfx2, h2);
        h = __builtin_elementwise_min(__builtin_elementwise_max(h, -lim), lim);
        shortx2 r = __builtin_bit_cast(shortx2, h);
        r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r, h, 1.0f, false);
        return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(__builtin_bit_cast(uint32_t, r), 1.0f, false));
    }
    static __device__ __forceinline__ void decodeIn(const uint32_t* raw, uint32_t* frag)
    {
#pragma unroll
        for (int d = 0; d < 4; ++d) frag[d] = roundTrip(raw[d]);
    }
};

// Signed or unsigned bytes on either side of v_mfma_i32_16x16x64_i8, which multiplies signed
// bytes only.  An unsigned byte u is run as the signed byte u ^ 0x80 = u - 128, and the sum is
// corrected afterwards:   sum (w^ + 128 a)(x^ + 128 b) = sum w^ x^ + 128 b sum w^ + 128 a sum x^
// + 16384 a b k   (a, b in {0,1}: matrix / vectors unsigned).  Row sums of w^ are formed once per
// workgroup from the staged fragments, sums of x^ per tile, both with v_sad_u8.
struct I8AnySign : I8Mma {
    static constexpr const char* kName = "i8-any-sign";
    static constexpr int kInEsz = 1, kInRawDW = 4;
    static constexpr bool kAnySign = true, kStreaming = true, kWideFragments = false;
    static __device__ __forceinline__ void decodeIn(const uint32_t* raw, uint32_t* frag) { I8Mma::decode(raw, frag); }
};

// signed sum of the four bytes of a dword
__device__ __forceinline__ int sumSignedBytes(uint32_t v)
{
    return (int)__builtin_amdgcn_sad_u8(v ^ 0x80808080u, 0u, 0u) - 512;
}
// 0x80 in every byte of dword i that lies below validBytes
__device__ __forceinline__ uint32_t signFlipMask(int i, int validBytes)
{
    const int nb = validBytes - 4 * i;
    return nb >= 4 ? 0x80808080u : nb <= 0 ? 0u : (0x80808080u & ((1u << (8 * nb)) - 1u));
}

// two fp32 values -> one dword of two 16-bit results
template <typename OutT>
__device__ __forceinline__ uint32_t pack16(float a, float b)
{
    if constexpr (std::is_same<OutT, half_t>::value) {
        const halfx2 h = {(half_t)a, (half_t)b};
        return __builtin_bit_cast(uint32_t, h);
    } else {
        const bf16x2 h = {(bf16_t)a, (bf16_t)b};
        return __builtin_bit_cast(uint32_t, h);
    }
}

// activation on an accumulator that becomes a 16-bit result: rounded to the result type first
// (the operator's T), then the activation in T's arithmetic
template <typename OutT>
__device__ __forceinline__ float activate16(float acc, int act, float slope)
{
    if constexpr (std::is_same<OutT, half_t>::value) {
        return (float)activateHalf((half_t)acc, act, slope);
    } else {
        float z = (float)(bf16_t)acc;
        if (act == kActRelu) z = z > 0.f ? z : 0.f;
        else if (act == kActLeakyRelu) { const float zs = (float)(bf16_t)(z * slope); z = z >= zs ? z : zs; }
        else if (act >= kActSigmoid) z = smoothActivation(z, act);
        return z;
    }
}

template <int DW>
__device__ __forceinline__ void loadSlotsVec(uint32_t (&s)[DW], const uint8_t* p)
{
    if constexpr (DW % 4 == 0) {
#pragma unroll
        for (int i = 0; i < DW / 4; ++i) {
            const u32x4 v = *(const u32x4*)(p + 16 * i);
            s[4 * i] = v.x; s[4 * i + 1] = v.y; s[4 * i + 2] = v.z; s[4 * i + 3] = v.w;
        }
    } else {
#pragma unroll
        for (int i = 0; i < DW / 2; ++i) {
            const u32x2 v = *(const u32x2*)(p + 8 * i);
            s[2 * i] = v.x; s[2 * i + 1] = v.y;
        }
    }
}

// mode 0: full-width vector loads, 1: masked dwords, 2: masked bytes
template <int DW>
__device__ __forceinline__ void loadSlots(uint32_t (&s)[DW], const uint8_t* p, int validBytes, int mode)
{
    if (mode == 0) {
        loadSlotsVec<DW>(s, p);
    } else if (mode == 1) {
#pragma unroll
        for (int i = 0; i < DW; ++i) s[i] = (4 * i < validBytes) ? *(const uint32_t*)(p + 4 * i) : 0u;
    } else {
#pragma unroll
        for (int i = 0; i < DW; ++i) {
            uint32_t v = 0;
#pragma unroll
            for (int b = 0; b < 4; ++b)
                if (4 * i + b < validBytes) v |= (uint32_t)p[4 * i + b] << (8 * b);
            s[i] = v;
        }
    }
}

template <int DW>
__device__ __forceinline__ void storeVec(uint8_t* o, const uint32_t (&pk)[DW])
{
    if constexpr (DW % 4 == 0) {
#pragma unroll
        for (int i = 0; i < DW / 4; ++i) {
            const u32x4 v = {pk[4 * i], pk[4 * i + 1], pk[4 * i + 2], pk[4 * i + 3]};
            ((u32x4*)o)[i] = v;
        }
    } else {
#pragma unroll
        for (int i = 0; i < DW / 2; ++i) {
            const u32x2 v = {pk[2 * i], pk[2 * i + 1]};
            ((u32x2*)o)[i] = v;
        }
    }
}

// Per-lane constants of a wave's output: lane group g owns rows [g*ROWS, (g+1)*ROWS) of the block.
template <class Fl, int MT>
struct LaneOut {
    typename Fl::Acc bias[MT];   // bias (and, for unsigned bytes, the per-row correction)
    int validRows;
};

template <class Fl, int MT>
__device__ __forceinline__ void loadBias(LaneOut<Fl, MT>& lo, const MatMulArgs& a, int rowBase)
{
    constexpr int ROWS = 4 * MT;
    lo.validRows = min(max(a.m - rowBase, 0), ROWS);
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int row = rowBase + 4 * t + r;
            if constexpr (Fl::kIsFloat)
                lo.bias[t][r] = (a.bias && row < a.m) ? loadAsFloat(a.bias + (size_t)row * elemSize(a.biasCt), a.biasCt) : 0.f;
            else
                lo.bias[t][r] = (a.bias && row < a.m) ? ((const int32_t*)a.bias)[row] : 0;
        }
}

// General epilogue of one 16-sample tile: every activation, ragged m, unaligned rows, `this += ...`.
template <class Fl, int MT, typename OutT>
__device__ __forceinline__ void storeGeneral(const typename Fl::Acc (&acc)[MT], const MatMulArgs& a, uint8_t* o, int validRows)
{
    constexpr int ROWS = 4 * MT;
    constexpr int OUT_DW = ROWS * (int)sizeof(OutT) / 4;
    uint32_t pk[OUT_DW];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        if constexpr (sizeof(OutT) == 2) {
            pk[2 * t] = pack16<OutT>(activate16<OutT>(acc[t][0], a.act, a.slope), activate16<OutT>(acc[t][1], a.act, a.slope));
            pk[2 * t + 1] = pack16<OutT>(activate16<OutT>(acc[t][2], a.act, a.slope), activate16<OutT>(acc[t][3], a.act, a.slope));
        } else if constexpr (Fl::kIsFloat) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float x = acc[t][r];
                if (a.act == kActRelu) x = x > 0.f ? x : 0.f;
                else if (a.act == kActLeakyRelu) x = fmaxf(x, x * a.slope);
                else if (a.act >= kActSigmoid) x = smoothActivation(x, a.act);
                pk[4 * t + r] = __builtin_bit_cast(uint32_t, x);
            }
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                int x = acc[t][r];
                if (a.act == kActRelu) x = x > 0 ? x : 0;
                pk[4 * t + r] = (uint32_t)x;
            }
        }
    }
    if (a.accumulate || validRows != ROWS || a.outAlign < (OUT_DW % 4 == 0 ? 16u : 8u)) {
        // element-wise tail: the member forms `this += ...`, ragged m, unaligned rows
        OutT* oe = (OutT*)o;
#pragma unroll
        for (int e = 0; e < ROWS; ++e) {
            if (e < validRows) {
                if constexpr (sizeof(OutT) == 2) {
                    const uint16_t bits = (uint16_t)(pk[e / 2] >> (16 * (e & 1)));
                    OutT v = __builtin_bit_cast(OutT, bits);
                    if (a.accumulate) v = (OutT)((float)oe[e] + (float)v);
                    oe[e] = v;
                } else {
                    OutT v = __builtin_bit_cast(OutT, pk[e]);
                    if (a.accumulate) v = oe[e] + v;
                    oe[e] = v;
                }
            }
        }
    } else {
        storeVec<OUT_DW>(o, pk);
    }
}

// Per-row correction of the unsigned-byte forms, added to the bias: 128 * sum_k w^[row][k] when the
// vectors are unsigned, plus 16384 * k when the matrix is unsigned too.  rowSum[t] holds, in lane
// 16*g+i, the sum of this lane's k-slots of row (i/4)*ROWS + 4t + i%4.
template <class Fl, int MT>
__device__ __forceinline__ void addUnsignedRowTerm(LaneOut<Fl, MT>& lo, int (&rowSum)[MT], const MatMulArgs& a, int g)
{
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int total = sumOverGroups(rowSum[t]);      // lane i (any group): row (i/4)*ROWS + 4t + i%4
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int mine = __shfl(total, 4 * g + r);   // row g*ROWS + 4t + r
            lo.bias[t][r] += 128 * mine + (a.matUnsigned ? 16384 * a.k : 0);
        }
    }
}

// LINES (streaming kernel only): the vectors on both sides are whole, aligned 128-byte lines, which the
// kernel then reads and writes with non-temporal accesses.
template <class Fl, int MT, int KT, int NT, typename OutT, bool FAST, bool LINES = false>
__global__ __launch_bounds__(256) void matmulKernel(const MatMulArgs a)
{
    constexpr int EPL = Fl::kEpl, FD = Fl::kFD, ESZ = Fl::kEsz, RAW = Fl::kRawDW;
    constexpr int IESZ = Fl::kInEsz, IRAW = Fl::kInRawDW;
    constexpr int SLOT_DW = IRAW * KT;        // input dwords per lane per 16-sample tile
    constexpr int ROWS = 4 * MT;              // output rows per lane
    constexpr int OUT_DW = ROWS * (int)sizeof(OutT) / 4;
    typedef typename Fl::Acc Acc;

    __shared__ __attribute__((aligned(16))) uint32_t ldsW[MT * KT * 64 * RAW];
    // Output rows of 128 bytes or more leave through a per-wave LDS transpose so that every
    // store instruction writes whole 128-byte lines (lane l -> 16 consecutive bytes of the
    // tile's output block) instead of 16-byte pieces of many lines.  Rows are padded by 16
    // bytes in LDS, which makes both the scattered writes and the linear reads conflict-free.
    constexpr int ROW_DW = 4 * OUT_DW;                      // dwords of one sample's output row
    constexpr bool LDS_STORE = FAST && ROW_DW >= 32;
    constexpr int STAGE_DW = LDS_STORE ? 16 * (ROW_DW + 4) : 4;
    __shared__ __attribute__((aligned(16))) uint32_t ldsStage[4 * STAGE_DW];

    const uint32_t gs = optGS((uint32_t)a.k);   // k-slots owned by one lane group

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, n = lane & 15;

    // ---- per-lane constants -------------------------------------------------------------
    const int rowBase = g * ROWS;
    const int colBase = (int)(g * gs);
    const int validBytes = min((int)gs, max(a.k - colBase, 0)) * IESZ;
    const int loadMode = (validBytes == SLOT_DW * 4 && a.inAlign >= (SLOT_DW % 4 == 0 ? 16u : 8u)) ? 0
                       : ((validBytes & 3) == 0 && a.inAlign >= 4u) ? 1 : 2;

    LaneOut<Fl, MT> lo;
    loadBias<Fl, MT>(lo, a, rowBase);
    const int validRows = lo.validRows;
    // ReLU as a lower bound: max(z, 0) when on, max(z, -inf) = z when off (FAST path)
    const float reluFloor = a.act == kActRelu ? 0.f : -__builtin_inff();
    const int reluFloorI = a.act == kActRelu ? 0 : (int)0x80000000;

    constexpr uint32_t TILE = 16 * NT;
    // FAST handles whole tiles only (the launcher sends the ragged tail to the general kernel),
    // so its loop has no per-lane predicates and the prefetch below is unconditional: with a
    // fixed number of loads and stores per iteration the compiler can wait for exactly the
    // current tile's loads while the next tile's stay in flight.
    const uint32_t numTiles = FAST ? a.batch / TILE : (a.batch + TILE - 1) / TILE;
    const uint32_t tileStride = gridDim.x * 4;
    uint32_t tile = blockIdx.x * 4 + wave;
    const bool haveTile = tile < numTiles;     // (no early return: every wave takes part in staging the matrix)

    const uint8_t* inLane = a.in + (size_t)colBase * IESZ;
    uint8_t* outLane = a.out + (size_t)rowBase * sizeof(OutT);
    const uint32_t lastSample = a.batch - 1;

    // One tile's input registers are loaded a whole tile ahead.  The two buffers swap roles
    // (no register copies: a copy would have to wait for the prefetch it is meant to hide).
    // LINE_LOADS (streaming kernel, rows of eight 16-byte chunks = one 128-byte line): a load instruction
    // of the wave covers eight whole rows, the eight lanes {n%8} x {g} x {n/8} of a row taking its
    // chunks 2g + n/8, which lets the loads be non-temporal (loadStream16).  The first instruction
    // fetches samples 0..7 of the tile, the second samples 8..15, so a lane ends up with chunk
    // 2g + n/8 of samples n%8 and 8 + n%8; the fragment it needs (chunks 2g and 2g+1 of sample n) is
    // completed by one exchange with the lane eight places away in its row (lineSwap, DPP).
    // (Measured: fp16 64x64 196 -> 188 us together with the non-temporal stores; where a sample's output
    // is several times its input, as for int8 128x128 with 512-byte rows of int32, the exchange costs
    // more than the loads gain, so those shapes keep the plain pattern.)
    constexpr bool LINE_LOADS = FAST && LINES && KT == 2 && IRAW == 4 && ROWS * 4 * (int)sizeof(OutT) <= 256;
    auto loadTile = [&](uint32_t (&buf)[NT][SLOT_DW], uint32_t t) {
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            if constexpr (LINE_LOADS) {
                const uint8_t* p = a.in + (size_t)(t * TILE + 16 * j + (n & 7)) * a.inStride + (2 * g + (n >> 3)) * 16;
                const u32x4 v0 = loadStream16(p), v1 = loadStream16(p + (size_t)8 * a.inStride);
                buf[j][0] = v0.x; buf[j][1] = v0.y; buf[j][2] = v0.z; buf[j][3] = v0.w;
                buf[j][4] = v1.x; buf[j][5] = v1.y; buf[j][6] = v1.z; buf[j][7] = v1.w;
            } else if constexpr (FAST) {
                loadSlotsVec<SLOT_DW>(buf[j], inLane + (size_t)(t * TILE + 16 * j + n) * a.inStride);
            } else {
                const uint32_t s = min(t * TILE + 16 * j + n, lastSample);
                loadSlots<SLOT_DW>(buf[j], inLane + (size_t)s * a.inStride, validBytes, loadMode);
            }
        }
    };

    // The first tile's vectors are requested before the matrix is staged: their trip to HBM and the
    // staging overlap.
    uint32_t bufA[NT][SLOT_DW], bufB[NT][SLOT_DW];
    if (haveTile) loadTile(bufA, tile);

    stageFragments<ESZ, EPL>(ldsW, a.mat, a.shape, a.transpose != 0, MT, KT, gs, (uint32_t)a.m, (uint32_t)a.k,
                             a.rowOff, (Fl::kAnySign && a.matUnsigned) ? 0x80u : 0u);
    __syncthreads();

    uint32_t afrag[MT][KT][FD];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
            Fl::decode(&ldsW[((t * KT + kt) * 64 + lane) * RAW], afrag[t][kt]);

    if constexpr (Fl::kAnySign) {
        if (a.inUnsigned) {
            int rowSum[MT];
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                rowSum[t] = 0;
#pragma unroll
                for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                    for (int d = 0; d < FD; ++d) rowSum[t] += sumSignedBytes(afrag[t][kt][d]);
            }
            addUnsignedRowTerm<Fl, MT>(lo, rowSum, a, g);
        }
    }
    auto computeStore = [&](const uint32_t (&bufIn)[NT][SLOT_DW], uint32_t t0) {
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            uint32_t slot[SLOT_DW];
#pragma unroll
            for (int d = 0; d < SLOT_DW; ++d) slot[d] = bufIn[j][d];
            if constexpr (LINE_LOADS) {
                // lanes 0..7 of a row keep their first register (sample n, chunk 2g) and take the partner's
                // first one (sample n, chunk 2g+1); lanes 8..15 keep their second and take the partner's second
                constexpr int kRowRor8 = 0x128;
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    const int r0 = (int)bufIn[j][d], r1 = (int)bufIn[j][4 + d];
                    slot[4 + d] = (uint32_t)__builtin_amdgcn_update_dpp(r1, r0, kRowRor8, 0xf, 0x3, false);
                    slot[d] = (uint32_t)__builtin_amdgcn_update_dpp(r0, r1, kRowRor8, 0xf, 0xc, false);
                }
            }
            const uint32_t (&buf)[SLOT_DW] = slot;
            Acc acc[MT];
#pragma unroll
            for (int t = 0; t < MT; ++t) acc[t] = lo.bias[t];
            int xSum = 0;       // unsigned matrix: sum of this lane's signed input bytes
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                uint32_t bfrag[FD];
                if constexpr (Fl::kAnySign) {
                    uint32_t x[IRAW];
#pragma unroll
                    for (int d = 0; d < IRAW; ++d) {
                        x[d] = buf[kt * IRAW + d];
                        if (a.inUnsigned) x[d] ^= FAST ? 0x80808080u : signFlipMask(kt * IRAW + d, validBytes);
                        if (a.matUnsigned) xSum += sumSignedBytes(x[d]);
                    }
                    Fl::decodeIn(x, bfrag);
                } else {
                    Fl::decodeIn(&buf[kt * IRAW], bfrag);
                }
#pragma unroll
                for (int t = 0; t < MT; ++t) acc[t] = Fl::mma(afrag[t][kt], bfrag, acc[t]);
            }
            if constexpr (Fl::kAnySign) {
                if (a.matUnsigned) {
                    const int add = 128 * sumOverGroups(xSum);
#pragma unroll
                    for (int t = 0; t < MT; ++t)
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[t][r] += add;
                }
            }

            const uint32_t sample = t0 * TILE + 16 * j + n;
            uint8_t* o = outLane + (size_t)sample * a.outStride;
            if constexpr (FAST) {
                uint32_t pk[OUT_DW];
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    if constexpr (sizeof(OutT) == 2) {
                        // max on the fp32 accumulator commutes with the rounding to 16 bits
                        pk[2 * t] = pack16<OutT>(fmaxf(acc[t][0], reluFloor), fmaxf(acc[t][1], reluFloor));
                        pk[2 * t + 1] = pack16<OutT>(fmaxf(acc[t][2], reluFloor), fmaxf(acc[t][3], reluFloor));
                    } else if constexpr (Fl::kIsFloat) {
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            pk[4 * t + r] = __builtin_bit_cast(uint32_t, fmaxf(acc[t][r], reluFloor));
                    } else {
#pragma unroll
                        for (int r = 0; r < 4; ++r) pk[4 * t + r] = (uint32_t)max(acc[t][r], reluFloorI);
                    }
                }
                if constexpr (LDS_STORE) {
                    uint32_t* st = ldsStage + wave * STAGE_DW;
                    u32x4* w = (u32x4*)(st + n * (ROW_DW + 4) + g * OUT_DW);
#pragma unroll
                    for (int i = 0; i < OUT_DW / 4; ++i) {
                        const u32x4 v = {pk[4 * i], pk[4 * i + 1], pk[4 * i + 2], pk[4 * i + 3]};
                        w[i] = v;
                    }
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                    constexpr int CPR = ROW_DW / 4;            // 16-byte chunks per row (power of two)
                    uint8_t* tileOut = a.out + (size_t)(t0 * TILE + 16 * j) * a.outStride;
#pragma unroll
                    for (int i = 0; i < ROW_DW / 16; ++i) {
                        const int c = i * 64 + lane, srow = c / CPR, ch = c % CPR;
                        const u32x4 v = *(const u32x4*)(st + srow * (ROW_DW + 4) + ch * 4);
                        uint8_t* dst = tileOut + (size_t)srow * a.outStride + ch * 16;
                        if constexpr (LINES) storeStream16(dst, v);      // in pieces of lines such stores crawl
                        else *(u32x4*)dst = v;
                    }
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                } else {
                    storeVec<OUT_DW>(o, pk);
                }
            } else {
                if (sample >= a.batch || validRows <= 0) continue;
                storeGeneral<Fl, MT, OutT>(acc, a, o, validRows);
            }
        }
    };

    while (haveTile) {
        // a prefetch past the end re-reads a valid tile instead of branching around the loads
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

// ---- any number of k-tiles: the block of the matrix lives in LDS ---------------------------------
// One workgroup stages the MT x KT fragments of its block of rows into dynamic LDS; a wave then
// walks the k-tiles of a 16-sample tile KC at a time, reading its vector slice from memory and the
// matrix fragments from LDS.  KT is a multiple of KC (fragments past the matrix hold zeros).
constexpr int kLargeKC = 4;
constexpr int kLargeLdsBytes = 128 * 1024;

template <class Fl, int MT, typename OutT>
__global__ __launch_bounds__(256) void matmulLargeKernel(const MatMulArgs a, const int KT)
{
    constexpr int EPL = Fl::kEpl, FD = Fl::kFD, ESZ = Fl::kEsz, RAW = Fl::kRawDW;
    constexpr int IESZ = Fl::kInEsz, IRAW = Fl::kInRawDW;
    constexpr int KC = kLargeKC, STEP_DW = KC * IRAW, ROWS = 4 * MT;
    typedef typename Fl::Acc Acc;
    extern __shared__ __attribute__((aligned(16))) uint32_t ldsDyn[];

    const uint32_t gs = optGS((uint32_t)a.k);
    stageFragments<ESZ, EPL>(ldsDyn, a.mat, a.shape, a.transpose != 0, MT, KT, gs, (uint32_t)a.m, (uint32_t)a.k,
                             a.rowOff, (Fl::kAnySign && a.matUnsigned) ? 0x80u : 0u);
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, n = lane & 15;
    const int rowBase = g * ROWS;
    const int colBase = (int)(g * gs);
    const int validBytes = min((int)gs, max(a.k - colBase, 0)) * IESZ;

    LaneOut<Fl, MT> lo;
    loadBias<Fl, MT>(lo, a, rowBase);
    if constexpr (Fl::kAnySign) {
        if (a.inUnsigned) {
            int rowSum[MT];
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                rowSum[t] = 0;
                for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                    for (int d = 0; d < RAW; ++d) rowSum[t] += sumSignedBytes(ldsDyn[((t * KT + kt) * 64 + lane) * RAW + d]);
            }
            addUnsignedRowTerm<Fl, MT>(lo, rowSum, a, g);
        }
    }

    const uint8_t* inLane = a.in + (size_t)colBase * IESZ;
    uint8_t* outLane = a.out + (size_t)rowBase * sizeof(OutT);
    const uint32_t numTiles = (a.batch + 15) / 16;
    for (uint32_t tile = blockIdx.x * 4 + wave; tile < numTiles; tile += gridDim.x * 4) {
        const uint32_t sample = tile * 16 + n;
        const uint8_t* p = inLane + (size_t)min(sample, a.batch - 1) * a.inStride;
        Acc acc[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[t] = lo.bias[t];
        int xSum = 0;
        for (int kc = 0; kc < KT; kc += KC) {
            const int off = kc * IRAW * 4;                         // byte offset of this step in the lane's slice
            const int vb = min(max(validBytes - off, 0), STEP_DW * 4);
            const int mode = (vb == STEP_DW * 4 && a.inAlign >= 16u && ((colBase * IESZ) & 15) == 0) ? 0 : ((vb & 3) == 0 && a.inAlign >= 4u) ? 1 : 2;
            uint32_t x[STEP_DW];
            loadSlots<STEP_DW>(x, p + off, vb, mode);
            if constexpr (Fl::kAnySign) {
#pragma unroll
                for (int d = 0; d < STEP_DW; ++d) {
                    if (a.inUnsigned) x[d] ^= signFlipMask(d, vb);
                    if (a.matUnsigned) xSum += sumSignedBytes(x[d]);
                }
            }
#pragma unroll
            for (int j = 0; j < KC; ++j) {
                uint32_t bfrag[FD];
                Fl::decodeIn(&x[j * IRAW], bfrag);
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    uint32_t af[FD];
                    Fl::decode(&ldsDyn[((t * KT + kc + j) * 64 + lane) * RAW], af);
                    acc[t] = Fl::mma(af, bfrag, acc[t]);
                }
            }
        }
        if constexpr (Fl::kAnySign) {
            if (a.matUnsigned) {
                const int add = 128 * sumOverGroups(xSum);
#pragma unroll
                for (int t = 0; t < MT; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[t][r] += add;
            }
        }
        if (sample < a.batch && lo.validRows > 0)
            storeGeneral<Fl, MT, OutT>(acc, a, outLane + (size_t)sample * a.outStride, lo.validRows);
    }
}

#ifndef CV_MATMUL_NT_SMALL
#define CV_MATMUL_NT_SMALL 2
#endif

template <int MT, int KT>
struct TileShape {
    // samples per wave-iteration: as many 16-sample tiles as the register budget allows
    static constexpr int NT = (MT * KT <= 8) ? CV_MATMUL_NT_SMALL : (MT * KT <= 16 ? 2 : 1);
};

template <class Fl, int MT, int KT, typename OutT, bool FAST, bool LINES = false>
hipError_t launchOne(hipStream_t stream, const MatMulArgs& a, int numCUs, bool append)
{
    constexpr int NT = TileShape<MT, KT>::NT;
    // Persistent grid: exactly as many workgroups as are resident at once, so that every wave
    // strides over the same number of tiles (a partial second round would run at a fraction of
    // the occupancy).  The residency of a kernel is fixed, so it is queried once.
    const int blocksPerCU = residentBlocksPerCU<matmulKernel<Fl, MT, KT, NT, OutT, FAST, LINES>>(256);
    const uint32_t tile = 16 * NT;
    const uint32_t numTiles = (a.batch + tile - 1) / tile;
    const uint32_t blocksNeeded = (numTiles + 3) / 4;
    const uint32_t blocksMax = (uint32_t)numCUs * (uint32_t)blocksPerCU;
    const uint32_t blocks = blocksNeeded < blocksMax ? blocksNeeded : blocksMax;
    noteKernel(append, "matmulKernel<%s,MT=%d,KT=%d,NT=%d,out=%dB,%s>", Fl::kName, MT, KT, NT,
               (int)sizeof(OutT), LINES ? "streaming,lines" : FAST ? "streaming" : "general");
    hipLaunchKernelGGL((matmulKernel<Fl, MT, KT, NT, OutT, FAST, LINES>), dim3(blocks), dim3(256), 0, stream, a);
    return hipGetLastError();
}

template <class Fl, int MT, int KT, typename OutT>
hipError_t launchShape(hipStream_t stream, const MatMulArgs& a, int numCUs, bool append)
{
    constexpr uint32_t slotBytes = Fl::kInRawDW * 4 * KT;
    constexpr uint32_t tile = 16 * TileShape<MT, KT>::NT;
    const bool fast = (uint32_t)a.k == 4u * Fl::kEpl * KT && a.m == 16 * MT &&
                      a.inAlign >= (slotBytes % 16 == 0 ? 16u : 8u) &&
                      a.outAlign >= ((4 * MT * sizeof(OutT)) % 16 == 0 ? 16u : 8u) &&
                      !a.accumulate && a.act <= kActRelu;
    if constexpr (!Fl::kStreaming) {
        return launchOne<Fl, MT, KT, OutT, false>(stream, a, numCUs, append);
    } else {
        if (!fast) return launchOne<Fl, MT, KT, OutT, false>(stream, a, numCUs, append);
        // whole tiles on the streaming kernel, the ragged tail (< one tile) on the general one
        const uint32_t whole = a.batch / tile * tile;
        if (whole) {
            MatMulArgs b = a;
            b.batch = whole;
            // rows of whole 128-byte lines on both sides (and an output row that leaves through the LDS transpose)
            constexpr bool kLinesShape = 16 * MT * sizeof(OutT) >= 128 && !Fl::kWideFragments;
            const bool lines = kLinesShape && (((uintptr_t)a.in | a.inStride | (uintptr_t)a.out | a.outStride) & 127u) == 0;
            hipError_t e;
            if constexpr (kLinesShape) {
                e = lines ? launchOne<Fl, MT, KT, OutT, true, true>(stream, b, numCUs, append)
                          : launchOne<Fl, MT, KT, OutT, true, false>(stream, b, numCUs, append);
            } else {
                e = launchOne<Fl, MT, KT, OutT, true, false>(stream, b, numCUs, append);
            }
            if (e != hipSuccess) return e;
        }
        if (whole == a.batch) return hipSuccess;
        MatMulArgs t = a;
        t.in += (size_t)whole * a.inStride;
        t.out += (size_t)whole * a.outStride;
        t.batch = a.batch - whole;
        return launchOne<Fl, MT, KT, OutT, false>(stream, t, numCUs, append || whole != 0);
    }
}

template <class Fl, int MT, typename OutT>
hipError_t launchLarge(hipStream_t stream, const MatMulArgs& a, int KT, int numCUs, bool append)
{
    const size_t ldsBytes = (size_t)MT * KT * 64 * Fl::kRawDW * 4;
    const hipError_t ea = allowDynamicLds<matmulLargeKernel<Fl, MT, OutT>>(kLargeLdsBytes);
    if (ea != hipSuccess) return ea;
    int perCU = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&perCU, matmulLargeKernel<Fl, MT, OutT>, 256, ldsBytes) != hipSuccess || perCU < 1) perCU = 1;
    const uint32_t numTiles = (a.batch + 15) / 16, need = (numTiles + 3) / 4;
    const uint32_t cap = (uint32_t)numCUs * (uint32_t)perCU;
    noteKernel(append, "matmulLargeKernel<%s,MT=%d,KT=%d,out=%dB>", Fl::kName, MT, KT, (int)sizeof(OutT));
    hipLaunchKernelGGL((matmulLargeKernel<Fl, MT, OutT>), dim3(need < cap ? need : cap), dim3(256), ldsBytes, stream, a, KT);
    return hipGetLastError();
}

// One block of at most 16*MTs rows at row a.rowOff (a.m = rows of the block; out and bias already
// point at the block's first row).
template <class Fl, typename OutT>
hipError_t dispatchBlock(hipStream_t stream, const MatMulArgs& a, int numCUs, bool append, int largeKT)
{
    const uint32_t mt = optMT((uint32_t)a.m), kt = optKT((uint32_t)a.k, Fl::kEpl);
    const int MTs = mt <= 1 ? 1 : mt <= 2 ? 2 : mt <= 4 ? 4 : mt <= 8 ? 8 : 0;
    if (!MTs) return hipErrorInvalidValue;
    if (largeKT) {
        switch (MTs) {
        case 1: return launchLarge<Fl, 1, OutT>(stream, a, largeKT, numCUs, append);
        case 2: return launchLarge<Fl, 2, OutT>(stream, a, largeKT, numCUs, append);
        case 4: return launchLarge<Fl, 4, OutT>(stream, a, largeKT, numCUs, append);
        default: return launchLarge<Fl, 8, OutT>(stream, a, largeKT, numCUs, append);
        }
    }
    const int KTs = kt <= 1 ? 1 : kt <= 2 ? 2 : kt <= 4 ? 4 : 0;
    if (!KTs) return hipErrorInvalidValue;
#define CV_CASE(M_, K_) \
    if (MTs == M_ && KTs == K_) return launchShape<Fl, M_, K_, OutT>(stream, a, numCUs, append);
    CV_CASE(1, 1) CV_CASE(1, 2)
    CV_CASE(2, 1) CV_CASE(2, 2)
    CV_CASE(4, 1) CV_CASE(4, 2)
    if constexpr (!Fl::kWideFragments) {
        CV_CASE(1, 4) CV_CASE(2, 4) CV_CASE(4, 4)
        CV_CASE(8, 1) CV_CASE(8, 2) CV_CASE(8, 4)
    }
#undef CV_CASE
    return hipErrorInvalidValue;
}

// Splits m into blocks of rows that one workgroup can hold: 128 rows while the fragments stay in
// registers (at most four k-tiles), else as many 16-row tiles (8, 4, 2 or 1) as fit the LDS budget.
// hipErrorInvalidValue when even one 16-row tile of k columns does not fit.
template <class Fl, typename OutT>
hipError_t dispatchShape(hipStream_t stream, const MatMulArgs& a, int numCUs)
{
    const uint32_t kt = optKT((uint32_t)a.k, Fl::kEpl);
    int blockTiles = 8, largeKT = 0;
    const bool inRegisters = Fl::kWideFragments ? (kt <= 2 && a.m <= 64) : kt <= 4;
    if (Fl::kWideFragments && inRegisters) blockTiles = 4;
    if (!inRegisters) {
        largeKT = (int)((kt + kLargeKC - 1) / kLargeKC * kLargeKC);
        const size_t tileBytes = (size_t)largeKT * 64 * Fl::kRawDW * 4;
        while (blockTiles > 1 && blockTiles * tileBytes > (size_t)kLargeLdsBytes) blockTiles /= 2;
        if (blockTiles * tileBytes > (size_t)kLargeLdsBytes) return hipErrorInvalidValue;
    }
    const int blockRows = 16 * blockTiles;
    const uint32_t biasEsz = a.bias ? elemSize(a.biasCt) : 0;
    for (int r0 = 0; r0 < a.m; r0 += blockRows) {
        MatMulArgs b = a;
        b.rowOff = (uint32_t)r0;
        b.m = a.m - r0 < blockRows ? a.m - r0 : blockRows;
        b.out = a.out + (size_t)r0 * sizeof(OutT);
        if (a.bias) b.bias = a.bias + (size_t)r0 * biasEsz;
        // an output row that starts inside a vector is only as aligned as its offset
        uint32_t al = a.outAlign;
        while (al > 1 && ((size_t)r0 * sizeof(OutT)) % al) al >>= 1;
        b.outAlign = al;
        const hipError_t e = dispatchBlock<Fl, OutT>(stream, b, numCUs, r0 != 0, largeKT);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

} // namespace
} // namespace cv
