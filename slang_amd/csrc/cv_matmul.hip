// cv_matmul.hip -- batched coopVecMatMul / coopVecMatMulAdd for gfx950.
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
#include "cv_device.h"
#include "cv_kernels.h"

namespace cv {

namespace {

template <int DW>
__device__ __forceinline__ void loadSlots(uint32_t (&s)[DW], const uint8_t* p, int validBytes, int mode)
{
    if (mode == 0) {
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

template <class Mma, int MT, int KT, int NT, typename OutT>
__global__ __launch_bounds__(256) void matmulKernel(const MatMulArgs a)
{
    constexpr int EPL = Mma::kEpl, FD = Mma::kFD, ESZ = Mma::kEsz, RAW = Mma::kRawDW;
    constexpr int SLOT_DW = RAW * KT;         // input dwords per lane per 16-sample tile
    constexpr int ROWS = 4 * MT;              // output rows per lane
    typedef typename Mma::Acc Acc;

    __shared__ __attribute__((aligned(16))) uint32_t ldsW[MT * KT * 64 * RAW];

    const uint32_t gs = optGS((uint32_t)a.k);   // k-slots owned by one lane group

    // ---- stage the matrix into LDS in fragment order ------------------------------------
    {
        const bool direct = a.shape.layout == kInferencingOptimal && !a.transpose &&
                            optMT(a.shape.rows) == (uint32_t)MT &&
                            optKT(a.shape.cols, EPL) == (uint32_t)KT;
        if (direct) {
            const u32x4* src = (const u32x4*)a.mat;
            u32x4* dst = (u32x4*)ldsW;
            for (int i = threadIdx.x; i < MT * KT * 64 * RAW / 4; i += 256) dst[i] = src[i];
        } else {
            uint8_t* dst = (uint8_t*)ldsW;
            for (int e = threadIdx.x; e < MT * KT * 64 * EPL; e += 256) {
                const int s = e % EPL, lane = (e / EPL) & 63, f = e / (EPL * 64);
                const int kt = f % KT, t = f / KT, g = lane >> 4, i = lane & 15;
                const uint32_t row = (uint32_t)((i >> 2) * ROWS + 4 * t + (i & 3));
                const uint32_t q = (uint32_t)(kt * EPL + s), col = g * gs + q;
                const bool valid = row < (uint32_t)a.m && q < gs && col < (uint32_t)a.k;
                const size_t off = valid ? (a.transpose ? elemOffset(a.shape, col, row)
                                                        : elemOffset(a.shape, row, col)) : 0;
                if constexpr (ESZ == 2) ((uint16_t*)dst)[e] = valid ? *(const uint16_t*)(a.mat + off) : (uint16_t)0;
                else                    dst[e] = valid ? a.mat[off] : (uint8_t)0;
            }
        }
    }
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, n = lane & 15;

    uint32_t afrag[MT][KT][FD];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
            Mma::decode(&ldsW[((t * KT + kt) * 64 + lane) * RAW], afrag[t][kt]);

    // ---- per-lane constants -------------------------------------------------------------
    const int rowBase = g * ROWS;
    const int validRows = min(max(a.m - rowBase, 0), ROWS);
    const int colBase = (int)(g * gs);
    const int validBytes = min((int)gs, max(a.k - colBase, 0)) * ESZ;
    // 0: full-width vector loads, 1: masked dwords, 2: masked bytes
    const int loadMode = (validBytes == SLOT_DW * 4 && a.inAlign >= (SLOT_DW % 4 == 0 ? 16u : 8u)) ? 0
                       : ((validBytes & 3) == 0 && a.inAlign >= 4u) ? 1 : 2;

    Acc biasv[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int row = rowBase + 4 * t + r;
            if constexpr (Mma::kIsFloat)
                biasv[t][r] = (a.bias && row < a.m) ? loadAsFloat(a.bias + (size_t)row * elemSize(a.biasCt), a.biasCt) : 0.f;
            else
                biasv[t][r] = (a.bias && row < a.m) ? ((const int32_t*)a.bias)[row] : 0;
        }

    constexpr uint32_t TILE = 16 * NT;
    const uint32_t numTiles = (a.batch + TILE - 1) / TILE;
    const uint32_t tileStride = gridDim.x * 4;
    uint32_t tile = blockIdx.x * 4 + wave;
    if (tile >= numTiles) return;

    const uint8_t* inLane = a.in + (size_t)colBase * ESZ;
    uint8_t* outLane = a.out + (size_t)rowBase * sizeof(OutT);
    const uint32_t lastSample = a.batch - 1;

    uint32_t cur[NT][SLOT_DW], nxt[NT][SLOT_DW];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const uint32_t s = min(tile * TILE + 16 * j + n, lastSample);
        loadSlots<SLOT_DW>(cur[j], inLane + (size_t)s * a.inStride, validBytes, loadMode);
    }

    for (; tile < numTiles; tile += tileStride) {
        const uint32_t nextTile = tile + tileStride;
        if (nextTile < numTiles) {
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                const uint32_t s = min(nextTile * TILE + 16 * j + n, lastSample);
                loadSlots<SLOT_DW>(nxt[j], inLane + (size_t)s * a.inStride, validBytes, loadMode);
            }
        }

#pragma unroll
        for (int j = 0; j < NT; ++j) {
            Acc acc[MT];
#pragma unroll
            for (int t = 0; t < MT; ++t) acc[t] = biasv[t];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                uint32_t bfrag[FD];
                Mma::decode(&cur[j][kt * RAW], bfrag);
#pragma unroll
                for (int t = 0; t < MT; ++t) acc[t] = Mma::mma(afrag[t][kt], bfrag, acc[t]);
            }

            const uint32_t sample = tile * TILE + 16 * j + n;
            if (sample < a.batch && validRows > 0) {
                OutT* o = (OutT*)(outLane + (size_t)sample * a.outStride);
                constexpr int OUT_DW = ROWS * (int)sizeof(OutT) / 4;
                uint32_t pk[OUT_DW];
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    if constexpr (sizeof(OutT) == 2) {
                        halfx2 lo, hi;
                        lo.x = activateHalf((half_t)acc[t][0], a.act, a.slope);
                        lo.y = activateHalf((half_t)acc[t][1], a.act, a.slope);
                        hi.x = activateHalf((half_t)acc[t][2], a.act, a.slope);
                        hi.y = activateHalf((half_t)acc[t][3], a.act, a.slope);
                        pk[2 * t] = __builtin_bit_cast(uint32_t, lo);
                        pk[2 * t + 1] = __builtin_bit_cast(uint32_t, hi);
                    } else if constexpr (Mma::kIsFloat) {
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            float x = acc[t][r];
                            if (a.act == kActRelu) x = x > 0.f ? x : 0.f;
                            else if (a.act == kActLeakyRelu) x = fmaxf(x, x * a.slope);
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
                    // element-wise tail: the member forms `this += ...` and ragged m
#pragma unroll
                    for (int e = 0; e < ROWS; ++e) {
                        if (e < validRows) {
                            if constexpr (sizeof(OutT) == 2) {
                                const uint16_t bits = (uint16_t)(pk[e / 2] >> (16 * (e & 1)));
                                half_t v = __builtin_bit_cast(half_t, bits);
                                if (a.accumulate) v = (half_t)((float)o[e] + (float)v);
                                o[e] = v;
                            } else {
                                OutT v = __builtin_bit_cast(OutT, pk[e]);
                                if (a.accumulate) v = o[e] + v;
                                o[e] = v;
                            }
                        }
                    }
                } else if constexpr (OUT_DW % 4 == 0) {
#pragma unroll
                    for (int i = 0; i < OUT_DW / 4; ++i) {
                        const u32x4 v = {pk[4 * i], pk[4 * i + 1], pk[4 * i + 2], pk[4 * i + 3]};
                        ((u32x4*)o)[i] = v;
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < OUT_DW / 2; ++i) {
                        const u32x2 v = {pk[2 * i], pk[2 * i + 1]};
                        ((u32x2*)o)[i] = v;
                    }
                }
            }
        }

#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int d = 0; d < SLOT_DW; ++d) cur[j][d] = nxt[j][d];
    }
}

template <class Mma, int MT, int KT, typename OutT>
hipError_t launchOne(hipStream_t stream, const MatMulArgs& a, int numCUs)
{
    // samples per wave-iteration: as many 16-sample tiles as the register budget allows
    constexpr int NT = (MT * KT <= 8) ? 4 : (MT * KT <= 16 ? 2 : 1);
    const uint32_t tile = 16 * NT;
    const uint32_t numTiles = (a.batch + tile - 1) / tile;
    const uint32_t blocksNeeded = (numTiles + 3) / 4;
    const uint32_t blocksMax = (uint32_t)numCUs * 4u;
    const uint32_t blocks = blocksNeeded < blocksMax ? blocksNeeded : blocksMax;
    hipLaunchKernelGGL((matmulKernel<Mma, MT, KT, NT, OutT>), dim3(blocks), dim3(256), 0, stream, a);
    return hipGetLastError();
}

template <class Mma, typename OutT>
hipError_t dispatchShape(hipStream_t stream, const MatMulArgs& a, int numCUs)
{
    const uint32_t mt = optMT((uint32_t)a.m), kt = optKT((uint32_t)a.k, Mma::kEpl);
    const int MTs = mt <= 1 ? 1 : mt <= 2 ? 2 : mt <= 4 ? 4 : mt <= 8 ? 8 : 0;
    const int KTs = kt <= 1 ? 1 : kt <= 2 ? 2 : kt <= 4 ? 4 : 0;
    if (!MTs || !KTs) return hipErrorInvalidValue;
#define CV_CASE(M_, K_) \
    if (MTs == M_ && KTs == K_) return launchOne<Mma, M_, K_, OutT>(stream, a, numCUs);
    CV_CASE(1, 1) CV_CASE(1, 2) CV_CASE(1, 4)
    CV_CASE(2, 1) CV_CASE(2, 2) CV_CASE(2, 4)
    CV_CASE(4, 1) CV_CASE(4, 2) CV_CASE(4, 4)
    CV_CASE(8, 1) CV_CASE(8, 2) CV_CASE(8, 4)
#undef CV_CASE
    return hipErrorInvalidValue;
}

} // namespace

hipError_t launchMatMul(hipStream_t stream, MmaKind kind, const MatMulArgs& a, int numCUs)
{
    if (a.batch == 0) return hipSuccess;
    switch (kind) {
    case MmaKind::F16:
        return a.outCt == kF32 ? dispatchShape<F16Mma, float>(stream, a, numCUs)
                               : dispatchShape<F16Mma, half_t>(stream, a, numCUs);
    case MmaKind::Fp8AsF16:
        return a.outCt == kF32 ? dispatchShape<Fp8AsF16Mma, float>(stream, a, numCUs)
                               : dispatchShape<Fp8AsF16Mma, half_t>(stream, a, numCUs);
    case MmaKind::Fp8Native:
        return a.outCt == kF32 ? dispatchShape<Fp8NativeMma, float>(stream, a, numCUs)
                               : dispatchShape<Fp8NativeMma, half_t>(stream, a, numCUs);
    case MmaKind::I8:
        return dispatchShape<I8Mma, int32_t>(stream, a, numCUs);
    }
    return hipErrorInvalidValue;
}

} // namespace cv
