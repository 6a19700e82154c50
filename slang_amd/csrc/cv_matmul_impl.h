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
#pragma once
#include "cv_device.h"
#include "cv_kernels.h"
#include "cv_launch.h"
#include "cv_error.h"

namespace cv {
namespace {

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

template <class Mma, int MT, int KT, int NT, typename OutT, bool FAST>
__global__ __launch_bounds__(256) void matmulKernel(const MatMulArgs a)
{
    constexpr int EPL = Mma::kEpl, FD = Mma::kFD, ESZ = Mma::kEsz, RAW = Mma::kRawDW;
    constexpr int SLOT_DW = RAW * KT;         // input dwords per lane per 16-sample tile
    constexpr int ROWS = 4 * MT;              // output rows per lane
    constexpr int OUT_DW = ROWS * (int)sizeof(OutT) / 4;
    typedef typename Mma::Acc Acc;

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
    if (tile >= numTiles) return;

    const uint8_t* inLane = a.in + (size_t)colBase * ESZ;
    uint8_t* outLane = a.out + (size_t)rowBase * sizeof(OutT);
    const uint32_t lastSample = a.batch - 1;

    // One tile's input registers are loaded a whole tile ahead.  The two buffers swap roles
    // (no register copies: a copy would have to wait for the prefetch it is meant to hide).
    auto loadTile = [&](uint32_t (&buf)[NT][SLOT_DW], uint32_t t) {
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            if constexpr (FAST) {
                loadSlotsVec<SLOT_DW>(buf[j], inLane + (size_t)(t * TILE + 16 * j + n) * a.inStride);
            } else {
                const uint32_t s = min(t * TILE + 16 * j + n, lastSample);
                loadSlots<SLOT_DW>(buf[j], inLane + (size_t)s * a.inStride, validBytes, loadMode);
            }
        }
    };

    auto computeStore = [&](const uint32_t (&buf)[NT][SLOT_DW], uint32_t t0) {
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            Acc acc[MT];
#pragma unroll
            for (int t = 0; t < MT; ++t) acc[t] = biasv[t];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                uint32_t bfrag[FD];
                Mma::decode(&buf[j][kt * RAW], bfrag);
#pragma unroll
                for (int t = 0; t < MT; ++t) acc[t] = Mma::mma(afrag[t][kt], bfrag, acc[t]);
            }

            const uint32_t sample = t0 * TILE + 16 * j + n;
            uint8_t* o = outLane + (size_t)sample * a.outStride;
            uint32_t pk[OUT_DW];
            if constexpr (FAST) {
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    if constexpr (sizeof(OutT) == 2) {
                        // max on the fp32 accumulator commutes with the rounding to fp16
                        halfx2 lo, hi;
                        lo.x = (half_t)fmaxf(acc[t][0], reluFloor); lo.y = (half_t)fmaxf(acc[t][1], reluFloor);
                        hi.x = (half_t)fmaxf(acc[t][2], reluFloor); hi.y = (half_t)fmaxf(acc[t][3], reluFloor);
                        pk[2 * t] = __builtin_bit_cast(uint32_t, lo);
                        pk[2 * t + 1] = __builtin_bit_cast(uint32_t, hi);
                    } else if constexpr (Mma::kIsFloat) {
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
                        *(u32x4*)(tileOut + (size_t)srow * a.outStride + ch * 16) = v;
                    }
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                } else {
                    storeVec<OUT_DW>(o, pk);
                }
            } else {
                if (sample >= a.batch || validRows <= 0) continue;
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
                                half_t v = __builtin_bit_cast(half_t, bits);
                                if (a.accumulate) v = (half_t)((float)oe[e] + (float)v);
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
        }
    };

    uint32_t bufA[NT][SLOT_DW], bufB[NT][SLOT_DW];
    loadTile(bufA, tile);
    while (true) {
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

#ifndef CV_MATMUL_NT_SMALL
#define CV_MATMUL_NT_SMALL 2
#endif

template <int MT, int KT>
struct TileShape {
    // samples per wave-iteration: as many 16-sample tiles as the register budget allows
    static constexpr int NT = (MT * KT <= 8) ? CV_MATMUL_NT_SMALL : (MT * KT <= 16 ? 2 : 1);
};

template <class Mma, int MT, int KT, typename OutT, bool FAST>
hipError_t launchOne(hipStream_t stream, const MatMulArgs& a, int numCUs, bool tailOfStreaming = false)
{
    constexpr int NT = TileShape<MT, KT>::NT;
    // Persistent grid: exactly as many workgroups as are resident at once, so that every wave
    // strides over the same number of tiles (a partial second round would run at a fraction of
    // the occupancy).  The residency of a kernel is fixed, so it is queried once.
    const int blocksPerCU = residentBlocksPerCU<matmulKernel<Mma, MT, KT, NT, OutT, FAST>>(256);
    const uint32_t tile = 16 * NT;
    const uint32_t numTiles = (a.batch + tile - 1) / tile;
    const uint32_t blocksNeeded = (numTiles + 3) / 4;
    const uint32_t blocksMax = (uint32_t)numCUs * (uint32_t)blocksPerCU;
    const uint32_t blocks = blocksNeeded < blocksMax ? blocksNeeded : blocksMax;
    noteKernel(tailOfStreaming, "matmulKernel<%s,MT=%d,KT=%d,NT=%d,out=%dB,%s>", Mma::kName, MT, KT, NT,
               (int)sizeof(OutT), FAST ? "streaming" : "general");
    hipLaunchKernelGGL((matmulKernel<Mma, MT, KT, NT, OutT, FAST>), dim3(blocks), dim3(256), 0, stream, a);
    return hipGetLastError();
}

template <class Mma, int MT, int KT, typename OutT>
hipError_t launchShape(hipStream_t stream, const MatMulArgs& a, int numCUs)
{
    constexpr uint32_t slotBytes = Mma::kRawDW * 4 * KT;
    constexpr uint32_t tile = 16 * TileShape<MT, KT>::NT;
    const bool fast = (uint32_t)a.k == 4u * Mma::kEpl * KT && a.m == 16 * MT &&
                      a.inAlign >= (slotBytes % 16 == 0 ? 16u : 8u) &&
                      a.outAlign >= ((4 * MT * sizeof(OutT)) % 16 == 0 ? 16u : 8u) &&
                      !a.accumulate && a.act <= kActRelu;
    if (!fast) return launchOne<Mma, MT, KT, OutT, false>(stream, a, numCUs);
    // whole tiles on the streaming kernel, the ragged tail (< one tile) on the general one
    const uint32_t whole = a.batch / tile * tile;
    if (whole) {
        MatMulArgs b = a;
        b.batch = whole;
        const hipError_t e = launchOne<Mma, MT, KT, OutT, true>(stream, b, numCUs);
        if (e != hipSuccess) return e;
    }
    if (whole == a.batch) return hipSuccess;
    MatMulArgs t = a;
    t.in += (size_t)whole * a.inStride;
    t.out += (size_t)whole * a.outStride;
    t.batch = a.batch - whole;
    return launchOne<Mma, MT, KT, OutT, false>(stream, t, numCUs, whole != 0);
}

template <class Mma, typename OutT>
hipError_t dispatchShape(hipStream_t stream, const MatMulArgs& a, int numCUs)
{
    const uint32_t mt = optMT((uint32_t)a.m), kt = optKT((uint32_t)a.k, Mma::kEpl);
    const int MTs = mt <= 1 ? 1 : mt <= 2 ? 2 : mt <= 4 ? 4 : mt <= 8 ? 8 : 0;
    const int KTs = kt <= 1 ? 1 : kt <= 2 ? 2 : kt <= 4 ? 4 : 0;
    if (!MTs || !KTs) return hipErrorInvalidValue;
#define CV_CASE(M_, K_) \
    if (MTs == M_ && KTs == K_) return launchShape<Mma, M_, K_, OutT>(stream, a, numCUs);
    CV_CASE(1, 1) CV_CASE(1, 2) CV_CASE(1, 4)
    CV_CASE(2, 1) CV_CASE(2, 2) CV_CASE(2, 4)
    CV_CASE(4, 1) CV_CASE(4, 2) CV_CASE(4, 4)
    CV_CASE(8, 1) CV_CASE(8, 2) CV_CASE(8, 4)
#undef CV_CASE
    return hipErrorInvalidValue;
}

} // namespace
} // namespace cv
