// cv_device.h -- device-side building blocks shared by the gfx950 kernels.
//
// Mapping used by every kernel here: one 64-lane wavefront works on tiles of 16 samples.
// Lane l = 16*g + n belongs to sample n of the tile and to lane group g.  A vector of P
// (padded) features is spread over the wave so that group g owns the contiguous quarter
// [g*P/4, (g+1)*P/4) of it -- which is at once the B-operand register layout of
// v_mfma_*_16x16x{32,64} (k-slots of group g) and, for the result D = W . X^T, the
// accumulator layout (rows 4g..4g+3 of every 16-row tile) under the row order of
// cv_layout.h.  A layer's accumulators therefore feed the next layer's MFMA without any
// cross-lane movement.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "cv_layout.h"

namespace cv {

typedef _Float16 half_t;
typedef _Float16 halfx2 __attribute__((ext_vector_type(2)));
typedef _Float16 halfx4 __attribute__((ext_vector_type(4)));
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef int intx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

enum : int { kActNone = 0, kActRelu = 1, kActLeakyRelu = 2, kActSigmoid = 3, kActTanh = 4, kActExp = 5,
             kActSine = 6, kActSilu = 7, kActQuickGelu = 8, kActCount = 9 };

// ---- MFMA flavours ---------------------------------------------------------------------
// Each flavour describes how elements lie in memory (kEsz bytes each; kEpl k-slots per lane
// per fragment = kRawDW dwords as loaded) and in the MFMA operand registers (kFD dwords per
// fragment after decode()), the accumulator type, and D += A.B.

struct F16Mma {
    static constexpr const char* kName = "f16";
    static constexpr int kEsz = 2, kEpl = 8, kRawDW = 4, kFD = 4;
    static constexpr bool kIsFloat = true;
    typedef floatx4 Acc;
    static __device__ __forceinline__ void decode(const uint32_t* raw, uint32_t* frag)
    {
        frag[0] = raw[0]; frag[1] = raw[1]; frag[2] = raw[2]; frag[3] = raw[3];
    }
    static __device__ __forceinline__ Acc mma(const uint32_t* a, const uint32_t* b, Acc c)
    {
        u32x4 av = {a[0], a[1], a[2], a[3]}, bv = {b[0], b[1], b[2], b[3]};
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(halfx8, av),
                                                      __builtin_bit_cast(halfx8, bv), c, 0, 0, 0);
    }
};

// OCP e4m3 operands on the fp8 matrix pipeline.  Measured on gfx950: this pipeline aligns the
// products of one instruction to the largest of them and keeps about 11 bits below it, so sums
// that cancel carry an absolute error of up to ~2^-12 * sum|terms|.
struct Fp8NativeMma {
    static constexpr const char* kName = "e4m3-fp8pipe";
    static constexpr int kEsz = 1, kEpl = 8, kRawDW = 2, kFD = 2;
    static constexpr bool kIsFloat = true;
    typedef floatx4 Acc;
    static __device__ __forceinline__ void decode(const uint32_t* raw, uint32_t* frag)
    {
        frag[0] = raw[0]; frag[1] = raw[1];
    }
    static __device__ __forceinline__ Acc mma(const uint32_t* a, const uint32_t* b, Acc c)
    {
        u32x2 av = {a[0], a[1]}, bv = {b[0], b[1]};
        return __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(__builtin_bit_cast(long, av),
                                                          __builtin_bit_cast(long, bv), c, 0, 0, 0);
    }
};

// OCP e4m3 in memory, decoded (exactly: e4m3 is a subset of fp16) to fp16 operands of the
// fp16 matrix pipeline, whose accumulation is fp32-grade.  This is the flavour that meets the
// fp32-accumulated parity bar for e4m3 matrices.
struct Fp8AsF16Mma {
    static constexpr const char* kName = "e4m3-f16pipe";
    static constexpr int kEsz = 1, kEpl = 8, kRawDW = 2, kFD = 4;
    static constexpr bool kIsFloat = true;
    typedef floatx4 Acc;
    static __device__ __forceinline__ void decode(const uint32_t* raw, uint32_t* frag)
    {
        frag[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(raw[0], 1.0f, false));
        frag[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(raw[0], 1.0f, true));
        frag[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(raw[1], 1.0f, false));
        frag[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(raw[1], 1.0f, true));
    }
    static __device__ __forceinline__ Acc mma(const uint32_t* a, const uint32_t* b, Acc c)
    {
        return F16Mma::mma(a, b, c);
    }
};

// bfloat16 operands (the library's extension type CV_BFLOAT16)
struct Bf16Mma {
    static constexpr const char* kName = "bf16";
    static constexpr int kEsz = 2, kEpl = 8, kRawDW = 4, kFD = 4;
    static constexpr bool kIsFloat = true;
    typedef floatx4 Acc;
    static __device__ __forceinline__ void decode(const uint32_t* raw, uint32_t* frag)
    {
        frag[0] = raw[0]; frag[1] = raw[1]; frag[2] = raw[2]; frag[3] = raw[3];
    }
    static __device__ __forceinline__ Acc mma(const uint32_t* a, const uint32_t* b, Acc c)
    {
        typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
        u32x4 av = {a[0], a[1], a[2], a[3]}, bv = {b[0], b[1], b[2], b[3]};
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, av), __builtin_bit_cast(bf16x8, bv), c, 0, 0, 0);
    }
};

// fp32 operands on v_mfma_f32_16x16x4_f32.  A fragment keeps the 8 k-slots per lane of the 16-bit
// flavours (so the InferencingOptimal form of an fp32 matrix is the same arrangement with 4-byte
// elements): eight instructions, the s-th multiplying slot s of every lane, i.e. the four k
// values {g*GS + 8*kt + s : g = 0..3}.
struct F32Mma {
    static constexpr const char* kName = "f32";
    static constexpr int kEsz = 4, kEpl = 8, kRawDW = 8, kFD = 8;
    static constexpr bool kIsFloat = true;
    typedef floatx4 Acc;
    static __device__ __forceinline__ void decode(const uint32_t* raw, uint32_t* frag)
    {
#pragma unroll
        for (int d = 0; d < 8; ++d) frag[d] = raw[d];
    }
    static __device__ __forceinline__ Acc mma(const uint32_t* a, const uint32_t* b, Acc c)
    {
#pragma unroll
        for (int s = 0; s < 8; ++s)
            c = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, a[s]), __builtin_bit_cast(float, b[s]), c, 0, 0, 0);
        return c;
    }
};

// OCP e5m2 in memory, decoded exactly to fp16 operands: an e5m2 value is the high byte of the
// binary16 with the same value
struct Bf8AsF16Mma {
    static constexpr const char* kName = "e5m2-f16pipe";
    static constexpr int kEsz = 1, kEpl = 8, kRawDW = 2, kFD = 4;
    static constexpr bool kIsFloat = true;
    typedef floatx4 Acc;
    static __device__ __forceinline__ void decode(const uint32_t* raw, uint32_t* frag)
    {
        // v_perm_b32: selector 0x0c = constant 0, 0..3 = bytes of the second source
        frag[0] = __builtin_amdgcn_perm(0u, raw[0], 0x010c000cu);
        frag[1] = __builtin_amdgcn_perm(0u, raw[0], 0x030c020cu);
        frag[2] = __builtin_amdgcn_perm(0u, raw[1], 0x010c000cu);
        frag[3] = __builtin_amdgcn_perm(0u, raw[1], 0x030c020cu);
    }
    static __device__ __forceinline__ Acc mma(const uint32_t* a, const uint32_t* b, Acc c)
    {
        return F16Mma::mma(a, b, c);
    }
};

struct I8Mma {   // int8 x int8 -> int32
    static constexpr const char* kName = "i8";
    static constexpr int kEsz = 1, kEpl = 16, kRawDW = 4, kFD = 4;
    static constexpr bool kIsFloat = false;
    typedef intx4 Acc;
    static __device__ __forceinline__ void decode(const uint32_t* raw, uint32_t* frag)
    {
        frag[0] = raw[0]; frag[1] = raw[1]; frag[2] = raw[2]; frag[3] = raw[3];
    }
    static __device__ __forceinline__ Acc mma(const uint32_t* a, const uint32_t* b, Acc c)
    {
        intx4 av = {(int)a[0], (int)a[1], (int)a[2], (int)a[3]};
        intx4 bv = {(int)b[0], (int)b[1], (int)b[2], (int)b[3]};
        return __builtin_amdgcn_mfma_i32_16x16x64_i8(av, bv, c, 0, 0, 0);
    }
};

// ---- floating-point mode ----------------------------------------------------------------
// MODE.FP16_OVFL (hardware mode register 1, bit 23).  While it is set, conversions to fp16 and to
// fp8 clamp an out-of-range result to the largest finite value (65504 / 448) instead of producing
// inf / NaN.  Measured on gfx950: with the bit set v_cvt_scalef32_pk_fp8_f16 equals the saturating
// OCP e4m3 quantiser for every one of the 65 536 fp16 inputs (NaN aside), so the explicit clamp to
// +-448 in front of it can go.  fp32 -> fp16 conversions clamp too while it is set, which is the
// same thing for a value that is quantised to e4m3 next, but not for a kernel's fp16 output: the
// bit is cleared around those.
template <bool ON>
__device__ __forceinline__ void setFp16OverflowClamp()
{
    __builtin_amdgcn_s_setreg(1 | (23 << 6) | (0 << 11), ON ? 1 : 0);
}

// Makes `v` pass through this point of the program: nothing that computes v can sink below it and
// nothing that uses v can rise above it.  Used on both sides of a mode switch, whose ordering
// against plain arithmetic the optimiser would not keep by itself.
template <class T>
__device__ __forceinline__ void pinHere(T& v) { asm volatile("" : "+v"(v)); }

// ---- the example's input encoding ---------------------------------------------------------
// MyNetwork::encodeInput (examples/mlp-training-coopvec/network.slang:35-38) on a float2 sample
// converted to half2 (kernels.slang:19): the CoopVec<half,4> (x, y, x*x, y*y) as two packed dwords.
__device__ __forceinline__ void encodeXYSquares(float x, float y, uint32_t& xy, uint32_t& squares)
{
    const halfx2 h = {(half_t)x, (half_t)y};
    xy = __builtin_bit_cast(uint32_t, h);
    squares = __builtin_bit_cast(uint32_t, h * h);
}
__device__ __forceinline__ void encodeXYSquares(const uint8_t* sample, uint32_t& xy, uint32_t& squares)
{
    encodeXYSquares(((const float*)sample)[0], ((const float*)sample)[1], xy, squares);
}

// groundtruth(x, y) of the example (network.slang:67-75), every operation in half
__device__ __forceinline__ void exampleGroundTruth(half_t x, half_t y, half_t (&gt)[4])
{
    const half_t one = (half_t)1.f, two = (half_t)2.f, hlf = (half_t)0.5f, c12 = (half_t)1.2f;
    gt[0] = (half_t)((x + y) / (half_t)(one + (half_t)(y * y)));
    gt[1] = (half_t)((half_t)(two * x) + y);
    gt[2] = (half_t)((half_t)((half_t)(hlf * x) * x) + (half_t)(c12 * y));
    gt[3] = (half_t)(x + (half_t)((half_t)(hlf * y) * y));
}

// ---- final sum over per-workgroup partials ---------------------------------------------------
// Streamed vectors (every byte is touched once per launch) go past the caches with non-temporal
// accesses: measured on an MI355X, a plain 512 MiB copy runs at 5.5-5.8 TB/s with ordinary 16-byte
// accesses and at 6.1-6.4 TB/s with non-temporal loads and stores.  Only where one instruction of
// a wave covers whole 128-byte lines: a line fetched in two halves by two non-temporal loads is
// fetched twice (lanes reading 16 bytes at a 32-byte pitch lost 4 % with them), and non-temporal
// stores of 16-byte pieces at a 128-byte pitch ran at 0.4 TB/s where ordinary ones reach 3 TB/s.
__device__ __forceinline__ u32x4 loadStream16(const void* p) { return __builtin_nontemporal_load((const u32x4*)p); }
__device__ __forceinline__ u32x2 loadStream8(const void* p) { return __builtin_nontemporal_load((const u32x2*)p); }
__device__ __forceinline__ void storeStream16(void* p, u32x4 v) { __builtin_nontemporal_store(v, (u32x4*)p); }
__device__ __forceinline__ void storeStream8(void* p, u32x2 v) { __builtin_nontemporal_store(v, (u32x2*)p); }

// v summed over the four 16-lane groups of a wave (lanes n, n+16, n+32, n+48), in every lane.
// v_permlane16_swap / v_permlane32_swap exchange rows between two registers; fed the same value
// twice they leave each lane with both values of its pair, so the exchange costs one VALU
// instruction and no LDS round trip.  The additions are those of v += shfl_xor(v, 16);
// v += shfl_xor(v, 32) (each sum has the same two operands).
// (The second result passes through an empty asm: without it the optimiser replaces it by the first
// one when the two are added as floats.)
__device__ __forceinline__ void swapRows16(uint32_t a, uint32_t& x, uint32_t& y)
{
    const u32x2 r = __builtin_amdgcn_permlane16_swap(a, a, false, false);
    x = r.x; y = r.y;
    asm volatile("" : "+v"(y));
}
__device__ __forceinline__ void swapHalves32(uint32_t a, uint32_t& x, uint32_t& y)
{
    const u32x2 r = __builtin_amdgcn_permlane32_swap(a, a, false, false);
    x = r.x; y = r.y;
    asm volatile("" : "+v"(y));
}
__device__ __forceinline__ float sumOverGroups(float v)
{
    uint32_t x, y;
    swapRows16(__builtin_bit_cast(uint32_t, v), x, y);
    v = __builtin_bit_cast(float, x) + __builtin_bit_cast(float, y);
    swapHalves32(__builtin_bit_cast(uint32_t, v), x, y);
    return __builtin_bit_cast(float, x) + __builtin_bit_cast(float, y);
}
__device__ __forceinline__ int sumOverGroups(int v)
{
    uint32_t x, y;
    swapRows16((uint32_t)v, x, y);
    swapHalves32(x + y, x, y);
    return (int)(x + y);
}

// Used by the second-stage kernels of the deterministic reductions.  A workgroup of kReduceWaves
// waves owns 64 consecutive values; every wave sums a contiguous share of the partials of the
// calling lane's value (src[b * stride], b < numPartials) with sixteen independent loads in
// flight, then wave 0 adds the wave sums in a fixed order.  Returns true in the lanes of wave 0
// (with the total); all threads of the workgroup must call it.
constexpr int kReduceWaves = 16;
__device__ __forceinline__ bool sumPartials(const float* src, size_t stride, uint32_t numPartials, bool inRange,
                                            float* red /* shared, kReduceWaves * 64 floats */, float& total)
{
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63u;
    const uint32_t per = (numPartials + kReduceWaves - 1u) / kReduceWaves;
    const uint32_t b0 = min(wave * per, numPartials), b1 = min(b0 + per, numPartials);
    float c = 0.f;
    if (inRange) {
        uint32_t b = b0;
        for (; b + 16 <= b1; b += 16) {
            float v[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) v[u] = src[(size_t)(b + u) * stride];
#pragma unroll
            for (int u = 0; u < 16; ++u) c += v[u];
        }
        for (; b < b1; ++b) c += src[(size_t)b * stride];
    }
    red[wave * 64 + lane] = c;
    __syncthreads();
    if (wave != 0) return false;
    float s = red[lane];
#pragma unroll
    for (int w = 1; w < kReduceWaves; ++w) s += red[w * 64 + lane];
    total = s;
    return true;
}

// ---- scalar helpers ---------------------------------------------------------------------

__device__ __forceinline__ float loadAsFloat(const uint8_t* p, int ct)
{
    switch (ct) {
    case kF16: return (float)*(const half_t*)p;
    case kF32: return *(const float*)p;
    case kBF16: return __builtin_bit_cast(float, (uint32_t)*(const uint16_t*)p << 16);
    }
    return 0.f;
}

// bfloat16 as a result element (conversions round to nearest even: v_cvt_pk_bf16_f32)
typedef __bf16 bf16_t;
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// fp32 -> OCP e4m3, saturating, round to nearest even; two values per call (bytes 0,1)
__device__ __forceinline__ uint32_t packE4M3Sat(float a, float b)
{
    // v_cvt_pk_fp8_f32 rounds to nearest even and produces NaN above the finite range:
    // clamp to +-448 first (v_med3 keeps NaN as NaN on the min/max path is not guaranteed,
    // so NaN inputs are not supported by the fused paths).
    a = __builtin_fminf(__builtin_fmaxf(a, -448.f), 448.f);
    b = __builtin_fminf(__builtin_fmaxf(b, -448.f), 448.f);
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false) & 0xffffu;
}

// four fp16 values (two packed dwords) -> four OCP e4m3 bytes, saturating at +-448, nearest even
// (v_cvt_scalef32_pk_fp8_f16 rounds like the fp32 route for every fp16 input within the clamp)
__device__ __forceinline__ uint32_t quantE4M3x4Sat(uint32_t h01bits, uint32_t h23bits)
{
    typedef short shortx2 __attribute__((ext_vector_type(2)));
    const halfx2 lim = {(half_t)448.f, (half_t)448.f};
    const halfx2 h01 = __builtin_elementwise_min(__builtin_elementwise_max(__builtin_bit_cast(halfx2, h01bits), -lim), lim);
    const halfx2 h23 = __builtin_elementwise_min(__builtin_elementwise_max(__builtin_bit_cast(halfx2, h23bits), -lim), lim);
    shortx2 r = __builtin_bit_cast(shortx2, h01);
    r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r, h01, 1.0f, false);
    r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r, h23, 1.0f, true);
    return __builtin_bit_cast(uint32_t, r);
}

// The neural module's smooth activations (source/standard-modules/neural/activations.slang:88-233)
// in fp32.  Sigmoid-like ones keep the source's branch that makes the exp() argument <= 0.
__device__ __forceinline__ float smoothActivation(float x, int act)
{
    switch (act) {
    case kActTanh: return tanhf(x);
    case kActExp: return expf(x);
    case kActSine: return sinf(x);
    case kActSigmoid: {
        const float ex = expf(x >= 0.f ? -x : x);
        return x >= 0.f ? 1.f / (1.f + ex) : ex / (1.f + ex); }
    case kActSilu: {
        const float ex = expf(x >= 0.f ? -x : x);
        return x >= 0.f ? x / (1.f + ex) : x * ex / (1.f + ex); }
    case kActQuickGelu: {
        const float sx = 1.702f * x;
        const float ex = expf(sx >= 0.f ? -sx : sx);
        return sx >= 0.f ? x / (1.f + ex) : x * ex / (1.f + ex); }
    }
    return x;
}

// activation on a value already rounded to fp16 (the carrier type is CoopVec<half>)
__device__ __forceinline__ half_t activateHalf(half_t z, int act, float slope)
{
    if (act == kActRelu) return z > (half_t)0 ? z : (half_t)0;
    if (act == kActLeakyRelu) {
        const half_t zs = (half_t)((float)z * slope);   // exact product, one rounding
        return z >= zs ? z : zs;
    }
    if (act >= kActSigmoid) return (half_t)smoothActivation((float)z, act);
    return z;
}

} // namespace cv
