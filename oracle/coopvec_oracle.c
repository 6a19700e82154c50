/*
 * coopvec_oracle.c -- CPU oracle for the cooperative-vector operators.
 *
 * TEST INFRASTRUCTURE ONLY: the checker for tests, the smoke check and the benchmark's
 * cpu_baseline leg.  The shipped library never links or calls it.  See coopvec_oracle.h.
 *
 * Parity status per function family:
 *   cvo_f32_to_f16_*, cvo_f16_to_f32 : pinned (IEEE 754 exhaustively against numpy; the
 *       software rule against the points the prelude's own algorithm fixes).
 *   cvo_*e4m3*                        : pinned (OCP FP8 spec table, reference points
 *       tests/hlsl-intrinsic/scalar-fp8.slang:24-43, substandard-fp-folding.slang:14-33).
 *   cvo_slang_*                       : pinned (every golden of tests/cooperative-vector/
 *       matrix-mul*.slang, outer-product.slang, reduce-sum-accumulate*.slang).
 *   cvo_ref_*                         : pinned (same goldens, fp64 brute force, closed forms
 *       of tests/neural/basic-ilayer-ffn-{forward,backward}-test.slang, finite differences).
 *   cvo_slang_adam_step               : pinned by multi-step closed forms of Adam (constant
 *       gradient, impulse response, iteration count, NaN/Inf rules); the reference has no golden.
 *   cvo_layout_* for the two Optimal layouts : PARITY UNPINNED against the reference (the
 *       reference delegates those layouts to the vendor driver); pinned only by invariants.
 */
#include "coopvec_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ===================================================================================== */
/* numerics                                                                              */
/* ===================================================================================== */

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* IEEE 754 binary32 -> binary16, round to nearest even. */
uint16_t cvo_f32_to_f16_rne(float f)
{
    uint32_t x = f32_bits(f);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? (0x0200u | ((ax >> 13) & 0x3ffu)) : 0u));
    if (ax >= 0x477ff000u) /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7c00u);
    if (ax < 0x33000001u) /* <= 2^-25 rounds to zero (2^-25 itself is a tie to even = 0) */
        return (uint16_t)sign;
    int e = (int)(ax >> 23) - 127;
    uint32_t m = (ax & 0x007fffffu) | 0x00800000u; /* 24-bit significand */
    int shift;                                     /* bits to drop */
    uint32_t he;
    if (e < -14) { shift = 13 + (-14 - e); he = 0; }        /* subnormal half */
    else         { shift = 13;             he = (uint32_t)(e + 15); }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half_ulp = 1u << (shift - 1);
    if (rem > half_ulp || (rem == half_ulp && (q & 1u))) q++;
    /* q holds the implicit bit for normals: (he<<10) + (q - 0x400) == ((he-1)<<10) + q */
    uint32_t out = (he == 0) ? q : (((he - 1u) << 10) + q);
    return (uint16_t)(sign | out);
}

/* The prelude's software conversion, restated from
 * prelude/slang-cpp-scalar-intrinsics.h:563-613 (same algorithm as
 * source/core/slang-math.h:212-236 and mlp-training-coopvec.cpp:400-425):
 * keeps one guard bit and adds it back, so exact ties round away from zero and
 * everything below 2^-24 flushes to zero. */
uint16_t cvo_f32_to_f16_slang(float f)
{
    uint32_t in = f32_bits(f);
    uint32_t bits = (in >> 16) & 0x8000u;
    uint32_t m = (in >> 12) & 0x07ffu;
    uint32_t e = (in >> 23) & 0xffu;
    if (e < 103u) return (uint16_t)bits;
    if (e == 0xffu) {
        m >>= 1;
        m += (uint32_t)(m == 0 && (in & 0x007fffffu));
        return (uint16_t)(bits | 0x7c00u | m);
    }
    if (e > 142u) return (uint16_t)(bits | 0x7c00u);
    if (e < 113u) {
        m |= 0x0800u;
        bits |= (m >> (114u - e)) + ((m >> (113u - e)) & 1u);
        return (uint16_t)bits;
    }
    bits |= ((e - 112u) << 10) | (m >> 1);
    bits += m & 1u;
    return (uint16_t)bits;
}

float cvo_f16_to_f32(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu;
    uint32_t m = h & 0x3ffu;
    if (e == 0) {
        if (m == 0) return bits_f32(sign);
        /* subnormal: m * 2^-24 */
        float v = (float)m * (1.0f / 16777216.0f);
        return (sign ? -v : v);
    }
    if (e == 0x1f) return bits_f32(sign | 0x7f800000u | (m << 13));
    return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
}

/* OCP 8-bit float E4M3 (bias 7, no infinities, S.1111.111 = NaN, max finite 448 = 0x7E):
 * saturating conversion, round to nearest even, NaN stays NaN. */
uint8_t cvo_f32_to_e4m3_sat(float f)
{
    uint32_t x = f32_bits(f);
    uint8_t sign = (uint8_t)((x >> 24) & 0x80u);
    uint32_t ax = x & 0x7fffffffu;
    if (ax > 0x7f800000u) return (uint8_t)(sign | 0x7fu);   /* NaN */
    float a = bits_f32(ax);
    if (a >= 448.0f) return (uint8_t)(sign | 0x7eu);        /* saturate (also +-inf) */
    /* spacing: normals 2^(e-3) for e>=-6; subnormals 2^-9 */
    int e;
    (void)frexpf(a, &e);        /* a = m*2^e, m in [0.5,1)  ->  floor(log2 a) = e-1 */
    int le = e - 1;
    if (a == 0.0f) return sign;
    if (le < -6) le = -6;
    float ulp = ldexpf(1.0f, le - 3);
    float qf = a / ulp;         /* exact: power-of-two scaling */
    float fl = floorf(qf);
    float rem = qf - fl;
    uint32_t q = (uint32_t)fl;
    if (rem > 0.5f || (rem == 0.5f && (q & 1u))) q++;
    /* q in [0,16]: value = q * ulp */
    uint32_t out;
    if (le == -6 && q < 8u) out = q;                               /* subnormal or zero */
    else {
        if (q == 16u) { q = 8u; le++; }
        out = ((uint32_t)(le + 7) << 3) | (q - 8u);
    }
    if (out > 0x7eu) out = 0x7eu;
    return (uint8_t)(sign | out);
}

float cvo_e4m3_to_f32(uint8_t b)
{
    uint32_t e = (b >> 3) & 0xfu, m = b & 7u;
    float v;
    if (e == 0xfu && m == 7u) return bits_f32(((uint32_t)(b & 0x80u) << 24) | 0x7fc00000u);
    if (e == 0) v = ldexpf((float)m, -9);
    else        v = ldexpf((float)(8u + m), (int)e - 10);
    return (b & 0x80u) ? -v : v;
}

/* ===================================================================================== */
/* type tables, hlsl.meta.slang:32577-32670                                              */
/* ===================================================================================== */

int cvo_component_packing_factor(int ct)
{
    return (ct == CVO_SINT8_PACKED || ct == CVO_UINT8_PACKED) ? 4 : 1;
}

int cvo_component_scalar_type(int ct)
{
    switch (ct) { /* values of SLANG_SCALAR_TYPE_*, include/slang.h:2139-2157 */
    case CVO_FLOAT_E4M3: return 17;
    case CVO_FLOAT_E5M2: return 18;
    case CVO_FLOAT16: return 7;
    case CVO_FLOAT32: return 8;
    case CVO_FLOAT64: return 9;
    case CVO_SINT8: case CVO_SINT8_PACKED: return 10;
    case CVO_SINT16: return 12;
    case CVO_SINT32: return 3;
    case CVO_SINT64: return 5;
    case CVO_UINT8: case CVO_UINT8_PACKED: return 11;
    case CVO_UINT16: return 13;
    case CVO_UINT32: return 4;
    case CVO_UINT64: return 6;
    }
    return -1;
}

/* No case for the two fp8 types: the fallback static_asserts on them (:32666-32668). */
int cvo_component_type_stride(int ct)
{
    switch (ct) {
    case CVO_FLOAT16: return 2;
    case CVO_FLOAT32: return 4;
    case CVO_FLOAT64: return 8;
    case CVO_SINT8: return 1;
    case CVO_SINT16: return 2;
    case CVO_SINT32: return 4;
    case CVO_SINT8_PACKED: return 4;
    case CVO_SINT64: return 8;
    case CVO_UINT8: return 1;
    case CVO_UINT16: return 2;
    case CVO_UINT32: return 4;
    case CVO_UINT8_PACKED: return 4;
    case CVO_UINT64: return 8;
    }
    return -1;
}

/* storage size of one element of a component type in this library's buffers (fp8 = 1) */
static int elem_size(int ct)
{
    switch (ct) {
    case CVO_FLOAT_E4M3: case CVO_FLOAT_E5M2: case CVO_SINT8: case CVO_UINT8: return 1;
    case CVO_FLOAT16: case CVO_SINT16: case CVO_UINT16: case CVO_BFLOAT16: return 2;
    case CVO_FLOAT32: case CVO_SINT32: case CVO_UINT32: case CVO_SINT8_PACKED:
    case CVO_UINT8_PACKED: return 4;
    case CVO_FLOAT64: case CVO_SINT64: case CVO_UINT64: return 8;
    }
    return -1;
}

/* ===================================================================================== */
/* Slang CPU-target semantics                                                            */
/* ===================================================================================== */

/* A value of the CoopVec element type T.  T is one of FLOAT16 (bits in .h), FLOAT32, FLOAT64,
 * SINT32, UINT32, SINT64, UINT64 (the integer pairs share their two's-complement bits). */
typedef union { uint16_t h; float f; int32_t i; uint32_t u; double d; int64_t i64; uint64_t u64; } tval;

static inline int t_supported(int T)
{
    return T == CVO_FLOAT16 || T == CVO_FLOAT32 || T == CVO_SINT32 || T == CVO_UINT32 ||
           T == CVO_FLOAT64 || T == CVO_SINT64 || T == CVO_UINT64;
}
static inline int t_size(int T)
{
    return T == CVO_FLOAT16 ? 2 : (T == CVO_FLOAT64 || T == CVO_SINT64 || T == CVO_UINT64) ? 8 : 4;
}

static inline uint16_t to_half(float f, int halfMode)
{
    return halfMode == CVO_HALF_SLANG_SOFT ? cvo_f32_to_f16_slang(f) : cvo_f32_to_f16_rne(f);
}

/* load<Wt>(p) then __arithmetic_cast<T>.  Wt is a scalar component type.  A source value is held as a
 * double (every half / float / double exactly), as an int64, or as a uint64 (UINT64 sources). */
static inline __attribute__((always_inline)) tval
load_cast(const uint8_t* p, int Wt, int T, int halfMode, int* ok)
{
    tval r; r.u64 = 0;
    int kind = 0;   /* 0: signed integer in `is`, 1: unsigned 64-bit in `us`, 2: float in `fs` */
    double fs = 0.0; int64_t is = 0; uint64_t us = 0;
    switch (Wt) {
    case CVO_FLOAT16: { uint16_t h; memcpy(&h, p, 2); fs = cvo_f16_to_f32(h); kind = 2; break; }
    case CVO_FLOAT32: { float f; memcpy(&f, p, 4); fs = f; kind = 2; break; }
    case CVO_FLOAT64: { memcpy(&fs, p, 8); kind = 2; break; }
    case CVO_SINT8: case CVO_SINT8_PACKED: { int8_t v; memcpy(&v, p, 1); is = v; break; }
    case CVO_UINT8: case CVO_UINT8_PACKED: { uint8_t v; memcpy(&v, p, 1); is = v; break; }
    case CVO_SINT16: { int16_t v; memcpy(&v, p, 2); is = v; break; }
    case CVO_UINT16: { uint16_t v; memcpy(&v, p, 2); is = v; break; }
    case CVO_SINT32: { int32_t v; memcpy(&v, p, 4); is = v; break; }
    case CVO_UINT32: { uint32_t v; memcpy(&v, p, 4); is = v; break; }
    case CVO_SINT64: { memcpy(&is, p, 8); break; }
    case CVO_UINT64: { memcpy(&us, p, 8); kind = 1; break; }
    default: *ok = 0; return r;
    }
    switch (T) {
    case CVO_FLOAT16: r.h = to_half(kind == 2 ? (float)fs : kind == 1 ? (float)us : (float)is, halfMode); break;
    case CVO_FLOAT32: r.f = kind == 2 ? (float)fs : kind == 1 ? (float)us : (float)is; break;
    case CVO_FLOAT64: r.d = kind == 2 ? fs : kind == 1 ? (double)us : (double)is; break;
    case CVO_SINT32:  r.i = kind == 2 ? (int32_t)fs : kind == 1 ? (int32_t)us : (int32_t)is; break;
    case CVO_UINT32:  r.u = kind == 2 ? (uint32_t)fs : kind == 1 ? (uint32_t)us : (uint32_t)is; break;
    case CVO_SINT64:  r.i64 = kind == 2 ? (int64_t)fs : kind == 1 ? (int64_t)us : is; break;
    case CVO_UINT64:  r.u64 = kind == 2 ? (uint64_t)fs : kind == 1 ? us : (uint64_t)is; break;
    default: *ok = 0;
    }
    return r;
}

static inline __attribute__((always_inline)) tval t_mul(tval a, tval b, int T, int halfMode)
{
    tval r; r.u64 = 0;
    switch (T) {
    case CVO_FLOAT16: r.h = to_half(cvo_f16_to_f32(a.h) * cvo_f16_to_f32(b.h), halfMode); break;
    case CVO_FLOAT32: r.f = a.f * b.f; break;
    case CVO_FLOAT64: r.d = a.d * b.d; break;
    case CVO_SINT64: case CVO_UINT64: r.u64 = a.u64 * b.u64; break;
    default:          r.u = a.u * b.u; break; /* two's complement wrap for both int types */
    }
    return r;
}

static inline __attribute__((always_inline)) tval t_add(tval a, tval b, int T, int halfMode)
{
    tval r; r.u64 = 0;
    switch (T) {
    case CVO_FLOAT16: r.h = to_half(cvo_f16_to_f32(a.h) + cvo_f16_to_f32(b.h), halfMode); break;
    case CVO_FLOAT32: r.f = a.f + b.f; break;
    case CVO_FLOAT64: r.d = a.d + b.d; break;
    case CVO_SINT64: case CVO_UINT64: r.u64 = a.u64 + b.u64; break;
    default:          r.u = a.u + b.u; break;
    }
    return r;
}

static inline void t_store(void* dst, int idx, tval v, int T)
{
    int sz = t_size(T);
    if (sz == 2) memcpy((uint8_t*)dst + 2 * idx, &v.h, 2);
    else if (sz == 8) memcpy((uint8_t*)dst + 8 * (size_t)idx, &v.u64, 8);
    else memcpy((uint8_t*)dst + 4 * idx, &v.u, 4);
}
static inline tval t_load(const void* src, int idx, int T)
{
    tval v; v.u64 = 0;
    int sz = t_size(T);
    if (sz == 2) memcpy(&v.h, (const uint8_t*)src + 2 * idx, 2);
    else if (sz == 8) memcpy(&v.u64, (const uint8_t*)src + 8 * (size_t)idx, 8);
    else memcpy(&v.u, (const uint8_t*)src + 4 * idx, 4);
    return v;
}

#define CVO_MAX_DIM 4096

/* hlsl.meta.slang:32835-32912 (matmul) followed by :33055-33100 (bias). */
static inline __attribute__((always_inline)) int
slang_matmul_impl(const void* input, int U, int packedK, int inInterp, int k,
                  void* result, int T, int M,
                  const uint8_t* mat, int32_t matOff, int matInterp,
                  int layout, int transpose, uint32_t stride,
                  const uint8_t* bias, int32_t biasOff, int biasInterp,
                  int accumulate, int halfMode)
{
    int ok = 1;
    if (!t_supported(T) || k < 0 || k > CVO_MAX_DIM || M < 0 || M > CVO_MAX_DIM) return -1;
    int wsz = cvo_component_type_stride(matInterp);
    if (wsz < 0 || cvo_component_packing_factor(matInterp) != 1) return -1;   /* :32803 */
    int packed = cvo_component_packing_factor(inInterp) != 1;
    if (!packed && k != packedK) return -1;                                   /* :32798 */
    tval v[CVO_MAX_DIM];
    if (k == packedK) {                                                       /* :32839-32843 */
        int usz = elem_size(U);
        if (usz < 0) return -1;
        for (int i = 0; i < k; ++i)
            v[i] = load_cast((const uint8_t*)input + (size_t)i * usz, U, T, halfMode, &ok);
    } else {                                                                  /* :32844-32856 */
        if (k != packedK * 4) return -1;
        if (U != CVO_UINT32 && U != CVO_SINT32) return -1;
        for (int i = 0; i < k; ++i) {
            int32_t n; memcpy(&n, (const uint8_t*)input + 4 * (i / 4), 4);
            int8_t s = (int8_t)((n >> ((i % 4) * 8)) & 0xff);
            v[i] = load_cast((const uint8_t*)&s, CVO_SINT8, T, halfMode, &ok);
        }
    }
    int swap = (transpose != 0) ^ (layout == CVO_COLUMN_MAJOR);               /* :32862-32863 */
    for (int i = 0; i < M; ++i) {
        tval r; r.u64 = 0;                                 /* CoopVec<T,M>(0): +0 in every T */
        for (int j = 0; j < k; ++j) {
            int row = swap ? j : i;
            int col = swap ? i : j;
            int32_t off = matOff + (int32_t)(row * stride + col * (uint32_t)wsz);   /* :32864 */
            tval w = load_cast(mat + off, matInterp, T, halfMode, &ok);
            r = t_add(r, t_mul(w, v[j], T, halfMode), T, halfMode);           /* :32869 */
        }
        if (biasInterp >= 0) {
            int bsz = cvo_component_type_stride(biasInterp);
            if (bsz < 0 || cvo_component_packing_factor(biasInterp) != 1) return -1;
            tval b = load_cast(bias + biasOff + i * bsz, biasInterp, T, halfMode, &ok);
            r = t_add(r, b, T, halfMode);                                     /* :33057-33061 */
        }
        if (accumulate)                                   /* this = this + matmul(...) :31510 */
            r = t_add(t_load(result, i, T), r, T, halfMode);
        t_store(result, i, r, T);
    }
    return ok ? 0 : -1;
}

int cvo_slang_matmul(const void* input, int inputType, int packedK, int inputInterp, int k,
                     void* result, int resultType, int M,
                     const void* matrix, int32_t matrixOffset, int matrixInterp,
                     int layout, int transpose, uint32_t matrixStride,
                     const void* bias, int32_t biasOffset, int biasInterp,
                     int accumulate, int halfMode)
{
    return slang_matmul_impl(input, inputType, packedK, inputInterp, k, result, resultType, M,
                             (const uint8_t*)matrix, matrixOffset, matrixInterp, layout,
                             transpose, matrixStride, (const uint8_t*)bias, biasOffset,
                             biasInterp, accumulate, halfMode);
}

/* hlsl.meta.slang:33261-33315.  a and b share the element type T; the product is formed in T,
 * cast to the matrix interpretation and added non-atomically. */
int cvo_slang_outer_product_accumulate(const void* a, int M, const void* b, int N, int T,
                                       void* matrix, int32_t matOff, uint32_t stride,
                                       int layout, int matInterp, int halfMode)
{
    if (!t_supported(T)) return -1;
    int wsz = cvo_component_type_stride(matInterp);
    if (wsz < 0 || cvo_component_packing_factor(matInterp) != 1) return -1;
    uint8_t* mat = (uint8_t*)matrix;
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j) {
            tval p = t_mul(t_load(a, i, T), t_load(b, j, T), T, halfMode);     /* :33266 */
            int row = (layout == CVO_COLUMN_MAJOR) ? j : i;                    /* :33267-33268 */
            int col = (layout == CVO_COLUMN_MAJOR) ? i : j;
            uint8_t* dst = mat + matOff + (int32_t)(row * stride + col * (uint32_t)wsz);
            float pf = 0.f; int64_t pi = 0; int pIsFloat = (T == CVO_FLOAT16 || T == CVO_FLOAT32);
            if (T == CVO_FLOAT16) pf = cvo_f16_to_f32(p.h);
            else if (T == CVO_FLOAT32) pf = p.f;
            else if (T == CVO_SINT32) pi = p.i;
            else pi = p.u;
            switch (matInterp) {                                               /* :33271-33312 */
            case CVO_FLOAT16: {
                uint16_t cur; memcpy(&cur, dst, 2);
                uint16_t add = to_half(pIsFloat ? pf : (float)pi, halfMode);
                uint16_t nv = to_half(cvo_f16_to_f32(cur) + cvo_f16_to_f32(add), halfMode);
                memcpy(dst, &nv, 2); break; }
            case CVO_FLOAT32: {
                float cur; memcpy(&cur, dst, 4);
                cur = cur + (pIsFloat ? pf : (float)pi);
                memcpy(dst, &cur, 4); break; }
            case CVO_SINT32: case CVO_UINT32: {
                uint32_t cur; memcpy(&cur, dst, 4);
                cur += pIsFloat ? (uint32_t)(int32_t)pf : (uint32_t)pi;
                memcpy(dst, &cur, 4); break; }
            case CVO_SINT8: case CVO_UINT8: {
                uint8_t cur; memcpy(&cur, dst, 1);
                cur = (uint8_t)(cur + (pIsFloat ? (uint8_t)(int8_t)pf : (uint8_t)pi));
                memcpy(dst, &cur, 1); break; }
            default: return -1;
            }
        }
    return 0;
}

/* hlsl.meta.slang:33344-33352: destination element type is T itself. */
int cvo_slang_reduce_sum_accumulate(const void* v, int N, int T, void* buffer, int32_t offset,
                                    int halfMode)
{
    if (!t_supported(T)) return -1;
    uint8_t* dst = (uint8_t*)buffer + offset;
    for (int i = 0; i < N; ++i)
        t_store(dst, i, t_add(t_load(dst, i, T), t_load(v, i, T), T, halfMode), T);
    return 0;
}

/* Specialised bodies so that the constant arguments fold the way slangc's constexpr
 * parameters do (interpretations, layout, stride are compile-time constants in Slang). */
static int dispatch_f16_rowmajor(uint32_t g0, uint32_t g1, uint32_t count, const uint8_t* in,
                                 size_t inStride, int k, uint8_t* out, size_t outStride, int M,
                                 const uint8_t* mat, int32_t matOff, uint32_t stride,
                                 const uint8_t* bias, int32_t biasOff, int hasBias, int halfMode)
{
    for (uint32_t g = g0; g < g1; ++g)
        for (uint32_t t = 0; t < 256; ++t) {
            uint32_t tid = g * 256u + t;
            if (tid >= count) continue;
            int rc = slang_matmul_impl(in + (size_t)tid * inStride, CVO_FLOAT16, k, CVO_FLOAT16, k,
                                       out + (size_t)tid * outStride, CVO_FLOAT16, M, mat, matOff,
                                       CVO_FLOAT16, CVO_ROW_MAJOR, 0, stride, bias, biasOff,
                                       hasBias ? CVO_FLOAT16 : -1, 0, halfMode);
            if (rc) return rc;
        }
    return 0;
}

static int dispatch_i8packed(uint32_t g0, uint32_t g1, uint32_t count, const uint8_t* in,
                             size_t inStride, int k, uint8_t* out, size_t outStride, int M,
                             const uint8_t* mat, int32_t matOff, int layout, uint32_t stride,
                             const uint8_t* bias, int32_t biasOff, int hasBias)
{
    for (uint32_t g = g0; g < g1; ++g)
        for (uint32_t t = 0; t < 256; ++t) {
            uint32_t tid = g * 256u + t;
            if (tid >= count) continue;
            int rc = slang_matmul_impl(in + (size_t)tid * inStride, CVO_UINT32, k / 4,
                                       CVO_SINT8_PACKED, k, out + (size_t)tid * outStride,
                                       CVO_SINT32, M, mat, matOff, CVO_SINT8, layout, 0, stride,
                                       bias, biasOff, hasBias ? CVO_SINT32 : -1, 0, CVO_HALF_RNE);
            if (rc) return rc;
        }
    return 0;
}

int cvo_slang_dispatch_matmul_add(uint32_t startGroup, uint32_t endGroup, uint32_t count,
                                  const void* input, size_t inputStride, int inputType,
                                  int packedK, int inputInterp, int k,
                                  void* output, size_t outputStride, int resultType, int M,
                                  const void* matrix, int32_t matrixOffset, int matrixInterp,
                                  int layout, int transpose, uint32_t matrixStride,
                                  const void* bias, int32_t biasOffset, int biasInterp,
                                  int halfMode)
{
    const uint8_t* in = (const uint8_t*)input; uint8_t* out = (uint8_t*)output;
    if (inputType == CVO_FLOAT16 && inputInterp == CVO_FLOAT16 && matrixInterp == CVO_FLOAT16 &&
        resultType == CVO_FLOAT16 && !transpose && layout != CVO_COLUMN_MAJOR &&
        (biasInterp < 0 || biasInterp == CVO_FLOAT16))
        return dispatch_f16_rowmajor(startGroup, endGroup, count, in, inputStride, k, out,
                                     outputStride, M, (const uint8_t*)matrix, matrixOffset,
                                     matrixStride, (const uint8_t*)bias, biasOffset,
                                     biasInterp >= 0, halfMode);
    if (inputType == CVO_UINT32 && inputInterp == CVO_SINT8_PACKED && matrixInterp == CVO_SINT8 &&
        resultType == CVO_SINT32 && !transpose && k == 4 * packedK &&
        (biasInterp < 0 || biasInterp == CVO_SINT32))
        return dispatch_i8packed(startGroup, endGroup, count, in, inputStride, k, out,
                                 outputStride, M, (const uint8_t*)matrix, matrixOffset, layout,
                                 matrixStride, (const uint8_t*)bias, biasOffset, biasInterp >= 0);
    for (uint32_t g = startGroup; g < endGroup; ++g)
        for (uint32_t t = 0; t < 256; ++t) {
            uint32_t tid = g * 256u + t;
            if (tid >= count) continue;
            int rc = slang_matmul_impl(in + (size_t)tid * inputStride, inputType, packedK,
                                       inputInterp, k, out + (size_t)tid * outputStride,
                                       resultType, M, (const uint8_t*)matrix, matrixOffset,
                                       matrixInterp, layout, transpose, matrixStride,
                                       (const uint8_t*)bias, biasOffset, biasInterp, 0, halfMode);
            if (rc) return rc;
        }
    return 0;
}

/* ===================================================================================== */
/* matrix layouts                                                                        */
/* ===================================================================================== */

/* k-slots one lane contributes to one MFMA fragment, by storage class */
static int frag_elems_per_lane(int ct)
{
    switch (ct) {
    case CVO_SINT8: case CVO_UINT8: return 16;        /* v_mfma_i32_16x16x64_i8: 16 B per lane */
    case CVO_FLOAT_E4M3: case CVO_FLOAT_E5M2: return 8; /* v_mfma_f32_16x16x32_fp8: 8 B */
    case CVO_FLOAT16: return 8;                         /* v_mfma_f32_16x16x32_f16: 16 B */
    case CVO_BFLOAT16: return 8;                        /* v_mfma_f32_16x16x32_bf16: 16 B */
    case CVO_FLOAT32: return 8;
    }
    return -1;
}

static int layout_ct_ok(int ct, int layout)
{
    if (elem_size(ct) < 0 || cvo_component_packing_factor(ct) != 1) return 0;
    if (layout == CVO_INFERENCING_OPTIMAL) return frag_elems_per_lane(ct) > 0;
    if (layout == CVO_TRAINING_OPTIMAL) return ct == CVO_FLOAT16 || ct == CVO_FLOAT32 || ct == CVO_BFLOAT16;
    return layout == CVO_ROW_MAJOR || layout == CVO_COLUMN_MAJOR;
}

size_t cvo_layout_matrix_size(uint32_t rows, uint32_t cols, int ct, int layout, size_t stride)
{
    if (rows == 0 || cols == 0 || !layout_ct_ok(ct, layout)) return 0;
    size_t esz = (size_t)elem_size(ct);
    switch (layout) {
    case CVO_ROW_MAJOR: {
        size_t s = stride ? stride : cols * esz;
        if (s < cols * esz) return 0;
        return (size_t)(rows - 1) * s + cols * esz; }
    case CVO_COLUMN_MAJOR: {
        size_t s = stride ? stride : rows * esz;
        if (s < rows * esz) return 0;
        return (size_t)(cols - 1) * s + rows * esz; }
    case CVO_INFERENCING_OPTIMAL: {
        size_t epl = (size_t)frag_elems_per_lane(ct);
        size_t mt = (rows + 15) / 16;
        size_t gs = ((cols + 15) / 16) * 4;          /* k-slots owned by one 16-lane group */
        size_t kt = (gs + epl - 1) / epl;
        return mt * kt * 64 * epl * esz; }
    case CVO_TRAINING_OPTIMAL:
        return (size_t)((rows + 15) / 16) * ((cols + 15) / 16) * 256 * esz;
    }
    return 0;
}

int64_t cvo_layout_elem_offset(uint32_t rows, uint32_t cols, int ct, int layout, size_t stride,
                               uint32_t r, uint32_t c)
{
    if (rows == 0 || cols == 0 || r >= rows || c >= cols || !layout_ct_ok(ct, layout)) return -1;
    size_t esz = (size_t)elem_size(ct);
    switch (layout) {
    case CVO_ROW_MAJOR:    return (int64_t)((size_t)r * (stride ? stride : cols * esz) + c * esz);
    case CVO_COLUMN_MAJOR: return (int64_t)((size_t)c * (stride ? stride : rows * esz) + r * esz);
    case CVO_INFERENCING_OPTIMAL: {
        /* Fragment-native tiles for D = W . X^T with W as the MFMA A operand.
         * Fragment (t,kt) holds, for lane = 16*g + i, EPL consecutive k-slots.
         *   row r  <-> group rg = r / (4*MT), tile t = (r % (4*MT)) / 4, i = 4*rg + r % 4
         *   col c  <-> group g = c / GS, slot q = c % GS, kt = q / EPL, s = q % EPL
         * so that lane group g owns the contiguous quarter [g*GS,(g+1)*GS) of the input vector
         * and the contiguous quarter [g*4MT,(g+1)*4MT) of the output vector. */
        size_t epl = (size_t)frag_elems_per_lane(ct);
        size_t mt = (rows + 15) / 16, mt4 = 4 * mt;
        size_t gs = ((cols + 15) / 16) * 4;
        size_t kt = (gs + epl - 1) / epl;
        size_t rg = r / mt4, rem = r % mt4, t = rem / 4, i = 4 * rg + rem % 4;
        size_t g = c / gs, q = c % gs, k = q / epl, s = q % epl;
        size_t lane = 16 * g + i;
        return (int64_t)((((t * kt + k) * 64 + lane) * epl + s) * esz); }
    case CVO_TRAINING_OPTIMAL: {
        /* MFMA accumulator-native 16x16 tiles, tile grid row-major; in a tile lane = 16*g + j
         * holds rows 4g..4g+3 of column j in consecutive elements. */
        size_t ct_ = (cols + 15) / 16;
        size_t tr = r / 16, tc = c / 16, rr = r % 16, cc = c % 16;
        size_t lane = 16 * (rr / 4) + cc;
        return (int64_t)((((tr * ct_ + tc) * 64 + lane) * 4 + rr % 4) * esz); }
    }
    return -1;
}

int cvo_layout_convert(void* dst, uint32_t rows, uint32_t cols, int dstCt, int dstLayout,
                       size_t dstStride, const void* src, int srcCt, int srcLayout,
                       size_t srcStride)
{
    size_t dsz = cvo_layout_matrix_size(rows, cols, dstCt, dstLayout, dstStride);
    size_t ssz = cvo_layout_matrix_size(rows, cols, srcCt, srcLayout, srcStride);
    if (!dsz || !ssz) return -1;
    if (dstCt != srcCt &&
        !((dstCt == CVO_FLOAT16 || dstCt == CVO_FLOAT32) && (srcCt == CVO_FLOAT16 || srcCt == CVO_FLOAT32)))
        return -1;
    if (dstLayout == CVO_INFERENCING_OPTIMAL || dstLayout == CVO_TRAINING_OPTIMAL)
        memset(dst, 0, dsz);
    int des = elem_size(dstCt), ses = elem_size(srcCt);
    for (uint32_t r = 0; r < rows; ++r)
        for (uint32_t c = 0; c < cols; ++c) {
            const uint8_t* s = (const uint8_t*)src +
                cvo_layout_elem_offset(rows, cols, srcCt, srcLayout, srcStride, r, c);
            uint8_t* d = (uint8_t*)dst +
                cvo_layout_elem_offset(rows, cols, dstCt, dstLayout, dstStride, r, c);
            if (dstCt == srcCt) memcpy(d, s, (size_t)des);
            else if (srcCt == CVO_FLOAT16) { uint16_t h; memcpy(&h, s, 2); float f = cvo_f16_to_f32(h); memcpy(d, &f, 4); }
            else { float f; memcpy(&f, s, 4); uint16_t h = cvo_f32_to_f16_rne(f); memcpy(d, &h, 2); }
            (void)ses;
        }
    return 0;
}

/* ===================================================================================== */
/* parity reference                                                                      */
/* ===================================================================================== */

static inline int decode_f32(const uint8_t* p, int ct, float* out)
{
    switch (ct) {
    case CVO_FLOAT16: { uint16_t h; memcpy(&h, p, 2); *out = cvo_f16_to_f32(h); return 0; }
    case CVO_FLOAT32: { memcpy(out, p, 4); return 0; }
    case CVO_FLOAT_E4M3: { *out = cvo_e4m3_to_f32(*p); return 0; }
    case CVO_FLOAT_E5M2: { *out = cvo_f16_to_f32((uint16_t)((uint16_t)*p << 8)); return 0; }   /* e5m2 = high byte of binary16 */
    case CVO_BFLOAT16: { uint16_t h; memcpy(&h, p, 2); *out = bits_f32((uint32_t)h << 16); return 0; } /* bf16 = high half of binary32 */
    case CVO_SINT8: { *out = (float)*(const int8_t*)p; return 0; }
    case CVO_UINT8: { *out = (float)*p; return 0; }
    }
    return -1;
}

/* Gather the (logical) M x k matrix into a dense row-major float array. */
static float* gather_matrix_f32(const void* matrix, size_t matrixOffset, int matInterp, int layout,
                                int transpose, uint32_t stride, int M, int k)
{
    float* W = (float*)malloc(sizeof(float) * (size_t)M * (size_t)k);
    if (!W) return NULL;
    /* memory holds `rows x cols`; with transpose the stored matrix is k x M */
    uint32_t rows = transpose ? (uint32_t)k : (uint32_t)M, cols = transpose ? (uint32_t)M : (uint32_t)k;
    const uint8_t* base = (const uint8_t*)matrix + matrixOffset;
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < k; ++j) {
            uint32_t r = transpose ? (uint32_t)j : (uint32_t)i, c = transpose ? (uint32_t)i : (uint32_t)j;
            int64_t off = cvo_layout_elem_offset(rows, cols, matInterp, layout, stride, r, c);
            if (off < 0 || decode_f32(base + off, matInterp, &W[(size_t)i * k + j])) { free(W); return NULL; }
        }
    return W;
}

int cvo_ref_matmul_f32(const void* x, size_t xStride, int xType, int k,
                       const void* matrix, size_t matrixOffset, int matrixInterp,
                       int layout, int transpose, uint32_t matrixStride, int M,
                       const void* bias, size_t biasOffset, int biasInterp,
                       uint32_t batch, float* out_f32, float* out_abs)
{
    int xsz = elem_size(xType);
    if (xsz < 0 || k <= 0 || M <= 0 || k > CVO_MAX_DIM) return -1;
    float* W = gather_matrix_f32(matrix, matrixOffset, matrixInterp, layout, transpose, matrixStride, M, k);
    if (!W) return -1;
    float* B = NULL;
    if (bias && biasInterp >= 0) {
        B = (float*)malloc(sizeof(float) * (size_t)M);
        int bsz = elem_size(biasInterp);
        for (int i = 0; i < M; ++i)
            if (bsz < 0 || decode_f32((const uint8_t*)bias + biasOffset + (size_t)i * bsz, biasInterp, &B[i])) { free(W); free(B); return -1; }
    }
    float xv[CVO_MAX_DIM];
    for (uint32_t b = 0; b < batch; ++b) {
        const uint8_t* xp = (const uint8_t*)x + (size_t)b * xStride;
        for (int j = 0; j < k; ++j)
            if (decode_f32(xp + (size_t)j * xsz, xType, &xv[j])) { free(W); free(B); return -1; }
        for (int i = 0; i < M; ++i) {
            const float* w = W + (size_t)i * k;
            volatile float acc = 0.f;   /* volatile: forbid reassociation / fma contraction */
            float ab = 0.f;
            for (int j = 0; j < k; ++j) {
                volatile float p = w[j] * xv[j];
                acc = acc + p;
                ab += fabsf(p);
            }
            if (B) { acc = acc + B[i]; ab += fabsf(B[i]); }
            out_f32[(size_t)b * M + i] = acc;
            if (out_abs) out_abs[(size_t)b * M + i] = ab;
        }
    }
    free(W); free(B);
    return 0;
}

int cvo_ref_matmul_i32(const void* x, size_t xStride, int xType, int k,
                       const void* matrix, size_t matrixOffset, int matrixInterp,
                       int layout, int transpose, uint32_t matrixStride, int M,
                       const void* bias, size_t biasOffset, int biasInterp,
                       uint32_t batch, int32_t* out)
{
    if (!(xType == CVO_SINT8 || xType == CVO_UINT8) || !(matrixInterp == CVO_SINT8 || matrixInterp == CVO_UINT8)) return -1;
    if (k <= 0 || M <= 0) return -1;
    float* Wf = gather_matrix_f32(matrix, matrixOffset, matrixInterp, layout, transpose, matrixStride, M, k);
    if (!Wf) return -1;
    for (uint32_t b = 0; b < batch; ++b) {
        const uint8_t* xp = (const uint8_t*)x + (size_t)b * xStride;
        for (int i = 0; i < M; ++i) {
            int64_t acc = 0;
            for (int j = 0; j < k; ++j) {
                int xv = (xType == CVO_SINT8) ? (int)(int8_t)xp[j] : (int)xp[j];
                acc += (int64_t)((int)Wf[(size_t)i * k + j]) * xv;
            }
            if (bias && biasInterp >= 0) {
                if (biasInterp != CVO_SINT32) { free(Wf); return -1; }
                int32_t bv; memcpy(&bv, (const uint8_t*)bias + biasOffset + 4 * (size_t)i, 4);
                acc += bv;
            }
            out[(size_t)b * M + i] = (int32_t)(uint32_t)(uint64_t)acc;   /* wraps like int32 */
        }
    }
    free(Wf);
    return 0;
}

/* The slope of a half network is a half value: fflayer.slang:64 builds it as CoopVec<NFloat, OutputSize>(0.001h). */
static inline float slope_as_half(float slope) { return cvo_f16_to_f32(cvo_f32_to_f16_rne(slope)); }

static inline uint16_t act_f16(uint16_t z, int act, float slope)
{
    float zf = cvo_f16_to_f32(z);
    switch (act) {
    case CVO_ACT_RELU: return (zf > 0.f) ? z : (uint16_t)((zf != zf) ? z : 0); /* max(z,0); NaN stays */
    case CVO_ACT_LEAKY_RELU: {
        /* max(out, out * slope) evaluated in half, fflayer.slang:64-65 */
        uint16_t zs = cvo_f32_to_f16_rne(zf * slope_as_half(slope));
        return (zf >= cvo_f16_to_f32(zs)) ? z : zs; }
    }
    return z;
}

static float** gather_layers(const CvoLayer* layers, int n)
{
    float** W = (float**)calloc((size_t)n, sizeof(float*));
    for (int l = 0; l < n; ++l) {
        W[l] = gather_matrix_f32(layers[l].weights, 0, layers[l].weightType, CVO_ROW_MAJOR, 0,
                                 layers[l].weightStride, layers[l].outDim, layers[l].inDim);
        if (!W[l]) { for (int q = 0; q < l; ++q) free(W[q]); free(W); return NULL; }
    }
    return W;
}

int cvo_ref_mlp_forward(const CvoLayer* layers, int numLayers,
                        const void* input, size_t inputStride, int inputType,
                        uint32_t batch, uint16_t* out, uint16_t* acts)
{
    if (numLayers <= 0) return -1;
    float** W = gather_layers(layers, numLayers);
    if (!W) return -1;
    size_t actOff[64]; size_t off = 0;
    if (numLayers > 64) return -1;
    for (int l = 0; l < numLayers; ++l) { actOff[l] = off; off += (size_t)batch * layers[l].outDim; }
    float cur[CVO_MAX_DIM], nxt[CVO_MAX_DIM];
    int isz = elem_size(inputType);
    for (uint32_t b = 0; b < batch; ++b) {
        const uint8_t* xp = (const uint8_t*)input + (size_t)b * inputStride;
        for (int j = 0; j < layers[0].inDim; ++j)
            if (decode_f32(xp + (size_t)j * isz, inputType, &cur[j])) return -1;
        for (int l = 0; l < numLayers; ++l) {
            const CvoLayer* L = &layers[l];
            if (L->weightType == CVO_FLOAT_E4M3)      /* quantise the carrier to e4m3 */
                for (int j = 0; j < L->inDim; ++j) cur[j] = cvo_e4m3_to_f32(cvo_f32_to_e4m3_sat(cur[j]));
            for (int i = 0; i < L->outDim; ++i) {
                const float* w = W[l] + (size_t)i * L->inDim;
                volatile float acc = 0.f;
                for (int j = 0; j < L->inDim; ++j) { volatile float p = w[j] * cur[j]; acc = acc + p; }
                if (L->bias) acc = acc + cvo_f16_to_f32(((const uint16_t*)L->bias)[i]);
                uint16_t z = cvo_f32_to_f16_rne(acc);
                uint16_t a = act_f16(z, L->activation, L->leakySlope);
                nxt[i] = cvo_f16_to_f32(a);
                if (acts) acts[actOff[l] + (size_t)b * L->outDim + i] = a;
                if (l == numLayers - 1) out[(size_t)b * L->outDim + i] = a;
            }
            memcpy(cur, nxt, sizeof(float) * (size_t)L->outDim);
        }
    }
    for (int l = 0; l < numLayers; ++l) free(W[l]);
    free(W);
    return 0;
}

int cvo_ref_mlp_train(const CvoLayer* layers, int numLayers,
                      const uint16_t* input, size_t inputStride,
                      const uint16_t* targets, float lossScale, uint32_t batch,
                      double** dW, double** dB, double* lossSum, int maxTieRule)
{
    if (numLayers <= 0 || numLayers > 64) return -1;
    float** W = gather_layers(layers, numLayers);
    if (!W) return -1;
    for (int l = 0; l < numLayers; ++l) {
        memset(dW[l], 0, sizeof(double) * (size_t)layers[l].inDim * layers[l].outDim);
        memset(dB[l], 0, sizeof(double) * (size_t)layers[l].outDim);
    }
    /* per-layer saved input x_l and pre-activation z_l, as fp32 images of fp16 values */
    float* xs = (float*)malloc(sizeof(float) * 65 * CVO_MAX_DIM);
    float* zs = (float*)malloc(sizeof(float) * 64 * CVO_MAX_DIM);
    double loss = 0.0;
    for (uint32_t b = 0; b < batch; ++b) {
        const uint16_t* xp = (const uint16_t*)((const uint8_t*)input + (size_t)b * inputStride);
        float* x0 = xs;
        float insum = 0.f;
        for (int j = 0; j < layers[0].inDim; ++j) { x0[j] = cvo_f16_to_f32(xp[j]); insum += x0[j]; }
        for (int l = 0; l < numLayers; ++l) {
            const CvoLayer* L = &layers[l];
            const float* cur = xs + (size_t)l * CVO_MAX_DIM;
            float* nxt = xs + (size_t)(l + 1) * CVO_MAX_DIM;
            float* z = zs + (size_t)l * CVO_MAX_DIM;
            for (int i = 0; i < L->outDim; ++i) {
                const float* w = W[l] + (size_t)i * L->inDim;
                volatile float acc = 0.f;
                for (int j = 0; j < L->inDim; ++j) { volatile float p = w[j] * cur[j]; acc = acc + p; }
                if (L->bias) acc = acc + cvo_f16_to_f32(((const uint16_t*)L->bias)[i]);
                uint16_t zh = cvo_f32_to_f16_rne(acc);
                z[i] = cvo_f16_to_f32(zh);
                nxt[i] = cvo_f16_to_f32(act_f16(zh, L->activation, L->leakySlope));
            }
        }
        /* loss and its seed gradient */
        const CvoLayer* LL = &layers[numLayers - 1];
        float g[CVO_MAX_DIM], gin[CVO_MAX_DIM];
        const float* y = xs + (size_t)numLayers * CVO_MAX_DIM;
        for (int i = 0; i < LL->outDim; ++i) {
            float t = targets ? cvo_f16_to_f32(targets[(size_t)b * LL->outDim + i])
                              : cvo_f16_to_f32(cvo_f32_to_f16_rne(sinf(insum)));
            float diff = cvo_f16_to_f32(cvo_f32_to_f16_rne(y[i] - t));
            loss += (double)diff * (double)diff;
            g[i] = cvo_f16_to_f32(cvo_f32_to_f16_rne(2.0f * diff * lossScale));
        }
        for (int l = numLayers - 1; l >= 0; --l) {
            const CvoLayer* L = &layers[l];
            const float* xin = xs + (size_t)l * CVO_MAX_DIM;
            const float* z = zs + (size_t)l * CVO_MAX_DIM;
            float dz[CVO_MAX_DIM];
            for (int i = 0; i < L->outDim; ++i) {
                float gi = g[i], zi = z[i], d;
                switch (L->activation) {
                case CVO_ACT_RELU:       /* max(z, 0): diff.meta.slang:2258-2277 */
                    d = (zi > 0.f) ? gi : ((zi == 0.f && maxTieRule) ? cvo_f16_to_f32(cvo_f32_to_f16_rne(0.5f * gi)) : 0.f);
                    break;
                case CVO_ACT_LEAKY_RELU: { /* max(z, z*s) */
                    float zsv = cvo_f16_to_f32(cvo_f32_to_f16_rne(zi * slope_as_half(L->leakySlope)));
                    float da, db;
                    if (zi > zsv) { da = gi; db = 0.f; }
                    else if (zi < zsv) { da = 0.f; db = gi; }
                    else if (maxTieRule) { da = db = cvo_f16_to_f32(cvo_f32_to_f16_rne(0.5f * gi)); }
                    else { da = gi; db = 0.f; }
                    float dbs = cvo_f16_to_f32(cvo_f32_to_f16_rne(db * slope_as_half(L->leakySlope)));
                    d = cvo_f16_to_f32(cvo_f32_to_f16_rne(da + dbs));
                    break; }
                default: d = gi;
                }
                dz[i] = d;
                dB[l][i] += (double)d;
                double* dwrow = dW[l] + (size_t)i * L->inDim;
                for (int j = 0; j < L->inDim; ++j) dwrow[j] += (double)d * (double)xin[j];
            }
            if (l > 0) {
                for (int j = 0; j < L->inDim; ++j) {
                    volatile float acc = 0.f;
                    for (int i = 0; i < L->outDim; ++i) { volatile float p = W[l][(size_t)i * L->inDim + j] * dz[i]; acc = acc + p; }
                    gin[j] = cvo_f16_to_f32(cvo_f32_to_f16_rne(acc));
                }
                memcpy(g, gin, sizeof(float) * (size_t)L->inDim);
            }
        }
    }
    if (lossSum) *lossSum = loss;
    free(xs); free(zs);
    for (int l = 0; l < numLayers; ++l) free(W[l]);
    free(W);
    return 0;
}

/* ===================================================================================== */
/* Adam (examples/mlp-training-coopvec/adam.slang:20-36, kernels.slang:29-45)            */
/* ===================================================================================== */

/* powNudge1/2 move the fp32 value of pow(beta1, it) / pow(beta2, it) by that many fp32 ulps before
 * it is rounded to half: pow is the one operation here that maths libraries are allowed to round
 * differently, and the tests use the nudges to show that a result differing from nudge (0,0) is such
 * a case. */
static float nudge_ulps(float v, int n)
{
    for (; n > 0; --n) v = nextafterf(v, INFINITY);
    for (; n < 0; ++n) v = nextafterf(v, -INFINITY);
    return v;
}

void cvo_slang_adam_step_nudged(CvoAdamState* states, uint16_t* params, uint16_t* grads, uint32_t count,
                                float beta1f, float beta2f, float epsf, float lrf, int halfMode,
                                int powNudge1, int powNudge2)
{
#define H(x) cvo_f16_to_f32(to_half((x), halfMode))     /* one rounding to half */
    const float beta1 = H(beta1f), beta2 = H(beta2f), eps = H(epsf), lr = H(lrf);
    for (uint32_t i = 0; i < count; ++i) {
        float g = cvo_f16_to_f32(grads[i]);
        if (g != g) { grads[i] = 0; continue; }                       /* kernels.slang:39-43 */
        CvoAdamState* st = &states[i];
        st->iteration++;
        if (isinf(g)) g = g > 0 ? H(10000.0f) : H(-10000.0f);          /* adam.slang:23-29 */
        float mean = cvo_f16_to_f32(st->mean), var = cvo_f16_to_f32(st->variance);
        const float omb1 = H(1.0f - beta1), omb2 = H(1.0f - beta2);
        mean = H(H(beta1 * mean) + H(omb1 * g));
        var = H(H(beta2 * var) + H(H(omb2 * g) * g));
        const float it = H((float)st->iteration);
        const float meanHat = H(mean / H(1.0f - H(nudge_ulps(powf(beta1, it), powNudge1))));
        const float varHat = H(var / H(1.0f - H(nudge_ulps(powf(beta2, it), powNudge2))));
        const float denom = H(sqrtf(H(fmaxf(0.0f, varHat) + eps)));
        const float p = cvo_f16_to_f32(params[i]);
        params[i] = to_half(p - H(H(lr * meanHat) / denom), halfMode);
        st->mean = to_half(mean, halfMode);
        st->variance = to_half(var, halfMode);
        grads[i] = 0;
    }
#undef H
}

void cvo_slang_adam_step(CvoAdamState* states, uint16_t* params, uint16_t* grads, uint32_t count,
                         float beta1f, float beta2f, float epsf, float lrf, int halfMode)
{
    cvo_slang_adam_step_nudged(states, params, grads, count, beta1f, beta2f, epsf, lrf, halfMode, 0, 0);
}

/* ===================================================================================== */
/* element-wise surface (hlsl.meta.slang:32043-32421, slang-ir-lower-coopvec.cpp:113-166, */
/* activations.slang) and its reverse-mode rules (diff.meta.slang:1948-2470)              */
/* ===================================================================================== */

static double ew_load(const void* p, int ct, size_t i)
{
    if (ct == CVO_FLOAT32) return (double)((const float*)p)[i];
    return (double)cvo_f16_to_f32(((const uint16_t*)p)[i]);
}

/* double -> half in one rounding: a float that is truncated towards zero with its last bit set whenever anything
 * was cut off (round to odd) carries enough to round to the 11 bits of a half exactly once */
static uint16_t ew_f64_to_f16(double v)
{
    float f = (float)v;
    if ((double)f != v && f == f && f - f == 0.0f) {
        uint32_t u;
        memcpy(&u, &f, 4);
        if (fabs((double)f) > fabs(v)) u -= 1u;
        u |= 1u;
        memcpy(&f, &u, 4);
    }
    return cvo_f32_to_f16_rne(f);
}

static void ew_store(void* p, int ct, size_t i, double v)
{
    if (ct == CVO_FLOAT32) ((float*)p)[i] = (float)v;
    else ((uint16_t*)p)[i] = ew_f64_to_f16(v);
}

static double ew_sigmoid(double x)
{
    /* activations.slang:101-108: the exp() argument is always <= 0 */
    const double ex = exp(x >= 0 ? -x : x);
    return x >= 0 ? 1.0 / (1.0 + ex) : ex / (1.0 + ex);
}

static int ew_operands(int op)
{
    switch (op) {
    case CVO_OP_ADD: case CVO_OP_SUB: case CVO_OP_MUL: case CVO_OP_DIV: case CVO_OP_MIN: case CVO_OP_MAX: case CVO_OP_STEP: return 2;
    case CVO_OP_CLAMP: case CVO_OP_FMA: return 3;
    }
    return 1;
}

static const double kLn2 = 0.69314718055994530941723212145818;

int cvo_elementwise(int op, int ct, size_t count, const void* a, const void* b, const void* c, void* out, float param)
{
    if (op < 0 || op >= CVO_OP_COUNT || (ct != CVO_FLOAT16 && ct != CVO_FLOAT32)) return -1;
    const int n = ew_operands(op);
    for (size_t i = 0; i < count; ++i) {
        const double x = ew_load(a, ct, i), y = n >= 2 ? ew_load(b, ct, i) : 0, z = n >= 3 ? ew_load(c, ct, i) : 0;
        double r = x;
        switch (op) {
        case CVO_OP_ADD: r = x + y; break;
        case CVO_OP_SUB: r = x - y; break;
        case CVO_OP_MUL: r = x * y; break;
        case CVO_OP_DIV: r = x / y; break;
        case CVO_OP_NEG: r = -x; break;
        case CVO_OP_MIN: r = x < y ? x : y; break;                      /* hlsl.meta.slang:32046-32067 */
        case CVO_OP_MAX: r = x > y ? x : y; break;
        case CVO_OP_CLAMP: r = fmin(fmax(x, y), z); break;              /* :32094-32111 */
        case CVO_OP_STEP: r = y >= x ? 1.0 : 0.0; break;                /* step(edge, x), :32210-32229 */
        case CVO_OP_SIN: r = sin(x); break;
        case CVO_OP_COS: r = cos(x); break;
        case CVO_OP_EXP: r = exp(x); break;
        case CVO_OP_LOG: r = log(x); break;
        case CVO_OP_LOG2: r = log2(x); break;
        case CVO_OP_EXP2: r = exp2(x); break;
        case CVO_OP_TANH: r = tanh(x); break;
        case CVO_OP_ATAN: r = atan(x); break;
        case CVO_OP_FMA: r = x * y + z; break;
        case CVO_OP_RELU: r = x > 0 ? x : 0; break;                     /* activations.slang:25-42 */
        case CVO_OP_LEAKY_RELU: r = x < 0 ? (double)param * x : x; break; /* :69-74 */
        case CVO_OP_SIGMOID: r = ew_sigmoid(x); break;
        case CVO_OP_SILU: r = x * ew_sigmoid(x); break;                 /* :186-193 */
        case CVO_OP_QUICK_GELU: r = x * ew_sigmoid(1.702 * x); break;   /* :215-223 */
        case CVO_OP_SCALE:                                              /* hlsl.meta.slang:32004: vector * T(scalar) */
            r = x * (ct == CVO_FLOAT16 ? (double)cvo_f16_to_f32(cvo_f32_to_f16_rne(param)) : (double)param); break;
        }
        ew_store(out, ct, i, r);
    }
    return 0;
}

int cvo_elementwise_backward(int op, int ct, size_t count, const void* a, const void* b, const void* c,
                             const void* dOut, void* dA, void* dB, void* dC, float param)
{
    if (op < 0 || op >= CVO_OP_COUNT || (ct != CVO_FLOAT16 && ct != CVO_FLOAT32)) return -1;
    const int n = ew_operands(op);
    for (size_t i = 0; i < count; ++i) {
        const double x = ew_load(a, ct, i), y = n >= 2 ? ew_load(b, ct, i) : 0, z = n >= 3 ? ew_load(c, ct, i) : 0;
        const double g = ew_load(dOut, ct, i);
        double dx = 0, dy = 0, dz = 0;
        switch (op) {
        case CVO_OP_ADD: dx = g; dy = g; break;
        case CVO_OP_SUB: dx = g; dy = -g; break;
        case CVO_OP_MUL: dx = y * g; dy = x * g; break;
        case CVO_OP_DIV: dx = g / y; dy = -x * g / (y * y); break;
        case CVO_OP_NEG: dx = -g; break;
        case CVO_OP_MIN:                                                 /* diff.meta.slang:2293-2300 */
            dx = x < y ? g : (x > y ? 0 : 0.5 * g);
            dy = y < x ? g : (y > x ? 0 : 0.5 * g);
            break;
        case CVO_OP_MAX:                                                 /* :2266-2273 */
            dx = x > y ? g : (x < y ? 0 : 0.5 * g);
            dy = y > x ? g : (y < x ? 0 : 0.5 * g);
            break;
        case CVO_OP_CLAMP:                                               /* :2413-2421 */
            dx = (x >= y && x <= z) ? g : 0;
            dy = x < y ? g : 0;
            dz = x > z ? g : 0;
            break;
        case CVO_OP_STEP: break;
        case CVO_OP_SIN: dx = cos(x) * g; break;                        /* :2104-2105 */
        case CVO_OP_COS: dx = -(sin(x) * g); break;                     /* :2108-2112 */
        case CVO_OP_EXP: dx = exp(x) * g; break;
        case CVO_OP_LOG: dx = g / x; break;
        case CVO_OP_LOG2: dx = g / (x * kLn2); break;                   /* :2134-2139 */
        case CVO_OP_EXP2: dx = exp2(x) * kLn2 * g; break;
        case CVO_OP_TANH: { const double t = tanh(x); dx = g - t * t * g; break; }   /* :2117-2124 */
        case CVO_OP_ATAN: dx = g / (x * x + 1.0); break;                /* :2152-2156 */
        case CVO_OP_FMA: dx = y * g; dy = x * g; dz = g; break;         /* :2441-2446 */
        case CVO_OP_RELU: dx = x > 0 ? g : (x < 0 ? 0 : 0.5 * g); break;
        case CVO_OP_LEAKY_RELU: dx = x < 0 ? (double)param * g : g; break;
        case CVO_OP_SIGMOID: { const double sg = ew_sigmoid(x); dx = sg * (1 - sg) * g; break; }
        case CVO_OP_SILU: { const double sg = ew_sigmoid(x); dx = (sg + x * sg * (1 - sg)) * g; break; }
        case CVO_OP_QUICK_GELU: { const double sg = ew_sigmoid(1.702 * x); dx = (sg + 1.702 * x * sg * (1 - sg)) * g; break; }
        case CVO_OP_SCALE: dx = (ct == CVO_FLOAT16 ? (double)cvo_f16_to_f32(cvo_f32_to_f16_rne(param)) : (double)param) * g; break;
        }
        if (dA) ew_store(dA, ct, i, dx);
        if (dB && n >= 2) ew_store(dB, ct, i, dy);
        if (dC && n >= 3) ew_store(dC, ct, i, dz);
    }
    return 0;
}

/* ===================================================================================== */
/* grid hashes (source/standard-modules/neural/hash-function.slang)                      */
/* ===================================================================================== */

typedef struct { uint64_t state, inc; } Pcg32;

static uint32_t pcg_next(Pcg32* r)                                    /* hash-function.slang:35-42 */
{
    const uint64_t old = r->state;
    r->state = old * 0x5851f42d4c957f2dULL + r->inc;
    const uint32_t xorshifted = (uint32_t)(((old >> 18) ^ old) >> 27);
    const uint32_t rot = (uint32_t)(old >> 59);
    return (xorshifted >> rot) | (xorshifted << ((~rot + 1u) & 31u));
}

static void pcg_init(Pcg32* r, uint64_t initstate, uint64_t initseq)  /* :25-32 */
{
    r->state = 0;
    r->inc = (initseq << 1) | 1u;
    pcg_next(r);
    r->state += initstate;
    pcg_next(r);
}

static void pcg_advance(Pcg32* r, int64_t delta)                      /* :45-65 */
{
    uint64_t curMult = 0x5851f42d4c957f2dULL, curPlus = r->inc, accMult = 1, accPlus = 0;
    for (uint64_t d = (uint64_t)delta; d > 0; d /= 2) {
        if (d & 1) { accMult *= curMult; accPlus = accPlus * curMult + curPlus; }
        curPlus = (curMult + 1) * curPlus;
        curMult *= curMult;
    }
    r->state = accMult * r->state + accPlus;
}

uint32_t cvo_grid_hash(int type, int dims, const uint32_t* pos)
{
    static const uint32_t prime[7] = {1958374283u, 2654435761u, 805459861u, 3674653429u, 2097192037u, 1434869437u, 2165219737u};
    static const uint32_t coherent[7] = {1u, 2654435761u, 805459861u, 3674653429u, 2097192037u, 1434869437u, 2165219737u};
    static const uint32_t reversed[7] = {2165219737u, 1434869437u, 2097192037u, 3674653429u, 805459861u, 2654435761u, 1958374283u};
    switch (type) {
    case 0: case 1: case 2: {                                           /* lcgHash, :69-78 */
        const uint32_t* f = type == 0 ? prime : type == 1 ? coherent : reversed;
        uint32_t r = 0;
        for (int i = 0; i < dims; ++i) r ^= pos[i] * f[i];
        return r; }
    case 3: {                                                           /* rngHash, :117-131 */
        const int bits = 64 / dims;
        uint64_t step = 0;
        for (int i = 0; i < dims; ++i) step ^= (uint64_t)pos[i] << (i * bits);
        Pcg32 rng;
        pcg_init(&rng, 1337, 1);
        pcg_advance(&rng, (int64_t)step);
        return pcg_next(&rng); }
    case 4: {                                                           /* baseConvertHash, :103-113 */
        uint32_t k = 0;
        for (int d = 0; d < dims; ++d) { k += pos[d]; k *= 2531011u; }
        return k; }
    }
    return 0;
}

/* ===================================================================================== */
/* permutohedral-lattice encoder (source/standard-modules/neural/permuto-encoder.slang)  */
/* ===================================================================================== */

void cvo_permuto_prepare_level(uint32_t level, int dims, uint32_t log2HashmapSize, float baseScale,
                               float log2PerLevelScale, uint32_t seed, CvoPermutoLevel* out)   /* :339-368 */
{
    const uint32_t size = 1u << log2HashmapSize;
    out->currentLevelIndex = level;
    out->featureTableSize = size;
    out->offsetOfFeatureTable = level * size;
    out->scale = baseScale * exp2f((float)level * log2PerLevelScale);
    Pcg32 rng;
    pcg_init(&rng, seed, 1);
    pcg_advance(&rng, (int64_t)(level * (uint32_t)dims));
    for (int d = 0; d < dims; ++d) {
        out->scalesPerDim[d] = out->scale * (1.0f / sqrtf((float)((d + 1) * (d + 2))));
        const float r = (float)pcg_next(&rng) * (1.0f / 4294967296.0f);
        out->shiftsPerDim[d] = r * 10.0f - 5.0f;
    }
}

/* geometry of one (sample, level): elevated point, closest remainder-0 point, rank (:74-152) */
static void permuto_geometry(int D, const float* pos, const CvoPermutoLevel* lv, float* elevated, int* rem0, int* rank)
{
    float sum = 0.0f;
    for (int dim = D - 1; dim >= 0; --dim) {
        const float cf = (pos[dim] + lv->shiftsPerDim[dim]) * lv->scalesPerDim[dim];
        elevated[dim + 1] = sum - (float)(dim + 1) * cf;
        sum += cf;
    }
    elevated[0] = sum;
    int isum = 0;
    for (int dim = 0; dim <= D; ++dim) {
        rank[dim] = 0;
        const float v = elevated[dim] * (1.0f / (float)(D + 1));
        const float up = ceilf(v) * (float)(D + 1), down = floorf(v) * (float)(D + 1);
        rem0[dim] = (up - elevated[dim] < elevated[dim] - down) ? (int)up : (int)down;
        isum += rem0[dim];
    }
    isum /= (D + 1);
    for (int dim = 0; dim < D; ++dim) {
        const float di = elevated[dim] - (float)rem0[dim];
        for (int other = dim + 1; other <= D; ++other) {
            if (di < elevated[other] - (float)rem0[other]) rank[dim]++;
            else rank[other]++;
        }
    }
    for (int dim = 0; dim <= D; ++dim) {
        rank[dim] += isum;
        if (rank[dim] < 0) { rank[dim] += D + 1; rem0[dim] += D + 1; }
        else if (rank[dim] > D) { rank[dim] -= D + 1; rem0[dim] -= D + 1; }
    }
}

static uint32_t permuto_vertex_index(int D, int F, const CvoPermutoLevel* lv, const int* rem0, const int* rank, int k)
{
    uint32_t key[CVO_PERMUTO_MAX_DIMS];
    for (int dim = 0; dim < D; ++dim) {                                  /* :296-304 */
        key[dim] = (uint32_t)(rem0[dim] + k);
        if (rank[dim] > D - k) key[dim] -= (uint32_t)(D + 1);
    }
    return lv->offsetOfFeatureTable * (uint32_t)F + (cvo_grid_hash(4, D, key) % lv->featureTableSize) * (uint32_t)F;
}

static float permuto_tab(const void* table, int ct, size_t i)
{
    return ct == CVO_FLOAT32 ? ((const float*)table)[i] : cvo_f16_to_f32(((const uint16_t*)table)[i]);
}
static float permuto_round(float v, int ct) { return ct == CVO_FLOAT32 ? v : cvo_f16_to_f32(cvo_f32_to_f16_rne(v)); }

int cvo_permuto_encode(int D, int F, int numLevels, float maxLevel, const CvoPermutoLevel* levels, int ct,
                       const void* positions, size_t count, const void* table, void* out)
{
    if (D < 1 || D > CVO_PERMUTO_MAX_DIMS || F < 1 || numLevels < 1 || (ct != CVO_FLOAT32 && ct != CVO_FLOAT16)) return -1;
    for (size_t s = 0; s < count; ++s) {
        float pos[CVO_PERMUTO_MAX_DIMS];
        for (int d = 0; d < D; ++d) pos[d] = permuto_tab(positions, ct, s * D + d);
        for (int l = 0; l < numLevels; ++l) {
            const CvoPermutoLevel* lv = &levels[l];
            float acc[64];
            for (int f = 0; f < F; ++f) acc[f] = 0.0f;
            if (!((float)lv->currentLevelIndex >= maxLevel + 1e-3f)) {   /* :259-262 */
                float elevated[CVO_PERMUTO_MAX_DIMS + 1], bary[CVO_PERMUTO_MAX_DIMS + 2];
                int rem0[CVO_PERMUTO_MAX_DIMS + 1], rank[CVO_PERMUTO_MAX_DIMS + 1];
                permuto_geometry(D, pos, lv, elevated, rem0, rank);
                for (int i = 0; i <= D + 1; ++i) bary[i] = 0.0f;        /* :166-179 */
                for (int dim = 0; dim <= D; ++dim) {
                    const float delta = (elevated[dim] - (float)rem0[dim]) * (1.0f / (float)(D + 1));
                    bary[D - rank[dim]] += delta;
                    bary[D + 1 - rank[dim]] -= delta;
                }
                bary[0] += 1.0f + bary[D + 1];
                for (int k = 0; k <= D; ++k) {
                    const uint32_t idx = permuto_vertex_index(D, F, lv, rem0, rank, k);
                    const float w = permuto_round(bary[k], ct);          /* T(weight) */
                    for (int f = 0; f < F; ++f)                          /* += T(weight) * featureVal, in T (:312-316) */
                        acc[f] = permuto_round(acc[f] + permuto_round(w * permuto_tab(table, ct, idx + f), ct), ct);
                }
            }
            for (int f = 0; f < F; ++f) {
                const size_t o = s * (size_t)(numLevels * F) + (size_t)lv->currentLevelIndex * F + f;
                if (ct == CVO_FLOAT32) ((float*)out)[o] = acc[f];
                else ((uint16_t*)out)[o] = cvo_f32_to_f16_rne(acc[f]);
            }
        }
    }
    return 0;
}

/* Reverse mode of the encoder in double: dPositions (overwritten) and dTable (accumulated, like the
 * reference's atomicAdd, :222-238). */
int cvo_permuto_encode_backward(int D, int F, int numLevels, float maxLevel, const CvoPermutoLevel* levels,
                                const float* positions, size_t count, const float* table, const float* dOut,
                                double* dPositions, double* dTable)
{
    if (D < 1 || D > CVO_PERMUTO_MAX_DIMS || F < 1 || numLevels < 1) return -1;
    for (size_t s = 0; s < count; ++s) {
        const float* pos = positions + s * D;
        for (int d = 0; d < D; ++d) dPositions[s * D + d] = 0.0;
        for (int l = 0; l < numLevels; ++l) {
            const CvoPermutoLevel* lv = &levels[l];
            if ((float)lv->currentLevelIndex >= maxLevel + 1e-3f) continue;
            float elevated[CVO_PERMUTO_MAX_DIMS + 1];
            int rem0[CVO_PERMUTO_MAX_DIMS + 1], rank[CVO_PERMUTO_MAX_DIMS + 1];
            permuto_geometry(D, pos, lv, elevated, rem0, rank);
            double bary[CVO_PERMUTO_MAX_DIMS + 2], dbary[CVO_PERMUTO_MAX_DIMS + 2];
            for (int i = 0; i <= D + 1; ++i) { bary[i] = 0.0; dbary[i] = 0.0; }
            for (int dim = 0; dim <= D; ++dim) {
                const double delta = ((double)elevated[dim] - (double)rem0[dim]) / (double)(D + 1);
                bary[D - rank[dim]] += delta;
                bary[D + 1 - rank[dim]] -= delta;
            }
            bary[0] += 1.0 + bary[D + 1];
            const float* g = dOut + s * (size_t)(numLevels * F) + (size_t)lv->currentLevelIndex * F;
            for (int k = 0; k <= D; ++k) {
                const uint32_t idx = permuto_vertex_index(D, F, lv, rem0, rank, k);
                for (int f = 0; f < F; ++f) {
                    dTable[idx + f] += bary[k] * (double)g[f];
                    dbary[k] += (double)table[idx + f] * (double)g[f];
                }
            }
            dbary[D + 1] += dbary[0];                                    /* wrap-around term */
            double delev[CVO_PERMUTO_MAX_DIMS + 1];
            for (int dim = 0; dim <= D; ++dim)
                delev[dim] = (dbary[D - rank[dim]] - dbary[D + 1 - rank[dim]]) / (double)(D + 1);
            /* elevate: e[dim+1] = sum - (dim+1) cf, sum += cf for dim = D-1..0, e[0] = sum */
            double dsum = delev[0];
            for (int dim = 0; dim < D; ++dim) {
                double dcf = dsum - (double)(dim + 1) * delev[dim + 1];
                dsum += delev[dim + 1];
                dPositions[s * D + dim] += dcf * (double)lv->scalesPerDim[dim];
            }
        }
    }
    return 0;
}
