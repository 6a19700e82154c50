// cv_layout.h -- byte layouts of cooperative-vector matrices, shared by host and device code.
//
// RowMajor / ColumnMajor follow the reference's addressing rule
// (source/slang/hlsl.meta.slang:32862-32864): element (r,c) lives at r*stride + c*elemSize,
// or c*stride + r*elemSize for ColumnMajor.
//
// The reference leaves InferencingOptimal / TrainingOptimal opaque (they belong to the vendor
// driver behind rhi::IDevice::getCooperativeVectorMatrixSize, call site
// examples/mlp-training-coopvec/mlp-training-coopvec.cpp:305).  Here they are defined by the
// gfx950 MFMA register fragments:
//
//  InferencingOptimal : the matrix is the A operand of D = W . X^T, split into fragments
//      (t, kt) of 64 lanes x EPL elements, stored [t][kt][lane][EPL].  Lane 16*g+i of fragment
//      (t,kt) holds W[row(t,i)][g*GS + kt*EPL + s], s < EPL, where GS = 4*ceil(K/16) is the
//      number of k-slots a 16-lane group owns and row(t,i) = (i/4)*4*MT + 4*t + i%4.
//      With that row order the accumulator of one layer is, register for register, the B
//      operand of the next layer, and lane group g owns a contiguous quarter of both the input
//      and the output vector.  Slots >= GS and rows/cols beyond the matrix hold zero.
//
//  TrainingOptimal    : accumulator-native 16x16 tiles, tile grid row-major; in a tile lane
//      16*g+j holds rows 4g..4g+3 of column j in four consecutive elements.
#pragma once
#include <stddef.h>
#include <stdint.h>

#if defined(__HIPCC__)
#define CV_HD __host__ __device__ inline
#else
#define CV_HD inline
#endif

namespace cv {

// CoopVecComponentType values (hlsl.meta.slang:32558-32575)
enum : int {
    kE4M3 = 0, kE5M2 = 1, kF16 = 2, kF32 = 3, kF64 = 4, kS8 = 5, kS16 = 6, kS32 = 7, kS64 = 8,
    kS8Packed = 9, kU8 = 10, kU16 = 11, kU32 = 12, kU64 = 13, kU8Packed = 14,
    kBF16 = 15          // the library's extension: bfloat16
};
enum : int { kRowMajor = 0, kColumnMajor = 1, kInferencingOptimal = 2, kTrainingOptimal = 3 };

// bytes of one stored element, 0 if the type is unknown
CV_HD uint32_t elemSize(int ct)
{
    switch (ct) {
    case kE4M3: case kE5M2: case kS8: case kU8: return 1;
    case kF16: case kS16: case kU16: case kBF16: return 2;
    case kF32: case kS32: case kU32: case kS8Packed: case kU8Packed: return 4;
    case kF64: case kS64: case kU64: return 8;
    }
    return 0;
}

// k-slots one lane contributes to one MFMA fragment (0: no InferencingOptimal form)
CV_HD uint32_t fragElemsPerLane(int ct)
{
    switch (ct) {
    case kS8: case kU8: return 16;                 // v_mfma_i32_16x16x64_i8
    case kE4M3: case kE5M2: return 8;              // v_mfma_f32_16x16x32_fp8_fp8
    case kF16: case kF32: case kBF16: return 8;    // v_mfma_f32_16x16x32_f16 / _bf16
    }
    return 0;
}

CV_HD bool layoutSupports(int ct, int layout)
{
    if (elemSize(ct) == 0 || ct == kS8Packed || ct == kU8Packed) return false;
    switch (layout) {
    case kRowMajor: case kColumnMajor: return true;
    case kInferencingOptimal: return fragElemsPerLane(ct) != 0;
    case kTrainingOptimal: return ct == kF16 || ct == kF32 || ct == kBF16;
    }
    return false;
}

struct MatrixShape {
    uint32_t rows, cols;
    int32_t ct, layout;
    size_t stride;     // Row/ColumnMajor: bytes between rows/columns (0 = packed)
};

CV_HD uint32_t optMT(uint32_t rows) { return (rows + 15u) / 16u; }
CV_HD uint32_t optGS(uint32_t cols) { return ((cols + 15u) / 16u) * 4u; }
CV_HD uint32_t optKT(uint32_t cols, uint32_t epl) { return (optGS(cols) + epl - 1u) / epl; }

CV_HD size_t matrixSize(const MatrixShape& s)
{
    if (s.rows == 0 || s.cols == 0 || !layoutSupports(s.ct, s.layout)) return 0;
    const size_t esz = elemSize(s.ct);
    switch (s.layout) {
    case kRowMajor: {
        const size_t st = s.stride ? s.stride : s.cols * esz;
        return st < s.cols * esz ? 0 : (size_t)(s.rows - 1) * st + s.cols * esz; }
    case kColumnMajor: {
        const size_t st = s.stride ? s.stride : s.rows * esz;
        return st < s.rows * esz ? 0 : (size_t)(s.cols - 1) * st + s.rows * esz; }
    case kInferencingOptimal: {
        const uint32_t epl = fragElemsPerLane(s.ct);
        return (size_t)optMT(s.rows) * optKT(s.cols, epl) * 64u * epl * esz; }
    case kTrainingOptimal:
        return (size_t)optMT(s.rows) * optMT(s.cols) * 256u * esz;
    }
    return 0;
}

// byte offset of element (r,c); the caller guarantees r < rows, c < cols and a valid shape
CV_HD size_t elemOffset(const MatrixShape& s, uint32_t r, uint32_t c)
{
    const size_t esz = elemSize(s.ct);
    switch (s.layout) {
    case kRowMajor:    return (size_t)r * (s.stride ? s.stride : s.cols * esz) + c * esz;
    case kColumnMajor: return (size_t)c * (s.stride ? s.stride : s.rows * esz) + r * esz;
    case kInferencingOptimal: {
        const uint32_t epl = fragElemsPerLane(s.ct);
        const uint32_t mt4 = 4u * optMT(s.rows), gs = optGS(s.cols), kt = optKT(s.cols, epl);
        const uint32_t rem = r % mt4, t = rem / 4u, i = 4u * (r / mt4) + (rem & 3u);
        const uint32_t g = c / gs, q = c % gs, k = q / epl, e = q % epl;
        return ((((size_t)t * kt + k) * 64u + 16u * g + i) * epl + e) * esz; }
    case kTrainingOptimal: {
        const uint32_t tc = optMT(s.cols);
        const uint32_t lane = 16u * ((r & 15u) / 4u) + (c & 15u);
        return ((((size_t)(r / 16u) * tc + c / 16u) * 64u + lane) * 4u + (r & 3u)) * esz; }
    }
    return 0;
}

} // namespace cv
