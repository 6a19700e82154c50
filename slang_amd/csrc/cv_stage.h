// cv_stage.h -- the one routine that brings a weight matrix from memory into LDS in MFMA fragment
// order; every kernel that keeps weights on chip stages them through it.
//
// Destination: fragments (t, kt), t < MT, kt < KT, stored [t][kt][lane][EPL] (the InferencingOptimal
// order of cv_layout.h).  Lane 16*g+i of fragment (t,kt) receives, for s < EPL,
//     L[rowOff + (i/4)*4*MT + 4*t + i%4][g*gs + kt*EPL + s]
// of the logical matrix L (rows x cols valid, everything else zero), where L(r,c) is element (r,c)
// of the matrix in memory, or element (c,r) when `transposed` (the matrix is used as its transpose:
// the backward pass reads W^T out of the same bytes).
//
// A source whose fragment order already matches is copied with 16-byte accesses.  Otherwise a
// thread gathers one lane-chunk (EPL elements) at a time: when the chunk is contiguous in memory
// (RowMajor used as it lies, ColumnMajor used transposed), whole and 8-byte aligned it is fetched
// with 8-byte loads, else element by element with zero fill.
#pragma once
#include "cv_device.h"

namespace cv {

// xorByte (1-byte types only): XORed into every valid element on the way, used to re-bias
// unsigned bytes to signed ones (u ^ 0x80 == u - 128 as int8); padding stays zero.
template <int ESZ, int EPL>
__device__ __forceinline__ void stageFragments(uint32_t* ldsDst, const uint8_t* w, const MatrixShape& shape,
                                               bool transposed, int MT, int KT, uint32_t gs, uint32_t rows,
                                               uint32_t cols, uint32_t rowOff = 0, uint32_t xorByte = 0,
                                               uint32_t firstThread = 0)
{
    constexpr int CHUNK = ESZ * EPL;              // bytes of one lane-chunk: 8, 16 or 32
    static_assert(ESZ == 1 || ESZ == 2 || ESZ == 4, "element size");
    static_assert(CHUNK % 8 == 0, "a lane-chunk is a whole number of 8-byte words");
    const int chunks = MT * KT * 64;
    const bool direct = shape.layout == kInferencingOptimal && !transposed && rowOff == 0 && xorByte == 0 &&
                        optMT(shape.rows) == (uint32_t)MT && optKT(shape.cols, EPL) == (uint32_t)KT &&
                        shape.rows == rows && shape.cols == cols;
    if (direct) {
        const u32x4* src = (const u32x4*)w;
        u32x4* dst = (u32x4*)ldsDst;
        for (int i = threadIdx.x; i < chunks * CHUNK / 16; i += blockDim.x) dst[i] = src[i];
        return;
    }
    const bool contiguous = (shape.layout == kRowMajor && !transposed) || (shape.layout == kColumnMajor && transposed);
    const uint32_t xorWord = xorByte * 0x01010101u;
    const int ROWS = 4 * MT;
    // firstThread: the thread that takes chunk 0.  A kernel that stages several small matrices gives each its own
    // part of the workgroup, so that their round trips to memory overlap instead of following one another.
    const uint32_t vt = threadIdx.x >= firstThread ? threadIdx.x - firstThread : threadIdx.x + blockDim.x - firstThread;
    for (int c = (int)vt; c < chunks; c += blockDim.x) {
        const int lane = c & 63, f = c >> 6;
        const int kt = f % KT, t = f / KT, g = lane >> 4, i = lane & 15;
        const uint32_t row = (uint32_t)((i >> 2) * ROWS + 4 * t + (i & 3));
        const uint32_t q0 = (uint32_t)(kt * EPL), col0 = g * gs + q0;
        int nvalid = 0;
        if (row < rows && q0 < gs && col0 < cols) {
            const uint32_t a = gs - q0, b = cols - col0;
            nvalid = (int)(a < b ? a : b);
            if (nvalid > EPL) nvalid = EPL;
        }
        uint32_t* d = ldsDst + (size_t)c * (CHUNK / 4);
        const uint32_t r = rowOff + row;
        const uint8_t* p0 = nvalid > 0 ? w + (transposed ? elemOffset(shape, col0, r) : elemOffset(shape, r, col0)) : w;
        if (contiguous && nvalid == EPL && ((uintptr_t)p0 & 7) == 0) {
#pragma unroll
            for (int i8 = 0; i8 < CHUNK / 8; ++i8) {
                const u32x2 x = ((const u32x2*)p0)[i8];
                ((u32x2*)d)[i8] = u32x2{x.x ^ xorWord, x.y ^ xorWord};
            }
        } else if (contiguous) {
            // a ragged or unaligned run of elements that lie side by side: all loads first (always-valid
            // addresses, masked afterwards), then the stores, so that the run costs one round trip to memory
            // instead of one per element (small networks spend most of their few microseconds here)
            uint32_t v[EPL];
#pragma unroll
            for (int s = 0; s < EPL; ++s) {
                const uint8_t* p = s < nvalid ? p0 + s * ESZ : w;
                if constexpr (ESZ == 4)      v[s] = *(const uint32_t*)p;
                else if constexpr (ESZ == 2) v[s] = *(const uint16_t*)p;
                else                         v[s] = (uint32_t)(*p ^ xorByte);
            }
#pragma unroll
            for (int s = 0; s < EPL; ++s) v[s] = s < nvalid ? v[s] : 0u;
            if constexpr (ESZ == 4) {
#pragma unroll
                for (int s = 0; s < EPL; ++s) d[s] = v[s];
            } else if constexpr (ESZ == 2) {
#pragma unroll
                for (int s = 0; s < EPL; s += 2) d[s / 2] = v[s] | (v[s + 1] << 16);
            } else {
#pragma unroll
                for (int s = 0; s < EPL; s += 4) d[s / 4] = v[s] | (v[s + 1] << 8) | (v[s + 2] << 16) | (v[s + 3] << 24);
            }
        } else {
            // element by element (kept as a loop: staging runs once per workgroup, and unrolled its code would be large)
#pragma nounroll
            for (int s = 0; s < EPL; ++s) {
                const bool valid = s < nvalid;
                const uint8_t* p = !valid ? w : contiguous ? p0 + s * ESZ
                                 : w + (transposed ? elemOffset(shape, col0 + s, r) : elemOffset(shape, r, col0 + s));
                if constexpr (ESZ == 4)      d[s] = valid ? *(const uint32_t*)p : 0u;
                else if constexpr (ESZ == 2) ((uint16_t*)d)[s] = valid ? *(const uint16_t*)p : (uint16_t)0;
                else                         ((uint8_t*)d)[s] = valid ? (uint8_t)(*p ^ xorByte) : (uint8_t)0;
            }
        }
    }
}

} // namespace cv
