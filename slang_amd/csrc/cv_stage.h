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

// The EPL elements of lane-chunk c (chunk = 64 * fragment + lane) of that arrangement, fetched from memory into
// CHUNK / 4 registers (zero where the matrix ends).  xorByte (1-byte types only): XORed into every valid element on the
// way, used to re-bias unsigned bytes to signed ones (u ^ 0x80 == u - 128 as int8); padding stays zero.
template <int ESZ, int EPL>
__device__ __forceinline__ void fetchFragmentChunk(uint32_t (&out)[ESZ * EPL / 4], const uint8_t* w, const MatrixShape& shape,
                                                   bool transposed, bool direct, int MT, int KT, uint32_t gs, uint32_t rows,
                                                   uint32_t cols, uint32_t rowOff, uint32_t xorByte, int c)
{
    constexpr int CHUNK = ESZ * EPL;              // bytes of one lane-chunk: 8, 16 or 32
    static_assert(ESZ == 1 || ESZ == 2 || ESZ == 4, "element size");
    static_assert(CHUNK % 8 == 0, "a lane-chunk is a whole number of 8-byte words");
    if (direct) {                                 // the source is in fragment order already
        if constexpr (CHUNK % 16 == 0) {
#pragma unroll
            for (int i16 = 0; i16 < CHUNK / 16; ++i16) {
                const u32x4 x = ((const u32x4*)(w + (size_t)c * CHUNK))[i16];
                out[4 * i16] = x.x; out[4 * i16 + 1] = x.y; out[4 * i16 + 2] = x.z; out[4 * i16 + 3] = x.w;
            }
        } else {
            const u32x2 x = *(const u32x2*)(w + (size_t)c * CHUNK);
            out[0] = x.x; out[1] = x.y;
        }
        return;
    }
    const uint32_t xorWord = xorByte * 0x01010101u;
    const int ROWS = 4 * MT;
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
    const uint32_t r = rowOff + row;
    if (shape.layout == kRowMajor || shape.layout == kColumnMajor) {
        // A linear layout: element (mr, mc) of the matrix in memory lies at mr * sr + mc * sc, and the chunk's
        // elements follow one another at a fixed step (the element size when they are neighbours in memory).  All
        // loads of the chunk are in flight together, from always-valid addresses, masked afterwards.
        const size_t line = shape.stride ? shape.stride : (size_t)(shape.layout == kRowMajor ? shape.cols : shape.rows) * ESZ;
        const size_t sr = shape.layout == kRowMajor ? line : (size_t)ESZ, sc = shape.layout == kRowMajor ? (size_t)ESZ : line;
        const size_t step = transposed ? sr : sc;
        const uint8_t* p0 = nvalid > 0 ? w + (transposed ? (size_t)col0 * sr + (size_t)r * sc : (size_t)r * sr + (size_t)col0 * sc) : w;
        if (step == (size_t)ESZ && nvalid == EPL && ((uintptr_t)p0 & 7) == 0) {
#pragma unroll
            for (int i8 = 0; i8 < CHUNK / 8; ++i8) {
                const u32x2 x = ((const u32x2*)p0)[i8];
                out[2 * i8] = x.x ^ xorWord; out[2 * i8 + 1] = x.y ^ xorWord;
            }
            return;
        }
        uint32_t v[EPL];
#pragma unroll
        for (int s = 0; s < EPL; ++s) {
            const uint8_t* p = s < nvalid ? p0 + (size_t)s * step : w;
            if constexpr (ESZ == 4)      v[s] = *(const uint32_t*)p;
            else if constexpr (ESZ == 2) v[s] = *(const uint16_t*)p;
            else                         v[s] = (uint32_t)(*p ^ xorByte);
        }
#pragma unroll
        for (int s = 0; s < EPL; ++s) v[s] = s < nvalid ? v[s] : 0u;
        if constexpr (ESZ == 4) {
#pragma unroll
            for (int s = 0; s < EPL; ++s) out[s] = v[s];
        } else if constexpr (ESZ == 2) {
#pragma unroll
            for (int s = 0; s < EPL; s += 2) out[s / 2] = v[s] | (v[s + 1] << 16);
        } else {
#pragma unroll
            for (int s = 0; s < EPL; s += 4) out[s / 4] = v[s] | (v[s + 1] << 8) | (v[s + 2] << 16) | (v[s + 3] << 24);
        }
        return;
    }
    // An Optimal layout that is not this fragment order (transposed, a block of rows, another tiling): element by
    // element through the layout's index map, kept as a loop (its code is long, and this path is rare).
#pragma unroll
    for (int d = 0; d < CHUNK / 4; ++d) out[d] = 0u;
#pragma nounroll
    for (int s = 0; s < nvalid; ++s) {
        const uint8_t* p = w + (transposed ? elemOffset(shape, col0 + s, r) : elemOffset(shape, r, col0 + s));
        uint32_t e;
        if constexpr (ESZ == 4)      e = *(const uint32_t*)p;
        else if constexpr (ESZ == 2) e = *(const uint16_t*)p;
        else                         e = (uint32_t)(*p ^ xorByte);
        constexpr int PER = 4 / ESZ;                   // elements per register
        const int d = s / PER, sh = (s % PER) * 8 * ESZ;
#pragma unroll
        for (int k = 0; k < CHUNK / 4; ++k) out[k] |= k == d ? e << sh : 0u;      // (no dynamic register index)
    }
}

template <int DW>
__device__ __forceinline__ void storeFragmentChunk(uint32_t* d, const uint32_t (&v)[DW])
{
    if constexpr (DW % 4 == 0) {
#pragma unroll
        for (int i = 0; i < DW; i += 4) *(u32x4*)(d + i) = u32x4{v[i], v[i + 1], v[i + 2], v[i + 3]};
    } else {
#pragma unroll
        for (int i = 0; i < DW; i += 2) *(u32x2*)(d + i) = u32x2{v[i], v[i + 1]};
    }
}

template <int ESZ, int EPL>
__host__ __device__ __forceinline__ bool fragmentSourceIsDirect(const MatrixShape& shape, bool transposed, int MT, int KT, uint32_t gs,
                                                       uint32_t rows, uint32_t cols, uint32_t rowOff, uint32_t xorByte)
{
    return shape.layout == kInferencingOptimal && !transposed && rowOff == 0 && xorByte == 0 &&
           optMT(shape.rows) == (uint32_t)MT && optKT(shape.cols, EPL) == (uint32_t)KT && optGS(shape.cols) == gs &&
           shape.rows == rows && shape.cols == cols;
}

// firstThread: the thread that takes chunk 0.  A kernel that stages several small matrices gives each its own
// part of the workgroup, so that their round trips to memory overlap instead of following one another.
template <int ESZ, int EPL>
__device__ __forceinline__ void stageFragments(uint32_t* ldsDst, const uint8_t* w, const MatrixShape& shape,
                                               bool transposed, int MT, int KT, uint32_t gs, uint32_t rows,
                                               uint32_t cols, uint32_t rowOff = 0, uint32_t xorByte = 0,
                                               uint32_t firstThread = 0)
{
    constexpr int DW = ESZ * EPL / 4;
    const int chunks = MT * KT * 64;
    const bool direct = fragmentSourceIsDirect<ESZ, EPL>(shape, transposed, MT, KT, gs, rows, cols, rowOff, xorByte);
    const uint32_t vt = threadIdx.x >= firstThread ? threadIdx.x - firstThread : threadIdx.x + blockDim.x - firstThread;
    for (int c = (int)vt; c < chunks; c += blockDim.x) {
        uint32_t v[DW];
        fetchFragmentChunk<ESZ, EPL>(v, w, shape, transposed, direct, MT, KT, gs, rows, cols, rowOff, xorByte, c);
        storeFragmentChunk<DW>(ldsDst + (size_t)c * DW, v);
    }
}

// One lane-chunk per thread in two passes, for kernels whose cost is launch latency: request() only issues loads, all
// from addresses that exist, and finish() masks and stores.  Between the two a kernel requests its other chunks and
// whatever else it needs at its start, so that all of it costs one round trip to memory.  Takes a matrix already in this
// fragment order (kChunkDirect), or a RowMajor one whose rows are whole aligned dwords (kChunkRowDwords: a chunk then is
// up to CHUNK / 4 neighbouring dwords of a row).  The kind is a template parameter, so that a request is straight-line
// code; chunkInFlightKind names it on the host (kChunkNone: the source goes through stageFragments).
enum : int { kChunkNone = 0, kChunkRowDwords = 1, kChunkDirect = 2 };
template <int ESZ, int EPL>
__host__ __device__ __forceinline__ int chunkInFlightKind(const uint8_t* w, const MatrixShape& shape, int MT, int KT, uint32_t gs,
                                                          uint32_t rows, uint32_t cols)
{
    if (shape.layout == kRowMajor)
        return ((uintptr_t)w & 3u) == 0 && (shape.stride & 3u) == 0 && ((size_t)shape.cols * ESZ & 3u) == 0 ? kChunkRowDwords : kChunkNone;
    return fragmentSourceIsDirect<ESZ, EPL>(shape, false, MT, KT, gs, rows, cols, 0, 0) ? kChunkDirect : kChunkNone;
}

// v: the chunk's dwords as they lie in memory; validBytes: how many of its bytes exist
template <int ESZ, int EPL, int KIND>
struct ChunkInFlight {
    static constexpr int CHUNK = ESZ * EPL, DW = CHUNK / 4;
    static_assert(ESZ <= 2 && (CHUNK == 8 || CHUNK == 16), "one or two 8-byte words per lane-chunk");
    static_assert(KIND == kChunkRowDwords || KIND == kChunkDirect, "kind of source");
    static __device__ __forceinline__ void request(uint32_t (&v)[DW], int& validBytes, const uint8_t* w, const MatrixShape& shape,
                                                   int MT, int KT, uint32_t gs, uint32_t rows, uint32_t cols, int c)
    {
        if constexpr (KIND == kChunkDirect) {
            validBytes = CHUNK;
            if constexpr (DW == 4) {
                const u32x4 x = *(const u32x4*)(w + (size_t)c * CHUNK);
                v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
            } else {
                const u32x2 x = *(const u32x2*)(w + (size_t)c * CHUNK);
                v[0] = x.x; v[1] = x.y;
            }
            return;
        }
        // (the geometry of fetchFragmentChunk)
        const int lane = c & 63, f = c >> 6;
        const int kt = f % KT, t = f / KT, g = lane >> 4, i = lane & 15;
        const uint32_t row = (uint32_t)((i >> 2) * 4 * MT + 4 * t + (i & 3));
        const uint32_t q0 = (uint32_t)(kt * EPL), col0 = g * gs + q0;
        int nvalid = 0;
        if (row < rows && q0 < gs && col0 < cols) {
            const uint32_t a = gs - q0, b = cols - col0;
            nvalid = (int)(a < b ? a : b);
            if (nvalid > EPL) nvalid = EPL;
        }
        validBytes = nvalid * ESZ;
        const size_t line = shape.stride ? shape.stride : (size_t)shape.cols * ESZ;
        const size_t first = nvalid > 0 ? (size_t)row * line + (size_t)col0 * ESZ : 0;
#pragma unroll
        for (int d = 0; d < DW; ++d) v[d] = *(const uint32_t*)(w + (4 * d < validBytes ? first + 4 * d : 0));
    }
    static __device__ __forceinline__ void finish(const uint32_t (&v)[DW], int validBytes, uint32_t* ldsDst)
    {
        uint32_t out[DW];
#pragma unroll
        for (int d = 0; d < DW; ++d) out[d] = 4 * d < validBytes ? v[d] : 0u;
        storeFragmentChunk<DW>(ldsDst, out);
    }
};

// The same in two passes, for kernels that stage several matrices: load() of every matrix first, then store() of
// every matrix, so that all of a thread's loads are in flight together and the whole staging costs one round trip to
// memory instead of one per matrix (fifteen of them, 14 us, at the head of the paired training kernel).  ITERS: chunks
// per thread, ceil(MT * KT * 64 / BLOCK) for the largest matrix staged through this object's type.
template <int ESZ, int EPL, int ITERS, int BLOCK>
struct FragmentStage {
    static constexpr int DW = ESZ * EPL / 4;
    uint32_t v[ITERS][DW];
    __device__ __forceinline__ void load(const uint8_t* w, const MatrixShape& shape, bool transposed, int MT, int KT, uint32_t gs,
                                         uint32_t rows, uint32_t cols)
    {
        const int chunks = MT * KT * 64;
        const bool direct = fragmentSourceIsDirect<ESZ, EPL>(shape, transposed, MT, KT, gs, rows, cols, 0, 0);
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int c = (int)threadIdx.x + it * BLOCK;
            // (a chunk past the end fetches chunk 0 and is dropped at store(): no branch around the loads)
            fetchFragmentChunk<ESZ, EPL>(v[it], w, shape, transposed, direct, MT, KT, gs, rows, cols, 0, 0, c < chunks ? c : 0);
        }
    }
    __device__ __forceinline__ void store(uint32_t* ldsDst, int MT, int KT) const
    {
        const int chunks = MT * KT * 64;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int c = (int)threadIdx.x + it * BLOCK;
            if (c < chunks) {
                storeFragmentChunk<DW>(ldsDst + (size_t)c * DW, v[it]);
            }
        }
    }
};

} // namespace cv
