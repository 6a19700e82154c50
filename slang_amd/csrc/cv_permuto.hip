// cv_permuto.hip -- input encoders of the neural module in front of the MLP, for gfx950.
//
// Replaces, for a whole batch of positions, PermutoEncoder::encode and its reverse mode
// (source/standard-modules/neural/permuto-encoder.slang:240-337, readFeatureValueBwd :222-238,
// prepareLevelInfo :339-368) and the grid hashes it is built on
// (source/standard-modules/neural/hash-function.slang:69-151).  One thread handles one position: it
// walks the levels, finds the enclosing simplex of the permutohedral lattice, and gathers D+1 hashed
// feature-table entries per level -- integer hashing plus scattered reads, bound by cache and HBM
// latency, not by arithmetic.  The reverse pass scatters with atomic adds, as the reference does.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstring>

#include "cv_device.h"
#include "cv_error.h"
#include "cv_kernels.h"
#include "cv_launch.h"
#include "cv_permuto_impl.h"

namespace cv {
namespace {

constexpr int kMaxDims = CV_PERMUTO_MAX_DIMS;
constexpr int kMaxLevels = CV_PERMUTO_MAX_LEVELS;

// ---- hashes (hash-function.slang) -----------------------------------------------------------
struct Pcg32 {
    uint64_t state, inc;
    __host__ __device__ uint32_t next()                               // :35-42
    {
        const uint64_t old = state;
        state = old * 0x5851f42d4c957f2dULL + inc;
        const uint32_t xorshifted = (uint32_t)(((old >> 18) ^ old) >> 27);
        const uint32_t rot = (uint32_t)(old >> 59);
        return (xorshifted >> rot) | (xorshifted << ((~rot + 1u) & 31u));
    }
    __host__ __device__ void init(uint64_t initstate, uint64_t initseq = 1)   // :25-32
    {
        state = 0;
        inc = (initseq << 1) | 1u;
        next();
        state += initstate;
        next();
    }
    __host__ __device__ void advance(int64_t delta)                    // :45-65
    {
        uint64_t curMult = 0x5851f42d4c957f2dULL, curPlus = inc, accMult = 1, accPlus = 0;
        for (uint64_t d = (uint64_t)delta; d > 0; d /= 2) {
            if (d & 1) { accMult *= curMult; accPlus = accPlus * curMult + curPlus; }
            curPlus = (curMult + 1) * curPlus;
            curMult *= curMult;
        }
        state = accMult * state + accPlus;
    }
};

__host__ __device__ inline uint32_t baseConvertHash(const uint32_t* pos, int dims)   // :103-113
{
    uint32_t k = 0;
    for (int d = 0; d < dims; ++d) { k += pos[d]; k *= 2531011u; }
    return k;
}

__host__ __device__ inline uint32_t gridHash(int type, const uint32_t* pos, int dims)
{
    const uint32_t prime[7] = {1958374283u, 2654435761u, 805459861u, 3674653429u, 2097192037u, 1434869437u, 2165219737u};
    switch (type) {
    case CV_HASH_PRIME: case CV_HASH_COHERENT_PRIME: case CV_HASH_REVERSED_PRIME: {   // lcgHash, :69-100
        uint32_t r = 0;
        for (int i = 0; i < dims; ++i) {
            uint32_t f = type == CV_HASH_REVERSED_PRIME ? prime[6 - i] : prime[i];
            if (type == CV_HASH_COHERENT_PRIME && i == 0) f = 1u;
            r ^= pos[i] * f;
        }
        return r; }
    case CV_HASH_RNG: {                                                // :117-131
        const int bits = 64 / dims;
        uint64_t step = 0;
        for (int i = 0; i < dims; ++i) step ^= (uint64_t)pos[i] << (i * bits);
        Pcg32 rng;
        rng.init(1337);
        rng.advance((int64_t)step);
        return rng.next(); }
    case CV_HASH_BASE_CONVERT: return baseConvertHash(pos, dims);
    }
    return 0;
}

__global__ __launch_bounds__(256) void gridHashKernel(int type, int dims, const uint8_t* pos, uint64_t stride, uint32_t* out, uint32_t batch)
{
    const uint32_t s = blockIdx.x * 256u + threadIdx.x;
    if (s >= batch) return;
    uint32_t p[7];
    for (int i = 0; i < dims; ++i) p[i] = ((const uint32_t*)(pos + (size_t)s * stride))[i];
    out[s] = gridHash(type, p, dims);
}

// ---- permutohedral lattice --------------------------------------------------------------------
struct PermutoArgs {
    CvPermutoDesc desc;
    const uint8_t* pos; uint64_t posStride;
    const uint8_t* table;
    uint8_t* out; uint64_t outStride;
    const uint8_t* dOut; uint64_t dOutStride;
    uint8_t* dPos; uint64_t dPosStride;
    float* dTable;
    uint32_t batch;
};

template <typename T, int D>
__global__ __launch_bounds__(256) void permutoEncodeKernel(const PermutoArgs a)
{
    const uint32_t s = blockIdx.x * 256u + threadIdx.x;
    if (s >= a.batch) return;
    const int F = a.desc.featureDimensionPerEntry;
    float pos[D];
#pragma unroll
    for (int d = 0; d < D; ++d) pos[d] = (float)((const T*)(a.pos + (size_t)s * a.posStride))[d];
    T* out = (T*)(a.out + (size_t)s * a.outStride);
    const T* table = (const T*)a.table;
    for (uint32_t l = 0; l < a.desc.maxLevels; ++l) {
        const CvPermutoLevelInfo& lv = a.desc.levelInfo[l];
        T* o = out + lv.currentLevelIndex * F;
        for (int f = 0; f < F; ++f) o[f] = (T)0.f;
        if ((float)lv.currentLevelIndex >= a.desc.maxLevel + 1e-3f) continue;   // zero padding beyond maxLevel, :259-262
        float elevated[D + 1], bary[D + 2];
        int rem0[D + 1], rank[D + 1];
        latticeGeometry<D>(pos, lv, elevated, rem0, rank);
        barycentricWeights<D>(elevated, rem0, rank, bary);
        uint32_t idx[D + 1];
        vertexIndices<D>(lv, F, rem0, rank, idx);
        for (int f0 = 0; f0 < F; f0 += 4) {                            // four features of the entry at a time
            T acc[4] = {(T)0.f, (T)0.f, (T)0.f, (T)0.f};
#pragma unroll
            for (int k = 0; k <= D; ++k) {
                const T w = (T)bary[k];
#pragma unroll
                for (int f = 0; f < 4; ++f)
                    if (f0 + f < F) acc[f] = (T)(acc[f] + (T)(w * table[idx[k] + f0 + f]));    // in T, vertex by vertex (:312-316)
            }
#pragma unroll
            for (int f = 0; f < 4; ++f)
                if (f0 + f < F) o[f0 + f] = acc[f];
        }
    }
}

// The same encoding with one thread per (position, level), the level running fastest: a wave's 64 results are
// consecutive in memory (one thread per position writes F elements at the pitch of a whole row, which the memory
// system does not merge: 2.1 bytes written per byte of output), no thread loops over levels, and a feature table that
// fits is held in LDS, where a gather of 64 scattered entries costs a few cycles instead of one cache line per lane.
// The arithmetic per (position, level) is that of permutoEncodeKernel, instruction for instruction.
template <typename T, int D, int F, bool LDS_TABLE>
__global__ __launch_bounds__(1024) void permutoEncodePairsKernel(const PermutoArgs a, uint32_t tableElems, uint32_t levelShift)
{
    typedef typename PermutoEntry<T, F>::type Entry;
    extern __shared__ __align__(16) uint8_t ldsRaw[];
    CvPermutoLevelInfo* levels = (CvPermutoLevelInfo*)ldsRaw;
    const T* ldsTable = (const T*)(ldsRaw + kMaxLevels * sizeof(CvPermutoLevelInfo));
    const uint32_t L = a.desc.maxLevels;
    {
        constexpr uint32_t words = sizeof(CvPermutoLevelInfo) / 4u;
        const uint32_t* src = (const uint32_t*)a.desc.levelInfo;
        for (uint32_t i = threadIdx.x; i < L * words; i += blockDim.x) ((uint32_t*)levels)[i] = src[i];
        if constexpr (LDS_TABLE) {
            const Entry* t = (const Entry*)a.table;
            Entry* dst = (Entry*)(ldsRaw + kMaxLevels * sizeof(CvPermutoLevelInfo));
            for (uint32_t i = threadIdx.x; i < tableElems / (uint32_t)F; i += blockDim.x) dst[i] = t[i];
        }
    }
    __syncthreads();
    const T* table = LDS_TABLE ? ldsTable : (const T*)a.table;
    const uint64_t pairs = (uint64_t)a.batch * L;
    for (uint64_t p = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; p < pairs; p += (uint64_t)gridDim.x * blockDim.x) {
        const uint32_t s = levelShift < 32u ? (uint32_t)(p >> levelShift) : (uint32_t)(p / L);
        const uint32_t l = (uint32_t)(p - (uint64_t)s * L);
        const CvPermutoLevelInfo& lv = levels[l];
        float pos[D];
#pragma unroll
        for (int d = 0; d < D; ++d) pos[d] = (float)((const T*)(a.pos + (size_t)s * a.posStride))[d];
        const Entry acc = permutoEncodeEntry<T, D, F>(pos, lv, table, a.desc.maxLevel);
        // (a streaming store: the encoded vectors are written once and read by the next kernel)
        __builtin_nontemporal_store(acc, (Entry*)((T*)(a.out + (size_t)s * a.outStride) + lv.currentLevelIndex * F));
    }
}

// Reverse mode for one position: adds bary[k] * dOut to the table gradient `dTable` (global memory, or a workgroup's
// private copy in LDS) and, if wanted, writes the position gradient.
// FT: the features per entry when they are 1, 2 or 4 (the loops over them unrolled, the loads of a level issued together:
// with a run-time count every element was a load and a wait of its own), else 0.
template <int D, int FT>
__device__ __forceinline__ void permutoBackwardOne(const PermutoArgs& a, uint32_t s, float* dTable)
{
    const int F = FT ? FT : a.desc.featureDimensionPerEntry;
    float pos[D], dpos[D];
#pragma unroll
    for (int d = 0; d < D; ++d) { pos[d] = ((const float*)(a.pos + (size_t)s * a.posStride))[d]; dpos[d] = 0.f; }
    const float* table = (const float*)a.table;
    const float* g = (const float*)(a.dOut + (size_t)s * a.dOutStride);
    for (uint32_t l = 0; l < a.desc.maxLevels; ++l) {
        const CvPermutoLevelInfo& lv = a.desc.levelInfo[l];
        if ((float)lv.currentLevelIndex >= a.desc.maxLevel + 1e-3f) continue;
        float elevated[D + 1], bary[D + 2], dbary[D + 2];
        int rem0[D + 1], rank[D + 1];
        latticeGeometry<D>(pos, lv, elevated, rem0, rank);
        barycentricWeights<D>(elevated, rem0, rank, bary);
#pragma unroll
        for (int i = 0; i <= D + 1; ++i) dbary[i] = 0.f;
        const float* gl = g + lv.currentLevelIndex * F;
        uint32_t idx[D + 1];
        vertexIndices<D>(lv, F, rem0, rank, idx);
        if constexpr (FT > 0) {
            float gv[FT], tv[D + 1][FT];
#pragma unroll
            for (int f = 0; f < FT; ++f) gv[f] = gl[f];
#pragma unroll
            for (int k = 0; k <= D; ++k)
#pragma unroll
                for (int f = 0; f < FT; ++f) tv[k][f] = table[idx[k] + f];
#pragma unroll
            for (int k = 0; k <= D; ++k) {
#pragma unroll
                for (int f = 0; f < FT; ++f) {
                    if (dTable) atomicAdd(dTable + idx[k] + f, bary[k] * gv[f]);    // readFeatureValueBwd, :222-238
                    dbary[k] += tv[k][f] * gv[f];
                }
            }
        } else {
#pragma unroll
            for (int k = 0; k <= D; ++k) {
                for (int f = 0; f < F; ++f) {
                    if (dTable) atomicAdd(dTable + idx[k] + f, bary[k] * gl[f]);    // readFeatureValueBwd, :222-238
                    dbary[k] += table[idx[k] + f] * gl[f];
                }
            }
        }
        if (!a.dPos) continue;
        dbary[D + 1] += dbary[0];                                      // the wrap-around term of barycentric[0]
        float delev[D + 1];
#pragma unroll
        for (int dim = 0; dim <= D; ++dim) {
            float plus = 0.f, minus = 0.f;
#pragma unroll
            for (int i = 0; i <= D + 1; ++i) {
                if (i == D - rank[dim]) plus = dbary[i];
                if (i == D + 1 - rank[dim]) minus = dbary[i];
            }
            delev[dim] = (plus - minus) * (1.0f / (float)(D + 1));
        }
        // elevate: e[dim+1] = sum - (dim+1) cf, sum += cf for dim = D-1..0, e[0] = sum
        float dsum = delev[0];
#pragma unroll
        for (int dim = 0; dim < D; ++dim) {
            const float dcf = dsum - (float)(dim + 1) * delev[dim + 1];
            dsum += delev[dim + 1];
            dpos[dim] += dcf * lv.scalesPerDim[dim];
        }
    }
    if (a.dPos) {
#pragma unroll
        for (int d = 0; d < D; ++d) ((float*)(a.dPos + (size_t)s * a.dPosStride))[d] = dpos[d];
    }
}

template <int D, int FT>
__global__ __launch_bounds__(256) void permutoBackwardKernel(const PermutoArgs a)
{
    const uint32_t s = blockIdx.x * 256u + threadIdx.x;
    if (s >= a.batch) return;
    permutoBackwardOne<D, FT>(a, s, a.dTable);
}

// A small feature table (the reference's own test: 2 048 floats) receives every position's atomic adds on a handful of
// addresses: 2^22 positions took 123 ms that way.  Here a workgroup accumulates into a private copy of the table in
// LDS and adds that copy to the table gradient once, at its end: the atomic traffic to memory shrinks by the number
// of positions per workgroup.
// As many copies of the table as fit (a power of two, up to 16) share the lanes of a wave among them: lanes of one
// instruction that add to the same address are served one after the other, and with 64 lanes on a level of a few hundred
// entries that is the common case (measured: 230 cycles per LDS atomic instruction with one copy).
template <int D, int FT>
__global__ __launch_bounds__(1024) void permutoBackwardLdsKernel(const PermutoArgs a, uint32_t tableElems, uint32_t copies)
{
    extern __shared__ float ldsTable[];
    for (uint32_t i = threadIdx.x; i < tableElems * copies; i += blockDim.x) ldsTable[i] = 0.f;
    __syncthreads();
    float* mine = ldsTable + (threadIdx.x & (copies - 1u)) * tableElems;
    for (uint64_t s = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; s < a.batch; s += (uint64_t)gridDim.x * blockDim.x)
        permutoBackwardOne<D, FT>(a, (uint32_t)s, mine);
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < tableElems; i += blockDim.x) {
        float v = ldsTable[i];
        for (uint32_t c = 1; c < copies; ++c) v += ldsTable[c * tableElems + i];
        if (v != 0.f) atomicAdd(a.dTable + i, v);
    }
}

// the table as the levels lay it out: offsets and sizes in entries, F elements per entry
uint64_t tableElements(const CvPermutoDesc& d)
{
    uint64_t n = 0;
    for (uint32_t l = 0; l < d.maxLevels; ++l) {
        const uint64_t e = ((uint64_t)d.levelInfo[l].offsetOfFeatureTable + d.levelInfo[l].featureTableSize) * (uint64_t)d.featureDimensionPerEntry;
        n = e > n ? e : n;
    }
    return n;
}

constexpr size_t kPairsLevelBytes = kMaxLevels * sizeof(CvPermutoLevelInfo);
constexpr size_t kPairsTableBytes = 144 * 1024;      // with the level records: within the 160 KB of a compute unit

template <typename T, int D, int F>
hipError_t launchEncodePairs(hipStream_t stream, const PermutoArgs& a)
{
    const uint64_t tableElems = tableElements(a.desc);
    const bool inLds = tableElems * sizeof(T) <= kPairsTableBytes;
    const size_t lds = kPairsLevelBytes + (inLds ? (size_t)tableElems * sizeof(T) : 0);
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    const uint64_t pairs = (uint64_t)a.batch * a.desc.maxLevels, want = (pairs + 1023u) / 1024u;
    const uint64_t cap = (uint64_t)cus * (lds <= 80 * 1024 ? 2u : 1u);
    const dim3 grid((uint32_t)(want < cap ? want : cap)), block(1024);
    const uint32_t L = a.desc.maxLevels;
    const uint32_t shift = (L & (L - 1u)) == 0u ? (uint32_t)__builtin_ctz(L) : 0xffffffffu;
    hipError_t e;
    if (inLds) {
        e = allowDynamicLds<permutoEncodePairsKernel<T, D, F, true>>((int)(kPairsLevelBytes + kPairsTableBytes));
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL((permutoEncodePairsKernel<T, D, F, true>), grid, block, lds, stream, a, (uint32_t)tableElems, shift);
    } else {
        hipLaunchKernelGGL((permutoEncodePairsKernel<T, D, F, false>), grid, block, lds, stream, a, (uint32_t)tableElems, shift);
    }
    return hipGetLastError();
}

// the kernel above takes entries of 4, 8 or 16 bytes at addresses that are multiples of their size
template <typename T>
bool pairsEligible(const PermutoArgs& a)
{
    const size_t eb = (size_t)a.desc.featureDimensionPerEntry * sizeof(T);
    const int F = a.desc.featureDimensionPerEntry;
    if (a.desc.dimensions > 4 || (F != 1 && F != 2 && F != 4 && F != 8) || eb > 16) return false;
    return (uintptr_t)a.table % eb == 0 && (uintptr_t)a.out % eb == 0 && a.outStride % eb == 0 && tableElements(a.desc) <= 0xffffffffull;
}

template <typename T>
hipError_t launchEncode(hipStream_t stream, const PermutoArgs& a)
{
    if (pairsEligible<T>(a)) {
        noteKernel(false, "permutoEncodePairsKernel<%s,D=%d,F=%d>", sizeof(T) == 4 ? "f32" : "f16", a.desc.dimensions, a.desc.featureDimensionPerEntry);
        switch (a.desc.dimensions * 16 + a.desc.featureDimensionPerEntry) {
#define CV_DF(N, G) case N * 16 + G: if constexpr (G * sizeof(T) <= 16) return launchEncodePairs<T, N, G>(stream, a); break;
        CV_DF(1, 1) CV_DF(1, 2) CV_DF(1, 4) CV_DF(1, 8) CV_DF(2, 1) CV_DF(2, 2) CV_DF(2, 4) CV_DF(2, 8)
        CV_DF(3, 1) CV_DF(3, 2) CV_DF(3, 4) CV_DF(3, 8) CV_DF(4, 1) CV_DF(4, 2) CV_DF(4, 4) CV_DF(4, 8)
#undef CV_DF
        }
    }
    noteKernel(false, "permutoEncodeKernel<%s,D=%d>", sizeof(T) == 4 ? "f32" : "f16", a.desc.dimensions);
    const dim3 grid((a.batch + 255) / 256), block(256);
    switch (a.desc.dimensions) {
#define CV_D(N) case N: hipLaunchKernelGGL((permutoEncodeKernel<T, N>), grid, block, 0, stream, a); break;
    CV_D(1) CV_D(2) CV_D(3) CV_D(4) CV_D(5) CV_D(6) CV_D(7) CV_D(8)
#undef CV_D
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launchBackward(hipStream_t stream, const PermutoArgs& a)
{
    const uint64_t tableElems = tableElements(a.desc);
    const int fe = a.desc.featureDimensionPerEntry, ft = (fe == 1 || fe == 2 || fe == 4) ? fe : 0;
    constexpr uint64_t kLdsTableBytes = 64 * 1024;
    if (a.dTable && tableElems * 4 <= kLdsTableBytes && a.batch >= 4096u) {
        int dev = 0, cus = 256;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
        uint32_t copies = 1;
        while (copies < 16u && (size_t)tableElems * 4 * (copies * 2u) <= 2 * kLdsTableBytes) copies *= 2u;
        const size_t lds = (size_t)tableElems * 4 * copies;
        // workgroups of 16 waves, one or two to a compute unit as the copies leave room
        const uint32_t want = (a.batch + 1023u) / 1024u, cap = (uint32_t)cus * (lds <= 80 * 1024 ? 2u : 1u);
        const dim3 grid(want < cap ? want : cap), block(1024);
        noteKernel(false, "permutoBackwardLdsKernel<D=%d,%u copies>", a.desc.dimensions, copies);
        switch (a.desc.dimensions * 8 + ft) {
#define CV_DF(N, G) case N * 8 + G: { \
            const hipError_t e = allowDynamicLds<permutoBackwardLdsKernel<N, G>>((int)(2 * kLdsTableBytes)); \
            if (e != hipSuccess) return e; \
            hipLaunchKernelGGL((permutoBackwardLdsKernel<N, G>), grid, block, lds, stream, a, (uint32_t)tableElems, copies); break; }
#define CV_D(N) CV_DF(N, 0) CV_DF(N, 1) CV_DF(N, 2) CV_DF(N, 4)
        CV_D(1) CV_D(2) CV_D(3) CV_D(4) CV_D(5) CV_D(6) CV_D(7) CV_D(8)
#undef CV_D
#undef CV_DF
        default: return hipErrorInvalidValue;
        }
        return hipGetLastError();
    }
    noteKernel(false, "permutoBackwardKernel<D=%d>", a.desc.dimensions);
    const dim3 grid((a.batch + 255) / 256), block(256);
    switch (a.desc.dimensions * 8 + ft) {
#define CV_DF(N, G) case N * 8 + G: hipLaunchKernelGGL((permutoBackwardKernel<N, G>), grid, block, 0, stream, a); break;
#define CV_D(N) CV_DF(N, 0) CV_DF(N, 1) CV_DF(N, 2) CV_DF(N, 4)
    CV_D(1) CV_D(2) CV_D(3) CV_D(4) CV_D(5) CV_D(6) CV_D(7) CV_D(8)
#undef CV_D
#undef CV_DF
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

} // namespace

CvResult checkPermutoDesc(const char* who, const CvPermutoDesc* d)
{
    if (!d) return failWith(CV_E_INVALID_ARG, "%s: desc is null", who);
    if (d->dimensions < 1 || d->dimensions > kMaxDims) return failWith(CV_E_INVALID_ARG, "%s: dimensions=%d (1..%d)", who, d->dimensions, kMaxDims);
    if (d->featureDimensionPerEntry < 1 || d->featureDimensionPerEntry > 64)
        return failWith(CV_E_INVALID_ARG, "%s: featureDimensionPerEntry=%d (1..64)", who, d->featureDimensionPerEntry);
    if (d->maxLevels < 1 || d->maxLevels > (uint32_t)kMaxLevels) return failWith(CV_E_INVALID_ARG, "%s: maxLevels=%u (1..%d)", who, d->maxLevels, kMaxLevels);
    if (d->elementType != CV_FLOAT32 && d->elementType != CV_FLOAT16)
        return failWith(CV_E_NOT_AVAILABLE, "%s: elementType %d (supported: FLOAT32, FLOAT16)", who, d->elementType);
    for (uint32_t l = 0; l < d->maxLevels; ++l)
        if (d->levelInfo[l].featureTableSize == 0 || d->levelInfo[l].currentLevelIndex >= d->maxLevels)
            return failWith(CV_E_INVALID_ARG, "%s: level %u: empty feature table or level index %u out of range", who, l, d->levelInfo[l].currentLevelIndex);
    return CV_OK;
}

} // namespace cv

extern "C" {

CV_API CvResult cvGridHash(void* stream, int32_t hashType, int32_t dimensions, const void* positions, size_t positionStride,
                           uint32_t* out, uint32_t batch)
{
    using namespace cv;
    if (hashType < CV_HASH_PRIME || hashType > CV_HASH_BASE_CONVERT) return failWith(CV_E_INVALID_ARG, "cvGridHash: unknown hash type %d", hashType);
    if (dimensions < 1 || dimensions > 7) return failWith(CV_E_INVALID_ARG, "cvGridHash: dimensions=%d (1..7, the prime table of the reference)", dimensions);
    if (batch == 0) return CV_OK;
    if (!positions || !out || (uintptr_t)positions % 4 || positionStride % 4 || (uintptr_t)out % 4 ||
        (batch > 1 && positionStride < (size_t)dimensions * 4))
        return failWith(CV_E_INVALID_ARG, "cvGridHash: null or misaligned argument");
    noteKernel(false, "gridHashKernel");
    hipLaunchKernelGGL(gridHashKernel, dim3((batch + 255) / 256), dim3(256), 0, (hipStream_t)stream, hashType, dimensions,
                       (const uint8_t*)positions, (uint64_t)positionStride, out, batch);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return failWith(CV_E_INTERNAL_FAIL, "cvGridHash launch: %s", hipGetErrorString(e));
    return CV_OK;
}

CV_API CvResult cvPermutoPrepareLevels(CvPermutoDesc* d, float baseScale, float log2PerLevelScale, float maxLevelRatio, uint32_t seed)
{
    using namespace cv;
    if (!d) return failWith(CV_E_INVALID_ARG, "cvPermutoPrepareLevels: desc is null");
    if (d->dimensions < 1 || d->dimensions > kMaxDims || d->maxLevels < 1 || d->maxLevels > (uint32_t)kMaxLevels || d->log2HashmapSize > 30)
        return failWith(CV_E_INVALID_ARG, "cvPermutoPrepareLevels: dimensions=%d maxLevels=%u log2HashmapSize=%u", d->dimensions, d->maxLevels, d->log2HashmapSize);
    const uint32_t size = 1u << d->log2HashmapSize;
    d->maxLevel = maxLevelRatio * (float)d->maxLevels;
    for (uint32_t level = 0; level < d->maxLevels; ++level) {          // prepareLevelInfo, permuto-encoder.slang:339-368
        CvPermutoLevelInfo& lv = d->levelInfo[level];
        memset(&lv, 0, sizeof(lv));
        lv.currentLevelIndex = level;
        lv.featureTableSize = size;
        lv.offsetOfFeatureTable = level * size;
        lv.scale = baseScale * exp2f((float)level * log2PerLevelScale);
        Pcg32 rng;
        rng.init(seed);
        rng.advance((int64_t)(level * (uint32_t)d->dimensions));
        for (int dim = 0; dim < d->dimensions; ++dim) {
            lv.scalesPerDim[dim] = lv.scale * (1.0f / sqrtf((float)((dim + 1) * (dim + 2))));
            const float r = (float)rng.next() * (1.0f / 4294967296.0f);
            lv.shiftsPerDim[dim] = r * 10.0f - 5.0f;
        }
    }
    return CV_OK;
}

CV_API CvResult cvPermutoEncode(void* stream, const CvPermutoDesc* desc, const void* positions, size_t positionStride,
                                const void* featureTable, void* out, size_t outStride, uint32_t batch)
{
    using namespace cv;
    CvResult rc = checkPermutoDesc("cvPermutoEncode", desc);
    if (CV_FAILED(rc)) return rc;
    if (batch == 0) return CV_OK;
    const uint32_t esz = desc->elementType == CV_FLOAT32 ? 4u : 2u;
    const size_t nOut = (size_t)desc->maxLevels * desc->featureDimensionPerEntry;
    if (!positions || !featureTable || !out || (uintptr_t)positions % esz || positionStride % esz || (uintptr_t)featureTable % esz ||
        (uintptr_t)out % esz || outStride % esz ||
        (batch > 1 && (positionStride < (size_t)desc->dimensions * esz || outStride < nOut * esz)))
        return failWith(CV_E_INVALID_ARG, "cvPermutoEncode: null, misaligned or overlapping-row argument");
    PermutoArgs a;
    memset(&a, 0, sizeof(a));
    a.desc = *desc;
    a.pos = (const uint8_t*)positions; a.posStride = positionStride; a.table = (const uint8_t*)featureTable;
    a.out = (uint8_t*)out; a.outStride = outStride; a.batch = batch;
    const hipError_t e = esz == 4 ? launchEncode<float>((hipStream_t)stream, a) : launchEncode<half_t>((hipStream_t)stream, a);
    if (e != hipSuccess) return failWith(CV_E_INTERNAL_FAIL, "cvPermutoEncode launch: %s", hipGetErrorString(e));
    return CV_OK;
}

CV_API CvResult cvPermutoEncodeBackward(void* stream, const CvPermutoDesc* desc, const void* positions, size_t positionStride,
                                        const void* featureTable, const void* dOut, size_t dOutStride,
                                        void* dPositions, size_t dPositionStride, void* dFeatureTable, uint32_t batch)
{
    using namespace cv;
    CvResult rc = checkPermutoDesc("cvPermutoEncodeBackward", desc);
    if (CV_FAILED(rc)) return rc;
    if (desc->elementType != CV_FLOAT32)
        return failWith(CV_E_NOT_AVAILABLE, "cvPermutoEncodeBackward: FLOAT32 data only (the table gradient is accumulated with fp32 atomic adds)");
    if (batch == 0) return CV_OK;
    const size_t nOut = (size_t)desc->maxLevels * desc->featureDimensionPerEntry;
    if (!positions || !featureTable || !dOut || (uintptr_t)positions % 4 || positionStride % 4 || (uintptr_t)featureTable % 4 ||
        (uintptr_t)dOut % 4 || dOutStride % 4 || (uintptr_t)dPositions % 4 || dPositionStride % 4 || (uintptr_t)dFeatureTable % 4 ||
        (batch > 1 && (positionStride < (size_t)desc->dimensions * 4 || dOutStride < nOut * 4 ||
                       (dPositions && dPositionStride < (size_t)desc->dimensions * 4))))
        return failWith(CV_E_INVALID_ARG, "cvPermutoEncodeBackward: null, misaligned or overlapping-row argument");
    PermutoArgs a;
    memset(&a, 0, sizeof(a));
    a.desc = *desc;
    a.pos = (const uint8_t*)positions; a.posStride = positionStride; a.table = (const uint8_t*)featureTable;
    a.dOut = (const uint8_t*)dOut; a.dOutStride = dOutStride;
    a.dPos = (uint8_t*)dPositions; a.dPosStride = dPositionStride; a.dTable = (float*)dFeatureTable; a.batch = batch;
    const hipError_t e = launchBackward((hipStream_t)stream, a);
    if (e != hipSuccess) return failWith(CV_E_INTERNAL_FAIL, "cvPermutoEncodeBackward launch: %s", hipGetErrorString(e));
    return CV_OK;
}

} // extern "C"
