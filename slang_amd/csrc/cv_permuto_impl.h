// cv_permuto_impl.h -- geometry of the permutohedral lattice shared by the encoder kernels.
//
// Device-side restatement of the per-level steps of PermutoEncoder::encode
// (source/standard-modules/neural/permuto-encoder.slang:240-337): elevate the position, find the closest
// remainder-0 lattice point and the ranks (:74-152), the barycentric weights (:166-179) and the hashed
// feature-table slots of the D+1 vertices of the enclosing simplex (:296-309).  Line numbers in the comments below refer
// to that file.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "coopvec.h"

namespace cv {

// elevated point, closest remainder-0 point and rank of one position on one level (:74-152)
template <int D>
__device__ __forceinline__ void latticeGeometry(const float* pos, const CvPermutoLevelInfo& lv, float* elevated, int* rem0, int* rank)
{
    float sum = 0.0f;
#pragma unroll
    for (int dim = D - 1; dim >= 0; --dim) {
        const float cf = (pos[dim] + lv.shiftsPerDim[dim]) * lv.scalesPerDim[dim];
        elevated[dim + 1] = sum - (float)(dim + 1) * cf;
        sum += cf;
    }
    elevated[0] = sum;
    int isum = 0;
#pragma unroll
    for (int dim = 0; dim <= D; ++dim) {
        rank[dim] = 0;
        const float v = elevated[dim] * (1.0f / (float)(D + 1));
        const float up = ceilf(v) * (float)(D + 1), down = floorf(v) * (float)(D + 1);
        rem0[dim] = (up - elevated[dim] < elevated[dim] - down) ? (int)up : (int)down;
        isum += rem0[dim];
    }
    isum /= (D + 1);
#pragma unroll
    for (int dim = 0; dim < D; ++dim) {
        const float di = elevated[dim] - (float)rem0[dim];
#pragma unroll
        for (int other = dim + 1; other <= D; ++other) {
            if (di < elevated[other] - (float)rem0[other]) rank[dim]++;
            else rank[other]++;
        }
    }
#pragma unroll
    for (int dim = 0; dim <= D; ++dim) {
        rank[dim] += isum;
        const int wrap = rank[dim] < 0 ? D + 1 : (rank[dim] > D ? -(D + 1) : 0);     // :146-156, as selects
        rank[dim] += wrap;
        rem0[dim] += wrap;
    }
}

// barycentric[k] of the remainder-k vertex (:166-179).  The reference indexes the array with the ranks
// (barycentric[D - rank] += delta, barycentric[D + 1 - rank] -= delta); the ranks being a permutation of 0..D, entry i
// receives the delta of the dimension ranked D - i and loses that of the dimension ranked D + 1 - i.  Here the deltas
// are first put in rank order by selects (registers cannot be indexed by a run-time value), then every entry is one
// difference: 0 + a - b and 0 - b + a round to the same value, also when a or b is a signed zero.
template <int D>
__device__ __forceinline__ void barycentricWeights(const float* elevated, const int* rem0, const int* rank, float* bary)
{
    float delta[D + 1], sorted[D + 1];
#pragma unroll
    for (int dim = 0; dim <= D; ++dim) delta[dim] = (elevated[dim] - (float)rem0[dim]) * (1.0f / (float)(D + 1));
#pragma unroll
    for (int r = 0; r <= D; ++r) {
        float v = delta[D];
#pragma unroll
        for (int dim = D - 1; dim >= 0; --dim) v = rank[dim] == r ? delta[dim] : v;
        sorted[r] = v;
    }
    bary[D + 1] = 0.0f - sorted[0];
#pragma unroll
    for (int i = 1; i <= D; ++i) bary[i] = (0.0f + sorted[D - i]) - sorted[D + 1 - i];
    bary[0] = (0.0f + sorted[D]) + (1.0f + bary[D + 1]);
}

// Feature-table offsets (in elements) of the D+1 vertices of the simplex (:296-309).  The key of vertex k is
// rem0[dim] + k, less D+1 in the dimensions ranked above D - k; baseConvertHash is linear modulo 2^32
// (hash = sum key[d] * c^(D-d)), so the hash of vertex k is that of vertex k-1 plus the sum of the multipliers, less
// (D+1) times the multiplier of the dimension ranked D+1-k: three integer multiplies per position instead of three per
// vertex, same 32-bit values.
template <int D>
__device__ __forceinline__ void vertexIndices(const CvPermutoLevelInfo& lv, int F, const int* rem0, const int* rank, uint32_t* idx)
{
    constexpr uint32_t c = 2531011u;
    uint32_t mult[D], all = 0u, p = c;
#pragma unroll
    for (int dim = D - 1; dim >= 0; --dim) { mult[dim] = p; all += p; p *= c; }
    uint32_t hash = 0u;
#pragma unroll
    for (int dim = 0; dim < D; ++dim) hash += (uint32_t)rem0[dim] * mult[dim];
    // (a table of 2^n entries, which is what prepareLevelInfo makes, is indexed with a mask: the general remainder
    // is a division by a run-time value, some forty instructions per vertex)
    const uint32_t size = lv.featureTableSize, base = lv.offsetOfFeatureTable * (uint32_t)F;
    const bool pow2 = (size & (size - 1u)) == 0u;
#pragma unroll
    for (int k = 0; k <= D; ++k) {
        if (k > 0) {
            uint32_t less = 0u;
#pragma unroll
            for (int dim = 0; dim < D; ++dim) less = rank[dim] == D + 1 - k ? (uint32_t)(D + 1) * mult[dim] : less;
            hash += all - less;
        }
        const uint32_t slot = pow2 ? (hash & (size - 1u)) : hash % size;
        idx[k] = base + slot * (uint32_t)F;
    }
}

// F consecutive elements of type T: one entry of the feature table, one level's share of an encoded vector
template <typename T, int F>
struct PermutoEntry { typedef T type __attribute__((ext_vector_type(F))); };

// One level of encode for one position (:259-317): zeros beyond maxLevel, else the entries of the simplex vertices
// weighted in T, vertex by vertex.  `table` may point to memory or to a copy of the table in LDS; entries are read
// whole, so `table` and every entry offset must be multiples of the entry size.
template <typename T, int D, int F>
__device__ __forceinline__ typename PermutoEntry<T, F>::type permutoEncodeEntry(const float* pos, const CvPermutoLevelInfo& lv, const T* table, float maxLevel)
{
    typedef typename PermutoEntry<T, F>::type Entry;
    Entry acc;
#pragma unroll
    for (int f = 0; f < F; ++f) acc[f] = (T)0.f;
    if (!((float)lv.currentLevelIndex >= maxLevel + 1e-3f)) {   // zero padding beyond maxLevel, :259-262
        float elevated[D + 1], bary[D + 2];
        int rem0[D + 1], rank[D + 1];
        latticeGeometry<D>(pos, lv, elevated, rem0, rank);
        barycentricWeights<D>(elevated, rem0, rank, bary);
        uint32_t idx[D + 1];
        vertexIndices<D>(lv, F, rem0, rank, idx);
        Entry e[D + 1];
#pragma unroll
        for (int k = 0; k <= D; ++k) e[k] = *(const Entry*)(table + idx[k]);
#pragma unroll
        for (int k = 0; k <= D; ++k) {
            const T w = (T)bary[k];
#pragma unroll
            for (int f = 0; f < F; ++f) acc[f] = (T)(acc[f] + (T)(w * e[k][f]));    // in T, vertex by vertex (:312-316)
        }
    }
    return acc;
}

} // namespace cv
