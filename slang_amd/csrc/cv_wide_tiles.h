// cv_wide_tiles.h -- geometry shared by the fused forward kernels that work on 32-sample tiles
// (v_mfma_f32_32x32x16_f16): lane l = 32*h + n belongs to sample n of the tile and to half h;
// register r of an accumulator tile T is row 8*(r/4) + 4*h + r%4 of that tile; as B operand of
// k-step s, lane (n,h) supplies k-slots 8*h .. 8*h+7 of that step.
#pragma once
#include "cv_device.h"

namespace cv {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

// hidden unit computed by MFMA row rho of 32-row tile T (H = hidden width / 32)
__host__ __device__ constexpr int wideUnitOfRow(int H, int T, int rho)
{
    return (2 * (rho / 16) + (rho % 8) / 4) * (8 * H) + 8 * T + 4 * ((rho % 16) / 8) + rho % 4;
}
// hidden unit consumed by element e of half h in k-step s
__host__ __device__ constexpr int wideUnitOfSlot(int H, int s, int h, int e)
{
    return (2 * (s % 2) + h) * (8 * H) + 8 * (s / 2) + e;
}

__device__ __forceinline__ floatx16 mfma32(const uint32_t* a, const uint32_t* b, floatx16 c)
{
    const u32x4 av = {a[0], a[1], a[2], a[3]}, bv = {b[0], b[1], b[2], b[3]};
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, av), __builtin_bit_cast(halfx8, bv), c, 0, 0, 0);
}

} // namespace
} // namespace cv
