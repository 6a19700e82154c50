// cv_convert.hip -- matrix layout conversion for gfx950.
//
// Replaces rhi::ICommandEncoder::convertCooperativeVectorMatrix (call site
// examples/mlp-training-coopvec/mlp-training-coopvec.cpp:203-236): copies a list of matrices
// between (component type, layout, stride) descriptions.  Destination-driven: one thread per
// destination element slot, so padding of the Optimal layouts is written (as zero) by the same
// pass and no two threads touch the same byte.  For Row/ColumnMajor destinations only logical
// elements are written; bytes between rows (stride padding) are left alone.
#include "cv_device.h"
#include "cv_kernels.h"
#include "cv_error.h"

namespace cv {

namespace {

// Inverse of cv::elemOffset for destination slot `e` (in elements).  Returns false for padding.
__device__ __forceinline__ bool slotToCoord(const MatrixShape& s, uint32_t e, uint32_t& r, uint32_t& c)
{
    switch (s.layout) {
    case kRowMajor: r = e / s.cols; c = e % s.cols; return true;
    case kColumnMajor: c = e / s.rows; r = e % s.rows; return true;
    case kInferencingOptimal: {
        const uint32_t epl = fragElemsPerLane(s.ct);
        const uint32_t mt4 = 4u * optMT(s.rows), gs = optGS(s.cols), kt = optKT(s.cols, epl);
        const uint32_t el = e % epl, lane = (e / epl) & 63u, f = e / (epl * 64u);
        const uint32_t k = f % kt, t = f / kt, g = lane >> 4, i = lane & 15u;
        const uint32_t q = k * epl + el;
        r = (i >> 2) * mt4 + 4u * t + (i & 3u);
        c = g * gs + q;
        return q < gs && r < s.rows && c < s.cols; }
    case kTrainingOptimal: {
        const uint32_t tc = optMT(s.cols);
        const uint32_t rr = e & 3u, lane = (e >> 2) & 63u, tile = e >> 8;
        r = (tile / tc) * 16u + (lane >> 4) * 4u + rr;
        c = (tile % tc) * 16u + (lane & 15u);
        return r < s.rows && c < s.cols; }
    }
    return false;
}

__global__ __launch_bounds__(256) void convertKernel(const ConvertArgs args)
{
    const ConvertItem& it = args.items[blockIdx.y];
    const MatrixShape src = it.srcShape, dst = it.dstShape;
    const uint32_t dEsz = elemSize(dst.ct), sEsz = elemSize(src.ct);
    const bool dstOptimal = dst.layout == kInferencingOptimal || dst.layout == kTrainingOptimal;
    const uint32_t slots = dstOptimal ? it.dstBytes / dEsz : dst.rows * dst.cols;
    for (uint32_t e = blockIdx.x * 256u + threadIdx.x; e < slots; e += gridDim.x * 256u) {
        uint32_t r, c;
        const bool valid = slotToCoord(dst, e, r, c);
        uint8_t* d = it.dst + (dstOptimal ? (size_t)e * dEsz : elemOffset(dst, r, c));
        const uint8_t* s = valid ? it.src + elemOffset(src, r, c) : nullptr;
        if (src.ct == dst.ct) {
            switch (dEsz) {
            case 1: *d = valid ? *s : (uint8_t)0; break;
            case 2: *(uint16_t*)d = valid ? *(const uint16_t*)s : (uint16_t)0; break;
            case 4: *(uint32_t*)d = valid ? *(const uint32_t*)s : 0u; break;
            case 8: *(uint64_t*)d = valid ? *(const uint64_t*)s : 0ull; break;
            }
        } else if (dst.ct == kF16) {   // FLOAT32 -> FLOAT16, round to nearest even
            *(half_t*)d = valid ? (half_t)*(const float*)s : (half_t)0;
        } else {                       // FLOAT16 -> FLOAT32
            *(float*)d = valid ? (float)*(const half_t*)s : 0.f;
        }
        (void)sEsz;
    }
}

} // namespace

hipError_t launchConvert(hipStream_t stream, const ConvertArgs& args)
{
    if (args.count == 0) return hipSuccess;
    uint32_t maxSlots = 1;
    for (uint32_t i = 0; i < args.count; ++i) {
        const ConvertItem& it = args.items[i];
        const bool opt = it.dstShape.layout == kInferencingOptimal || it.dstShape.layout == kTrainingOptimal;
        const uint32_t slots = opt ? it.dstBytes / elemSize(it.dstShape.ct) : it.dstShape.rows * it.dstShape.cols;
        if (slots > maxSlots) maxSlots = slots;
    }
    uint32_t bx = (maxSlots + 255u) / 256u;
    if (bx > 1024u) bx = 1024u;
    noteKernel(false, "convertKernel");
    hipLaunchKernelGGL(convertKernel, dim3(bx, args.count), dim3(256), 0, stream, args);
    return hipGetLastError();
}

} // namespace cv
