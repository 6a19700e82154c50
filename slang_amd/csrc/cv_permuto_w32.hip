// cv_permuto_w32.hip -- permutohedral encoder of 32 features fused in front of the 32-sample-tile forward kernel.
#include "cv_permuto_wide.h"

namespace cv {

hipError_t launchPermutoWide16In32(hipStream_t stream, const CvPermutoDesc& desc, const void* positions, uint64_t positionStride,
                                   const void* featureTable, uint32_t tableElems, const MlpArgs& mlp, int numCUs, int H, int NH)
{
    PermutoWideArgs pa;
    pa.mlp = mlp; pa.desc = desc; pa.pos = (const uint8_t*)positions; pa.posStride = positionStride;
    pa.table = (const uint8_t*)featureTable; pa.tableElems = tableElems;
    return launchPermutoWide16K<32>(stream, pa, numCUs, H, NH);
}

} // namespace cv
