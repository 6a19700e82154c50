// cv_mlp_f16w32.hip -- 32-sample-tile fused forward MLP, fp16 networks with 32 inputs per sample.
#include "cv_mlp_wide16.h"

namespace cv {

hipError_t launchMlpWide16In32(hipStream_t stream, const MlpArgs& a, int numCUs, int H, int NH)
{
    return launchMlpWide16K<32>(stream, a, numCUs, H, NH);
}

} // namespace cv
