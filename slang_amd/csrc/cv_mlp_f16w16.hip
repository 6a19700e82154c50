// cv_mlp_f16w16.hip -- 32-sample-tile fused forward MLP, fp16 networks with 16 inputs per sample.
#include "cv_mlp_wide16.h"

namespace cv {

hipError_t launchMlpWide16In16(hipStream_t stream, const MlpArgs& a, int numCUs, int H, int NH)
{
    return launchMlpWide16K<16>(stream, a, numCUs, H, NH);
}

} // namespace cv
