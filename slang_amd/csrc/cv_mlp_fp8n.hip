// cv_mlp_fp8n.hip -- e4m3 instantiations of the fused forward MLP on the fp8 matrix pipeline.
#include "cv_mlp_stream.h"

namespace cv {

hipError_t launchMlpFp8Native(hipStream_t stream, const MlpArgs& a, int numCUs)
{
    return dispatchMlp<Fp8NativeMma>(stream, a, numCUs);
}

} // namespace cv
