// cv_mlp_fp8.hip -- e4m3 instantiations of the fused forward MLP on the fp16 matrix pipeline
// (exact decode of weights and of the re-quantised carrier; fp32-grade accumulation).
#include "cv_mlp_stream.h"

namespace cv {

hipError_t launchMlpFp8AsF16(hipStream_t stream, const MlpArgs& a, int numCUs)
{
    return dispatchMlp<Fp8AsF16Mma>(stream, a, numCUs);
}

} // namespace cv
