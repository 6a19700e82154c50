// cv_mlp_f16.hip -- fp16 instantiations of the fused forward MLP, and the dispatcher.
#include "cv_mlp_stream.h"

namespace cv {

hipError_t launchMlpFp8AsF16(hipStream_t stream, const MlpArgs& a, int numCUs);
hipError_t launchMlpFp8Native(hipStream_t stream, const MlpArgs& a, int numCUs);

hipError_t launchMlpForward(hipStream_t stream, MmaKind kind, const MlpArgs& a, int numCUs)
{
    if (a.batch == 0) return hipSuccess;
    switch (kind) {
    case MmaKind::F16: return dispatchMlp<F16Mma>(stream, a, numCUs);
    case MmaKind::Fp8AsF16: return launchMlpFp8AsF16(stream, a, numCUs);
    case MmaKind::Fp8Native: return launchMlpFp8Native(stream, a, numCUs);
    default: break;
    }
    return hipErrorInvalidValue;
}

} // namespace cv
