// cv_mlp_fp8.hip -- e4m3 instantiations of the fused forward MLP on the fp16 matrix pipeline
// (exact decode of weights and of the re-quantised carrier; fp32-grade accumulation).
#include "cv_mlp_stream.h"
#include "cv_mlp_wide.h"

namespace cv {

hipError_t launchMlpFp8AsF16(hipStream_t stream, const MlpArgs& a, int numCUs)
{
    int H, NH, OQ;
    if (mlpWideEligible(a, H, NH, OQ)) {      // 32-sample tiles where the network allows them
        const hipError_t e = launchMlpWide(stream, a, numCUs, H, NH, OQ);
        if (e != hipErrorInvalidValue) return e;
    }
    return dispatchMlp<Fp8AsF16Mma>(stream, a, numCUs);
}

} // namespace cv
