// cv_matmul_fp8b.hip -- further 8-bit float instantiations of the batched matMul kernel: fp16
// vectors interpreted as e4m3 (quantised on load) against an e4m3 matrix, and e5m2 vectors and
// matrix; both run as exactly equal fp16 operands on the fp16 matrix pipeline.
#include "cv_matmul_impl.h"

namespace cv {

hipError_t launchMatMulF16VecAsE4M3(hipStream_t stream, const MatMulArgs& a, int numCUs)
{
    return a.outCt == kF32 ? dispatchShape<F16VecAsE4M3, float>(stream, a, numCUs)
                           : dispatchShape<F16VecAsE4M3, half_t>(stream, a, numCUs);
}

hipError_t launchMatMulBf8AsF16(hipStream_t stream, const MatMulArgs& a, int numCUs)
{
    return a.outCt == kF32 ? dispatchShape<VecAsMatrix<Bf8AsF16Mma>, float>(stream, a, numCUs)
                           : dispatchShape<VecAsMatrix<Bf8AsF16Mma>, half_t>(stream, a, numCUs);
}

} // namespace cv
