// cv_matmul_bf16.hip -- bfloat16 instantiations of the batched matMul kernel
// (v_mfma_f32_16x16x32_bf16; results as bfloat16 or fp32).
#include "cv_matmul_impl.h"

namespace cv {

hipError_t launchMatMulBf16(hipStream_t stream, const MatMulArgs& a, int numCUs)
{
    return a.outCt == kF32 ? dispatchShape<VecAsMatrix<Bf16Mma>, float>(stream, a, numCUs)
                           : dispatchShape<VecAsMatrix<Bf16Mma>, bf16_t>(stream, a, numCUs);
}

} // namespace cv
