// cv_matmul_f32.hip -- fp32 instantiations of the batched matMul kernel
// (v_mfma_f32_16x16x4_f32; fp32 vectors, matrix, bias and results).
#include "cv_matmul_impl.h"

namespace cv {

hipError_t launchMatMulF32(hipStream_t stream, const MatMulArgs& a, int numCUs)
{
    return dispatchShape<VecAsMatrix<F32Mma>, float>(stream, a, numCUs);
}

} // namespace cv
