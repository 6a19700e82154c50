// cv_matmul_i8.hip -- int8 -> int32 instantiations of the batched matMul kernel (bit-exact):
// signed bytes on both sides, and the flavour that takes unsigned bytes on either side.
#include "cv_matmul_impl.h"

namespace cv {

hipError_t launchMatMulI8(hipStream_t stream, const MatMulArgs& a, int numCUs)
{
    return dispatchShape<VecAsMatrix<I8Mma>, int32_t>(stream, a, numCUs);
}

hipError_t launchMatMulI8AnySign(hipStream_t stream, const MatMulArgs& a, int numCUs)
{
    return dispatchShape<I8AnySign, int32_t>(stream, a, numCUs);
}

} // namespace cv
