// cv_matmul_fp8.hip -- e4m3 instantiations of the batched matMul kernel: decoded to fp16
// operands on the fp16 matrix pipeline (default), or native on the fp8 matrix pipeline.
#include "cv_matmul_impl.h"

namespace cv {

hipError_t launchMatMulFp8AsF16(hipStream_t stream, const MatMulArgs& a, int numCUs)
{
    return a.outCt == kF32 ? dispatchShape<VecAsMatrix<Fp8AsF16Mma>, float>(stream, a, numCUs)
                           : dispatchShape<VecAsMatrix<Fp8AsF16Mma>, half_t>(stream, a, numCUs);
}

hipError_t launchMatMulFp8Native(hipStream_t stream, const MatMulArgs& a, int numCUs)
{
    return a.outCt == kF32 ? dispatchShape<VecAsMatrix<Fp8NativeMma>, float>(stream, a, numCUs)
                           : dispatchShape<VecAsMatrix<Fp8NativeMma>, half_t>(stream, a, numCUs);
}

} // namespace cv
