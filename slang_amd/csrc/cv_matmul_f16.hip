// cv_matmul_f16.hip -- fp16 instantiations of the batched matMul kernel, and the dispatcher.
#include "cv_matmul_impl.h"

namespace cv {

hipError_t launchMatMulFp8AsF16(hipStream_t stream, const MatMulArgs& a, int numCUs);
hipError_t launchMatMulFp8Native(hipStream_t stream, const MatMulArgs& a, int numCUs);
hipError_t launchMatMulF16VecAsE4M3(hipStream_t stream, const MatMulArgs& a, int numCUs);
hipError_t launchMatMulBf8AsF16(hipStream_t stream, const MatMulArgs& a, int numCUs);
hipError_t launchMatMulBf16(hipStream_t stream, const MatMulArgs& a, int numCUs);
hipError_t launchMatMulI8(hipStream_t stream, const MatMulArgs& a, int numCUs);
hipError_t launchMatMulI8AnySign(hipStream_t stream, const MatMulArgs& a, int numCUs);
hipError_t launchMatMulF32(hipStream_t stream, const MatMulArgs& a, int numCUs);

hipError_t launchMatMul(hipStream_t stream, MmaKind kind, const MatMulArgs& a, int numCUs)
{
    if (a.batch == 0) return hipSuccess;
    switch (kind) {
    case MmaKind::F16:
        return a.outCt == kF32 ? dispatchShape<VecAsMatrix<F16Mma>, float>(stream, a, numCUs)
                               : dispatchShape<VecAsMatrix<F16Mma>, half_t>(stream, a, numCUs);
    case MmaKind::Fp8AsF16: return launchMatMulFp8AsF16(stream, a, numCUs);
    case MmaKind::Fp8Native: return launchMatMulFp8Native(stream, a, numCUs);
    case MmaKind::F16VecAsE4M3: return launchMatMulF16VecAsE4M3(stream, a, numCUs);
    case MmaKind::Bf8AsF16: return launchMatMulBf8AsF16(stream, a, numCUs);
    case MmaKind::Bf16: return launchMatMulBf16(stream, a, numCUs);
    case MmaKind::I8: return launchMatMulI8(stream, a, numCUs);
    case MmaKind::I8AnySign: return launchMatMulI8AnySign(stream, a, numCUs);
    case MmaKind::F32: return launchMatMulF32(stream, a, numCUs);
    case MmaKind::Scalar: return launchMatMulScalar(stream, a, numCUs);
    }
    return hipErrorInvalidValue;
}

} // namespace cv
