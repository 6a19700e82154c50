// cv_adam.hip -- the example's parameter update on gfx950.
//
// Replaces the adjustParameters dispatch of examples/mlp-training-coopvec
// (kernels.slang:29-45 -> AdamOptimizer::step, adam.slang:20-36; host side
// mlp-training-coopvec.cpp:238-250): one thread per fp16 parameter, every operation evaluated in
// half exactly as the Slang source spells it (each product, sum, quotient, pow and sqrt rounded to
// fp16), NaN gradients cleared and skipped, infinite ones replaced by +-10000, gradient zeroed.
// Pure streaming: 12 bytes read and written per parameter.
#include <hip/hip_runtime.h>

#include "cv_device.h"
#include "cv_error.h"

namespace cv {
namespace {

struct AdamState { half_t mean, variance; int32_t iteration; };   // adam.slang:5-10

__device__ __forceinline__ half_t H(float x) { return (half_t)x; }

__global__ __launch_bounds__(256) void adamKernel(AdamState* states, half_t* params, half_t* grads, uint32_t count,
                                                  float beta1f, float beta2f, float epsf, float lrf)
{
    const uint32_t tid = blockIdx.x * 256u + threadIdx.x;
    if (tid >= count) return;
    float g = (float)grads[tid];
    if (g != g) { grads[tid] = (half_t)0; return; }
    const float beta1 = (float)H(beta1f), beta2 = (float)H(beta2f), eps = (float)H(epsf), lr = (float)H(lrf);
    AdamState st = states[tid];
    st.iteration++;
    if (__builtin_isinf(g)) g = g > 0 ? (float)H(10000.0f) : (float)H(-10000.0f);
    float mean = (float)st.mean, var = (float)st.variance;
    const float omb1 = (float)H(1.0f - beta1), omb2 = (float)H(1.0f - beta2);
    mean = (float)H((float)H(beta1 * mean) + (float)H(omb1 * g));
    var = (float)H((float)H(beta2 * var) + (float)H((float)H(omb2 * g) * g));
    const float it = (float)H((float)st.iteration);
    const float meanHat = (float)H(mean / (float)H(1.0f - (float)H(powf(beta1, it))));
    const float varHat = (float)H(var / (float)H(1.0f - (float)H(powf(beta2, it))));
    const float denom = (float)H(sqrtf((float)H(fmaxf(0.0f, varHat) + eps)));
    params[tid] = H((float)params[tid] - (float)H((float)H(lr * meanHat) / denom));
    st.mean = H(mean);
    st.variance = H(var);
    states[tid] = st;
    grads[tid] = (half_t)0;
}

} // namespace
} // namespace cv

extern "C" CV_API CvResult cvAdamStep(void* stream, void* states, void* params, void* gradients, uint32_t count,
                                      float beta1, float beta2, float epsilon, float learningRate)
{
    if (count == 0) return CV_OK;
    if (!states || !params || !gradients) return cv::failWith(CV_E_INVALID_ARG, "cvAdamStep: null argument");
    if ((uintptr_t)states % 4 || (uintptr_t)params % 2 || (uintptr_t)gradients % 2)
        return cv::failWith(CV_E_INVALID_ARG, "cvAdamStep: misaligned argument");
    cv::noteKernel(false, "adamKernel");
    hipLaunchKernelGGL(cv::adamKernel, dim3((count + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                       (cv::AdamState*)states, (cv::half_t*)params, (cv::half_t*)gradients, count, beta1, beta2,
                       epsilon, learningRate);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return cv::failWith(CV_E_INTERNAL_FAIL, "cvAdamStep launch: %s", hipGetErrorString(e));
    return CV_OK;
}
