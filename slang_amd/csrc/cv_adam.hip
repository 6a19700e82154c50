// cv_adam.hip -- the example's parameter update on gfx950.
//
// Replaces the adjustParameters dispatch of examples/mlp-training-coopvec
// (kernels.slang:29-45 -> AdamOptimizer::step, adam.slang:20-36; host side
// mlp-training-coopvec.cpp:238-250): one thread per fp16 parameter, every operation evaluated in
// half exactly as the Slang source spells it (each product, sum, quotient, pow and sqrt rounded to
// fp16), NaN gradients cleared and skipped, infinite ones replaced by +-10000, gradient zeroed.
// Pure streaming: 12 bytes read and written per parameter.
#include <hip/hip_runtime.h>

#include <string.h>

#include "coopvec.h"
#include "cv_device.h"
#include "cv_error.h"

namespace cv {
namespace {

struct AdamState { half_t mean, variance; int32_t iteration; };   // adam.slang:5-10

__device__ __forceinline__ half_t H(float x) { return (half_t)x; }

struct AdamConstants { float beta1, beta2, eps, lr; };

// AdamOptimizer::step (adam.slang:20-36) behind the guards of adjustParameters (kernels.slang:39-43) for one
// parameter; returns false when the gradient is NaN (the update is skipped; the caller clears the gradient either way)
// pow(beta1, t) and pow(beta2, t) as half, for the half-rounded step count t (adam.slang:30-31).  The two powf are
// two thirds of the update's instructions, and all parameters of a network normally share one step count, so a
// workgroup evaluates them once for the count `shared` (its first state's) and a lane whose own count differs
// evaluates them itself: same function, same arguments, same bits.
struct AdamPowers { float it, p1, p2; };

__device__ __forceinline__ AdamPowers adamPowers(float it, const AdamConstants& k)
{
    return AdamPowers{it, (float)H(powf((float)H(k.beta1), it)), (float)H(powf((float)H(k.beta2), it))};
}

__device__ __forceinline__ bool adamUpdate(AdamState& st, half_t& param, float g, const AdamConstants& k, const AdamPowers& shared)
{
    if (g != g) return false;
    const float beta1 = (float)H(k.beta1), beta2 = (float)H(k.beta2), eps = (float)H(k.eps), lr = (float)H(k.lr);
    st.iteration++;
    if (__builtin_isinf(g)) g = g > 0 ? (float)H(10000.0f) : (float)H(-10000.0f);
    float mean = (float)st.mean, var = (float)st.variance;
    const float omb1 = (float)H(1.0f - beta1), omb2 = (float)H(1.0f - beta2);
    mean = (float)H((float)H(beta1 * mean) + (float)H(omb1 * g));
    var = (float)H((float)H(beta2 * var) + (float)H((float)H(omb2 * g) * g));
    const float it = (float)H((float)st.iteration);
    AdamPowers pw = shared;
    if (it != shared.it) pw = adamPowers(it, k);
    const float meanHat = (float)H(mean / (float)H(1.0f - pw.p1));
    const float varHat = (float)H(var / (float)H(1.0f - pw.p2));
    const float denom = (float)H(sqrtf((float)H(fmaxf(0.0f, varHat) + eps)));
    param = H((float)param - (float)H((float)H(lr * meanHat) / denom));
    st.mean = H(mean);
    st.variance = H(var);
    return true;
}

// the powers for the step count that follows the one stored in `first`, evaluated by the first wave of the workgroup
__device__ __forceinline__ AdamPowers sharedAdamPowers(const AdamState* first, const AdamConstants& k, float* lds /* 3 floats */)
{
    if (threadIdx.x < 64u) {
        const AdamPowers pw = adamPowers((float)H((float)(first->iteration + 1)), k);
        if (threadIdx.x == 0) { lds[0] = pw.it; lds[1] = pw.p1; lds[2] = pw.p2; }
    }
    __syncthreads();
    return AdamPowers{lds[0], lds[1], lds[2]};
}

__global__ __launch_bounds__(1024) void adamKernel(AdamState* states, half_t* params, half_t* grads, uint32_t count,
                                                   AdamConstants k)
{
    __shared__ float ldsPowers[3];
    const uint32_t tid = blockIdx.x * 1024u + threadIdx.x;
    const bool on = tid < count;
    const uint32_t i = on ? tid : count - 1u;
    AdamState st = states[i];                 // requested before the powers are worked out
    half_t p = params[i];
    const float g = (float)grads[i];
    const AdamPowers shared = sharedAdamPowers(states + blockIdx.x * 1024u, k, ldsPowers);
    if (!on) return;
    if (adamUpdate(st, p, g, k, shared)) {
        params[tid] = p;
        states[tid] = st;
    }
    grads[tid] = (half_t)0;
}

// The same with four consecutive parameters per thread: 8-byte accesses to the parameters and gradients, two of 16 bytes to
// the states, all of them streaming (every byte is touched once); for counts that are a multiple of four at addresses
// aligned to those accesses.
__global__ __launch_bounds__(256) void adamKernel4(AdamState* states, half_t* params, half_t* grads, uint32_t quads, AdamConstants k)
{
    __shared__ float ldsPowers[3];
    const uint32_t tid = blockIdx.x * 256u + threadIdx.x;
    const bool on = tid < quads;
    const uint32_t q = on ? tid : quads - 1u;
    const u32x4 s01 = __builtin_nontemporal_load((const u32x4*)(states + 4u * q));
    const u32x4 s23 = __builtin_nontemporal_load((const u32x4*)(states + 4u * q) + 1);
    const u32x2 pw = __builtin_nontemporal_load((const u32x2*)(params + 4u * q));
    const u32x2 gw = __builtin_nontemporal_load((const u32x2*)(grads + 4u * q));
    const AdamPowers shared = sharedAdamPowers(states + blockIdx.x * 1024u, k, ldsPowers);
    if (!on) return;
    const uint32_t sIn[8] = {s01.x, s01.y, s01.z, s01.w, s23.x, s23.y, s23.z, s23.w};
    uint32_t sOut[8];
    half_t p[4], g[4];
    *(u32x2*)p = pw;
    *(u32x2*)g = gw;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        AdamState st;
        const halfx2 mv = __builtin_bit_cast(halfx2, sIn[2 * i]);
        st.mean = mv.x; st.variance = mv.y; st.iteration = (int32_t)sIn[2 * i + 1];
        half_t pi = p[i];
        if (adamUpdate(st, pi, (float)g[i], k, shared)) {
            p[i] = pi;
            sOut[2 * i] = __builtin_bit_cast(uint32_t, halfx2{st.mean, st.variance});
            sOut[2 * i + 1] = (uint32_t)st.iteration;
        } else {
            sOut[2 * i] = sIn[2 * i]; sOut[2 * i + 1] = sIn[2 * i + 1];
        }
    }
    __builtin_nontemporal_store(*(const u32x2*)p, (u32x2*)(params + 4u * tid));
    __builtin_nontemporal_store(u32x4{sOut[0], sOut[1], sOut[2], sOut[3]}, (u32x4*)(states + 4u * tid));
    __builtin_nontemporal_store(u32x4{sOut[4], sOut[5], sOut[6], sOut[7]}, (u32x4*)(states + 4u * tid) + 1);
    __builtin_nontemporal_store(u32x2{0u, 0u}, (u32x2*)(grads + 4u * tid));
}

// The same update for a whole network, read straight from the gradient buffers the training step fills: the example
// first copies every weight gradient from its TrainingOptimal buffer to a row-major one
// (mlp-training-coopvec.cpp:203-236) and clears the TrainingOptimal segment at the top of the next iteration
// (:183-188); here a thread finds its gradient element through the layout's index map and leaves a zero behind.
struct AdamLayer {
    uint8_t* weights; uint8_t* wGrad; AdamState* wStates;
    half_t* biases; uint8_t* bGrad; AdamState* bStates;
    MatrixShape wShape, gShape;
    uint32_t first;          // index of the layer's first element among all threads' elements
    uint32_t weightCount, biasCount;
};
constexpr int kMaxAdamLayers = 8;
struct AdamLayersArgs {
    AdamLayer layers[kMaxAdamLayers];
    int32_t numLayers;
    int32_t gradCt;          // kF16 or kF32
    uint32_t total;
    AdamConstants k;
};

__global__ __launch_bounds__(256) void adamLayersKernel(const AdamLayersArgs a)
{
    __shared__ float ldsPowers[3];
    // (a thread past the last element works on the last one and leaves before it stores: no branch around the requests)
    const uint32_t own = blockIdx.x * 256u + threadIdx.x;
    const bool on = own < a.total;
    const uint32_t tid = on ? own : a.total - 1u;
    int l = 0;
#pragma unroll
    for (int i = 1; i < kMaxAdamLayers; ++i)
        if (i < a.numLayers && tid >= a.layers[i].first) l = i;
    const AdamLayer& ly = a.layers[l];
    const uint32_t e = tid - ly.first;
    half_t* param; uint8_t* grad; AdamState* state;
    if (e < ly.weightCount) {
        const uint32_t o = e / ly.wShape.cols, i = e - o * ly.wShape.cols;
        param = (half_t*)(ly.weights + elemOffset(ly.wShape, o, i));
        grad = ly.wGrad + elemOffset(ly.gShape, o, i);
        state = ly.wStates + e;
    } else {
        const uint32_t o = e - ly.weightCount;
        param = ly.biases + o;
        grad = ly.bGrad + (size_t)o * (a.gradCt == kF32 ? 4u : 2u);
        state = ly.bStates + o;
    }
    // Requested before the powers are worked out, and nothing is done with them until then: one trip to memory for the
    // step count, the state, the parameter and the gradient together.  (A half gradient is read as the two bytes it is;
    // an fp32 one as four, from an address that holds four either way.)
    AdamState st = *state;
    half_t p = *param;
    const bool wide = a.gradCt == kF32;
    const uint32_t gbits = wide ? *(const uint32_t*)grad : (uint32_t)*(const uint16_t*)grad;
    const AdamPowers shared = sharedAdamPowers(a.layers[0].wStates, a.k, ldsPowers);
    if (!on) return;
    // an fp32 gradient buffer holds the sum the half buffer of the example would have held unrounded: rounded here
    const float g = wide ? (float)H(__builtin_bit_cast(float, gbits)) : (float)__builtin_bit_cast(half_t, (uint16_t)gbits);
    if (adamUpdate(st, p, g, a.k, shared)) {
        *param = p;
        *state = st;
    }
    if (wide) *(float*)grad = 0.f; else *(half_t*)grad = (half_t)0;
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
    if (count % 4u == 0 && (uintptr_t)states % 16 == 0 && (uintptr_t)params % 8 == 0 && (uintptr_t)gradients % 8 == 0) {
        cv::noteKernel(false, "adamKernel4");
        hipLaunchKernelGGL(cv::adamKernel4, dim3((count / 4u + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                           (cv::AdamState*)states, (cv::half_t*)params, (cv::half_t*)gradients, count / 4u,
                           cv::AdamConstants{beta1, beta2, epsilon, learningRate});
    } else {
        cv::noteKernel(false, "adamKernel");
        hipLaunchKernelGGL(cv::adamKernel, dim3((count + 1023) / 1024), dim3(1024), 0, (hipStream_t)stream,
                           (cv::AdamState*)states, (cv::half_t*)params, (cv::half_t*)gradients, count,
                           cv::AdamConstants{beta1, beta2, epsilon, learningRate});
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return cv::failWith(CV_E_INTERNAL_FAIL, "cvAdamStep launch: %s", hipGetErrorString(e));
    return CV_OK;
}

extern "C" CV_API CvResult cvMlpAdamStep(void* stream, const CvMlpDesc* mlp, void* const* weightStates, void* const* biasStates,
                                         float beta1, float beta2, float epsilon, float learningRate)
{
    using namespace cv;
    const char* who = "cvMlpAdamStep";
    if (!mlp || !mlp->layers || !weightStates) return failWith(CV_E_INVALID_ARG, "%s: null argument", who);
    if (mlp->numLayers < 1 || mlp->numLayers > kMaxAdamLayers)
        return failWith(CV_E_INVALID_ARG, "%s: numLayers=%d (1..%d)", who, mlp->numLayers, kMaxAdamLayers);
    if (mlp->weightType != CV_FLOAT16 || mlp->biasType != CV_FLOAT16)
        return failWith(CV_E_NOT_AVAILABLE, "%s: the optimizer's arithmetic is half (adam.slang:3): FLOAT16 parameters only", who);
    if (mlp->gradType != CV_FLOAT16 && mlp->gradType != CV_FLOAT32)
        return failWith(CV_E_NOT_AVAILABLE, "%s: gradType %d (FLOAT16 or FLOAT32)", who, mlp->gradType);
    AdamLayersArgs a;
    memset(&a, 0, sizeof(a));
    a.numLayers = mlp->numLayers; a.gradCt = mlp->gradType;
    a.k = AdamConstants{beta1, beta2, epsilon, learningRate};
    const uint32_t gEsz = elemSize(mlp->gradType);
    uint64_t total = 0;
    for (int l = 0; l < mlp->numLayers; ++l) {
        const CvMlpLayer& L = mlp->layers[l];
        if (L.inputSize <= 0 || L.outputSize <= 0) return failWith(CV_E_INVALID_ARG, "%s: layer %d is %dx%d", who, l, L.outputSize, L.inputSize);
        if (!L.weights || !L.weightsGrad || !weightStates[l])
            return failWith(CV_E_INVALID_ARG, "%s: layer %d: weights, weightsGrad and weightStates are needed", who, l);
        if ((L.biases != nullptr) != (L.biasesGrad != nullptr) || (L.biases && (!biasStates || !biasStates[l])))
            return failWith(CV_E_INVALID_ARG, "%s: layer %d: biases, biasesGrad and biasStates go together", who, l);
        AdamLayer& o = a.layers[l];
        const bool wOpt = L.weightLayout == CV_LAYOUT_INFERENCING_OPTIMAL || L.weightLayout == CV_LAYOUT_TRAINING_OPTIMAL;
        const bool gOpt = L.gradLayout == CV_LAYOUT_INFERENCING_OPTIMAL || L.gradLayout == CV_LAYOUT_TRAINING_OPTIMAL;
        o.wShape = MatrixShape{(uint32_t)L.outputSize, (uint32_t)L.inputSize, CV_FLOAT16, L.weightLayout, wOpt ? 0 : (size_t)L.weightStride};
        o.gShape = MatrixShape{(uint32_t)L.outputSize, (uint32_t)L.inputSize, mlp->gradType, L.gradLayout, gOpt ? 0 : (size_t)L.gradStride};
        if (L.weightLayout < 0 || L.weightLayout > 3 || L.gradLayout < 0 || L.gradLayout > 3 || matrixSize(o.wShape) == 0 || matrixSize(o.gShape) == 0)
            return failWith(CV_E_INVALID_ARG, "%s: layer %d: layout/stride of the weights or of their gradient", who, l);
        if ((uintptr_t)L.weights % 2 || (uintptr_t)L.weightsGrad % gEsz || (uintptr_t)weightStates[l] % 4 ||
            (!wOpt && L.weightStride % 2) || (!gOpt && L.gradStride % gEsz) || (uintptr_t)L.biases % 2 || (uintptr_t)L.biasesGrad % gEsz ||
            (L.biases && (uintptr_t)biasStates[l] % 4))
            return failWith(CV_E_INVALID_ARG, "%s: layer %d: misaligned argument", who, l);
        o.weights = (uint8_t*)const_cast<void*>(L.weights); o.wGrad = (uint8_t*)L.weightsGrad; o.wStates = (AdamState*)weightStates[l];
        o.biases = (half_t*)const_cast<void*>(L.biases); o.bGrad = (uint8_t*)L.biasesGrad;
        o.bStates = L.biases ? (AdamState*)biasStates[l] : nullptr;
        o.first = (uint32_t)total;
        o.weightCount = (uint32_t)L.outputSize * (uint32_t)L.inputSize;
        o.biasCount = L.biases ? (uint32_t)L.outputSize : 0u;
        total += (uint64_t)o.weightCount + o.biasCount;
        if (total > 0xffffffffull) return failWith(CV_E_NOT_AVAILABLE, "%s: more than 2^32 parameters", who);
    }
    a.total = (uint32_t)total;
    noteKernel(false, "adamLayersKernel<%d layers>", mlp->numLayers);
    hipLaunchKernelGGL(adamLayersKernel, dim3((a.total + 255) / 256), dim3(256), 0, (hipStream_t)stream, a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return failWith(CV_E_INTERNAL_FAIL, "%s launch: %s", who, hipGetErrorString(e));
    return CV_OK;
}
