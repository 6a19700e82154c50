// cv_neural.hip -- the neural module's network parameter block on gfx950: whole-network layout
// conversion and the FFLayer chain evaluated from such a block.
//
// Replaces NetworkParameterLayoutConverter (source/standard-modules/neural/
// network-parameter-layout-converter.slang:469-555; per-layer rules :288-440; sizes :96-135) and
// FFLayer.eval / the parameter-offset bookkeeping of FFLayer (source/standard-modules/neural/
// layers.slang:34-110).  Portable layout: per layer row-major weight[Out][In], then bias[Out] only if
// the layer's bit of the bias mask is set.  Optimal layout: per layer the envelope weight
// [align16(Out)][align16(In)] followed by a bias slot of align16(Out) elements, whether or not the layer
// has a bias; padding is zero.  Only the order of the weights inside the envelope is the target's:
// here it is the accumulator-native 16x16 tile of v_mfma_f32_16x16x32_f16 (cv_layout.h,
// TrainingOptimal), which the fused kernels read and the training step writes directly.  The reference's
// own three orders are provided as well, so that a block written by another target can be read.
#include <hip/hip_runtime.h>

#include <cstring>

#include "cv_device.h"
#include "cv_error.h"
#include "cv_kernels.h"

namespace cv {
namespace {

__host__ __device__ inline int align16(int v) { return (v + 15) / 16 * 16; }

// element offset of weight (outputIndex, inputIndex) inside a layer's padded envelope
__host__ __device__ inline int physicalWeightOffset(int order, int inputSize, int outputSize, int o, int i)
{
    const int pin = align16(inputSize), pout = align16(outputSize);
    const int ot = o / 16, it = i / 16, oi = o % 16, ii = i % 16;
    switch (order) {
    case CV_NEURAL_ORDER_NATIVE: {           // tile grid row-major over (outputTile, inputTile); lane 16g+j holds rows 4g..4g+3 of column j
        const int lane = 16 * (oi / 4) + ii;
        return (ot * (pin / 16) + it) * 256 + lane * 4 + (oi & 3); }
    case CV_NEURAL_ORDER_TILED_ROW_MAJOR:    // the reference's SPIR-V rule (:161-166 of the converter)
        return (ot * (pin / 16) + it) * 256 + oi * 16 + ii;
    case CV_NEURAL_ORDER_PADDED_ROW_MAJOR:   // the reference's Metal rule (:167-170)
        return o * pin + i;
    case CV_NEURAL_ORDER_CUDA_MATRIX_B: {    // the reference's CUDA rule (:155-160, rowMajorToCudaNativeLayout :59-72)
        const int row = ii, col = oi;        // (inputInTile, outputInTile)
        const int rowGroup = row < 8 ? 0 : 1, rowInGroup = row - 8 * rowGroup, tidLocal = rowInGroup / 2, pair = rowInGroup % 2;
        const int sub = col < 8 ? 0 : 1, gid = col - 8 * sub;
        return (it * (pout / 16) + ot) * 256 + (gid * 4 + tidLocal) * 8 + sub * 4 + rowGroup * 2 + pair; }
    }
    return 0;
}

struct NeuralArgs {
    CvNeuralNetworkDesc net;
    const uint8_t* src;
    uint8_t* dst;
    uint32_t total;           // elements of the destination
};

// One thread per destination element.  TO_OPTIMAL: destination = optimal block (padding written as 0);
// otherwise destination = portable block.  The search over layers is a short scalar loop.
template <typename T, bool TO_OPTIMAL>
__global__ __launch_bounds__(256) void neuralConvertKernel(const NeuralArgs a)
{
    const uint32_t e = blockIdx.x * 256u + threadIdx.x;
    if (e >= a.total) return;
    const T* src = (const T*)a.src;
    T* dst = (T*)a.dst;
    uint32_t logical = 0, physical = 0;
    for (int l = 0; l < a.net.layerCount; ++l) {
        const int in = a.net.dims[l], out = a.net.dims[l + 1];
        const bool hasBias = (a.net.biasMask >> l) & 1ull;
        const uint32_t wl = (uint32_t)(in * out), wp = (uint32_t)(align16(in) * align16(out));
        const uint32_t nl = wl + (hasBias ? (uint32_t)out : 0u), np = wp + (uint32_t)align16(out);
        if constexpr (TO_OPTIMAL) {
            if (e < physical + np) {
                const uint32_t q = e - physical;
                T v = (T)0.f;
                if (q >= wp) {                                   // bias slot
                    const uint32_t o = q - wp;
                    if (hasBias && o < (uint32_t)out) v = src[logical + wl + o];
                    dst[e] = v;
                    return;
                }
                // invert the order: find (o, i) of physical weight index q
                int o, i;
                const int pin = align16(in), pout = align16(out);
                const int tile = (int)q / 256, r = (int)q % 256;
                switch (a.net.order) {
                case CV_NEURAL_ORDER_NATIVE: {
                    const int lane = r / 4, oi = 4 * (lane / 16) + (r & 3), ii = lane % 16;
                    o = (tile / (pin / 16)) * 16 + oi; i = (tile % (pin / 16)) * 16 + ii; break; }
                case CV_NEURAL_ORDER_TILED_ROW_MAJOR:
                    o = (tile / (pin / 16)) * 16 + r / 16; i = (tile % (pin / 16)) * 16 + r % 16; break;
                case CV_NEURAL_ORDER_PADDED_ROW_MAJOR:
                    o = (int)q / pin; i = (int)q % pin; break;
                default: {                                       // CUDA MatrixB (cudaNativeLayoutToRowMajor, :74-94)
                    const int lane = r / 8, localPos = r % 8, gid = lane / 4, tidLocal = lane % 4;
                    const int sub = localPos / 4, rowGroup = (localPos % 4) / 2, pair = localPos % 2;
                    const int row = rowGroup * 8 + tidLocal * 2 + pair, col = sub * 8 + gid;
                    o = (tile % (pout / 16)) * 16 + col; i = (tile / (pout / 16)) * 16 + row; break; }
                }
                if (o < out && i < in) v = src[logical + (uint32_t)(o * in + i)];
                dst[e] = v;
                return;
            }
        } else {
            if (e < logical + nl) {
                const uint32_t q = e - logical;
                if (q >= wl) { dst[e] = src[physical + wp + (q - wl)]; return; }
                const int o = (int)q / in, i = (int)q % in;
                dst[e] = src[physical + (uint32_t)physicalWeightOffset(a.net.order, in, out, o, i)];
                return;
            }
        }
        logical += nl; physical += np;
    }
}

CvResult checkNet(const char* who, const CvNeuralNetworkDesc* n)
{
    if (!n) return failWith(CV_E_INVALID_ARG, "%s: desc is null", who);
    if (n->layerCount < 1 || n->layerCount > CV_NEURAL_MAX_LAYERS) return failWith(CV_E_INVALID_ARG, "%s: layerCount=%d (1..%d)", who, n->layerCount, CV_NEURAL_MAX_LAYERS);
    for (int l = 0; l <= n->layerCount; ++l)
        if (n->dims[l] < 1) return failWith(CV_E_INVALID_ARG, "%s: dims[%d]=%d", who, l, n->dims[l]);
    if (n->elementType != CV_FLOAT32 && n->elementType != CV_FLOAT16)
        return failWith(CV_E_NOT_AVAILABLE, "%s: elementType %d (supported: FLOAT32, FLOAT16)", who, n->elementType);
    if (n->order < CV_NEURAL_ORDER_NATIVE || n->order > CV_NEURAL_ORDER_CUDA_MATRIX_B) return failWith(CV_E_INVALID_ARG, "%s: unknown order %d", who, n->order);
    // the kernels index a layer's elements with 32-bit integers: a layer of 2^31 padded elements or more is refused
    for (int l = 0; l < n->layerCount; ++l) {
        const uint64_t pin = ((uint64_t)n->dims[l] + 15u) / 16u * 16u, pout = ((uint64_t)n->dims[l + 1] + 15u) / 16u * 16u;
        if (pin * pout + pout >= (1ull << 31))
            return failWith(CV_E_NOT_AVAILABLE, "%s: layer %d (%d -> %d) has 2^31 padded elements or more", who, l, n->dims[l], n->dims[l + 1]);
    }
    return CV_OK;
}

void networkCounts(const CvNeuralNetworkDesc& n, size_t* logical, size_t* physical)
{
    size_t l = 0, p = 0;
    for (int i = 0; i < n.layerCount; ++i) {
        const int in = n.dims[i], out = n.dims[i + 1];
        l += (size_t)in * out + (((n.biasMask >> i) & 1ull) ? (size_t)out : 0);
        p += (size_t)align16(in) * align16(out) + (size_t)align16(out);
    }
    *logical = l; *physical = p;
}

template <bool TO_OPTIMAL>
CvResult convert(const char* who, void* stream, const CvNeuralNetworkDesc* n, const void* src, void* dst)
{
    CvResult rc = checkNet(who, n);
    if (CV_FAILED(rc)) return rc;
    const uint32_t esz = n->elementType == CV_FLOAT32 ? 4u : 2u;
    if (!src || !dst || (uintptr_t)src % esz || (uintptr_t)dst % esz) return failWith(CV_E_INVALID_ARG, "%s: null or misaligned buffer", who);
    size_t logical, physical;
    networkCounts(*n, &logical, &physical);
    const size_t total = TO_OPTIMAL ? physical : logical;
    if (total > 0xffffffffull) return failWith(CV_E_INVALID_ARG, "%s: network too large", who);
    NeuralArgs a;
    memset(&a, 0, sizeof(a));
    a.net = *n; a.src = (const uint8_t*)src; a.dst = (uint8_t*)dst; a.total = (uint32_t)total;
    const dim3 grid((uint32_t)((total + 255) / 256)), block(256);
    noteKernel(false, "neuralConvertKernel<%s,%s>", esz == 4 ? "f32" : "f16", TO_OPTIMAL ? "toOptimal" : "toPortable");
    if (esz == 4) hipLaunchKernelGGL((neuralConvertKernel<float, TO_OPTIMAL>), grid, block, 0, (hipStream_t)stream, a);
    else          hipLaunchKernelGGL((neuralConvertKernel<half_t, TO_OPTIMAL>), grid, block, 0, (hipStream_t)stream, a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return failWith(CV_E_INTERNAL_FAIL, "%s launch: %s", who, hipGetErrorString(e));
    return CV_OK;
}

// Per-layer CvMlpLayer records pointing into a parameter block (and, for training, a gradient block of
// the same layout: the DifferentialPtrPair of layers.slang:21-25).
CvResult layersFromBlock(const char* who, const CvNeuralNetworkDesc* n, int32_t optimal, const void* params, void* grads,
                         const int32_t* activations, const float* leakySlopes, CvMlpLayer* out)
{
    CvResult rc = checkNet(who, n);
    if (CV_FAILED(rc)) return rc;
    const size_t esz = n->elementType == CV_FLOAT32 ? 4u : 2u;
    if (optimal && n->order != CV_NEURAL_ORDER_NATIVE)
        return failWith(CV_E_NOT_AVAILABLE, "%s: an optimal-layout block must be in CV_NEURAL_ORDER_NATIVE order (convert it first)", who);
    if (n->layerCount > kMaxMlpLayers) return failWith(CV_E_NOT_AVAILABLE, "%s: at most %d layers", who, kMaxMlpLayers);
    if (!params) return failWith(CV_E_INVALID_ARG, "%s: params is null", who);
    size_t off = 0;
    for (int l = 0; l < n->layerCount; ++l) {
        const int in = n->dims[l], o = n->dims[l + 1];
        const bool hasBias = (n->biasMask >> l) & 1ull;
        const size_t wElems = optimal ? (size_t)align16(in) * align16(o) : (size_t)in * o;   // FFLayer::WeightStorageSize, layers.slang:63-66
        const size_t bElems = optimal ? (size_t)align16(o) : (hasBias ? (size_t)o : 0);       // FFLayer::BiasStorageSize, :68-71
        CvMlpLayer& L = out[l];
        memset(&L, 0, sizeof(L));
        L.weights = (const uint8_t*)params + off * esz;
        L.biases = hasBias ? (const uint8_t*)params + (off + wElems) * esz : nullptr;
        if (grads) {
            L.weightsGrad = (uint8_t*)grads + off * esz;
            L.biasesGrad = hasBias ? (uint8_t*)grads + (off + wElems) * esz : nullptr;
        }
        L.inputSize = in; L.outputSize = o;
        L.weightLayout = L.gradLayout = optimal ? CV_LAYOUT_TRAINING_OPTIMAL : CV_LAYOUT_ROW_MAJOR;
        L.weightStride = L.gradStride = optimal ? 0u : (uint32_t)(in * esz);
        L.activation = activations ? activations[l] : CV_ACT_NONE;
        L.leakySlope = leakySlopes ? leakySlopes[l] : 0.f;
        off += wElems + bElems;
    }
    return CV_OK;
}

} // namespace
} // namespace cv

extern "C" {

CV_API CvResult cvNeuralNetworkSize(const CvNeuralNetworkDesc* net, size_t* elementCountLogical, size_t* elementCountPhysical)
{
    using namespace cv;
    CvResult rc = checkNet("cvNeuralNetworkSize", net);
    if (CV_FAILED(rc)) return rc;
    size_t l, p;
    networkCounts(*net, &l, &p);
    if (elementCountLogical) *elementCountLogical = l;
    if (elementCountPhysical) *elementCountPhysical = p;
    return CV_OK;
}

CV_API CvResult cvNeuralToOptimalLayout(void* stream, const CvNeuralNetworkDesc* net, const void* portable, void* optimal)
{
    return cv::convert<true>("cvNeuralToOptimalLayout", stream, net, portable, optimal);
}

CV_API CvResult cvNeuralToPortableLayout(void* stream, const CvNeuralNetworkDesc* net, const void* optimal, void* portable)
{
    return cv::convert<false>("cvNeuralToPortableLayout", stream, net, optimal, portable);
}

CV_API CvResult cvNeuralMlpForward(void* stream, const CvNeuralNetworkDesc* net, int32_t optimalLayout, const void* params,
                                   const int32_t* activations, const float* leakySlopes,
                                   const void* input, size_t inputStride, void* output, size_t outputStride, uint32_t batch)
{
    CvMlpLayer layers[cv::kMaxMlpLayers];
    CvResult rc = cv::layersFromBlock("cvNeuralMlpForward", net, optimalLayout, params, nullptr, activations, leakySlopes, layers);
    if (CV_FAILED(rc)) return rc;
    const int32_t T = net->elementType;      // vectors, parameters and results share the network's element type
    CvMlpDesc mlp = {layers, net->layerCount, T, T, T, T, CV_FLOAT16, 0, CV_ENCODE_NONE};
    return cvMlpForward(stream, &mlp, input, inputStride, output, outputStride, batch);
}

CV_API CvResult cvNeuralMlpTrainStep(void* stream, const CvNeuralNetworkDesc* net, int32_t optimalLayout, const void* params,
                                     void* paramGrads, const int32_t* activations, const float* leakySlopes,
                                     const void* input, size_t inputStride, const void* targets, size_t targetStride,
                                     float lossScale, uint32_t batch, float* lossSum, void* workspace, size_t workspaceBytes)
{
    CvMlpLayer layers[cv::kMaxMlpLayers];
    if (!paramGrads) return cv::failWith(CV_E_INVALID_ARG, "cvNeuralMlpTrainStep: paramGrads is null");
    CvResult rc = cv::layersFromBlock("cvNeuralMlpTrainStep", net, optimalLayout, params, paramGrads, activations, leakySlopes, layers);
    if (CV_FAILED(rc)) return rc;
    const int32_t T = net->elementType;      // the gradient block has the parameters' type and layout
    CvMlpDesc mlp = {layers, net->layerCount, T, T, T, T, T, 0, CV_ENCODE_NONE};
    if (!workspace) {       // size query
        size_t need = 0;
        rc = cvMlpTrainStepWorkspaceSize(&mlp, batch, &need);
        if (CV_FAILED(rc)) return rc;
        return cv::failWith(CV_E_BUFFER_TOO_SMALL, "cvNeuralMlpTrainStep: workspace of %zu bytes needed", need);
    }
    return cvMlpTrainStep(stream, &mlp, input, inputStride, targets, targetStride, lossScale, batch, lossSum, workspace, workspaceBytes);
}

CV_API CvResult cvNeuralMlpTrainStepWorkspaceSize(const CvNeuralNetworkDesc* net, uint32_t batch, size_t* outBytes)
{
    CvMlpLayer layers[cv::kMaxMlpLayers];
    alignas(16) static const uint8_t dummy[16] = {};      // stands for a parameter block: only its alignment is looked at
    CvResult rc = cv::layersFromBlock("cvNeuralMlpTrainStepWorkspaceSize", net, 0, dummy, nullptr, nullptr, nullptr, layers);
    if (CV_FAILED(rc)) return rc;
    const int32_t T = net->elementType;
    CvMlpDesc mlp = {layers, net->layerCount, T, T, T, T, T, 0, CV_ENCODE_NONE};
    return cvMlpTrainStepWorkspaceSize(&mlp, batch, outBytes);
}

} // extern "C"
