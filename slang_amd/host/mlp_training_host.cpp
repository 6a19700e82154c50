// mlp_training_host.cpp -- host program that trains the example's 4 -> 16 -> 4 network on MI355X
// through the C-ABI of include/coopvec.h.
//
// Counterpart of examples/mlp-training-coopvec/mlp-training-coopvec.cpp (execute(), :76-262): the
// same three-segment parameter buffer with 64-byte sub-allocations (:92-126, :265-315), the same
// seeded initialisation (srand(1072), rand(), the reference's float->half rule, :128-137,
// :400-425), the same 16 samples (:163-170) and the same per-iteration order (:178-260):
//   clear the training-optimal gradient segment -> learnGradient -> convert TrainingOptimal to
//   RowMajor -> adjustParameters (Adam) -> every 10 iterations read back the loss.
// What the Slang kernels do per thread is done here by cvMlpTrainStep / cvConvertMatrices /
// cvAdamStep.  The input encoding (x, y, x^2, y^2) (network.slang:35-38) and the ground truth
// (network.slang:67-75) are evaluated by the training kernel in half, as the shader would.
//
// Two forms of the iteration, same parameters bit for bit:
//   --unfused : the example's five steps as listed above (memset, 2 kernels, convert, Adam);
//   default   : cvMlpTrainStep + cvMlpAdamStep, which reads the TrainingOptimal gradients where they lie and leaves
//               them at zero, so the convert and the clear go away; ten iterations (the interval at which the loss is
//               read back) are recorded once into a HIP graph of thirty kernels, and one graph launch runs them.
// The loss printed is the one the example prints: the largest per-sample loss of the iteration (learnGradient's
// WaveActiveMax + atomic max, kernels.slang:21-26), followed by the mean.
//
//   mlp_training_host [iterations=1000] [--unfused] [--time]
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "coopvec.h"

typedef _Float16 NFloat;

static const int kLayerSizes[] = {4, 16, 4};
static const int kLayerCount = sizeof(kLayerSizes) / sizeof(int) - 1;

#define HIP_OK(x)                                                                      \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            fprintf(stderr, "%s failed: %s\n", #x, hipGetErrorString(e_));             \
            return 1;                                                                  \
        }                                                                              \
    } while (0)
#define CV_OK_OR_FAIL(x)                                                               \
    do {                                                                               \
        CvResult r_ = (x);                                                             \
        if (CV_FAILED(r_)) {                                                           \
            fprintf(stderr, "%s failed: %s\n", #x, cvGetLastErrorMessage());           \
            return 1;                                                                  \
        }                                                                              \
    } while (0)

struct LayerAllocation {
    size_t weightsOffset, weightsSize, biasOffset, biasSize;
    size_t weightsGradOffset, biasGradOffset, weightsGradTrainingOffset, weightsGradTrainingSize;
};

// The reference initialises its parameters with this float -> half rule (guard bit added back:
// ties away from zero, everything below 2^-24 flushed), not with IEEE nearest-even.
static uint16_t referenceFloatToHalf(float value)
{
    uint32_t in;
    memcpy(&in, &value, 4);
    uint32_t out = (in >> 16) & 0x8000u;
    uint32_t mant = (in >> 12) & 0x07ffu;
    const uint32_t expo = (in >> 23) & 0xffu;
    if (expo < 103u) return (uint16_t)out;
    if (expo > 142u) return (uint16_t)(out | 0x7c00u | (uint32_t)(expo == 255u && (in & 0x007fffffu)));
    if (expo < 113u) {
        mant |= 0x0800u;
        return (uint16_t)(out | ((mant >> (114u - expo)) + ((mant >> (113u - expo)) & 1u)));
    }
    out |= ((expo - 112u) << 10) | (mant >> 1);
    return (uint16_t)(out + (mant & 1u));
}

int main(int argc, char** argv)
{
    int iterations = 1000;
    bool unfused = false, timeIt = false;
    for (int i = 1; i < argc; i++) {
        if (!strcmp(argv[i], "--unfused")) unfused = true;
        else if (!strcmp(argv[i], "--time")) timeIt = true;
        else iterations = atoi(argv[i]);
    }

    // ---- buffer plan: | weights_i bias_i ... | row-major grads ... | training-optimal weight grads |
    std::vector<LayerAllocation> layers(kLayerCount);
    size_t bufferSize = 0;
    auto alloc64 = [&](size_t size) {
        const size_t offset = bufferSize;
        bufferSize += (size + 63) / 64 * 64;
        return offset;
    };
    for (int i = 0; i < kLayerCount; i++) {
        layers[i].weightsSize = (size_t)kLayerSizes[i] * kLayerSizes[i + 1] * sizeof(NFloat);
        layers[i].weightsOffset = alloc64(layers[i].weightsSize);
        layers[i].biasSize = (size_t)kLayerSizes[i + 1] * sizeof(NFloat);
        layers[i].biasOffset = alloc64(layers[i].biasSize);
    }
    const size_t gradientOffset = bufferSize;
    for (int i = 0; i < kLayerCount; i++) {
        layers[i].weightsGradOffset = alloc64(layers[i].weightsSize);
        layers[i].biasGradOffset = alloc64(layers[i].biasSize);
    }
    const size_t gradientTrainingOffset = bufferSize;
    for (int i = 0; i < kLayerCount; i++) {
        CV_OK_OR_FAIL(cvGetMatrixSize(kLayerSizes[i + 1], kLayerSizes[i], CV_FLOAT16, CV_LAYOUT_TRAINING_OPTIMAL, 0,
                                      &layers[i].weightsGradTrainingSize));
        layers[i].weightsGradTrainingOffset = alloc64(layers[i].weightsGradTrainingSize);
    }

    // ---- seeded initial contents, in the reference's order: parameters first, then the inputs
    std::vector<uint16_t> initParams;
    srand(1072);
    for (size_t i = 0; i < bufferSize / sizeof(NFloat); i++)
        initParams.push_back(referenceFloatToHalf(rand() / (float)RAND_MAX * 2.0f - 1.0f));
    const int inputCount = 32, sampleCount = inputCount / 2;
    std::vector<float> inputData;
    for (int i = 0; i < inputCount; i++) inputData.push_back(rand() / (float)RAND_MAX);

    // the float2 samples go to the device as they are (`uniform float2* inputs`, kernels.slang:12): the
    // training step converts them to half2, encodes (x, y, x*x, y*y) and evaluates groundtruth(x, y) itself
    uint8_t* params = nullptr;
    void *adamStates = nullptr, *dInputs = nullptr, *workspace = nullptr;
    float* dLoss = nullptr;      // [0] sum, [1] max of the per-sample losses
    const size_t paramCount = bufferSize / sizeof(NFloat);
    HIP_OK(hipMalloc((void**)&params, bufferSize));
    HIP_OK(hipMemcpy(params, initParams.data(), bufferSize, hipMemcpyHostToDevice));
    HIP_OK(hipMalloc(&adamStates, paramCount * 8));
    HIP_OK(hipMemset(adamStates, 0, paramCount * 8));
    HIP_OK(hipMalloc(&dInputs, inputData.size() * sizeof(float)));
    HIP_OK(hipMemcpy(dInputs, inputData.data(), inputData.size() * sizeof(float), hipMemcpyHostToDevice));
    HIP_OK(hipMalloc((void**)&dLoss, 2 * sizeof(float)));
    // the gradient segments start from zero (the reference's random fill there would be noise)
    HIP_OK(hipMemset(params + gradientOffset, 0, bufferSize - gradientOffset));

    // ---- the network: per layer {weights, weightsGrad, biases, biasesGrad} like :146-158
    CvMlpLayer net[kLayerCount];
    CvMatrixDesc srcDescs[kLayerCount], dstDescs[kLayerCount];
    for (int i = 0; i < kLayerCount; i++) {
        memset(&net[i], 0, sizeof(net[i]));
        net[i].weights = params + layers[i].weightsOffset;
        net[i].weightsGrad = params + layers[i].weightsGradTrainingOffset;
        net[i].biases = params + layers[i].biasOffset;
        net[i].biasesGrad = params + layers[i].biasGradOffset;
        net[i].inputSize = kLayerSizes[i];
        net[i].outputSize = kLayerSizes[i + 1];
        net[i].weightLayout = CV_LAYOUT_ROW_MAJOR;
        net[i].weightStride = kLayerSizes[i] * sizeof(NFloat);
        net[i].gradLayout = CV_LAYOUT_TRAINING_OPTIMAL;
        net[i].activation = CV_ACT_LEAKY_RELU;              // max(z, z * 0.001h), fflayer.slang:63-65
        net[i].leakySlope = (float)(NFloat)0.001f;
        srcDescs[i] = CvMatrixDesc{(uint32_t)kLayerSizes[i + 1], (uint32_t)kLayerSizes[i], CV_FLOAT16,
                                   CV_LAYOUT_TRAINING_OPTIMAL, layers[i].weightsGradTrainingSize,
                                   layers[i].weightsGradTrainingOffset, 0};
        dstDescs[i] = CvMatrixDesc{(uint32_t)kLayerSizes[i + 1], (uint32_t)kLayerSizes[i], CV_FLOAT16,
                                   CV_LAYOUT_ROW_MAJOR, layers[i].weightsSize, layers[i].weightsGradOffset,
                                   (size_t)kLayerSizes[i] * sizeof(NFloat)};
    }
    CvMlpDesc mlp = {net, kLayerCount, CV_FLOAT32, CV_FLOAT16, CV_FLOAT16, CV_FLOAT16, CV_FLOAT16, 0, CV_ENCODE_XY_SQUARES, dLoss + 1};
    size_t workspaceBytes = 0;
    CV_OK_OR_FAIL(cvMlpTrainStepWorkspaceSize(&mlp, sampleCount, &workspaceBytes));
    HIP_OK(hipMalloc(&workspace, workspaceBytes));
    // Adam states: one record per element of the parameter buffer, at the element's own index (adjustParameters'
    // states[tid]); a layer's weights and biases find theirs at their offsets
    void *weightStates[kLayerCount], *biasStates[kLayerCount];
    for (int i = 0; i < kLayerCount; i++) {
        weightStates[i] = (uint8_t*)adamStates + layers[i].weightsOffset / sizeof(NFloat) * 8;
        biasStates[i] = (uint8_t*)adamStates + layers[i].biasOffset / sizeof(NFloat) * 8;
    }

    hipStream_t stream = nullptr;
    HIP_OK(hipStreamCreate(&stream));
    auto unfusedIteration = [&]() -> int {
        HIP_OK(hipMemsetAsync(params + gradientTrainingOffset, 0, bufferSize - gradientTrainingOffset, stream));
        CV_OK_OR_FAIL(cvMlpTrainStep(stream, &mlp, dInputs, 2 * sizeof(float), nullptr, 0, 1.0f, sampleCount, dLoss,
                                     workspace, workspaceBytes));
        CV_OK_OR_FAIL(cvConvertMatrices(stream, params, dstDescs, params, srcDescs, kLayerCount));
        CV_OK_OR_FAIL(cvAdamStep(stream, adamStates, params, params + gradientOffset,
                                 (uint32_t)((gradientTrainingOffset - gradientOffset) / sizeof(NFloat)), 0.9f, 0.999f,
                                 1e-7f, 0.01f));
        return 0;
    };
    auto fusedIteration = [&]() -> int {
        CV_OK_OR_FAIL(cvMlpTrainStep(stream, &mlp, dInputs, 2 * sizeof(float), nullptr, 0, 1.0f, sampleCount, dLoss,
                                     workspace, workspaceBytes));
        CV_OK_OR_FAIL(cvMlpAdamStep(stream, &mlp, weightStates, biasStates, 0.9f, 0.999f, 1e-7f, 0.01f));
        return 0;
    };
    hipGraphExec_t graphExec = nullptr;
    hipEvent_t t0, t1;
    HIP_OK(hipEventCreate(&t0));
    HIP_OK(hipEventCreate(&t1));
    HIP_OK(hipEventRecord(t0, stream));
    const int kGraphIterations = 10;
    for (int k = 0; k < iterations;) {
        int done = 1;
        if (unfused) {
            if (unfusedIteration()) return 1;
        } else if (k < kGraphIterations || iterations - k < kGraphIterations) {
            // the first ten iterations run as plain launches (the library looks up its kernels' residency once per
            // device), and so does a tail shorter than the graph
            if (fusedIteration()) return 1;
            if (k + 1 == kGraphIterations) {
                hipGraph_t graph = nullptr;
                HIP_OK(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
                for (int j = 0; j < kGraphIterations; j++)
                    if (fusedIteration()) return 1;
                HIP_OK(hipStreamEndCapture(stream, &graph));
                HIP_OK(hipGraphInstantiate(&graphExec, graph, nullptr, nullptr, 0));
                HIP_OK(hipGraphDestroy(graph));
            }
        } else {
            HIP_OK(hipGraphLaunch(graphExec, stream));
            done = kGraphIterations;
        }
        k += done;
        if (k % 10 == 0 && !timeIt) {
            float loss[2] = {0.f, 0.f};
            HIP_OK(hipStreamSynchronize(stream));
            HIP_OK(hipMemcpy(loss, dLoss, sizeof(loss), hipMemcpyDeviceToHost));
            printf("Loss after %d iterations: %f (mean %f)\n", k, loss[1], loss[0] / sampleCount);
        }
    }
    HIP_OK(hipEventRecord(t1, stream));
    HIP_OK(hipStreamSynchronize(stream));
    if (timeIt) {
        float ms = 0.f;
        HIP_OK(hipEventElapsedTime(&ms, t0, t1));
        printf("%s iteration: %.2f us (%d iterations)\n", unfused ? "unfused" : "fused (ten per graph launch)", ms * 1e3f / iterations, iterations);
    }
    // a digest of the parameters, so that two runs can be compared bit for bit
    std::vector<uint16_t> finalParams(gradientOffset / sizeof(NFloat));
    HIP_OK(hipMemcpy(finalParams.data(), params, gradientOffset, hipMemcpyDeviceToHost));
    uint64_t digest = 1469598103934665603ull;
    for (int i = 0; i < kLayerCount; i++) {
        for (size_t e = 0; e < layers[i].weightsSize / 2; e++) digest = (digest ^ finalParams[layers[i].weightsOffset / 2 + e]) * 1099511628211ull;
        for (size_t e = 0; e < layers[i].biasSize / 2; e++) digest = (digest ^ finalParams[layers[i].biasOffset / 2 + e]) * 1099511628211ull;
    }
    printf("Parameter digest: %016llx\n", (unsigned long long)digest);
    HIP_OK(hipDeviceSynchronize());
    return 0;
}
