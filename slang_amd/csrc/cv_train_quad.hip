// cv_train_quad.hip -- instantiations and launcher of the fused fp16 training step for 128-wide hidden layers.
#include "cv_train_quad.h"
#include "cv_error.h"

namespace cv {

namespace {

// (16-feature tiles of the input, hidden layers): up to 32 inputs, one or two hidden layers, the wider of 65..128 units (ReLU or leaky
// ReLU), up to 16 outputs without activation
#define CV_TRAIN_QUAD_SHAPES(X) X(1, 1) X(1, 2) X(2, 1) X(2, 2)

template <int IT0, int NH>
hipError_t launchQuad(hipStream_t stream, const TrainLaunch& t, int numCUs)
{
    typedef TrainNet<IT0, 1, 8, NH, 1> Net;
    TrainArgs ta;
    ta.mlp = t.mlp;
    ta.targets = t.targets;
    ta.targetStride = t.targetStride;
    ta.lossScale = t.lossScale;
    ta.partials = t.workspace;
    ta.wantLossMax = t.lossMax ? 1 : 0;
    ta.finishInKernel = 0;
    // one workgroup (a group of four waves, rounds of 64 samples) per compute unit, fewer for a small batch
    const uint32_t rounds = (t.mlp.batch + 63u) / 64u;
    const uint32_t blocks = rounds < (uint32_t)numCUs ? rounds : (uint32_t)numCUs;
    const TrainReduceArgs ra = makeTrainReduceArgs<Net>(t, blocks);
    ta.finish = ra;
    // (the leaky instantiation also takes an activation behind the last layer)
    bool leaky = t.mlp.layers[Net::L - 1].act != kActNone;
    for (int l = 0; l + 1 < Net::L; ++l) leaky = leaky || t.mlp.layers[l].act == kActLeakyRelu;
    noteKernel(false, "mlpTrainQuadKernel<IT0=%d,HT=8,hidden=%d,MTL=1,%s> + mlpTrainReduceKernel", IT0, NH, leaky ? "leaky-or-relu" : "relu/none");
    if (leaky) hipLaunchKernelGGL((mlpTrainQuadKernel<Net, true>), dim3(blocks), dim3(256), 0, stream, ta);
    else       hipLaunchKernelGGL((mlpTrainQuadKernel<Net, false>), dim3(blocks), dim3(256), 0, stream, ta);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    constexpr uint32_t total = Net::totalGradTiles * 256 + Net::totalDbTiles * 16 + 1;
    hipLaunchKernelGGL((mlpTrainReduceKernel<Net>), dim3((total + 63) / 64), dim3(64 * kReduceWaves), 0, stream, ra);
    return hipGetLastError();
}

// the shape of a network this kernel takes: (input tiles, hidden layers), or (0, 0)
void classifyQuad(const MlpArgs& a, int& it0, int& nh)
{
    it0 = nh = 0;
    const int L = a.numLayers;
    if (L < 2 || L > 3 || a.inEncoding != kEncodeNone) return;
    if (a.layers[0].in < 1 || a.layers[0].in > 32 || a.layers[L - 1].out > 16 ||
        (a.layers[L - 1].act != kActNone && a.layers[L - 1].act != kActRelu && a.layers[L - 1].act != kActLeakyRelu)) return;
    // (the caller sends networks here whose widest hidden layer has 65 to 128 units; a narrower one is padded)
    for (int l = 0; l + 1 < L; ++l)
        if (optMT((uint32_t)a.layers[l].out) > 8u || (a.layers[l].act != kActRelu && a.layers[l].act != kActLeakyRelu)) return;
    it0 = (int)optMT((uint32_t)a.layers[0].in);
    nh = L - 1;
}

} // namespace

size_t trainQuadWorkspaceBytes(const MlpArgs& a, int numCUs)
{
    int it0, nh;
    classifyQuad(a, it0, nh);
#define CV_X(I0, NH) if (it0 == I0 && nh == NH) return (size_t)numCUs * TrainNet<I0, 1, 8, NH, 1>::partialFloats * sizeof(float);
    CV_TRAIN_QUAD_SHAPES(CV_X)
#undef CV_X
    return 0;
}

hipError_t launchMlpTrainQuad(hipStream_t stream, const TrainLaunch& t, int numCUs)
{
    int it0, nh;
    classifyQuad(t.mlp, it0, nh);
#define CV_X(I0, NH) if (it0 == I0 && nh == NH) return launchQuad<I0, NH>(stream, t, numCUs);
    CV_TRAIN_QUAD_SHAPES(CV_X)
#undef CV_X
    return hipErrorInvalidValue;
}

} // namespace cv
