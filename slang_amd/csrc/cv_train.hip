// cv_train.hip -- instantiations and launcher of the fused fp16 training step.
#include "cv_train_impl.h"
#include "cv_train_pair.h"
#include "cv_error.h"
#include <algorithm>

namespace cv {

namespace {

// (input feature tiles, input k-tiles, hidden tiles, hidden layers, output tiles)
#define CV_TRAIN_SHAPES(X) \
    X(1, 1, 1, 1, 1) X(1, 1, 1, 2, 1) X(1, 1, 1, 3, 1) \
    X(1, 1, 2, 1, 1) X(1, 1, 2, 2, 1) X(1, 1, 2, 3, 1) X(1, 1, 2, 4, 1) X(2, 1, 2, 1, 1) X(2, 1, 2, 2, 1) X(2, 1, 2, 3, 1) X(2, 1, 2, 4, 1) \
    X(1, 1, 4, 1, 1) X(1, 1, 4, 2, 1) X(1, 1, 4, 3, 1) X(1, 1, 4, 4, 1) X(2, 1, 4, 1, 1) X(2, 1, 4, 2, 1) X(2, 1, 4, 3, 1) X(2, 1, 4, 4, 1)

struct Shape { int it0, kt0, ht, nhid, mtl; bool ok; };

Shape classify(const MlpArgs& a)
{
    Shape s{0, 0, 0, 0, 0, false};
    const int L = a.numLayers;
    if (L < 2) return s;
    s.it0 = (int)optMT((uint32_t)a.layers[0].in);
    s.kt0 = (int)optKT((uint32_t)a.layers[0].in, 8);
    // the widest hidden layer decides the tiling: 1, 2, 4 or 8 tiles of 16 units; narrower hidden layers are padded to it
    // (rows and columns of zeros in the staged weights)
    int widest = 0;
    for (int l = 0; l + 1 < L; ++l) widest = std::max(widest, (int)optMT((uint32_t)a.layers[l].out));
    s.ht = widest <= 2 ? widest : widest <= 4 ? 4 : widest <= 8 ? 8 : widest;
    s.nhid = L - 1;
    // (16-wide networks with four hidden layers or more than 16 inputs have no instantiation of their own)
    if (s.ht == 1 && (s.nhid > 3 || s.it0 > 1)) s.ht = 2;
    s.mtl = (int)optMT((uint32_t)a.layers[L - 1].out);
    s.ok = true;
    return s;
}

// workgroups of the fused kernels per compute unit (the workspace holds one partial for each).  Two of the paired kernel
// would fit for 32-wide networks (71 KB of LDS, under 128 registers) and were slower: 80 against 72 us for 8-32-32-32-4.
template <class Net>
constexpr int kWorkgroupsPerCU = 1;

template <class Net>
hipError_t launchNet(hipStream_t stream, const TrainLaunch& t, int numCUs)
{
    TrainArgs ta;
    ta.mlp = t.mlp;
    ta.targets = t.targets;
    ta.targetStride = t.targetStride;
    ta.lossScale = t.lossScale;
    ta.partials = t.workspace;
    ta.wantLossMax = t.lossMax ? 1 : 0;
    // one resident workgroup per compute unit, fewer when the batch has less work than that: a workgroup takes four
    // 16-sample tiles (on 64-wide networks four 32-sample rounds) at a time, and every workgroup launched writes a
    // partial that the second kernel reads (the example's 16 samples: one workgroup instead of 256)
    // the paired kernel's LDS: weights, transposes, biases, four pairs' tiles of a round (64-wide networks with four hidden
    // layers and more than 16 inputs exceed it and run on the one-wave kernel)
    constexpr int kPairLdsBytes = 4 * ((Net::totalFrags + (Net::totalTFrags > 0 ? Net::totalTFrags : 1)) * 256 + Net::totalBiasTiles * 16 +
                                       4 * Net::totalXTiles * 256 + 8 * Net::MTMAX * 256 + 12);
    constexpr bool kPairShape = (Net::HT == 4 || Net::HT == 2) && kPairLdsBytes <= 160 * 1024;
    const uint32_t units = kPairShape ? (t.mlp.batch + 31u) / 32u : ((t.mlp.batch + 15u) / 16u + 3u) / 4u;
    const uint32_t resident = (uint32_t)numCUs * (uint32_t)kWorkgroupsPerCU<Net>;
    const uint32_t blocks = units < resident ? (units ? units : 1u) : resident;
    const TrainReduceArgs ra = makeTrainReduceArgs<Net>(t, blocks);
    constexpr uint32_t total = Net::totalGradTiles * 256 + Net::totalDbTiles * 16 + 1;
    // ReLU on every hidden layer and none on the last one gets the straight-line instantiation
    bool plain = t.mlp.layers[Net::L - 1].act == kActNone;
    for (int l = 0; l + 1 < Net::L; ++l) plain = plain && t.mlp.layers[l].act == kActRelu;
    // (the paired kernel also takes hidden layers with leaky ReLU, the example's activation)
    bool leaky = !plain;
    for (int l = 0; l < Net::L; ++l)
        leaky = leaky && (t.mlp.layers[l].act == kActRelu || t.mlp.layers[l].act == kActLeakyRelu || (l + 1 == Net::L && t.mlp.layers[l].act == kActNone));
    // straight-line input loads: float2 samples of the example's encoding, or slices of whole aligned dwords
    const bool xy = t.mlp.inEncoding == kEncodeXYSquares;
    const bool dwords = !xy && t.mlp.layers[0].in % 2 == 0 && t.mlp.inAlign >= 4u;
    const int variant = !plain || !(xy || dwords) ? 0 : xy ? 2 : 1;
    const bool pairLeaky = kPairShape && leaky && (dwords || xy);
    // a launch of one workgroup of the one-wave-per-SIMD kernel finishes the step itself
    ta.finishInKernel = (blocks == 1 && !(kPairShape && (variant != 0 || pairLeaky))) ? 1 : 0;
    ta.finish = ra;
    noteKernel(false, "mlpTrainKernel<IT0=%d,KT0=%d,HT=%d,hidden=%d,MTL=%d,%s> + mlpTrainReduceKernel", Net::IT0, Net::KT0,
               Net::HT, Net::L - 1, Net::MTL,
               variant == 0 ? "runtime-act,any-input" : variant == 1 ? "relu/none,dword-input" : "relu/none,xy-input");
    // 64- and 32-wide networks with these activations run on the two-waves-per-SIMD kernel
    constexpr bool kPair = kPairShape;
    if constexpr (kPair) {
        if (variant != 0 || pairLeaky)
            noteKernel(false, "mlpTrainPairKernel<IT0=%d,KT0=%d,HT=%d,hidden=%d,MTL=%d,%s,%s> + mlpTrainReduceKernel", Net::IT0,
                       Net::KT0, Net::HT, Net::L - 1, Net::MTL, pairLeaky ? "leaky-or-relu" : "relu/none", xy ? "xy-input" : "dword-input");
        if (pairLeaky && xy)   hipLaunchKernelGGL((mlpTrainPairKernel<Net, kLoadXY, true>), dim3(blocks), dim3(512), 0, stream, ta);
        else if (pairLeaky)    hipLaunchKernelGGL((mlpTrainPairKernel<Net, kLoadDwords, true>), dim3(blocks), dim3(512), 0, stream, ta);
        else if (variant == 1) hipLaunchKernelGGL((mlpTrainPairKernel<Net, kLoadDwords>), dim3(blocks), dim3(512), 0, stream, ta);
        else if (variant == 2) hipLaunchKernelGGL((mlpTrainPairKernel<Net, kLoadXY>), dim3(blocks), dim3(512), 0, stream, ta);
    } else {
        if (variant == 1)      hipLaunchKernelGGL((mlpTrainKernel<Net, kActRelu, kActNone, kLoadDwords>), dim3(blocks), dim3(256), 0, stream, ta);
        else if (variant == 2) hipLaunchKernelGGL((mlpTrainKernel<Net, kActRelu, kActNone, kLoadXY>), dim3(blocks), dim3(256), 0, stream, ta);
    }
    if (variant == 0 && !pairLeaky) hipLaunchKernelGGL((mlpTrainKernel<Net, -1, -1, kLoadAny>), dim3(blocks), dim3(256), 0, stream, ta);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (ta.finishInKernel) return hipSuccess;
    hipLaunchKernelGGL((mlpTrainReduceKernel<Net>), dim3((total + 63) / 64), dim3(64 * kReduceWaves), 0, stream, ra);
    return hipGetLastError();
}

} // namespace

size_t trainWorkspaceBytes(const MlpArgs& a, int numCUs)
{
    const Shape s = classify(a);
    if (!s.ok) return 0;
    if (s.ht == 8) return trainQuadWorkspaceBytes(a, numCUs);
#define CV_X(I0, K0, HT, NH, ML) \
    if (s.it0 == I0 && s.kt0 == K0 && s.ht == HT && s.nhid == NH && s.mtl == ML) \
        return (size_t)numCUs * kWorkgroupsPerCU<TrainNet<I0, K0, HT, NH, ML>> * TrainNet<I0, K0, HT, NH, ML>::partialFloats * sizeof(float);
    CV_TRAIN_SHAPES(CV_X)
#undef CV_X
    return 0;
}

hipError_t launchMlpTrain(hipStream_t stream, const TrainLaunch& t, int numCUs)
{
    if (t.mlp.batch == 0) return hipSuccess;
    const Shape s = classify(t.mlp);
    if (!s.ok) return hipErrorInvalidValue;
    if (s.ht == 8) return launchMlpTrainQuad(stream, t, numCUs);
    if (trainTeamTakes(t)) return launchMlpTrainTeam(stream, t, numCUs);
#define CV_X(I0, K0, HT, NH, ML) \
    if (s.it0 == I0 && s.kt0 == K0 && s.ht == HT && s.nhid == NH && s.mtl == ML) \
        return launchNet<TrainNet<I0, K0, HT, NH, ML>>(stream, t, numCUs);
    CV_TRAIN_SHAPES(CV_X)
#undef CV_X
    return hipErrorInvalidValue;
}

} // namespace cv
