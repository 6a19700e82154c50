// cv_train_team.hip -- instantiations and launcher of the fused fp16 training step whose waves share a tile by kind of work.
#include "cv_train_team.h"
#include "cv_error.h"

namespace cv {

namespace {

template <int NH>
hipError_t launchTeam(hipStream_t stream, const TrainLaunch& t, int numCUs)
{
    typedef TrainNet<1, 1, 4, NH, 1> Net;
    TrainArgs ta;
    ta.mlp = t.mlp;
    ta.targets = t.targets;
    ta.targetStride = t.targetStride;
    ta.lossScale = t.lossScale;
    ta.partials = t.workspace;
    ta.wantLossMax = t.lossMax ? 1 : 0;
    ta.finishInKernel = 0;
    // one workgroup per compute unit = two teams, each with tiles of 32 samples of its own
    const uint32_t pairsOfTiles = ((t.mlp.batch + 31u) / 32u + 1u) / 2u;
    const uint32_t blocks = pairsOfTiles < (uint32_t)numCUs ? pairsOfTiles : (uint32_t)numCUs;
    const TrainReduceArgs ra = makeTrainReduceArgs<Net>(t, blocks);
    ta.finish = ra;
    noteKernel(false, "mlpTrainTeamKernel<inputs<=16,hidden=%dx64,outputs<=16,relu/none,dword-input> + mlpTrainReduceKernel", NH);
    hipLaunchKernelGGL((mlpTrainTeamKernel<Net>), dim3(blocks), dim3(512), 0, stream, ta);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    constexpr uint32_t total = Net::totalGradTiles * 256 + Net::totalDbTiles * 16 + 1;
    hipLaunchKernelGGL((mlpTrainReduceKernel<Net>), dim3((total + 63) / 64), dim3(64 * kReduceWaves), 0, stream, ra);
    return hipGetLastError();
}

} // namespace

bool trainTeamTakes(const TrainLaunch& t)
{
    const MlpArgs& a = t.mlp;
    const int L = a.numLayers;
    if (!t.splitByRole || L < 2 || L > 5 || a.batch < kTrainTeamMinBatch) return false;
    if (a.inEncoding != kEncodeNone || a.layers[0].in > 16 || a.layers[0].in % 2 != 0 || a.inAlign < 4u) return false;
    if (a.layers[L - 1].out > 16 || a.layers[L - 1].act != kActNone) return false;
    for (int l = 0; l < L; ++l) {
        if (l + 1 < L && (a.layers[l].out != 64 || a.layers[l].act != kActRelu)) return false;
        const int layout = a.layers[l].shape.layout;
        if (layout != kRowMajor && layout != kColumnMajor) return false;
    }
    return true;
}

hipError_t launchMlpTrainTeam(hipStream_t stream, const TrainLaunch& t, int numCUs)
{
    switch (t.mlp.numLayers - 1) {
    case 1: return launchTeam<1>(stream, t, numCUs);
    case 2: return launchTeam<2>(stream, t, numCUs);
    case 3: return launchTeam<3>(stream, t, numCUs);
    case 4: return launchTeam<4>(stream, t, numCUs);
    }
    return hipErrorInvalidValue;
}

} // namespace cv
