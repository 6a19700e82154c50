// cv_mlp_f16.hip -- fp16 instantiations of the fused forward MLP, and the dispatcher.
#include "cv_mlp_stream.h"

namespace cv {

hipError_t launchMlpFp8AsF16(hipStream_t stream, const MlpArgs& a, int numCUs);
hipError_t launchMlpFp8Native(hipStream_t stream, const MlpArgs& a, int numCUs);
hipError_t launchMlpWide16In8(hipStream_t stream, const MlpArgs& a, int numCUs, int H, int NH);
hipError_t launchMlpWide16In16(hipStream_t stream, const MlpArgs& a, int numCUs, int H, int NH);
hipError_t launchMlpWide16In32(hipStream_t stream, const MlpArgs& a, int numCUs, int H, int NH);

// true when the 32-sample-tile kernel (cv_mlp_wide16.h) can take this call; see mlpWide16Eligible there
static bool wide16Shape(const MlpArgs& a, int& H, int& NH, int& K0)
{
    const int L = a.numLayers;
    if (L < 2 || L > 5 || a.inEncoding != kEncodeNone || a.inHalfAsE4M3 || a.noWideTiles) return false;
    K0 = a.layers[0].in;
    if (K0 != 8 && K0 != 16 && K0 != 32) return false;
    if (a.inStride != 2u * (uint64_t)K0 || ((uintptr_t)a.in & 15u) != 0 || a.batch == 0 || a.batch > (1u << 31)) return false;
    const int width = a.layers[0].out;
    if (width != 32 && width != 64) return false;
    // (hidden layers all ReLU or all leaky ReLU)
    const int hiddenAct = a.layers[0].act;
    if (hiddenAct != kActRelu && hiddenAct != kActLeakyRelu) return false;
    for (int l = 0; l < L; ++l) {
        if (l + 1 < L && (a.layers[l].out != width || a.layers[l].act != hiddenAct)) return false;
        if (l > 0 && a.layers[l].in != width) return false;
    }
    // (the last layer: none or ReLU; a leaky network's may be leaky ReLU as well)
    if (a.layers[L - 1].act != kActNone && a.layers[L - 1].act != kActRelu &&
        !(a.layers[L - 1].act == kActLeakyRelu && a.layers[0].act == kActLeakyRelu)) return false;
    if (a.layers[L - 1].out > 32) return false;
    H = width / 32; NH = L - 1;
    // 64-byte rows with one or two hidden layers are bound by their memory traffic, which the streaming kernel
    // moves faster (whole rows through LDS): 71 against 82 us for 32-64-64-8 over 2^22 samples
    // (a leaky network has no streaming instantiation and stays here: 32-64-64-8 over 2^22 samples 191 us on the 16-sample kernel)
    if (K0 == 32 && NH < 3 && hiddenAct == kActRelu) return false;
    return true;
}

hipError_t launchMlpForward(hipStream_t stream, MmaKind kind, const MlpArgs& a, int numCUs)
{
    if (a.batch == 0) return hipSuccess;
    switch (kind) {
    case MmaKind::F16: {
        int H, NH, K0;
        if (wide16Shape(a, H, NH, K0)) {      // 32-sample tiles where the network allows them
            const hipError_t e = K0 == 8 ? launchMlpWide16In8(stream, a, numCUs, H, NH)
                               : K0 == 16 ? launchMlpWide16In16(stream, a, numCUs, H, NH)
                                          : launchMlpWide16In32(stream, a, numCUs, H, NH);
            if (e != hipErrorInvalidValue) return e;
        }
        return dispatchMlp<F16Mma>(stream, a, numCUs); }
    case MmaKind::Fp8AsF16: return launchMlpFp8AsF16(stream, a, numCUs);
    case MmaKind::Fp8Native: return launchMlpFp8Native(stream, a, numCUs);
    default: break;
    }
    return hipErrorInvalidValue;
}

} // namespace cv
