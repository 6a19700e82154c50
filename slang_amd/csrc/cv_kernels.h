// cv_kernels.h -- host-callable launchers of the gfx950 kernels (internal to the library).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "coopvec.h"
#include "cv_layout.h"

namespace cv {

// ---- batched matMul[Add] ------------------------------------------------------------------
struct MatMulArgs {
    const uint8_t* in;      // sample s at in + s*inStride
    uint8_t* out;           // sample s at out + s*outStride
    const uint8_t* mat;     // matrix base (offset already applied)
    const uint8_t* bias;    // bias base (offset already applied) or nullptr
    uint64_t inStride, outStride;
    MatrixShape shape;      // the matrix as it lies in memory
    int32_t transpose;      // memory holds k x m and is used transposed
    int32_t m, k;
    int32_t inCt;           // element type of the input vectors in memory
    int32_t biasCt;
    int32_t outCt;          // kF16, kF32 or kS32
    int32_t act;
    float slope;
    int32_t accumulate;
    uint32_t batch;
    uint32_t inAlign, outAlign;   // largest power of two (<= 16) dividing base address and stride
    uint32_t rowOff;              // first matrix row of the block this launch computes (set by the launcher)
    int32_t inUnsigned, matUnsigned;   // MmaKind::I8AnySign: which side holds unsigned bytes
};

enum class MmaKind : int {
    F16 = 0, Fp8AsF16 = 1, Fp8Native = 2, I8 = 3,
    Bf16 = 4,            // bfloat16 vectors and matrix
    Bf8AsF16 = 5,        // e5m2 vectors and matrix, decoded to fp16 operands
    F16VecAsE4M3 = 6,    // fp16 vectors quantised to e4m3 on load, e4m3 matrix (matMul only)
    I8AnySign = 7,       // signed/unsigned bytes on either side (matMul only)
    F32 = 8,             // fp32 vectors and matrix (matMul only)
    Scalar = 9           // combinations without a matrix instruction (16/32-bit integers, mixed forms): cv_matmul_scalar.hip
};

// Returns hipSuccess, or hipErrorInvalidValue when no kernel covers (m,k): k beyond what one
// 16-row block of the matrix can hold in LDS.
hipError_t launchMatMul(hipStream_t stream, MmaKind kind, const MatMulArgs& args, int numCUs);
// the scalar definition evaluated as written, for the combinations MmaKind::Scalar stands for
hipError_t launchMatMulScalar(hipStream_t stream, const MatMulArgs& args, int numCUs);

// ---- fused forward MLP --------------------------------------------------------------------
constexpr int kMaxMlpLayers = 8;
struct MlpLayerArgs {
    const uint8_t* w;       // weights base
    const uint8_t* bias;    // fp16 biases or nullptr
    MatrixShape shape;      // out x in as it lies in memory
    int32_t in, out;
    int32_t act;
    float slope;
};
struct MlpArgs {
    MlpLayerArgs layers[kMaxMlpLayers];
    int32_t numLayers;
    const uint8_t* in;
    uint8_t* out;           // fp16 [batch][lastOut]
    uint64_t inStride, outStride;
    uint32_t batch;
    uint32_t inAlign, outAlign;
    int32_t inEncoding;     // kEncodeNone, or kEncodeXYSquares: a sample is a float2, layer 0 sees (x, y, x*x, y*y)
    int32_t inHalfAsE4M3;   // e4m3 networks: the vectors in memory are fp16 and are quantised to e4m3 as they are loaded
    int32_t noWideTiles;    // keep to the kernels on 16-sample tiles (cross-checks)
};
enum : int { kEncodeNone = 0, kEncodeXYSquares = 1 };
// hipErrorInvalidValue when no built-in specialisation covers the layer shapes
hipError_t launchMlpForward(hipStream_t stream, MmaKind kind, const MlpArgs& args, int numCUs);
// any layer sizes up to 128 (weights read from LDS); hipErrorInvalidValue beyond that
hipError_t launchMlpGeneric(hipStream_t stream, MmaKind kind, const MlpArgs& args, int numCUs);
// permutohedral encoding of fp16 positions fused in front of an fp16 network (weights in LDS, every dimension <= 128);
// hipErrorInvalidValue for encoders or networks the kernel does not take
hipError_t launchPermutoMlp(hipStream_t stream, const CvPermutoDesc& desc, const void* positions, uint64_t positionStride,
                            const void* featureTable, const MlpArgs& mlp, int numCUs);
// CV_OK, or the reason why an encoder description is malformed (recorded as the thread's last error)
CvResult checkPermutoDesc(const char* who, const CvPermutoDesc* desc);
// the fp16 run-time-size kernel that also leaves every layer's pre-activations (tapZ[l]) and activations (tapX[l]) in
// memory as [batch][out_l] halfs, where the pointer is not null; hipErrorInvalidValue beyond its limits
hipError_t launchMlpGenericTaps(hipStream_t stream, const MlpArgs& args, uint8_t* const* tapZ, uint8_t* const* tapX, int numCUs);
// networks of one type T = float (MmaKind::F32) or bfloat16 (MmaKind::Bf16): vectors, weights, biases, results;
// same limits as launchMlpGeneric
hipError_t launchMlpFloat(hipStream_t stream, MmaKind kind, const MlpArgs& args, int numCUs);

// ---- fused training step ------------------------------------------------------------------
struct TrainLaunch {
    MlpArgs mlp;                 // layers, input, batch
    const uint8_t* targets;      // fp16 [batch][lastOut] or nullptr
    uint64_t targetStride;
    float lossScale;
    // gradient destinations, per layer
    uint8_t* wGrad[kMaxMlpLayers];
    uint8_t* bGrad[kMaxMlpLayers];
    MatrixShape gradShape[kMaxMlpLayers];
    int32_t gradCt;
    int32_t carrierCt;           // kF16, or kF32 for a network of float (layer-by-layer step only)
    float* lossSum;
    float* lossMax;              // optional: max over the samples of the per-sample loss
    float* workspace;            // partials
    int32_t splitByRole;         // take the kernel of launchMlpTrainTeam where trainTeamTakes() says it applies
};
// Bytes of workspace the training step needs for this network on a device with numCUs compute
// units; 0 when no built-in specialisation covers the layer shapes.
size_t trainWorkspaceBytes(const MlpArgs& shapes, int numCUs);
hipError_t launchMlpTrain(hipStream_t stream, const TrainLaunch& args, int numCUs);
// The fused step whose waves share a tile of samples by kind of work (forward, backward, weight gradients) and keep the
// weights in registers: up to 16 inputs, one to four ReLU hidden layers of 64 units, up to 16 outputs without activation,
// Row/ColumnMajor weights, batches of at least kTrainTeamMinBatch samples.  Same workspace and partials as launchMlpTrain,
// which calls it for a step that asks for it (splitByRole) where trainTeamTakes() says it applies.
// The fused step for 128-wide hidden layers (one or two of them, ReLU; up to 32 inputs, up to 16 outputs without
// activation): bytes of workspace, 0 where it does not apply; launchMlpTrain / trainWorkspaceBytes call these.
size_t trainQuadWorkspaceBytes(const MlpArgs& shapes, int numCUs);
hipError_t launchMlpTrainQuad(hipStream_t stream, const TrainLaunch& args, int numCUs);
constexpr uint32_t kTrainTeamMinBatch = 16384;
bool trainTeamTakes(const TrainLaunch& args);
hipError_t launchMlpTrainTeam(hipStream_t stream, const TrainLaunch& args, int numCUs);
// The same step layer by layer through the batched kernels, for any layer sizes: per-layer vectors
// of the whole batch are parked in the workspace, whose size therefore grows with mlp.batch.
size_t trainGeneralWorkspaceBytes(const MlpArgs& shapesAndBatch, int numCUs, int carrierCt);
hipError_t launchMlpTrainGeneral(hipStream_t stream, const TrainLaunch& args, int numCUs);

// ---- batched outer-product / reduce-sum accumulate ---------------------------------------
struct OuterArgs {
    const uint8_t* a; const uint8_t* b;   // fp16 [batch][m], [batch][n]
    uint64_t aStride, bStride;
    uint32_t aAlign, bAlign;
    int32_t m, n;
    uint32_t batch;
    uint8_t* mat;                          // destination (offset applied)
    MatrixShape shape;                     // m x n, FLOAT16 or FLOAT32, any layout
    float* partials;
};
size_t outerWorkspaceBytes(int m, int n, uint32_t batch, int numCUs);
hipError_t launchOuterProduct(hipStream_t stream, const OuterArgs& args, int numCUs);

// fp32 vectors into an fp32 matrix on the matrix pipeline (cv_accum_f32.hip); b == nullptr with n == 1 is the reduce-sum form
size_t outerF32WorkspaceBytes(int m, int n, uint32_t batch, int numCUs);
hipError_t launchOuterProductF32(hipStream_t stream, const uint8_t* a, uint64_t aStride, int m, const uint8_t* b, uint64_t bStride,
                                 int n, uint32_t batch, uint8_t* mat, const MatrixShape& shape, void* workspace, int numCUs);

// The scalar definition of both accumulate operators for every plain element type (cv_accum_scalar.hip):
// matrix[i][j] += cast<MatT>(a[i] * b[j]) summed over the batch; b == nullptr with n == 1 is the reduce-sum form.
bool isPlainComponent(int ct);
size_t accumScalarWorkspaceBytes(int m, int n, uint32_t batch);
hipError_t launchAccumScalar(hipStream_t stream, const uint8_t* a, uint64_t aStride, int m, const uint8_t* b, uint64_t bStride,
                             int n, int tCt, uint32_t batch, uint8_t* mat, const MatrixShape& shape, void* workspace);

struct ReduceSumArgs {
    const uint8_t* v;                      // fp16 [batch][n]
    uint64_t vStride;
    int32_t n, colsPerGroup;
    uint32_t batch;
    uint8_t* buf;                          // destination (offset applied)
    int32_t bufCt;                         // kF16 or kF32
    float* partials;
};
size_t reduceSumWorkspaceBytes(uint32_t batch, int numCUs);
hipError_t launchReduceSum(hipStream_t stream, const ReduceSumArgs& args, int numCUs);

// ---- layout conversion --------------------------------------------------------------------
struct ConvertItem {
    const uint8_t* src;
    uint8_t* dst;
    MatrixShape srcShape, dstShape;
    uint32_t dstBytes;      // bytes of the destination to cover (padding is zero-filled)
};
constexpr int kMaxConvertItems = 32;   // keeps ConvertArgs under the 4 KB kernel-argument limit
struct ConvertArgs {
    ConvertItem items[kMaxConvertItems];
    uint32_t count;
};
hipError_t launchConvert(hipStream_t stream, const ConvertArgs& args);

} // namespace cv
