/*
 * coopvec.h -- C-ABI of the MI355X (gfx950) cooperative-vector library.
 *
 * The library serves the operator surface Slang declares for CoopVec<T,N>
 * (source/slang/hlsl.meta.slang:32540-33841) and the two host calls the example
 * examples/mlp-training-coopvec/mlp-training-coopvec.cpp makes on slang-rhi
 * (getCooperativeVectorMatrixSize :305, convertCooperativeVectorMatrix :227).
 *
 * Slang maps one logical vector to one shader thread; here one call processes a whole
 * batch of vectors ("samples"): sample s of a batch lives at `base + s * stride` bytes.
 * Arguments that are `constexpr` in Slang (interpretations, k, layout, transpose, stride)
 * select a kernel specialisation; everything else is a device pointer or byte offset.
 *
 * Conventions
 *   - every pointer named *device* memory is a plain HIP device address owned by the caller;
 *     the library never allocates or frees device memory (scratch comes in as `workspace`);
 *   - every call is asynchronous on the given stream (a `hipStream_t` passed as void*;
 *     NULL = the default stream) and returns a SlangResult-compatible code
 *     (include/slang.h:1377-1464): 0 = OK, negative = failure; nothing throws;
 *   - calls are thread-compatible: the only global state is a per-thread error string and
 *     per-device caches of immutable device facts (compute-unit count, kernel residency), kept
 *     in atomics / call_once;
 *   - vectors must start at 16-byte-aligned addresses (hlsl.meta.slang:30761-30764,
 *     30874-30878); matrices and biases at 64-byte-aligned addresses like the example's
 *     sub-allocations (mlp-training-coopvec.cpp:273-279).
 */
#ifndef COOPVEC_H
#define COOPVEC_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(_WIN32)
#define CV_API __declspec(dllexport)
#else
#define CV_API __attribute__((visibility("default")))
#endif

/* ---- result codes: numerically equal to SLANG_OK / SLANG_E_* (include/slang.h:1400-1464) */
typedef int32_t CvResult;
#define CV_OK                  ((CvResult)0)
#define CV_FAIL                ((CvResult)0x80004005)
#define CV_E_NOT_IMPLEMENTED   ((CvResult)0x80004001)
#define CV_E_INVALID_ARG       ((CvResult)0x80070057)
#define CV_E_BUFFER_TOO_SMALL  ((CvResult)0x82000001)
#define CV_E_INTERNAL_FAIL     ((CvResult)0x82000006)
#define CV_E_NOT_AVAILABLE     ((CvResult)0x82000007)
#define CV_FAILED(r)           ((r) < 0)

/* ---- CoopVecMatrixLayout (hlsl.meta.slang:32547-32553, include/slang.h:948-955) */
typedef enum CvMatrixLayout {
    CV_LAYOUT_ROW_MAJOR = 0,
    CV_LAYOUT_COLUMN_MAJOR = 1,
    CV_LAYOUT_INFERENCING_OPTIMAL = 2,
    CV_LAYOUT_TRAINING_OPTIMAL = 3
} CvMatrixLayout;

/* ---- CoopVecComponentType (hlsl.meta.slang:32558-32575), same numeric values.  Used both
 *      for interpretations and for the element type of a vector in memory. */
typedef enum CvComponentType {
    CV_FLOAT_E4M3 = 0, CV_FLOAT_E5M2 = 1, CV_FLOAT16 = 2, CV_FLOAT32 = 3, CV_FLOAT64 = 4,
    CV_SINT8 = 5, CV_SINT16 = 6, CV_SINT32 = 7, CV_SINT64 = 8, CV_SINT8_PACKED = 9,
    CV_UINT8 = 10, CV_UINT16 = 11, CV_UINT32 = 12, CV_UINT64 = 13, CV_UINT8_PACKED = 14,
    /* extension: bfloat16 operands (v_mfma_f32_16x16x32_bf16).  Slang's CoopVecComponentType has no
     * such entry (SLANG_SCALAR_TYPE_BFLOAT16 = 16 exists as a scalar type only, include/slang.h:2155);
     * accepted by cvMatMul, cvGetMatrixSize and cvConvertMatrices. */
    CV_BFLOAT16 = 15,
    CV_COMPONENT_NONE = -1
} CvComponentType;

/* ---- the host API's numbering of the same types: rhi::CooperativeVectorComponentType
 *      (include/slang-gfx.h:1748-1765), which is what the example passes to
 *      getCooperativeVectorMatrixSize and puts into CooperativeVectorMatrixDesc.componentType
 *      (mlp-training-coopvec.cpp:212,220,308).  It differs from the shader-side numbering above
 *      (Float16 is 0 there, FLOAT_E4M3 is 0 here): every entry point of this library takes
 *      CvComponentType, so a caller holding an rhi value converts it first. */
typedef enum CvRhiComponentType {
    CV_RHI_FLOAT16 = 0, CV_RHI_FLOAT32 = 1, CV_RHI_FLOAT64 = 2,
    CV_RHI_SINT8 = 3, CV_RHI_SINT16 = 4, CV_RHI_SINT32 = 5, CV_RHI_SINT64 = 6,
    CV_RHI_UINT8 = 7, CV_RHI_UINT16 = 8, CV_RHI_UINT32 = 9, CV_RHI_UINT64 = 10,
    CV_RHI_SINT8_PACKED = 11, CV_RHI_UINT8_PACKED = 12, CV_RHI_FLOAT_E4M3 = 13, CV_RHI_FLOAT_E5M2 = 14
} CvRhiComponentType;

/* Activation fused behind a matMulAdd.  RELU is max(z, 0) as the neural module defines it
 * (source/standard-modules/neural/activations.slang:25-42); the kernels evaluate it with the packed fp16
 * maximum, which returns 0 for a NaN z (the scalar definition keeps the NaN): NaN results of a fused RELU,
 * in cvMatMul and in the fused networks alike, are outside the parity claim; LEAKY_RELU is the example's
 * max(z, z * slope) evaluated in half (examples/mlp-training-coopvec/fflayer.slang:64-65). */
typedef enum CvActivation {
    CV_ACT_NONE = 0, CV_ACT_RELU = 1, CV_ACT_LEAKY_RELU = 2,
    /* the remaining activations of the neural module (activations.slang:88-233), evaluated on the
     * fp16 (or fp32) result element: in fp32, rounded once */
    CV_ACT_SIGMOID = 3, CV_ACT_TANH = 4, CV_ACT_EXP = 5, CV_ACT_SINE = 6, CV_ACT_SILU = 7, CV_ACT_QUICK_GELU = 8
} CvActivation;

/* Flags of CvMatMulDesc / CvMlpDesc.
 * By default FLOAT_E4M3 operands are decoded (exactly) to fp16 and multiplied on the fp16
 * matrix pipeline, whose accumulation is fp32-grade: that path meets the fp32-accumulated
 * parity bar.  CV_FLAG_FP8_MATRIX_PIPELINE multiplies them on the fp8 matrix pipeline
 * instead; gfx950 aligns the products of one such instruction to the largest of them and
 * keeps about 11 bits below it, so results that cancel carry an absolute error of up to
 * ~2^-12 * sum|terms|.  No effect on other types. */
#define CV_FLAG_FP8_MATRIX_PIPELINE 1u
/* cvMlpTrainStep[WorkspaceSize]: take the layer-by-layer step (the one that serves any layer sizes)
 * also where a fused kernel exists.  Same rounding points; for cross-checking the two. */
#define CV_FLAG_LAYERWISE_TRAINING 2u
/* cvMlpForward: keep to the kernels that work on 16-sample tiles (cross-checks of the 32-sample-tile kernels) */
#define CV_FLAG_FORWARD_TILE16 4u
/* cvMlpTrainStep: where it applies (fp16, up to 16 inputs, one to four RELU hidden layers of 64 units, up to 16 outputs
 * without activation, Row/ColumnMajor weights, at least 16384 samples) take the fused kernel whose waves share a tile of
 * samples by kind of work (forward, backward, weight gradients) and keep the weights in registers.  Same rounding points
 * and the same bar as the default kernels, in which every wave takes whole samples through the step; measured slower
 * than those on MI355X (8-64-64-64-64-1 at 2^20 samples: 151 against 124 us), hence not the default. */
#define CV_FLAG_TRAIN_SPLIT_BY_ROLE 8u

/* Mirrors the fields the example fills in rhi::CooperativeVectorMatrixDesc
 * (mlp-training-coopvec.cpp:204-225).  `offset` is in bytes from the buffer handed to
 * cvConvertMatrices; rowColumnStride is bytes between rows (RowMajor) or columns
 * (ColumnMajor), 0 = tightly packed, ignored for the Optimal layouts. */
typedef struct CvMatrixDesc {
    uint32_t rowCount;
    uint32_t colCount;
    int32_t  componentType;   /* CvComponentType */
    int32_t  layout;          /* CvMatrixLayout */
    size_t   size;
    size_t   offset;
    size_t   rowColumnStride;
} CvMatrixDesc;

/* Shape of include/slang.h:5215-5229 CooperativeVectorCombination, with component types. */
typedef struct CvCombination {
    int32_t  inputType;
    int32_t  inputInterpretation;
    uint32_t inputPackingFactor;
    int32_t  matrixInterpretation;
    int32_t  biasInterpretation;   /* CV_COMPONENT_NONE: no bias operand */
    int32_t  resultType;
    int32_t  transpose;
} CvCombination;

/* ------------------------------------------------------------------------------------ */
/* library                                                                              */
/* ------------------------------------------------------------------------------------ */

/* Version of this ABI (major<<16 | minor). */
CV_API uint32_t cvGetVersion(void);
/* Message describing the last failure on the calling thread ("" if none). */
CV_API const char* cvGetLastErrorMessage(void);
/* Diagnostics: the kernel specialisation(s) the calling thread's last operator call launched
 * (e.g. "matmulKernel<f16,MT=4,KT=2,NT=2,out=f16,streaming>"); "" before the first launch. */
CV_API const char* cvGetLastKernelName(void);
/* Helpers replacing hlsl.meta.slang:32578-32593 / :32596-32633 / :32636-32670. */
CV_API int32_t cvComponentPackingFactor(int32_t componentType);
CV_API int32_t cvComponentScalarType(int32_t componentType);      /* SLANG_SCALAR_TYPE_* or -1 */
CV_API int32_t cvComponentTypeStride(int32_t componentType);      /* bytes, -1 if unknown */
/* rhi::CooperativeVectorComponentType -> CvComponentType and back; CV_COMPONENT_NONE (-1) for a
 * value outside the enum. */
CV_API int32_t cvComponentTypeFromRhi(int32_t rhiComponentType);
CV_API int32_t cvComponentTypeToRhi(int32_t componentType);
/* The (type, interpretation) combinations cvMatMul accepts, in the shape a host compares
 * against ICooperativeTypesMetadata (include/slang.h:5231-5273).  Returns the total count;
 * fills at most `capacity` entries. */
CV_API uint32_t cvQuerySupportedCombinations(CvCombination* out, uint32_t capacity);

/* ------------------------------------------------------------------------------------ */
/* host surface: size query and layout conversion                                       */
/* ------------------------------------------------------------------------------------ */

/* Replaces rhi::IDevice::getCooperativeVectorMatrixSize (call site
 * mlp-training-coopvec.cpp:305-311).  Size in bytes (multiple of 64 for Optimal layouts). */
CV_API CvResult cvGetMatrixSize(uint32_t rowCount, uint32_t colCount, int32_t componentType,
                                int32_t layout, size_t rowColumnStride, size_t* outSize);

/* Replaces rhi::ICommandEncoder::convertCooperativeVectorMatrix (call site
 * mlp-training-coopvec.cpp:227-232): converts `count` matrices from srcDescs[i] inside
 * srcBuffer to dstDescs[i] inside dstBuffer in one launch.  Row/column counts must match;
 * component types must match or be a FLOAT16/FLOAT32 pair (round to nearest even).
 * Padding of Optimal destinations is written as zero.  Source and destination ranges must
 * not overlap.  At most 64 matrices per call. */
CV_API CvResult cvConvertMatrices(void* stream, void* dstBuffer, const CvMatrixDesc* dstDescs,
                                  const void* srcBuffer, const CvMatrixDesc* srcDescs,
                                  uint32_t count);

/* ------------------------------------------------------------------------------------ */
/* operator surface                                                                     */
/* ------------------------------------------------------------------------------------ */

/* coopVecMatMul / coopVecMatMulAdd / coopVecMatMul[Add]Packed over a batch
 * (hlsl.meta.slang:32786-33190; IR operand order slang-ir-insts.lua:1694-1718):
 *
 *   output[s][i] = act( cast<resultType>( sum_{j<k} W[i][j] * input[s][j]  + bias[i] ) )
 *
 * W is M x k unless `transpose`, in which case memory holds k x M and is used transposed.
 * Float types accumulate in fp32, integer types in int32 (exact).
 * Type combinations: those with a matrix instruction (cvQuerySupportedCombinations lists all), and, for
 * the rest of the fallback's switch (hlsl.meta.slang:32866-32907), every mix of SINT8/16/32/64, UINT8/16/32/64,
 * FLOAT16, FLOAT32 and FLOAT64 for vector, matrix, bias and result (FLOAT16/32/64, SINT32/64 or UINT32/64):
 * these run as the scalar definition, operands cast to the result type first, RowMajor / ColumnMajor only.
 * There, as in the fallback (hlsl.meta.slang:32839-32856), a packed inputInterpretation (32-bit elements of four
 * sign-extended bytes) goes with every matrix type, and a plain inputInterpretation other than the stored
 * type is accepted and changes nothing: the stored elements are cast to the result type.
 * accumulate != 0 gives the member forms matMulAccum / matMulAddAccum
 * (hlsl.meta.slang:31476-31650): output += result (activation must be NONE).
 */
typedef struct CvMatMulDesc {
    /* vectors */
    const void* input;          /* device; sample s at input + s*inputStride */
    size_t      inputStride;    /* bytes */
    int32_t     inputType;      /* element type of CoopVec<U,PackedK> in memory */
    int32_t     inputInterpretation;
    int32_t     k;              /* logical input length; == 4*PackedK for *_PACKED */
    void*       output;         /* device; sample s at output + s*outputStride */
    size_t      outputStride;
    int32_t     resultType;     /* element type T of CoopVec<T,M> */
    int32_t     m;
    /* matrix */
    const void* matrix;         /* device */
    size_t      matrixOffset;   /* bytes */
    int32_t     matrixInterpretation;
    int32_t     layout;         /* CvMatrixLayout */
    int32_t     transpose;
    uint32_t    matrixStride;   /* bytes; ignored for Optimal layouts */
    /* bias (optional) */
    const void* bias;           /* device or NULL (coopVecMatMul) */
    size_t      biasOffset;
    int32_t     biasInterpretation;
    /* extras */
    int32_t     activation;     /* CvActivation */
    float       leakySlope;     /* rounded to half where resultType is FLOAT16 (the example's slope is a vector of the layer's
                                 * element type, fflayer.slang:64) */
    int32_t     accumulate;
    uint32_t    batch;          /* number of samples */
    uint32_t    flags;          /* CV_FLAG_* */
} CvMatMulDesc;

CV_API CvResult cvMatMul(void* stream, const CvMatMulDesc* desc);

/* coopVecOuterProductAccumulate over a batch (hlsl.meta.slang:33227-33316):
 *   Mat[i][j] += sum_s a[s][i] * b[s][j]
 * The per-sample atomics of the reference are replaced by an MFMA contraction over the batch,
 * per-workgroup fp32 partials in `workspace` and one fixed-order reduction, so the result is
 * bitwise reproducible.  That kernel takes FLOAT16 vectors and a FLOAT16 or FLOAT32 matrix in any of the four
 * layouts; FLOAT32 vectors into a FLOAT32 matrix have one of the same kind on the fp32 matrix instruction (each
 * product enters its sum through a fused multiply-add; a batch of one sample gives the bits of the reference).
 * Every other pair of the fallback's types (FLOAT16/32/64 and the 8/16/32/64-bit integers for the
 * vectors and for the matrix, :33261-33315) runs as the scalar definition: the product in the vectors' type,
 * cast to the matrix type, summed over the batch (integers modulo 2^width: bit-exact with the reference;
 * floats in fp32, fp64 for a FLOAT64 matrix, in a fixed order), RowMajor / ColumnMajor (fp32 also the Optimal
 * layouts). */
CV_API CvResult cvOuterProductAccumulateWorkspaceSize(int32_t m, int32_t n, uint32_t batch,
                                                      size_t* outBytes);
CV_API CvResult cvOuterProductAccumulate(void* stream,
                                         const void* a, size_t aStride, int32_t m,
                                         const void* b, size_t bStride, int32_t n,
                                         int32_t elementType, uint32_t batch,
                                         void* matrix, size_t matrixOffset, uint32_t matrixStride,
                                         int32_t layout, int32_t matrixInterpretation,
                                         void* workspace, size_t workspaceBytes);

/* coopVecReduceSumAccumulate over a batch (hlsl.meta.slang:33330-33353):
 *   buffer[i] += sum_s v[s][i]
 * `bufferType` is the vectors' type (the reference's rule); FLOAT16 vectors also go into a FLOAT32 buffer
 * (what "bias gradients into fp32 buffers" needs).  Vectors of FLOAT16/32/64 and of the 8/16/32/64-bit
 * integers (these modulo 2^width, bit-exact with the reference).  Deterministic. */
CV_API CvResult cvReduceSumAccumulateWorkspaceSize(int32_t n, uint32_t batch, size_t* outBytes);
CV_API CvResult cvReduceSumAccumulate(void* stream, const void* v, size_t vStride, int32_t n,
                                      int32_t elementType, uint32_t batch,
                                      void* buffer, size_t offset, int32_t bufferType,
                                      void* workspace, size_t workspaceBytes);

/* ------------------------------------------------------------------------------------ */
/* element-wise surface of CoopVec<T,N>                                                  */
/* ------------------------------------------------------------------------------------ */

/* The per-component operators and math functions Slang declares on CoopVec<T,N>
 * (arithmetic: slang-ir-lower-coopvec.cpp:113-166; min/max/clamp/step hlsl.meta.slang:32043-32229;
 * sin..fma :32231-32421) and the neural module's activations (activations.slang), over a batch:
 *   out[s][i] = op(a[s][i], b[s][i], c[s][i])
 * elementType is FLOAT16 or FLOAT32 (all operands and the result); FLOAT16 evaluates in fp32 and
 * rounds once.  The operators Slang declares on integer vectors -- ADD, SUB, MUL, DIV, NEG, MIN, MAX, CLAMP
 * (hlsl.meta.slang:32115-32229) -- also take SINT8/16/32/64 and UINT8/16/32/64 (two's complement, wrapping; the
 * quotients C leaves undefined are x / 0 = 0 and MIN / -1 = MIN) and FLOAT64, which takes STEP and FMA as well.
 * Operands an operator does not take are ignored (may be NULL).  `param` is the
 * slope of CV_OP_LEAKY_RELU and the scalar of CV_OP_SCALE (converted to the element type first).  FLOAT16 fma is
 * rounded once from the exact a*b + c.  In-place use (out == a) is allowed. */
typedef enum CvElementwiseOp {
    CV_OP_ADD = 0, CV_OP_SUB = 1, CV_OP_MUL = 2, CV_OP_DIV = 3, CV_OP_NEG = 4,
    CV_OP_MIN = 5, CV_OP_MAX = 6, CV_OP_CLAMP = 7 /* clamp(a, b, c) */, CV_OP_STEP = 8 /* step(edge = a, x = b) */,
    CV_OP_SIN = 9, CV_OP_COS = 10, CV_OP_EXP = 11, CV_OP_LOG = 12, CV_OP_LOG2 = 13, CV_OP_EXP2 = 14,
    CV_OP_TANH = 15, CV_OP_ATAN = 16, CV_OP_FMA = 17 /* a*b + c */,
    CV_OP_RELU = 18, CV_OP_LEAKY_RELU = 19 /* a < 0 ? param*a : a */, CV_OP_SIGMOID = 20, CV_OP_SILU = 21,
    CV_OP_QUICK_GELU = 22,
    CV_OP_SCALE = 23 /* a * T(param): vector times scalar, hlsl.meta.slang:32004, :32038 */,
    CV_OP_COUNT = 24
} CvElementwiseOp;

CV_API CvResult cvElementwise(void* stream, int32_t op, int32_t elementType, int32_t n, uint32_t batch,
                              const void* a, size_t aStride, const void* b, size_t bStride,
                              const void* c, size_t cStride, void* out, size_t outStride, float param);

/* CoopVec<T,N>(CoopVec<U,N>) / CoopVec.copyFrom (hlsl.meta.slang:30683-30730) over a batch:
 *   dst[s][i] = T(src[s][i])
 * between any two of FLOAT16/32/64, BFLOAT16 and the 8/16/32/64-bit integers.  Integer -> integer keeps the low bits;
 * to a float type: one rounding to nearest even of the exact source value (also from fp64 and from 64-bit
 * integers to FLOAT16 / BFLOAT16); float -> integer: towards zero (what C leaves undefined is
 * fixed as NaN -> 0 and out-of-range values saturated to 32 bits, 64 for 64-bit targets, then cut to the low bits). */
CV_API CvResult cvVectorCast(void* stream, int32_t n, uint32_t batch, const void* src, size_t srcStride, int32_t srcType,
                             void* dst, size_t dstStride, int32_t dstType);

/* Reverse-mode derivative of the same operators, by Slang's rules (diff.meta.slang:1948-2470: the
 * larger operand of max / smaller of min takes dOut and a tie splits it in halves, clamp passes
 * dOut to x inside [min, max] including the bounds and to the bound it was clamped to otherwise):
 *   dA[s][i] = d op / d a * dOut[s][i], likewise dB, dC (overwritten, not accumulated).
 * Gradient outputs that are NULL, or that the operator has no operand for, are skipped.  FLOAT16 / FLOAT32 only. */
CV_API CvResult cvElementwiseBackward(void* stream, int32_t op, int32_t elementType, int32_t n, uint32_t batch,
                                      const void* a, size_t aStride, const void* b, size_t bStride,
                                      const void* c, size_t cStride, const void* dOut, size_t dOutStride,
                                      void* dA, size_t dAStride, void* dB, size_t dBStride,
                                      void* dC, size_t dCStride, float param);

/* ------------------------------------------------------------------------------------ */
/* input encoders of the neural module                                                  */
/* ------------------------------------------------------------------------------------ */

/* gridHash<Type, Dimensions> (source/standard-modules/neural/hash-function.slang:134-151) of `batch`
 * integer grid positions [batch][dimensions] (uint32): out[s] = hash(positions[s]).  Integer work,
 * bit-exact. */
typedef enum CvHashType {
    CV_HASH_PRIME = 0, CV_HASH_COHERENT_PRIME = 1, CV_HASH_REVERSED_PRIME = 2, CV_HASH_RNG = 3, CV_HASH_BASE_CONVERT = 4
} CvHashType;
CV_API CvResult cvGridHash(void* stream, int32_t hashType, int32_t dimensions, const void* positions,
                           size_t positionStride, uint32_t* out, uint32_t batch);

/* PermutoEncoder (source/standard-modules/neural/permuto-encoder.slang): a multi-level hash encoding
 * on the permutohedral lattice.  CvPermutoLevelInfo mirrors PerLevelInfo (:22-30), CvPermutoDesc the
 * generic arguments <T, Dimensions, FeatureDimensionPerEntry, Log2HashmapSize, MaxLevels> plus
 * HyperParameters (:38-42). */
#define CV_PERMUTO_MAX_DIMS 8
#define CV_PERMUTO_MAX_LEVELS 16
typedef struct CvPermutoLevelInfo {
    uint32_t currentLevelIndex;
    uint32_t offsetOfFeatureTable;   /* in entries */
    uint32_t featureTableSize;       /* hashmap size of this level, in entries */
    float    scale;
    float    scalesPerDim[CV_PERMUTO_MAX_DIMS];
    float    shiftsPerDim[CV_PERMUTO_MAX_DIMS];
} CvPermutoLevelInfo;
typedef struct CvPermutoDesc {
    int32_t  dimensions;                 /* 1..8 */
    int32_t  featureDimensionPerEntry;
    uint32_t log2HashmapSize;
    uint32_t maxLevels;                  /* 1..16 */
    int32_t  elementType;                /* T: FLOAT32 or FLOAT16 -- positions, feature table and output */
    float    maxLevel;                   /* maxLevelRatio * maxLevels; levels >= maxLevel + 1e-3 encode as zeros */
    CvPermutoLevelInfo levelInfo[CV_PERMUTO_MAX_LEVELS];
} CvPermutoDesc;

/* prepareLevelInfo (:339-368) for every level, on the host: fills maxLevel and levelInfo from
 * dimensions, log2HashmapSize and maxLevels (scale = baseScale * 2^(level * log2PerLevelScale),
 * per-dimension scales, PCG32 shifts drawn from `seed`). */
CV_API CvResult cvPermutoPrepareLevels(CvPermutoDesc* desc, float baseScale, float log2PerLevelScale,
                                       float maxLevelRatio, uint32_t seed);
/* encode (:240-337): out[s] = the maxLevels * featureDimensionPerEntry interpolated features of
 * positions[s]; the feature table holds (sum of level sizes) * featureDimensionPerEntry elements. */
CV_API CvResult cvPermutoEncode(void* stream, const CvPermutoDesc* desc, const void* positions, size_t positionStride,
                                const void* featureTable, void* out, size_t outStride, uint32_t batch);
/* bwd_diff of encode for FLOAT32 data: dPositions[s] (overwritten; may be NULL) and dFeatureTable
 * (+=, atomic adds like readFeatureValueBwd :222-238; may be NULL). */
CV_API CvResult cvPermutoEncodeBackward(void* stream, const CvPermutoDesc* desc, const void* positions, size_t positionStride,
                                        const void* featureTable, const void* dOut, size_t dOutStride,
                                        void* dPositions, size_t dPositionStride, void* dFeatureTable, uint32_t batch);

/* ------------------------------------------------------------------------------------ */
/* fused MLP: the example's FeedForwardLayer chain                                       */
/* ------------------------------------------------------------------------------------ */

/* One layer; pointers are arranged like the example's per-layer 4 x u64 block
 * {weights, weightsGrad, biases, biasesGrad} (mlp-training-coopvec.cpp:146-158,
 * fflayer.slang:9-12). */
typedef struct CvMlpLayer {
    const void* weights;        /* device */
    void*       weightsGrad;    /* device or NULL (forward only) */
    const void* biases;         /* device or NULL */
    void*       biasesGrad;     /* device or NULL */
    int32_t     inputSize;
    int32_t     outputSize;
    int32_t     weightLayout;   /* layout of `weights` */
    uint32_t    weightStride;   /* bytes, Row/ColumnMajor only */
    int32_t     gradLayout;     /* layout of `weightsGrad` */
    uint32_t    gradStride;
    int32_t     activation;     /* CvActivation applied to this layer's output */
    float       leakySlope;     /* taken in the vectors' type: rounded to half for a network of half vectors, as the example
                                 * builds it (fflayer.slang:64, CoopVec<NFloat, OutputSize>(0.001h)) */
} CvMlpLayer;

/* Encoding applied to a sample in front of layer 0.
 * CV_ENCODE_XY_SQUARES is the example's MyNetwork::encodeInput (network.slang:35-38): a sample is a
 * float2 (x, y) in memory (`uniform float2* inputs`, kernels.slang:12); it is converted to half2
 * (kernels.slang:19) and layer 0 sees the CoopVec<half,4> (x, y, x*x, y*y), the squares rounded to half.
 * Needs inputType FLOAT32, FLOAT16 weights and a first layer of 4 inputs.  With this encoding and
 * targets == NULL, cvMlpTrainStep differentiates the example's own loss (network.slang:58-75): the
 * squared distance of the 4 outputs from groundtruth(x, y), evaluated in half. */
typedef enum CvInputEncoding { CV_ENCODE_NONE = 0, CV_ENCODE_XY_SQUARES = 1 } CvInputEncoding;

typedef struct CvMlpDesc {
    const CvMlpLayer* layers;   /* host array */
    int32_t  numLayers;
    int32_t  inputType;         /* element type of the input vectors in memory */
    int32_t  weightType;        /* matrix interpretation of every layer: FLOAT16 or FLOAT_E4M3; FLOAT32 or BFLOAT16 for
                                   a network of that one type (vectors, biases, results and targets too; BFLOAT16 forward
                                   only, FLOAT32 also trains: layer by layer, FLOAT32 gradients) */
    int32_t  biasType;          /* FLOAT16 (weightType for FLOAT32 / BFLOAT16 networks) */
    int32_t  outputType;        /* FLOAT16 (weightType for FLOAT32 / BFLOAT16 networks) */
    int32_t  gradType;          /* FLOAT16 or FLOAT32: element type of weightsGrad/biasesGrad */
    uint32_t flags;             /* CV_FLAG_* */
    int32_t  inputEncoding;     /* CvInputEncoding */
    float*   lossMax;           /* device, optional (NULL: not wanted): cvMlpTrainStep overwrites it with max_s loss_s, the
                                   figure the example's learnGradient leaves in its loss buffer (WaveActiveMax + atomic max
                                   over a cleared buffer, kernels.slang:21-26) */
} CvMlpDesc;

/* y = layer_{n-1}( ... layer_0(x) ): every layer is coopVecMatMulAdd + activation with
 * CoopVec<half> as the carrier between layers; with weightType FLOAT_E4M3 the carrier is
 * re-quantised to OCP e4m3 (saturating) in front of every layer; with weightType FLOAT32 / BFLOAT16 the
 * carrier is CoopVec<float> / bfloat16 (the FFLayer<float, ...> chain of the neural module).  Activations stay in
 * registers between layers. */
CV_API CvResult cvMlpForward(void* stream, const CvMlpDesc* mlp,
                             const void* input, size_t inputStride,
                             void* output, size_t outputStride, uint32_t batch);

/* encode + network in one kernel.  A Slang thread hands the result of PermutoEncoder::encode
 * (source/standard-modules/neural/permuto-encoder.slang:319-337) straight to the first layer of its
 * network (layers.slang:34-110; network.slang:41-47), so the encoded vector never exists in memory;
 * this is that composition for a batch: output[s] = mlp(encode(positions[s])), bit for bit what
 * cvPermutoEncode followed by cvMlpForward returns.  FLOAT16 encoders (1..4 dimensions, 1, 2 or 4
 * features per entry, level records in level order) in front of FLOAT16 networks of at least two
 * layers whose first layer takes maxLevels * featureDimensionPerEntry inputs, every dimension <= 128;
 * CV_E_NOT_AVAILABLE otherwise (call the two entry points instead).  The feature table must be aligned
 * to one entry. */
CV_API CvResult cvPermutoMlpForward(void* stream, const CvPermutoDesc* desc, const void* positions, size_t positionStride,
                                    const void* featureTable, const CvMlpDesc* mlp, void* output, size_t outputStride,
                                    uint32_t batch);

/* Forward + reverse pass of loss_s = sum_i (y[s][i] - target[s][i])^2 with seed `lossScale`
 * (the example: bwd_diff(loss)(network, x, y, 1.0h), kernels.slang:20): accumulates
 * sum_s dY (x) X into every layer's weightsGrad and sum_s dY into biasesGrad ("+=").
 * targets == NULL selects target = sin(sum of the sample's inputs) for every output (with
 * inputEncoding CV_ENCODE_XY_SQUARES: the example's groundtruth(x, y)).
 * lossSum (device, optional, one float) is overwritten with sum_s loss_s; mlp->lossMax, if set, with max_s loss_s.
 * The fused kernel for 64-wide networks runs pairs of waves that wait for each other with a bounded spin; should such a
 * wait ever time out (only a defect of the kernel could cause that), the step is void: lossSum, lossMax and every
 * gradient sum the step adds are NaN, whether or not the loss outputs are requested.  A NaN loss for any other reason
 * (NaN samples) has the same effect. */
CV_API CvResult cvMlpTrainStepWorkspaceSize(const CvMlpDesc* mlp, uint32_t batch, size_t* outBytes);
CV_API CvResult cvMlpTrainStep(void* stream, const CvMlpDesc* mlp,
                               const void* input, size_t inputStride,
                               const void* targets, size_t targetStride,
                               float lossScale, uint32_t batch, float* lossSum,
                               void* workspace, size_t workspaceBytes);

/* cvMlpTrainStep for callers that cannot allocate device memory or carry a workspace around:
 * code under HIP graph capture, tight training loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference.  Same arguments, kernels and results (bit for bit) as
 * cvMlpTrainStep, but the per-workgroup gradient partials go to an array of
 * CV_NOALLOC_SCRATCH_BYTES that is part of the library's device image (every GPU the library
 * runs on holds one copy until the process ends).  Networks whose partials do not fit get
 * CV_E_NOT_AVAILABLE.  The call allocates and frees nothing; the first call on a device looks up
 * the array's address (make that call outside a graph capture).  All calls on one GPU share the
 * array: calls that may overlap on one GPU (different streams, different threads) race. */
#define CV_NOALLOC_SCRATCH_BYTES ((size_t)16 << 20)
CV_API CvResult cvMlpTrainStepNoAlloc(void* stream, const CvMlpDesc* mlp,
                                      const void* input, size_t inputStride,
                                      const void* targets, size_t targetStride,
                                      float lossScale, uint32_t batch, float* lossSum);

/* ------------------------------------------------------------------------------------ */
/* the neural module's network parameter block                                          */
/* ------------------------------------------------------------------------------------ */

/* NetworkParameterLayoutConverter<T, BiasMask, D0, D1, ...>
 * (source/standard-modules/neural/network-parameter-layout-converter.slang:469-555) and the FFLayer
 * chain over such a block (layers.slang:34-110).  dims[0..layerCount] are D0..Dn; bit l of biasMask
 * says whether layer l (D_l -> D_{l+1}) has a bias.
 *   portable layout: per layer row-major weight[Out][In], then bias[Out] if the layer has one;
 *   optimal layout : per layer weight envelope [align16(Out)][align16(In)], then a bias slot of
 *                    align16(Out) elements (reserved for every layer), padding zero.
 * `order` is the order of the weights inside an envelope: NATIVE is this library's (accumulator-native
 * 16x16 tiles, i.e. CV_LAYOUT_TRAINING_OPTIMAL per layer: what the fused kernels read and write); the
 * other three are the reference's SPIR-V, Metal and CUDA orders (:137-172), so that blocks can be
 * exchanged with those targets. */
#define CV_NEURAL_MAX_LAYERS 64
typedef enum CvNeuralWeightOrder {
    CV_NEURAL_ORDER_NATIVE = 0, CV_NEURAL_ORDER_TILED_ROW_MAJOR = 1, CV_NEURAL_ORDER_PADDED_ROW_MAJOR = 2,
    CV_NEURAL_ORDER_CUDA_MATRIX_B = 3
} CvNeuralWeightOrder;
typedef struct CvNeuralNetworkDesc {
    int32_t  layerCount;
    int32_t  dims[CV_NEURAL_MAX_LAYERS + 1];
    uint64_t biasMask;
    int32_t  elementType;     /* T: FLOAT32 or FLOAT16 */
    int32_t  order;           /* CvNeuralWeightOrder */
} CvNeuralNetworkDesc;

/* ElementCountLogical / ElementCountPhysical (:477-480). */
CV_API CvResult cvNeuralNetworkSize(const CvNeuralNetworkDesc* net, size_t* elementCountLogical, size_t* elementCountPhysical);
/* toOptimalLayout (:487-516) / toPortableLayout (:524-553) of the whole block in one launch. */
CV_API CvResult cvNeuralToOptimalLayout(void* stream, const CvNeuralNetworkDesc* net, const void* portable, void* optimal);
CV_API CvResult cvNeuralToPortableLayout(void* stream, const CvNeuralNetworkDesc* net, const void* optimal, void* portable);
/* The FFLayer chain y = Activation_l(W_l x + b_l) (layers.slang:90-110) over a FLOAT16 or FLOAT32 parameter block
 * (vectors and results have the block's element type),
 * in the portable (LinearLayout; optimalLayout = 0) or the optimal layout in NATIVE order
 * (optimalLayout = 1); layer l's bias sits WeightStorageSize elements behind its weights (:93-96).
 * activations / leakySlopes: one CvActivation / slope per layer (NULL: none).  Served by cvMlpForward. */
CV_API CvResult cvNeuralMlpForward(void* stream, const CvNeuralNetworkDesc* net, int32_t optimalLayout, const void* params,
                                   const int32_t* activations, const float* leakySlopes,
                                   const void* input, size_t inputStride, void* output, size_t outputStride, uint32_t batch);
/* bwd_diff through the chain with a gradient block laid out like the parameter block (the
 * DifferentialPtrPair of layers.slang:21-25): gradients are accumulated in the block's element type (FLOAT16 or
 * FLOAT32) at the same element offsets.  Served by cvMlpTrainStep (same loss, targets, workspace rules). */
CV_API CvResult cvNeuralMlpTrainStepWorkspaceSize(const CvNeuralNetworkDesc* net, uint32_t batch, size_t* outBytes);
CV_API CvResult cvNeuralMlpTrainStep(void* stream, const CvNeuralNetworkDesc* net, int32_t optimalLayout, const void* params,
                                     void* paramGrads, const int32_t* activations, const float* leakySlopes,
                                     const void* input, size_t inputStride, const void* targets, size_t targetStride,
                                     float lossScale, uint32_t batch, float* lossSum, void* workspace, size_t workspaceBytes);

/* ------------------------------------------------------------------------------------ */
/* parameter update of the example                                                      */
/* ------------------------------------------------------------------------------------ */

/* Replaces the adjustParameters dispatch (examples/mlp-training-coopvec/kernels.slang:29-45,
 * AdamOptimizer::step adam.slang:20-36, host side mlp-training-coopvec.cpp:238-250) over `count`
 * fp16 parameters: `states` are AdamState records {half mean; half variance; int iteration}
 * (8 bytes each), `gradients` fp16 (zeroed by the call; NaN gradients are cleared and skipped,
 * infinite ones taken as +-10000).  All arithmetic in half, as the Slang source spells it.
 * The example's constants: beta1 0.9, beta2 0.999, epsilon 1e-7, learningRate 0.01. */
CV_API CvResult cvAdamStep(void* stream, void* states, void* params, void* gradients, uint32_t count,
                           float beta1, float beta2, float epsilon, float learningRate);

/* The same update for every parameter of a network in one launch, read straight from the gradient buffers
 * cvMlpTrainStep fills: it replaces convertCooperativeVectorMatrix (TrainingOptimal -> RowMajor,
 * mlp-training-coopvec.cpp:203-236) + adjustParameters (:238-250) of the example's iteration, and the clear of the
 * gradient segment at the top of the next one (:183-188), since every gradient element it reads is left at zero.
 * Layer l: `weights` (FLOAT16, any layout, updated in place), `weightsGrad` (gradType FLOAT16 or FLOAT32, any layout; an
 * FLOAT32 sum is rounded to half first), `biases` / `biasesGrad` (or both NULL).  weightStates[l] holds one AdamState per
 * weight in row-major order [outputSize][inputSize], biasStates[l] one per bias.  Results equal
 * cvConvertMatrices + cvAdamStep bit for bit. */
CV_API CvResult cvMlpAdamStep(void* stream, const CvMlpDesc* mlp, void* const* weightStates, void* const* biasStates,
                              float beta1, float beta2, float epsilon, float learningRate);

#ifdef __cplusplus
}
#endif
#endif /* COOPVEC_H */
