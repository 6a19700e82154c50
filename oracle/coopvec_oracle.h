/*
 * coopvec_oracle.h -- CPU oracle for the cooperative-vector operators.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library or its Python host
 * layer links, loads or calls this code; it is used by tests/, by the smoke
 * check and by the benchmark's cpu_baseline leg as the checker / reported
 * baseline.
 *
 * Two families of functions live here:
 *
 *  (1) cvo_slang_*  : a literal restatement of what Slang's CPU target executes
 *      for the operators, i.e. the `default:` arms of `__target_switch` in
 *      source/slang/hlsl.meta.slang (matmul :32835-32912, bias :33043-33103,
 *      outer product :33261-33315, reduce-sum :33344-33352) on top of the
 *      prelude's `half` (prelude/slang-cpp-scalar-intrinsics.h:563-741).
 *      Pinned by the reference's own golden vectors (tests/cooperative-vector).
 *
 *  (2) cvo_ref_*    : the parity reference the north star defines: products
 *      accumulated sequentially in fp32 (or exactly in int32), one rounding to
 *      the result type at the end.  Pinned by the same goldens, by fp64 brute
 *      force and by closed forms.
 *
 *  (3) cvo_layout_* : the byte layouts of this library's InferencingOptimal /
 *      TrainingOptimal matrices.  The reference leaves those layouts opaque
 *      (vendor driver), so they are pinned only by invariants (round trip,
 *      zero padding, size rules): "parity unpinned" against any vendor layout.
 */
#ifndef COOPVEC_ORACLE_H
#define COOPVEC_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* CoopVecComponentType, numeric values as declared in hlsl.meta.slang:32558-32575 */
enum {
    CVO_FLOAT_E4M3 = 0, CVO_FLOAT_E5M2 = 1, CVO_FLOAT16 = 2, CVO_FLOAT32 = 3, CVO_FLOAT64 = 4,
    CVO_SINT8 = 5, CVO_SINT16 = 6, CVO_SINT32 = 7, CVO_SINT64 = 8, CVO_SINT8_PACKED = 9,
    CVO_UINT8 = 10, CVO_UINT16 = 11, CVO_UINT32 = 12, CVO_UINT64 = 13, CVO_UINT8_PACKED = 14,
    /* not in the reference's enum: bfloat16 operands of the matrix cores, the library's extension */
    CVO_BFLOAT16 = 15
};
/* CoopVecMatrixLayout, hlsl.meta.slang:32547-32553 == include/slang.h:948-955 */
enum { CVO_ROW_MAJOR = 0, CVO_COLUMN_MAJOR = 1, CVO_INFERENCING_OPTIMAL = 2, CVO_TRAINING_OPTIMAL = 3 };
/* how `half` arithmetic rounds: IEEE round-to-nearest-even (`_Float16`), or the prelude's
 * software struct (ties away from zero, prelude/slang-cpp-scalar-intrinsics.h:604-612) */
enum { CVO_HALF_RNE = 0, CVO_HALF_SLANG_SOFT = 1 };
/* activations understood by the fused-MLP reference */
enum { CVO_ACT_NONE = 0, CVO_ACT_RELU = 1, CVO_ACT_LEAKY_RELU = 2 };

/* ---- numerics ---------------------------------------------------------------------- */
uint16_t cvo_f32_to_f16_rne(float f);
uint16_t cvo_f32_to_f16_slang(float f);
float    cvo_f16_to_f32(uint16_t h);
uint8_t  cvo_f32_to_e4m3_sat(float f);
float    cvo_e4m3_to_f32(uint8_t b);

/* ---- type tables (hlsl.meta.slang:32577-32670) ------------------------------------- */
int cvo_component_packing_factor(int ct);
int cvo_component_scalar_type(int ct);   /* SLANG_SCALAR_TYPE_* value, -1 if none */
int cvo_component_type_stride(int ct);   /* bytes; -1 where the fallback has no case */

/* ---- Slang CPU-target semantics ------------------------------------------------------ */
/* One thread's coopVecMatMul[Add]Packed.  `inputType`/`resultType` are the CoopVec element
 * types U and T given as component types.  biasInterp < 0 means "no bias" (coopVecMatMul).
 * accumulate != 0 gives the member forms matMulAccum/matMulAddAccum (result += ...).
 * Returns 0, or -1 for a combination the fallback cannot compile. */
int cvo_slang_matmul(const void* input, int inputType, int packedK, int inputInterp, int k,
                     void* result, int resultType, int M,
                     const void* matrix, int32_t matrixOffset, int matrixInterp,
                     int layout, int transpose, uint32_t matrixStride,
                     const void* bias, int32_t biasOffset, int biasInterp,
                     int accumulate, int halfMode);

int cvo_slang_outer_product_accumulate(const void* a, int M, const void* b, int N, int elemType,
                                       void* matrix, int32_t matrixOffset, uint32_t matrixStride,
                                       int layout, int matrixInterp, int halfMode);

int cvo_slang_reduce_sum_accumulate(const void* v, int N, int elemType,
                                    void* buffer, int32_t offset, int halfMode);

/* A whole dispatch of `[numthreads(256,1,1)]` threads over groups [startGroup,endGroup),
 * one sample per thread, shaped like the wrapper slangc emits for the CPU target
 * (source/slang/slang-emit-cpp.cpp:2255-2280).  Loads the K-vector of thread `tid` at
 * byte offset tid*inputStride, stores the M-vector at tid*outputStride. */
int cvo_slang_dispatch_matmul_add(uint32_t startGroup, uint32_t endGroup, uint32_t count,
                                  const void* input, size_t inputStride, int inputType,
                                  int packedK, int inputInterp, int k,
                                  void* output, size_t outputStride, int resultType, int M,
                                  const void* matrix, int32_t matrixOffset, int matrixInterp,
                                  int layout, int transpose, uint32_t matrixStride,
                                  const void* bias, int32_t biasOffset, int biasInterp,
                                  int halfMode);

/* ---- parity reference -------------------------------------------------------------- */
/* Batched layer:  y[b][i] = cast<T>( sum_j W[i][j]*x[b][j]  (+ bias[i]) ).
 * Float paths: operands decoded to fp32, products and running sum in fp32, j ascending, bias
 * added last in fp32; `out_f32` receives the unrounded fp32 value, `out_abs` (optional) the
 * sum of |terms| (+|bias|) used by tests as a cancellation floor.  Integer path: exact int32.
 * W is read through cvo_layout_elem_offset, so every layout is accepted. */
int cvo_ref_matmul_f32(const void* x, size_t xStride, int xType, int k,
                       const void* matrix, size_t matrixOffset, int matrixInterp,
                       int layout, int transpose, uint32_t matrixStride, int M,
                       const void* bias, size_t biasOffset, int biasInterp,
                       uint32_t batch, float* out_f32, float* out_abs);
int cvo_ref_matmul_i32(const void* x, size_t xStride, int xType, int k,
                       const void* matrix, size_t matrixOffset, int matrixInterp,
                       int layout, int transpose, uint32_t matrixStride, int M,
                       const void* bias, size_t biasOffset, int biasInterp,
                       uint32_t batch, int32_t* out);

/* One layer description for the fused-MLP reference.  Weights are row-major
 * [outDim][inDim] elements of `weightType` (FLOAT16 or FLOAT_E4M3) with stride in bytes. */
typedef struct CvoLayer {
    int inDim, outDim;
    int weightType;
    const void* weights; uint32_t weightStride;
    const void* bias;      /* fp16 [outDim] or NULL */
    int activation;        /* CVO_ACT_* */
    float leakySlope;      /* fp16-representable */
} CvoLayer;

/* Forward pass with the carrier type CoopVec<half>: every layer output is rounded to fp16
 * (RNE) before the activation; for weightType FLOAT_E4M3 the layer's input is quantised to
 * OCP e4m3 (saturating) before the products.  `inputType` is FLOAT16 or FLOAT_E4M3 (bytes).
 * out: fp16 [batch][lastOutDim].  If `acts` is not NULL it receives every layer's fp16
 * output (after activation) back to back per layer: layer l block is [batch][outDim_l]. */
int cvo_ref_mlp_forward(const CvoLayer* layers, int numLayers,
                        const void* input, size_t inputStride, int inputType,
                        uint32_t batch, uint16_t* out, uint16_t* acts);

/* Training step for an fp16 MLP, per-sample loss sum_i (y_i - t_i)^2 with seed
 * dLoss = lossScale (the example calls bwd_diff(loss)(..., 1.0h)).  All carrier values
 * (activations, dY, dX) are rounded to fp16 as CoopVec<half> does; weight and bias gradients
 * are summed over the batch in fp64 and returned as doubles, row-major [outDim][inDim] per
 * layer then [outDim], so that any accumulation order on the GPU can be compared to them.
 * targets: fp16 [batch][lastOutDim], or NULL for target = fp16(sinf(sum of the fp16 inputs))
 * broadcast to every output.  maxTieRule != 0 applies Slang's derivative of max at a tie
 * (0.5 each, source/slang/diff.meta.slang:2258-2277). */
int cvo_ref_mlp_train(const CvoLayer* layers, int numLayers,
                      const uint16_t* input, size_t inputStride,
                      const uint16_t* targets, float lossScale, uint32_t batch,
                      double** dW, double** dB, double* lossSum, int maxTieRule);

/* ---- matrix layouts ---------------------------------------------------------------- */
/* Bytes needed for rows x cols of component type ct in `layout`; stride (bytes between rows
 * for RowMajor / between columns for ColumnMajor, 0 = tightly packed) is ignored for the
 * Optimal layouts.  0 on an invalid argument. */
size_t  cvo_layout_matrix_size(uint32_t rows, uint32_t cols, int ct, int layout, size_t stride);
/* Byte offset of element (r,c) from the start of the matrix, -1 if invalid. */
int64_t cvo_layout_elem_offset(uint32_t rows, uint32_t cols, int ct, int layout, size_t stride,
                               uint32_t r, uint32_t c);
/* Copy/convert one matrix.  Padding of Optimal destinations is zero-filled.  Component types
 * may differ between FLOAT16 and FLOAT32 (RNE); otherwise they must match. */
int cvo_layout_convert(void* dst, uint32_t rows, uint32_t cols, int dstCt, int dstLayout,
                       size_t dstStride, const void* src, int srcCt, int srcLayout,
                       size_t srcStride);

/* ---- Adam parameter update (examples/mlp-training-coopvec) ----------------------------- */
/* AdamState of adam.slang:5-10: { half mean; half variance; int iteration } = 8 bytes. */
typedef struct CvoAdamState { uint16_t mean, variance; int32_t iteration; } CvoAdamState;
/* One dispatch of adjustParameters (kernels.slang:29-45) + AdamOptimizer::step (adam.slang:20-36)
 * over `count` fp16 parameters: every operation in half (each result rounded), NaN gradients are
 * cleared and skipped, infinite ones replaced by +-10000, the gradient is zeroed afterwards.
 * The reference has no golden for the optimizer; pinned by what the mathematics of Adam fixes
 * over several steps (tests/test_adam.py): a constant gradient g gives bias-corrected moments g and
 * g^2, so every step moves the parameter by lr*sign(g); one gradient followed by zeros gives the
 * closed-form decay beta1^(n-1)(1-beta1)/(1-beta1^n) over sqrt of the same in beta2; the iteration
 * counter; NaN skips, infinities clip. */
void cvo_slang_adam_step(CvoAdamState* states, uint16_t* params, uint16_t* grads, uint32_t count,
                         float beta1, float beta2, float epsilon, float learningRate, int halfMode);
/* Same, with the fp32 values of pow(beta1, it) and pow(beta2, it) moved by powNudge1 / powNudge2
 * ulps before they are rounded to half (pow is the one operation maths libraries may round
 * differently). */
void cvo_slang_adam_step_nudged(CvoAdamState* states, uint16_t* params, uint16_t* grads, uint32_t count,
                                float beta1, float beta2, float epsilon, float learningRate, int halfMode,
                                int powNudge1, int powNudge2);

/* ---- element-wise surface ------------------------------------------------------------- */
/* Operator numbers of the C-ABI's CvElementwiseOp. */
enum {
    CVO_OP_ADD = 0, CVO_OP_SUB, CVO_OP_MUL, CVO_OP_DIV, CVO_OP_NEG, CVO_OP_MIN, CVO_OP_MAX, CVO_OP_CLAMP, CVO_OP_STEP,
    CVO_OP_SIN, CVO_OP_COS, CVO_OP_EXP, CVO_OP_LOG, CVO_OP_LOG2, CVO_OP_EXP2, CVO_OP_TANH, CVO_OP_ATAN, CVO_OP_FMA,
    CVO_OP_RELU, CVO_OP_LEAKY_RELU, CVO_OP_SIGMOID, CVO_OP_SILU, CVO_OP_QUICK_GELU, CVO_OP_SCALE, CVO_OP_COUNT
};
/* out[i] = op(a[i], b[i], c[i]) over `count` elements of type ct (FLOAT16 or FLOAT32), evaluated in
 * double and rounded once: the per-component functions of CoopVec<T,N> (hlsl.meta.slang:32043-32421)
 * and the neural module's activations (activations.slang).  Pinned by the primal CHECK values of
 * tests/autodiff/coopvec.slang (tests/test_oracle_elementwise.py). */
int cvo_elementwise(int op, int ct, size_t count, const void* a, const void* b, const void* c, void* out, float param);
/* dA/dB/dC[i] = d op / d operand * dOut[i], by the rules of diff.meta.slang:1948-2470 (ties of min/max
 * split dOut in halves; clamp passes dOut to x on the closed interval).  Pinned by the gradient CHECK
 * values of tests/autodiff/coopvec.slang and by central differences. */
int cvo_elementwise_backward(int op, int ct, size_t count, const void* a, const void* b, const void* c,
                             const void* dOut, void* dA, void* dB, void* dC, float param);

/* ---- grid hashes and the permutohedral encoder of the neural module --------------------- */
/* gridHash<Type, Dimensions> (hash-function.slang:134-151): type 0 Prime, 1 CoherentPrime,
 * 2 ReversedPrime, 3 Rng (PCG32, seed 1337), 4 BaseConvert.  Pinned by all 22 values of
 * tests/neural/hash-function-test.slang. */
uint32_t cvo_grid_hash(int type, int dims, const uint32_t* pos);

#define CVO_PERMUTO_MAX_DIMS 8
/* PermutoEncoder::PerLevelInfo (permuto-encoder.slang:22-30) */
typedef struct CvoPermutoLevel {
    uint32_t currentLevelIndex, offsetOfFeatureTable, featureTableSize;
    float scale;
    float scalesPerDim[CVO_PERMUTO_MAX_DIMS], shiftsPerDim[CVO_PERMUTO_MAX_DIMS];
} CvoPermutoLevel;
/* prepareLevelInfo (:339-368).  Pinned by tests/neural/permuto-encoder-precomputed-constants.slang. */
void cvo_permuto_prepare_level(uint32_t level, int dims, uint32_t log2HashmapSize, float baseScale,
                               float log2PerLevelScale, uint32_t seed, CvoPermutoLevel* out);
/* encode (:240-337) of `count` positions [count][D] of type ct (FLOAT32/FLOAT16, also the type of the
 * feature table and of out [count][numLevels*F]).  Pinned by the 128 forward values of
 * tests/neural/permuto-reference-data.slang (to that test's own epsilon 0.1). */
int cvo_permuto_encode(int D, int F, int numLevels, float maxLevel, const CvoPermutoLevel* levels, int ct,
                       const void* positions, size_t count, const void* table, void* out);
/* reverse mode for fp32 data, evaluated in double: dPositions [count][D] overwritten, dTable accumulated.
 * Pinned by EXPECTED_DL_DPOS / EXPECTED_DL_DPARAMS of the same file. */
int cvo_permuto_encode_backward(int D, int F, int numLevels, float maxLevel, const CvoPermutoLevel* levels,
                                const float* positions, size_t count, const float* table, const float* dOut,
                                double* dPositions, double* dTable);

#ifdef __cplusplus
}
#endif
#endif
