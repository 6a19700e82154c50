// cv_train_general.hip -- the training step for networks outside the fused kernel's tile shapes.
//
// The same computation as the fused step (the example's learnGradient, kernels.slang:9-27:
// forward, bwd_diff of the squared-error loss, fflayer.slang:29-58), layer by layer over the
// whole batch, with the per-layer vectors parked in the caller's workspace instead of registers:
//
//   forward   Z_l = W_l X_l + b_l   (batched matMulAdd kernel, fp16 result)
//             X_{l+1} = act(Z_l)    (element-wise, half arithmetic)
//   loss      diff = half(y - t), lossSum += diff^2, g = half(2 diff lossScale)
//   backward  dZ_l = g * act'(Z_l)  (Slang's max rule: whole gradient to the larger operand, half
//                                    to each at a tie, diff.meta.slang:2258-2277)
//             db_l += sum_s dZ_l    (batched reduce-sum accumulate kernel)
//             dW_l += sum_s dZ_l (x) X_l   (batched outer-product accumulate kernel)
//             g = half(W_l^T dZ_l)  (batched matMul kernel on the transposed matrix)
//
// Every rounding point is the fused kernel's (and the oracle's); all reductions run in a fixed
// order, so the result is bitwise reproducible.  Any layer sizes the matMul kernels serve.
//
// Networks of T = float (the neural module's FFLayer<float, ...>) run the same steps with every "half" above
// read as float: fp32 matMul kernels, element-wise steps in float, gradients summed by the scalar accumulate
// kernels into fp32 destinations.
#include <cstring>

#include "cv_device.h"
#include "cv_kernels.h"
#include "cv_error.h"

namespace cv {

namespace {

constexpr size_t kAlign = 256;
size_t alignUp(size_t v) { return (v + kAlign - 1) / kAlign * kAlign; }

// Where each per-layer array lives in the workspace (byte offsets).
struct GeneralPlan {
    size_t x0;                        // encoded network input (only with an input encoding)
    size_t z[kMaxMlpLayers];          // pre-activations, fp16 [batch][out_l]
    size_t act[kMaxMlpLayers];        // activations (== z[l] where the layer has no activation)
    size_t gA, gB;                    // gradient ping-pong buffers, fp16 [batch][widest layer]
    size_t lossPartials;              // one float per workgroup of the loss kernel
    size_t partials;                  // scratch of the accumulate kernels
    size_t total;
    uint32_t lossBlocks;
};

constexpr uint32_t kLossSamplesPerBlock = 1024;

GeneralPlan makePlan(const MlpArgs& a, int numCUs, int carrierCt)
{
    const size_t esz = elemSize(carrierCt);
    GeneralPlan p{};
    const int L = a.numLayers;
    const size_t batch = a.batch ? a.batch : 1;
    size_t off = 0;
    int widest = a.layers[0].in;
    p.x0 = off;
    if (a.inEncoding != kEncodeNone) off += alignUp(batch * 4 * 2);      // (fp16 networks only)
    for (int l = 0; l < L; ++l) {
        const size_t bytes = alignUp(batch * (size_t)a.layers[l].out * esz);
        p.z[l] = off; off += bytes;
        // (room for the activations is reserved whether or not the layer has one: the size then depends on the
        // layer sizes and the batch alone, which is all a size query knows)
        p.act[l] = a.layers[l].act == kActNone ? p.z[l] : off;
        off += bytes;
        if (a.layers[l].out > widest) widest = a.layers[l].out;
    }
    const size_t gBytes = alignUp(batch * (size_t)widest * esz);
    p.gA = off; off += gBytes;
    p.gB = off; off += gBytes;
    p.lossBlocks = (uint32_t)((batch + kLossSamplesPerBlock - 1) / kLossSamplesPerBlock);
    p.lossPartials = off; off += alignUp((size_t)p.lossBlocks * 2 * sizeof(float));      // sums, then maxima
    size_t part = reduceSumWorkspaceBytes((uint32_t)batch, numCUs);
    for (int l = 0; l < L; ++l) {
        const size_t o = outerWorkspaceBytes(a.layers[l].out, a.layers[l].in, (uint32_t)batch, numCUs);
        if (o > part) part = o;
        if (carrierCt != kF16) {
            const size_t sc = accumScalarWorkspaceBytes(a.layers[l].out, a.layers[l].in, (uint32_t)batch);
            if (sc > part) part = sc;
            const size_t mp = outerF32WorkspaceBytes(a.layers[l].out, a.layers[l].in, (uint32_t)batch, numCUs);
            if (mp > part) part = mp;
        }
    }
    p.partials = off; off += alignUp(part);
    p.total = off;
    return p;
}

// ---- element-wise kernels ---------------------------------------------------------------------

// float2 samples -> the example's encoded input (x, y, x*x, y*y) in half
__global__ __launch_bounds__(256) void encodeXYKernel(const uint8_t* in, uint64_t inStride, uint32_t batch, uint32_t* x0)
{
    const uint32_t s = blockIdx.x * 256u + threadIdx.x;
    if (s >= batch) return;
    uint32_t xy, sq;
    encodeXYSquares(in + (size_t)s * inStride, xy, sq);
    x0[2 * s] = xy; x0[2 * s + 1] = sq;
}

// activation and its derivative rule in the carrier type T
template <typename T> __device__ __forceinline__ T activateT(T z, int act, float slope);
template <> __device__ __forceinline__ half_t activateT<half_t>(half_t z, int act, float slope) { return activateHalf(z, act, slope); }
template <> __device__ __forceinline__ float activateT<float>(float z, int act, float slope)
{
    if (act == kActRelu) return z > 0.f ? z : 0.f;
    if (act == kActLeakyRelu) return fmaxf(z, z * slope);      // as the fp32 matMul kernels apply it
    return z;
}

// dz = g * act'(z), every product and sum rounded to T
template <typename T>
__device__ __forceinline__ T activationGrad(T g, T z, int act, float slope)
{
    const T halfG = (T)(0.5f * (float)g);
    if (act == kActRelu) return z > (T)0 ? g : (z == (T)0 ? halfG : (T)0);
    if (act == kActLeakyRelu) {
        const T zs = (T)((float)z * slope);
        T da, db;
        if (z > zs) { da = g; db = (T)0; }
        else if (z < zs) { da = (T)0; db = g; }
        else { da = halfG; db = halfG; }
        const T dbs = (T)((float)db * slope);
        return (T)((float)da + (float)dbs);
    }
    return g;
}

// 16 bytes per thread and step where the arrays allow it, the rest one by one
template <typename T>
__global__ __launch_bounds__(256) void activationKernel(const T* z, T* out, size_t count, int act, float slope)
{
    constexpr int PER = 16 / sizeof(T);
    typedef T Vec __attribute__((ext_vector_type(PER)));
    const size_t tid = (size_t)blockIdx.x * 256u + threadIdx.x, nthreads = (size_t)gridDim.x * 256u;
    const size_t chunks = count / PER;
    for (size_t c = tid; c < chunks; c += nthreads) {
        const Vec v = ((const Vec*)z)[c];
        Vec r;
#pragma unroll
        for (int i = 0; i < PER; ++i) r[i] = activateT<T>(v[i], act, slope);
        ((Vec*)out)[c] = r;
    }
    for (size_t i = chunks * PER + tid; i < count; i += nthreads) out[i] = activateT<T>(z[i], act, slope);
}

template <typename T>
__global__ __launch_bounds__(256) void activationGradKernel(const T* g, const T* z, T* dz, size_t count, int act, float slope)
{
    constexpr int PER = 16 / sizeof(T);
    typedef T Vec __attribute__((ext_vector_type(PER)));
    const size_t tid = (size_t)blockIdx.x * 256u + threadIdx.x, nthreads = (size_t)gridDim.x * 256u;
    const size_t chunks = count / PER;
    for (size_t c = tid; c < chunks; c += nthreads) {
        const Vec gv = ((const Vec*)g)[c], zv = ((const Vec*)z)[c];
        Vec r;
#pragma unroll
        for (int i = 0; i < PER; ++i) r[i] = activationGrad<T>(gv[i], zv[i], act, slope);
        ((Vec*)dz)[c] = r;
    }
    for (size_t i = chunks * PER + tid; i < count; i += nthreads) dz[i] = activationGrad<T>(g[i], z[i], act, slope);
}

struct LossArgs {
    const void* y;              // network output, [batch][outDim] of the carrier type
    const void* z;              // last layer's pre-activation
    void* dz;                   // gradient at the last layer's pre-activation
    const uint8_t* targets; uint64_t targetStride;
    const uint8_t* in; uint64_t inStride;   // network input as the caller passed it
    int32_t inDim, outDim, inEncoding;
    int32_t act; float slope;
    float lossScale;
    uint32_t batch;
    float* partials;            // per workgroup: the sum of its samples' losses, and behind all sums the largest one
    uint32_t numBlocks;
};

// One thread per sample; a workgroup's squared errors are summed in a fixed order.
template <typename T>
__global__ __launch_bounds__(256) void lossGradKernel(const LossArgs a)
{
    const T* const y = (const T*)a.y; const T* const z = (const T*)a.z; T* const dzOut = (T*)a.dz;
    __shared__ float red[256];
    __shared__ uint32_t maxBits;        // the largest per-sample loss as bits (non-negative floats order like integers)
    if (threadIdx.x == 0) maxBits = 0u;
    __syncthreads();
    float loss = 0.f, lossMax = 0.f;
    const uint32_t first = blockIdx.x * kLossSamplesPerBlock;
    for (uint32_t s = first + threadIdx.x; s < min(first + kLossSamplesPerBlock, a.batch); s += 256u) {
        const uint8_t* xin = a.in + (size_t)s * a.inStride;
        const bool exampleLoss = !a.targets && a.inEncoding == kEncodeXYSquares;
        half_t gt[4] = {(half_t)0, (half_t)0, (half_t)0, (half_t)0};
        float tgtAll = 0.f;
        if (exampleLoss) {
            exampleGroundTruth((half_t)((const float*)xin)[0], (half_t)((const float*)xin)[1], gt);
        } else if (!a.targets) {
            // sin(sum of the inputs), summed quarter by quarter like the fused kernel's lane groups
            const int gs = (int)optGS((uint32_t)a.inDim);
            float part[4] = {0.f, 0.f, 0.f, 0.f};
            for (int g = 0; g < 4; ++g)
                for (int q = 0; q < gs; ++q) {
                    const int j = g * gs + q;
                    if (j < a.inDim) part[g] += (float)((const T*)xin)[j];
                }
            // lane group g adds the partner groups in the order g^1, then the pair sums: (p0+p1)+(p2+p3)
            tgtAll = (float)(T)sinf((part[0] + part[1]) + (part[2] + part[3]));
        }
        float sampleLoss = 0.f;
        // one element: the same arithmetic in the same order, whichever way its operands were fetched
        auto element = [&](int i, T yv, T zv, float tv) -> T {
            const T diff = (T)((float)yv - tv);
            loss += (float)diff * (float)diff;
            sampleLoss += (float)diff * (float)diff;
            const T g = (T)(2.0f * (float)diff * a.lossScale);
            (void)i;
            return activationGrad<T>(g, zv, a.act, a.slope);
        };
        constexpr int EPC = 16 / (int)sizeof(T);                   // elements of a 16-byte piece
        const size_t e0 = (size_t)s * a.outDim;
        const bool pieces = a.outDim % EPC == 0 && (((uintptr_t)a.y | (uintptr_t)a.z | (uintptr_t)a.dz) & 15u) == 0 &&
                            (!a.targets || (((uintptr_t)a.targets | a.targetStride) & 15u) == 0);
        if (pieces) {
            // rows of whole aligned 16-byte pieces: three loads and one store per piece instead of per element
            for (int i0 = 0; i0 < a.outDim; i0 += EPC) {
                T yv[EPC], zv[EPC], tvv[EPC], gv[EPC];
                *(u32x4*)yv = *(const u32x4*)(y + e0 + i0);
                *(u32x4*)zv = *(const u32x4*)(z + e0 + i0);
                if (a.targets) *(u32x4*)tvv = *(const u32x4*)(a.targets + (size_t)s * a.targetStride + sizeof(T) * i0);
#pragma unroll
                for (int k = 0; k < EPC; ++k) {
                    const float tv = a.targets ? (float)tvv[k] : (exampleLoss ? (float)gt[(i0 + k) & 3] : tgtAll);
                    gv[k] = element(i0 + k, yv[k], zv[k], tv);
                }
                *(u32x4*)(dzOut + e0 + i0) = *(const u32x4*)gv;
            }
        } else {
            for (int i = 0; i < a.outDim; ++i) {
                const float tv = a.targets ? (float)*(const T*)(a.targets + (size_t)s * a.targetStride + sizeof(T) * i)
                                           : (exampleLoss ? (float)gt[i & 3] : tgtAll);
                dzOut[e0 + i] = element(i, y[e0 + i], z[e0 + i], tv);
            }
        }
        lossMax = (sampleLoss > lossMax || sampleLoss != sampleLoss) ? sampleLoss : lossMax;
    }
    red[threadIdx.x] = loss;
    atomicMax(&maxBits, __builtin_bit_cast(uint32_t, lossMax));
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        a.partials[blockIdx.x] = red[0];
        a.partials[a.numBlocks + blockIdx.x] = __builtin_bit_cast(float, maxBits);
    }
}

// the sum (fixed order: a thread's strided share, sixteen neighbouring threads per lane of the first wave, then lanes
// 32 ... 1 places apart) and the maximum of the per-workgroup loss partials
__global__ __launch_bounds__(1024) void lossFinalKernel(const float* partials, uint32_t n, float* lossSum, float* lossMax)
{
    __shared__ float red[1024];
    __shared__ uint32_t maxBits;
    if (threadIdx.x == 0) maxBits = 0u;
    __syncthreads();
    float c = 0.f;
    uint32_t m = 0u;
    for (uint32_t i = threadIdx.x; i < n; i += 1024u) {
        c += partials[i];
        const uint32_t b = __builtin_bit_cast(uint32_t, partials[n + i]);     // non-negative floats or NaN: ordered like their bits
        m = b > m ? b : m;
    }
    red[threadIdx.x] = c;
    if (m) atomicMax(&maxBits, m);
    __syncthreads();
    if (threadIdx.x < 64u) {
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < 16; ++k) s += red[threadIdx.x * 16 + k];
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) s += __shfl_xor(s, d, 64);
        if (threadIdx.x == 0) {
            if (lossSum) *lossSum = s;
            if (lossMax) *lossMax = __builtin_bit_cast(float, maxBits);
        }
    }
}

uint32_t gridFor(size_t count, int numCUs)
{
    const size_t need = (count / 8 + 255) / 256, cap = (size_t)numCUs * 8;
    return (uint32_t)(need < cap ? (need ? need : 1) : cap);
}

uint32_t alignOfPtr(const void* p, uint64_t stride)
{
    uint32_t al = 16;
    while (al > 1 && (((uintptr_t)p | stride) & (al - 1))) al >>= 1;
    return al;
}

} // namespace

size_t trainGeneralWorkspaceBytes(const MlpArgs& a, int numCUs, int carrierCt)
{
    if (a.numLayers < 2) return 0;
    return makePlan(a, numCUs, carrierCt).total;
}

hipError_t launchMlpTrainGeneral(hipStream_t stream, const TrainLaunch& t, int numCUs)
{
    const MlpArgs& a = t.mlp;
    const uint32_t batch = a.batch;
    if (batch == 0) return hipSuccess;
    const int L = a.numLayers;
    if (L < 2) return hipErrorInvalidValue;
    const int ct = t.carrierCt;                 // kF16 or kF32: vectors, weights, biases
    const bool f32 = ct == kF32;
    const uint64_t esz = elemSize(ct);
    const MmaKind mma = f32 ? MmaKind::F32 : MmaKind::F16;
    const GeneralPlan p = makePlan(a, numCUs, ct);
    uint8_t* ws = (uint8_t*)t.workspace;
    hipError_t e;

    // ---- network input ------------------------------------------------------------------------
    const uint8_t* x = a.in;
    uint64_t xStride = a.inStride;
    if (a.inEncoding == kEncodeXYSquares) {
        hipLaunchKernelGGL(encodeXYKernel, dim3((batch + 255) / 256), dim3(256), 0, stream, a.in, a.inStride, batch, (uint32_t*)(ws + p.x0));
        if ((e = hipGetLastError()) != hipSuccess) return e;
        x = ws + p.x0; xStride = 8;
    }

    // ---- forward ------------------------------------------------------------------------------
    const uint8_t* xl[kMaxMlpLayers];
    uint64_t xlStride[kMaxMlpLayers];
    // fp16 networks up to 128 wide: one launch of the run-time-size forward kernel that leaves every layer's
    // pre-activations and activations where the per-layer launches below would (same arithmetic, same bits); the input
    // is read once and no vector makes a second trip through memory
    bool forwardDone = false;
    if (!f32) {
        MlpArgs fa = a;
        fa.in = x; fa.inStride = xStride; fa.inEncoding = kEncodeNone;
        fa.inAlign = alignOfPtr(fa.in, fa.inStride);
        fa.out = ws + p.act[L - 1]; fa.outStride = (uint64_t)a.layers[L - 1].out * esz;
        fa.outAlign = alignOfPtr(fa.out, fa.outStride);
        fa.inHalfAsE4M3 = 0;
        uint8_t* tapZ[kMaxMlpLayers] = {};
        uint8_t* tapX[kMaxMlpLayers] = {};
        for (int l = 0; l < L; ++l) {
            const bool last = l + 1 == L;
            if (!last || p.z[l] != p.act[l]) tapZ[l] = ws + p.z[l];
            if (!last && p.act[l] != p.z[l]) tapX[l] = ws + p.act[l];
        }
        e = launchMlpGenericTaps(stream, fa, tapZ, tapX, numCUs);
        if (e == hipSuccess) forwardDone = true;
        else if (e != hipErrorInvalidValue) return e;
    }
    for (int l = 0; l < L; ++l) {
        const MlpLayerArgs& ly = a.layers[l];
        xl[l] = x; xlStride[l] = xStride;
        if (forwardDone) {
            x = ws + p.act[l]; xStride = (uint64_t)ly.out * esz;
            continue;
        }
        MatMulArgs m;
        memset(&m, 0, sizeof(m));
        m.in = x; m.inStride = xStride;
        m.out = ws + p.z[l]; m.outStride = (uint64_t)ly.out * esz;
        m.mat = ly.w; m.bias = ly.bias; m.biasCt = ct;
        m.shape = ly.shape; m.transpose = 0; m.m = ly.out; m.k = ly.in;
        m.inCt = ct; m.outCt = ct; m.act = kActNone; m.batch = batch;
        m.inAlign = alignOfPtr(m.in, m.inStride); m.outAlign = alignOfPtr(m.out, m.outStride);
        if ((e = launchMatMul(stream, mma, m, numCUs)) != hipSuccess) return e;
        if (ly.act != kActNone) {
            const size_t count = (size_t)batch * ly.out;
            if (f32) hipLaunchKernelGGL(activationKernel<float>, dim3(gridFor(count, numCUs)), dim3(256), 0, stream,
                                        (const float*)(ws + p.z[l]), (float*)(ws + p.act[l]), count, ly.act, ly.slope);
            else hipLaunchKernelGGL(activationKernel<half_t>, dim3(gridFor(count, numCUs)), dim3(256), 0, stream,
                                    (const half_t*)(ws + p.z[l]), (half_t*)(ws + p.act[l]), count, ly.act, ly.slope);
            if ((e = hipGetLastError()) != hipSuccess) return e;
        }
        x = ws + p.act[l]; xStride = (uint64_t)ly.out * esz;
    }

    // ---- loss and the gradient at the last pre-activation -----------------------------------------
    {
        const MlpLayerArgs& ly = a.layers[L - 1];
        LossArgs la;
        la.y = ws + p.act[L - 1]; la.z = ws + p.z[L - 1];
        la.dz = ws + p.gA;
        la.targets = t.targets; la.targetStride = t.targetStride;
        la.in = a.in; la.inStride = a.inStride;
        la.inDim = a.layers[0].in; la.outDim = ly.out; la.inEncoding = a.inEncoding;
        la.act = ly.act; la.slope = ly.slope; la.lossScale = t.lossScale; la.batch = batch;
        la.partials = (float*)(ws + p.lossPartials);
        la.numBlocks = p.lossBlocks;
        if (f32) hipLaunchKernelGGL(lossGradKernel<float>, dim3(p.lossBlocks), dim3(256), 0, stream, la);
        else hipLaunchKernelGGL(lossGradKernel<half_t>, dim3(p.lossBlocks), dim3(256), 0, stream, la);
        if ((e = hipGetLastError()) != hipSuccess) return e;
        if (t.lossSum || t.lossMax) {
            hipLaunchKernelGGL(lossFinalKernel, dim3(1), dim3(1024), 0, stream, (const float*)(ws + p.lossPartials), p.lossBlocks, t.lossSum, t.lossMax);
            if ((e = hipGetLastError()) != hipSuccess) return e;
        }
    }

    // ---- backward -----------------------------------------------------------------------------
    size_t dzOff = p.gA, otherOff = p.gB;
    for (int l = L - 1; l >= 0; --l) {
        const MlpLayerArgs& ly = a.layers[l];
        const uint8_t* dz = ws + dzOff;
        const uint64_t dzStride = (uint64_t)ly.out * esz;
        if (f32) {
            // fp32 vectors: into fp32 gradients on the matrix pipeline's fp32 instruction, into half ones through the
            // scalar accumulate kernels (db: the reduce-sum form, b == 1)
            const bool pipe = t.gradCt == kF32;
            if (t.bGrad[l]) {
                const MatrixShape bs{(uint32_t)ly.out, 1u, t.gradCt, kRowMajor, (size_t)elemSize(t.gradCt)};
                e = pipe ? launchOuterProductF32(stream, dz, dzStride, ly.out, nullptr, 0, 1, batch, t.bGrad[l], bs, ws + p.partials, numCUs)
                         : launchAccumScalar(stream, dz, dzStride, ly.out, nullptr, 0, 1, ct, batch, t.bGrad[l], bs, ws + p.partials);
                if (e != hipSuccess) return e;
            }
            if (t.wGrad[l]) {
                e = pipe ? launchOuterProductF32(stream, dz, dzStride, ly.out, xl[l], xlStride[l], ly.in, batch, t.wGrad[l], t.gradShape[l],
                                                 ws + p.partials, numCUs)
                         : launchAccumScalar(stream, dz, dzStride, ly.out, xl[l], xlStride[l], ly.in, ct, batch, t.wGrad[l], t.gradShape[l],
                                             ws + p.partials);
                if (e != hipSuccess) return e;
            }
        }
        if (!f32 && t.bGrad[l]) {
            for (int c0 = 0; c0 < ly.out; c0 += 256) {      // the reduce kernel takes up to 256 columns
                const int n = ly.out - c0 < 256 ? ly.out - c0 : 256;
                ReduceSumArgs r;
                memset(&r, 0, sizeof(r));
                r.v = dz + (size_t)c0 * 2; r.vStride = dzStride; r.n = n;
                r.colsPerGroup = (((n + 3) / 4) + 1) / 2 * 2;
                r.batch = batch; r.buf = t.bGrad[l] + (size_t)c0 * elemSize(t.gradCt); r.bufCt = t.gradCt;
                r.partials = (float*)(ws + p.partials);
                if ((e = launchReduceSum(stream, r, numCUs)) != hipSuccess) return e;
            }
        }
        if (!f32 && t.wGrad[l]) {
            OuterArgs o;
            memset(&o, 0, sizeof(o));
            o.a = dz; o.aStride = dzStride; o.aAlign = alignOfPtr(o.a, o.aStride);
            o.b = xl[l]; o.bStride = xlStride[l]; o.bAlign = alignOfPtr(o.b, o.bStride);
            o.m = ly.out; o.n = ly.in; o.batch = batch;
            o.mat = t.wGrad[l]; o.shape = t.gradShape[l];
            o.partials = (float*)(ws + p.partials);
            if ((e = launchOuterProduct(stream, o, numCUs)) != hipSuccess) return e;
        }
        if (l == 0) break;
        // g = W^T dZ (rounded to half), then through the previous layer's activation
        const MlpLayerArgs& prev = a.layers[l - 1];
        const bool prevAct = prev.act != kActNone;
        MatMulArgs m;
        memset(&m, 0, sizeof(m));
        m.in = dz; m.inStride = dzStride;
        m.out = ws + otherOff; m.outStride = (uint64_t)ly.in * esz;
        m.mat = ly.w; m.shape = ly.shape; m.transpose = 1; m.m = ly.in; m.k = ly.out;
        m.inCt = ct; m.outCt = ct; m.act = kActNone; m.batch = batch;
        m.inAlign = alignOfPtr(m.in, m.inStride); m.outAlign = alignOfPtr(m.out, m.outStride);
        if ((e = launchMatMul(stream, mma, m, numCUs)) != hipSuccess) return e;
        if (prevAct) {
            // in place: element i of dz depends on element i of g only
            const size_t count = (size_t)batch * ly.in;
            if (f32) hipLaunchKernelGGL(activationGradKernel<float>, dim3(gridFor(count, numCUs)), dim3(256), 0, stream,
                                        (const float*)(ws + otherOff), (const float*)(ws + p.z[l - 1]), (float*)(ws + otherOff),
                                        count, prev.act, prev.slope);
            else hipLaunchKernelGGL(activationGradKernel<half_t>, dim3(gridFor(count, numCUs)), dim3(256), 0, stream,
                                    (const half_t*)(ws + otherOff), (const half_t*)(ws + p.z[l - 1]), (half_t*)(ws + otherOff),
                                    count, prev.act, prev.slope);
            if ((e = hipGetLastError()) != hipSuccess) return e;
        }
        const size_t tmp = dzOff; dzOff = otherOff; otherOff = tmp;
    }
    noteKernel(false, "layer-by-layer training step: matmulKernel/activationKernel (forward), lossGradKernel, "
                      "reduceSum + outerProduct + transposed matmulKernel + activationGradKernel per layer (backward)");
    return hipSuccess;
}

} // namespace cv
