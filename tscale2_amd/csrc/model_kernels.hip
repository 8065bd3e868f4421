// Kernels around the layer stack: label embedding, final soft-max / loss gradient and 16-bit transposed copies for the
// final layer's bf16 products (the reference runs them in fp16: src/gpt/compute/gpu_final.cuh:223-296, gpu_embedding.cuh:126-218).
#include "vec.h"
#include "internal.h"

namespace
{
// state0[t] = sum over labels of +-E[label] * scale (ComputeEmbedding, src/gpt/compute/cpu_transformer.cpp:76-100); one workgroup per row
template <class TEmb>
__global__ void __launch_bounds__(256) EmbedForward(int len, int dim, const int *labelPtr, const uint32_t *labels, const uint8_t *embed,
    int64_t ldEmb, float mult, const float *scalePtr, float *state, int64_t ldState)
{
    int t = blockIdx.x;
    float s = mult * (scalePtr ? *scalePtr : 1.f);
    for (int col = threadIdx.x * 4; col < dim; col += 1024) {
        F4 acc = ZeroF4();
        if (t < len) {
            for (int k = labelPtr[t]; k < labelPtr[t + 1]; ++k) {
                uint32_t label = labels[k];
                float w = (label & 0x80000000u) ? -s : s;
                label &= 0x7fffffffu;
                acc = acc + Load4<TEmb>(embed + (int64_t)label * ldEmb + col * TEmb::SIZE) * w;
            }
        }
        Store4<TF32>((uint8_t *)state + (int64_t)t * ldState + col * 4, acc);
    }
}

// deltaLabel[label] += +-grad[t]  (src/gpt/compute/cpu_transformer.cpp:182-197); fp32 atomics, delta cleared by the caller
__global__ void __launch_bounds__(256) EmbedBackward(int len, int dim, const int *labelPtr, const uint32_t *labels, const float *grad, int64_t ldGrad,
    float *delta, int64_t ldDelta)
{
    int t = blockIdx.x;
    for (int k = labelPtr[t]; k < labelPtr[t + 1]; ++k) {
        uint32_t label = labels[k];
        float w = (label & 0x80000000u) ? -1.f : 1.f;
        label &= 0x7fffffffu;
        for (int col = threadIdx.x; col < dim; col += 256) {
            atomicAdd(delta + (int64_t)label * ldDelta / 4 + col, grad[(int64_t)t * ldGrad / 4 + col] * w);
        }
    }
}

// SoftMax base 2 with running max starting at 0 and the (onehot - p) gradient (src/gpt/compute/cpu_transformer.cpp:12-37,146-159).
// One workgroup per row; logits fp32 [row][vocab] are overwritten by probabilities when keepProb, grad is bf16.  Two passes over the
// row with 16-byte accesses: the first finds the maximum and the sum together (the sum is rescaled whenever a lane's maximum grows),
// the second, served by the caches, writes the gradient.  vocab is a multiple of 4.
__global__ void __launch_bounds__(256) FinalSoftmaxGrad(int vocab, float *logits, int64_t ldLogits, const float *bias, const int *target,
    float gradMult, bf16_t *grad, int64_t ldGrad, float *lossSum, int keepProb)
{
    __shared__ float redM[4], redS[4];
    int t = blockIdx.x;
    int tid = threadIdx.x;
    float *row = (float *)((uint8_t *)logits + (int64_t)t * ldLogits);
    bf16_t *grow = (bf16_t *)((uint8_t *)grad + (int64_t)t * ldGrad);
    int tg = target[t];
    if (tg < 0) {
        for (int k = tid * 4; k < vocab; k += 1024) {
            *(uint2 *)(grow + k) = make_uint2(0, 0);
        }
        if (!keepProb) {
            return;
        }
    }
    // lane-local running maximum m (of the logits without bias, never below 0) and sum of 2^(x + bias - m)
    float m = 0, sum = 0;
    for (int k0 = tid * 4; k0 < vocab; k0 += 4096) {
        float4 x[4], bv[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int k = k0 + i * 1024;
            bool in = k < vocab;
            x[i] = in ? *(const float4 *)(row + k) : make_float4(-1e30f, -1e30f, -1e30f, -1e30f);
            bv[i] = in ? *(const float4 *)(bias + k) : make_float4(0, 0, 0, 0);
        }
        float mNew = m;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            mNew = fmaxf(mNew, fmaxf(fmaxf(x[i].x, x[i].y), fmaxf(x[i].z, x[i].w)));
        }
        sum *= exp2f(m - mNew);
        m = mNew;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            sum += (exp2f(x[i].x + bv[i].x - m) + exp2f(x[i].y + bv[i].y - m)) + (exp2f(x[i].z + bv[i].z - m) + exp2f(x[i].w + bv[i].w - m));
        }
    }
    float mx = WaveMax(m);
    if ((tid & 63) == 0) {
        redM[tid >> 6] = mx;
    }
    __syncthreads();
    mx = fmaxf(fmaxf(redM[0], redM[1]), fmaxf(redM[2], redM[3]));
    sum = WaveSum(sum * exp2f(m - mx));
    if ((tid & 63) == 0) {
        redS[tid >> 6] = sum;
    }
    __syncthreads();
    float scale = 1 / ((redS[0] + redS[1]) + (redS[2] + redS[3]));
    for (int k0 = tid * 4; k0 < vocab; k0 += 4096) {
        float4 x[4], bv[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int k = k0 + i * 1024;
            bool in = k < vocab;
            x[i] = in ? *(const float4 *)(row + k) : make_float4(0, 0, 0, 0);
            bv[i] = in ? *(const float4 *)(bias + k) : make_float4(0, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int k = k0 + i * 1024;
            if (k >= vocab) {
                continue;
            }
            float p[4] = {exp2f(x[i].x + bv[i].x - mx) * scale, exp2f(x[i].y + bv[i].y - mx) * scale, exp2f(x[i].z + bv[i].z - mx) * scale,
                exp2f(x[i].w + bv[i].w - mx) * scale};
            if (keepProb) {
                *(float4 *)(row + k) = make_float4(p[0], p[1], p[2], p[3]);
            }
            if (tg >= 0) {
                float g[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    g[e] = ((k + e == tg ? 1.f : 0.f) - p[e]) * gradMult;
                    if (k + e == tg && lossSum) {
                        atomicAdd(lossSum, logf(p[e]));
                    }
                }
                *(uint2 *)(grow + k) = make_uint2(PackBf16x2(g[0], g[1]), PackBf16x2(g[2], g[3]));
            }
        }
    }
}

// dst[x][t] = bf16(src[t][x]) for t < rows, 0 up to rowsRound; 64x64 tiles through LDS
template <class TSrc>
__global__ void __launch_bounds__(256) TransposeToBf16(int rows, int rowsRound, int cols, const uint8_t *src, int64_t ldSrc, uint8_t *dst, int64_t ldDst)
{
    __shared__ float tile[64][65];
    int x0 = blockIdx.x * 64, t0 = blockIdx.y * 64;
    int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int r = ty; r < 64; r += 4) {
        int t = t0 + r, x = x0 + tx;
        float v = 0;
        if (t < rows && x < cols) {
            const uint8_t *p = src + (int64_t)t * ldSrc + (int64_t)x * TSrc::SIZE;
            if (TSrc::SIZE == 2) {
                v = Bf16ToFloat(*(const bf16_t *)p);
            } else if (std::is_same<TSrc, TI8>::value) {
                v = (float)*(const int8_t *)p;
            } else {
                v = __builtin_amdgcn_cvt_f32_fp8((int)*p, 0);
            }
        }
        tile[r][tx] = v;
    }
    __syncthreads();
    for (int r = ty; r < 64; r += 4) {
        int x = x0 + r, t = t0 + tx;
        if (x < cols && t < rowsRound) {
            *(bf16_t *)(dst + (int64_t)x * ldDst + (int64_t)t * 2) = FloatToBf16(tile[tx][r]);
        }
    }
}

// dst[x][t] = src[t][x] for 2-byte elements, zeros for rows <= t < rowsRound; 64x64 tiles, 16-byte loads and stores.
// cols and rowsRound are multiples of 8, rows of both matrices 16-byte aligned.
__global__ void __launch_bounds__(256) Transpose16(int rows, int rowsRound, int cols, const uint8_t *src, int64_t ldSrc, uint8_t *dst, int64_t ldDst)
{
    constexpr int PITCH = 66; // 2-byte elements per LDS row: column reads of neighbouring lanes fall into different banks
    __shared__ __attribute__((aligned(16))) uint16_t tile[64 * PITCH];
    int x0 = blockIdx.x * 64, t0 = blockIdx.y * 64;
    int tid = threadIdx.x;
    int lc = tid & 7, lr = tid >> 3; // 8 lanes x 16 bytes per row, 32 rows per pass
    v4i raw[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        int t = t0 + lr + 32 * k, x = x0 + lc * 8;
        raw[k] = (t < rows && x < cols) ? *(const v4i *)(src + (int64_t)t * ldSrc + (int64_t)x * 2) : (v4i){0, 0, 0, 0};
    }
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        uint32_t *d = (uint32_t *)(tile + (lr + 32 * k) * PITCH + lc * 8);
        d[0] = (uint32_t)raw[k][0];
        d[1] = (uint32_t)raw[k][1];
        d[2] = (uint32_t)raw[k][2];
        d[3] = (uint32_t)raw[k][3];
    }
    __syncthreads();
    // thread -> destination row x (64 of them), 8 consecutive t (8 blocks): 2 units per thread
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        int u = tid + 256 * k;
        int tb = u & 7, xr = u >> 3;
        uint32_t w[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            uint32_t lo = tile[(tb * 8 + 2 * e) * PITCH + xr];
            uint32_t hi = tile[(tb * 8 + 2 * e + 1) * PITCH + xr];
            w[e] = lo | (hi << 16);
        }
        int x = x0 + xr, t = t0 + tb * 8;
        if (x < cols && t < rowsRound) {
            *(uint4 *)(dst + (int64_t)x * ldDst + (int64_t)t * 2) = make_uint4(w[0], w[1], w[2], w[3]);
        }
    }
}

__global__ void ZeroBytes(uint8_t *p, int64_t ld, int rowBytes)
{
    uint8_t *row = p + (int64_t)blockIdx.x * ld;
    for (int x = threadIdx.x * 4; x < rowBytes; x += blockDim.x * 4) {
        *(uint32_t *)(row + x) = 0;
    }
}
// The same for IEEE-half logits (the reference keeps its logit window in half, src/gpt/compute/gpu_final.cuh:173-189): eight values
// per 16-byte load, no probabilities kept
__global__ void __launch_bounds__(256) FinalSoftmaxGradHalf(int vocab, const _Float16 *logits, int64_t ldLogits, const float *bias, const int *target,
    float gradMult, bf16_t *grad, int64_t ldGrad, float *lossSum)
{
    typedef _Float16 v8h __attribute__((ext_vector_type(8)));
    __shared__ float redM[4], redS[4];
    int t = blockIdx.x;
    int tid = threadIdx.x;
    const _Float16 *row = (const _Float16 *)((const uint8_t *)logits + (int64_t)t * ldLogits);
    bf16_t *grow = (bf16_t *)((uint8_t *)grad + (int64_t)t * ldGrad);
    int tg = target[t];
    if (tg < 0) {
        for (int k = tid * 8; k < vocab; k += 2048) {
            *(uint4 *)(grow + k) = make_uint4(0, 0, 0, 0);
        }
        return;
    }
    float m = 0, sum = 0;
    for (int k0 = tid * 8; k0 < vocab; k0 += 4096) {
        float x[2][8], bv[2][8];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            int k = k0 + i * 2048;
            bool in = k < vocab;
            v8h h = in ? *(const v8h *)(row + k) : (v8h)(_Float16)-60000.f;
            float4 b0 = in ? *(const float4 *)(bias + k) : make_float4(0, 0, 0, 0);
            float4 b1 = in ? *(const float4 *)(bias + k + 4) : make_float4(0, 0, 0, 0);
            const float bb[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                x[i][e] = (float)h[e];
                bv[i][e] = bb[e];
            }
        }
        float mNew = m;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                mNew = fmaxf(mNew, x[i][e]);
            }
        }
        sum *= exp2f(m - mNew);
        m = mNew;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                sum += exp2f(x[i][e] + bv[i][e] - m);
            }
        }
    }
    float mx = WaveMax(m);
    if ((tid & 63) == 0) {
        redM[tid >> 6] = mx;
    }
    __syncthreads();
    mx = fmaxf(fmaxf(redM[0], redM[1]), fmaxf(redM[2], redM[3]));
    sum = WaveSum(sum * exp2f(m - mx));
    if ((tid & 63) == 0) {
        redS[tid >> 6] = sum;
    }
    __syncthreads();
    float scale = 1 / ((redS[0] + redS[1]) + (redS[2] + redS[3]));
    for (int k = tid * 8; k < vocab; k += 2048) {
        v8h h = *(const v8h *)(row + k); // second read of the row: served by L2
        float4 b0 = *(const float4 *)(bias + k), b1 = *(const float4 *)(bias + k + 4);
        const float bb[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
        float g[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            float pr = exp2f((float)h[e] + bb[e] - mx) * scale;
            g[e] = ((k + e == tg ? 1.f : 0.f) - pr) * gradMult;
            if (k + e == tg && lossSum) {
                atomicAdd(lossSum, logf(pr));
            }
        }
        *(uint4 *)(grow + k) = make_uint4(PackBf16x2(g[0], g[1]), PackBf16x2(g[2], g[3]), PackBf16x2(g[4], g[5]), PackBf16x2(g[6], g[7]));
    }
}
// The same for rows of at most ROW_ROUNDS * 8192 logits, with the row read once and one exponential per logit: a workgroup of 1024
// threads walks rows with a grid stride and a thread keeps its logits in registers.  It takes its own maximum first (packed half
// max), replaces every logit by 2^(logit + bias - own reference) as a half (a number in [0, 1] with 11 significant bits, more than
// the bf16 gradient keeps) while summing in fp32, and after the workgroup reduction the gradient is that half times one per-thread
// factor.  The next row's loads are in flight during all of this.  Arithmetic per logit: two conversions, two adds, one v_exp_f32,
// one sum, one multiply - the two-pass kernel above is bound by its VALU work (two exponentials per logit), not by memory.
constexpr int ROW_ROUNDS = 7; // up to 57344 logits; 2 x 28 registers of row data per thread

__global__ void __launch_bounds__(1024) FinalSoftmaxGradHalfRow(int rows, int vocab, const _Float16 *logits, int64_t ldLogits, const float *bias,
    const int *target, float gradMult, bf16_t *grad, int64_t ldGrad, float *lossSum)
{
    typedef _Float16 v8h __attribute__((ext_vector_type(8)));
    __shared__ float redM[16], redS[16];
    const int tid = threadIdx.x;
    v8h cur[ROW_ROUNDS], nxt[ROW_ROUNDS];
    auto prefetch = [&](int t) {
        const _Float16 *row = (const _Float16 *)((const uint8_t *)logits + (int64_t)t * ldLogits);
#pragma unroll
        for (int i = 0; i < ROW_ROUNDS; ++i) {
            int k = tid * 8 + i * 8192;
            nxt[i] = k < vocab ? *(const v8h *)(row + k) : (v8h)(_Float16)-60000.f;
        }
    };
    int t = blockIdx.x;
    if (t < rows) {
        prefetch(t);
    }
    // a thread meets the same columns in every row: the largest bias among them, added to its reference, keeps the halves in [0, 1]
    float biasTop = 0;
#pragma unroll
    for (int i = 0; i < ROW_ROUNDS; ++i) {
        int k = tid * 8 + i * 8192;
        if (k < vocab) {
            float4 b0 = *(const float4 *)(bias + k), b1 = *(const float4 *)(bias + k + 4);
            biasTop = fmaxf(fmaxf(fmaxf(biasTop, fmaxf(b0.x, b0.y)), fmaxf(b0.z, b0.w)), fmaxf(fmaxf(b1.x, b1.y), fmaxf(b1.z, b1.w)));
        }
    }
    for (; t < rows; t += gridDim.x) {
#pragma unroll
        for (int i = 0; i < ROW_ROUNDS; ++i) {
            cur[i] = nxt[i];
        }
        if (t + (int)gridDim.x < rows) {
            prefetch(t + gridDim.x);
        }
        bf16_t *grow = (bf16_t *)((uint8_t *)grad + (int64_t)t * ldGrad);
        const int tg = target[t];
        if (tg < 0) { // (workgroup-uniform) no label: zero gradient
            for (int k = tid * 8; k < vocab; k += 8192) {
                *(uint4 *)(grow + k) = make_uint4(0, 0, 0, 0);
            }
            continue;
        }
        // own reference: the largest logit (not below 0, as in the two-pass kernel) plus the largest bias of the thread's columns
        v8h hm = cur[0];
#pragma unroll
        for (int i = 1; i < ROW_ROUNDS; ++i) {
            hm = __builtin_elementwise_max(hm, cur[i]);
        }
        float m = 0;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            m = fmaxf(m, (float)hm[e]);
        }
        m += biasTop;
        float sum = 0;
#pragma unroll
        for (int i = 0; i < ROW_ROUNDS; ++i) {
            int k = tid * 8 + i * 8192;
            if (k < vocab) {
                float4 b0 = *(const float4 *)(bias + k), b1 = *(const float4 *)(bias + k + 4);
                const float bb[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
                v8h ex;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    float w = __builtin_amdgcn_exp2f((float)cur[i][e] + (bb[e] - m)); // hardware exp2: below 2^-126 flushed to zero
                    sum += w;
                    ex[e] = (_Float16)w;
                }
                cur[i] = ex;
            }
        }
        float mx = WaveMax(m);
        if ((tid & 63) == 0) {
            redM[tid >> 6] = mx;
        }
        __syncthreads();
        mx = redM[0];
#pragma unroll
        for (int w = 1; w < 16; ++w) {
            mx = fmaxf(mx, redM[w]);
        }
        const float own = __builtin_amdgcn_exp2f(m - mx); // own reference -> row reference
        sum = WaveSum(sum * own);
        if ((tid & 63) == 0) {
            redS[tid >> 6] = sum;
        }
        __syncthreads();
        float total = 0;
#pragma unroll
        for (int w = 0; w < 16; ++w) {
            total += redS[w];
        }
        const float scale = own / total;       // half -> probability
        const float negScale = -scale * gradMult; // half -> gradient of a logit that is not the label
#pragma unroll
        for (int i = 0; i < ROW_ROUNDS; ++i) {
            int k = tid * 8 + i * 8192;
            if (k < vocab) {
                float g[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    g[e] = (float)cur[i][e] * negScale;
                }
                if ((unsigned)(tg - k) < 8u) { // the label's chunk (one thread of the workgroup)
                    float pr = 0;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        pr = e == tg - k ? (float)cur[i][e] * scale : pr;
                    }
                    const float gt = (1.f - pr) * gradMult;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        g[e] = e == tg - k ? gt : g[e];
                    }
                    if (lossSum) {
                        atomicAdd(lossSum, logf(pr));
                    }
                }
                *(uint4 *)(grow + k) = make_uint4(PackBf16x2(g[0], g[1]), PackBf16x2(g[2], g[3]), PackBf16x2(g[4], g[5]), PackBf16x2(g[6], g[7]));
            }
        }
        __syncthreads(); // the reduction slots are free again
    }
}
} // namespace

#define STREAM ((hipStream_t)stream)

int Ts2EmbedForward(int len, int lenRound, int dim, const int *labelPtr, const uint32_t *labels, const ts2_mat *embed, int embType, float mult,
    const float *scalePtr, const ts2_mat *state, void *stream)
{
    if (embType == TS2_I8) {
        hipLaunchKernelGGL((EmbedForward<TI8>), dim3(lenRound), dim3(256), 0, STREAM, len, dim, labelPtr, labels, (const uint8_t *)embed->ptr,
            embed->strideBytes, mult, scalePtr, (float *)state->ptr, state->strideBytes);
    } else if (embType == TS2_E4M3) {
        hipLaunchKernelGGL((EmbedForward<TE4M3>), dim3(lenRound), dim3(256), 0, STREAM, len, dim, labelPtr, labels, (const uint8_t *)embed->ptr,
            embed->strideBytes, mult, scalePtr, (float *)state->ptr, state->strideBytes);
    } else {
        return TS2_ERR_UNSUPPORTED;
    }
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

int Ts2EmbedBackward(int len, int dim, const int *labelPtr, const uint32_t *labels, const ts2_mat *grad, const ts2_mat *delta, int labelCount,
    void *stream)
{
    hipLaunchKernelGGL(ZeroBytes, dim3(labelCount), dim3(256), 0, STREAM, (uint8_t *)delta->ptr, delta->strideBytes, dim * 4);
    TS2_CHECK_LAUNCH();
    hipLaunchKernelGGL(EmbedBackward, dim3(len), dim3(256), 0, STREAM, len, dim, labelPtr, labels, (const float *)grad->ptr, grad->strideBytes,
        (float *)delta->ptr, delta->strideBytes);
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

int Ts2FinalSoftmaxGradHalf(int rows, int vocab, const ts2_mat *logits, const float *bias, const int *target, float gradMult, const ts2_mat *grad,
    float *lossSum, void *stream)
{
    if (vocab % 8 || (logits->strideBytes & 15) || (grad->strideBytes & 15) || ((uintptr_t)logits->ptr & 15) || ((uintptr_t)grad->ptr & 15) ||
        ((uintptr_t)bias & 15)) {
        return TS2_ERR_ALIGN;
    }
    if (vocab >= 2048 && vocab <= ROW_ROUNDS * 8192) {
        const int wgs = rows < 512 ? rows : 512; // one workgroup of 16 waves per CU is resident (registers); two per CU in the queue
        hipLaunchKernelGGL(FinalSoftmaxGradHalfRow, dim3(wgs), dim3(1024), 0, STREAM, rows, vocab, (const _Float16 *)logits->ptr,
            logits->strideBytes, bias, target, gradMult, (bf16_t *)grad->ptr, grad->strideBytes, lossSum);
    } else {
        hipLaunchKernelGGL(FinalSoftmaxGradHalf, dim3(rows), dim3(256), 0, STREAM, vocab, (const _Float16 *)logits->ptr, logits->strideBytes, bias,
            target, gradMult, (bf16_t *)grad->ptr, grad->strideBytes, lossSum);
    }
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

int Ts2FinalSoftmaxGrad(int rows, int vocab, const ts2_mat *logits, const float *bias, const int *target, float gradMult, const ts2_mat *grad,
    float *lossSum, int keepProb, void *stream)
{
    hipLaunchKernelGGL(FinalSoftmaxGrad, dim3(rows), dim3(256), 0, STREAM, vocab, (float *)logits->ptr, logits->strideBytes, bias, target, gradMult,
        (bf16_t *)grad->ptr, grad->strideBytes, lossSum, keepProb);
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

// dst[t][x] = bf16(src[t][x]) for 8-bit src (exact), rows <= t < rowsRound zero; a lane converts 8 consecutive elements
template <class TSrc>
__global__ void __launch_bounds__(256) RowsToBf16(int rows, int rowsRound, int cols8, const uint8_t *src, int64_t ldSrc, uint8_t *dst, int64_t ldDst)
{
    const long total = (long)rowsRound * cols8;
    for (long u = (long)blockIdx.x * 256 + threadIdx.x; u < total; u += (long)gridDim.x * 256) {
        const int t = (int)(u / cols8), c = (int)(u % cols8);
        uint32_t out[4] = {0, 0, 0, 0};
        if (t < rows) {
            const uint2 in = *(const uint2 *)(src + (int64_t)t * ldSrc + c * 8);
            const uint32_t w[2] = {in.x, in.y};
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
                float lo, hi;
                if (std::is_same<TSrc, TI8>::value) {
                    lo = (float)(int8_t)(w[e >> 2] >> (8 * (e & 3)));
                    hi = (float)(int8_t)(w[e >> 2] >> (8 * ((e + 1) & 3)));
                } else {
                    lo = (e & 3) == 0 ? __builtin_amdgcn_cvt_f32_fp8((int)w[e >> 2], 0) : __builtin_amdgcn_cvt_f32_fp8((int)w[e >> 2], 2);
                    hi = (e & 3) == 0 ? __builtin_amdgcn_cvt_f32_fp8((int)w[e >> 2], 1) : __builtin_amdgcn_cvt_f32_fp8((int)w[e >> 2], 3);
                }
                out[e >> 1] = PackBf16x2(lo, hi);
            }
        }
        *(uint4 *)(dst + (int64_t)t * ldDst + c * 16) = make_uint4(out[0], out[1], out[2], out[3]);
    }
}

int Ts2RowsToBf16(int rows, int rowsRound, int cols, const ts2_mat *src, int srcType, const ts2_mat *dst, void *stream)
{
    if ((cols & 7) || (src->strideBytes & 7) || (dst->strideBytes & 15) || ((uintptr_t)src->ptr & 7) || ((uintptr_t)dst->ptr & 15)) {
        return TS2_ERR_ALIGN;
    }
    const long total = (long)rowsRound * (cols / 8);
    const dim3 grid((unsigned)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192));
    if (srcType == TS2_I8) {
        hipLaunchKernelGGL((RowsToBf16<TI8>), grid, dim3(256), 0, STREAM, rows, rowsRound, cols / 8, (const uint8_t *)src->ptr, src->strideBytes,
            (uint8_t *)dst->ptr, dst->strideBytes);
    } else if (srcType == TS2_E4M3) {
        hipLaunchKernelGGL((RowsToBf16<TE4M3>), grid, dim3(256), 0, STREAM, rows, rowsRound, cols / 8, (const uint8_t *)src->ptr, src->strideBytes,
            (uint8_t *)dst->ptr, dst->strideBytes);
    } else {
        return TS2_ERR_UNSUPPORTED;
    }
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

int Ts2TransposeToBf16(int rows, int rowsRound, int cols, const ts2_mat *src, int srcType, const ts2_mat *dst, void *stream)
{
    dim3 grid((cols + 63) / 64, (rowsRound + 63) / 64);
    const uint8_t *s = (const uint8_t *)src->ptr;
    uint8_t *d = (uint8_t *)dst->ptr;
    if (srcType == TS2_I8) {
        hipLaunchKernelGGL((TransposeToBf16<TI8>), grid, dim3(256), 0, STREAM, rows, rowsRound, cols, s, src->strideBytes, d, dst->strideBytes);
    } else if (srcType == TS2_E4M3) {
        hipLaunchKernelGGL((TransposeToBf16<TE4M3>), grid, dim3(256), 0, STREAM, rows, rowsRound, cols, s, src->strideBytes, d, dst->strideBytes);
    } else if (srcType == TS2_BF16) {
        if (cols % 8 == 0 && rowsRound % 8 == 0 && src->strideBytes % 16 == 0 && dst->strideBytes % 16 == 0 && (uintptr_t)s % 16 == 0 &&
            (uintptr_t)d % 16 == 0) {
            hipLaunchKernelGGL(Transpose16, grid, dim3(256), 0, STREAM, rows, rowsRound, cols, s, src->strideBytes, d, dst->strideBytes);
        } else {
            hipLaunchKernelGGL((TransposeToBf16<TBF16>), grid, dim3(256), 0, STREAM, rows, rowsRound, cols, s, src->strideBytes, d, dst->strideBytes);
        }
    } else {
        return TS2_ERR_UNSUPPORTED;
    }
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

__global__ void FillFloatsKernel(float *p, int n, float v)
{
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        p[i] = v;
    }
}

int Ts2FillFloats(float *p, int n, float v, void *stream)
{
    hipLaunchKernelGGL(FillFloatsKernel, dim3((n + 255) / 256), dim3(256), 0, STREAM, p, n, v);
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

int Ts2ZeroRows(const ts2_mat *m, int rows, int rowBytes, void *stream)
{
    hipLaunchKernelGGL(ZeroBytes, dim3(rows), dim3(256), 0, STREAM, (uint8_t *)m->ptr, m->strideBytes, rowBytes);
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}
