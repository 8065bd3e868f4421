// Bandwidth-bound fused gradient kernels (tile norm forward/backward + residual add, dynamic gradient scaling, gated sigmoid
// forward/backward, per-row and per-k-tile int8 quantisation, 8-bit transposes).
//
// Mapping for gfx950: one 128-wide tile is held by 32 lanes x 4 elements, so a 64-wide wavefront processes two tiles per
// instruction with 16-byte (fp32), 8-byte (bf16) or 4-byte (8-bit) accesses per lane; reductions stay inside the 32-lane group
// (5 cross-lane steps).  Workgroups are 256 threads (8 tiles in flight) and grids cover every (row, tile) once, so each launch puts
// thousands of workgroups on the 256 CUs; consecutive 32-lane groups walk consecutive tiles of a row, i.e. HBM accesses are fully
// coalesced 512-byte (fp32) runs.  The reference launches one 32-thread block per (tile, row) (src/lib/cuda/cuda_graph.cuh:359-365).
#include "vec.h"
#include "internal.h"

namespace
{
struct Mat {
    uint8_t *p;
    int64_t ld;
};

__host__ __device__ __forceinline__ Mat M(const ts2_mat &m)
{
    Mat r = {(uint8_t *)m.ptr, m.strideBytes};
    return r;
}

template <class TT> __device__ __forceinline__ void *At(const Mat &m, int row, int col)
{
    return m.p + (int64_t)row * m.ld + (int64_t)col * TT::SIZE;
}

__device__ __forceinline__ float &ScaleAt(const Mat &m, int tile, int row)
{
    return *(float *)(m.p + (int64_t)tile * m.ld + (int64_t)row * 4);
}

// Every 32-lane group owns U consecutive rows of one tile column and issues the loads of all U rows before it touches any of them:
// with one row per group a wave has a single 4-16 byte load per lane in flight and the kernels sit at 30-50 % of what a copy reaches.
constexpr int U = 4;

// first row and tile of this 32-lane group; returns false when the whole group is out of range
__device__ __forceinline__ bool Unit(int rows, int tiles, int *row0, int *tile, int *lane32)
{
    long u = ((long)blockIdx.x * blockDim.x + threadIdx.x) >> 5;
    *lane32 = threadIdx.x & 31;
    long rb = u / tiles;
    *tile = (int)(u - rb * tiles);
    *row0 = (int)(rb * U);
    return *row0 < rows;
}

inline dim3 GridFor(int rows, int tiles)
{
    long units = (long)((rows + U - 1) / U) * tiles;
    return dim3((unsigned)((units * 32 + 255) / 256));
}

// non-negative float max through the integer ordering, like the reference's atomicMax((int*)p, __float_as_int(x))
__device__ __forceinline__ void AtomicMaxPos(float *p, float v)
{
    atomicMax((int *)p, __float_as_int(v));
}

// lanes 0..U-1 of the group store the U per-row scalars of one tile column (16 contiguous bytes)
__device__ __forceinline__ void StoreScales(const Mat &m, int tile, int row0, int rows, int h, const float (&v)[U])
{
    float mine = 0;
#pragma unroll
    for (int k = 0; k < U; ++k) {
        mine = h == k ? v[k] : mine;
    }
    if (h < U && row0 + h < rows) {
        ScaleAt(m, tile, row0 + h) = mine;
    }
}

// --------------------------------------------------------------------------------------------------------------------------
template <class TSrc, class TDst>
__global__ void __launch_bounds__(256) LayerNormalizeStateVecs(int len, int lenRound, int tiles, float vecScale, Mat state, Mat normState, Mat normScale)
{
    int t0, tile, h;
    if (!Unit(lenRound, tiles, &t0, &tile, &h)) {
        return;
    }
    int col = tile * TILE + h * 4;
    F4 v[U];
    float discr[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
        v[k] = t0 + k < len ? Load4<TSrc>(At<TSrc>(state, t0 + k, col)) : ZeroF4();
    }
#pragma unroll
    for (int k = 0; k < U; ++k) {
        discr[k] = 0;
        float sum2 = Half32Sum(HSum(v[k] * v[k]));
        if (sum2 > 0) {
            discr[k] = sqrtf(sum2 / TILE) * vecScale;
            v[k] = v[k] * (1 / discr[k]);
        }
        if (t0 + k < lenRound) {
            Store4<TDst>(At<TDst>(normState, t0 + k, col), v[k]);
        }
    }
    StoreScales(normScale, tile, t0, lenRound, h, discr);
}

// Every workgroup walks many units and issues ONE atomic max at the end: one atomic per unit (the reference's scheme,
// gpu_layer_norm.cuh:111-114) serialises half a million updates of a single address at this problem size.
template <class TNorm, class TFast, bool FINAL>
__global__ void __launch_bounds__(256) BackpropLayerNormalize(int len, int rows, int tiles, Mat normState, Mat stateScale, Mat dNormState,
    const float *combinerScale, const float *gradScale, const float *gradMult, Mat stateGrad, Mat stateGradFast, float *nextMaxNorm)
{
    __shared__ float red[8];
    const int h = threadIdx.x & 31;
    const long units = (long)((rows + U - 1) / U) * tiles;
    float s = 1;
    if (!FINAL) {
        if (combinerScale) {
            s *= *combinerScale;
        }
        if (gradScale) {
            s *= *gradScale;
        }
    }
    const float gm = (!FINAL && gradMult) ? *gradMult : 1.f;
    float gmax = 0;
    for (long u = ((long)blockIdx.x * 256 + threadIdx.x) >> 5; u < units; u += (long)gridDim.x * 8) {
        long rb = u / tiles;
        int tile = (int)(u - rb * tiles);
        int t0 = (int)rb * U;
        int col = tile * TILE + h * 4;
        F4 vec[U], grad[U], prev[U];
        float sc[U];
#pragma unroll
        for (int k = 0; k < U; ++k) {
            int t = t0 + k;
            bool live = t < len;
            vec[k] = live ? Load4<TNorm>(At<TNorm>(normState, t, col)) : ZeroF4();
            grad[k] = live ? Load4<TF32>(At<TF32>(dNormState, t, col)) : ZeroF4();
            prev[k] = (live && !FINAL) ? Load4<TF32>(At<TF32>(stateGrad, t, col)) : ZeroF4();
            sc[k] = live ? ScaleAt(stateScale, tile, t) : 0.f;
        }
#pragma unroll
        for (int k = 0; k < U; ++k) {
            int t = t0 + k;
            if (t >= rows) {
                continue;
            }
            F4 g = ZeroF4();
            if (t < len) {
                g = FINAL ? grad[k] : grad[k] * s;
                g = TileNormBackprop(vec[k] * sc[k], g);
                if (!FINAL) {
                    g = g + prev[k];
                }
                gmax = fmaxf(gmax, HMaxAbs(g));
            }
            Store4<TF32>(At<TF32>(stateGrad, t, col), g);
            Store4<TFast>(At<TFast>(stateGradFast, t, col), g * gm);
        }
    }
    gmax = Half32Max(gmax);
    if (h == 0) {
        red[threadIdx.x >> 5] = gmax;
    }
    __syncthreads();
    if (threadIdx.x == 0 && nextMaxNorm) {
        float m = fmaxf(fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])), fmaxf(fmaxf(red[4], red[5]), fmaxf(red[6], red[7])));
        AtomicMaxPos(nextMaxNorm, m);
    }
}

// e4m3 norm state and e4m3 fast gradient with eight elements per lane (a tile = 16 lanes, 16-byte accesses to the fp32 arrays): the
// form the fp8 model runs.  Same arithmetic per element as BackpropLayerNormalize; Row16Sum is defined with the 8-wide LoLU kernel.
__device__ __forceinline__ float Row16SumFwd(float v);

template <bool FINAL>
__global__ void __launch_bounds__(256) BackpropLayerNormalize8(int len, int rows, int tiles, Mat normState, Mat stateScale, Mat dNormState,
    const float *combinerScale, const float *gradScale, const float *gradMult, Mat stateGrad, Mat stateGradFast, float *nextMaxNorm)
{
    __shared__ float red[4];
    const int l16 = threadIdx.x & 15;
    const long units = (long)rows * tiles;
    float s = 1;
    if (!FINAL) {
        if (combinerScale) {
            s *= *combinerScale;
        }
        if (gradScale) {
            s *= *gradScale;
        }
    }
    const float gm = (!FINAL && gradMult) ? *gradMult : 1.f;
    float gmax = 0;
    // every lane of a wave takes part in every iteration (the reductions are cross-lane): the loop bound is wave-uniform
    const long unitFirst = ((long)blockIdx.x * 256 + (threadIdx.x & ~63)) >> 4;
    for (long ub = unitFirst; ub < units; ub += (long)gridDim.x * 16) {
        const long u = ub + ((threadIdx.x & 63) >> 4);
        const bool any = u < units;
        const int t = any ? (int)(u / tiles) : 0;
        const int tile = any ? (int)(u - (long)t * tiles) : 0;
        const int col = tile * TILE + l16 * 8;
        const bool live = any && t < len;
        uint2 nv = live ? *(const uint2 *)At<TE4M3>(normState, t, col) : make_uint2(0, 0);
        F4 g0 = live ? Load4<TF32>(At<TF32>(dNormState, t, col)) : ZeroF4();
        F4 g1 = live ? Load4<TF32>(At<TF32>(dNormState, t, col + 4)) : ZeroF4();
        F4 p0 = (live && !FINAL) ? Load4<TF32>(At<TF32>(stateGrad, t, col)) : ZeroF4();
        F4 p1 = (live && !FINAL) ? Load4<TF32>(At<TF32>(stateGrad, t, col + 4)) : ZeroF4();
        const float sc = live ? ScaleAt(stateScale, tile, t) : 0.f;
        float src[8], g[8];
        const float nf[8] = {__builtin_amdgcn_cvt_f32_fp8((int)nv.x, 0), __builtin_amdgcn_cvt_f32_fp8((int)nv.x, 1), __builtin_amdgcn_cvt_f32_fp8((int)nv.x, 2),
            __builtin_amdgcn_cvt_f32_fp8((int)nv.x, 3), __builtin_amdgcn_cvt_f32_fp8((int)nv.y, 0), __builtin_amdgcn_cvt_f32_fp8((int)nv.y, 1),
            __builtin_amdgcn_cvt_f32_fp8((int)nv.y, 2), __builtin_amdgcn_cvt_f32_fp8((int)nv.y, 3)};
        const float gin[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
        const float prev[8] = {p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w};
        float sum2 = 0, dp = 0;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            src[e] = nf[e] * sc;
            g[e] = FINAL ? gin[e] : gin[e] * s;
            sum2 += src[e] * src[e];
            dp += src[e] * g[e];
        }
        sum2 = Row16SumFwd(sum2);
        dp = Row16SumFwd(dp);
        if (!any) {
            continue;
        }
        float sigma = 0, scale = 0;
        if (sum2 != 0) {
            float inv = 1 / sum2;
            sigma = dp * inv;
            scale = sqrtf(TILE * inv);
        }
        float out[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            float x = 0;
            if (live) {
                x = sum2 != 0 ? (g[e] - src[e] * sigma) * scale : 0.f;
                if (!FINAL) {
                    x += prev[e];
                }
                gmax = fmaxf(gmax, fabsf(x));
            }
            out[e] = x;
        }
        Store4<TF32>(At<TF32>(stateGrad, t, col), MakeF4(out[0], out[1], out[2], out[3]));
        Store4<TF32>(At<TF32>(stateGrad, t, col + 4), MakeF4(out[4], out[5], out[6], out[7]));
        uint32_t lo = CvtPkE4m3(out[0] * gm, out[1] * gm) | (CvtPkE4m3(out[2] * gm, out[3] * gm) << 16);
        uint32_t hi = CvtPkE4m3(out[4] * gm, out[5] * gm) | (CvtPkE4m3(out[6] * gm, out[7] * gm) << 16);
        *(uint2 *)At<TE4M3>(stateGradFast, t, col) = make_uint2(lo, hi);
    }
    gmax = WaveMax(gmax);
    if ((threadIdx.x & 63) == 0) {
        red[threadIdx.x >> 6] = gmax;
    }
    __syncthreads();
    if (threadIdx.x == 0 && nextMaxNorm) {
        AtomicMaxPos(nextMaxNorm, fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])));
    }
}

__device__ __forceinline__ float ComputeGradMult(float gradMaxNorm)
{
    if (gradMaxNorm == 0) {
        return 1;
    }
    return __uint_as_float(__float_as_uint(128.f / gradMaxNorm) & 0xff800000u);
}

template <class TFast>
__global__ void __launch_bounds__(256) ScaleGrad(int len, int tiles, const float *gradMaxNorm, const float *prevGradMult, Mat grad, Mat gradFast,
    float *gradScaleOut, float *gradMultOut)
{
    int t0, tile, h;
    float gradMult = ComputeGradMult(*gradMaxNorm);
    bool rewrite = !prevGradMult || gradMult != *prevGradMult;
    if (Unit(len, tiles, &t0, &tile, &h) && rewrite) {
        int col = tile * TILE + h * 4;
        F4 v[U];
#pragma unroll
        for (int k = 0; k < U; ++k) {
            v[k] = t0 + k < len ? Load4<TF32>(At<TF32>(grad, t0 + k, col)) : ZeroF4();
        }
#pragma unroll
        for (int k = 0; k < U; ++k) {
            if (t0 + k < len) {
                Store4<TFast>(At<TFast>(gradFast, t0 + k, col), v[k] * gradMult);
            }
        }
    }
}

// published after the rewrite kernel so that a caller may pass the same cell as prevGradMult and gradMultOut
__global__ void PublishGradMult(const float *gradMaxNorm, float *gradScaleOut, float *gradMultOut)
{
    float gradMult = ComputeGradMult(*gradMaxNorm);
    if (gradScaleOut) {
        *gradScaleOut = 1 / gradMult;
    }
    if (gradMultOut) {
        *gradMultOut = gradMult;
    }
}

template <class TDst>
__global__ void __launch_bounds__(256) MatrixLoLU(int len, int lenRound, int tiles, Mat gate, Mat vals, float resMult, Mat res)
{
    int t0, tile, h;
    if (!Unit(lenRound, tiles, &t0, &tile, &h)) {
        return;
    }
    int col = tile * TILE + h * 4;
    F4 g[U], v[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
        bool live = t0 + k < len;
        g[k] = live ? Load4<TBF16>(At<TBF16>(gate, t0 + k, col)) : ZeroF4();
        v[k] = live ? Load4<TBF16>(At<TBF16>(vals, t0 + k, col)) : ZeroF4();
    }
#pragma unroll
    for (int k = 0; k < U; ++k) {
        if (t0 + k < lenRound) {
            Store4<TDst>(At<TDst>(res, t0 + k, col), t0 + k < len ? v[k] * LoLU4(g[k]) * resMult : ZeroF4());
        }
    }
}

// The e4m3 result from bf16 inputs with eight elements per lane (16-byte loads, 8-byte stores; no reduction in this kernel, so the
// tile structure does not matter): the form the model's FFN and attention forward use.  Two row segments per lane in flight.
__global__ void __launch_bounds__(256) MatrixLoLU8(int len, int lenRound, int dim8, Mat gate, Mat vals, float resMult, Mat res)
{
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    const long total = (long)lenRound * dim8;
    const long stride = (long)gridDim.x * 256;
    uint4 g[2], v[2];
    long id[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        id[k] = idx + k * stride;
        const int t = (int)(id[k] / dim8), c = (int)(id[k] - (long)t * dim8) * 8;
        const bool live = id[k] < total && t < len;
        g[k] = live ? *(const uint4 *)At<TBF16>(gate, t, c) : make_uint4(0, 0, 0, 0);
        v[k] = live ? *(const uint4 *)At<TBF16>(vals, t, c) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        if (id[k] >= total) {
            continue;
        }
        const int t = (int)(id[k] / dim8), c = (int)(id[k] - (long)t * dim8) * 8;
        const uint32_t gw[4] = {g[k].x, g[k].y, g[k].z, g[k].w}, vw[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
        uint32_t out[2] = {0, 0};
        if (t < len) {
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                float g0 = __uint_as_float(gw[w] << 16), g1 = __uint_as_float(gw[w] & 0xffff0000u);
                float v0 = __uint_as_float(vw[w] << 16), v1 = __uint_as_float(vw[w] & 0xffff0000u);
                out[w >> 1] |= CvtPkE4m3(v0 * LoLU1(g0) * resMult, v1 * LoLU1(g1) * resMult) << ((w & 1) * 16);
            }
        }
        *(uint2 *)At<TE4M3>(res, t, c) = make_uint2(out[0], out[1]);
    }
}

// Sixteen elements per lane: two 16-byte loads per input (the second is served by the line the first brought in) and one 16-byte store
__global__ void __launch_bounds__(256) MatrixLoLU16(int len, int lenRound, int dim16, Mat gate, Mat vals, float resMult, Mat res)
{
    const long id = (long)blockIdx.x * 256 + threadIdx.x;
    const long total = (long)lenRound * dim16;
    if (id >= total) {
        return;
    }
    const int t = (int)(id / dim16), c = (int)(id - (long)t * dim16) * 16;
    uint32_t out[4] = {0, 0, 0, 0};
    if (t < len) {
        const uint4 g0 = *(const uint4 *)At<TBF16>(gate, t, c), g1 = *(const uint4 *)At<TBF16>(gate, t, c + 8);
        const uint4 v0 = *(const uint4 *)At<TBF16>(vals, t, c), v1 = *(const uint4 *)At<TBF16>(vals, t, c + 8);
        const uint32_t gw[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w}, vw[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            float ga = __uint_as_float(gw[w] << 16), gb = __uint_as_float(gw[w] & 0xffff0000u);
            float va = __uint_as_float(vw[w] << 16), vb = __uint_as_float(vw[w] & 0xffff0000u);
            out[w >> 1] |= CvtPkE4m3(va * LoLU1(ga) * resMult, vb * LoLU1(gb) * resMult) << ((w & 1) * 16);
        }
    }
    *(uint4 *)At<TE4M3>(res, t, c) = make_uint4(out[0], out[1], out[2], out[3]);
}

// MODE 0: FFN (tile-norm backward of vals fused); MODE 1: attention (dScale fused)
template <class TGrad, class TOutG, class TOutV, int MODE>
__global__ void __launch_bounds__(256) BackpropLoLU(int len, int lenRound, int tiles, Mat gate, Mat vals, float valsScale, Mat valsSrcTileScale,
    Mat gradArr, Mat gradGate, Mat gradVals, Mat dScale)
{
    int t0, tile, h;
    if (!Unit(lenRound, tiles, &t0, &tile, &h)) {
        return;
    }
    int col = tile * TILE + h * 4;
    F4 g[U], v[U], grad[U];
    float ts[U], ds[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
        int t = t0 + k;
        bool live = t < len;
        g[k] = live ? Load4<TBF16>(At<TBF16>(gate, t, col)) : ZeroF4();
        v[k] = live ? Load4<TBF16>(At<TBF16>(vals, t, col)) : ZeroF4();
        grad[k] = live ? Load4<TGrad>(At<TGrad>(gradArr, t, col)) : ZeroF4();
        ts[k] = (MODE == 0 && live) ? ScaleAt(valsSrcTileScale, tile, t) : 0.f;
    }
#pragma unroll
    for (int k = 0; k < U; ++k) {
        int t = t0 + k;
        ds[k] = 0;
        if (t >= lenRound) {
            continue;
        }
        F4 resGate = ZeroF4(), resVals = ZeroF4();
        if (t < len) {
            F4 vv = v[k] * valsScale;
            F4 mult = LoLU4(g[k]);
            resGate = grad[k] * vv * LoLUGrad4(mult);
            resVals = grad[k] * mult;
            if (MODE == 0) {
                // un-normalised source = normalised * (tile scale / valsScale)
                F4 src = vv * (ts[k] / valsScale);
                resVals = TileNormBackprop(src, resVals);
            } else {
                ds[k] = Half32Sum(HSum(vv * resVals));
            }
        }
        Store4<TOutG>(At<TOutG>(gradGate, t, col), resGate);
        Store4<TOutV>(At<TOutV>(gradVals, t, col), resVals);
    }
    if (MODE == 1) {
        StoreScales(dScale, tile, t0, lenRound, h, ds);
    }
}

// The FFN flavour (MODE 0) for bf16 gradients and e4m3 results with eight elements per lane: a 128-wide tile is 16 lanes, so a wave
// holds four (row, tile) units, the tile sums are four DPP steps inside a row of 16 lanes, loads are 16 bytes and stores 8.  Two
// units per lane in flight.  Same arithmetic per element as BackpropLoLU<.., 0>.
__device__ __forceinline__ float Row16Sum(float v);
__device__ __forceinline__ float Row16SumFwd(float v)
{
    return Row16Sum(v);
}

__device__ __forceinline__ float Row16Sum(float v)
{
    v += LaneDpp<DPP_XOR1>(v);
    v += LaneDpp<DPP_XOR2>(v);
    v += LaneDpp<DPP_HALF_MIRROR>(v);
    v += LaneDpp<DPP_MIRROR>(v);
    return v;
}

__global__ void __launch_bounds__(256) BackpropLoLU8(int len, int lenRound, int tiles, Mat gate, Mat vals, float valsScale, Mat valsSrcTileScale,
    Mat gradArr, Mat gradGate, Mat gradVals)
{
    constexpr int UU = 2;
    const int l16 = threadIdx.x & 15;
    const long unit0 = ((long)blockIdx.x * 256 + threadIdx.x) >> 4; // (row, tile) units; consecutive units = consecutive tiles of a row
    const long units = (long)lenRound * tiles;
    const long stride = ((long)gridDim.x * 256) >> 4;
    uint4 g[UU], v[UU], gr[UU];
    float ts[UU];
    int row[UU], col[UU];
    bool any[UU], live[UU];
#pragma unroll
    for (int k = 0; k < UU; ++k) {
        long u = unit0 + k * stride;
        any[k] = u < units;
        row[k] = any[k] ? (int)(u / tiles) : 0;
        int tile = any[k] ? (int)(u - (long)row[k] * tiles) : 0;
        col[k] = tile * TILE + l16 * 8;
        live[k] = any[k] && row[k] < len;
        g[k] = live[k] ? *(const uint4 *)At<TBF16>(gate, row[k], col[k]) : make_uint4(0, 0, 0, 0);
        v[k] = live[k] ? *(const uint4 *)At<TBF16>(vals, row[k], col[k]) : make_uint4(0, 0, 0, 0);
        gr[k] = live[k] ? *(const uint4 *)At<TBF16>(gradArr, row[k], col[k]) : make_uint4(0, 0, 0, 0);
        ts[k] = live[k] ? ScaleAt(valsSrcTileScale, tile, row[k]) : 0.f;
    }
#pragma unroll
    for (int k = 0; k < UU; ++k) {
        const uint32_t gw[4] = {g[k].x, g[k].y, g[k].z, g[k].w}, vw[4] = {v[k].x, v[k].y, v[k].z, v[k].w}, rw[4] = {gr[k].x, gr[k].y, gr[k].z, gr[k].w};
        float resGate[8], resVals[8], src[8];
        float sum2 = 0, dp = 0;
        const float srcMult = ts[k] / valsScale;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint32_t sh = (e & 1) ? 0xffff0000u : 0u;
            float ge = (e & 1) ? __uint_as_float(gw[e >> 1] & sh) : __uint_as_float(gw[e >> 1] << 16);
            float ve = (e & 1) ? __uint_as_float(vw[e >> 1] & sh) : __uint_as_float(vw[e >> 1] << 16);
            float de = (e & 1) ? __uint_as_float(rw[e >> 1] & sh) : __uint_as_float(rw[e >> 1] << 16);
            float vv = ve * valsScale;
            float mult = LoLU1(ge);
            resGate[e] = de * vv * (mult * (1 - mult) * 2.f);
            resVals[e] = de * mult;
            // un-normalised source = normalised * (tile scale / valsScale)
            src[e] = vv * srcMult;
            sum2 += src[e] * src[e];
            dp += src[e] * resVals[e];
        }
        sum2 = Row16Sum(sum2);
        dp = Row16Sum(dp);
        if (!any[k]) {
            continue;
        }
        uint32_t og[2] = {0, 0}, ov[2] = {0, 0};
        if (live[k]) {
            float sigma = 0, scale = 0;
            if (sum2 != 0) {
                float inv = 1 / sum2;
                sigma = dp * inv;
                scale = sqrtf(TILE * inv);
            }
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                float a0 = sum2 != 0 ? (resVals[2 * w] - src[2 * w] * sigma) * scale : 0.f;
                float a1 = sum2 != 0 ? (resVals[2 * w + 1] - src[2 * w + 1] * sigma) * scale : 0.f;
                ov[w >> 1] |= CvtPkE4m3(a0, a1) << ((w & 1) * 16);
                og[w >> 1] |= CvtPkE4m3(resGate[2 * w], resGate[2 * w + 1]) << ((w & 1) * 16);
            }
        }
        *(uint2 *)At<TE4M3>(gradGate, row[k], col[k]) = make_uint2(og[0], og[1]);
        *(uint2 *)At<TE4M3>(gradVals, row[k], col[k]) = make_uint2(ov[0], ov[1]);
    }
}

// A 128 x 128 block of bytes staged in LDS as [t][x] (pitch PITCH) goes out transposed: dst[x][t], 16 bytes (16 t) per store.
// thread -> (tq = block of 16 t, xq = x quad)
template <int PITCH> __device__ __forceinline__ void TransposeOut128(const uint8_t *buf, const Mat &dst, int xBlock, int tBlock, int tid)
{
    const int tq = tid & 7, xq = tid >> 3;
    uint32_t out[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint8_t *b = buf + (tq * 16 + j * 4) * PITCH + xq * 4;
        uint32_t r0 = *(const uint32_t *)(b);
        uint32_t r1 = *(const uint32_t *)(b + PITCH);
        uint32_t r2 = *(const uint32_t *)(b + 2 * PITCH);
        uint32_t r3 = *(const uint32_t *)(b + 3 * PITCH);
        // 4x4 byte transpose.  __builtin_amdgcn_perm(hi, lo, sel): result byte i = byte sel[i] of {hi:lo} (lo = bytes 0-3)
        uint32_t a = __builtin_amdgcn_perm(r1, r0, 0x05010400); // r0.b0 r1.b0 r0.b1 r1.b1
        uint32_t bb = __builtin_amdgcn_perm(r1, r0, 0x07030602); // r0.b2 r1.b2 r0.b3 r1.b3
        uint32_t c = __builtin_amdgcn_perm(r3, r2, 0x05010400);
        uint32_t d = __builtin_amdgcn_perm(r3, r2, 0x07030602);
        out[0][j] = __builtin_amdgcn_perm(c, a, 0x05040100); // column 0: r0.b0 r1.b0 r2.b0 r3.b0
        out[1][j] = __builtin_amdgcn_perm(c, a, 0x07060302);
        out[2][j] = __builtin_amdgcn_perm(d, bb, 0x05040100);
        out[3][j] = __builtin_amdgcn_perm(d, bb, 0x07060302);
    }
    int x = xBlock + xq * 4;
    int tcol = tBlock + tq * 16;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        *(uint4 *)(dst.p + (int64_t)(x + i) * dst.ld + tcol) = make_uint4(out[i][0], out[i][1], out[i][2], out[i][3]);
    }
}

// BackpropLoLU8 that also leaves the transposed copies of both results (gradGateT, gradValsT: [dim][lenRound]) which the delta
// products of the two matrices contract over: a workgroup takes a block of 128 rows x one tile, computes it 16 rows at a time with
// the arithmetic of BackpropLoLU8, stores the row-major bytes and stages them in LDS for the transposed stores.  Saves reading both
// results back for their transposes.
__global__ void __launch_bounds__(256) BackpropLoLU8T(int len, int lenRound, Mat gate, Mat vals, float valsScale, Mat valsSrcTileScale, Mat gradArr,
    Mat gradGate, Mat gradVals, Mat gradGateT, Mat gradValsT)
{
    constexpr int PITCH = 132;
    __shared__ __attribute__((aligned(16))) uint8_t bufG[128 * PITCH], bufV[128 * PITCH];
    const int tid = threadIdx.x, l16 = tid & 15, lr = tid >> 4;
    const int tile = blockIdx.x, tBlock = blockIdx.y * 128;
    const int col = tile * TILE + l16 * 8;
    for (int r0 = 0; r0 < 128; r0 += 64) {
        uint4 g[4], v[4], gr[4];
        float ts[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int row = tBlock + r0 + k * 16 + lr;
            const bool live = row < len;
            g[k] = live ? *(const uint4 *)At<TBF16>(gate, row, col) : make_uint4(0, 0, 0, 0);
            v[k] = live ? *(const uint4 *)At<TBF16>(vals, row, col) : make_uint4(0, 0, 0, 0);
            gr[k] = live ? *(const uint4 *)At<TBF16>(gradArr, row, col) : make_uint4(0, 0, 0, 0);
            ts[k] = live ? ScaleAt(valsSrcTileScale, tile, row) : 0.f;
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int r = r0 + k * 16 + lr, row = tBlock + r;
            const uint32_t gw[4] = {g[k].x, g[k].y, g[k].z, g[k].w}, vw[4] = {v[k].x, v[k].y, v[k].z, v[k].w}, rw[4] = {gr[k].x, gr[k].y, gr[k].z, gr[k].w};
            float resGate[8], resVals[8], src[8];
            float sum2 = 0, dp = 0;
            const float srcMult = ts[k] / valsScale;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t sh = 0xffff0000u;
                float ge = (e & 1) ? __uint_as_float(gw[e >> 1] & sh) : __uint_as_float(gw[e >> 1] << 16);
                float ve = (e & 1) ? __uint_as_float(vw[e >> 1] & sh) : __uint_as_float(vw[e >> 1] << 16);
                float de = (e & 1) ? __uint_as_float(rw[e >> 1] & sh) : __uint_as_float(rw[e >> 1] << 16);
                float vv = ve * valsScale;
                float mult = LoLU1(ge);
                resGate[e] = de * vv * (mult * (1 - mult) * 2.f);
                resVals[e] = de * mult;
                src[e] = vv * srcMult;
                sum2 += src[e] * src[e];
                dp += src[e] * resVals[e];
            }
            sum2 = Row16Sum(sum2);
            dp = Row16Sum(dp);
            uint32_t og[2] = {0, 0}, ov[2] = {0, 0};
            if (row < len) {
                float sigma = 0, scale = 0;
                if (sum2 != 0) {
                    float inv = 1 / sum2;
                    sigma = dp * inv;
                    scale = sqrtf(TILE * inv);
                }
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    float a0 = sum2 != 0 ? (resVals[2 * w] - src[2 * w] * sigma) * scale : 0.f;
                    float a1 = sum2 != 0 ? (resVals[2 * w + 1] - src[2 * w + 1] * sigma) * scale : 0.f;
                    ov[w >> 1] |= CvtPkE4m3(a0, a1) << ((w & 1) * 16);
                    og[w >> 1] |= CvtPkE4m3(resGate[2 * w], resGate[2 * w + 1]) << ((w & 1) * 16);
                }
            }
            *(uint2 *)At<TE4M3>(gradGate, row, col) = make_uint2(og[0], og[1]);
            *(uint2 *)At<TE4M3>(gradVals, row, col) = make_uint2(ov[0], ov[1]);
            *(uint32_t *)(bufG + r * PITCH + l16 * 8) = og[0];
            *(uint32_t *)(bufG + r * PITCH + l16 * 8 + 4) = og[1];
            *(uint32_t *)(bufV + r * PITCH + l16 * 8) = ov[0];
            *(uint32_t *)(bufV + r * PITCH + l16 * 8 + 4) = ov[1];
        }
    }
    __syncthreads();
    TransposeOut128<PITCH>(bufG, gradGateT, tile * TILE, tBlock, tid);
    TransposeOut128<PITCH>(bufV, gradValsT, tile * TILE, tBlock, tid);
}

// The attention flavour (MODE 1) with eight elements per lane: bf16 gate, values and gradient in, e4m3 gate gradient and bf16 value
// gradient out, and the per-(head, row) sum <values, value gradient> that the attention backward subtracts (dScale).
__global__ void __launch_bounds__(256) BackpropLoLUAtt8(int len, int lenRound, int tiles, Mat gate, Mat vals, float valsScale, Mat gradArr,
    Mat gradGate, Mat gradVals, Mat dScale)
{
    constexpr int UU = 2;
    const int l16 = threadIdx.x & 15;
    const long unit0 = ((long)blockIdx.x * 256 + threadIdx.x) >> 4; // (row, tile) units; consecutive units = consecutive tiles of a row
    const long units = (long)lenRound * tiles;
    const long stride = ((long)gridDim.x * 256) >> 4;
    uint4 g[UU], v[UU], gr[UU];
    int row[UU], tile[UU];
    bool any[UU], live[UU];
#pragma unroll
    for (int k = 0; k < UU; ++k) {
        long u = unit0 + k * stride;
        any[k] = u < units;
        row[k] = any[k] ? (int)(u / tiles) : 0;
        tile[k] = any[k] ? (int)(u - (long)row[k] * tiles) : 0;
        const int col = tile[k] * TILE + l16 * 8;
        live[k] = any[k] && row[k] < len;
        g[k] = live[k] ? *(const uint4 *)At<TBF16>(gate, row[k], col) : make_uint4(0, 0, 0, 0);
        v[k] = live[k] ? *(const uint4 *)At<TBF16>(vals, row[k], col) : make_uint4(0, 0, 0, 0);
        gr[k] = live[k] ? *(const uint4 *)At<TBF16>(gradArr, row[k], col) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int k = 0; k < UU; ++k) {
        const uint32_t gw[4] = {g[k].x, g[k].y, g[k].z, g[k].w}, vw[4] = {v[k].x, v[k].y, v[k].z, v[k].w}, rw[4] = {gr[k].x, gr[k].y, gr[k].z, gr[k].w};
        float resGate[8], resVals[8];
        float dp = 0;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint32_t sh = 0xffff0000u;
            float ge = (e & 1) ? __uint_as_float(gw[e >> 1] & sh) : __uint_as_float(gw[e >> 1] << 16);
            float ve = (e & 1) ? __uint_as_float(vw[e >> 1] & sh) : __uint_as_float(vw[e >> 1] << 16);
            float de = (e & 1) ? __uint_as_float(rw[e >> 1] & sh) : __uint_as_float(rw[e >> 1] << 16);
            float vv = ve * valsScale;
            float mult = LoLU1(ge);
            resGate[e] = de * vv * (mult * (1 - mult) * 2.f);
            resVals[e] = de * mult;
            dp += vv * resVals[e];
        }
        dp = Row16Sum(dp); // zero for rows past len: their inputs were read as zero
        if (!any[k]) {
            continue;
        }
        const int col = tile[k] * TILE + l16 * 8;
        uint32_t og[2] = {0, 0}, ov[4] = {0, 0, 0, 0};
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            og[w >> 1] |= CvtPkE4m3(resGate[2 * w], resGate[2 * w + 1]) << ((w & 1) * 16);
            ov[w] = PackBf16x2(resVals[2 * w], resVals[2 * w + 1]);
        }
        *(uint2 *)At<TE4M3>(gradGate, row[k], col) = make_uint2(og[0], og[1]);
        *(uint4 *)At<TBF16>(gradVals, row[k], col) = make_uint4(ov[0], ov[1], ov[2], ov[3]);
        if (l16 == 0) {
            ScaleAt(dScale, tile[k], row[k]) = dp;
        }
    }
}

// Workgroups walk rows with a grid stride; a row stays in registers between the abs-max pass and the quantise pass when it has at
// most 4096 elements (REG) and the next row is fetched before the current one is reduced, so a workgroup always has loads in
// flight.  Longer rows are read twice (the second read is served by L2).
template <class TSrc, bool REG>
__global__ void __launch_bounds__(256) NormalizeVecsRowMax(int len, int lenRound, int dim, Mat src, const float *colScale, Mat dst, float *rowScale,
    float *rowAbsMax, uint32_t seed)
{
    __shared__ float red[2][4], redPlain[2][4];
    const int tid = threadIdx.x;
    F4 next[4];
    auto fetch = [&](int t) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int col = tid * 4 + i * 1024;
            next[i] = (REG && t < len && col < dim) ? Load4<TSrc>(At<TSrc>(src, t, col)) : ZeroF4();
        }
    };
    fetch(blockIdx.x);
    int phase = 0;
    for (int t = blockIdx.x; t < lenRound; t += gridDim.x, phase ^= 1) {
        if (t >= len) {
            for (int col = tid * 4; col < dim; col += 1024) {
                *(uint32_t *)At<TI8>(dst, t, col) = 0;
            }
            if (tid == 0) {
                rowScale[t] = 0;
                if (rowAbsMax) {
                    rowAbsMax[t] = 0;
                }
            }
            continue;
        }
        float mx = 0, plain = 0; // plain: abs-max of the row before the column scales (what the delta's k-tile scale is built from)
        F4 keep[4];
        if (REG) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                keep[i] = next[i];
            }
            fetch(t + gridDim.x);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                plain = fmaxf(plain, HMaxAbs(keep[i]));
            }
            if (colScale) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    int col = tid * 4 + i * 1024;
                    if (col < dim) {
                        keep[i] = keep[i] * Load4<TF32>(colScale + col);
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                mx = fmaxf(mx, HMaxAbs(keep[i]));
            }
        } else {
            for (int col = tid * 4; col < dim; col += 1024) {
                F4 v = Load4<TSrc>(At<TSrc>(src, t, col));
                plain = fmaxf(plain, HMaxAbs(v));
                if (colScale) {
                    v = v * Load4<TF32>(colScale + col);
                }
                mx = fmaxf(mx, HMaxAbs(v));
            }
        }
        mx = WaveMax(mx);
        plain = WaveMax(plain);
        if ((tid & 63) == 0) {
            red[phase][tid >> 6] = mx;
            redPlain[phase][tid >> 6] = plain;
        }
        __syncthreads(); // the two phases of the exchange arrays make one barrier per row enough
        mx = fmaxf(fmaxf(red[phase][0], red[phase][1]), fmaxf(red[phase][2], red[phase][3]));
        if (tid == 0 && rowAbsMax) {
            rowAbsMax[t] = fmaxf(fmaxf(redPlain[phase][0], redPlain[phase][1]), fmaxf(redPlain[phase][2], redPlain[phase][3]));
        }
        float discr = 0, mult = 0;
        if (mx > 0) {
            discr = mx / 127;
            mult = 1 / discr;
        }
        if (REG) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                int col = tid * 4 + i * 1024;
                if (col < dim) {
                    if (seed) {
                        *(uint32_t *)At<TI8>(dst, t, col) = QuantDither4(keep[i].x, keep[i].y, keep[i].z, keep[i].w, mult, DitherWord(seed, t, col >> 2));
                    } else {
                        Store4<TI8>(At<TI8>(dst, t, col), keep[i] * mult);
                    }
                }
            }
        } else {
            for (int col = tid * 4; col < dim; col += 1024) {
                F4 v = Load4<TSrc>(At<TSrc>(src, t, col));
                if (colScale) {
                    v = v * Load4<TF32>(colScale + col);
                }
                if (seed) {
                    *(uint32_t *)At<TI8>(dst, t, col) = QuantDither4(v.x, v.y, v.z, v.w, mult, DitherWord(seed, t, col >> 2));
                } else {
                    Store4<TI8>(At<TI8>(dst, t, col), v * mult);
                }
            }
        }
        if (tid == 0) {
            rowScale[t] = discr;
        }
    }
}

// The same quantiser with one wave per row for bf16 rows of NCH * 512 elements (at most 4096): a lane holds NCH chunks of 8
// consecutive elements (16-byte loads, 8-byte stores, each instruction of the wave covering 1 KB / 512 B of the row), the row
// maxima are wave reductions, and no workgroup barrier or LDS exchange is left.  Same arithmetic per element as NormalizeVecsRowMax.
template <int NCH>
__global__ void __launch_bounds__(256) NormalizeRowsWave(int len, int lenRound, Mat src, const float *colScale, Mat dst, float *rowScale, float *rowAbsMax,
    uint32_t seed)
{
    const int lane = threadIdx.x & 63;
    const int nWaves = gridDim.x * 4;
    // the column scales of the lane's chunks stay in registers for all the rows the wave walks
    F4 cs[NCH][2];
    if (colScale) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            cs[i][0] = Load4<TF32>(colScale + (i * 64 + lane) * 8);
            cs[i][1] = Load4<TF32>(colScale + (i * 64 + lane) * 8 + 4);
        }
    }
    for (int t = blockIdx.x * 4 + (threadIdx.x >> 6); t < lenRound; t += nWaves) {
        uint8_t *out = dst.p + (int64_t)t * dst.ld;
        if (t >= len) {
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                *(uint2 *)(out + (i * 64 + lane) * 8) = make_uint2(0u, 0u);
            }
            if (lane == 0) {
                rowScale[t] = 0;
                if (rowAbsMax) {
                    rowAbsMax[t] = 0;
                }
            }
            continue;
        }
        const uint8_t *in = src.p + (int64_t)t * src.ld;
        uint4 raw[NCH];
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            raw[i] = *(const uint4 *)(in + (i * 64 + lane) * 16);
        }
        F4 v[NCH][2];
        float mx = 0, plain = 0;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            v[i][0] = MakeF4(__uint_as_float(raw[i].x << 16), __uint_as_float(raw[i].x & 0xffff0000u), __uint_as_float(raw[i].y << 16),
                __uint_as_float(raw[i].y & 0xffff0000u));
            v[i][1] = MakeF4(__uint_as_float(raw[i].z << 16), __uint_as_float(raw[i].z & 0xffff0000u), __uint_as_float(raw[i].w << 16),
                __uint_as_float(raw[i].w & 0xffff0000u));
            plain = fmaxf(plain, fmaxf(HMaxAbs(v[i][0]), HMaxAbs(v[i][1])));
            if (colScale) {
                v[i][0] = v[i][0] * cs[i][0];
                v[i][1] = v[i][1] * cs[i][1];
            }
            mx = fmaxf(mx, fmaxf(HMaxAbs(v[i][0]), HMaxAbs(v[i][1])));
        }
        mx = WaveMax(mx);
        plain = WaveMax(plain);
        float discr = 0, mult = 0;
        if (mx > 0) {
            discr = mx / 127;
            mult = 1 / discr;
        }
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            if (seed) {
                const int col4 = (i * 64 + lane) * 2;
                *(uint2 *)(out + (i * 64 + lane) * 8) =
                    make_uint2(QuantDither4(v[i][0].x, v[i][0].y, v[i][0].z, v[i][0].w, mult, DitherWord(seed, t, col4)),
                        QuantDither4(v[i][1].x, v[i][1].y, v[i][1].z, v[i][1].w, mult, DitherWord(seed, t, col4 + 1)));
                continue;
            }
            F4 a = v[i][0] * mult, b = v[i][1] * mult;
            uint32_t lo = (uint32_t)(CvtToI8(a.x) & 0xff) | ((uint32_t)(CvtToI8(a.y) & 0xff) << 8) | ((uint32_t)(CvtToI8(a.z) & 0xff) << 16) |
                          ((uint32_t)(CvtToI8(a.w) & 0xff) << 24);
            uint32_t hi = (uint32_t)(CvtToI8(b.x) & 0xff) | ((uint32_t)(CvtToI8(b.y) & 0xff) << 8) | ((uint32_t)(CvtToI8(b.z) & 0xff) << 16) |
                          ((uint32_t)(CvtToI8(b.w) & 0xff) << 24);
            *(uint2 *)(out + (i * 64 + lane) * 8) = make_uint2(lo, hi);
        }
        if (lane == 0) {
            rowScale[t] = discr;
            if (rowAbsMax) {
                rowAbsMax[t] = plain;
            }
        }
    }
}

__global__ void FillFloats(float *p, int n, float v)
{
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        p[i] = v;
    }
}

// tileMax[kt] = max over the k-tile's rows of rowAbsMax[t] * |rowMult[t]|: the k-tile abs-max when the row maxima are already known
__global__ void __launch_bounds__(256) TileMaxFromRows(int len, const float *rowAbsMax, const float *rowMult, int kTile, float *tileMax)
{
    __shared__ float red[4];
    int t0 = blockIdx.x * kTile;
    float mx = 0;
    for (int t = t0 + threadIdx.x; t < t0 + kTile && t < len; t += 256) {
        float m = rowAbsMax[t];
        if (rowMult) {
            m *= fabsf(rowMult[t]);
        }
        mx = fmaxf(mx, m);
    }
    mx = WaveMax(mx);
    if ((threadIdx.x & 63) == 0) {
        red[threadIdx.x >> 6] = mx;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        tileMax[blockIdx.x] = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    }
}

// abs-max of 16 raw bytes holding fp32 or bf16 values
template <class TSrc> __device__ __forceinline__ float AbsMax16(v4i raw)
{
    float m = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        uint32_t w = (uint32_t)raw[e];
        if (TSrc::SIZE == 4) {
            m = fmaxf(m, fabsf(__uint_as_float(w)));
        } else {
            m = fmaxf(m, fmaxf(fabsf(__uint_as_float(w << 16)), fabsf(__uint_as_float(w & 0xffff0000u))));
        }
    }
    return m;
}

// grid (row bytes / 4096 rounded up, len/ROWS): a workgroup reduces ROWS rows x 4096 bytes with 16-byte loads, four rows in flight,
// and issues one atomic.  ROWS divides 128, hence kTile.
template <class TSrc>
__global__ void __launch_bounds__(256) TileAbsMax(int len, int dim, Mat src, const float *rowMult, int kTile, float *tileMax)
{
    constexpr int ROWS = 16;
    __shared__ float red[4];
    int tid = threadIdx.x;
    int byteCol = blockIdx.x * 4096 + tid * 16;
    int t0 = blockIdx.y * ROWS;
    float mx = 0;
    if (byteCol < dim * TSrc::SIZE) {
        for (int r = 0; r < ROWS; r += 4) {
            v4i raw[4];
            float rm[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                int t = t0 + r + k;
                raw[k] = t < len ? *(const v4i *)(src.p + (int64_t)t * src.ld + byteCol) : (v4i){0, 0, 0, 0};
                rm[k] = (rowMult && t < len) ? fabsf(rowMult[t]) : 1.f;
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                mx = fmaxf(mx, AbsMax16<TSrc>(raw[k]) * rm[k]);
            }
        }
    }
    mx = WaveMax(mx);
    if ((tid & 63) == 0) {
        red[tid >> 6] = mx;
    }
    __syncthreads();
    if (tid == 0) {
        mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        AtomicMaxPos(&tileMax[t0 / kTile], mx);
    }
}

// 128 (rows t) x 128 (columns x) tile.  Loads are 16 bytes per lane with four rows in flight, conversion, byte tile in LDS, then
// every thread transposes a 16 (t) x 4 (x) block with v_perm_b32 and stores 16 bytes to each of 4 destination rows; 8 neighbouring
// lanes cover the 128 bytes of one destination row.
template <class TSrc, bool QUANT>
__global__ void __launch_bounds__(256) TransposeQuant(int len, int lenRound, Mat src, const float *rowMult, const float *tileMax, int kTile,
    const int *rowIndex, Mat dst, float *tileScale, const float *rowAbsMax, uint32_t seed)
{
    constexpr int PITCH = 132;
    __shared__ __attribute__((aligned(16))) uint8_t buf[128 * PITCH];
    int tid = threadIdx.x;
    int xBlock = blockIdx.x * 128;
    int tBlock = blockIdx.y * 128;
    constexpr int SB = QUANT ? TSrc::SIZE : 1;     // source bytes per element
    constexpr int LPR = 128 * SB / 16;             // lanes per row: 8 (1-byte), 16 (bf16), 32 (fp32)
    constexpr int RPP = 256 / LPR;                 // rows per pass
    constexpr int EPL = 16 / SB;                   // elements per lane
    const int lr = tid / LPR, lc = tid % LPR;
    float mult = 0, tm = 0;
    if (QUANT) {
        if (rowAbsMax) {
            // the k-tile's abs-max from the row maxima (max over its rows of rowAbsMax[t] * |rowMult[t]|), as TileMaxFromRows forms it
            __shared__ float redT[4];
            const int k0 = (tBlock / kTile) * kTile;
            float mx = 0;
            for (int t = k0 + tid; t < k0 + kTile && t < len; t += 256) {
                const int sr = rowIndex ? rowIndex[t] : t; // (a gathered tile: the maxima of the rows that land in it)
                if (sr < 0) {
                    continue;
                }
                float m = rowAbsMax[sr];
                if (rowMult) {
                    m *= fabsf(rowMult[sr]);
                }
                mx = fmaxf(mx, m);
            }
            mx = WaveMax(mx);
            if ((tid & 63) == 0) {
                redT[tid >> 6] = mx;
            }
            __syncthreads();
            tm = fmaxf(fmaxf(redT[0], redT[1]), fmaxf(redT[2], redT[3]));
        } else {
            tm = tileMax[tBlock / kTile];            // one 128-row block lies inside one k-tile (kTile is a multiple of 128)
        }
        mult = tm > 0 ? 1 / (tm / 127) : 0.f;        // same two roundings as scale = max/127, mult = 1/scale
    }
    for (int r0 = 0; r0 < 128; r0 += RPP * 4) {
        v4i raw[4];
        float rm[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            int r = r0 + k * RPP + lr;
            int t = tBlock + r;
            raw[k] = (v4i){0, 0, 0, 0};
            rm[k] = 0;
            if (t < len) {
                int srcRow = rowIndex ? rowIndex[t] : t;
                if (srcRow >= 0) {
                    raw[k] = *(const v4i *)(src.p + (int64_t)srcRow * src.ld + (int64_t)(xBlock + lc * EPL) * SB);
                    rm[k] = (QUANT && rowMult) ? rowMult[srcRow] : 1.f;
                }
            }
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            int r = r0 + k * RPP + lr;
            uint8_t *d = buf + r * PITCH + lc * EPL;
            if (!QUANT) {
                *(uint32_t *)d = (uint32_t)raw[k][0];
                *(uint32_t *)(d + 4) = (uint32_t)raw[k][1];
                *(uint32_t *)(d + 8) = (uint32_t)raw[k][2];
                *(uint32_t *)(d + 12) = (uint32_t)raw[k][3];
            } else {
                float f[EPL];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    uint32_t w = (uint32_t)raw[k][e];
                    if (SB == 4) {
                        f[e] = __uint_as_float(w);
                    } else {
                        f[(2 * e) % EPL] = __uint_as_float(w << 16);
                        f[(2 * e + 1) % EPL] = __uint_as_float(w & 0xffff0000u);
                    }
                }
                uint32_t packed[EPL / 4];
#pragma unroll
                for (int q = 0; q < EPL / 4; ++q) {
                    packed[q] = 0;
                    // (the dither's row is the position in the contraction, its column the gradient's)
                    const uint32_t word = seed ? DitherWord(seed, tBlock + r, (xBlock + lc * EPL) / 4 + q) : 0u;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float x = f[q * 4 + e];
                        if (rowMult) {
                            x = x * rm[k];
                        }
                        const float y = seed ? __builtin_fmaf(x, mult, DitherOffset(word, e)) : x * mult;
                        packed[q] |= (uint32_t)(CvtToI8(y) & 0xff) << (8 * e);
                    }
                }
                *(uint32_t *)d = packed[0];
                if (EPL == 8) {
                    *(uint32_t *)(d + 4) = packed[EPL / 4 - 1];
                }
            }
        }
    }
    __syncthreads();
    TransposeOut128<PITCH>(buf, dst, xBlock, tBlock, tid);
    if (QUANT && tileScale && blockIdx.x == 0 && tid == 0) {
        tileScale[tBlock / kTile] = tm > 0 ? tm / 127 : 1.f;
    }
}


// rope pairs are (cos, sin) interleaved: lane holds two pairs
__device__ __forceinline__ F4 ApplyRope4(F4 v, F4 rope, float dir)
{
    float s0 = rope.y * dir, s1 = rope.w * dir;
    return MakeF4(v.x * rope.x - v.y * s0, v.x * s0 + v.y * rope.x, v.z * rope.z - v.w * s1, v.z * s1 + v.w * rope.z);
}

template <class TSrc>
__global__ void __launch_bounds__(256) RowTileNormalizeRope(int len, int lenRound, int tiles, Mat src, float srcMult, int normalize, float vecScale,
    Mat rope, Mat dst, Mat tileScale)
{
    int t0, tile, h;
    if (!Unit(lenRound, tiles, &t0, &tile, &h)) {
        return;
    }
    int col = tile * TILE + h * 4;
    F4 v[U], rp[U];
    float discr[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
        bool live = t0 + k < len;
        v[k] = live ? Load4<TSrc>(At<TSrc>(src, t0 + k, col)) : ZeroF4();
        rp[k] = (live && rope.p) ? Load4<TF32>(At<TF32>(rope, t0 + k, h * 4)) : ZeroF4();
    }
#pragma unroll
    for (int k = 0; k < U; ++k) {
        discr[k] = 0;
        if (t0 + k >= lenRound) {
            continue;
        }
        F4 x = v[k] * srcMult;
        if (t0 + k < len) {
            if (normalize) {
                float sum2 = Half32Sum(HSum(x * x));
                if (sum2 > 0) {
                    discr[k] = sqrtf(sum2 / TILE) * vecScale;
                    x = x * (1 / discr[k]);
                }
            }
            if (rope.p) {
                x = ApplyRope4(x, rp[k], 1.f);
            }
        }
        Store4<TBF16>(At<TBF16>(dst, t0 + k, col), x);
    }
    if (normalize) {
        StoreScales(tileScale, tile, t0, lenRound, h, discr);
    }
}

template <class TGrad, class TDst>
__global__ void __launch_bounds__(256) BackpropRowTileNormalizeRope(int len, int lenRound, int tiles, Mat grad, float gradMult, Mat srcNorm,
    Mat srcTileScale, Mat rope, Mat dst)
{
    int t0, tile, h;
    if (!Unit(lenRound, tiles, &t0, &tile, &h)) {
        return;
    }
    int col = tile * TILE + h * 4;
    F4 g[U], sn[U], rp[U];
    float sc[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
        int t = t0 + k;
        bool live = t < len;
        g[k] = live ? Load4<TGrad>(At<TGrad>(grad, t, col)) : ZeroF4();
        sn[k] = (live && srcNorm.p) ? Load4<TBF16>(At<TBF16>(srcNorm, t, col)) : ZeroF4();
        sc[k] = (live && srcNorm.p) ? ScaleAt(srcTileScale, tile, t) : 0.f;
        rp[k] = (live && rope.p) ? Load4<TF32>(At<TF32>(rope, t, h * 4)) : ZeroF4();
    }
#pragma unroll
    for (int k = 0; k < U; ++k) {
        int t = t0 + k;
        if (t >= lenRound) {
            continue;
        }
        F4 x = g[k] * gradMult;
        if (t < len) {
            if (srcNorm.p) {
                x = TileNormBackprop(sn[k] * sc[k], x);
            }
            if (rope.p) {
                x = ApplyRope4(x, rp[k], -1.f);
            }
        }
        Store4<TDst>(At<TDst>(dst, t, col), x);
    }
}

// bf16 gradient -> e4m3 with eight elements per lane (a tile = 16 lanes, the tile sums are four DPP steps, the rotated pairs sit in
// one lane): the form the model's attention backward uses.  Same arithmetic per element as BackpropRowTileNormalizeRope.
__global__ void __launch_bounds__(256) BackpropRowTileNormalizeRope8(int len, int lenRound, int tiles, Mat grad, float gradMult, Mat srcNorm,
    Mat srcTileScale, Mat rope, Mat dst)
{
    constexpr int UU = 2;
    const int l16 = threadIdx.x & 15;
    const long unit0 = ((long)blockIdx.x * 256 + threadIdx.x) >> 4;
    const long units = (long)lenRound * tiles;
    const long stride = ((long)gridDim.x * 256) >> 4;
    uint4 g[UU], sn[UU];
    F4 rp[UU][2];
    float sc[UU];
    int row[UU], col[UU];
    bool any[UU], live[UU];
#pragma unroll
    for (int k = 0; k < UU; ++k) {
        long u = unit0 + k * stride;
        any[k] = u < units;
        row[k] = any[k] ? (int)(u / tiles) : 0;
        int tile = any[k] ? (int)(u - (long)row[k] * tiles) : 0;
        col[k] = tile * TILE + l16 * 8;
        live[k] = any[k] && row[k] < len;
        g[k] = live[k] ? *(const uint4 *)At<TBF16>(grad, row[k], col[k]) : make_uint4(0, 0, 0, 0);
        sn[k] = (live[k] && srcNorm.p) ? *(const uint4 *)At<TBF16>(srcNorm, row[k], col[k]) : make_uint4(0, 0, 0, 0);
        sc[k] = (live[k] && srcNorm.p) ? ScaleAt(srcTileScale, tile, row[k]) : 0.f;
        rp[k][0] = (live[k] && rope.p) ? Load4<TF32>(At<TF32>(rope, row[k], l16 * 8)) : ZeroF4();
        rp[k][1] = (live[k] && rope.p) ? Load4<TF32>(At<TF32>(rope, row[k], l16 * 8 + 4)) : ZeroF4();
    }
#pragma unroll
    for (int k = 0; k < UU; ++k) {
        const uint32_t gw[4] = {g[k].x, g[k].y, g[k].z, g[k].w}, sw[4] = {sn[k].x, sn[k].y, sn[k].z, sn[k].w};
        float x[8], src[8];
        float sum2 = 0, dp = 0;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            float ge = (e & 1) ? __uint_as_float(gw[e >> 1] & 0xffff0000u) : __uint_as_float(gw[e >> 1] << 16);
            float se = (e & 1) ? __uint_as_float(sw[e >> 1] & 0xffff0000u) : __uint_as_float(sw[e >> 1] << 16);
            x[e] = ge * gradMult;
            src[e] = se * sc[k];
            sum2 += src[e] * src[e];
            dp += src[e] * x[e];
        }
        if (srcNorm.p) { // uniform
            sum2 = Row16Sum(sum2);
            dp = Row16Sum(dp);
        }
        if (!any[k]) {
            continue;
        }
        uint32_t out[2] = {0, 0};
        if (live[k]) {
            if (srcNorm.p) {
                float sigma = 0, scale = 0;
                if (sum2 != 0) {
                    float inv = 1 / sum2;
                    sigma = dp * inv;
                    scale = sqrtf(TILE * inv);
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    x[e] = sum2 != 0 ? (x[e] - src[e] * sigma) * scale : 0.f;
                }
            }
            if (rope.p) {
                F4 lo = ApplyRope4(MakeF4(x[0], x[1], x[2], x[3]), rp[k][0], -1.f);
                F4 hi = ApplyRope4(MakeF4(x[4], x[5], x[6], x[7]), rp[k][1], -1.f);
                x[0] = lo.x; x[1] = lo.y; x[2] = lo.z; x[3] = lo.w;
                x[4] = hi.x; x[5] = hi.y; x[6] = hi.z; x[7] = hi.w;
            }
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                out[w >> 1] |= CvtPkE4m3(x[2 * w], x[2 * w + 1]) << ((w & 1) * 16);
            }
        }
        *(uint2 *)At<TE4M3>(dst, row[k], col[k]) = make_uint2(out[0], out[1]);
    }
}

// sum of `splits` fp32 partial products (slabs of [rows][cols]) -> packed delta: per row and 128-column tile scale = maxabs/127,
// bytes = sat_i8(rne(v/scale)), TileScale[tile][row] = scale: the arithmetic of the GEMM's ROW_TILE_MAXNORM epilogue applied to the sum
__global__ void __launch_bounds__(256) PackDelta(int rows, int tiles, int splits, const uint8_t *partial, int64_t ldPartial, int64_t slab, float alpha,
    const float *alphaPtr, Mat delta, Mat tileScale)
{
    int t0, tile, h;
    if (!Unit(rows, tiles, &t0, &tile, &h)) {
        return;
    }
    float scale = alpha;
    if (alphaPtr) {
        scale *= *alphaPtr;
    }
    int col = tile * TILE + h * 4;
    F4 v[U];
    float discr[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
        v[k] = ZeroF4();
    }
    for (int sIdx = 0; sIdx < splits; ++sIdx) {
#pragma unroll
        for (int k = 0; k < U; ++k) {
            if (t0 + k < rows) {
                v[k] = v[k] + Load4<TF32>(partial + sIdx * slab + (int64_t)(t0 + k) * ldPartial + (int64_t)col * 4);
            }
        }
    }
#pragma unroll
    for (int k = 0; k < U; ++k) {
        float mx = Half32Max(HMaxAbs(v[k])) * fabsf(scale);
        discr[k] = 0;
        float mult = 0;
        if (mx > 0) {
            discr[k] = mx / 127;
            mult = 1 / discr[k];
        }
        if (t0 + k < rows) {
            Store4<TI8>(At<TI8>(delta, t0 + k, col), v[k] * scale * mult);
        }
    }
    StoreScales(tileScale, tile, t0, rows, h, discr);
}

bool MatOk(const ts2_mat *m, int rows, int cols, int elemSize)
{
    return m && m->ptr && m->y >= rows && m->x >= cols && (m->strideBytes % 4) == 0 && m->strideBytes >= (int64_t)cols * elemSize;
}

int ElemSize(int type)
{
    switch (type) {
    case TS2_F32:
    case TS2_I32:
        return 4;
    case TS2_BF16:
        return 2;
    default:
        return 1;
    }
}
} // namespace

#define STREAM ((hipStream_t)stream)

extern "C" int ts2_layer_normalize_state_vecs(const ts2_mat *state, int32_t stateType, int32_t len, int32_t lenRound, float vecScale,
    const ts2_mat *normState, int32_t normType, const ts2_mat *normStateScale, void *stream)
{
    if (!state || !normState || !normStateScale) {
        return TS2_ERR_NULL;
    }
    int dim = state->x;
    if (dim % TILE || lenRound < len || !MatOk(state, len, dim, ElemSize(stateType)) || !MatOk(normState, lenRound, dim, ElemSize(normType)) ||
        !MatOk(normStateScale, dim / TILE, lenRound, 4)) {
        return TS2_ERR_SHAPE;
    }
    int tiles = dim / TILE;
    TS2_DISPATCH_TYPE(stateType, TS, TS2_DISPATCH_TYPE(normType, TD,
        hipLaunchKernelGGL((LayerNormalizeStateVecs<TS, TD>), GridFor(lenRound, tiles), dim3(256), 0, STREAM, len, lenRound, tiles, vecScale,
            M(*state), M(*normState), M(*normStateScale))));
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

static int BackpropNormImpl(bool final, int len, int rows, const ts2_mat *normState, int normType, const ts2_mat *stateScale,
    const ts2_mat *dNormState, const float *combinerScale, const float *gradScale, const float *gradMult, const ts2_mat *stateGrad,
    const ts2_mat *stateGradFast, int fastType, float *nextMaxNorm, void *stream)
{
    if (!normState || !stateScale || !dNormState || !stateGrad || !stateGradFast) {
        return TS2_ERR_NULL;
    }
    int dim = dNormState->x;
    if (dim % TILE || !MatOk(normState, len, dim, ElemSize(normType)) || !MatOk(stateScale, dim / TILE, len, 4) ||
        !MatOk(dNormState, len, dim, 4) || !MatOk(stateGrad, rows, dim, 4) || !MatOk(stateGradFast, rows, dim, ElemSize(fastType))) {
        return TS2_ERR_SHAPE;
    }
    if (normType == TS2_F32 || (fastType != TS2_BF16 && fastType != TS2_E4M3)) {
        return TS2_ERR_UNSUPPORTED;
    }
    int tiles = dim / TILE;
    long nUnits = (long)rows * tiles;
    dim3 bnGrid((unsigned)((nUnits + 7) / 8 < 4096 ? (nUnits + 7) / 8 : 4096));
    if (normType == TS2_E4M3 && fastType == TS2_E4M3 && (((uintptr_t)normState->ptr | normState->strideBytes | (uintptr_t)stateGradFast->ptr |
                                                         stateGradFast->strideBytes) & 7) == 0 &&
        Aligned16(dNormState->ptr, dNormState->strideBytes) && Aligned16(stateGrad->ptr, stateGrad->strideBytes)) {
        dim3 grid8((unsigned)((nUnits + 15) / 16 < 8192 ? (nUnits + 15) / 16 : 8192));
        if (final) {
            hipLaunchKernelGGL((BackpropLayerNormalize8<true>), grid8, dim3(256), 0, STREAM, len, rows, tiles, M(*normState), M(*stateScale),
                M(*dNormState), combinerScale, gradScale, gradMult, M(*stateGrad), M(*stateGradFast), nextMaxNorm);
        } else {
            hipLaunchKernelGGL((BackpropLayerNormalize8<false>), grid8, dim3(256), 0, STREAM, len, rows, tiles, M(*normState), M(*stateScale),
                M(*dNormState), combinerScale, gradScale, gradMult, M(*stateGrad), M(*stateGradFast), nextMaxNorm);
        }
        TS2_CHECK_LAUNCH();
        return TS2_OK;
    }
#define LAUNCH_BN(TN, TFA)                                                                                                                 \
    if (final)                                                                                                                             \
        hipLaunchKernelGGL((BackpropLayerNormalize<TN, TFA, true>), bnGrid, dim3(256), 0, STREAM, len, rows, tiles,         \
            M(*normState), M(*stateScale), M(*dNormState), combinerScale, gradScale, gradMult, M(*stateGrad), M(*stateGradFast), nextMaxNorm); \
    else                                                                                                                                   \
        hipLaunchKernelGGL((BackpropLayerNormalize<TN, TFA, false>), bnGrid, dim3(256), 0, STREAM, len, rows, tiles,        \
            M(*normState), M(*stateScale), M(*dNormState), combinerScale, gradScale, gradMult, M(*stateGrad), M(*stateGradFast), nextMaxNorm)
    if (fastType == TS2_BF16) {
        TS2_DISPATCH_TYPE(normType, TN, LAUNCH_BN(TN, TBF16));
    } else {
        TS2_DISPATCH_TYPE(normType, TN, LAUNCH_BN(TN, TE4M3));
    }
#undef LAUNCH_BN
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_backprop_layer_normalize(const ts2_mat *normState, int32_t normType, const ts2_mat *stateScale, const ts2_mat *dNormState,
    const float *combinerScale, const float *gradScale, const float *gradMult, const ts2_mat *stateGrad, const ts2_mat *stateGradFast,
    int32_t fastType, float *nextLayerGradMaxNorm, int32_t len, void *stream)
{
    return BackpropNormImpl(false, len, len, normState, normType, stateScale, dNormState, combinerScale, gradScale, gradMult, stateGrad,
        stateGradFast, fastType, nextLayerGradMaxNorm, stream);
}

extern "C" int ts2_backprop_final_normalize(int32_t len, int32_t lenRound, const ts2_mat *normState, int32_t normType, const ts2_mat *stateScale,
    const ts2_mat *dNormState, const ts2_mat *stateGrad, const ts2_mat *stateGradFast, int32_t fastType, float *nextLayerGradMaxNorm,
    void *stream)
{
    return BackpropNormImpl(true, len, lenRound, normState, normType, stateScale, dNormState, nullptr, nullptr, nullptr, stateGrad, stateGradFast,
        fastType, nextLayerGradMaxNorm, stream);
}

extern "C" int ts2_scale_grad(const float *gradMaxNorm, const float *prevGradMult, const ts2_mat *grad, const ts2_mat *gradFast, int32_t fastType,
    int32_t len, float *gradScaleOut, float *gradMultOut, void *stream)
{
    if (!gradMaxNorm || !grad || !gradFast) {
        return TS2_ERR_NULL;
    }
    int dim = grad->x;
    if (dim % TILE || !MatOk(grad, len, dim, 4) || !MatOk(gradFast, len, dim, ElemSize(fastType))) {
        return TS2_ERR_SHAPE;
    }
    int tiles = dim / TILE;
    if (fastType == TS2_BF16) {
        hipLaunchKernelGGL((ScaleGrad<TBF16>), GridFor(len, tiles), dim3(256), 0, STREAM, len, tiles, gradMaxNorm, prevGradMult, M(*grad),
            M(*gradFast), gradScaleOut, gradMultOut);
    } else if (fastType == TS2_E4M3) {
        hipLaunchKernelGGL((ScaleGrad<TE4M3>), GridFor(len, tiles), dim3(256), 0, STREAM, len, tiles, gradMaxNorm, prevGradMult, M(*grad),
            M(*gradFast), gradScaleOut, gradMultOut);
    } else {
        return TS2_ERR_UNSUPPORTED;
    }
    TS2_CHECK_LAUNCH();
    hipLaunchKernelGGL(PublishGradMult, dim3(1), dim3(1), 0, STREAM, gradMaxNorm, gradScaleOut, gradMultOut);
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_matrix_lolu(int32_t len, int32_t lenRound, const ts2_mat *gate, const ts2_mat *vals, float resMult, const ts2_mat *res,
    int32_t resType, void *stream)
{
    if (!gate || !vals || !res) {
        return TS2_ERR_NULL;
    }
    int dim = res->x;
    if (dim % TILE || !MatOk(gate, len, dim, 2) || !MatOk(vals, len, dim, 2) || !MatOk(res, lenRound, dim, ElemSize(resType))) {
        return TS2_ERR_SHAPE;
    }
    int tiles = dim / TILE;
    if (resType == TS2_E4M3 && Aligned16(gate->ptr, gate->strideBytes) && Aligned16(vals->ptr, vals->strideBytes) &&
        Aligned16(res->ptr, res->strideBytes)) {
        const long lanes = (long)lenRound * (dim / 16);
        hipLaunchKernelGGL(MatrixLoLU16, dim3((unsigned)((lanes + 255) / 256)), dim3(256), 0, STREAM, len, lenRound, dim / 16, M(*gate), M(*vals),
            resMult, M(*res));
        TS2_CHECK_LAUNCH();
        return TS2_OK;
    }
    if (resType == TS2_E4M3 && Aligned16(gate->ptr, gate->strideBytes) && Aligned16(vals->ptr, vals->strideBytes) &&
        (((uintptr_t)res->ptr | res->strideBytes) & 7) == 0) {
        const long lanes = ((long)lenRound * (dim / 8) + 1) / 2;
        hipLaunchKernelGGL(MatrixLoLU8, dim3((unsigned)((lanes + 255) / 256)), dim3(256), 0, STREAM, len, lenRound, dim / 8, M(*gate), M(*vals),
            resMult, M(*res));
        TS2_CHECK_LAUNCH();
        return TS2_OK;
    }
    TS2_DISPATCH_TYPE(resType, TD,
        hipLaunchKernelGGL((MatrixLoLU<TD>), GridFor(lenRound, tiles), dim3(256), 0, STREAM, len, lenRound, tiles, M(*gate), M(*vals), resMult,
            M(*res)));
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

template <int MODE>
static int BackpropLoluImpl(int len, int lenRound, const ts2_mat *gate, const ts2_mat *vals, float valsScale, const ts2_mat *tileScale,
    const ts2_mat *grad, int gradType, const ts2_mat *gradGate, int ggType, const ts2_mat *gradVals, int gvType, const ts2_mat *dScale, void *stream)
{
    if (!gate || !vals || !grad || !gradGate || !gradVals || (MODE == 0 ? !tileScale : !dScale)) {
        return TS2_ERR_NULL;
    }
    int dim = grad->x;
    if (dim % TILE || !MatOk(gate, len, dim, 2) || !MatOk(vals, len, dim, 2) || !MatOk(grad, len, dim, ElemSize(gradType)) ||
        !MatOk(gradGate, lenRound, dim, ElemSize(ggType)) || !MatOk(gradVals, lenRound, dim, ElemSize(gvType))) {
        return TS2_ERR_SHAPE;
    }
    if (MODE == 0 ? !MatOk(tileScale, dim / TILE, len, 4) : !MatOk(dScale, dim / TILE, lenRound, 4)) {
        return TS2_ERR_SHAPE;
    }
    int tiles = dim / TILE;
    Mat ts = MODE == 0 ? M(*tileScale) : Mat{nullptr, 0};
    Mat ds = MODE == 1 ? M(*dScale) : Mat{nullptr, 0};
    if ((gradType != TS2_BF16 && gradType != TS2_F32) || (ggType != TS2_BF16 && ggType != TS2_E4M3) || (gvType != TS2_BF16 && gvType != TS2_E4M3)) {
        return TS2_ERR_UNSUPPORTED;
    }
    if (MODE == 0 && gradType == TS2_BF16 && ggType == TS2_E4M3 && gvType == TS2_E4M3 && Aligned16(gate->ptr, gate->strideBytes) &&
        Aligned16(vals->ptr, vals->strideBytes) && Aligned16(grad->ptr, grad->strideBytes) &&
        (((uintptr_t)gradGate->ptr | gradGate->strideBytes | (uintptr_t)gradVals->ptr | gradVals->strideBytes) & 7) == 0) {
        const long lanes = ((long)lenRound * tiles * 16 + 1) / 2;
        hipLaunchKernelGGL(BackpropLoLU8, dim3((unsigned)((lanes + 255) / 256)), dim3(256), 0, STREAM, len, lenRound, tiles, M(*gate), M(*vals), valsScale,
            ts, M(*grad), M(*gradGate), M(*gradVals));
        TS2_CHECK_LAUNCH();
        return TS2_OK;
    }
    if (MODE == 1 && gradType == TS2_BF16 && ggType == TS2_E4M3 && gvType == TS2_BF16 && Aligned16(gate->ptr, gate->strideBytes) &&
        Aligned16(vals->ptr, vals->strideBytes) && Aligned16(grad->ptr, grad->strideBytes) && Aligned16(gradVals->ptr, gradVals->strideBytes) &&
        (((uintptr_t)gradGate->ptr | gradGate->strideBytes) & 7) == 0) {
        const long lanes = ((long)lenRound * tiles * 16 + 1) / 2;
        hipLaunchKernelGGL(BackpropLoLUAtt8, dim3((unsigned)((lanes + 255) / 256)), dim3(256), 0, STREAM, len, lenRound, tiles, M(*gate), M(*vals),
            valsScale, M(*grad), M(*gradGate), M(*gradVals), ds);
        TS2_CHECK_LAUNCH();
        return TS2_OK;
    }
#define LAUNCH_BL(TG, TOG, TOV)                                                                                                            \
    hipLaunchKernelGGL((BackpropLoLU<TG, TOG, TOV, MODE>), GridFor(lenRound, tiles), dim3(256), 0, STREAM, len, lenRound, tiles, M(*gate),  \
        M(*vals), valsScale, ts, M(*grad), M(*gradGate), M(*gradVals), ds)
    if (gradType == TS2_BF16) {
        if (ggType == TS2_BF16 && gvType == TS2_BF16) {
            LAUNCH_BL(TBF16, TBF16, TBF16);
        } else if (ggType == TS2_E4M3 && gvType == TS2_E4M3) {
            LAUNCH_BL(TBF16, TE4M3, TE4M3);
        } else if (ggType == TS2_E4M3 && gvType == TS2_BF16) {
            LAUNCH_BL(TBF16, TE4M3, TBF16);
        } else {
            return TS2_ERR_UNSUPPORTED;
        }
    } else {
        if (ggType == TS2_BF16 && gvType == TS2_BF16) {
            LAUNCH_BL(TF32, TBF16, TBF16);
        } else if (ggType == TS2_E4M3 && gvType == TS2_E4M3) {
            LAUNCH_BL(TF32, TE4M3, TE4M3);
        } else if (ggType == TS2_E4M3 && gvType == TS2_BF16) {
            LAUNCH_BL(TF32, TE4M3, TBF16);
        } else {
            return TS2_ERR_UNSUPPORTED;
        }
    }
#undef LAUNCH_BL
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_backprop_row_tile_normalize_lolu(int32_t len, int32_t lenRound, const ts2_mat *gate, const ts2_mat *vals, float valsScale,
    const ts2_mat *valsSrcTileScale, const ts2_mat *grad, int32_t gradType, const ts2_mat *gradGate, const ts2_mat *gradVals,
    int32_t gradOutType, void *stream)
{
    return BackpropLoluImpl<0>(len, lenRound, gate, vals, valsScale, valsSrcTileScale, grad, gradType, gradGate, gradOutType, gradVals,
        gradOutType, nullptr, stream);
}

extern "C" int ts2_backprop_lolu_dscale(int32_t len, int32_t lenRound, const ts2_mat *gate, const ts2_mat *vals, float valsScale,
    const ts2_mat *grad, int32_t gradType, const ts2_mat *gradGate, int32_t gradGateType, const ts2_mat *gradVals, int32_t gradValsType,
    const ts2_mat *dScale, void *stream)
{
    return BackpropLoluImpl<1>(len, lenRound, gate, vals, valsScale, nullptr, grad, gradType, gradGate, gradGateType, gradVals, gradValsType,
        dScale, stream);
}

extern "C" int ts2_tile_max_from_rows(int32_t len, const float *rowAbsMax, const float *rowMult, int32_t kTile, float *tileMax, void *stream)
{
    if (!rowAbsMax || !tileMax) {
        return TS2_ERR_NULL;
    }
    if (kTile <= 0 || kTile % 128 || len <= 0) {
        return TS2_ERR_SHAPE;
    }
    hipLaunchKernelGGL(TileMaxFromRows, dim3((len + kTile - 1) / kTile), dim3(256), 0, STREAM, len, rowAbsMax, rowMult, kTile, tileMax);
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_normalize_vecs_row_max_dither(int32_t len, int32_t lenRound, const ts2_mat *src, int32_t srcType, const float *colScale,
    const ts2_mat *dst, float *rowScale, float *rowAbsMax, uint32_t ditherSeed, void *stream);

extern "C" int ts2_normalize_vecs_row_max2(int32_t len, int32_t lenRound, const ts2_mat *src, int32_t srcType, const float *colScale,
    const ts2_mat *dst, float *rowScale, float *rowAbsMax, void *stream)
{
    return ts2_normalize_vecs_row_max_dither(len, lenRound, src, srcType, colScale, dst, rowScale, rowAbsMax, 0, stream);
}

extern "C" int ts2_normalize_vecs_row_max(int32_t len, int32_t lenRound, const ts2_mat *src, int32_t srcType, const float *colScale,
    const ts2_mat *dst, float *rowScale, void *stream)
{
    return ts2_normalize_vecs_row_max2(len, lenRound, src, srcType, colScale, dst, rowScale, nullptr, stream);
}

extern "C" int ts2_normalize_vecs_row_max_dither(int32_t len, int32_t lenRound, const ts2_mat *src, int32_t srcType, const float *colScale,
    const ts2_mat *dst, float *rowScale, float *rowAbsMax, uint32_t ditherSeed, void *stream)
{
    if (!src || !dst || !rowScale) {
        return TS2_ERR_NULL;
    }
    int dim = dst->x;
    if (dim % 4 || lenRound < len || !MatOk(src, len, dim, ElemSize(srcType)) || !MatOk(dst, lenRound, dim, 1)) {
        return TS2_ERR_SHAPE;
    }
    const bool reg = dim <= 4096;
    if (srcType == TS2_BF16 && dim % 512 == 0 && dim <= 4096 && Aligned16(src->ptr, src->strideBytes) && (((uintptr_t)dst->ptr | dst->strideBytes) & 7) == 0 &&
        (!colScale || ((uintptr_t)colScale & 15) == 0)) {
        // with column scales a wave walks several rows (the scales stay in registers), else one row per wave
        const int wgs = (lenRound + 3) / 4;
        const dim3 grid(colScale && wgs > 2048 ? 2048 : wgs);
#define LAUNCH_RW(N) hipLaunchKernelGGL((NormalizeRowsWave<N>), grid, dim3(256), 0, STREAM, len, lenRound, M(*src), colScale, M(*dst), rowScale, rowAbsMax, ditherSeed)
        switch (dim / 512) {
        case 1: LAUNCH_RW(1); break;
        case 2: LAUNCH_RW(2); break;
        case 3: LAUNCH_RW(3); break;
        case 4: LAUNCH_RW(4); break;
        case 5: LAUNCH_RW(5); break;
        case 6: LAUNCH_RW(6); break;
        case 7: LAUNCH_RW(7); break;
        default: LAUNCH_RW(8); break;
        }
#undef LAUNCH_RW
        TS2_CHECK_LAUNCH();
        return TS2_OK;
    }
#define LAUNCH_RM(TS, REG) hipLaunchKernelGGL((NormalizeVecsRowMax<TS, REG>), dim3(lenRound < 4096 ? lenRound : 4096), dim3(256), 0, STREAM, len, lenRound, dim, M(*src), colScale, M(*dst), rowScale, rowAbsMax, ditherSeed)
    if (srcType == TS2_BF16) {
        if (reg) {
            LAUNCH_RM(TBF16, true);
        } else {
            LAUNCH_RM(TBF16, false);
        }
    } else if (srcType == TS2_F32) {
        if (reg) {
            LAUNCH_RM(TF32, true);
        } else {
            LAUNCH_RM(TF32, false);
        }
    } else {
        return TS2_ERR_UNSUPPORTED;
    }
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_tile_absmax(int32_t len, const ts2_mat *src, int32_t srcType, const float *rowMult, int32_t kTile, float *tileMax, int32_t clear,
    void *stream)
{
    if (!src || !tileMax) {
        return TS2_ERR_NULL;
    }
    int dim = src->x;
    if (dim % 4 || kTile <= 0 || kTile % 128 || !MatOk(src, len, dim, ElemSize(srcType))) {
        return TS2_ERR_SHAPE;
    }
    if (((uintptr_t)src->ptr % 16) || (src->strideBytes % 16) || ((int64_t)dim * ElemSize(srcType)) % 16) {
        return TS2_ERR_ALIGN;
    }
    int nTiles = (len + kTile - 1) / kTile;
    if (clear) {
        hipLaunchKernelGGL(FillFloats, dim3((nTiles + 255) / 256), dim3(256), 0, STREAM, tileMax, nTiles, 0.f);
        TS2_CHECK_LAUNCH();
    }
    dim3 grid((dim * ElemSize(srcType) + 4095) / 4096, (len + 15) / 16);
    if (srcType == TS2_BF16) {
        hipLaunchKernelGGL((TileAbsMax<TBF16>), grid, dim3(256), 0, STREAM, len, dim, M(*src), rowMult, kTile, tileMax);
    } else if (srcType == TS2_F32) {
        hipLaunchKernelGGL((TileAbsMax<TF32>), grid, dim3(256), 0, STREAM, len, dim, M(*src), rowMult, kTile, tileMax);
    } else {
        return TS2_ERR_UNSUPPORTED;
    }
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_transpose_quant(int32_t len, int32_t lenRound, const ts2_mat *src, int32_t srcType, const float *rowMult, const float *tileMax,
    int32_t kTile, const int32_t *rowIndex, const ts2_mat *dstT, int32_t dstType, float *tileScale, void *stream)
{
    return Ts2TransposeQuantRows(len, lenRound, src, srcType, rowMult, tileMax, nullptr, kTile, rowIndex, dstT, dstType, tileScale, stream);
}

extern "C" int ts2_transpose_quant_dither(int32_t len, int32_t lenRound, const ts2_mat *src, int32_t srcType, const float *rowMult, const float *tileMax,
    int32_t kTile, const int32_t *rowIndex, const ts2_mat *dstT, int32_t dstType, float *tileScale, uint32_t ditherSeed, void *stream)
{
    return Ts2TransposeQuantRows(len, lenRound, src, srcType, rowMult, tileMax, nullptr, kTile, rowIndex, dstT, dstType, tileScale, stream, ditherSeed);
}

// ts2_transpose_quant whose k-tile maxima may come from the row maxima instead (rowAbsMax, with tileMax null; with a row index: the
// maxima of the rows gathered into the tile): the kernel then forms each k-tile's maximum itself and the separate
// ts2_tile_max_from_rows launch is not needed
int Ts2TransposeQuantRows(int len, int lenRound, const ts2_mat *src, int srcType, const float *rowMult, const float *tileMax, const float *rowAbsMax,
    int kTile, const int *rowIndex, const ts2_mat *dstT, int dstType, float *tileScale, void *stream, uint32_t ditherSeed)
{
    if (!src || !dstT) {
        return TS2_ERR_NULL;
    }
    int dim = dstT->y;
    if (dim % 128 || lenRound % 128 || lenRound < len || dstT->x < lenRound || src->x < dim || (dstT->strideBytes % 4) ||
        dstT->strideBytes < lenRound) {
        return TS2_ERR_SHAPE;
    }
    if (((uintptr_t)src->ptr % 16) || (src->strideBytes % 16) || ((uintptr_t)dstT->ptr % 16) || (dstT->strideBytes % 16)) {
        return TS2_ERR_ALIGN;
    }
    dim3 grid(dim / 128, lenRound / 128);
    bool quant = dstType == TS2_I8 && (srcType == TS2_BF16 || srcType == TS2_F32);
    if (quant) {
        if ((!tileMax && !rowAbsMax) || kTile <= 0 || kTile % 128) {
            return TS2_ERR_SHAPE;
        }
        if (tileMax) {
            rowAbsMax = nullptr;
        }
        if (srcType == TS2_BF16) {
            hipLaunchKernelGGL((TransposeQuant<TBF16, true>), grid, dim3(256), 0, STREAM, len, lenRound, M(*src), rowMult, tileMax, kTile, rowIndex,
                M(*dstT), tileScale, rowAbsMax, ditherSeed);
        } else {
            hipLaunchKernelGGL((TransposeQuant<TF32, true>), grid, dim3(256), 0, STREAM, len, lenRound, M(*src), rowMult, tileMax, kTile, rowIndex,
                M(*dstT), tileScale, rowAbsMax, ditherSeed);
        }
    } else if (ElemSize(srcType) == 1 && dstType == srcType) {
        hipLaunchKernelGGL((TransposeQuant<TI8, false>), grid, dim3(256), 0, STREAM, len, lenRound, M(*src), nullptr, nullptr, 128, rowIndex,
            M(*dstT), nullptr, nullptr, 0u);
    } else {
        return TS2_ERR_UNSUPPORTED;
    }
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_row_tile_normalize_rope(int32_t len, int32_t lenRound, const ts2_mat *src, int32_t srcType, float srcMult, int32_t normalize,
    float vecScale, const ts2_mat *ropeBuf, const ts2_mat *dst, const ts2_mat *tileScale, void *stream)
{
    if (!src || !dst || (normalize && !tileScale)) {
        return TS2_ERR_NULL;
    }
    int dim = dst->x;
    if (dim % TILE || !MatOk(src, len, dim, ElemSize(srcType)) || !MatOk(dst, lenRound, dim, 2) ||
        (normalize && !MatOk(tileScale, dim / TILE, lenRound, 4)) || (ropeBuf && !MatOk(ropeBuf, len, TILE, 4))) {
        return TS2_ERR_SHAPE;
    }
    int tiles = dim / TILE;
    Mat rope = ropeBuf ? M(*ropeBuf) : Mat{nullptr, 0};
    Mat ts = normalize ? M(*tileScale) : Mat{nullptr, 0};
    if (srcType == TS2_F32) {
        hipLaunchKernelGGL((RowTileNormalizeRope<TF32>), GridFor(lenRound, tiles), dim3(256), 0, STREAM, len, lenRound, tiles, M(*src), srcMult,
            normalize, vecScale, rope, M(*dst), ts);
    } else if (srcType == TS2_BF16) {
        hipLaunchKernelGGL((RowTileNormalizeRope<TBF16>), GridFor(lenRound, tiles), dim3(256), 0, STREAM, len, lenRound, tiles, M(*src), srcMult,
            normalize, vecScale, rope, M(*dst), ts);
    } else {
        return TS2_ERR_UNSUPPORTED;
    }
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_backprop_row_tile_normalize_rope(int32_t len, int32_t lenRound, const ts2_mat *grad, int32_t gradType, float gradMult,
    const ts2_mat *srcNorm, const ts2_mat *srcTileScale, const ts2_mat *ropeBuf, const ts2_mat *dst, int32_t dstType, void *stream)
{
    if (!grad || !dst || (srcNorm && !srcTileScale)) {
        return TS2_ERR_NULL;
    }
    int dim = dst->x;
    if (dim % TILE || !MatOk(grad, len, dim, ElemSize(gradType)) || !MatOk(dst, lenRound, dim, ElemSize(dstType)) ||
        (srcNorm && (!MatOk(srcNorm, len, dim, 2) || !MatOk(srcTileScale, dim / TILE, len, 4))) || (ropeBuf && !MatOk(ropeBuf, len, TILE, 4))) {
        return TS2_ERR_SHAPE;
    }
    int tiles = dim / TILE;
    Mat rope = ropeBuf ? M(*ropeBuf) : Mat{nullptr, 0};
    Mat sn = srcNorm ? M(*srcNorm) : Mat{nullptr, 0};
    Mat st = srcNorm ? M(*srcTileScale) : Mat{nullptr, 0};
    if (gradType != TS2_F32 && gradType != TS2_BF16) {
        return TS2_ERR_UNSUPPORTED;
    }
    if (gradType == TS2_BF16 && dstType == TS2_E4M3 && Aligned16(grad->ptr, grad->strideBytes) && (!srcNorm || Aligned16(srcNorm->ptr, srcNorm->strideBytes)) &&
        (!ropeBuf || Aligned16(ropeBuf->ptr, ropeBuf->strideBytes)) && (((uintptr_t)dst->ptr | dst->strideBytes) & 7) == 0) {
        const long lanes = ((long)lenRound * tiles * 16 + 1) / 2;
        hipLaunchKernelGGL(BackpropRowTileNormalizeRope8, dim3((unsigned)((lanes + 255) / 256)), dim3(256), 0, STREAM, len, lenRound, tiles, M(*grad),
            gradMult, sn, st, rope, M(*dst));
        TS2_CHECK_LAUNCH();
        return TS2_OK;
    }
#define LAUNCH_BR(TG, TD)                                                                                                                  \
    hipLaunchKernelGGL((BackpropRowTileNormalizeRope<TG, TD>), GridFor(lenRound, tiles), dim3(256), 0, STREAM, len, lenRound, tiles, M(*grad), \
        gradMult, sn, st, rope, M(*dst))
    if (gradType == TS2_F32) {
        TS2_DISPATCH_TYPE(dstType, TD, LAUNCH_BR(TF32, TD));
    } else {
        TS2_DISPATCH_TYPE(dstType, TD, LAUNCH_BR(TBF16, TD));
    }
#undef LAUNCH_BR
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_pack_delta(const ts2_mat *partial, int32_t splits, int64_t slabBytes, int32_t rows, int32_t cols, float alpha, const float *alphaPtr,
    const ts2_mat *delta, const ts2_mat *deltaTileScale, void *stream)
{
    if (!partial || !delta || !deltaTileScale) {
        return TS2_ERR_NULL;
    }
    if (cols % TILE || splits < 1 || !MatOk(partial, rows, cols, 4) || !MatOk(delta, rows, cols, 1) || !MatOk(deltaTileScale, cols / TILE, rows, 4) ||
        (slabBytes & 15) || (partial->strideBytes & 15) || ((uintptr_t)partial->ptr & 15)) {
        return TS2_ERR_SHAPE;
    }
    int tiles = cols / TILE;
    hipLaunchKernelGGL(PackDelta, GridFor(rows, tiles), dim3(256), 0, STREAM, rows, tiles, splits, (const uint8_t *)partial->ptr, partial->strideBytes,
        slabBytes, alpha, alphaPtr, M(*delta), M(*deltaTileScale));
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_backprop_row_tile_normalize_lolu_t(int32_t len, int32_t lenRound, const ts2_mat *gate, const ts2_mat *vals, float valsScale,
    const ts2_mat *valsSrcTileScale, const ts2_mat *grad, const ts2_mat *gradGate, const ts2_mat *gradVals, const ts2_mat *gradGateT,
    const ts2_mat *gradValsT, void *stream)
{
    if (!gate || !vals || !valsSrcTileScale || !grad || !gradGate || !gradVals || !gradGateT || !gradValsT) {
        return TS2_ERR_NULL;
    }
    int dim = grad->x;
    if (dim % TILE || lenRound % 128 || lenRound < len || !MatOk(gate, len, dim, 2) || !MatOk(vals, len, dim, 2) || !MatOk(grad, len, dim, 2) ||
        !MatOk(gradGate, lenRound, dim, 1) || !MatOk(gradVals, lenRound, dim, 1) || !MatOk(gradGateT, dim, lenRound, 1) ||
        !MatOk(gradValsT, dim, lenRound, 1) || !MatOk(valsSrcTileScale, dim / TILE, len, 4)) {
        return TS2_ERR_SHAPE;
    }
    if (!Aligned16(gate->ptr, gate->strideBytes) || !Aligned16(vals->ptr, vals->strideBytes) || !Aligned16(grad->ptr, grad->strideBytes) ||
        !Aligned16(gradGateT->ptr, gradGateT->strideBytes) || !Aligned16(gradValsT->ptr, gradValsT->strideBytes) ||
        (((uintptr_t)gradGate->ptr | gradGate->strideBytes | (uintptr_t)gradVals->ptr | gradVals->strideBytes) & 7)) {
        return TS2_ERR_ALIGN;
    }
    hipLaunchKernelGGL(BackpropLoLU8T, dim3(dim / TILE, lenRound / 128), dim3(256), 0, STREAM, len, lenRound, M(*gate), M(*vals), valsScale,
        M(*valsSrcTileScale), M(*grad), M(*gradGate), M(*gradVals), M(*gradGateT), M(*gradValsT));
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}
