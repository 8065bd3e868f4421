// Mixture-of-experts routing, grouping, gather / combine and the fused gate backward over expert-grouped rows.
// The grouped GEMMs themselves are ts2_gemm_nt with tileGroup / groupOffsets.
#include "vec.h"

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

constexpr int RB = 256; // (token, slot) entries per counting block

// one wave per token: top-k by repeated arg-max (ties -> lowest index), weights as in CpuMoe (layer_moe.cu:287-327)
template <class TSrc>
__global__ void __launch_bounds__(256) MoeCalcSampleExpertLists(int len, int experts, int selected, Mat moeArr, int *sampleExpertIds,
    float *sampleExpertWeights)
{
    int t = blockIdx.x * 4 + (threadIdx.x >> 6);
    int lane = threadIdx.x & 63;
    if (t >= len) {
        return;
    }
    constexpr int PER = 4; // up to 256 experts
    float val[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        int x = lane + 64 * i;
        val[i] = -1e10f;
        if (x < experts) {
            const typename TSrc::T *row = (const typename TSrc::T *)(moeArr.p + (int64_t)t * moeArr.ld);
            if (TSrc::SIZE == 4) {
                val[i] = ((const float *)row)[x];
            } else {
                val[i] = Bf16ToFloat(((const bf16_t *)row)[x]);
            }
        }
    }
    float maxVal = 0, sum2 = 0;
    float myW = 0;
    int myIdx = 0;
    for (int z = 0; z < selected; ++z) {
        float top = -1e10f;
        int topIdx = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            if (val[i] > top) {
                top = val[i];
                topIdx = lane + 64 * i;
            }
        }
        if (topIdx == 0x7fffffff) {
            topIdx = lane; // every remaining value is the -1e10 sentinel
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            float ot = __shfl_xor(top, o, 64);
            int oi = __shfl_xor(topIdx, o, 64);
            if (ot > top || (ot == top && oi < topIdx)) {
                top = ot;
                topIdx = oi;
            }
        }
        if (z == 0) {
            maxVal = top;
        }
        float w = expf((top - maxVal) * 0.5f);
        sum2 += w * w;
        if (lane == z) {
            myW = w;
            myIdx = topIdx;
        }
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            if (lane + 64 * i == topIdx) {
                val[i] = -1e10f;
            }
        }
    }
    float scale = sqrtf((float)experts) * sqrtf(1 / sum2);
    if (lane < selected) {
        sampleExpertIds[t * selected + lane] = myIdx;
        sampleExpertWeights[t * selected + lane] = myW * scale;
    }
}

// stable counting sort, step 1: rank of every entry among earlier entries of its block with the same expert + block histogram
__global__ void __launch_bounds__(RB) MoeLocalRank(int total, int experts, const int *sampleExpertIds, int *sampleExpertOffset, int *blockCounts)
{
    __shared__ int ids[RB];
    int i = blockIdx.x * RB + threadIdx.x;
    int e = i < total ? sampleExpertIds[i] : -1;
    ids[threadIdx.x] = e;
    for (int x = threadIdx.x; x < experts; x += RB) {
        blockCounts[blockIdx.x * experts + x] = 0;
    }
    __syncthreads();
    if (e >= 0) {
        int rank = 0;
        for (int j = 0; j < (int)threadIdx.x; ++j) {
            rank += ids[j] == e;
        }
        sampleExpertOffset[i] = rank;
        atomicAdd(&blockCounts[blockIdx.x * experts + e], 1);
    }
}

// step 2 (one workgroup): per expert exclusive prefix over blocks, padded expert offsets, tile -> expert table.  The blocks are cut
// into 1024/experts chunks (experts <= 256) that are summed by different threads, so no thread walks a long chain of dependent loads.
// (the two serial passes over a thread's blocks are chains of dependent global accesses: with useLds the table is staged in LDS,
// scanned there and written back, all with coalesced accesses - 48 -> a few microseconds for 256 blocks x 64 experts)
__global__ void __launch_bounds__(1024) MoeOffsets(int nBlocks, int experts, int lenMoe, int *blockCountsGlobal, int *expertOffset, int *xpTileExpertId,
    int useLds)
{
    extern __shared__ int stage[];
    constexpr int NT = 1024; // threads: experts x chunks of blocks; the passes over a chunk are serial, so many short chunks
    __shared__ int chunkSum[NT];
    __shared__ int counts[NT];
    int *blockCounts = useLds ? stage : blockCountsGlobal;
    if (useLds) {
        for (int i = threadIdx.x; i < nBlocks * experts; i += NT) {
            stage[i] = blockCountsGlobal[i];
        }
        __syncthreads();
    }
    const int chunks = NT / experts > 0 ? NT / experts : 1;
    const int e = threadIdx.x % experts, ch = threadIdx.x / experts;
    const int per = (nBlocks + chunks - 1) / chunks;
    const int b0 = ch * per, b1 = min(nBlocks, b0 + per);
    const bool active = ch < chunks && threadIdx.x < experts * chunks;
    int sum = 0;
    if (active) {
        for (int b = b0; b < b1; ++b) {
            sum += blockCounts[b * experts + e];
        }
    }
    chunkSum[threadIdx.x] = active ? sum : 0;
    __syncthreads();
    if (active) {
        int base = 0;
        for (int c = 0; c < ch; ++c) {
            base += chunkSum[c * experts + e];
        }
        int run = base;
        for (int b = b0; b < b1; ++b) {
            int c = blockCounts[b * experts + e];
            blockCounts[b * experts + e] = run;
            run += c;
        }
        if (ch == chunks - 1) {
            counts[e] = (run + TILE - 1) & ~(TILE - 1);
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int off = 0;
        for (int x = 0; x < experts; ++x) {
            expertOffset[x] = off;
            off += counts[x];
        }
        expertOffset[experts] = off;
        expertOffset[experts + 1] = lenMoe;
    }
    __syncthreads();
    if (useLds) {
        for (int i = threadIdx.x; i < nBlocks * experts; i += NT) {
            blockCountsGlobal[i] = stage[i];
        }
    }
    for (int x = threadIdx.x; x <= experts; x += NT) {
        int kStart = expertOffset[x] / TILE, kFinish = expertOffset[x + 1] / TILE;
        int res = x == experts ? -1 : x;
        for (int k = kStart; k < kFinish; ++k) {
            xpTileExpertId[k] = res;
        }
    }
}

__global__ void MoeInitXp(int lenMoe, int *xpSampleId, float *xpSampleWeight)
{
    int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t < lenMoe) {
        xpSampleId[t] = -1;
        xpSampleWeight[t] = 0;
    }
}

// step 3: final position inside the expert = block base + local rank; fill the grouped-row tables
__global__ void __launch_bounds__(RB) MoeFillXp(int total, int experts, int selected, const int *sampleExpertIds, const float *sampleExpertWeights,
    int *sampleExpertOffset, const int *blockCounts, const int *expertOffset, int *xpSampleId, float *xpSampleWeight)
{
    int i = blockIdx.x * RB + threadIdx.x;
    if (i >= total) {
        return;
    }
    int e = sampleExpertIds[i];
    int off = blockCounts[blockIdx.x * experts + e] + sampleExpertOffset[i];
    sampleExpertOffset[i] = off;
    int dst = expertOffset[e] + off;
    xpSampleId[dst] = i / selected;
    xpSampleWeight[dst] = sampleExpertWeights[i];
}

// gather rows: 16 bytes per lane
__global__ void __launch_bounds__(256) MoeGroupSamples(int lenMoe, int rowBytes, Mat src, const int *xpSampleId, Mat dst)
{
    int chunksPerRow = rowBytes / 16;
    long id = (long)blockIdx.x * 256 + threadIdx.x;
    int row = (int)(id / chunksPerRow);
    int c = (int)(id - (long)row * chunksPerRow);
    if (row >= lenMoe) {
        return;
    }
    int s = xpSampleId[row];
    v4i v = {0, 0, 0, 0};
    if (s >= 0) {
        v = *(const v4i *)(src.p + (int64_t)s * src.ld + c * 16);
    }
    *(v4i *)(dst.p + (int64_t)row * dst.ld + c * 16) = v;
}

template <class TDst>
__global__ void __launch_bounds__(256) MatrixLoLUmoe(int lenMoe, int tiles, const float *xpSampleWeight, Mat gate, Mat vals, float resMult, Mat res)
{
    long u = ((long)blockIdx.x * 256 + threadIdx.x) >> 5;
    int h = threadIdx.x & 31;
    int t = (int)(u / tiles), tile = (int)(u % tiles);
    if (t >= lenMoe) {
        return;
    }
    int col = tile * TILE + h * 4;
    float moe = xpSampleWeight[t];
    F4 v = ZeroF4();
    if (moe != 0) {
        F4 g = Load4<TBF16>(At<TBF16>(gate, t, col));
        v = Load4<TBF16>(At<TBF16>(vals, t, col)) * LoLU4(g) * (moe * resMult);
    }
    Store4<TDst>(At<TDst>(res, t, col), v);
}

// sum over the 16 lanes of a row of the wave (one 128-wide tile at 8 elements per lane)
__device__ __forceinline__ float Row16Sum(float v)
{
    v += LaneDpp<DPP_XOR1>(v);
    v += LaneDpp<DPP_XOR2>(v);
    v += LaneDpp<DPP_HALF_MIRROR>(v);
    v += LaneDpp<DPP_MIRROR>(v);
    return v;
}

// e4m3 results, sixteen elements per lane (two 16-byte loads per input, one 16-byte store): the arithmetic of MatrixLoLUmoe
__global__ void __launch_bounds__(256) MatrixLoLUmoe16(int lenMoe, int dim16, const float *xpSampleWeight, Mat gate, Mat vals, float resMult, Mat res)
{
    const long id = (long)blockIdx.x * 256 + threadIdx.x;
    if (id >= (long)lenMoe * dim16) {
        return;
    }
    const int t = (int)(id / dim16), c = (int)(id - (long)t * dim16) * 16;
    const float moe = xpSampleWeight[t];
    uint32_t out[4] = {0, 0, 0, 0};
    if (moe != 0) {
        const uint4 g0 = *(const uint4 *)At<TBF16>(gate, t, c), g1 = *(const uint4 *)At<TBF16>(gate, t, c + 8);
        const uint4 v0 = *(const uint4 *)At<TBF16>(vals, t, c), v1 = *(const uint4 *)At<TBF16>(vals, t, c + 8);
        const uint32_t gw[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w}, vw[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
        const float f = moe * resMult;
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            float ga = __uint_as_float(gw[w] << 16), gb = __uint_as_float(gw[w] & 0xffff0000u);
            float va = __uint_as_float(vw[w] << 16), vb = __uint_as_float(vw[w] & 0xffff0000u);
            out[w >> 1] |= CvtPkE4m3(va * LoLU1(ga) * f, vb * LoLU1(gb) * f) << ((w & 1) * 16);
        }
    }
    *(uint4 *)At<TE4M3>(res, t, c) = make_uint4(out[0], out[1], out[2], out[3]);
}

// one workgroup (8 x 32 lanes) per grouped row so that the routing-weight gradient is a plain block reduction
template <class TGrad, class TOut>
__global__ void __launch_bounds__(256) BackpropRowTileNormalizeLoLUmoe(int tiles, const float *xpSampleWeight, Mat gate, Mat vals, float valsScale,
    Mat valsSrcTileScale, Mat gradArr, float gradMult, Mat gradGate, Mat gradVals, float *dExpertWeight)
{
    __shared__ float red[8];
    int t = blockIdx.x;
    int h = threadIdx.x & 31, grp = threadIdx.x >> 5;
    float moe = xpSampleWeight[t];
    float gm = 0;
    for (int tile = grp; tile < tiles; tile += 8) {
        int col = tile * TILE + h * 4;
        F4 resGate = ZeroF4(), resVals = ZeroF4();
        if (moe != 0) {
            F4 g = Load4<TBF16>(At<TBF16>(gate, t, col));
            F4 v = Load4<TBF16>(At<TBF16>(vals, t, col)) * valsScale;
            F4 grad = Load4<TGrad>(At<TGrad>(gradArr, t, col)) * gradMult;
            F4 mult = LoLU4(g);
            resGate = grad * v * LoLUGrad4(mult) * moe;
            resVals = grad * mult * moe;
            gm += HSum(grad * v * mult);
            F4 src = v * (ScaleAt(valsSrcTileScale, tile, t) / valsScale);
            resVals = TileNormBackprop(src, resVals);
        }
        Store4<TOut>(At<TOut>(gradGate, t, col), resGate);
        Store4<TOut>(At<TOut>(gradVals, t, col), resVals);
    }
    gm = Half32Sum(gm);
    if (h == 0) {
        red[grp] = gm;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        dExpertWeight[t] = ((red[0] + red[1]) + (red[2] + red[3])) + ((red[4] + red[5]) + (red[6] + red[7]));
    }
}

// The fp8 model's types (bf16 gradient in, e4m3 out): one wave per grouped row, a tile is 16 lanes of 8 elements (16-byte loads,
// 8-byte stores), four tiles per pass, and the routing-weight gradient is a wave reduction: no LDS, no workgroup barrier, no idle
// lanes at expert widths below 1024.  Per element the arithmetic of BackpropRowTileNormalizeLoLUmoe.
__global__ void __launch_bounds__(256) BackpropRowTileNormalizeLoLUmoe8(int lenMoe, int tiles, const float *xpSampleWeight, Mat gate, Mat vals,
    float valsScale, Mat valsSrcTileScale, Mat gradArr, float gradMult, Mat gradGate, Mat gradVals, float *dExpertWeight)
{
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6); // wave-uniform
    if (t >= lenMoe) {
        return;
    }
    const int lane = threadIdx.x & 63, l16 = lane & 15, q = lane >> 4;
    const float moe = xpSampleWeight[t];
    float gm = 0;
    for (int tile0 = 0; tile0 < tiles; tile0 += 4) {
        const int tile = tile0 + q;
        const bool any = tile < tiles;
        const bool live = any && moe != 0;
        const int col = (any ? tile : 0) * TILE + l16 * 8;
        uint4 g = make_uint4(0, 0, 0, 0), v = g, gr = g;
        float ts = 0;
        if (live) {
            g = *(const uint4 *)At<TBF16>(gate, t, col);
            v = *(const uint4 *)At<TBF16>(vals, t, col);
            gr = *(const uint4 *)At<TBF16>(gradArr, t, col);
            ts = ScaleAt(valsSrcTileScale, tile, t);
        }
        const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, vw[4] = {v.x, v.y, v.z, v.w}, rw[4] = {gr.x, gr.y, gr.z, gr.w};
        float resGate[8], resVals[8], src[8];
        float sum2 = 0, dp = 0;
        const float srcMult = ts / valsScale;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float ge = (e & 1) ? __uint_as_float(gw[e >> 1] & 0xffff0000u) : __uint_as_float(gw[e >> 1] << 16);
            const float ve = (e & 1) ? __uint_as_float(vw[e >> 1] & 0xffff0000u) : __uint_as_float(vw[e >> 1] << 16);
            const float de = ((e & 1) ? __uint_as_float(rw[e >> 1] & 0xffff0000u) : __uint_as_float(rw[e >> 1] << 16)) * gradMult;
            const float vv = ve * valsScale;
            const float mult = LoLU1(ge);
            resGate[e] = de * vv * (mult * (1 - mult) * 2.f) * moe;
            resVals[e] = de * mult * moe;
            gm += de * vv * mult;
            src[e] = vv * srcMult;
            sum2 += src[e] * src[e];
            dp += src[e] * resVals[e];
        }
        sum2 = Row16Sum(sum2);
        dp = Row16Sum(dp);
        if (!any) {
            continue;
        }
        uint32_t og[2] = {0, 0}, ov[2] = {0, 0};
        if (live) {
            float sigma = 0, scale = 0;
            if (sum2 != 0) {
                const float inv = 1 / sum2;
                sigma = dp * inv;
                scale = sqrtf(TILE * inv);
            }
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const float a0 = sum2 != 0 ? (resVals[2 * w] - src[2 * w] * sigma) * scale : 0.f;
                const float a1 = sum2 != 0 ? (resVals[2 * w + 1] - src[2 * w + 1] * sigma) * scale : 0.f;
                ov[w >> 1] |= CvtPkE4m3(a0, a1) << ((w & 1) * 16);
                og[w >> 1] |= CvtPkE4m3(resGate[2 * w], resGate[2 * w + 1]) << ((w & 1) * 16);
            }
        }
        *(uint2 *)At<TE4M3>(gradGate, t, col) = make_uint2(og[0], og[1]);
        *(uint2 *)At<TE4M3>(gradVals, t, col) = make_uint2(ov[0], ov[1]);
    }
    gm = WaveSum(gm);
    if (lane == 0) {
        dExpertWeight[t] = gm;
    }
}

// CpuBackpropMoe (layer_moe.cu:330-358) restricted to the selected experts (all other terms are zero); one wave per token
template <class TDst>
__global__ void __launch_bounds__(256) BackpropMoe(int len, int lenRound, int bufferDim, int experts, int selected, const int *sampleExpertIds,
    const float *sampleExpertWeights, const int *sampleExpertOffset, const int *expertOffset, const float *dExpertWeight, Mat dMoe)
{
    int t = blockIdx.x * 4 + (threadIdx.x >> 6);
    int lane = threadIdx.x & 63;
    if (t >= lenRound) {
        return;
    }
    uint8_t *row = dMoe.p + (int64_t)t * dMoe.ld;
    auto store = [&](int x, float v) {
        if (TDst::SIZE == 4) {
            ((float *)row)[x] = v;
        } else if (TDst::SIZE == 2) {
            ((bf16_t *)row)[x] = FloatToBf16(v);
        } else {
            row[x] = (uint8_t)(CvtPkE4m3(v, 0.f) & 0xff);
        }
    };
    for (int x = lane; x < bufferDim; x += 64) {
        store(x, 0.f);
    }
    if (t >= len) {
        return;
    }
    float moeScale = sqrtf((float)experts);
    float w = 0, g = 0;
    int e = -1;
    if (lane < selected) {
        int idx = t * selected + lane;
        e = sampleExpertIds[idx];
        w = sampleExpertWeights[idx] / moeScale;
        g = dExpertWeight[expertOffset[e] + sampleExpertOffset[idx]] * moeScale;
    }
    float avrg = WaveSum(w * g);
    // the zero fill above and the scatter below touch the same row from the same wave: order them
    __builtin_amdgcn_s_waitcnt(0);
    __builtin_amdgcn_wave_barrier();
    if (e >= 0) {
        store(e, (w * g - w * w * avrg) * 0.5f);
    }
}

template <class TSrc>
__global__ void __launch_bounds__(256) CombineExperts(int len, int tiles, int selected, Mat src, const int *sampleExpertIds,
    const int *sampleExpertOffset, const int *expertOffset, float alpha, const float *alphaPtr, Mat res, int add)
{
    long u = ((long)blockIdx.x * 256 + threadIdx.x) >> 5;
    int h = threadIdx.x & 31;
    int t = (int)(u / tiles), tile = (int)(u % tiles);
    if (t >= len) {
        return;
    }
    int col = tile * TILE + h * 4;
    F4 sum = ZeroF4();
    for (int k = 0; k < selected; ++k) {
        int idx = t * selected + k;
        int row = expertOffset[sampleExpertIds[idx]] + sampleExpertOffset[idx];
        sum = sum + Load4<TSrc>(At<TSrc>(src, row, col));
    }
    float s = alpha;
    if (alphaPtr) {
        s *= *alphaPtr;
    }
    sum = sum * s;
    if (add) {
        sum = sum + Load4<TF32>(At<TF32>(res, t, col));
    }
    Store4<TF32>(At<TF32>(res, t, col), sum);
}

// 16-bit experts' results: a lane takes 8 consecutive elements (16-byte loads), a tile is 16 lanes, and the rows of all selected
// experts are looked up before the first of them is read, so their loads are in flight together.  The sums are formed in the order
// of the slots, like CombineExperts.
__global__ void __launch_bounds__(256) CombineExperts8(int len, int tiles, int selected, Mat src, const int *sampleExpertIds,
    const int *sampleExpertOffset, const int *expertOffset, float alpha, const float *alphaPtr, Mat res, int add)
{
    const long unit = ((long)blockIdx.x * 256 + threadIdx.x) >> 4;
    const int l16 = threadIdx.x & 15;
    if (unit >= (long)len * tiles) {
        return;
    }
    const int t = (int)(unit / tiles), tile = (int)(unit - (long)t * tiles);
    const int col = tile * TILE + l16 * 8;
    float sum[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    F4 old0 = ZeroF4(), old1 = ZeroF4();
    if (add) {
        old0 = Load4<TF32>(At<TF32>(res, t, col));
        old1 = Load4<TF32>(At<TF32>(res, t, col + 4));
    }
    constexpr int KB = 4; // slots per batch of loads
    for (int k0 = 0; k0 < selected; k0 += KB) {
        int row[KB];
        uint4 v[KB];
#pragma unroll
        for (int k = 0; k < KB; ++k) {
            const int idx = t * selected + (k0 + k < selected ? k0 + k : selected - 1);
            row[k] = expertOffset[sampleExpertIds[idx]] + sampleExpertOffset[idx];
        }
#pragma unroll
        for (int k = 0; k < KB; ++k) {
            v[k] = *(const uint4 *)At<TBF16>(src, row[k], col);
        }
#pragma unroll
        for (int k = 0; k < KB; ++k) {
            if (k0 + k < selected) {
                const uint32_t w[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    sum[e] += (e & 1) ? __uint_as_float(w[e >> 1] & 0xffff0000u) : __uint_as_float(w[e >> 1] << 16);
                }
            }
        }
    }
    float s = alpha;
    if (alphaPtr) {
        s *= *alphaPtr;
    }
    F4 r0 = MakeF4(sum[0], sum[1], sum[2], sum[3]) * s, r1 = MakeF4(sum[4], sum[5], sum[6], sum[7]) * s;
    if (add) {
        r0 = r0 + old0;
        r1 = r1 + old1;
    }
    Store4<TF32>(At<TF32>(res, t, col), r0);
    Store4<TF32>(At<TF32>(res, t, col + 4), r1);
}

// The same for up to KB (<= 4) selected experts with U consecutive tokens per lane: the three dependent loads that lead to a row's
// data (slot -> expert, expert -> first row, row -> data) are issued for all U tokens side by side, so that U * selected row loads of
// a lane are in flight together instead of `selected` at the end of one chain.
template <int U, int KB>
__global__ void __launch_bounds__(256) CombineExperts8U(int len, int tiles, int selected, Mat src, const int *sampleExpertIds,
    const int *sampleExpertOffset, const int *expertOffset, float alpha, const float *alphaPtr, Mat res, int add)
{
    const long unit = ((long)blockIdx.x * 256 + threadIdx.x) >> 4;
    const int l16 = threadIdx.x & 15;
    const long nUnits = (long)((len + U - 1) / U) * tiles;
    if (unit >= nUnits) {
        return;
    }
    const int t0 = (int)(unit / tiles) * U, tile = (int)(unit % tiles);
    const int col = tile * TILE + l16 * 8;
    int ids[U][KB], off[U][KB], row[U][KB];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int k = 0; k < KB; ++k) {
            const int t = t0 + u < len ? t0 + u : len - 1;
            const int idx = t * selected + (k < selected ? k : selected - 1);
            ids[u][k] = sampleExpertIds[idx];
            off[u][k] = sampleExpertOffset[idx];
        }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int k = 0; k < KB; ++k) {
            row[u][k] = expertOffset[ids[u][k]] + off[u][k];
        }
    }
    uint4 v[U][KB];
    F4 old0[U], old1[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int k = 0; k < KB; ++k) {
            if (k < selected) {
                v[u][k] = *(const uint4 *)At<TBF16>(src, row[u][k], col);
            }
        }
        old0[u] = ZeroF4();
        old1[u] = ZeroF4();
        if (add && t0 + u < len) {
            old0[u] = Load4<TF32>(At<TF32>(res, t0 + u, col));
            old1[u] = Load4<TF32>(At<TF32>(res, t0 + u, col + 4));
        }
    }
    float s = alpha;
    if (alphaPtr) {
        s *= *alphaPtr;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        if (t0 + u >= len) {
            break;
        }
        float sum[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int k = 0; k < KB; ++k) {
            if (k < selected) {
                const uint32_t w[4] = {v[u][k].x, v[u][k].y, v[u][k].z, v[u][k].w};
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    sum[e] += (e & 1) ? __uint_as_float(w[e >> 1] & 0xffff0000u) : __uint_as_float(w[e >> 1] << 16);
                }
            }
        }
        F4 r0 = MakeF4(sum[0], sum[1], sum[2], sum[3]) * s, r1 = MakeF4(sum[4], sum[5], sum[6], sum[7]) * s;
        if (add) {
            r0 = r0 + old0[u];
            r1 = r1 + old1[u];
        }
        Store4<TF32>(At<TF32>(res, t0 + u, col), r0);
        Store4<TF32>(At<TF32>(res, t0 + u, col + 4), r1);
    }
}

// 128x128 byte-tile transposes over a batch of slabs
__global__ void __launch_bounds__(256) TransposeU8Batched(const uint8_t *src, int64_t srcStride, int64_t srcSlab, uint8_t *dst, int64_t dstStride,
    int64_t dstSlab)
{
    constexpr int PITCH = 132;
    __shared__ __attribute__((aligned(16))) uint8_t buf[128 * PITCH];
    int tid = threadIdx.x;
    const uint8_t *s = src + blockIdx.z * srcSlab + (int64_t)blockIdx.y * 128 * srcStride + blockIdx.x * 128;
    uint8_t *d = dst + blockIdx.z * dstSlab + (int64_t)blockIdx.x * 128 * dstStride + blockIdx.y * 128;
    int h = tid & 31;
    for (int r = tid >> 5; r < 128; r += 8) {
        *(uint32_t *)(buf + r * PITCH + h * 4) = *(const uint32_t *)(s + (int64_t)r * srcStride + h * 4);
    }
    __syncthreads();
    int tq = tid & 31;
    for (int xq = tid >> 5; xq < 32; xq += 8) {
        uint32_t r0 = *(const uint32_t *)(buf + (tq * 4 + 0) * PITCH + xq * 4);
        uint32_t r1 = *(const uint32_t *)(buf + (tq * 4 + 1) * PITCH + xq * 4);
        uint32_t r2 = *(const uint32_t *)(buf + (tq * 4 + 2) * PITCH + xq * 4);
        uint32_t r3 = *(const uint32_t *)(buf + (tq * 4 + 3) * PITCH + xq * 4);
        uint32_t a = __builtin_amdgcn_perm(r1, r0, 0x05010400);
        uint32_t b = __builtin_amdgcn_perm(r1, r0, 0x07030602);
        uint32_t c = __builtin_amdgcn_perm(r3, r2, 0x05010400);
        uint32_t e = __builtin_amdgcn_perm(r3, r2, 0x07030602);
        *(uint32_t *)(d + (int64_t)(xq * 4 + 0) * dstStride + tq * 4) = __builtin_amdgcn_perm(c, a, 0x05040100);
        *(uint32_t *)(d + (int64_t)(xq * 4 + 1) * dstStride + tq * 4) = __builtin_amdgcn_perm(c, a, 0x07060302);
        *(uint32_t *)(d + (int64_t)(xq * 4 + 2) * dstStride + tq * 4) = __builtin_amdgcn_perm(e, b, 0x05040100);
        *(uint32_t *)(d + (int64_t)(xq * 4 + 3) * dstStride + tq * 4) = __builtin_amdgcn_perm(e, b, 0x07060302);
    }
}

bool TablesOk(const ts2_moe_tables *t)
{
    return t && t->sampleExpertIds && t->sampleExpertWeights && t->sampleExpertOffset && t->expertOffset && t->xpTileExpertId && t->xpSampleId &&
           t->xpSampleWeight;
}
} // namespace

#define STREAM ((hipStream_t)stream)

// Routing tables from the select logits; blockCounts is the counting sort's scratch: [ceil(len*selected/RB)][experts] ints, every entry in
// use written by MoeLocalRank before it is read, so it needs no clearing between calls.
// the dynamic LDS size MoeOffsets may ask for (a function attribute, set once; not a stream operation)
static bool MoeOffsetsLdsReady()
{
    static std::atomic<bool> attrDone{false};
    return Ts2SetDynamicLds(attrDone, (const void *)MoeOffsets, 150 * 1024);
}

static int MoeRoute(int32_t len, int32_t lenMoe, int32_t experts, int32_t selected, const ts2_mat *select, int32_t selectType,
    const ts2_moe_tables *tb, int *blockCounts, void *stream)
{
    if (selectType == TS2_F32) {
        hipLaunchKernelGGL((MoeCalcSampleExpertLists<TF32>), dim3((len + 3) / 4), dim3(256), 0, STREAM, len, experts, selected, M(*select),
            tb->sampleExpertIds, tb->sampleExpertWeights);
    } else if (selectType == TS2_BF16) {
        hipLaunchKernelGGL((MoeCalcSampleExpertLists<TBF16>), dim3((len + 3) / 4), dim3(256), 0, STREAM, len, experts, selected, M(*select),
            tb->sampleExpertIds, tb->sampleExpertWeights);
    } else {
        return TS2_ERR_UNSUPPORTED;
    }
    TS2_CHECK_LAUNCH();
    int total = len * selected;
    int nBlocks = (total + RB - 1) / RB;
    hipLaunchKernelGGL(MoeLocalRank, dim3(nBlocks), dim3(RB), 0, STREAM, total, experts, tb->sampleExpertIds, tb->sampleExpertOffset, blockCounts);
    TS2_CHECK_LAUNCH();
    const size_t tableBytes = (size_t)nBlocks * experts * 4;
    const int useLds = tableBytes <= 150 * 1024;
    if (!MoeOffsetsLdsReady()) {
        return TS2_ERR_LAUNCH;
    }
    hipLaunchKernelGGL(MoeOffsets, dim3(1), dim3(1024), useLds ? tableBytes : 0, STREAM, nBlocks, experts, lenMoe, blockCounts, tb->expertOffset,
        tb->xpTileExpertId, useLds);
    TS2_CHECK_LAUNCH();
    hipLaunchKernelGGL(MoeInitXp, dim3((lenMoe + 255) / 256), dim3(256), 0, STREAM, lenMoe, tb->xpSampleId, tb->xpSampleWeight);
    TS2_CHECK_LAUNCH();
    hipLaunchKernelGGL(MoeFillXp, dim3(nBlocks), dim3(RB), 0, STREAM, total, experts, selected, tb->sampleExpertIds, tb->sampleExpertWeights,
        tb->sampleExpertOffset, blockCounts, tb->expertOffset, tb->xpSampleId, tb->xpSampleWeight);
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

static int MoeRouteShapeOk(int32_t len, int32_t lenMoe, int32_t experts, int32_t selected, const ts2_mat *select)
{
    return !(len <= 0 || experts <= 0 || experts > 256 || selected <= 0 || selected > experts || selected > 64 || lenMoe % TILE ||
             (int64_t)lenMoe < (int64_t)len * selected + (int64_t)TILE * experts || select->x < experts || select->y < len);
}

extern "C" int ts2_moe_route(int32_t len, int32_t lenMoe, int32_t experts, int32_t selected, const ts2_mat *select, int32_t selectType,
    const ts2_moe_tables *tb, void *stream)
{
    if (!select || !TablesOk(tb) || !tb->blockCounts) {
        return TS2_ERR_NULL;
    }
    if (!MoeRouteShapeOk(len, lenMoe, experts, selected, select)) {
        return TS2_ERR_SHAPE;
    }
    return MoeRoute(len, lenMoe, experts, selected, select, selectType, tb, tb->blockCounts, stream);
}

// ---- the routing entry point that allocates nothing and takes no workspace: the counting sort's scratch is a file-scope device array.
// Every device the library runs on holds its own copy of the array at its own address (until the process ends); the name below is only
// the host-side handle of the symbol, never a device address: host code uses the per-device pointer hipGetSymbolAddress returns.
static __device__ __align__(256) int g_moeRouteScratch[TS2_MOE_ROUTE_STATIC_INTS];

namespace
{
constexpr int MAX_DEVICES = 64;
std::atomic<int *> g_moeRouteScratchPtr[MAX_DEVICES]; // zero-initialised (static storage)

// device address of this device's copy of the scratch array (resolved once per device, with that device current)
int *MoeRouteScratch()
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
        return nullptr;
    }
    int *p = g_moeRouteScratchPtr[dev].load(std::memory_order_acquire);
    if (!p) {
        void *sym = nullptr;
        if (hipGetSymbolAddress(&sym, HIP_SYMBOL(g_moeRouteScratch)) != hipSuccess || !sym) {
            (void)hipGetLastError();
            return nullptr;
        }
        p = (int *)sym;
        g_moeRouteScratchPtr[dev].store(p, std::memory_order_release); // two threads racing here store the same address
    }
    return p;
}
} // namespace

// Everything ts2_moe_route_static does on its first call on a device that is not a stream operation (the scratch symbol's address, which
// loads the code object and registers the array, and MoeOffsets' LDS attribute), for callers that make that first call under stream
// capture: ts2_device_info runs it for the current device.
int Ts2MoeRouteSetup()
{
    return MoeRouteScratch() && MoeOffsetsLdsReady() ? TS2_OK : TS2_ERR_LAUNCH;
}

extern "C" int ts2_moe_route_static(int32_t len, int32_t lenMoe, int32_t experts, int32_t selected, const ts2_mat *select, int32_t selectType,
    const ts2_moe_tables *tb, void *stream)
{
    if (!select || !TablesOk(tb)) {
        return TS2_ERR_NULL;
    }
    if (!MoeRouteShapeOk(len, lenMoe, experts, selected, select)) {
        return TS2_ERR_SHAPE;
    }
    const int64_t nBlocks = ((int64_t)len * selected + RB - 1) / RB;
    if (nBlocks * experts > TS2_MOE_ROUTE_STATIC_INTS) {
        return TS2_ERR_SHAPE; // beyond the fixed scratch: use ts2_moe_route with a caller-owned blockCounts
    }
    int *scratch = MoeRouteScratch();
    if (!scratch) {
        return TS2_ERR_LAUNCH;
    }
    return MoeRoute(len, lenMoe, experts, selected, select, selectType, tb, scratch, stream);
}

extern "C" int ts2_moe_group_samples(int32_t lenMoe, int32_t elemSize, const ts2_mat *src, const int32_t *xpSampleId, const ts2_mat *dst, void *stream)
{
    if (!src || !dst || !xpSampleId) {
        return TS2_ERR_NULL;
    }
    int rowBytes = dst->x * elemSize;
    if (rowBytes % 16 || dst->y < lenMoe || src->x < dst->x || !Aligned16(src->ptr, src->strideBytes) || !Aligned16(dst->ptr, dst->strideBytes)) {
        return TS2_ERR_SHAPE;
    }
    long chunks = (long)lenMoe * (rowBytes / 16);
    hipLaunchKernelGGL(MoeGroupSamples, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, STREAM, lenMoe, rowBytes, M(*src), xpSampleId, M(*dst));
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_matrix_lolu_moe(int32_t lenMoe, const float *xpSampleWeight, const ts2_mat *gate, const ts2_mat *vals, float resMult,
    const ts2_mat *res, int32_t resType, void *stream)
{
    if (!xpSampleWeight || !gate || !vals || !res) {
        return TS2_ERR_NULL;
    }
    int dim = res->x;
    if (dim % TILE || gate->y < lenMoe || vals->y < lenMoe || res->y < lenMoe || gate->x < dim || vals->x < dim) {
        return TS2_ERR_SHAPE;
    }
    int tiles = dim / TILE;
    long units = (long)lenMoe * tiles;
    if (resType == TS2_E4M3 && Aligned16(gate->ptr, gate->strideBytes) && Aligned16(vals->ptr, vals->strideBytes) &&
        Aligned16(res->ptr, res->strideBytes)) {
        const long lanes = (long)lenMoe * (dim / 16);
        hipLaunchKernelGGL(MatrixLoLUmoe16, dim3((unsigned)((lanes + 255) / 256)), dim3(256), 0, STREAM, lenMoe, dim / 16, xpSampleWeight, M(*gate),
            M(*vals), resMult, M(*res));
        TS2_CHECK_LAUNCH();
        return TS2_OK;
    }
    dim3 grid((unsigned)((units * 32 + 255) / 256));
    TS2_DISPATCH_TYPE(resType, TD,
        hipLaunchKernelGGL((MatrixLoLUmoe<TD>), grid, dim3(256), 0, STREAM, lenMoe, tiles, xpSampleWeight, M(*gate), M(*vals), resMult, M(*res)));
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_backprop_row_tile_normalize_lolu_moe(int32_t lenMoe, const float *xpSampleWeight, const ts2_mat *gate, const ts2_mat *vals,
    float valsScale, const ts2_mat *valsSrcTileScale, const ts2_mat *grad, int32_t gradType, float gradMult, const ts2_mat *gradGate,
    const ts2_mat *gradVals, int32_t gradOutType, float *dExpertWeight, void *stream)
{
    if (!xpSampleWeight || !gate || !vals || !valsSrcTileScale || !grad || !gradGate || !gradVals || !dExpertWeight) {
        return TS2_ERR_NULL;
    }
    int dim = grad->x;
    if (dim % TILE || gate->y < lenMoe || vals->y < lenMoe || grad->y < lenMoe || gradGate->y < lenMoe || gradVals->y < lenMoe ||
        valsSrcTileScale->y < dim / TILE || valsSrcTileScale->x < lenMoe) {
        return TS2_ERR_SHAPE;
    }
    int tiles = dim / TILE;
#define LAUNCH_M(TG, TO)                                                                                                                   \
    hipLaunchKernelGGL((BackpropRowTileNormalizeLoLUmoe<TG, TO>), dim3(lenMoe), dim3(256), 0, STREAM, tiles, xpSampleWeight, M(*gate), M(*vals), \
        valsScale, M(*valsSrcTileScale), M(*grad), gradMult, M(*gradGate), M(*gradVals), dExpertWeight)
    if (gradType == TS2_BF16 && gradOutType == TS2_E4M3 && Aligned16(gate->ptr, gate->strideBytes) && Aligned16(vals->ptr, vals->strideBytes) &&
        Aligned16(grad->ptr, grad->strideBytes) && (((uintptr_t)gradGate->ptr | gradGate->strideBytes | (uintptr_t)gradVals->ptr | gradVals->strideBytes) & 7) == 0) {
        hipLaunchKernelGGL(BackpropRowTileNormalizeLoLUmoe8, dim3((lenMoe + 3) / 4), dim3(256), 0, STREAM, lenMoe, tiles, xpSampleWeight, M(*gate),
            M(*vals), valsScale, M(*valsSrcTileScale), M(*grad), gradMult, M(*gradGate), M(*gradVals), dExpertWeight);
    } else if (gradType == TS2_BF16 && gradOutType == TS2_BF16) {
        LAUNCH_M(TBF16, TBF16);
    } else if (gradType == TS2_BF16 && gradOutType == TS2_E4M3) {
        LAUNCH_M(TBF16, TE4M3);
    } else if (gradType == TS2_F32 && gradOutType == TS2_BF16) {
        LAUNCH_M(TF32, TBF16);
    } else if (gradType == TS2_F32 && gradOutType == TS2_E4M3) {
        LAUNCH_M(TF32, TE4M3);
    } else {
        return TS2_ERR_UNSUPPORTED;
    }
#undef LAUNCH_M
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_backprop_moe(int32_t len, int32_t lenRound, int32_t experts, int32_t selected, const ts2_moe_tables *tb,
    const float *dExpertWeight, const ts2_mat *dMoe, int32_t dMoeType, void *stream)
{
    if (!TablesOk(tb) || !dExpertWeight || !dMoe) {
        return TS2_ERR_NULL;
    }
    if (dMoe->x < experts || dMoe->y < lenRound || selected > 64) {
        return TS2_ERR_SHAPE;
    }
    dim3 grid((lenRound + 3) / 4);
    if (dMoeType == TS2_F32) {
        hipLaunchKernelGGL((BackpropMoe<TF32>), grid, dim3(256), 0, STREAM, len, lenRound, dMoe->x, experts, selected, tb->sampleExpertIds,
            tb->sampleExpertWeights, tb->sampleExpertOffset, tb->expertOffset, dExpertWeight, M(*dMoe));
    } else if (dMoeType == TS2_BF16) {
        hipLaunchKernelGGL((BackpropMoe<TBF16>), grid, dim3(256), 0, STREAM, len, lenRound, dMoe->x, experts, selected, tb->sampleExpertIds,
            tb->sampleExpertWeights, tb->sampleExpertOffset, tb->expertOffset, dExpertWeight, M(*dMoe));
    } else if (dMoeType == TS2_E4M3) {
        hipLaunchKernelGGL((BackpropMoe<TE4M3>), grid, dim3(256), 0, STREAM, len, lenRound, dMoe->x, experts, selected, tb->sampleExpertIds,
            tb->sampleExpertWeights, tb->sampleExpertOffset, tb->expertOffset, dExpertWeight, M(*dMoe));
    } else {
        return TS2_ERR_UNSUPPORTED;
    }
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_combine_experts(int32_t len, int32_t selected, const ts2_mat *src, int32_t srcType, const ts2_moe_tables *tb, float alpha,
    const float *alphaPtr, const ts2_mat *res, int32_t add, void *stream)
{
    if (!src || !res || !TablesOk(tb)) {
        return TS2_ERR_NULL;
    }
    int dim = res->x;
    if (dim % TILE || res->y < len || src->x < dim) {
        return TS2_ERR_SHAPE;
    }
    int tiles = dim / TILE;
    long units = (long)len * tiles;
    dim3 grid((unsigned)((units * 32 + 255) / 256));
    if (srcType == TS2_BF16 && Aligned16(src->ptr, src->strideBytes) && Aligned16(res->ptr, res->strideBytes)) {
        if (selected <= 4) {
            const long unitsU = (long)((len + 3) / 4) * tiles;
            const dim3 gridU((unsigned)((unitsU * 16 + 255) / 256));
            if (selected <= 2) {
                hipLaunchKernelGGL((CombineExperts8U<4, 2>), gridU, dim3(256), 0, STREAM, len, tiles, selected, M(*src), tb->sampleExpertIds,
                    tb->sampleExpertOffset, tb->expertOffset, alpha, alphaPtr, M(*res), add);
            } else {
                hipLaunchKernelGGL((CombineExperts8U<4, 4>), gridU, dim3(256), 0, STREAM, len, tiles, selected, M(*src), tb->sampleExpertIds,
                    tb->sampleExpertOffset, tb->expertOffset, alpha, alphaPtr, M(*res), add);
            }
            TS2_CHECK_LAUNCH();
            return TS2_OK;
        }
        hipLaunchKernelGGL(CombineExperts8, dim3((unsigned)((units * 16 + 255) / 256)), dim3(256), 0, STREAM, len, tiles, selected, M(*src),
            tb->sampleExpertIds, tb->sampleExpertOffset, tb->expertOffset, alpha, alphaPtr, M(*res), add);
    } else if (srcType == TS2_BF16) {
        hipLaunchKernelGGL((CombineExperts<TBF16>), grid, dim3(256), 0, STREAM, len, tiles, selected, M(*src), tb->sampleExpertIds,
            tb->sampleExpertOffset, tb->expertOffset, alpha, alphaPtr, M(*res), add);
    } else if (srcType == TS2_F32) {
        hipLaunchKernelGGL((CombineExperts<TF32>), grid, dim3(256), 0, STREAM, len, tiles, selected, M(*src), tb->sampleExpertIds,
            tb->sampleExpertOffset, tb->expertOffset, alpha, alphaPtr, M(*res), add);
    } else {
        return TS2_ERR_UNSUPPORTED;
    }
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_transpose_u8_batched(int32_t batch, int32_t rows, int32_t cols, const void *src, int64_t srcStride, int64_t srcSlabBytes,
    void *dst, int64_t dstStride, int64_t dstSlabBytes, void *stream)
{
    if (!src || !dst) {
        return TS2_ERR_NULL;
    }
    if (batch <= 0 || rows % 128 || cols % 128 || srcStride % 4 || dstStride % 4) {
        return TS2_ERR_SHAPE;
    }
    hipLaunchKernelGGL(TransposeU8Batched, dim3(cols / 128, rows / 128, batch), dim3(256), 0, STREAM, (const uint8_t *)src, srcStride,
        srcSlabBytes, (uint8_t *)dst, dstStride, dstSlabBytes);
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}
