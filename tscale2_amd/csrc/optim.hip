// Optimiser apply on the device: packed delta -> fp32 master weights -> requantised fast weights.  The kernels of
// src/gpt/matrix/agpu_cuda.cuh:29-101 and agpu_cuda.cu:9-134 (UnpackDeltaKernel, MatrixRowSum2Kernel, UpdateGlobalRowDisp, AddGradientKernel,
// ConvertMatrixKernel) and the call order of TAgpuCudaModelMatrix::{AddDelta, ApplyGradientImpl, Convert} (agpu_cuda.cuh:398-428,484-590);
// the CPU twin is THostModelMatrix::AddDelta (src/gpt/matrix/host_matrix.cpp:25-145).
//
// All of it is bandwidth bound.  Mapping for gfx950: a workgroup of 256 threads walks rows with a grid stride, a lane owns 4 consecutive
// floats of every 1024-element segment of the row and issues the loads of all its operands for a segment pair before it touches any of
// them; row sums are wave reductions plus one LDS exchange.  Beyond the reference's kernel-per-step sequence there is one fused path for
// the common case "one delta, apply now" (no accumulation across micro-batches): the packed delta is never expanded into an fp32 gradient
// array - its row sums are taken from the bytes (1 B/element read) and AddGradient reads the bytes again - 23 B/element of traffic where
// the unpack / row-sum / add / convert sequence moves 34.
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

__device__ __forceinline__ float BlockSum256(float v, float *red)
{
    v = WaveSum(v);
    __syncthreads(); // red may still be read by the previous row's sum
    if ((threadIdx.x & 63) == 0) {
        red[threadIdx.x >> 6] = v;
    }
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

// delta element source: fp32 array, or packed i8 + one fp32 scale per (row, 128-column tile) laid out [tile][row]
template <bool PACKED> struct DeltaSrc {
    Mat d, ts;
    __device__ __forceinline__ F4 Load(int y, int x) const
    {
        if (PACKED) {
            float s = *(const float *)(ts.p + (int64_t)(x >> 7) * ts.ld + (int64_t)y * 4);
            return Load4<TI8>(d.p + (int64_t)y * d.ld + x) * s;
        }
        return Load4<TF32>(d.p + (int64_t)y * d.ld + (int64_t)x * 4);
    }
};

// UnpackDeltaKernel<ADD_TO_TARGET> (agpu_cuda.cuh:35-49)
template <int ADD> __global__ void __launch_bounds__(256) UnpackDelta(int xSize, int ySize, DeltaSrc<true> src, Mat dst)
{
    for (int y = blockIdx.x; y < ySize; y += gridDim.x) {
        for (int x = threadIdx.x * 4; x < xSize; x += 1024) {
            F4 v = src.Load(y, x);
            float *p = (float *)(dst.p + (int64_t)y * dst.ld) + x;
            if (ADD) {
                v = v + Load4<TF32>(p);
            }
            Store4<TF32>(p, v);
        }
    }
}

// MatrixRowSum2Kernel (agpu_cuda.cu:33-52), also straight from a packed delta
template <bool PACKED> __global__ void __launch_bounds__(256) RowSum2(int xSize, int ySize, DeltaSrc<PACKED> src, float *sum2arr)
{
    __shared__ float red[4];
    for (int y = blockIdx.x; y < ySize; y += gridDim.x) {
        float s0 = 0, s1 = 0;
        int x = threadIdx.x * 4;
        for (; x + 1024 < xSize; x += 2048) {
            F4 a = src.Load(y, x), b = src.Load(y, x + 1024);
            s0 += HSum(a * a);
            s1 += HSum(b * b);
        }
        if (x < xSize) {
            F4 a = src.Load(y, x);
            s0 += HSum(a * a);
        }
        float s = BlockSum256(s0 + s1, red);
        if (threadIdx.x == 0) {
            sum2arr[y] = s;
        }
    }
}

__device__ __forceinline__ float CalcRowScale(float rowDisp)
{
    return rowDisp > 0 ? 1 / sqrtf(rowDisp) : 0.f;
}

// UpdateGlobalRowDisp (agpu_cuda.cu:60-109): one workgroup.  With rowDispStep > 1 the reference walks the blocks one after the other
// with a block-wide sum each; here every wave takes blocks of its own.
__global__ void __launch_bounds__(1024) UpdateGlobalRowDisp(int xSize, int ySize, int rowDispSize, int rowDispStep, const float *deltaSum2arr,
    const ts2_add_gradient_params *pParams, float *sumWeightArr, float *rowDispArr, float *rowScaleArr)
{
    const ts2_add_gradient_params params = *pParams;
    float sumWeight = sumWeightArr[0];
    sumWeight = sumWeight * params.dispDecay + 1;
    const float rowDispNorm = 1 / sumWeight;
    if (rowDispStep == 1) {
        for (int y = threadIdx.x; y < ySize; y += 1024) {
            float rowDisp = (rowDispArr[y] * params.dispDecay) + (deltaSum2arr[y] / xSize);
            rowDispArr[y] = rowDisp;
            rowScaleArr[y] = CalcRowScale(rowDisp * rowDispNorm);
        }
    } else {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        for (int blockId = wave; blockId < rowDispSize; blockId += 16) {
            const int blkStart = blockId * rowDispStep;
            float sum2 = 0;
            for (int k = lane; k < rowDispStep; k += 64) {
                sum2 += deltaSum2arr[blkStart + k];
            }
            sum2 = WaveSum(sum2);
            float disp = sum2 / ((float)xSize * rowDispStep);
            float rowDisp = (rowDispArr[blockId] * params.dispDecay) + disp;
            float rowScale = CalcRowScale(rowDisp * rowDispNorm);
            if (lane == 0) {
                rowDispArr[blockId] = rowDisp;
            }
            for (int k = lane; k < rowDispStep; k += 64) {
                rowScaleArr[blkStart + k] = rowScale;
            }
        }
    }
    __syncthreads(); // every thread has read sumWeightArr[0]
    if (threadIdx.x == 0) {
        sumWeightArr[0] = sumWeight;
    }
}

// AddGradientKernel (agpu_cuda.cu:112-139): moving average of the normalised delta, weight decay, step, row sums of the new weights
template <bool PACKED>
__global__ void __launch_bounds__(256) AddGradient(int xSize, int ySize, DeltaSrc<PACKED> delta, const ts2_add_gradient_params *pParams,
    const float *rowScale, const float *sparsity, Mat avgGrad, Mat weights, float *weightsRowSum2arr)
{
    __shared__ float red[4];
    const ts2_add_gradient_params params = *pParams;
    const float stepMult = params.stepMult * sqrtf(sparsity[0]);
    const float shrinkMult = 1 - stepMult * params.l2Reg; // GetShrinkMult, src/gpt/train_config/train_step.h:29
    const float betaMult = 1 - params.beta1;
    for (int y = blockIdx.x; y < ySize; y += gridDim.x) {
        const float deltaScale = rowScale[y];
        float *ag = (float *)(avgGrad.p + (int64_t)y * avgGrad.ld);
        float *wr = (float *)(weights.p + (int64_t)y * weights.ld);
        float sum2 = 0;
        for (int x0 = threadIdx.x * 4; x0 < xSize; x0 += 2048) {
            const bool two = x0 + 1024 < xSize;
            F4 d[2], oldAG[2], w[2];
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                if (k == 0 || two) {
                    int x = x0 + k * 1024;
                    d[k] = delta.Load(y, x);
                    oldAG[k] = Load4<TF32>(ag + x);
                    w[k] = Load4<TF32>(wr + x);
                }
            }
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                if (k == 0 || two) {
                    int x = x0 + k * 1024;
                    F4 dl = d[k] * deltaScale;
                    F4 newAG = oldAG[k] * params.beta1 + dl * betaMult;
                    F4 totalDelta = newAG * params.weight1 + dl * params.weight0;
                    F4 val = w[k] * shrinkMult + totalDelta * stepMult;
                    sum2 += HSum(val * val);
                    Store4<TF32>(ag + x, newAG);
                    Store4<TF32>(wr + x, val);
                }
            }
        }
        float s = BlockSum256(sum2, red);
        if (threadIdx.x == 0) {
            weightsRowSum2arr[y] = s;
        }
    }
}

// first half of ConvertMatrixKernel (agpu_cuda.cuh:65-101): sko = rms of the whole matrix from the row sums, mult = 32 / sko (0 for a zero
// matrix).  The reference recomputes this in every workgroup of the conversion; here one small launch leaves both scalars on the device.
__global__ void __launch_bounds__(1024) MatrixSko(int totalXSize, int totalYSize, const float *sum2arr, float *resDiscrScale, float *convertMult)
{
    __shared__ float red[16];
    float sum2 = 0;
    for (int k = threadIdx.x; k < totalYSize; k += 1024) {
        sum2 += sum2arr[k];
    }
    sum2 = WaveSum(sum2);
    if ((threadIdx.x & 63) == 0) {
        red[threadIdx.x >> 6] = sum2;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float tot = 0;
        for (int i = 0; i < 16; ++i) {
            tot += red[i];
        }
        float sko = sqrtf(tot / ((float)totalXSize * (float)totalYSize));
        float discrScale = sko * (1 / 32.f); // MODEL_DISCR_SCALE, src/gpt/model_params/model_dim.h:9
        convertMult[0] = sko == 0 ? 0.f : 1 / discrScale;
        resDiscrScale[0] = sko;
    }
}

// second half: fast = cvt(weights * mult), rows ySize .. yBufSize cleared
template <class TDst>
__global__ void __launch_bounds__(256) ConvertMatrix(int xSize, int ySize, int yBufSize, Mat matr, const float *convertMult, Mat dst)
{
    const float mult = convertMult[0];
    for (int y = blockIdx.x; y < yBufSize; y += gridDim.x) {
        uint8_t *drow = dst.p + (int64_t)y * dst.ld;
        if (y < ySize) {
            const float *srow = (const float *)(matr.p + (int64_t)y * matr.ld);
            for (int x0 = threadIdx.x * 4; x0 < xSize; x0 += 2048) {
                const bool two = x0 + 1024 < xSize;
                F4 a = Load4<TF32>(srow + x0), b = two ? Load4<TF32>(srow + x0 + 1024) : ZeroF4();
                Store4<TDst>(drow + (int64_t)x0 * TDst::SIZE, a * mult);
                if (two) {
                    Store4<TDst>(drow + (int64_t)(x0 + 1024) * TDst::SIZE, b * mult);
                }
            }
        } else {
            for (int x = threadIdx.x * 4; x < xSize; x += 1024) {
                Store4<TDst>(drow + (int64_t)x * TDst::SIZE, ZeroF4());
            }
        }
    }
}

int RowGrid(int rows)
{
    return rows < 8192 ? rows : 8192;
}

bool F32Ok(const ts2_mat *m, int x, int y)
{
    return m && m->ptr && m->x >= x && m->y >= y && Aligned16(m->ptr, m->strideBytes);
}

bool PackedOk(const ts2_mat *delta, const ts2_mat *tileScale, int x, int y)
{
    return delta && tileScale && delta->ptr && tileScale->ptr && delta->x >= x && delta->y >= y && (((uintptr_t)delta->ptr | delta->strideBytes) & 3) == 0 &&
           tileScale->y >= x / 128 && tileScale->x >= y && (tileScale->strideBytes & 3) == 0;
}
} // namespace

#define STREAM ((hipStream_t)stream)

extern "C" int ts2_unpack_delta(int32_t xSize, int32_t ySize, const ts2_mat *delta, const ts2_mat *tileScale, const ts2_mat *dst, int32_t addToTarget,
    void *stream)
{
    if (xSize <= 0 || ySize <= 0 || xSize % 128) {
        return TS2_ERR_SHAPE;
    }
    if (!PackedOk(delta, tileScale, xSize, ySize) || !F32Ok(dst, xSize, ySize)) {
        return TS2_ERR_SHAPE;
    }
    DeltaSrc<true> src = {M(*delta), M(*tileScale)};
    if (addToTarget) {
        hipLaunchKernelGGL(UnpackDelta<1>, dim3(RowGrid(ySize)), dim3(256), 0, STREAM, xSize, ySize, src, M(*dst));
    } else {
        hipLaunchKernelGGL(UnpackDelta<0>, dim3(RowGrid(ySize)), dim3(256), 0, STREAM, xSize, ySize, src, M(*dst));
    }
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_matrix_row_sum2(int32_t xSize, int32_t ySize, const ts2_mat *matr, float *sum2arr, void *stream)
{
    if (xSize <= 0 || ySize <= 0 || xSize % 128 || !F32Ok(matr, xSize, ySize)) {
        return TS2_ERR_SHAPE;
    }
    if (!sum2arr) {
        return TS2_ERR_NULL;
    }
    DeltaSrc<false> src = {M(*matr), {nullptr, 0}};
    hipLaunchKernelGGL(RowSum2<false>, dim3(RowGrid(ySize)), dim3(256), 0, STREAM, xSize, ySize, src, sum2arr);
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_packed_delta_row_sum2(int32_t xSize, int32_t ySize, const ts2_mat *delta, const ts2_mat *tileScale, float *sum2arr, void *stream)
{
    if (xSize <= 0 || ySize <= 0 || xSize % 128 || !PackedOk(delta, tileScale, xSize, ySize)) {
        return TS2_ERR_SHAPE;
    }
    if (!sum2arr) {
        return TS2_ERR_NULL;
    }
    DeltaSrc<true> src = {M(*delta), M(*tileScale)};
    hipLaunchKernelGGL(RowSum2<true>, dim3(RowGrid(ySize)), dim3(256), 0, STREAM, xSize, ySize, src, sum2arr);
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_update_global_row_disp(int32_t xSize, int32_t ySize, int32_t rowDispSize, const float *deltaSum2arr,
    const ts2_add_gradient_params *params, float *sumWeight, float *rowDisp, float *rowScale, void *stream)
{
    if (!deltaSum2arr || !params || !sumWeight || !rowDisp || !rowScale) {
        return TS2_ERR_NULL;
    }
    if (xSize <= 0 || ySize <= 0 || rowDispSize <= 0 || ySize % rowDispSize) {
        return TS2_ERR_SHAPE;
    }
    hipLaunchKernelGGL(UpdateGlobalRowDisp, dim3(1), dim3(1024), 0, STREAM, xSize, ySize, rowDispSize, ySize / rowDispSize, deltaSum2arr, params,
        sumWeight, rowDisp, rowScale);
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

static int AddGradientImpl(int xSize, int ySize, const ts2_mat *grad, const ts2_mat *packed, const ts2_mat *tileScale,
    const ts2_add_gradient_params *params, const float *rowScale, const float *sparsity, const ts2_mat *avgGrad, const ts2_mat *weights,
    float *weightsRowSum2, void *stream)
{
    if (!params || !rowScale || !sparsity || !weightsRowSum2) {
        return TS2_ERR_NULL;
    }
    if (xSize <= 0 || ySize <= 0 || xSize % 128 || !F32Ok(avgGrad, xSize, ySize) || !F32Ok(weights, xSize, ySize)) {
        return TS2_ERR_SHAPE;
    }
    if (packed) {
        if (!PackedOk(packed, tileScale, xSize, ySize)) {
            return TS2_ERR_SHAPE;
        }
        DeltaSrc<true> src = {M(*packed), M(*tileScale)};
        hipLaunchKernelGGL(AddGradient<true>, dim3(RowGrid(ySize)), dim3(256), 0, STREAM, xSize, ySize, src, params, rowScale, sparsity, M(*avgGrad),
            M(*weights), weightsRowSum2);
    } else {
        if (!F32Ok(grad, xSize, ySize)) {
            return TS2_ERR_SHAPE;
        }
        DeltaSrc<false> src = {M(*grad), {nullptr, 0}};
        hipLaunchKernelGGL(AddGradient<false>, dim3(RowGrid(ySize)), dim3(256), 0, STREAM, xSize, ySize, src, params, rowScale, sparsity, M(*avgGrad),
            M(*weights), weightsRowSum2);
    }
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_add_gradient(int32_t xSize, int32_t ySize, const ts2_mat *grad, const ts2_add_gradient_params *params, const float *rowScale,
    const float *sparsity, const ts2_mat *avgGrad, const ts2_mat *weights, float *weightsRowSum2, void *stream)
{
    return AddGradientImpl(xSize, ySize, grad, nullptr, nullptr, params, rowScale, sparsity, avgGrad, weights, weightsRowSum2, stream);
}

extern "C" int ts2_convert_matrix(int32_t xSize, int32_t ySize, int32_t yBufSize, int32_t totalXSize, int32_t totalYSize, const ts2_mat *weights,
    const float *sum2arr, const ts2_mat *fast, int32_t fastType, float *matrixScale, float *convertMult, void *stream)
{
    if (!sum2arr || !fast || !fast->ptr || !matrixScale || !convertMult) {
        return TS2_ERR_NULL;
    }
    if (xSize <= 0 || ySize <= 0 || xSize % 128 || yBufSize < ySize || totalXSize < xSize || totalYSize < ySize || !F32Ok(weights, xSize, ySize) ||
        fast->x < xSize || fast->y < yBufSize || (((uintptr_t)fast->ptr | fast->strideBytes) & 3)) {
        return TS2_ERR_SHAPE;
    }
    hipLaunchKernelGGL(MatrixSko, dim3(1), dim3(1024), 0, STREAM, totalXSize, totalYSize, sum2arr, matrixScale, convertMult);
    TS2_CHECK_LAUNCH();
    if (fastType == TS2_I8) {
        hipLaunchKernelGGL(ConvertMatrix<TI8>, dim3(RowGrid(yBufSize)), dim3(256), 0, STREAM, xSize, ySize, yBufSize, M(*weights), convertMult, M(*fast));
    } else if (fastType == TS2_E4M3) {
        hipLaunchKernelGGL(ConvertMatrix<TE4M3>, dim3(RowGrid(yBufSize)), dim3(256), 0, STREAM, xSize, ySize, yBufSize, M(*weights), convertMult, M(*fast));
    } else if (fastType == TS2_BF16) {
        hipLaunchKernelGGL(ConvertMatrix<TBF16>, dim3(RowGrid(yBufSize)), dim3(256), 0, STREAM, xSize, ySize, yBufSize, M(*weights), convertMult, M(*fast));
    } else {
        return TS2_ERR_UNSUPPORTED;
    }
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

// TAgpuCudaModelMatrix::Convert (agpu_cuda.cuh:412-428): row sums of the weights, then the conversion
extern "C" int ts2_opt_convert(const ts2_opt_matrix *m, void *stream)
{
    if (!m) {
        return TS2_ERR_NULL;
    }
    int rc = ts2_matrix_row_sum2(m->xSize, m->ySize, &m->weights, m->weightsRowSum2, stream);
    if (rc) {
        return rc;
    }
    return ts2_convert_matrix(m->xSize, m->ySize, m->yBufSize, m->xSize, m->ySize, &m->weights, m->weightsRowSum2, &m->fast, m->fastType, m->matrixScale,
        m->convertMult, stream);
}

// TAgpuCudaModelMatrix::AddDelta(packed, bm) + ApplyGradientImpl (agpu_cuda.cuh:484-590) on one device
extern "C" int ts2_opt_add_delta(const ts2_opt_matrix *m, const ts2_mat *delta, const ts2_mat *tileScale, int32_t backpropMode,
    const ts2_add_gradient_params *params, void *stream)
{
    if (!m || !delta || !tileScale) {
        return TS2_ERR_NULL;
    }
    const bool add = backpropMode & TS2_BM_GRAD_ADD, apply = backpropMode & TS2_BM_GRAD_APPLY;
    int rc;
    if (!add && apply) {
        // one delta, applied now: the fp32 gradient array is never written
        rc = ts2_packed_delta_row_sum2(m->xSize, m->ySize, delta, tileScale, m->gradRowSum2, stream);
        if (rc) {
            return rc;
        }
        rc = ts2_update_global_row_disp(m->xSize, m->ySize, m->rowDispSize, m->gradRowSum2, params, m->sumWeight, m->rowDisp, m->rowScale, stream);
        if (rc) {
            return rc;
        }
        rc = AddGradientImpl(m->xSize, m->ySize, nullptr, delta, tileScale, params, m->rowScale, m->sparsity, &m->avgGrad, &m->weights,
            m->weightsRowSum2, stream);
    } else {
        rc = ts2_unpack_delta(m->xSize, m->ySize, delta, tileScale, &m->grad, add, stream);
        if (rc || !apply) {
            return rc;
        }
        rc = ts2_matrix_row_sum2(m->xSize, m->ySize, &m->grad, m->gradRowSum2, stream);
        if (rc) {
            return rc;
        }
        rc = ts2_update_global_row_disp(m->xSize, m->ySize, m->rowDispSize, m->gradRowSum2, params, m->sumWeight, m->rowDisp, m->rowScale, stream);
        if (rc) {
            return rc;
        }
        rc = ts2_add_gradient(m->xSize, m->ySize, &m->grad, params, m->rowScale, m->sparsity, &m->avgGrad, &m->weights, m->weightsRowSum2, stream);
    }
    if (rc) {
        return rc;
    }
    return ts2_convert_matrix(m->xSize, m->ySize, m->yBufSize, m->xSize, m->ySize, &m->weights, m->weightsRowSum2, &m->fast, m->fastType, m->matrixScale,
        m->convertMult, stream);
}
