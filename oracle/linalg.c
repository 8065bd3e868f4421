/* CPU oracle (test infrastructure only): the three matrix products of the reference's CPU path and the integer semantics of
 * its int8 GEMM cores.  Loop order and accumulation order follow the reference exactly; OpenMP only splits independent
 * output rows, so results do not depend on the thread count. */
#include "oracle.h"
#include <math.h>
#include <stddef.h>
#include <string.h>

/* src/gpt/compute/cpu_util.cpp:7-27  MulForward: res[t][k] = (sum_x vec[t][x]*kqv[k][x]) * sqrtf(1/dim) */
void orc_mul_forward(const float *vec, const float *kqv, float *res, int len, int dim, int rDim)
{
    float normScale = sqrtf(1.0f / dim);
#pragma omp parallel for schedule(static)
    for (int t = 0; t < len; ++t) {
        for (int k = 0; k < rDim; ++k) {
            float r = 0;
            for (int x = 0; x < dim; ++x) {
                r += vec[(size_t)t * dim + x] * kqv[(size_t)k * dim + x];
            }
            res[(size_t)t * rDim + k] = r * normScale;
        }
    }
}

/* src/gpt/compute/cpu_util.cpp:30-47  MulBackwardWithAccum: vecGrad[t][x] += (sum_k resGrad[t][k]*kqv[k][x]) * sqrtf(1/dim) */
void orc_mul_backward_accum(float *vecGrad, const float *kqv, const float *resGrad, int len, int dim, int rDim)
{
    float normScale = sqrtf(1.0f / dim);
#pragma omp parallel for schedule(static)
    for (int t = 0; t < len; ++t) {
        for (int x = 0; x < dim; ++x) {
            float r = 0;
            for (int k = 0; k < rDim; ++k) {
                r += resGrad[(size_t)t * rDim + k] * kqv[(size_t)k * dim + x];
            }
            vecGrad[(size_t)t * dim + x] += r * normScale;
        }
    }
}

/* src/gpt/compute/cpu_util.cpp:50-67  SumRankOne: delta[k][x] = sum_t resGrad[t][k]*vec[t][x]  (no scale) */
void orc_sum_rank_one(const float *vec, float *delta, const float *resGrad, int len, int dim, int rDim)
{
#pragma omp parallel for schedule(static)
    for (int k = 0; k < rDim; ++k) {
        for (int x = 0; x < dim; ++x) {
            float r = 0;
            for (int t = 0; t < len; ++t) {
                r += resGrad[(size_t)t * rDim + k] * vec[(size_t)t * dim + x];
            }
            delta[(size_t)k * dim + x] = 0 + r;
        }
    }
}

/* Integer contract of the reference's int8 GEMM cores, src/lib/cuda/cuda_i8.cuh:157-196:
 * C[m][n] = sum_k A[m][k]*B[n][k], both operands K-contiguous, exact int32 accumulation. */
void orc_gemm_i8_nt(const int8_t *a, const int8_t *b, int32_t *c, int m, int n, int k)
{
#pragma omp parallel for schedule(static)
    for (int y = 0; y < m; ++y) {
        for (int x = 0; x < n; ++x) {
            int32_t s = 0;
            for (int z = 0; z < k; ++z) {
                s += (int32_t)a[(size_t)y * k + z] * (int32_t)b[(size_t)x * k + z];
            }
            c[(size_t)y * n + x] = s;
        }
    }
}

/* src/lib/cuda/cuda_i8.cuh:200-260 Int8MatMulKernelRowScale with the TStoreScaled / TStoreAddScaled epilogue
 * (src/lib/cuda/cuda_matmul.cuh:420-436,467-490): c[m][n] (+)= (float(acc_i32) * aRowScale[m]) * alpha */
void orc_gemm_i8_nt_rowscale(const int8_t *a, const float *aRowScale, const int8_t *b, float alpha, float *c, int m, int n, int k, int add)
{
#pragma omp parallel for schedule(static)
    for (int y = 0; y < m; ++y) {
        for (int x = 0; x < n; ++x) {
            int32_t s = 0;
            for (int z = 0; z < k; ++z) {
                s += (int32_t)a[(size_t)y * k + z] * (int32_t)b[(size_t)x * k + z];
            }
            float v = ((float)s * (aRowScale ? aRowScale[y] : 1.0f)) * alpha;
            if (add) {
                c[(size_t)y * n + x] += v;
            } else {
                c[(size_t)y * n + x] = v;
            }
        }
    }
}

/* Delta GEMM with one scale per kTile contraction rows (the role of Int8MatMulYScaleKernel, src/lib/cuda/cuda_i8.cuh:264-320).
 * The reference rescales and re-rounds its int32 accumulator between tiles (a lossy step that depends on tile order); the
 * contract here keeps each tile's int32 sum exact and adds the tiles in fp32, in tile order:
 *   c[m][n] = alpha * sum_tile ( kTileScale[tile] * float(sum_{k in tile} A[m][k]*B[n][k]) ) */
void orc_gemm_i8_nt_ktile(const int8_t *a, const int8_t *b, const float *kTileScale, int kTile, float alpha, float *c, int m, int n, int k)
{
#pragma omp parallel for schedule(static)
    for (int y = 0; y < m; ++y) {
        for (int x = 0; x < n; ++x) {
            float acc = 0;
            for (int z0 = 0; z0 < k; z0 += kTile) {
                int32_t s = 0;
                int z1 = z0 + kTile < k ? z0 + kTile : k;
                for (int z = z0; z < z1; ++z) {
                    s += (int32_t)a[(size_t)y * k + z] * (int32_t)b[(size_t)x * k + z];
                }
                acc += kTileScale[z0 / kTile] * (float)s;
            }
            c[(size_t)y * n + x] = acc * alpha;
        }
    }
}

/* generic fp32 C (+)= alpha * A*B^T in double accumulation: the yardstick for fp8/bf16 GEMM tolerances */
void orc_gemm_f32_nt(const float *a, const float *b, float *c, int m, int n, int k, float alpha, int add)
{
#pragma omp parallel for schedule(static)
    for (int y = 0; y < m; ++y) {
        for (int x = 0; x < n; ++x) {
            double s = 0;
            for (int z = 0; z < k; ++z) {
                s += (double)a[(size_t)y * k + z] * (double)b[(size_t)x * k + z];
            }
            float v = (float)(s * alpha);
            if (add) {
                c[(size_t)y * n + x] += v;
            } else {
                c[(size_t)y * n + x] = v;
            }
        }
    }
}
