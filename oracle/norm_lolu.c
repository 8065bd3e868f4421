/* CPU oracle (test infrastructure only): tile RMS normalisation and the gated sigmoid ("LoLU"), forward and backward. */
#include "oracle.h"
#include <math.h>
#include <stddef.h>

/* src/gpt/compute/cpu_util.cpp:72-99  NormalizeState: per head (= per tile) y = x*sqrt(headDim/sum x^2), 0 if the tile is 0 */
void orc_normalize_state(const float *state, float *res, int len, int dim, int headCount)
{
    int headDim = dim / headCount;
#pragma omp parallel for schedule(static)
    for (int t = 0; t < len; ++t) {
        for (int h = 0; h < headCount; ++h) {
            const float *src = state + (size_t)t * dim + h * headDim;
            float *dst = res + (size_t)t * dim + h * headDim;
            float sum2 = 0;
            for (int x = 0; x < headDim; ++x) {
                sum2 += src[x] * src[x];
            }
            if (sum2 == 0) {
                for (int x = 0; x < headDim; ++x) {
                    dst[x] = 0;
                }
            } else {
                float scale = sqrtf(headDim / sum2);
                for (int x = 0; x < headDim; ++x) {
                    dst[x] = src[x] * scale;
                }
            }
        }
    }
}

/* src/gpt/compute/cpu_util.cpp:102-134  NormalizeStateBackward: dx = sqrt(n/sum2)*(dy - x*<x,dy>/sum2); grad may alias dNorm */
void orc_normalize_state_backward(const float *state, const float *dNorm, float *grad, int len, int dim, int headCount)
{
    int headDim = dim / headCount;
#pragma omp parallel for schedule(static)
    for (int t = 0; t < len; ++t) {
        for (int h = 0; h < headCount; ++h) {
            const float *src = state + (size_t)t * dim + h * headDim;
            const float *dn = dNorm + (size_t)t * dim + h * headDim;
            float *dst = grad + (size_t)t * dim + h * headDim;
            float sum2 = 0;
            float dp = 0;
            for (int x = 0; x < headDim; ++x) {
                sum2 += src[x] * src[x];
                dp += src[x] * dn[x];
            }
            if (sum2 == 0) {
                for (int x = 0; x < headDim; ++x) {
                    dst[x] = 0;
                }
            } else {
                float sigma = dp / sum2;
                float scale = sqrtf(headDim / sum2);
                for (int x = 0; x < headDim; ++x) {
                    dst[x] = scale * (dn[x] - src[x] * sigma);
                }
            }
        }
    }
}

/* src/gpt/compute/cpu_util.cpp:139-151  CpuComputeLolu: logistic of 2*x clamped at +-20 */
static float ComputeLolu(float x)
{
    float arg = x * ORC_LOLU_SCALE;
    if (arg < -20) {
        return 0;
    } else if (arg > 20) {
        return 1;
    } else {
        float w = expf(arg);
        return w / (1 + w);
    }
}

/* src/gpt/compute/cpu_util.cpp:154-167  LoLU */
void orc_lolu(const float *gate, const float *vals, float *res, int len, int dim)
{
    size_t n = (size_t)len * dim;
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) {
        float mult = ComputeLolu(gate[i]);
        res[i] = mult * vals[i];
    }
}

/* src/gpt/compute/cpu_util.cpp:170-188  BackpropLoLU */
void orc_backprop_lolu(const float *gate, const float *vals, const float *grad, float *gradGate, float *gradVals, int len, int dim)
{
    size_t n = (size_t)len * dim;
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) {
        float mult = ComputeLolu(gate[i]);
        float g = grad[i];
        gradGate[i] = g * vals[i] * mult * (1 - mult) * ORC_LOLU_SCALE;
        gradVals[i] = g * mult;
    }
}
