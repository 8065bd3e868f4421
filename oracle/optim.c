/* CPU oracle (test infrastructure only): the optimiser step that turns a delta into new master weights. */
#include "oracle.h"
#include <math.h>
#include <string.h>

/* inverse of Compress (src/gpt/matrix/delta.cpp:155-179), what UnpackDeltaKernel computes (src/gpt/matrix/agpu_cuda.cuh:35-49):
 * dst[y][x] (+)= delta[y][x] * tileScale[x/128][y] */
void orc_unpack_delta(const int8_t *delta, const float *tileScale, float *dst, int ySize, int xSize, int add)
{
    for (int y = 0; y < ySize; ++y) {
        for (int x = 0; x < xSize; ++x) {
            float v = (float)delta[(size_t)y * xSize + x] * tileScale[(size_t)(x / 128) * ySize + y];
            dst[(size_t)y * xSize + x] = add ? dst[(size_t)y * xSize + x] + v : v;
        }
    }
}

/* THostModelMatrix::AddDelta (src/gpt/matrix/host_matrix.cpp:112-145) with TMatrixDeltaAddCtx::AddRow (:45-77), for a dense fp32 delta
 * (the reference's host delta carries one scale and one sum of squares per row; their product with the row is the dense delta here):
 *   sumWeight = sumWeight * dispDecay + 1
 *   per block of rowDispStep = ySize / rowDispSize rows: disp = sum of squares / (rowDispStep * xSize);
 *       rowDisp = rowDisp * dispDecay + disp;  normScale = 1 / sqrt(rowDisp / sumWeight)
 *   per element: d = delta * normScale;  avg = avg * beta1 + d * (1 - beta1);  total = avg * weight1 + d * weight0;
 *       w = w * (1 - step * l2Reg) + total * step,  step = rate * sqrt(sparsity)       (GetShrinkMult, train_step.h:29)
 *   rows whose delta is all zero take d = 0 (AddRow without a delta, :45-58).
 * rowScaleOut [ySize] (may be NULL) receives normScale per row (0 where the dispersion is 0, the device's CalcRowScale guard,
 * agpu_cuda.cu:55-58); returns the sum of squares of the new weights (Sum2). */
double orc_apply_delta(float *weights, float *avgGrad, const float *delta, int ySize, int xSize, int rowDispSize, float *rowDisp, float *sumWeight,
    float sparsity, const orc_train_step *st, float *rowScaleOut)
{
    int rowDispStep = ySize / rowDispSize;
    float step = st->rate * sqrtf(sparsity);
    float shrinkMult = 1 - step * st->l2Reg;
    float betaMult1 = 1 - st->beta1;
    *sumWeight = *sumWeight * st->dispDecay + 1;
    float rowDispNorm = 1 / *sumWeight;
    double newSum2 = 0;
    for (int blockId = 0; blockId < rowDispSize; ++blockId) {
        int blkStart = blockId * rowDispStep;
        float sum2 = 0;
        for (int y = blkStart; y < blkStart + rowDispStep; ++y) {
            float rowSum2 = 0;
            for (int x = 0; x < xSize; ++x) {
                float d = delta[(size_t)y * xSize + x];
                rowSum2 += d * d;
            }
            sum2 += rowSum2;
        }
        float disp = sum2 / ((float)rowDispStep * xSize);
        rowDisp[blockId] = (rowDisp[blockId] * st->dispDecay) + disp;
        float v = rowDisp[blockId] * rowDispNorm;
        float normScale = v > 0 ? 1 / sqrtf(v) : 0;
        for (int y = blkStart; y < blkStart + rowDispStep; ++y) {
            if (rowScaleOut) {
                rowScaleOut[y] = normScale;
            }
            for (int x = 0; x < xSize; ++x) {
                size_t i = (size_t)y * xSize + x;
                float d = delta[i] * normScale;
                float avg = avgGrad[i] * st->beta1 + d * betaMult1;
                float total = avg * st->weight1 + d * st->weight0;
                float val = weights[i] * shrinkMult + total * step;
                avgGrad[i] = avg;
                weights[i] = val;
                newSum2 += (double)val * val;
            }
        }
    }
    return newSum2;
}
