/* CPU oracle (test infrastructure only): mixture-of-experts routing of the reference CPU layer. */
#include "oracle.h"
#include <math.h>
#include <stdlib.h>

/* src/gpt/compute/layer_moe.cu:287-327 CpuMoe: pick selectedCount largest logits (first index wins ties),
 * w = exp((s - max) * 0.5), then scale so that sum w^2 = expertCount; unselected experts get 0 */
void orc_cpu_moe(int len, int expertCount, int selectedCount, const float *moeSrc, float *res)
{
    float moeScale = sqrtf(expertCount);
    float *srcVec = (float *)malloc(sizeof(float) * expertCount);
    for (int t = 0; t < len; ++t) {
        float maxVal = -1e10f;
        for (int x = 0; x < expertCount; ++x) {
            float val = moeSrc[(size_t)t * expertCount + x];
            srcVec[x] = val;
            res[(size_t)t * expertCount + x] = 0;
            maxVal = maxVal > val ? maxVal : val;
        }
        float sum2 = 0;
        for (int z = 0; z < selectedCount; ++z) {
            float top = -1e10;
            int topIdx = 0;
            for (int x = 0; x < expertCount; ++x) {
                if (srcVec[x] > top) {
                    top = srcVec[x];
                    topIdx = x;
                }
            }
            float w = expf((top - maxVal) * ORC_MOE_SCALE);
            res[(size_t)t * expertCount + topIdx] = w;
            srcVec[topIdx] = -1e10;
            sum2 += w * w;
        }
        float scale = moeScale * sqrtf(1 / sum2);
        for (int x = 0; x < expertCount; ++x) {
            res[(size_t)t * expertCount + x] *= scale;
        }
    }
    free(srcVec);
}

/* src/gpt/compute/layer_moe.cu:330-358 CpuBackpropMoe: in place on dMoe;
 * with w^ = w/sqrt(E), g^ = g*sqrt(E): ds = (w^ g^ - w^2 sum(w^ g^)) * 0.5 */
void orc_cpu_backprop_moe(int len, int expertCount, const float *moe, float *dMoe)
{
    float moeScale = sqrtf(expertCount);
    float *srcVec = (float *)malloc(sizeof(float) * expertCount);
    float *gradVec = (float *)malloc(sizeof(float) * expertCount);
    for (int t = 0; t < len; ++t) {
        for (int x = 0; x < expertCount; ++x) {
            srcVec[x] = moe[(size_t)t * expertCount + x] / moeScale;
            gradVec[x] = dMoe[(size_t)t * expertCount + x] * moeScale;
        }
        float avrgGrad = 0;
        for (int x = 0; x < expertCount; ++x) {
            avrgGrad += srcVec[x] * gradVec[x];
        }
        for (int x = 0; x < expertCount; ++x) {
            float w = srcVec[x];
            dMoe[(size_t)t * expertCount + x] = (w * gradVec[x] - w * w * avrgGrad) * ORC_MOE_SCALE;
        }
    }
    free(srcVec);
    free(gradVec);
}

/* src/gpt/compute/layer_moe.cu:361-377 ScaleExperts: rg[t][expert slab] *= moe[t][expert]; width = total columns */
void orc_scale_experts(int len, int expertCount, int width, const float *moe, float *rg)
{
    int expertSize = width / expertCount;
    for (int t = 0; t < len; ++t) {
        for (int e = 0; e < expertCount; ++e) {
            float scale = moe[(size_t)t * expertCount + e];
            for (int x = e * expertSize; x < (e + 1) * expertSize; ++x) {
                rg[(size_t)t * width + x] *= scale;
            }
        }
    }
}

/* src/gpt/compute/layer_moe.cu:379-403 BackpropScaleExperts: gradMoe[t][e] = <rgSrc, gradRg> over the slab; gradRg *= moe */
void orc_backprop_scale_experts(int len, int expertCount, int width, const float *moe, const float *rgSrc, float *gradMoe, float *gradRg)
{
    int expertSize = width / expertCount;
    for (int t = 0; t < len; ++t) {
        for (int e = 0; e < expertCount; ++e) {
            float scale = moe[(size_t)t * expertCount + e];
            float g = 0;
            for (int x = e * expertSize; x < (e + 1) * expertSize; ++x) {
                float grad = gradRg[(size_t)t * width + x];
                g += rgSrc[(size_t)t * width + x] * grad;
                gradRg[(size_t)t * width + x] *= scale;
            }
            gradMoe[(size_t)t * expertCount + e] = g;
        }
    }
}

/* src/gpt/compute/layer_moe.cu:406-422 FwdContractMatrix: src[[expert][e]][x] -> res[e][[expert][x]] */
void orc_fwd_contract_matrix(const float *src, float *res, int xpCount, int eSize, int xSize)
{
    for (int xp = 0; xp < xpCount; ++xp) {
        for (int e = 0; e < eSize; ++e) {
            for (int x = 0; x < xSize; ++x) {
                res[(size_t)e * xpCount * xSize + xp * xSize + x] = src[((size_t)xp * eSize + e) * xSize + x];
            }
        }
    }
}

/* src/gpt/compute/layer_moe.cu:424-440 BwdContractMatrix: src[e][[expert][x]] -> res[[expert][e]][x] */
void orc_bwd_contract_matrix(const float *src, float *res, int xpCount, int eSize, int xSize)
{
    for (int xp = 0; xp < xpCount; ++xp) {
        for (int e = 0; e < eSize; ++e) {
            for (int x = 0; x < xSize; ++x) {
                res[((size_t)xp * eSize + e) * xSize + x] = src[(size_t)e * xpCount * xSize + xp * xSize + x];
            }
        }
    }
}
