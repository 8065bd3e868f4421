// Host-side model description helpers of the step driver: the layer schedule a model depth stands for and the RoPE table.
// They replace InitAlibi (src/gpt/model_params/model_dim.cpp:82-158, the ALIBI_V3 branch that every model string of the reference
// selects) and FillRopeBuf (src/gpt/att/rope.cpp:4-38), so that a caller of ts2_model_* needs nothing but this library to set a model up.
#include "../../include/ts2_abi.h"
#include <math.h>
#include <vector>

namespace
{
struct TLayerEntry {
    int type;
    int attId;
    float slope;
};
} // namespace

extern "C" int ts2_model_schedule(int32_t depth, int32_t moeExpertCount, int32_t wideWindow, int32_t maxLayers, int32_t *layerType,
    int32_t *layerAttId, float *layerSlope, int32_t *attWidth, int32_t *attTypeCount)
{
    if (!layerType || !layerAttId || !layerSlope || !attWidth || !attTypeCount) {
        return TS2_ERR_NULL;
    }
    if (depth < 0 || wideWindow <= 0 || maxLayers < 0) {
        return TS2_ERR_SHAPE;
    }
    const int mlp = moeExpertCount > 0 ? TS2_LT_MOE : TS2_LT_FFN;
    std::vector<TLayerEntry> layers;
    std::vector<int> widths;
    if (depth == 1) {
        // the reference's attention-profiling special case: one wide attention with a slope, one MLP
        widths = {wideWindow};
        layers = {{TS2_LT_ATT, 0, 0.1f}, {mlp, 0, 0.f}};
    } else {
        // attention types: previous token only, 64 tokens, the wide window.  `depth` counts layer pairs; a group is two pairs.  The first
        // groups (a sixth of them, at least one) look one token back and keep dense MLPs; the others alternate a sloped 64-token window
        // with the wide window, each followed by the model's MLP kind.
        widths = {1, 64, wideWindow};
        const int groups = (depth + 1) / 2;
        const int narrow = groups / 6 > 1 ? groups / 6 : 1;
        for (int g = 0; g < groups && depth > 0; ++g) {
            if (g < narrow) {
                for (int rep = 0; rep < 2; ++rep) {
                    layers.push_back({TS2_LT_ATT, 0, 0.f});
                    layers.push_back({TS2_LT_FFN, 0, 0.f});
                }
            } else {
                layers.push_back({TS2_LT_ATT, 1, 0.5f});
                layers.push_back({mlp, 0, 0.f});
                layers.push_back({TS2_LT_ATT, 2, 0.f});
                layers.push_back({mlp, 0, 0.f});
            }
        }
    }
    if ((int)layers.size() > maxLayers) {
        return TS2_ERR_SHAPE;
    }
    for (size_t i = 0; i < layers.size(); ++i) {
        layerType[i] = layers[i].type;
        layerAttId[i] = layers[i].attId;
        layerSlope[i] = layers[i].slope;
    }
    for (size_t i = 0; i < widths.size(); ++i) {
        attWidth[i] = widths[i];
    }
    *attTypeCount = (int)widths.size();
    return (int)layers.size();
}

extern "C" int ts2_fill_rope_buf(float *buf, int32_t width, int32_t ropeLen)
{
    if (!buf) {
        return TS2_ERR_NULL;
    }
    if (width <= 0 || (width & 1) || ropeLen < 0) {
        return TS2_ERR_SHAPE;
    }
    // theta = 5e5; frequency of pair j: theta^(-2j / width) (the logarithm in float, the power in double, as the reference evaluates it)
    const float logTheta = logf(500000.f);
    std::vector<float> freq(width / 2);
    for (int j = 0; j < width / 2; ++j) {
        freq[j] = (float)exp(-logTheta * (j * 2. / width));
    }
    for (int t = 0; t < ropeLen; ++t) {
        float *row = buf + (size_t)t * width;
        for (int j = 0; j < width / 2; ++j) {
            const float angle = t * freq[j];
            row[2 * j] = cosf(angle);
            row[2 * j + 1] = sinf(angle);
        }
    }
    return TS2_OK;
}
