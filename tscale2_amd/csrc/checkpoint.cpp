// Checkpoint and weight-exchange formats of the reference trainer, host side (no device code):
//   * the SAVELOAD layout of TModelParams (src/gpt/model_params/model_params.h:7-18 over model_matrix.h:61-70 and model_dim.h:118-178), as
//     the reference's binary saver writes it (src/util/bin_saver.h: plain structs and arrays of them as raw bytes, vectors as a 64-bit
//     count + elements, 2-D arrays as 64-bit x and y sizes + rows): read into a ts2_checkpoint, queried per matrix, written back byte for
//     byte;
//   * the fp16-row wire format of model_matrix.cpp:6-58 (PackMatrix / AddPackedMatrix): per row a float rms, then - unless it is zero -
//     the row divided by it as IEEE halves.
// A checkpoint read here feeds ts2_model_set_master (weights, dispersion granularity, sparsity) matrix by matrix.
#include "../../include/ts2_abi.h"
#include <math.h>
#include <string.h>
#include <vector>

namespace
{
struct TReader {
    const uint8_t *p;
    int64_t size, pos = 0;
    bool ok = true;
    bool Raw(void *dst, int64_t n)
    {
        if (!ok || n < 0 || pos + n > size) {
            ok = false;
            return false;
        }
        memcpy(dst, p + pos, (size_t)n);
        pos += n;
        return true;
    }
    template <class T> T Get()
    {
        T v = T();
        Raw(&v, sizeof(T));
        return v;
    }
};

struct TWriter {
    uint8_t *p;
    int64_t cap, pos = 0;
    void Raw(const void *src, int64_t n)
    {
        if (p && pos + n <= cap) {
            memcpy(p + pos, src, (size_t)n);
        }
        pos += n; // keeps counting past the capacity: the caller learns the size it needs
    }
    template <class T> void Put(T v) { Raw(&v, sizeof(T)); }
};

struct TMatrixRec {
    int64_t xSize = 0, ySize = 0;        // Matr
    std::vector<float> weights;
    int64_t gxSize = 0, gySize = 0;      // Grad1 (the moving average of the normalised gradient)
    std::vector<float> grad1;
    float sumWeight = 0;
    std::vector<float> rowDisp;
    float sparsity = 0;
};

bool ReadArray2D(TReader &r, int64_t *x, int64_t *y, std::vector<float> *data)
{
    *x = r.Get<int64_t>();
    *y = r.Get<int64_t>();
    if (!r.ok || *x < 0 || *y < 0 || (*x && *y > (r.size - r.pos) / 4 / *x)) {
        r.ok = false;
        return false;
    }
    data->resize((size_t)(*x * *y));
    return *x * *y == 0 || r.Raw(data->data(), *x * *y * 4);
}

bool ReadMatrix(TReader &r, TMatrixRec *m)
{
    ReadArray2D(r, &m->xSize, &m->ySize, &m->weights);
    ReadArray2D(r, &m->gxSize, &m->gySize, &m->grad1);
    m->sumWeight = r.Get<float>();
    int64_t n = r.Get<int64_t>();
    if (!r.ok || n < 0 || n > (r.size - r.pos) / 4) {
        r.ok = false;
        return false;
    }
    m->rowDisp.resize((size_t)n);
    if (n) {
        r.Raw(m->rowDisp.data(), n * 4);
    }
    m->sparsity = r.Get<float>();
    return r.ok;
}

void WriteMatrix(TWriter &w, const TMatrixRec &m)
{
    w.Put<int64_t>(m.xSize);
    w.Put<int64_t>(m.ySize);
    w.Raw(m.weights.data(), (int64_t)m.weights.size() * 4);
    w.Put<int64_t>(m.gxSize);
    w.Put<int64_t>(m.gySize);
    w.Raw(m.grad1.data(), (int64_t)m.grad1.size() * 4);
    w.Put<float>(m.sumWeight);
    w.Put<int64_t>((int64_t)m.rowDisp.size());
    w.Raw(m.rowDisp.data(), (int64_t)m.rowDisp.size() * 4);
    w.Put<float>(m.sparsity);
}

bool ReadMatrixVec(TReader &r, std::vector<TMatrixRec> *v)
{
    int64_t n = r.Get<int64_t>();
    if (!r.ok || n < 0 || n > 64) {
        r.ok = false;
        return false;
    }
    v->resize((size_t)n);
    for (TMatrixRec &m : *v) {
        if (!ReadMatrix(r, &m)) {
            return false;
        }
    }
    return true;
}

// IEEE half <-> float, round to nearest even (_mm256_cvtps_ph(x, 0) / _mm256_cvtph_ps, src/gpt/model_params/sse_utils.h:105-130)
uint16_t FloatToHalf(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    x &= 0x7fffffffu;
    if (x >= 0x7f800000u) {
        return (uint16_t)(sign | 0x7c00u | (x > 0x7f800000u ? 0x200u : 0)); // inf / nan
    }
    if (x >= 0x477ff000u) {
        return (uint16_t)(sign | 0x7c00u); // rounds to infinity
    }
    if (x < 0x33000001u) {
        return (uint16_t)sign; // below half of the smallest denormal
    }
    int e = (int)(x >> 23) - 127;
    uint32_t mant = (x & 0x7fffffu) | 0x800000u;
    int shift = e >= -14 ? 13 : 13 + (-14 - e); // bits dropped
    uint32_t h = mant >> shift;
    uint32_t rem = mant & ((1u << shift) - 1), halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (h & 1))) {
        ++h;
    }
    if (e >= -14) {
        h += (uint32_t)(e + 14) << 10; // mant's hidden bit adds the 1 of the exponent field; a carry from rounding moves up correctly
    }
    return (uint16_t)(sign | h);
}

float HalfToFloat(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 31, m = h & 0x3ffu, x;
    if (e == 0) {
        if (m == 0) {
            x = sign;
        } else {
            int s = 0;
            while (!(m & 0x400u)) {
                m <<= 1;
                ++s;
            }
            x = sign | ((uint32_t)(127 - 15 + 1 - s) << 23) | ((m & 0x3ffu) << 13);
        }
    } else if (e == 31) {
        x = sign | 0x7f800000u | (m << 13);
    } else {
        x = sign | ((e + 127 - 15) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &x, 4);
    return f;
}
} // namespace

struct ts2_checkpoint {
    int32_t dims[10];
    int64_t labelCount = 0, inputTokenCount = 0, outputTokenCount = 0;
    std::vector<int32_t> attTypes; // (Width, Type) pairs
    std::vector<int32_t> layers;   // (LayerType, AlibiSlope bits, AttentionTypeId) triples
    uint64_t flags = 0, docStartToken = 0;
    int64_t fragLen = 0;
    std::vector<std::vector<TMatrixRec>> layerMatr;
    std::vector<TMatrixRec> modelMatr;
    std::vector<float> bias;
};

extern "C" ts2_checkpoint *ts2_checkpoint_parse(const void *bytes, int64_t size)
{
    if (!bytes || size <= 0) {
        return nullptr;
    }
    TReader r = {(const uint8_t *)bytes, size};
    ts2_checkpoint *c = new ts2_checkpoint();
    r.Raw(c->dims, sizeof(c->dims)); // TModelDims: ten ints, one by one
    c->labelCount = r.Get<int64_t>();
    c->inputTokenCount = r.Get<int64_t>();
    c->outputTokenCount = r.Get<int64_t>();
    int64_t n = r.Get<int64_t>(); // TVector<TAttentionType>: plain structs, one chunk
    if (r.ok && n >= 0 && n <= 64) {
        c->attTypes.resize((size_t)n * 2);
        r.Raw(c->attTypes.data(), n * 8);
    } else {
        r.ok = false;
    }
    n = r.Get<int64_t>(); // TVector<TLayerParams>
    if (r.ok && n >= 0 && n <= 4096) {
        c->layers.resize((size_t)n * 3);
        r.Raw(c->layers.data(), n * 12);
    } else {
        r.ok = false;
    }
    c->flags = r.Get<uint64_t>();
    c->docStartToken = r.Get<uint64_t>();
    c->fragLen = r.Get<int64_t>();
    n = r.Get<int64_t>(); // LayerArr: vector of { MatrArr }
    if (r.ok && n >= 0 && n <= 4096) {
        c->layerMatr.resize((size_t)n);
        for (auto &v : c->layerMatr) {
            if (!ReadMatrixVec(r, &v)) {
                break;
            }
        }
    } else {
        r.ok = false;
    }
    ReadMatrixVec(r, &c->modelMatr);
    n = r.Get<int64_t>();
    if (r.ok && n >= 0 && n <= (r.size - r.pos) / 4) {
        c->bias.resize((size_t)n);
        if (n) {
            r.Raw(c->bias.data(), n * 4);
        }
    } else {
        r.ok = false;
    }
    if (!r.ok || r.pos != size || c->layerMatr.size() != c->layers.size() / 3) {
        delete c;
        return nullptr;
    }
    return c;
}

extern "C" void ts2_checkpoint_free(ts2_checkpoint *c)
{
    delete c;
}

extern "C" int64_t ts2_checkpoint_write(const ts2_checkpoint *c, void *out, int64_t cap)
{
    if (!c) {
        return TS2_ERR_NULL;
    }
    TWriter w = {(uint8_t *)out, out ? cap : 0};
    w.Raw(c->dims, sizeof(c->dims));
    w.Put<int64_t>(c->labelCount);
    w.Put<int64_t>(c->inputTokenCount);
    w.Put<int64_t>(c->outputTokenCount);
    w.Put<int64_t>((int64_t)c->attTypes.size() / 2);
    w.Raw(c->attTypes.data(), (int64_t)c->attTypes.size() * 4);
    w.Put<int64_t>((int64_t)c->layers.size() / 3);
    w.Raw(c->layers.data(), (int64_t)c->layers.size() * 4);
    w.Put<uint64_t>(c->flags);
    w.Put<uint64_t>(c->docStartToken);
    w.Put<int64_t>(c->fragLen);
    w.Put<int64_t>((int64_t)c->layerMatr.size());
    for (const auto &v : c->layerMatr) {
        w.Put<int64_t>((int64_t)v.size());
        for (const TMatrixRec &m : v) {
            WriteMatrix(w, m);
        }
    }
    w.Put<int64_t>((int64_t)c->modelMatr.size());
    for (const TMatrixRec &m : c->modelMatr) {
        WriteMatrix(w, m);
    }
    w.Put<int64_t>((int64_t)c->bias.size());
    w.Raw(c->bias.data(), (int64_t)c->bias.size() * 4);
    return w.pos;
}

extern "C" int ts2_checkpoint_get_info(const ts2_checkpoint *c, ts2_checkpoint_info *out)
{
    if (!c || !out) {
        return TS2_ERR_NULL;
    }
    memset(out, 0, sizeof(*out));
    out->dim = c->dims[0];
    out->qDim = c->dims[1];
    out->ttDim = c->dims[2];
    out->expertDim = c->dims[3];
    out->headCount = c->dims[4];
    out->ffnTiles = c->dims[5];
    out->moeExpertCount = c->dims[6];
    out->moeSelected = c->dims[7];
    out->kvRep = c->dims[8];
    out->depth = c->dims[9];
    out->labelCount = c->labelCount;
    out->inputTokenCount = c->inputTokenCount;
    out->outputTokenCount = c->outputTokenCount;
    out->attTypeCount = (int32_t)(c->attTypes.size() / 2);
    out->layerCount = (int32_t)(c->layers.size() / 3);
    out->flags = c->flags;
    out->docStartToken = c->docStartToken;
    out->fragLen = c->fragLen;
    out->biasCount = (int32_t)c->bias.size();
    out->bias = c->bias.data();
    return TS2_OK;
}

extern "C" int ts2_checkpoint_att_type(const ts2_checkpoint *c, int32_t id, int32_t *width, int32_t *type)
{
    if (!c || id < 0 || id >= (int)(c->attTypes.size() / 2)) {
        return TS2_ERR_SHAPE;
    }
    if (width) {
        *width = c->attTypes[(size_t)id * 2];
    }
    if (type) {
        *type = c->attTypes[(size_t)id * 2 + 1];
    }
    return TS2_OK;
}

extern "C" int ts2_checkpoint_layer(const ts2_checkpoint *c, int32_t layer, int32_t *layerType, float *alibiSlope, int32_t *attTypeId, int32_t *matrixCount)
{
    if (!c || layer < 0 || layer >= (int)c->layerMatr.size()) {
        return TS2_ERR_SHAPE;
    }
    if (layerType) {
        *layerType = c->layers[(size_t)layer * 3];
    }
    if (alibiSlope) {
        memcpy(alibiSlope, &c->layers[(size_t)layer * 3 + 1], 4);
    }
    if (attTypeId) {
        *attTypeId = c->layers[(size_t)layer * 3 + 2];
    }
    if (matrixCount) {
        *matrixCount = (int32_t)c->layerMatr[(size_t)layer].size();
    }
    return TS2_OK;
}

extern "C" int ts2_checkpoint_matrix(const ts2_checkpoint *c, int32_t layer, int32_t matrixId, ts2_checkpoint_matrix_view *out)
{
    if (!c || !out) {
        return TS2_ERR_NULL;
    }
    const std::vector<TMatrixRec> *v = nullptr;
    if (layer == -1) {
        v = &c->modelMatr;
    } else if (layer >= 0 && layer < (int)c->layerMatr.size()) {
        v = &c->layerMatr[(size_t)layer];
    }
    if (!v || matrixId < 0 || matrixId >= (int)v->size()) {
        return TS2_ERR_SHAPE;
    }
    const TMatrixRec &m = (*v)[(size_t)matrixId];
    out->xSize = (int32_t)m.xSize;
    out->ySize = (int32_t)m.ySize;
    out->weights = m.weights.data();
    out->avgGrad = (m.gxSize == m.xSize && m.gySize == m.ySize) ? m.grad1.data() : nullptr;
    out->sumWeight = m.sumWeight;
    out->rowDisp = m.rowDisp.data();
    out->rowDispSize = (int32_t)m.rowDisp.size();
    out->sparsity = m.sparsity;
    return TS2_OK;
}

// PackMatrix, src/gpt/model_params/model_matrix.cpp:6-30 (FP16_PACK): per row the rms as a float, then the row / rms as halves unless the
// rms is zero.  Returns the byte count (it keeps counting past cap so that a NULL / short buffer yields the size needed).
extern "C" int64_t ts2_pack_matrix_fp16(const float *matr, int32_t xSize, int32_t ySize, void *out, int64_t cap)
{
    if (!matr || xSize <= 0 || ySize <= 0 || xSize % 16) {
        return TS2_ERR_SHAPE;
    }
    TWriter w = {(uint8_t *)out, out ? cap : 0};
    std::vector<uint16_t> row((size_t)xSize);
    for (int y = 0; y < ySize; ++y) {
        const float *src = matr + (size_t)y * xSize;
        // CalcRowSum2 (sse_utils.h): eight lanes of partial sums, added up at the end (HorizontalSum)
        float lane[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int x = 0; x < xSize; x += 8) {
            for (int k = 0; k < 8; ++k) {
                lane[k] += src[x + k] * src[x + k];
            }
        }
        // HorizontalSum, src/util/sse_util.h:33-52: (x0+x4 + x2+x6) + (x1+x5 + x3+x7)
        float sum2 = ((lane[0] + lane[4]) + (lane[2] + lane[6])) + ((lane[1] + lane[5]) + (lane[3] + lane[7]));
        float sko = sqrtf(sum2 / xSize);
        w.Put<float>(sko);
        if (sko != 0) {
            float mult = 1 / sko;
            for (int x = 0; x < xSize; ++x) {
                row[(size_t)x] = FloatToHalf(src[x] * mult);
            }
            w.Raw(row.data(), (int64_t)xSize * 2);
        }
    }
    return w.pos;
}

// AddPackedMatrix, model_matrix.cpp:33-58: matr[y][x] += half * (rms * scale)
extern "C" int ts2_add_packed_matrix_fp16(float *matr, int32_t xSize, int32_t ySize, const void *in, int64_t size, float scale)
{
    if (!matr || !in || xSize <= 0 || ySize <= 0 || xSize % 16) {
        return TS2_ERR_SHAPE;
    }
    TReader r = {(const uint8_t *)in, size};
    std::vector<uint16_t> row((size_t)xSize);
    for (int y = 0; y < ySize; ++y) {
        float discrScale = r.Get<float>();
        if (!r.ok) {
            return TS2_ERR_SHAPE;
        }
        if (discrScale != 0) {
            if (!r.Raw(row.data(), (int64_t)xSize * 2)) {
                return TS2_ERR_SHAPE;
            }
            float mult = discrScale * scale;
            float *dst = matr + (size_t)y * xSize;
            for (int x = 0; x < xSize; ++x) {
                dst[x] += HalfToFloat(row[(size_t)x]) * mult;
            }
        }
    }
    return r.pos == size ? TS2_OK : TS2_ERR_SHAPE;
}
