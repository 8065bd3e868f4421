// Test infrastructure only: thin extern "C" wrappers around the reference's own host-compilable CPU sources,
// built by oracle/Makefile from the files where they lie under $(REF)/src into oracle/_ref/libts2ref.so.
// No reference source is copied here; this file only marshals flat arrays into the reference's containers.
// Wrapped reference entry points:
//   src/gpt/compute/cpu_util.cpp:7-186      MulForward, MulBackwardWithAccum, SumRankOne, NormalizeState(+Backward), LoLU(+Backprop)
//   src/gpt/compute/layer_att_reference.h   ComputeDScale, TAttentionComputer::{ComputeValLookup, GradQ, GradK}
//   src/gpt/att/rope.cpp:30-86              FillRopeBuf, ApplyRope
//   src/gpt/att/att.cpp:25-55               TransposeAttention
//   src/gpt/att/sliding_window.cpp:269-306  InitLabelData (labels, targets, spans)
//   src/gpt/model_params/model_dim.cpp      InitModelDescrImpl (layer schedule of a model string)
//   src/gpt/model_params/sse_utils.h:56-204 ConvertArray (fp32->i8), ConvertToFp8e4m3;  src/util/fp8.h:4-21 ConvertE4toFloat
#include <util/pch.h>
#include <math.h>
#include <gpt/compute/cpu_util.h>
#include <gpt/compute/layer_att_reference.h>
#include <gpt/att/rope.h>
#include <gpt/att/att.h>
#include <gpt/att/sliding_window.h>
#include <gpt/data/data.h>
#include <gpt/model_params/model_dim.h>
#include <gpt/model_params/sse_utils.h>
#include <util/fp8.h>
#include <lib/random/mersenne.h>
#include <util/mem_io.h>
#include <gpt/model_params/model_params.h>

static void ToArr(TArray2D<float> *p, const float *src, yint ySize, yint xSize)
{
    p->SetSizes(xSize, ySize);
    for (yint y = 0; y < ySize; ++y) {
        memcpy(p->GetRow(y), src + y * xSize, sizeof(float) * xSize);
    }
}

static void FromArr(float *dst, const TArray2D<float> &a)
{
    yint xSize = a.GetXSize();
    for (yint y = 0; y < a.GetYSize(); ++y) {
        memcpy(dst + y * xSize, a.GetRow(y), sizeof(float) * xSize);
    }
}

static void ToAtt(TAttentionInfo *p, int len, const int *spanPtr, const int *spans)
{
    p->Init();
    for (int t = 0; t < len; ++t) {
        for (int k = spanPtr[t]; k < spanPtr[t + 1]; ++k) {
            p->AddSpan(TAttentionSpan(spans[k * 2], spans[k * 2 + 1]));
        }
        p->AddSample();
    }
}

extern "C" {

void ref_mul_forward(const float *vec, const float *kqv, float *res, int len, int dim, int rDim)
{
    TArray2D<float> v, m;
    ToArr(&v, vec, len, dim);
    ToArr(&m, kqv, rDim, dim);
    FromArr(res, MulForward(v, m));
}

void ref_mul_backward_accum(float *vecGrad, const float *kqv, const float *resGrad, int len, int dim, int rDim)
{
    TArray2D<float> g, m, r;
    ToArr(&g, vecGrad, len, dim);
    ToArr(&m, kqv, rDim, dim);
    ToArr(&r, resGrad, len, rDim);
    MulBackwardWithAccum(&g, m, r);
    FromArr(vecGrad, g);
}

void ref_sum_rank_one(const float *vec, float *delta, const float *resGrad, int len, int dim, int rDim)
{
    TArray2D<float> v, d, r;
    ToArr(&v, vec, len, dim);
    ToArr(&r, resGrad, len, rDim);
    SumRankOne(v, &d, r);
    FromArr(delta, d);
}

void ref_normalize_state(const float *state, float *res, int len, int dim, int headCount)
{
    TArray2D<float> s;
    ToArr(&s, state, len, dim);
    FromArr(res, NormalizeState(s, headCount));
}

void ref_normalize_state_backward(const float *state, const float *dNorm, float *grad, int len, int dim, int headCount)
{
    TArray2D<float> s, d, g;
    ToArr(&s, state, len, dim);
    ToArr(&d, dNorm, len, dim);
    NormalizeStateBackward(s, headCount, d, &g);
    FromArr(grad, g);
}

void ref_lolu(const float *gate, const float *vals, float *res, int len, int dim)
{
    TArray2D<float> g, v, r;
    ToArr(&g, gate, len, dim);
    ToArr(&v, vals, len, dim);
    LoLU(g, v, &r);
    FromArr(res, r);
}

void ref_backprop_lolu(const float *gate, const float *vals, const float *grad, float *gradGate, float *gradVals, int len, int dim)
{
    TArray2D<float> g, v, d, gg, gv;
    ToArr(&g, gate, len, dim);
    ToArr(&v, vals, len, dim);
    ToArr(&d, grad, len, dim);
    BackpropLoLU(g, v, d, &gg, &gv);
    FromArr(gradGate, gg);
    FromArr(gradVals, gv);
}

void ref_fill_rope_buf(float *buf, int width, int ropeLen)
{
    TArray2D<float> r;
    FillRopeBuf(&r, width, ropeLen);
    FromArr(buf, r);
}

void ref_apply_rope(const float *ropeBuf, int width, int ropeLen, float dir, float *p, int len, int dim)
{
    TArray2D<float> r, v;
    ToArr(&r, ropeBuf, ropeLen, width);
    ToArr(&v, p, len, dim);
    ApplyRope(r, dir, &v);
    FromArr(p, v);
}

// returns number of spans of the transposed graph; outputs sized by the caller (at most edge count)
int ref_transpose_attention(int len, const int *spanPtr, const int *spans, int *resPtr, int *resSpans, int maxSpans)
{
    TAttentionInfo att;
    ToAtt(&att, len, spanPtr, spans);
    TAttentionInfo rev = TransposeAttention(att);
    yint n = YSize(rev.Spans);
    if (n > maxSpans) {
        return -1;
    }
    for (yint k = 0; k <= len; ++k) {
        resPtr[k] = rev.SpanPtr[k];
    }
    for (yint k = 0; k < n; ++k) {
        resSpans[k * 2] = rev.Spans[k].Start;
        resSpans[k * 2 + 1] = rev.Spans[k].Finish;
    }
    return (int)n;
}

// full attention forward + backward of the reference's CPU computer
// q,k [len][heads*qDim], v,dVal [len][heads*ttDim]; outputs same shapes; sumWeight,maxDP,dScale [heads][len]
void ref_attention(int len, int heads, int qDim, int ttDim, float alibiSlope, float attScaleMult, const int *spanPtr, const int *spans,
    const float *q, const float *k, const float *v, const float *dVal, float *valLookup, float *sumWeight, float *maxDP, float *dScale,
    float *dq, float *dk, float *dv)
{
    TModelDims dims;
    dims.QDim = qDim;
    dims.TTDim = ttDim;
    dims.HeadCount = heads;
    TAttentionInfo att;
    ToAtt(&att, len, spanPtr, spans);
    TAttentionInfo rev = TransposeAttention(att);
    TArray2D<float> aq, ak, av, ad, val, ds, gq, gk, gv;
    ToArr(&aq, q, len, heads * qDim);
    ToArr(&ak, k, len, heads * qDim);
    ToArr(&av, v, len, heads * ttDim);
    TAttentionComputer comp(dims, alibiSlope, attScaleMult);
    comp.ComputeValLookup(len, dims, aq, ak, av, att, &val);
    FromArr(valLookup, val);
    FromArr(sumWeight, comp.SumWeight);
    FromArr(maxDP, comp.MaxDP);
    if (dVal) {
        ToArr(&ad, dVal, len, heads * ttDim);
        ComputeDScale(dims, val, ad, &ds);
        FromArr(dScale, ds);
        TAttentionComputer::TGradData gd(dims, aq, ak, av, ad, ds);
        comp.GradQ(len, dims, gd, att, &gq);
        comp.GradK(len, dims, gd, rev, &gk, &gv);
        FromArr(dq, gq);
        FromArr(dk, gk);
        FromArr(dv, gv);
    }
}

void ref_convert_i8(signed char *dst, const float *src, int xSize, float mult)
{
    // ConvertArray needs 32-byte aligned input and a multiple of 32 elements
    float *buf = (float *)aligned_alloc(32, sizeof(float) * xSize);
    i8 *out = (i8 *)aligned_alloc(32, xSize);
    memcpy(buf, src, sizeof(float) * xSize);
    ConvertArray(out, buf, xSize, _mm256_set1_ps(mult));
    memcpy(dst, out, xSize);
    free(buf);
    free(out);
}

void ref_convert_e4m3(unsigned char *dst, const float *src, int xSize, float mult)
{
    float *buf = (float *)aligned_alloc(32, sizeof(float) * xSize);
    memcpy(buf, src, sizeof(float) * xSize);
    ConvertToFp8e4m3((e4m3 *)dst, buf, xSize, _mm256_set1_ps(mult));
    free(buf);
}

float ref_e4m3_to_float(int code)
{
    return ConvertE4toFloat((i8)code);
}

// layer schedule of a model string: per layer {type, attentionTypeId, slope}; attention widths per type
int ref_model_descr(const char *descr, int *dims10, int *layerType, int *layerAttId, float *layerSlope, int maxLayers, int *attWidth, int *attTypeCount)
{
    TModelDescr md;
    InitModelDescrImpl(&md, descr, 0, 0, 0, 0);
    int *d = dims10;
    d[0] = md.Dims.Dim; d[1] = md.Dims.QDim; d[2] = md.Dims.TTDim; d[3] = md.Dims.ExpertDim; d[4] = md.Dims.HeadCount;
    d[5] = md.Dims.FfnTiles; d[6] = md.Dims.MoeExpertCount; d[7] = md.Dims.MoeSelected; d[8] = md.Dims.KVrep; d[9] = md.Dims.Depth;
    yint n = YSize(md.LayerArr);
    if (n > maxLayers) {
        return -1;
    }
    for (yint k = 0; k < n; ++k) {
        layerType[k] = md.LayerArr[k].LayerType;
        layerAttId[k] = md.LayerArr[k].AttentionTypeId;
        layerSlope[k] = md.LayerArr[k].AlibiSlope;
    }
    *attTypeCount = (int)YSize(md.AttentionTypeArr);
    for (yint k = 0; k < YSize(md.AttentionTypeArr); ++k) {
        attWidth[k] = md.AttentionTypeArr[k].Width;
    }
    return (int)n;
}

// node construction for a batch of equal-length fragments, noise labels disabled, tokenDrop = 1 (never drop)
// tokens/targets [fragCount][fragLen] (target < 0 = undefined); outputs: labelPtr[n+1], labels (<= 3n), targets pairs, per att type CSR spans
int ref_init_label_data(const char *descr, int vocab, int fragCount, int fragLen, const int *tokens, const int *targets, int *labelCount,
    int *labelPtr, unsigned *labels, int *targetCount, int *targetPairs, int attType, int *spanPtr, int *spans)
{
    TModelDescr md;
    InitModelDescr(&md, descr, vocab, vocab, MPF_DISABLE_NOISE_LABELS);
    *labelCount = (int)md.LabelCount;
    TVector<TFragment> fragArr;
    fragArr.resize(fragCount);
    for (int f = 0; f < fragCount; ++f) {
        for (int t = 0; t < fragLen; ++t) {
            fragArr[f].Text.push_back(tokens[f * fragLen + t]);
            int tg = targets[f * fragLen + t];
            fragArr[f].Target.push_back(tg < 0 ? UNDEFINED_TOKEN : (TBPEToken)tg);
        }
    }
    TXRng rng(1313);
    TBatchNodes nodes;
    InitLabelData(md, rng, 1.0f, fragArr, ATT_GRAPH_TRAIN_LOSS, &nodes);
    yint n = nodes.GetNodeCount();
    for (yint k = 0; k <= n; ++k) {
        labelPtr[k] = nodes.Labels.LabelPtr[k];
    }
    for (yint k = 0; k < YSize(nodes.Labels.LabelArr); ++k) {
        labels[k] = nodes.Labels.LabelArr[k];
    }
    *targetCount = (int)YSize(nodes.Target);
    for (yint k = 0; k < YSize(nodes.Target); ++k) {
        targetPairs[k * 2] = (int)nodes.Target[k].Node;
        targetPairs[k * 2 + 1] = (int)nodes.Target[k].TargetId;
    }
    const TAttentionInfo &att = nodes.AttArr[attType];
    for (yint k = 0; k <= n; ++k) {
        spanPtr[k] = att.SpanPtr[k];
    }
    for (yint k = 0; k < YSize(att.Spans); ++k) {
        spans[k * 2] = att.Spans[k].Start;
        spans[k * 2 + 1] = att.Spans[k].Finish;
    }
    return (int)n;
}


// the input of the reference's own sort test (TestCudaSort, src/lib/cuda/cuda_sort.cu:232-247): n draws of TMersenne<ui32>(seed).GenRandReal3()
void ref_mersenne_real3(unsigned seed, int n, float *out)
{
    TMersenne<ui32> rng(seed);
    for (int i = 0; i < n; ++i) {
        out[i] = (float)rng.GenRandReal3();
    }
}


// a checkpoint as the reference writes it: a TModelParams laid out like AllocateModel does (src/gpt/model_params/model_params.cpp:142-163)
// for a model string, every matrix filled from a small deterministic generator (InitModel's threads are not needed for the format), the
// optimiser state of one matrix set, serialised with SAVELOAD (TModelParams, model_params.h:7-18) into memory.
// Returns the byte count (or -needed when cap is too small).
static float CkValue(unsigned *state)
{
    *state = *state * 1664525u + 1013904223u;
    return ((int)(*state >> 8) % 2001 - 1000) * (1.f / 1024);
}

static void CkFill(TModelMatrix *mm, unsigned *state)
{
    TArray2D<float> a, g;
    a.SetSizes(mm->GetXSize(), mm->GetYSize());
    g.SetSizes(mm->GetXSize(), mm->GetYSize());
    for (yint y = 0; y < mm->GetYSize(); ++y) {
        for (yint x = 0; x < mm->GetXSize(); ++x) {
            a[y][x] = CkValue(state);
            g[y][x] = CkValue(state) * 0.25f;
        }
    }
    mm->SetMatrix(a);
    mm->GetGrad1() = g;
}

long ref_make_checkpoint(const char *descr, int vocab, unsigned seed, char *out, long cap)
{
    TModelDescr md;
    InitModelDescr(&md, descr, vocab, vocab, MPF_DISABLE_NOISE_LABELS);
    TModelParams params;
    params.ModelDescr = md;
    yint dim = md.Dims.Dim;
    params.MatrArr.resize(MP_MODEL_COUNT);
    params.MatrArr[MP_MODEL_EMBED].SetSizesPerRowDisp(dim, md.LabelCount, 1);
    params.MatrArr[MP_MODEL_FINAL].SetSizesPerRowDisp(dim, md.OutputTokenCount, 1);
    yint depth = YSize(md.LayerArr);
    params.LayerArr.resize(depth);
    for (yint d = 0; d < depth; ++d) {
        TModelParams::TAttentionMatrices &dst = params.LayerArr[d];
        dst.MatrArr.resize(MP_MAX_COUNT);
        yint ptr = 0;
        md.EnumLayerMatrices(d, [&](yint xSize, yint ySize, float noise, float moeFraction) {
            dst.MatrArr[ptr++].SetSizesPerMatrixDisp(xSize, ySize, moeFraction);
        });
        dst.MatrArr.resize(ptr);
    }
    unsigned state = seed;
    params.ForEachModelMatrix([&](TModelMatrix &mm) { CkFill(&mm, &state); });
    params.Bias.resize(vocab);
    for (int k = 0; k < vocab; ++k) {
        params.Bias[k] = 0.01f * k;
    }
    {
        TVector<float> rd(params.MatrArr[MP_MODEL_FINAL].GetRowDisp().size(), 0.f);
        for (yint k = 0; k < YSize(rd); ++k) {
            rd[k] = 0.125f + k;
        }
        params.MatrArr[MP_MODEL_FINAL].SetRowDisp(2.5f, rd);
        params.LayerArr[0].MatrArr[0].SetRowDisp(1.5f, TVector<float>(1, 0.75f));
    }
    TVector<char> data;
    SerializeMem(IO_WRITE, &data, params);
    if ((long)data.size() > cap) {
        return -(long)data.size();
    }
    memcpy(out, data.data(), data.size());
    return (long)data.size();
}

// PackMatrix / AddPackedMatrix (src/gpt/model_params/model_matrix.cpp:6-58): the fp16-row wire format
long ref_pack_matrix(const float *matr, int xSize, int ySize, char *out, long cap)
{
    // (the AVX code of the reference reads and writes rows with aligned accesses)
    float *m = (float *)aligned_alloc(64, sizeof(float) * xSize * ySize);
    memcpy(m, matr, sizeof(float) * xSize * ySize);
    TVector<char> data;
    {
        TMemStream f(&data);
        {
            TBufferedStream bufIO(IO_WRITE, f);
            PackMatrix(bufIO, THost2DPtr<float>(m, xSize * sizeof(float), xSize, ySize));
        }
        f.Swap(&data);
    }
    free(m);
    if ((long)data.size() > cap) {
        return -(long)data.size();
    }
    memcpy(out, data.data(), data.size());
    return (long)data.size();
}

void ref_add_packed_matrix(float *matr, int xSize, int ySize, const char *in, long size, float scale)
{
    float *m = (float *)aligned_alloc(64, sizeof(float) * xSize * ySize);
    memcpy(m, matr, sizeof(float) * xSize * ySize);
    TVector<char> data(in, in + size);
    {
        TMemStream f(&data);
        TBufferedStream bufIO(IO_READ, f);
        AddPackedMatrix(THost2DPtr<float>(m, xSize * sizeof(float), xSize, ySize), bufIO, scale);
    }
    memcpy(matr, m, sizeof(float) * xSize * ySize);
    free(m);
}

}
