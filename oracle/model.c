/* CPU oracle (test infrastructure only): the reference's CPU layers and one full training step (forward, loss gradient,
 * backward through all layers, embedding delta).  Deltas are the raw fp32 matrices the reference hands to HostApplyDelta. */
#include "oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>

static float *NewF(size_t n)
{
    return (float *)calloc(n ? n : 1, sizeof(float));
}

static void AddTo(float *dst, const float *src, size_t n)
{
    for (size_t i = 0; i < n; ++i) {
        dst[i] += src[i] * 1;
    }
}

/* src/gpt/compute/cpu_util.h:86-95 MatmulBackprop / MatmulBackpropNoScale: dSrc += dDst*W/sqrt(in); delta = SumRankOne(src, dDst) */
static void MatmulBackprop(const float *w, float *delta, const float *src, const float *dstGrad, float *srcGrad, int len, int dim, int rDim)
{
    orc_mul_backward_accum(srcGrad, w, dstGrad, len, dim, rDim);
    if (delta) {
        orc_sum_rank_one(src, delta, dstGrad, len, dim, rDim);
    }
}

/* ---------------------------------------------------------------------------------------------------------------------------
 * FFN: src/gpt/compute/layer_ffn.cu:190-211 (forward) and :213-248 (backward) */
static void FfnCompute(const orc_dims *d, const orc_layer *l, int len, const float *prevState, float *normState, float *wide,
    float *wideNorm, float *gate, float *rg)
{
    int dim = d->dim, ffn = d->ffnDim;
    orc_normalize_state(prevState, normState, len, dim, dim / ORC_STATE_NORM_TILE);
    orc_mul_forward(normState, l->w[0], wide, len, dim, ffn);
    orc_normalize_state(wide, wideNorm, len, ffn, ffn / 128);
    orc_mul_forward(normState, l->w[1], gate, len, dim, ffn);
    orc_lolu(gate, wideNorm, rg, len, ffn);
}

static void FfnForward(const orc_dims *d, const orc_layer *l, int len, const float *prevState, float *state)
{
    int dim = d->dim, ffn = d->ffnDim;
    size_t nd = (size_t)len * dim, nf = (size_t)len * ffn;
    float *normState = NewF(nd), *wide = NewF(nf), *wideNorm = NewF(nf), *gate = NewF(nf), *rg = NewF(nf), *delta = NewF(nd);
    FfnCompute(d, l, len, prevState, normState, wide, wideNorm, gate, rg);
    orc_mul_forward(rg, l->w[2], delta, len, ffn, dim);
    memcpy(state, prevState, sizeof(float) * nd);
    AddTo(state, delta, nd);
    free(normState); free(wide); free(wideNorm); free(gate); free(rg); free(delta);
}

static void FfnBackward(const orc_dims *d, const orc_layer *l, int len, const float *prevState, float *grad)
{
    int dim = d->dim, ffn = d->ffnDim;
    size_t nd = (size_t)len * dim, nf = (size_t)len * ffn;
    float *normState = NewF(nd), *wide = NewF(nf), *wideNorm = NewF(nf), *gate = NewF(nf), *rg = NewF(nf);
    float *dNormState = NewF(nd), *drg = NewF(nf), *dgate = NewF(nf), *dwide = NewF(nf), *dsg = NewF(nd);
    FfnCompute(d, l, len, prevState, normState, wide, wideNorm, gate, rg);
    MatmulBackprop(l->w[2], l->delta[2], rg, grad, drg, len, ffn, dim);
    orc_backprop_lolu(gate, wideNorm, drg, dgate, dwide, len, ffn);
    orc_normalize_state_backward(wide, dwide, dwide, len, ffn, ffn / 128);
    MatmulBackprop(l->w[0], l->delta[0], normState, dwide, dNormState, len, dim, ffn);
    MatmulBackprop(l->w[1], l->delta[1], normState, dgate, dNormState, len, dim, ffn);
    orc_normalize_state_backward(prevState, dNormState, dsg, len, dim, dim / ORC_STATE_NORM_TILE);
    AddTo(grad, dsg, nd);
    free(normState); free(wide); free(wideNorm); free(gate); free(rg);
    free(dNormState); free(drg); free(dgate); free(dwide); free(dsg);
}

/* ---------------------------------------------------------------------------------------------------------------------------
 * attention: src/gpt/compute/layer_att.cu:368-405 (forward) and :407-482 (backward) */
typedef struct {
    float *normState, *qSrc, *kSrc, *gate, *vSrc, *q, *k, *v, *val, *rg, *sumWeight, *maxDP;
} TAttBufs;

static void AttAlloc(TAttBufs *b, const orc_dims *d, int len)
{
    size_t nd = (size_t)len * d->dim, nq = (size_t)len * d->qDim * d->headCount, nt = (size_t)len * d->ttDim * d->headCount;
    b->normState = NewF(nd);
    b->qSrc = NewF(nq); b->kSrc = NewF(nq); b->q = NewF(nq); b->k = NewF(nq);
    b->gate = NewF(nt); b->vSrc = NewF(nt); b->v = NewF(nt); b->val = NewF(nt); b->rg = NewF(nt);
    b->sumWeight = NewF((size_t)len * d->headCount);
    b->maxDP = NewF((size_t)len * d->headCount);
}

static void AttFree(TAttBufs *b)
{
    free(b->normState); free(b->qSrc); free(b->kSrc); free(b->q); free(b->k); free(b->gate); free(b->vSrc); free(b->v);
    free(b->val); free(b->rg); free(b->sumWeight); free(b->maxDP);
}

static void AttCompute(const orc_dims *d, const orc_layer *l, const orc_common *c, int len, const float *prevState, TAttBufs *b)
{
    int dim = d->dim, heads = d->headCount, qSum = d->qDim * heads, ttSum = d->ttDim * heads;
    int a = l->attTypeId;
    orc_normalize_state(prevState, b->normState, len, dim, dim / ORC_STATE_NORM_TILE);
    orc_mul_forward(b->normState, l->w[0], b->qSrc, len, dim, qSum);
    orc_mul_forward(b->normState, l->w[1], b->kSrc, len, dim, qSum);
    orc_mul_forward(b->normState, l->w[3], b->gate, len, dim, ttSum);
    orc_mul_forward(b->normState, l->w[2], b->vSrc, len, dim, ttSum);
    orc_normalize_state(b->qSrc, b->q, len, qSum, heads);
    memcpy(b->k, b->kSrc, sizeof(float) * (size_t)len * qSum);
    orc_normalize_state(b->vSrc, b->v, len, ttSum, heads);
    orc_apply_rope(c->ropeBuf, d->qDim, 1, b->q, len, qSum);
    orc_apply_rope(c->ropeBuf, d->qDim, 1, b->k, len, qSum);
    orc_attention_forward(len, heads, d->qDim, d->ttDim, l->alibiSlope, 1.0f, c->spanPtr[a], c->spans[a], b->q, b->k, b->v, b->val,
        b->sumWeight, b->maxDP);
    orc_lolu(b->gate, b->val, b->rg, len, ttSum);
}

static void AttForward(const orc_dims *d, const orc_layer *l, const orc_common *c, int len, const float *prevState, float *state)
{
    size_t nd = (size_t)len * d->dim;
    TAttBufs b;
    AttAlloc(&b, d, len);
    AttCompute(d, l, c, len, prevState, &b);
    float *delta = NewF(nd);
    orc_mul_forward(b.rg, l->w[4], delta, len, d->ttDim * d->headCount, d->dim);
    memcpy(state, prevState, sizeof(float) * nd);
    AddTo(state, delta, nd);
    free(delta);
    AttFree(&b);
}

static void AttBackward(const orc_dims *d, const orc_layer *l, const orc_common *c, int len, const float *prevState, float *grad)
{
    int dim = d->dim, heads = d->headCount, qSum = d->qDim * heads, ttSum = d->ttDim * heads;
    int a = l->attTypeId;
    size_t nd = (size_t)len * dim, nq = (size_t)len * qSum, nt = (size_t)len * ttSum;
    TAttBufs b;
    AttAlloc(&b, d, len);
    AttCompute(d, l, c, len, prevState, &b);
    float *dNormState = NewF(nd), *drg = NewF(nt), *dgate = NewF(nt), *dVal = NewF(nt), *dScale = NewF((size_t)len * heads);
    float *dQ = NewF(nq), *dK = NewF(nq), *dV = NewF(nt), *dsg = NewF(nd);
    /* combiner backprop */
    MatmulBackprop(l->w[4], l->delta[4], b.rg, grad, drg, len, ttSum, dim);
    /* lolu backprop */
    orc_backprop_lolu(b.gate, b.val, drg, dgate, dVal, len, ttSum);
    /* attention backprop */
    orc_compute_dscale(len, heads, d->ttDim, b.val, dVal, dScale);
    orc_attention_grad_q(len, heads, d->qDim, d->ttDim, l->alibiSlope, 1.0f, c->spanPtr[a], c->spans[a], b.q, b.k, b.v, dVal, dScale,
        b.sumWeight, b.maxDP, dQ);
    orc_attention_grad_k(len, heads, d->qDim, d->ttDim, l->alibiSlope, 1.0f, c->revPtr[a], c->revSpans[a], b.q, b.k, b.v, dVal, dScale,
        b.sumWeight, b.maxDP, dK, dV);
    orc_apply_rope(c->ropeBuf, d->qDim, -1, dQ, len, qSum);
    orc_apply_rope(c->ropeBuf, d->qDim, -1, dK, len, qSum);
    orc_normalize_state_backward(b.qSrc, dQ, dQ, len, qSum, heads);
    orc_normalize_state_backward(b.vSrc, dV, dV, len, ttSum, heads);
    /* matmul backprop */
    MatmulBackprop(l->w[0], l->delta[0], b.normState, dQ, dNormState, len, dim, qSum);
    MatmulBackprop(l->w[1], l->delta[1], b.normState, dK, dNormState, len, dim, qSum);
    MatmulBackprop(l->w[2], l->delta[2], b.normState, dV, dNormState, len, dim, ttSum);
    MatmulBackprop(l->w[3], l->delta[3], b.normState, dgate, dNormState, len, dim, ttSum);
    orc_normalize_state_backward(prevState, dNormState, dsg, len, dim, dim / ORC_STATE_NORM_TILE);
    AddTo(grad, dsg, nd);
    free(dNormState); free(drg); free(dgate); free(dVal); free(dScale); free(dQ); free(dK); free(dV); free(dsg);
    AttFree(&b);
}

/* ---------------------------------------------------------------------------------------------------------------------------
 * MoE: src/gpt/compute/layer_moe.cu:458-486 (forward) and :488-537 (backward); every expert is evaluated densely */
typedef struct {
    float *normState, *wide, *wideNorm, *gate, *moeSrc, *rgSrc, *moe, *rg, *contractFwd;
} TMoeBufs;

static void MoeAlloc(TMoeBufs *b, const orc_dims *d, int len)
{
    int moeDim = d->expertDim * d->expertCount;
    size_t nd = (size_t)len * d->dim, nm = (size_t)len * moeDim, ne = (size_t)len * d->expertCount;
    b->normState = NewF(nd);
    b->wide = NewF(nm); b->wideNorm = NewF(nm); b->gate = NewF(nm); b->rgSrc = NewF(nm); b->rg = NewF(nm);
    b->moeSrc = NewF(ne); b->moe = NewF(ne);
    b->contractFwd = NewF((size_t)d->dim * moeDim);
}

static void MoeFree(TMoeBufs *b)
{
    free(b->normState); free(b->wide); free(b->wideNorm); free(b->gate); free(b->rgSrc); free(b->rg); free(b->moeSrc); free(b->moe);
    free(b->contractFwd);
}

static void MoeCompute(const orc_dims *d, const orc_layer *l, int len, const float *prevState, TMoeBufs *b)
{
    int dim = d->dim, E = d->expertCount, moeDim = d->expertDim * E;
    orc_normalize_state(prevState, b->normState, len, dim, dim / ORC_STATE_NORM_TILE);
    orc_mul_forward(b->normState, l->w[0], b->wide, len, dim, moeDim);
    orc_normalize_state(b->wide, b->wideNorm, len, moeDim, moeDim / 128);
    orc_mul_forward(b->normState, l->w[1], b->gate, len, dim, moeDim);
    orc_mul_forward(b->normState, l->w[3], b->moeSrc, len, dim, E);
    orc_lolu(b->gate, b->wideNorm, b->rgSrc, len, moeDim);
    orc_cpu_moe(len, E, d->moeSelected, b->moeSrc, b->moe);
    memcpy(b->rg, b->rgSrc, sizeof(float) * (size_t)len * moeDim);
    orc_scale_experts(len, E, moeDim, b->moe, b->rg);
    /* contract matrix [E*dim][xp] -> [dim][E*xp] */
    orc_fwd_contract_matrix(l->w[2], b->contractFwd, E, dim, d->expertDim);
}

static void MoeForward(const orc_dims *d, const orc_layer *l, int len, const float *prevState, float *state)
{
    size_t nd = (size_t)len * d->dim;
    int moeDim = d->expertDim * d->expertCount;
    TMoeBufs b;
    MoeAlloc(&b, d, len);
    MoeCompute(d, l, len, prevState, &b);
    float *delta = NewF(nd);
    orc_mul_forward(b.rg, b.contractFwd, delta, len, moeDim, d->dim);
    memcpy(state, prevState, sizeof(float) * nd);
    AddTo(state, delta, nd);
    free(delta);
    MoeFree(&b);
}

static void MoeBackward(const orc_dims *d, const orc_layer *l, int len, const float *prevState, float *grad)
{
    int dim = d->dim, E = d->expertCount, moeDim = d->expertDim * E;
    size_t nd = (size_t)len * dim, nm = (size_t)len * moeDim, ne = (size_t)len * E;
    TMoeBufs b;
    MoeAlloc(&b, d, len);
    MoeCompute(d, l, len, prevState, &b);
    float *dNormState = NewF(nd), *drg = NewF(nm), *dMoe = NewF(ne), *dgate = NewF(nm), *dwide = NewF(nm), *dsg = NewF(nd);
    /* ContractMatmulBackprop, src/gpt/compute/layer_moe.cu:443-452 */
    orc_mul_backward_accum(drg, b.contractFwd, grad, len, moeDim, dim);
    if (l->delta[2]) {
        float *delta = NewF((size_t)dim * moeDim);
        orc_sum_rank_one(b.rg, delta, grad, len, moeDim, dim);
        orc_bwd_contract_matrix(delta, l->delta[2], E, dim, d->expertDim);
        free(delta);
    }
    orc_backprop_scale_experts(len, E, moeDim, b.moe, b.rgSrc, dMoe, drg);
    orc_cpu_backprop_moe(len, E, b.moe, dMoe);
    MatmulBackprop(l->w[3], l->delta[3], b.normState, dMoe, dNormState, len, dim, E);
    orc_backprop_lolu(b.gate, b.wideNorm, drg, dgate, dwide, len, moeDim);
    orc_normalize_state_backward(b.wide, dwide, dwide, len, moeDim, moeDim / 128);
    MatmulBackprop(l->w[0], l->delta[0], b.normState, dwide, dNormState, len, dim, moeDim);
    MatmulBackprop(l->w[1], l->delta[1], b.normState, dgate, dNormState, len, dim, moeDim);
    orc_normalize_state_backward(prevState, dNormState, dsg, len, dim, dim / ORC_STATE_NORM_TILE);
    AddTo(grad, dsg, nd);
    free(dNormState); free(drg); free(dMoe); free(dgate); free(dwide); free(dsg);
    MoeFree(&b);
}

/* src/gpt/compute/layer.h:66-67 TLayerBase::ComputeForward / ComputeBackward */
void orc_layer_forward(const orc_dims *d, const orc_layer *l, const orc_common *c, int len, const float *prevState, float *state)
{
    if (l->type == ORC_LT_FFN) {
        FfnForward(d, l, len, prevState, state);
    } else if (l->type == ORC_LT_ATT) {
        AttForward(d, l, c, len, prevState, state);
    } else if (l->type == ORC_LT_MOE) {
        MoeForward(d, l, len, prevState, state);
    } else {
        abort();
    }
}

void orc_layer_backward(const orc_dims *d, const orc_layer *l, const orc_common *c, int len, const float *prevState, float *grad)
{
    if (l->type == ORC_LT_FFN) {
        FfnBackward(d, l, len, prevState, grad);
    } else if (l->type == ORC_LT_ATT) {
        AttBackward(d, l, c, len, prevState, grad);
    } else if (l->type == ORC_LT_MOE) {
        MoeBackward(d, l, len, prevState, grad);
    } else {
        abort();
    }
}

/* src/gpt/model_params/model_dim.cpp:82-158 InitAlibi, the ALIBI_V3 branch (no RNN flags): attention types {1, 64, wide};
 * depth 1 is a profiling special case (one wide attention with slope 0.1 + one ffn/moe) */
int orc_model_schedule(int depth, int moeExpertCount, int wideWindow, int *layerType, int *layerAttId, float *layerSlope, int maxLayers,
    int *attWidth, int *attTypeCount)
{
    int n = 0;
#define ADD(lt, id, sl)                                                                                                                    \
    do {                                                                                                                                   \
        if (n >= maxLayers)                                                                                                                \
            return -1;                                                                                                                     \
        layerType[n] = lt;                                                                                                                 \
        layerAttId[n] = id;                                                                                                                \
        layerSlope[n] = sl;                                                                                                                \
        ++n;                                                                                                                               \
    } while (0)
    int ffn = moeExpertCount > 0 ? ORC_LT_MOE : ORC_LT_FFN;
    if (depth == 1) {
        attWidth[0] = wideWindow;
        *attTypeCount = 1;
        ADD(ORC_LT_ATT, 0, 0.1f);
        ADD(ffn, 0, 0);
        return n;
    }
    attWidth[0] = 1;
    attWidth[1] = 64;
    attWidth[2] = wideWindow;
    *attTypeCount = 3;
    if (depth > 0) {
        int groupCount = (depth + 1) / 2;
        int w1count = groupCount / 6 > 1 ? groupCount / 6 : 1;
        for (int k = 0; k < w1count; ++k) {
            ADD(ORC_LT_ATT, 0, 0.0f);
            ADD(ORC_LT_FFN, 0, 0);
            ADD(ORC_LT_ATT, 0, 0.0f);
            ADD(ORC_LT_FFN, 0, 0);
        }
        for (int k = w1count; k < groupCount; ++k) {
            ADD(ORC_LT_ATT, 1, 0.5f);
            ADD(ffn, 0, 0);
            ADD(ORC_LT_ATT, 2, 0.0f);
            ADD(ffn, 0, 0);
        }
    }
#undef ADD
    return n;
}

/* src/gpt/compute/cpu_transformer.cpp:76-100 ComputeEmbedding: state0[t] = sum over labels of +-embed[label] */
void orc_embedding_forward(int len, int dim, const int *labelPtr, const uint32_t *labels, const float *embed, float *state)
{
    memset(state, 0, sizeof(float) * (size_t)len * dim);
    for (int t = 0; t < len; ++t) {
        for (int k = labelPtr[t]; k < labelPtr[t + 1]; ++k) {
            uint32_t label = labels[k];
            float w = (label & 0x80000000u) ? -1 : 1;
            label &= 0x7fffffffu;
            for (int x = 0; x < dim; ++x) {
                state[(size_t)t * dim + x] += embed[(size_t)label * dim + x] * w;
            }
        }
    }
}

/* src/gpt/compute/cpu_transformer.cpp:182-197 embedding delta */
void orc_embedding_backward(int len, int dim, int labelCount, const int *labelPtr, const uint32_t *labels, const float *grad, float *deltaLabel)
{
    memset(deltaLabel, 0, sizeof(float) * (size_t)labelCount * dim);
    for (int t = 0; t < len; ++t) {
        for (int k = labelPtr[t]; k < labelPtr[t + 1]; ++k) {
            uint32_t label = labels[k];
            float w = (label & 0x80000000u) ? -1 : 1;
            label &= 0x7fffffffu;
            for (int x = 0; x < dim; ++x) {
                deltaLabel[(size_t)label * dim + x] += grad[(size_t)t * dim + x] * w;
            }
        }
    }
}

/* src/gpt/compute/cpu_transformer.cpp:12-37 SoftMax: base 2, running max starts at 0, double sum */
void orc_softmax2(const float *logits, const float *bias, float *pred, int len, int dim)
{
#pragma omp parallel for schedule(static)
    for (int t = 0; t < len; ++t) {
        float maxVal = 0;
        for (int k = 0; k < dim; ++k) {
            maxVal = fmaxf(maxVal, logits[(size_t)t * dim + k]);
        }
        double sumWeight = 0;
        for (int k = 0; k < dim; ++k) {
            float val = logits[(size_t)t * dim + k];
            float w = exp2f(val + bias[k] - maxVal);
            pred[(size_t)t * dim + k] = w;
            sumWeight += w;
        }
        float scale = 1 / sumWeight;
        for (int k = 0; k < dim; ++k) {
            pred[(size_t)t * dim + k] *= scale;
        }
    }
}

/* src/gpt/compute/cpu_transformer.cpp:119-172: final norm, logits/ln2, softmax2, gradient (onehot - p) on target nodes scaled by
 * (1/ln2)*ln2, dState through the final matrix and the final norm; deltaFinal = SumRankOne(finalNormState, gradArr).
 * pred is [len][vocab] (out), grad is [len][dim] (out, overwritten), targetPairs = {node, targetId}. */
void orc_final_backward(int len, int dim, int vocab, const float *lastState, const float *finalW, const float *bias, int targetCount,
    const int *targetPairs, float *pred, float *grad, float *deltaFinal)
{
    size_t nd = (size_t)len * dim, nv = (size_t)len * vocab;
    float *finalNorm = NewF(nd), *logits = NewF(nv), *gradArr = NewF(nv), *normStateGrad = NewF(nd);
    float finalMult = 1.f / ORC_LOG2; /* FINAL_LAYER_SOFTMAX_SCALE / LOG2 */
    orc_normalize_state(lastState, finalNorm, len, dim, dim / ORC_STATE_NORM_TILE);
    orc_mul_forward(finalNorm, finalW, logits, len, dim, vocab);
    for (size_t i = 0; i < nv; ++i) {
        logits[i] *= finalMult;
    }
    orc_softmax2(logits, bias, pred, len, vocab);
    for (int k = 0; k < targetCount; ++k) {
        int node = targetPairs[k * 2], target = targetPairs[k * 2 + 1];
        for (int q = 0; q < vocab; ++q) {
            gradArr[(size_t)node * vocab + q] += -pred[(size_t)node * vocab + q];
        }
        gradArr[(size_t)node * vocab + target] += 1;
    }
    float gs = finalMult * ORC_LOG2;
    for (size_t i = 0; i < nv; ++i) {
        gradArr[i] *= gs;
    }
    orc_mul_backward_accum(normStateGrad, finalW, gradArr, len, dim, vocab);
    if (deltaFinal) {
        orc_sum_rank_one(finalNorm, deltaFinal, gradArr, len, dim, vocab);
    }
    orc_normalize_state_backward(lastState, normStateGrad, grad, len, dim, dim / ORC_STATE_NORM_TILE);
    free(finalNorm); free(logits); free(gradArr); free(normStateGrad);
}

/* src/gpt/compute/cpu_transformer.cpp:128-198 ComputeBackprop.  states is [(depth+1)][len][dim] (out); stateGrad0 [len][dim] is the
 * gradient that reaches the embedding.  Returns the mean log2-free train log-loss (natural log of the target probability). */
double orc_model_step(const orc_dims *d, int depth, orc_layer *layers, const orc_common *c, int len, int labelCount, int vocab,
    const int *labelPtr, const uint32_t *labels, const float *embed, const float *finalW, const float *bias, int targetCount,
    const int *targetPairs, float *states, float *stateGrad0, float *deltaEmbed, float *deltaFinal)
{
    size_t nd = (size_t)len * d->dim;
    orc_embedding_forward(len, d->dim, labelPtr, labels, embed, states);
    for (int k = 0; k < depth; ++k) {
        orc_layer_forward(d, &layers[k], c, len, states + nd * k, states + nd * (k + 1));
    }
    float *pred = NewF((size_t)len * vocab);
    orc_final_backward(len, d->dim, vocab, states + nd * depth, finalW, bias, targetCount, targetPairs, pred, stateGrad0, deltaFinal);
    double loss = 0;
    for (int k = 0; k < targetCount; ++k) {
        loss += log(pred[(size_t)targetPairs[k * 2] * vocab + targetPairs[k * 2 + 1]]);
    }
    free(pred);
    for (int k = depth - 1; k >= 0; --k) {
        orc_layer_backward(d, &layers[k], c, len, states + nd * k, stateGrad0);
    }
    if (deltaEmbed) {
        orc_embedding_backward(len, d->dim, labelCount, labelPtr, labels, stateGrad0, deltaEmbed);
    }
    return targetCount ? loss / targetCount : 0;
}
