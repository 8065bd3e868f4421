/* CPU oracle (test infrastructure only): RoPE tables, the span graph and the base-2 "sink" attention of the reference CPU path. */
#include "oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* src/gpt/att/rope.cpp:4-38  TRopeComputer + FillRopeBuf: theta = 500000, buf[t][2j] = cos(t*f_j), buf[t][2j+1] = sin(t*f_j) */
void orc_fill_rope_buf(float *buf, int width, int ropeLen)
{
    float theta = 500000;
    float *freq = (float *)malloc(sizeof(float) * (width / 2));
    for (int k = 0; k < width / 2; ++k) {
        freq[k] = (float)exp(-logf(theta) * (k * 2. / width));
    }
    for (int t = 0; t < ropeLen; ++t) {
        for (int k = 0; k < width; k += 2) {
            float angle = t * freq[k / 2];
            buf[(size_t)t * width + k] = cosf(angle);
            buf[(size_t)t * width + k + 1] = sinf(angle);
        }
    }
    free(freq);
}

/* src/gpt/att/rope.cpp:54-86  ReferenceApplyRope / ApplyRope: rotate pairs in every head; row t uses table row t */
void orc_apply_rope(const float *ropeBuf, int width, float dir, float *p, int len, int dim)
{
    for (int t = 0; t < len; ++t) {
        for (int offset = 0; offset < dim; offset += width) {
            for (int k = 0; k < width; k += 2) {
                float *v0 = &p[(size_t)t * dim + offset + k];
                float *v1 = &p[(size_t)t * dim + offset + k + 1];
                float cosValue = ropeBuf[(size_t)t * width + k];
                float sinValue = ropeBuf[(size_t)t * width + k + 1] * dir;
                float r0 = *v0 * cosValue - *v1 * sinValue;
                float r1 = *v0 * sinValue + *v1 * cosValue;
                *v0 = r0;
                *v1 = r1;
            }
        }
    }
}

/* src/gpt/att/att.cpp:25-55  TransposeAttention: for every edge (from -> to) extend or open a span of "from" rows at "to".
 * Spans are {start, finish} pairs, inclusive.  Returns the span count or -1 if maxSpans is too small. */
int orc_transpose_attention(int len, const int *spanPtr, const int *spans, int *resPtr, int *resSpans, int maxSpans)
{
    /* two passes: count spans per target, then fill */
    int *cnt = (int *)calloc(len + 1, sizeof(int));
    int *last = (int *)malloc(sizeof(int) * len);
    for (int t = 0; t < len; ++t) {
        last[t] = -2;
    }
    for (int from = 0; from < len; ++from) {
        for (int k = spanPtr[from]; k < spanPtr[from + 1]; ++k) {
            for (int to = spans[k * 2]; to <= spans[k * 2 + 1]; ++to) {
                if (last[to] != from - 1 || cnt[to] == 0) {
                    cnt[to] += 1;
                }
                last[to] = from;
            }
        }
    }
    int total = 0;
    for (int t = 0; t < len; ++t) {
        resPtr[t] = total;
        total += cnt[t];
    }
    resPtr[len] = total;
    if (total > maxSpans) {
        free(cnt);
        free(last);
        return -1;
    }
    for (int t = 0; t < len; ++t) {
        cnt[t] = 0;
        last[t] = -2;
    }
    for (int from = 0; from < len; ++from) {
        for (int k = spanPtr[from]; k < spanPtr[from + 1]; ++k) {
            for (int to = spans[k * 2]; to <= spans[k * 2 + 1]; ++to) {
                if (cnt[to] > 0 && last[to] == from - 1) {
                    resSpans[(resPtr[to] + cnt[to] - 1) * 2 + 1] = from;
                } else {
                    int idx = resPtr[to] + cnt[to];
                    resSpans[idx * 2] = from;
                    resSpans[idx * 2 + 1] = from;
                    cnt[to] += 1;
                }
                last[to] = from;
            }
        }
    }
    free(cnt);
    free(last);
    return total;
}

/* src/gpt/att/sliding_window.cpp:111-118,236 (AddAttSpans with finishOffset = 1) over src/gpt/att/sliding_window.cpp:269-306:
 * row t of a fragment starting at row p attends [max(p, t - window), t - 1]; no span when that range is empty */
void orc_make_causal_spans(int fragCount, int fragLen, int window, int *spanPtr, int *spans, int *spanCount)
{
    int n = 0;
    spanPtr[0] = 0;
    for (int f = 0; f < fragCount; ++f) {
        int ptr = f * fragLen;
        for (int t = 0; t < fragLen; ++t) {
            int docStart = 0;
            int attStart = t - window > docStart ? t - window : docStart;
            int attFinish = t - 1;
            if (attFinish >= attStart) {
                spans[n * 2] = attStart + ptr;
                spans[n * 2 + 1] = attFinish + ptr;
                ++n;
            }
            spanPtr[ptr + t + 1] = n;
        }
    }
    *spanCount = n;
}

/* src/gpt/compute/layer_att_reference.h:29-45  TAttentionComputer ctor + CalcDP */
static float AttDotScale(int qDim, float attScaleMult)
{
    return sqrtf(1.0f / qDim) * (ORC_ATT_DOTPRODUCT_SCALE / ORC_LOG2) * attScaleMult;
}

static inline float CalcDP(const float *q, const float *k, int qSum, int headQDim, int qOffset, int from, int to, float attDotScale, float slope)
{
    float sum = 0;
    for (int x = 0; x < headQDim; ++x) {
        sum += q[(size_t)from * qSum + qOffset + x] * k[(size_t)to * qSum + qOffset + x];
    }
    float dp = sum * attDotScale;
    dp += -slope * (from - to);
    return dp;
}

/* src/gpt/compute/layer_att_reference.h:47-96  ComputeValLookup: running max starts at 0, a zero vector of weight 2^-max is always
 * in the denominator.  sumWeight/maxDP are [heads][len]. */
void orc_attention_forward(int len, int heads, int qDim, int ttDim, float alibiSlope, float attScaleMult, const int *spanPtr,
    const int *spans, const float *q, const float *k, const float *v, float *valLookup, float *sumWeight, float *maxDPArr)
{
    int qSum = qDim * heads;
    int ttSum = ttDim * heads;
    float ads = AttDotScale(qDim, attScaleMult);
#pragma omp parallel for schedule(dynamic, 16) collapse(2)
    for (int head = 0; head < heads; ++head) {
        for (int from = 0; from < len; ++from) {
            int qOffset = head * qDim;
            int ttOffset = head * ttDim;
            float acc[1024];
            float maxDP = 0;
            for (int a = spanPtr[from]; a < spanPtr[from + 1]; ++a) {
                for (int to = spans[a * 2]; to <= spans[a * 2 + 1]; ++to) {
                    float dp = CalcDP(q, k, qSum, qDim, qOffset, from, to, ads, alibiSlope);
                    maxDP = fmaxf(maxDP, dp);
                }
            }
            float sw = exp2f(-maxDP);
            for (int x = 0; x < ttDim; ++x) {
                acc[x] = 0;
            }
            for (int a = spanPtr[from]; a < spanPtr[from + 1]; ++a) {
                for (int to = spans[a * 2]; to <= spans[a * 2 + 1]; ++to) {
                    float dp = CalcDP(q, k, qSum, qDim, qOffset, from, to, ads, alibiSlope);
                    float w = exp2f(dp - maxDP);
                    sw += w;
                    for (int x = 0; x < ttDim; ++x) {
                        acc[x] += w * v[(size_t)to * ttSum + ttOffset + x];
                    }
                }
            }
            sumWeight[(size_t)head * len + from] = sw;
            maxDPArr[(size_t)head * len + from] = maxDP;
            float sw1 = 1 / sw;
            for (int x = 0; x < ttDim; ++x) {
                valLookup[(size_t)from * ttSum + ttOffset + x] = acc[x] * sw1;
            }
        }
    }
}

/* src/gpt/compute/layer_att_reference.h:6-21  ComputeDScale: dScale[head][t] = <dValLookup, valLookup> over the head */
void orc_compute_dscale(int len, int heads, int ttDim, const float *valLookup, const float *dValLookup, float *dScale)
{
    int ttSum = ttDim * heads;
    for (int i = 0; i < heads * len; ++i) {
        dScale[i] = 0;
    }
    for (int t = 0; t < len; ++t) {
        for (int k = 0; k < ttSum; ++k) {
            int head = k / ttDim;
            dScale[(size_t)head * len + t] += dValLookup[(size_t)t * ttSum + k] * valLookup[(size_t)t * ttSum + k];
        }
    }
}

/* src/gpt/compute/layer_att_reference.h:119-138  CalcDDot */
static inline float CalcDDot(const float *v, const float *dVal, const float *dScale, int len, int ttSum, int ttDim, int head, int ttOffset,
    int from, int to, float dp, float maxDP, float sumWeight, float ads)
{
    float w = exp2f(dp - maxDP) / sumWeight;
    float dW = 0;
    for (int x = 0; x < ttDim; ++x) {
        float dValLookup = dVal[(size_t)from * ttSum + ttOffset + x];
        float val = v[(size_t)to * ttSum + ttOffset + x];
        dW += dValLookup * val;
    }
    float ds = dScale[(size_t)head * len + from];
    float dDot = w * (dW - ds) * ads * ORC_LOG2;
    return dDot;
}

/* src/gpt/compute/layer_att_reference.h:140-170  GradQ */
void orc_attention_grad_q(int len, int heads, int qDim, int ttDim, float alibiSlope, float attScaleMult, const int *spanPtr,
    const int *spans, const float *q, const float *k, const float *v, const float *dVal, const float *dScale, const float *sumWeight,
    const float *maxDPArr, float *dq)
{
    int qSum = qDim * heads;
    int ttSum = ttDim * heads;
    float ads = AttDotScale(qDim, attScaleMult);
    memset(dq, 0, sizeof(float) * (size_t)len * qSum);
#pragma omp parallel for schedule(dynamic, 16) collapse(2)
    for (int head = 0; head < heads; ++head) {
        for (int from = 0; from < len; ++from) {
            int qOffset = head * qDim;
            int ttOffset = head * ttDim;
            for (int a = spanPtr[from]; a < spanPtr[from + 1]; ++a) {
                float sw = sumWeight[(size_t)head * len + from];
                float maxDP = maxDPArr[(size_t)head * len + from];
                for (int to = spans[a * 2]; to <= spans[a * 2 + 1]; ++to) {
                    float dp = CalcDP(q, k, qSum, qDim, qOffset, from, to, ads, alibiSlope);
                    float dDot = CalcDDot(v, dVal, dScale, len, ttSum, ttDim, head, ttOffset, from, to, dp, maxDP, sw, ads);
                    for (int x = 0; x < qDim; ++x) {
                        dq[(size_t)from * qSum + qOffset + x] += dDot * k[(size_t)to * qSum + qOffset + x];
                    }
                }
            }
        }
    }
}

/* src/gpt/compute/layer_att_reference.h:172-210  GradK over the transposed span graph -> dk, dv */
void orc_attention_grad_k(int len, int heads, int qDim, int ttDim, float alibiSlope, float attScaleMult, const int *revPtr,
    const int *revSpans, const float *q, const float *k, const float *v, const float *dVal, const float *dScale, const float *sumWeight,
    const float *maxDPArr, float *dk, float *dv)
{
    int qSum = qDim * heads;
    int ttSum = ttDim * heads;
    float ads = AttDotScale(qDim, attScaleMult);
    memset(dk, 0, sizeof(float) * (size_t)len * qSum);
    memset(dv, 0, sizeof(float) * (size_t)len * ttSum);
#pragma omp parallel for schedule(dynamic, 16) collapse(2)
    for (int head = 0; head < heads; ++head) {
        for (int to = 0; to < len; ++to) {
            int qOffset = head * qDim;
            int ttOffset = head * ttDim;
            for (int a = revPtr[to]; a < revPtr[to + 1]; ++a) {
                for (int from = revSpans[a * 2]; from <= revSpans[a * 2 + 1]; ++from) {
                    float sw = sumWeight[(size_t)head * len + from];
                    float maxDP = maxDPArr[(size_t)head * len + from];
                    float dp = CalcDP(q, k, qSum, qDim, qOffset, from, to, ads, alibiSlope);
                    float dDot = CalcDDot(v, dVal, dScale, len, ttSum, ttDim, head, ttOffset, from, to, dp, maxDP, sw, ads);
                    float w = exp2f(dp - maxDP) / sw;
                    for (int x = 0; x < qDim; ++x) {
                        dk[(size_t)to * qSum + qOffset + x] += dDot * q[(size_t)from * qSum + qOffset + x];
                    }
                    for (int x = 0; x < ttDim; ++x) {
                        dv[(size_t)to * ttSum + ttOffset + x] += w * dVal[(size_t)from * ttSum + ttOffset + x];
                    }
                }
            }
        }
    }
}
