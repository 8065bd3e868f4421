/* CPU oracle (test infrastructure only): number-format conversions and the quantised containers the backward reads and writes. */
#include "oracle.h"
#include <math.h>
#include <string.h>
#include <limits.h>

static inline uint32_t FloatBits(float x)
{
    uint32_t u;
    memcpy(&u, &x, 4);
    return u;
}

static inline float BitsFloat(uint32_t u)
{
    float x;
    memcpy(&x, &u, 4);
    return x;
}

/* src/gpt/model_params/sse_utils.h:56-71 PackFloatToInt8: _mm256_cvtps_epi32 (round to nearest even; NaN and anything outside
 * int32 become INT_MIN) followed by two signed saturating packs, so the result saturates to [-128, 127] */
int8_t orc_cvt_i8(float x)
{
    int32_t i;
    if (!(x > -2147483648.0f && x < 2147483648.0f)) {
        i = INT_MIN;
    } else {
        i = (int32_t)nearbyintf(x);
    }
    if (i < -128) {
        i = -128;
    }
    if (i > 127) {
        i = 127;
    }
    return (int8_t)i;
}

/* src/gpt/model_params/sse_utils.h:73-78 ConvertArray */
void orc_convert_i8(int8_t *dst, const float *src, int n, float mult)
{
    for (int i = 0; i < n; ++i) {
        dst[i] = orc_cvt_i8(src[i] * mult);
    }
}

/* src/gpt/model_params/sse_utils.h:161-204 ConvertToFp8e4m3, one element: add half an ulp of the 3-bit mantissa when the first
 * dropped bit is set, truncate; exponent above 15 -> 0x7f, below 0 -> 0; exponent field 0 keeps the normal mantissa bits;
 * finally 0x7f -> 0x7e and 0xff -> 0xfe */
uint8_t orc_cvt_e4m3(float vec)
{
    uint32_t roundBits = FloatBits(vec);
    float round0 = BitsFloat(roundBits & 0xFF800000u);
    float round1 = BitsFloat(roundBits & 0xFF880000u);
    vec = vec + (round1 - round0);
    uint32_t bits = FloatBits(vec);
    int32_t sign = (int32_t)(bits >> 31);
    int32_t exponent = (int32_t)((bits & 0x7F800000u) >> 23);
    int32_t mantissa = (int32_t)((bits & 0x007FFFFFu) >> 20);
    exponent -= 127 - 7;
    int32_t fp8dw = (int32_t)(((uint32_t)sign << 7) | ((uint32_t)exponent << 3) | (uint32_t)mantissa);
    int32_t maxAbs = (sign << 7) | 0x7f;
    if (exponent > 15) {
        fp8dw = maxAbs;
    }
    if (0 > exponent) {
        fp8dw = 0;
    }
    /* _mm_packus_epi32 then _mm_packus_epi16: saturate to [0, 255] */
    if (fp8dw < 0) {
        fp8dw = 0;
    }
    if (fp8dw > 255) {
        fp8dw = 255;
    }
    uint8_t r = (uint8_t)fp8dw;
    if (r > 0xfe) {
        r = 0xfe;
    }
    if ((int8_t)r > 0x7e) {
        r = 0x7e;
    }
    return r;
}

void orc_convert_e4m3(uint8_t *dst, const float *src, int n, float mult)
{
    for (int i = 0; i < n; ++i) {
        dst[i] = orc_cvt_e4m3(src[i] * mult);
    }
}

/* src/util/fp8.h:4-21 ConvertE4toFloat: bias 7, 3 mantissa bits, denormals, no NaN/Inf codes (0x7f decodes as 480) */
float orc_e4m3_to_float(int code)
{
    int x = code & 0xff;
    if (x == 0) {
        return 0;
    }
    float sign = (x & 0x80) ? -1.f : 1.f;
    int e = (x >> 3) & 15;
    int m = x & 7;
    if (e == 0 && m > 0) {
        return sign * exp2f(1 - 7) * (0 + exp2f(-3) * m);
    } else {
        return sign * exp2f(e - 7) * (1 + exp2f(-3) * m);
    }
}

/* Device-side conversion rule of the reference, src/lib/cuda/cuda_util.cuh:88-102 (cvt.rn.satfinite.e4m3x2.f32): round to nearest
 * even onto the e4m3 grid including denormals, saturate to +-448.  This is the rule the GPU kernels implement. */
uint8_t orc_cvt_e4m3_rne(float x)
{
    uint8_t sign = (FloatBits(x) >> 31) ? 0x80 : 0;
    float a = fabsf(x);
    if (!(a == a)) {
        return sign | 0x7f;
    }
    if (a >= 448.f) {
        return sign | 0x7e;
    }
    /* quantum: 2^-9 below 2^-6 (denormal range), else 2^(floor(log2 a) - 3) */
    int e;
    (void)frexpf(a, &e); /* a = f * 2^e, f in [0.5, 1) -> floor(log2 a) = e - 1 */
    int ex = e - 1;
    if (ex < -6) {
        ex = -6;
    }
    float q = ldexpf(1.f, ex - 3);
    float r = nearbyintf(a / q) * q; /* exact: a/q has at most 24 bits, ties to even */
    if (r >= 448.f) {
        return sign | 0x7e;
    }
    if (r == 0) {
        return sign;
    }
    if (r < ldexpf(1.f, -6)) {
        return sign | (uint8_t)(r / ldexpf(1.f, -9));
    }
    int e2;
    float f = frexpf(r, &e2); /* r = f*2^e2, f in [0.5,1) */
    int be = (e2 - 1) + 7;
    int m = (int)((f * 2 - 1) * 8);
    return sign | (uint8_t)((be << 3) | m);
}

/* the same rule over an array, result decoded back to fp32 (the value the device stores): used by the same-contract model of the tests */
void orc_round_e4m3_rne(float *dst, const float *src, long n)
{
#pragma omp parallel for schedule(static)
    for (long i = 0; i < n; ++i) {
        uint8_t c = orc_cvt_e4m3_rne(src[i]);
        float v = orc_e4m3_to_float(c & 0x7f);
        dst[i] = (c & 0x80) ? -v : v;
    }
}

/* src/gpt/matrix/quant.h:42-62 TQuantizedMatrix::Convert (i8): scale = rms of the matrix; fast = sat_i8(rne(w / (rms/32))).
 * Returns the matrix scale (rms).  The reference sums squares in 8 AVX lanes; the summation here is in double. */
float orc_quantize_matrix_i8(const float *w, int8_t *fast, int ySize, int xSize)
{
    double sum2 = 0;
    size_t n = (size_t)ySize * xSize;
    for (size_t i = 0; i < n; ++i) {
        sum2 += (double)w[i] * w[i];
    }
    float sko = sqrtf((float)sum2 / ((float)xSize * ySize));
    float discrScale = sko * ORC_MODEL_DISCR_SCALE;
    float mult = (sko == 0) ? 0 : (1 / discrScale);
    for (size_t i = 0; i < n; ++i) {
        fast[i] = orc_cvt_i8(w[i] * mult);
    }
    return sko;
}

/* same container for e4m3 weights: src/gpt/matrix/quant.cpp:78-82 -> ConvertToFp8e4m3 */
float orc_quantize_matrix_e4m3(const float *w, uint8_t *fast, int ySize, int xSize)
{
    double sum2 = 0;
    size_t n = (size_t)ySize * xSize;
    for (size_t i = 0; i < n; ++i) {
        sum2 += (double)w[i] * w[i];
    }
    float sko = sqrtf((float)sum2 / ((float)xSize * ySize));
    float discrScale = sko * ORC_MODEL_DISCR_SCALE;
    float mult = (sko == 0) ? 0 : (1 / discrScale);
    for (size_t i = 0; i < n; ++i) {
        fast[i] = orc_cvt_e4m3(w[i] * mult);
    }
    return sko;
}

/* src/gpt/matrix/quant.h:64-79 GetFastFloatData: w = float(fast) * scale, scale = 1/32 (noScale) or rms/32 */
void orc_dequant_i8(const int8_t *fast, float *w, int n, float scale)
{
    for (int i = 0; i < n; ++i) {
        w[i] = (float)fast[i] * scale;
    }
}

void orc_dequant_e4m3(const uint8_t *fast, float *w, int n, float scale)
{
    for (int i = 0; i < n; ++i) {
        w[i] = orc_e4m3_to_float(fast[i]) * scale;
    }
}

/* src/gpt/matrix/delta.cpp:155-179 Compress: per (row, 128-column tile) scale = maxabs/127, delta = sat_i8(rne(x/scale));
 * tileScale is [xSize/128][ySize]; an all-zero tile gets scale 0 and its bytes are left untouched */
void orc_compress_delta(const float *data, int8_t *delta, float *tileScale, int ySize, int xSize)
{
    for (int y = 0; y < ySize; ++y) {
        int tileId = 0;
        for (int xOffset = 0; xOffset < xSize; xOffset += 128) {
            float maxVal = 0;
            for (int x = 0; x < 128; ++x) {
                float a = fabsf(data[(size_t)y * xSize + xOffset + x]);
                maxVal = maxVal > a ? maxVal : a;
            }
            if (maxVal == 0) {
                tileScale[(size_t)tileId * ySize + y] = 0;
            } else {
                float scale = maxVal / 127;
                float mult = 1 / scale;
                tileScale[(size_t)tileId * ySize + y] = scale;
                orc_convert_i8(delta + (size_t)y * xSize + xOffset, data + (size_t)y * xSize + xOffset, 128, mult);
            }
            ++tileId;
        }
    }
}

/* src/gpt/compute/row_scale.cuh:12-43 NormalizeVecsRowMaxKernel without its random dither: per row scale = maxabs/127
 * (src/lib/cuda/cuda_util.cuh:366-378), dst = sat_i8(rne(x * (1/scale))), zero rows get scale 0 and zero bytes */
void orc_quant_rowmax_i8(const float *src, int8_t *dst, float *rowScale, int len, int dim)
{
    for (int t = 0; t < len; ++t) {
        float maxVal = 0;
        for (int x = 0; x < dim; ++x) {
            float a = fabsf(src[(size_t)t * dim + x]);
            maxVal = maxVal > a ? maxVal : a;
        }
        float discrScale = 0;
        float mult = 0;
        if (maxVal > 0) {
            discrScale = maxVal / 127;
            mult = 1 / discrScale;
        }
        for (int x = 0; x < dim; ++x) {
            dst[(size_t)t * dim + x] = orc_cvt_i8(src[(size_t)t * dim + x] * mult);
        }
        rowScale[t] = discrScale;
    }
}

/* The same with the noise NormalizeVecsRowMaxKernel adds before it rounds (src/gpt/compute/row_scale.cuh:32-35:
 * buf[d] = buf[d] * mult + rng.GenUniformFloat() - 0.5f): noise[t][x] in (-0.5, 0.5) is handed in by the caller (the reference draws it
 * from an LCG seeded with the row's own bits; the library under test from a counter-based hash).  One fused multiply-add per element. */
void orc_quant_rowmax_i8_noise(const float *src, const float *noise, int8_t *dst, float *rowScale, int len, int dim)
{
    for (int t = 0; t < len; ++t) {
        float maxVal = 0;
        for (int x = 0; x < dim; ++x) {
            float a = fabsf(src[(size_t)t * dim + x]);
            maxVal = maxVal > a ? maxVal : a;
        }
        float discrScale = 0;
        float mult = 0;
        if (maxVal > 0) {
            discrScale = maxVal / 127;
            mult = 1 / discrScale;
        }
        for (int x = 0; x < dim; ++x) {
            dst[(size_t)t * dim + x] = orc_cvt_i8(fmaf(src[(size_t)t * dim + x], mult, noise[(size_t)t * dim + x]));
        }
        rowScale[t] = discrScale;
    }
}

/* orc_quant_ktile_i8 (below) with the same noise in its requantisation */
void orc_quant_ktile_i8_noise(const float *src, const float *noise, int8_t *dst, float *tileScale, int len, int dim, int kTile)
{
    for (int t0 = 0; t0 < len; t0 += kTile) {
        int t1 = t0 + kTile < len ? t0 + kTile : len;
        float maxVal = 0;
        for (int t = t0; t < t1; ++t) {
            for (int x = 0; x < dim; ++x) {
                float a = fabsf(src[(size_t)t * dim + x]);
                maxVal = maxVal > a ? maxVal : a;
            }
        }
        float scale = maxVal > 0 ? maxVal / 127 : 1;
        float mult = 1 / scale;
        for (int t = t0; t < t1; ++t) {
            for (int x = 0; x < dim; ++x) {
                dst[(size_t)t * dim + x] = orc_cvt_i8(fmaf(src[(size_t)t * dim + x], mult, noise[(size_t)t * dim + x]));
            }
        }
        tileScale[t0 / kTile] = scale;
    }
}

/* Role of ShuffleMaxScaleTransposeKernel (src/gpt/compute/matmul_fwdbwd.cuh:209-280) without the sort and the dither: every
 * kTile consecutive rows share one scale = maxabs(tile)/127 (1 for an all-zero tile), requantised from the fp32 source.
 * Output stays row-major [len][dim]; the transposed copy the reference writes is a layout choice of its GEMM. */
void orc_quant_ktile_i8(const float *src, int8_t *dst, float *tileScale, int len, int dim, int kTile)
{
    for (int t0 = 0; t0 < len; t0 += kTile) {
        int t1 = t0 + kTile < len ? t0 + kTile : len;
        float maxVal = 0;
        for (int t = t0; t < t1; ++t) {
            for (int x = 0; x < dim; ++x) {
                float a = fabsf(src[(size_t)t * dim + x]);
                maxVal = maxVal > a ? maxVal : a;
            }
        }
        float scale = maxVal > 0 ? maxVal / 127 : 1;
        float mult = 1 / scale;
        for (int t = t0; t < t1; ++t) {
            for (int x = 0; x < dim; ++x) {
                dst[(size_t)t * dim + x] = orc_cvt_i8(src[(size_t)t * dim + x] * mult);
            }
        }
        tileScale[t0 / kTile] = scale;
    }
}

/* src/gpt/compute/gpu_grad_scale.cuh:33-41 ComputeGradMult with src/lib/cuda/cuda_util.cuh:390-393 TruncateToPow2 */
float orc_grad_mult(float maxNorm)
{
    if (maxNorm == 0) {
        return 1;
    }
    return BitsFloat(FloatBits(128.f / maxNorm) & 0xff800000u);
}

/* fp32 -> bf16 -> fp32, round to nearest even: the storage rounding of 16-bit activations on the GPU path */
float orc_bf16_round(float x)
{
    uint32_t u = FloatBits(x);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        return x;
    }
    uint32_t r = u + 0x7fffu + ((u >> 16) & 1u);
    return BitsFloat(r & 0xffff0000u);
}
