// 4-element-per-lane vector access for the bandwidth-bound kernels: a group of 32 lanes holds one 128-wide tile
// (the "warp vec" of the reference, src/lib/cuda/vec_util.cuh:67,168-273, re-cut for 64-wide wavefronts: one wave = two tiles).
#pragma once
#include "common.h"

struct F4 {
    float x, y, z, w;
};

__device__ __forceinline__ F4 MakeF4(float a, float b, float c, float d)
{
    F4 r = {a, b, c, d};
    return r;
}

__device__ __forceinline__ F4 ZeroF4()
{
    return MakeF4(0, 0, 0, 0);
}

__device__ __forceinline__ F4 operator*(F4 a, float s)
{
    return MakeF4(a.x * s, a.y * s, a.z * s, a.w * s);
}

__device__ __forceinline__ F4 operator*(F4 a, F4 b)
{
    return MakeF4(a.x * b.x, a.y * b.y, a.z * b.z, a.w * b.w);
}

__device__ __forceinline__ F4 operator+(F4 a, F4 b)
{
    return MakeF4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
}

__device__ __forceinline__ F4 operator-(F4 a, F4 b)
{
    return MakeF4(a.x - b.x, a.y - b.y, a.z - b.z, a.w - b.w);
}

__device__ __forceinline__ float HSum(F4 a)
{
    return (a.x + a.y) + (a.z + a.w);
}

__device__ __forceinline__ float HMaxAbs(F4 a)
{
    return fmaxf(fmaxf(fabsf(a.x), fabsf(a.y)), fmaxf(fabsf(a.z), fabsf(a.w)));
}

// element type tags
struct TF32 {
    typedef float T;
    static constexpr int SIZE = 4;
};
struct TBF16 {
    typedef bf16_t T;
    static constexpr int SIZE = 2;
};
struct TI8 {
    typedef int8_t T;
    static constexpr int SIZE = 1;
};
struct TE4M3 {
    typedef uint8_t T;
    static constexpr int SIZE = 1;
};

template <class TT> __device__ __forceinline__ F4 Load4(const void *p);

template <> __device__ __forceinline__ F4 Load4<TF32>(const void *p)
{
    float4 v = *(const float4 *)p;
    return MakeF4(v.x, v.y, v.z, v.w);
}

template <> __device__ __forceinline__ F4 Load4<TBF16>(const void *p)
{
    uint2 v = *(const uint2 *)p;
    return MakeF4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xffff0000u));
}

template <> __device__ __forceinline__ F4 Load4<TI8>(const void *p)
{
    int v = *(const int *)p;
    return MakeF4((float)(int8_t)(v & 0xff), (float)(int8_t)((v >> 8) & 0xff), (float)(int8_t)((v >> 16) & 0xff), (float)(v >> 24));
}

template <> __device__ __forceinline__ F4 Load4<TE4M3>(const void *p)
{
    int v = *(const int *)p;
    return MakeF4(__builtin_amdgcn_cvt_f32_fp8(v, 0), __builtin_amdgcn_cvt_f32_fp8(v, 1), __builtin_amdgcn_cvt_f32_fp8(v, 2),
        __builtin_amdgcn_cvt_f32_fp8(v, 3));
}

template <class TT> __device__ __forceinline__ void Store4(void *p, F4 v);

template <> __device__ __forceinline__ void Store4<TF32>(void *p, F4 v)
{
    *(float4 *)p = make_float4(v.x, v.y, v.z, v.w);
}

template <> __device__ __forceinline__ void Store4<TBF16>(void *p, F4 v)
{
    *(uint2 *)p = make_uint2(PackBf16x2(v.x, v.y), PackBf16x2(v.z, v.w));
}

template <> __device__ __forceinline__ void Store4<TI8>(void *p, F4 v)
{
    uint32_t r = (uint32_t)(CvtToI8(v.x) & 0xff) | ((uint32_t)(CvtToI8(v.y) & 0xff) << 8) | ((uint32_t)(CvtToI8(v.z) & 0xff) << 16) |
                 ((uint32_t)(CvtToI8(v.w) & 0xff) << 24);
    *(uint32_t *)p = r;
}

template <> __device__ __forceinline__ void Store4<TE4M3>(void *p, F4 v)
{
    *(uint32_t *)p = CvtPkE4m3(v.x, v.y) | (CvtPkE4m3(v.z, v.w) << 16);
}

// dispatch a lambda-like functor over the storage types the ABI accepts
#define TS2_DISPATCH_TYPE(code, TT, ...)                                                                                                   \
    switch (code) {                                                                                                                        \
    case TS2_F32: {                                                                                                                        \
        typedef TF32 TT;                                                                                                                   \
        __VA_ARGS__;                                                                                                                       \
    } break;                                                                                                                               \
    case TS2_BF16: {                                                                                                                       \
        typedef TBF16 TT;                                                                                                                  \
        __VA_ARGS__;                                                                                                                       \
    } break;                                                                                                                               \
    case TS2_I8: {                                                                                                                         \
        typedef TI8 TT;                                                                                                                    \
        __VA_ARGS__;                                                                                                                       \
    } break;                                                                                                                               \
    case TS2_E4M3: {                                                                                                                       \
        typedef TE4M3 TT;                                                                                                                  \
        __VA_ARGS__;                                                                                                                       \
    } break;                                                                                                                               \
    default:                                                                                                                               \
        return TS2_ERR_UNSUPPORTED;                                                                                                        \
    }

// tile-norm backward of one 128-wide tile spread over 32 lanes (TileNormalizeBackpropWarpVec, src/lib/cuda/vec_util.cuh:116-129):
// src = un-normalised source vector, grad = gradient of the normalised vector; returns the gradient of the source
__device__ __forceinline__ F4 TileNormBackprop(F4 src, F4 grad)
{
    float sum2 = Half32Sum(HSum(src * src));
    if (sum2 == 0) {
        return ZeroF4();
    }
    float dp = Half32Sum(HSum(src * grad));
    float inv = 1 / sum2; // one division per tile; the two quotients below differ from dp/sum2 and TILE/sum2 by an ulp at most
    float sigma = dp * inv;
    float scale = sqrtf(TILE * inv);
    return (grad - src * sigma) * scale;
}

// logistic gate of the reference (ComputeLoLU, src/gpt/compute/gpu_lolu.cuh:11-22): sigmoid(2x) with the +-20 clamps
__device__ __forceinline__ float LoLU1(float x)
{
    // 1 / (1 + e^-2x) with the hardware exp2 and reciprocal (about 1 ulp each): these kernels are otherwise bound by their VALU
    // instruction count.  Above the upper clamp (2x > 20) e^-2x < 2^-24 and the result is exactly 1 without a test; for large
    // negative x the exponential overflows to +inf, whose reciprocal is 0, so no intermediate can be NaN.
    float w = __builtin_amdgcn_exp2f(x * -2.88539008177792681f);
    float r = __builtin_amdgcn_rcpf(1 + w);
    return x < -10.f ? 0.f : r;
}

__device__ __forceinline__ F4 LoLU4(F4 g)
{
    return MakeF4(LoLU1(g.x), LoLU1(g.y), LoLU1(g.z), LoLU1(g.w));
}

__device__ __forceinline__ F4 LoLUGrad4(F4 m)
{
    return MakeF4(m.x * (1 - m.x) * 2.f, m.y * (1 - m.y) * 2.f, m.z * (1 - m.z) * 2.f, m.w * (1 - m.w) * 2.f);
}
