// Shared device/host helpers for the gfx950 kernels.  64-wide wavefronts throughout.
#pragma once
#include <hip/hip_runtime.h>
#include <atomic>
#include <stdint.h>
#include "../../include/ts2_abi.h"

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef unsigned short bf16_t; // raw storage of a bfloat16

constexpr int WAVE = 64;
constexpr int TILE = 128; // STATE_NORM_TILE / MM_TILE of the reference (model_dim.h:20, cuda_matmul.cuh:10)

#define TS2_CHECK_LAUNCH()                                                                                                                 \
    do {                                                                                                                                   \
        if (hipGetLastError() != hipSuccess)                                                                                               \
            return TS2_ERR_LAUNCH;                                                                                                         \
    } while (0)

// Raises a kernel's dynamic-LDS limit once per call site.  `done` is the call site's own flag; the attribute call is idempotent, so two
// host threads that both find the flag clear simply both set it.
inline bool Ts2SetDynamicLds(std::atomic<bool> &done, const void *kernel, int bytes)
{
    if (done.load(std::memory_order_acquire)) {
        return true;
    }
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
        return false;
    }
    done.store(true, std::memory_order_release);
    return true;
}

__device__ __forceinline__ float Bf16ToFloat(bf16_t x)
{
    return __uint_as_float(((uint32_t)x) << 16);
}

// round to nearest even; NaN stays NaN (v_cvt_pk_bf16_f32 of gfx950)
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef float v2f __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t PackBf16x2(float lo, float hi)
{
    v2f f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, v2bf));
}

// two fp32 -> packed IEEE half, round to nearest even
typedef _Float16 v2h __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t PackF16x2(float lo, float hi)
{
    v2f f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, v2h));
}

__device__ __forceinline__ bf16_t FloatToBf16(float x)
{
    return (bf16_t)(PackBf16x2(x, 0.f) & 0xffffu);
}

// fp32 -> i8, round to nearest even, saturate: cvt.rni.sat.s8.f32 of the reference (cuda_util.cuh:61-66)
__device__ __forceinline__ int CvtToI8(float x)
{
    float r = rintf(x);
    r = fminf(fmaxf(r, -128.f), 127.f);
    return (int)r;
}

// fp32 -> e4m3 (OCP), round to nearest even, saturate to +-448: cvt.rn.satfinite.e4m3x2.f32 of the reference (cuda_util.cuh:88-102)
__device__ __forceinline__ uint32_t CvtPkE4m3(float a, float b)
{
    a = fminf(fmaxf(a, -448.f), 448.f);
    b = fminf(fmaxf(b, -448.f), 448.f);
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false) & 0xffffu;
}

__device__ __forceinline__ float E4m3ToFloat(uint32_t byte)
{
    return __builtin_amdgcn_cvt_f32_fp8((int)byte, 0);
}

// Dither of the int8 quantisers (the role of the uniform noise NormalizeVecsRowMaxKernel adds before it rounds,
// src/gpt/compute/row_scale.cuh:32-35: rounding to nearest of x + u, u uniform in (-0.5, 0.5), is unbiased).  The noise is a counter-based
// hash of (seed, row, column / 4): one 32-bit word serves four neighbouring columns, byte b standing for the offset (b - 127.5) / 256.
// The offsets of a row depend on nothing but (seed, row, column), so a test can hand the same array to the CPU restatement.
__device__ __forceinline__ uint32_t DitherWord(uint32_t seed, int row, int col4)
{
    uint32_t h = seed ^ ((uint32_t)row * 0x9E3779B1u) ^ ((uint32_t)col4 * 0x85EBCA6Bu);
    h ^= h >> 16;
    h *= 0x7FEB352Du;
    h ^= h >> 15;
    h *= 0x846CA68Bu;
    h ^= h >> 16;
    return h;
}

__device__ __forceinline__ float DitherOffset(uint32_t word, int j)
{
    return ((float)((word >> (8 * j)) & 255u) - 127.5f) * (1.f / 256);
}

// sat_i8(rne(x * mult + offset)) of four neighbouring columns, one fused multiply-add each
__device__ __forceinline__ uint32_t QuantDither4(float x0, float x1, float x2, float x3, float mult, uint32_t word)
{
    return (uint32_t)(CvtToI8(__builtin_fmaf(x0, mult, DitherOffset(word, 0))) & 0xff) |
           ((uint32_t)(CvtToI8(__builtin_fmaf(x1, mult, DitherOffset(word, 1))) & 0xff) << 8) |
           ((uint32_t)(CvtToI8(__builtin_fmaf(x2, mult, DitherOffset(word, 2))) & 0xff) << 16) |
           ((uint32_t)(CvtToI8(__builtin_fmaf(x3, mult, DitherOffset(word, 3))) & 0xff) << 24);
}

// Cross-lane exchange without the LDS crossbar: DPP modifiers inside a row of 16 lanes (they fold into the consuming VALU
// instruction), v_permlane16_swap / v_permlane32_swap of gfx950 across rows.  A butterfly reduction over 1, 2, 4, 8 uses
// quad_perm, quad_perm, row_half_mirror and row_mirror: once the quads (the 8-lane halves) hold one value each, the mirrored lane
// supplies the other quad's (half's) value, so every lane ends with the same bits as with xor-shuffles.
enum { DPP_XOR1 = 0xB1, DPP_XOR2 = 0x4E, DPP_HALF_MIRROR = 0x141, DPP_MIRROR = 0x140 };

template <int CTRL> __device__ __forceinline__ float LaneDpp(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

template <int CTRL> __device__ __forceinline__ int LaneDpp(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}

// value of lane ^ 1
__device__ __forceinline__ float LaneXor1(float v)
{
    return LaneDpp<DPP_XOR1>(v);
}

// (a, b): lanes of rows 0,2 get (own, row+1's), lanes of rows 1,3 get (row-1's, own) -- any symmetric combination of a and b is
// the xor-16 butterfly step
__device__ __forceinline__ void LaneSwap16(float v, float *a, float *b)
{
    const unsigned u = __float_as_uint(v);
    auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const unsigned r0 = r[0], r1 = r[1]; // through scalars: a bit_cast applied to r[1] directly reads element 0
    *a = __uint_as_float(r0);
    *b = __uint_as_float(r1);
}

__device__ __forceinline__ void LaneSwap32(float v, float *a, float *b)
{
    const unsigned u = __float_as_uint(v);
    auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const unsigned r0 = r[0], r1 = r[1]; // through scalars: a bit_cast applied to r[1] directly reads element 0
    *a = __uint_as_float(r0);
    *b = __uint_as_float(r1);
}

// reductions inside each aligned group of 32 lanes (one 128-wide tile held as 4 floats per lane)
__device__ __forceinline__ float Half32Sum(float v)
{
    v += LaneDpp<DPP_XOR1>(v);
    v += LaneDpp<DPP_XOR2>(v);
    v += LaneDpp<DPP_HALF_MIRROR>(v);
    v += LaneDpp<DPP_MIRROR>(v);
    float a, b;
    LaneSwap16(v, &a, &b);
    return a + b;
}

__device__ __forceinline__ float Half32Max(float v)
{
    v = fmaxf(v, LaneDpp<DPP_XOR1>(v));
    v = fmaxf(v, LaneDpp<DPP_XOR2>(v));
    v = fmaxf(v, LaneDpp<DPP_HALF_MIRROR>(v));
    v = fmaxf(v, LaneDpp<DPP_MIRROR>(v));
    float a, b;
    LaneSwap16(v, &a, &b);
    return fmaxf(a, b);
}

// wave-wide reductions
__device__ __forceinline__ float WaveSum(float v)
{
    v = Half32Sum(v);
    float a, b;
    LaneSwap32(v, &a, &b);
    return a + b;
}

__device__ __forceinline__ float WaveMax(float v)
{
    v = Half32Max(v);
    float a, b;
    LaneSwap32(v, &a, &b);
    return fmaxf(a, b);
}

__device__ __forceinline__ void LaneSwap16(int v, int *a, int *b)
{
    auto r = __builtin_amdgcn_permlane16_swap((unsigned)v, (unsigned)v, false, false);
    *a = (int)r[0];
    *b = (int)r[1];
}

__device__ __forceinline__ void LaneSwap32(int v, int *a, int *b)
{
    auto r = __builtin_amdgcn_permlane32_swap((unsigned)v, (unsigned)v, false, false);
    *a = (int)r[0];
    *b = (int)r[1];
}

__device__ __forceinline__ int WaveMaxInt(int v)
{
    v = max(v, LaneDpp<DPP_XOR1>(v));
    v = max(v, LaneDpp<DPP_XOR2>(v));
    v = max(v, LaneDpp<DPP_HALF_MIRROR>(v));
    v = max(v, LaneDpp<DPP_MIRROR>(v));
    int a, b;
    LaneSwap16(v, &a, &b);
    v = max(a, b);
    LaneSwap32(v, &a, &b);
    return max(a, b);
}

__device__ __forceinline__ int WaveMinInt(int v)
{
    return -WaveMaxInt(-v); // callers keep away from INT_MIN
}

static inline bool Aligned16(const void *p, int64_t stride)
{
    return (((uintptr_t)p) & 15) == 0 && (stride & 15) == 0;
}
