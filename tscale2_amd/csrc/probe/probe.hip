// Machine probes used for pricing the kernels: what the matrix cores and HBM actually sustain on the device the library runs on.
// The published MFMA peak assumes the boost clock; with operands that toggle like real data the chip is power limited well below it,
// so a kernel's distance from "what the MFMA pipe sustains with nothing else running" is reported next to its fraction of the
// published peak.  These entry points have no counterpart in the reference.
#include "../common.h"
#include "../../../include/ts2_probe.h"

namespace {

// TYPE 0: i8 32x32x32, 1: e4m3 32x32x64, 2: bf16 32x32x16.  Each wave keeps 4 independent accumulators busy; operands are either
// small constants (few toggling bits) or hashed bit patterns that are different in every lane and rotate between MFMAs.
template <int TYPE> __global__ void __launch_bounds__(256) MfmaRate(int iters, int randomData, int *out)
{
    v8i a8[2], b8[2];
    uint32_t h = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            h = h * 1664525u + 1013904223u;
            uint32_t x = h ^ (h >> 13);
            h = h * 1664525u + 1013904223u;
            uint32_t y = h ^ (h >> 13);
            if (!randomData) {
                x = 0x01010101u;
                y = 0x01010101u;
            }
            if (TYPE == 1) { // no e4m3 NaN codes
                x &= 0xFEFEFEFEu;
                y &= 0xFEFEFEFEu;
            }
            if (TYPE == 2) { // bf16 values in +-[1, 2)
                x = (x & 0x807F807Fu) | 0x3F803F80u;
                y = (y & 0x807F807Fu) | 0x3F803F80u;
            }
            a8[q][e] = (int)x;
            b8[q][e] = (int)y;
        }
    }
    v4i a[4], b[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            a[j][e] = a8[j >> 1][(j & 1) * 4 + e];
            b[j][e] = b8[j >> 1][(j & 1) * 4 + e];
        }
    }
    v16i c[4] = {};
    v16f f[4] = {};
    for (int i = 0; i < iters; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (TYPE == 0) {
                c[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[j], b[(j + i) & 3], c[j], 0, 0, 0);
            } else if (TYPE == 1) {
                f[j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8[j & 1], b8[(j >> 1) ^ (i & 1)], f[j], 0, 0, 0, 0, 0, 0);
            } else {
                f[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a[j]), __builtin_bit_cast(v8bf, b[(j + i) & 3]), f[j], 0, 0, 0);
            }
        }
    }
    int s = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        s += c[j][0] + (int)f[j][0];
    }
    out[blockIdx.x * 256 + threadIdx.x] = s;
}

// four independent 16-byte loads in flight per lane and streaming (non-temporal) accesses: the access pattern the bandwidth kernels use
__global__ void __launch_bounds__(256) CopyRate(const v4i *__restrict__ src, v4i *__restrict__ dst, int64_t n16)
{
    constexpr int U = 4;
    int64_t stride = (int64_t)gridDim.x * 256 * U;
    for (int64_t i = (int64_t)blockIdx.x * 256 * U + threadIdx.x; i < n16; i += stride) {
        v4i v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (i + u * 256 < n16) {
                v[u] = __builtin_nontemporal_load(&src[i + u * 256]);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (i + u * 256 < n16) {
                __builtin_nontemporal_store(v[u], &dst[i + u * 256]);
            }
        }
    }
}

template <class TLaunch> int TimeIt(hipStream_t stream, float *ms, const TLaunch &launch)
{
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
        return TS2_ERR_LAUNCH;
    }
    launch(); // warm-up
    (void)hipEventRecord(e0, stream);
    launch();
    (void)hipEventRecord(e1, stream);
    int rc = hipEventSynchronize(e1) == hipSuccess && hipGetLastError() == hipSuccess ? TS2_OK : TS2_ERR_LAUNCH;
    if (rc == TS2_OK) {
        (void)hipEventElapsedTime(ms, e0, e1);
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return rc;
}

int CuCount()
{
    int dev = 0, cu = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
        return 0;
    }
    return cu;
}

} // namespace

extern "C" int ts2_probe_mfma_rate(int32_t abType, int32_t randomData, int32_t iters, int32_t *scratch, int64_t scratchInts, double *topsOut,
    void *streamV)
{
    hipStream_t stream = (hipStream_t)streamV;
    const int cu = CuCount();
    if (cu <= 0 || iters <= 0 || !scratch || !topsOut || scratchInts < (int64_t)cu * 256) {
        return TS2_ERR_SHAPE;
    }
    float ms = 0;
    int rc;
    double ops;
    if (abType == TS2_I8) {
        ops = 2.0 * 32 * 32 * 32;
        rc = TimeIt(stream, &ms, [&] { hipLaunchKernelGGL(MfmaRate<0>, dim3(cu), dim3(256), 0, stream, iters, randomData, scratch); });
    } else if (abType == TS2_E4M3) {
        ops = 2.0 * 32 * 32 * 64;
        rc = TimeIt(stream, &ms, [&] { hipLaunchKernelGGL(MfmaRate<1>, dim3(cu), dim3(256), 0, stream, iters, randomData, scratch); });
    } else if (abType == TS2_BF16) {
        ops = 2.0 * 32 * 32 * 16;
        rc = TimeIt(stream, &ms, [&] { hipLaunchKernelGGL(MfmaRate<2>, dim3(cu), dim3(256), 0, stream, iters, randomData, scratch); });
    } else {
        return TS2_ERR_UNSUPPORTED;
    }
    if (rc != TS2_OK) {
        return rc;
    }
    *topsOut = ops * 4.0 * iters * 4.0 * cu / (ms * 1e-3) / 1e12;
    return TS2_OK;
}

extern "C" int ts2_probe_copy_rate(const void *src, void *dst, int64_t bytes, double *gbPerSecOut, void *streamV)
{
    hipStream_t stream = (hipStream_t)streamV;
    const int cu = CuCount();
    if (cu <= 0 || bytes <= 0 || bytes % 16 || !src || !dst || !gbPerSecOut) {
        return TS2_ERR_SHAPE;
    }
    float ms = 0;
    int rc = TimeIt(stream, &ms, [&] { hipLaunchKernelGGL(CopyRate, dim3(cu * 128), dim3(256), 0, stream, (const v4i *)src, (v4i *)dst, bytes / 16); });
    if (rc != TS2_OK) {
        return rc;
    }
    *gbPerSecOut = 2.0 * bytes / (ms * 1e-3) / 1e9; // read + write
    return TS2_OK;
}

// One wave that samples the shader clock while other kernels run: every `periodTicks` ticks of the constant 100 MHz counter
// (s_memrealtime) it records how far the core-clock counter (s_memtime) advanced.  Bounded: `samples` periods, then it exits.
__global__ void ClockMonitor(uint64_t *out, int samples, int periodTicks)
{
    if (threadIdx.x != 0) {
        return;
    }
    for (int i = 0; i < samples; ++i) {
        const uint64_t r0 = __builtin_amdgcn_s_memrealtime();
        const uint64_t c0 = __builtin_amdgcn_s_memtime();
        uint64_t r1 = r0;
        while (r1 - r0 < (uint64_t)periodTicks) {
            __builtin_amdgcn_s_sleep(8);
            r1 = __builtin_amdgcn_s_memrealtime();
        }
        const uint64_t c1 = __builtin_amdgcn_s_memtime();
        out[2 * i] = r1 - r0;
        out[2 * i + 1] = c1 - c0;
    }
}

extern "C" int ts2_probe_clock_monitor(uint64_t *out, int32_t samples, int32_t periodTicks, void *streamV)
{
    if (!out || samples <= 0 || samples > (1 << 20) || periodTicks <= 0 || periodTicks > 100000000) {
        return TS2_ERR_SHAPE;
    }
    hipLaunchKernelGGL(ClockMonitor, dim3(1), dim3(64), 0, (hipStream_t)streamV, out, samples, periodTicks);
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}
