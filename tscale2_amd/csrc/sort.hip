// Sort of the gradient rows by their scale for the int8 delta product: the order of the reference's HistSortFloatsStableKernel
// (src/lib/cuda/cuda_sort.cu:115-186) - ascending in the top 13 bits of the positive float (sign, exponent, four mantissa bits), rows
// that share those bits in DEscending row order (its single warp hands out the slots of a bin from the end) - so that the 128..512
// consecutive rows of a k-tile have like magnitudes and their common int8 scale wastes few bits (matmul_fwdbwd.cuh:210-231,325).
//
// The reference builds a histogram with atomics and lets one warp scatter serially.  Here: one workgroup of 16 waves runs two stable
// least-significant-digit radix passes (6 + 7 bits) over the rows taken in reverse order; a wave owns a contiguous run of positions,
// ranks equal digits inside a 64-lane step with ballots and keeps per-(wave, digit) running offsets in LDS, so the result is
// deterministic and independent of atomic ordering.  About 20 microseconds for 32768 rows.
//
// Fewer than 500 rows: the reference sorts exactly instead (PerformRegularSort, cuda_sort.cu:50-60,117-120: ascending by value, equal
// values by ascending row, a strict total order, so its sorting network has one possible result).  Here each row counts the rows that
// precede it in that order.
#include "common.h"

namespace
{
constexpr int SORT_THREADS = 1024, SORT_WAVES = SORT_THREADS / 64;
constexpr int SORT_BITS = 13;

__device__ __forceinline__ uint32_t SortKey(const float *rowAbsMax, const float *rowMult, int row)
{
    float v = rowAbsMax[row];
    if (rowMult) {
        v *= fabsf(rowMult[row]);
    }
    return __float_as_uint(fabsf(v)) >> (31 - SORT_BITS);
}

// one stable pass over digit (key >> SHIFT) & (2^BITS - 1); FIRST: position j holds row len-1-j, else row in[j]
template <int SHIFT, int BITS, bool FIRST>
__device__ __forceinline__ void RadixPass(int len, const float *rowAbsMax, const float *rowMult, const int *in, int *out, int *cnt /*[SORT_WAVES][128]*/,
    int *total /*[128]*/)
{
    constexpr int ND = 1 << BITS;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int chunk = ((len + SORT_WAVES - 1) / SORT_WAVES + 63) / 64 * 64;
    const int j0 = wave * chunk, j1 = min(len, j0 + chunk);
    for (int i = tid; i < SORT_WAVES * 128; i += SORT_THREADS) {
        cnt[i] = 0;
    }
    __syncthreads();
    // count
    for (int j = j0 + lane; j < j1; j += 64) {
        int row = FIRST ? len - 1 - j : in[j];
        int d = (SortKey(rowAbsMax, rowMult, row) >> SHIFT) & (ND - 1);
        atomicAdd(&cnt[wave * 128 + d], 1);
    }
    __syncthreads();
    // offsets: cnt[w][d] <- number of elements with a smaller digit + those of earlier waves with the same digit
    if (tid < ND) {
        int run = 0;
        for (int w = 0; w < SORT_WAVES; ++w) {
            int c = cnt[w * 128 + tid];
            cnt[w * 128 + tid] = run;
            run += c;
        }
        total[tid] = run;
    }
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int d = 0; d < ND; ++d) {
            int c = total[d];
            total[d] = run;
            run += c;
        }
    }
    __syncthreads();
    // scatter, 64 positions of the wave's run per step, in order
    for (int jb = j0; jb < j1; jb += 64) {
        const int j = jb + lane;
        const bool active = j < j1;
        int row = 0, d = 0;
        if (active) {
            row = FIRST ? len - 1 - j : in[j];
            d = (SortKey(rowAbsMax, rowMult, row) >> SHIFT) & (ND - 1);
        }
        unsigned long long same = __ballot(active);
#pragma unroll
        for (int b = 0; b < BITS; ++b) {
            unsigned long long bal = __ballot(active && ((d >> b) & 1));
            same &= ((d >> b) & 1) ? bal : ~bal;
        }
        if (active) {
            const int rank = __popcll(same & ((1ull << lane) - 1ull));
            const int base = total[d] + cnt[wave * 128 + d];
            out[base + rank] = row;
            if (rank == 0) {
                cnt[wave * 128 + d] += __popcll(same); // the next step of this wave reads it after this write (LDS is in order per wave)
            }
        }
    }
}

constexpr int SORT_EXACT_BELOW = 500;

__global__ void __launch_bounds__(512) ExactSortRows(int len, const float *rowAbsMax, const float *rowMult, int *order)
{
    __shared__ uint32_t key[512];
    const int tid = threadIdx.x;
    if (tid < len) {
        float v = rowAbsMax[tid];
        if (rowMult) {
            v *= fabsf(rowMult[tid]);
        }
        key[tid] = __float_as_uint(fabsf(v)); // non-negative floats order as their bits
    }
    __syncthreads();
    if (tid < len) {
        const uint32_t mine = key[tid];
        int rank = 0;
        for (int j = 0; j < len; ++j) {
            const uint32_t other = key[j];
            rank += other < mine || (other == mine && j < tid);
        }
        order[rank] = tid;
    }
}

__global__ void __launch_bounds__(SORT_THREADS) HistSortRows(int len, const float *rowAbsMax, const float *rowMult, int *order, int *tmp)
{
    __shared__ int cnt[SORT_WAVES * 128];
    __shared__ int total[128];
    RadixPass<0, 6, true>(len, rowAbsMax, rowMult, nullptr, tmp, cnt, total);
    __threadfence();
    __syncthreads();
    RadixPass<6, 7, false>(len, rowAbsMax, rowMult, tmp, order, cnt, total);
}
} // namespace

extern "C" int ts2_sort_rows_by_scale(int32_t len, const float *rowAbsMax, const float *rowMult, int32_t *order, int32_t *tmp, void *stream)
{
    if (!rowAbsMax || !order || !tmp) {
        return TS2_ERR_NULL;
    }
    if (len <= 0) {
        return TS2_ERR_SHAPE;
    }
    if (len < SORT_EXACT_BELOW) {
        hipLaunchKernelGGL(ExactSortRows, dim3(1), dim3(512), 0, (hipStream_t)stream, len, rowAbsMax, rowMult, order);
        TS2_CHECK_LAUNCH();
        return TS2_OK;
    }
    hipLaunchKernelGGL(HistSortRows, dim3(1), dim3(SORT_THREADS), 0, (hipStream_t)stream, len, rowAbsMax, rowMult, order, tmp);
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}
