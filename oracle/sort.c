/* CPU oracle (test infrastructure only): the approximate stable sort of positive floats that orders the gradient rows of the int8 delta
 * product in the reference. */
#include "oracle.h"
#include <stdlib.h>
#include <string.h>

static uint32_t Bits(float x)
{
    uint32_t u;
    memcpy(&u, &x, 4);
    return u;
}

/* src/lib/cuda/cuda_sort.cu:115-186 HistSortFloatsStableKernel: values must be >= 0.
 *   nodeCount < 500 (unless forceHist): PerformRegularSort (:50-60) = exact sort by (score, node id) ascending (Order, :11-18);
 *   else: bin = top 13 bits of the float; bins ascending; inside a bin the single warp that scatters takes node ids in ascending order
 *   and hands out the bin's slots from its END (ptr = atomicAdd(&hist[bin], -1) - 1 on the inclusive prefix sum), i.e. descending
 *   node id.  (Lanes of one warp step that hit the same bin are served in lane order: that is what the reference's own test hash,
 *   1749808112 for TMersenne(1313), cuda_sort.cu:247, pins.) */
void orc_hist_sort_stable(const float *val, int nodeCount, int *order, int forceHist)
{
    if (nodeCount < 500 && !forceHist) {
        for (int i = 0; i < nodeCount; ++i) {
            order[i] = i;
        }
        /* insertion sort with the reference's comparison; small by construction */
        for (int i = 1; i < nodeCount; ++i) {
            int x = order[i], j = i - 1;
            while (j >= 0 && (val[order[j]] > val[x] || (val[order[j]] == val[x] && order[j] > x))) {
                order[j + 1] = order[j];
                --j;
            }
            order[j + 1] = x;
        }
        return;
    }
    enum { N_BITS = 13, SZ = 1 << N_BITS };
    int *hist = (int *)calloc(SZ, sizeof(int));
    for (int i = 0; i < nodeCount; ++i) {
        hist[Bits(val[i]) >> (31 - N_BITS)] += 1;
    }
    int run = 0;
    for (int b = 0; b < SZ; ++b) { /* inclusive prefix sum */
        run += hist[b];
        hist[b] = run;
    }
    for (int i = 0; i < nodeCount; ++i) {
        uint32_t bin = Bits(val[i]) >> (31 - N_BITS);
        int ptr = --hist[bin];
        order[ptr] = i;
    }
    free(hist);
}

/* CalcResultHash of the reference's sort test (cuda_sort.cu:222-229) over the node ids in sorted order */
uint32_t orc_sort_result_hash(const int *order, int n)
{
    uint64_t res = 0xdeadf00dull;
    for (int i = 0; i < n; ++i) {
        res = res * 0x2349057ull + (uint64_t)(int64_t)order[i];
    }
    return (uint32_t)(res >> 32);
}
