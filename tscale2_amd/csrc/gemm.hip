// NT GEMM on gfx950 MFMA for 8-bit (i8, e4m3) and bf16 operands:  C[m][n] (op)= scale * sum_k A[m][k] * B[n][k]
//
// Replaces the reference's GEMM cores (src/lib/cuda/cuda_i8.cuh:157-320, src/lib/cuda/cuda_matmul.cuh:396-416,
// src/lib/cuda/sm90_fp8.cuh:171-217) with one CDNA4 design:
//   * a workgroup = 4 wavefronts (2x2), each wave owns a (32*WTM) x (32*WTN) block of C as WTM x WTN MFMA 32x32 accumulators
//     (WTM = WTN = 4 -> 256x256 workgroup tile, 256 accumulator registers per lane; 2 -> 128x128; 4x2 -> 256x128 for the
//     k-tile-scaled int8 product, which carries a second, fp32 accumulator set); an 8-wave 256x256 variant puts two waves on a SIMD;
//   * K advances 128 bytes per step; A and B tiles go global -> LDS with global_load_lds_dwordx4, no staging registers and no
//     ds_write.  GemmNTRing (the 256x256 tile) keeps three stages of A and two of B (all 160 KB of LDS): A is loaded two steps
//     ahead, B one, one load at a time between the MFMAs.  GemmNTDirect (the other tiles, k-tile scales, expert groups) has two
//     stages.  Stages are separate static arrays so that operand reads of one never wait for the loads into another.  In all of
//     them 16-byte chunks are XOR-swizzled by (row/2)%8: the deposited loads and the ds_read_b128 operand fetches are bank-conflict free;
//   * operand fragments are read one K-slice ahead of the MFMAs that use them (two fragment sets), one barrier per step;
//   * MFMA: v_mfma_i32_32x32x32_i8, v_mfma_f32_32x32x64_f8f6f4 (fp8 x fp8), v_mfma_f32_32x32x16_bf16;
//   * workgroup ids are remapped so that each of the 8 XCDs (which receive ids round-robin) works on a compact band of C tiles
//     and its L2 sees every A/B panel only a few times;
//   * epilogues are fused: per-row scale, alpha, device scalar, store/accumulate in fp32/bf16, raw i32, packed int8 delta (row-tile
//     max-normalise), row-tile normalise + RoPE to bf16, per-k-tile scales (exact int32 per tile, fp32 across tiles); the contraction
//     can be cut into stored slices (deterministic split-K) or expert groups (MoE), and several products can be added into one
//     result in one launch.
#include "gemm_epilogue.h"
#include <stdlib.h>

using namespace gemmk;

namespace
{

// ---------------------------------------------------------------------------------------------------------------------------
// Two-stage loop with direct global -> LDS loads (global_load_lds_dwordx4): no staging registers and no ds_write instructions.  A
// wave-level load deposits 64 x 16 bytes contiguously in LDS, i.e. one block of 8 tile rows; which 16-byte chunk of the row a lane fetches is
// chosen so that the block lands already XOR-swizzled.  The two LDS stages are separate static arrays: the compiler can then prove
// that the operand reads of one stage do not alias the in-flight loads into the other and does not serialise them.

// SEG: two products into the same accumulators (C = alpha0 A0 B0^T + alpha1 A1 B1^T with the same k), the second operand pair and its
// factors in segA[0], segB[0], segAlpha[0], segAlphaPtr[0]; with tileGroup both B operands take the tile's slab.
template <int TYPE, int WTM, int WTN, int CT, int EPI, bool KT, int WM = 2, int WN = 2, bool SEG = false>
__global__ void __launch_bounds__(64 * WM * WN, (WM * WN) / 4) GemmNTDirect(GemmP p)
{
    typedef typename AccT<TYPE>::type TAcc;
    constexpr int NW = WM * WN; // waves per workgroup
    constexpr int BM = 32 * WTM * WM;
    constexpr int BN = 32 * WTN * WN;
    // plain 16-bit results of the 128x128 e4m3 tile leave through the row-owning epilogue (a lane owns a row: operands swapped)
    constexpr bool SWAPC = TYPE == T_FP8 && WTM == 2 && WTN == 2 && WM == 2 && WN == 2 && !KT &&
                           (CT == C_BF16NORM || ((CT == C_BF16 || CT == C_F16) && EPI == TS2_EPI_STORE));
    __shared__ __attribute__((aligned(1024))) uint8_t sA0[BM * BKB];
    __shared__ __attribute__((aligned(1024))) uint8_t sB0[BN * BKB];
    __shared__ __attribute__((aligned(1024))) uint8_t sA1[BM * BKB];
    __shared__ __attribute__((aligned(1024))) uint8_t sB1[BN * BKB];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WN;
    const int wn = wave % WN;

    int tm, tn;
    const int tilesMN = p.tilesM * p.tilesN;
    int bid = blockIdx.x;
    MapTile(bid, tilesMN, p.tilesM, p.tilesN, &tm, &tn, p.mapGroup ? p.mapGroup : 8);
    const int rowBase = tm * BM;
    const int colBase = tn * BN;
    int kSteps = p.kBytes / BKB;
    int kBeg = 0;
    if (p.tileGroup) {
        int g = p.tileGroup[rowBase / TILE];
        if (g < 0) {
            return;
        }
        p.b += (int64_t)g * p.bSlab;
        if (SEG) {
            p.segB[0] += (int64_t)g * p.bSlab;
        }
    }
    if (p.groupOffsets) {
        int g = blockIdx.y;
        kBeg = p.groupOffsets[g] * (TYPE == T_BF16 ? 2 : 1) / BKB;
        kSteps = p.groupOffsets[g + 1] * (TYPE == T_BF16 ? 2 : 1) / BKB - kBeg;
        p.c += (int64_t)g * p.cSlab;
        if (p.tileScale) {
            p.tileScale += (int64_t)g * p.tileScaleSlab;
        }
    }

    if (p.splits > 1) {
        // deterministic split of the contraction: slice y of p.splits, partial product to its own slab of C
        int per = (kSteps + p.splits - 1) / p.splits;
        kBeg = blockIdx.y * per;
        kSteps = kSteps - kBeg < per ? kSteps - kBeg : per;
        kSteps = kSteps < 0 ? 0 : kSteps;
        p.c += (int64_t)blockIdx.y * p.splitSlab;
    }

    // loader: wave w fills the 8-row blocks w, w+4, w+8, ... of each operand tile; inside a block lane -> (row = lane/8, slot = lane%8)
    // and the slot holds chunk slot ^ ((row >> 1) & 7) of the row.  All blocks of one wave have the same parity, so the chunk is fixed.
    const int lrow = wave * 8 + (lane >> 3);
    const int lchunk = (lane & 7) ^ ((lrow >> 1) & 7);
    // address = wave-uniform base (scalar registers) + one 32-bit per-lane offset per operand
    const int64_t aTileOff = (int64_t)rowBase * p.lda + (int64_t)kBeg * BKB, bTileOff = (int64_t)colBase * p.ldb + (int64_t)kBeg * BKB;
    const uint8_t *gaTile = p.a + aTileOff;
    const uint8_t *gbTile = p.b + bTileOff;
    const uint32_t gaLane = (uint32_t)(lrow * (int)p.lda + lchunk * 16);
    const uint32_t gbLane = (uint32_t)(lrow * (int)p.ldb + lchunk * 16);
    constexpr int LA = BM / (8 * NW);
    constexpr int LB = BN / (8 * NW);
#define DIRECT_LOAD(SA, SB, STEP)                                                                                                          \
    do {                                                                                                                                   \
        _Pragma("unroll") for (int i = 0; i < LA; ++i) __builtin_amdgcn_global_load_lds(                                                   \
            TS2_GLB_PTR(gaTile + ((int64_t)i * (8 * NW) * p.lda + (int64_t)(STEP)*BKB) + gaLane), TS2_LDS_PTR(SA + (wave + NW * i) * 1024), 16, 0, 0); \
        _Pragma("unroll") for (int i = 0; i < LB; ++i) __builtin_amdgcn_global_load_lds(                                                   \
            TS2_GLB_PTR(gbTile + ((int64_t)i * (8 * NW) * p.ldb + (int64_t)(STEP)*BKB) + gbLane), TS2_LDS_PTR(SB + (wave + NW * i) * 1024), 16, 0, 0); \
    } while (0)

    TAcc acc[WTM][WTN];
    v16f facc[KT ? WTM : 1][KT ? WTN : 1];
#pragma unroll
    for (int i = 0; i < WTM; ++i) {
#pragma unroll
        for (int j = 0; j < WTN; ++j) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                acc[i][j][e] = 0;
            }
        }
    }
    if (KT) {
#pragma unroll
        for (int i = 0; i < (KT ? WTM : 1); ++i) {
#pragma unroll
            for (int j = 0; j < (KT ? WTN : 1); ++j) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    facc[i][j][e] = 0;
                }
            }
        }
    }
    const int half = lane >> 5;
    const int l32 = lane & 31;
    const int aRow0 = wm * (32 * WTM) + l32;
    const int bRow0 = wn * (32 * WTN) + l32;
    constexpr int NS = TYPE == T_FP8 ? 2 : 4;
    typedef typename std::conditional<TYPE == T_FP8, v8i, v4i>::type TFrag;
    TFrag fa[2][WTM], fb[2][WTN];
    auto loadOne = [&](const uint8_t *base, int row, int sl) -> TFrag {
        if constexpr (TYPE == T_FP8) {
            int ch = sl * 4 + half * 2;
            v4i lo = *(const v4i *)(base + SwizzleOffset(row, ch));
            v4i hi = *(const v4i *)(base + SwizzleOffset(row, ch + 1));
            return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        } else {
            return *(const v4i *)(base + SwizzleOffset(row, sl * 2 + half));
        }
    };
    auto mfma = [&](TFrag a, TFrag b, TAcc c) -> TAcc {
        if constexpr (TYPE == T_I8) {
            return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
        } else if constexpr (TYPE == T_FP8) {
            return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
        } else {
            return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
        }
    };
#define LOAD_FRAGS(SET, SA, SB, SL)                                                                                                        \
    do {                                                                                                                                   \
        _Pragma("unroll") for (int i = 0; i < WTM; ++i) fa[SET][i] = loadOne(SA, aRow0 + 32 * i, SL);                                      \
        _Pragma("unroll") for (int j = 0; j < WTN; ++j) fb[SET][j] = loadOne(SB, bRow0 + 32 * j, SL);                                      \
    } while (0)
#define MFMA_ROWS(SET, I0, I1)                                                                                                             \
    do {                                                                                                                                   \
        _Pragma("unroll") for (int i = I0; i < I1; ++i) _Pragma("unroll") for (int j = 0; j < WTN; ++j) acc[i][j] =                        \
            mfma(SWAPC ? fb[SET][j] : fa[SET][i], SWAPC ? fa[SET][i] : fb[SET][j], acc[i][j]);                                             \
    } while (0)
#define WAIT_VM0() __builtin_amdgcn_s_waitcnt(0x0F70) /* vmcnt(0): the direct loads have landed in LDS */
    const int tileSteps = KT ? p.kTileBytes / BKB : 0;
    // one K step computing from stage (CA, CB) while the next tile streams into (NA, NB)
#define STEP(CA, CB, NA, NB, S)                                                                                                            \
    do {                                                                                                                                   \
        const bool more_ = (S) + 1 < kSteps;                                                                                               \
        if (more_) {                                                                                                                       \
            DIRECT_LOAD(NA, NB, (S) + 1);                                                                                                  \
        }                                                                                                                                  \
        _Pragma("unroll") for (int sl = 0; sl < NS - 1; ++sl)                                                                              \
        {                                                                                                                                  \
            if ((sl & 1) == 0) {                                                                                                           \
                LOAD_FRAGS(1, CA, CB, sl + 1);                                                                                             \
                MFMA_ROWS(0, 0, WTM);                                                                                                      \
            } else {                                                                                                                       \
                LOAD_FRAGS(0, CA, CB, sl + 1);                                                                                             \
                MFMA_ROWS(1, 0, WTM);                                                                                                      \
            }                                                                                                                              \
        }                                                                                                                                  \
        __builtin_amdgcn_sched_barrier(0);                                                                                                 \
        MFMA_ROWS(1, 0, WTM / 2);                                                                                                          \
        __builtin_amdgcn_sched_barrier(0);                                                                                                 \
        WAIT_VM0();                                                                                                                        \
        __syncthreads();                                                                                                                   \
        if (more_) {                                                                                                                       \
            LOAD_FRAGS(0, NA, NB, 0);                                                                                                      \
        }                                                                                                                                  \
        __builtin_amdgcn_sched_barrier(0);                                                                                                 \
        MFMA_ROWS(1, WTM / 2, WTM);                                                                                                        \
        if (KT) {                                                                                                                          \
            if ((kBeg + (S) + 1) % tileSteps == 0 || (S) + 1 == kSteps) {                                                                  \
                float sc = p.kTileScale[(kBeg + (S)) / tileSteps];                                                                         \
                _Pragma("unroll") for (int i = 0; i < (KT ? WTM : 1); ++i) _Pragma("unroll") for (int j = 0; j < (KT ? WTN : 1); ++j)      \
                    _Pragma("unroll") for (int e = 0; e < 16; ++e)                                                                         \
                {                                                                                                                          \
                    facc[i][j][e] += sc * (float)acc[i][j][e];                                                                             \
                    acc[i][j][e] = 0;                                                                                                      \
                }                                                                                                                          \
            }                                                                                                                              \
        }                                                                                                                                  \
    } while (0)

    float segUnits = 0; // SEG: the one factor the epilogue applies
    for (int seg = 0; seg < (SEG ? 2 : 1); ++seg) {
    if (SEG && seg == 1) {
        gaTile = p.segA[0] + aTileOff;
        gbTile = p.segB[0] + bTileOff;
    }
    if (kSteps > 0) {
        DIRECT_LOAD(sA0, sB0, 0);
    }
    WAIT_VM0();
    __syncthreads();
    if (kSteps > 0) {
        LOAD_FRAGS(0, sA0, sB0, 0);
    }
    // two steps per iteration so that each stage is a compile-time array; an odd tail step is peeled off behind the loop
    int s = 0;
    for (; s + 1 < kSteps; s += 2) {
        STEP(sA0, sB0, sA1, sB1, s);
        STEP(sA1, sB1, sA0, sB0, s + 1);
    }
    if (s < kSteps) {
        STEP(sA0, sB0, sA1, sB1, s);
    }
    if constexpr (SEG && TYPE != T_I8) {
        if (seg == 0) {
            // the epilogue applies one factor to the sum: the second product's, unless that is zero (an all-zero matrix has scale 0; the
            // product then contributes nothing and is skipped, and the first product's factor stays)
            float cur = p.alpha, nxt = p.segAlpha[0];
            if (p.alphaPtr) {
                cur *= *p.alphaPtr;
            }
            if (p.segAlphaPtr[0]) {
                nxt *= *p.segAlphaPtr[0];
            }
            segUnits = cur;
            if (nxt == 0) {
                __syncthreads();
                break;
            }
            segUnits = nxt;
            if (cur != nxt) {
                const float ratio = cur / nxt;
#pragma unroll
                for (int i = 0; i < WTM; ++i) {
#pragma unroll
                    for (int j = 0; j < WTN; ++j) {
#pragma unroll
                        for (int e = 0; e < 16; ++e) {
                            acc[i][j][e] *= ratio;
                        }
                    }
                }
            }
            __syncthreads(); // every wave has read its last operands of this product before the stages are refilled
        }
    }
    } // products
    if constexpr (SEG && TYPE != T_I8) {
        p.alpha = segUnits;
        p.alphaPtr = nullptr;
    }
#undef STEP
#undef LOAD_FRAGS
#undef MFMA_ROWS
#undef DIRECT_LOAD
#undef WAIT_VM0
    __syncthreads();
    if constexpr (SWAPC) {
        uint8_t *waveLds = wave == 0 ? sA0 : wave == 1 ? sB0 : wave == 2 ? sA1 : sB1;
        NormEpilogueRows<TYPE, CT == C_BF16NORM, CT == C_F16, 2, 2>(p, acc, waveLds, (float *)(sA0 + 8192), rowBase, colBase, wm, wn, lane);
    } else {
        Epilogue<TYPE, WTM, WTN, CT, EPI, KT>(p, acc, facc, sA0, rowBase, colBase, wm, wn, half, l32);
    }
}

// ---------------------------------------------------------------------------------------------------------------------------
// 256x256 tile, 4 waves, with the operand stages as a ring: three 32 KB stages of A (the M side: tokens, streamed once from HBM) and
// two of B (the N side: the smaller, cache-resident operand) = all 160 KB of LDS.  The loads of step S are B of step S+1 and A of
// step S+2, so an A line has two full steps to arrive and a B line one; they are issued one at a time between the MFMAs (a burst of
// sixteen 1 KB loads blocks the wave's instruction issue for about as long as the transfer takes).  Loads complete in order, so
// "all but the newest LA" (vmcnt) at the end of a step means A(S+1) and B(S+1) have landed.  Steps past the end of K reload the last
// step (harmless: the target stage is free) so that the loop body has no branches.  The stage arrays are separate static arrays
// (the compiler then knows that operand reads do not alias the loads in flight), hence six steps per loop iteration.
// WT = 2 is the same pipeline on a 128x128 tile (wave tile 64x64): the stages are 16 KB, the ring 80 KB, and two workgroups share a
// CU, so that one's start-up and stores fall into the other's main loop - for products whose workgroups are short (a contraction of
// 512 .. 2048 bytes: the expert-grouped products, whose 128-row tiles each take their expert's slab of B, tileGroup).  e4m3 only.
template <int TYPE, int CT, int EPI, bool TN = false, int WT = 4> __global__ void __launch_bounds__(256, WT == 4 ? 1 : 2) GemmNTRing(GemmP p)
{
    typedef typename AccT<TYPE>::type TAcc;
    constexpr int WTM = WT, WTN = WT, WN = 2, NW = 4, BM = 64 * WT, BN = 64 * WT;
    static_assert(WT == 4 || (WT == 2 && TYPE == T_FP8 && !TN), "the 128x128 ring takes e4m3 operands with the contraction along the rows");
    static_assert(!TN || TYPE != T_I8, "contraction-major operands: e4m3 and bf16");
    // the 16-bit and the packed-delta epilogues work on transposed blocks (a lane owns a row): the MFMAs take their operands the other way round
    constexpr bool SWAPC = ((CT == C_BF16NORM || ((CT == C_BF16 || CT == C_F16) && EPI == TS2_EPI_STORE)) && !TN) || (CT == C_I8PACK && WT == 4);
    constexpr int ESZ = TYPE == T_BF16 ? 2 : 1;
    constexpr int KR = BKB / ESZ; // contraction rows of a step (K-major operands)
    __shared__ __attribute__((aligned(1024))) uint8_t sA0[BM * BKB];
    __shared__ __attribute__((aligned(1024))) uint8_t sA1[BM * BKB];
    __shared__ __attribute__((aligned(1024))) uint8_t sA2[BM * BKB];
    __shared__ __attribute__((aligned(1024))) uint8_t sB0[BN * BKB];
    __shared__ __attribute__((aligned(1024))) uint8_t sB1[BN * BKB];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6); // wave-uniform: LDS targets and tile rows of the loader stay scalar
    const int wm = wave / WN;
    const int wn = wave % WN;
    int tm, tn;
    MapTile(blockIdx.x, p.tilesM * p.tilesN, p.tilesM, p.tilesN, &tm, &tn, p.mapGroup ? p.mapGroup : 8);
    const int rowBase = tm * BM;
    const int colBase = tn * BN;
    int kSteps = p.kBytes / BKB;
    int kBeg = 0;
    if (p.groupOffsets) {
        int g = blockIdx.y;
        kBeg = p.groupOffsets[g] * (TYPE == T_BF16 ? 2 : 1) / BKB;
        kSteps = p.groupOffsets[g + 1] * (TYPE == T_BF16 ? 2 : 1) / BKB - kBeg;
        p.c += (int64_t)g * p.cSlab;
        if (p.tileScale) {
            p.tileScale += (int64_t)g * p.tileScaleSlab;
        }
    }
    if (p.splits > 1) {
        int per = (kSteps + p.splits - 1) / p.splits;
        kBeg = blockIdx.y * per;
        kSteps = kSteps - kBeg < per ? kSteps - kBeg : per;
        kSteps = kSteps < 0 ? 0 : kSteps;
        p.c += (int64_t)blockIdx.y * p.splitSlab;
    }
    // NT: a wave-level load fills 8 tile rows of 128 K bytes, chunks swizzled by (row / 2) % 8.
    // K-major operands (TN), e4m3: a stage is 128 K rows of 256 tile-row bytes; a wave-level load fills 4 of them, and the 32-byte
    // granules of a row are XOR-swizzled by (K row) % 8 so that the transposing reads below (8 K rows x 32 bytes per half wave) hit
    // every bank once.  bf16: 64 K rows of 512 bytes, two per wave-level load; the 64-byte granules (32 tile rows) are XOR-swizzled by
    // (K row) % 4: a half wave of the 16-bit transposing read takes 64 bytes from each of 4 consecutive K rows.
    const int lrow = !TN ? wave * 8 + (lane >> 3) : TYPE == T_BF16 ? wave * 2 + (lane >> 5) : wave * 4 + (lane >> 4);
    const int lchunk = !TN               ? (lane & 7) ^ ((lrow >> 1) & 7)
                       : TYPE == T_BF16 ? (lane & 31) ^ ((lrow & 3) << 2)
                                        : (((((lane & 15) >> 1) ^ (((wave & 1) << 2) | (lane >> 4))) << 1) | (lane & 1));
    const int64_t aTileOff = TN ? (int64_t)kBeg * KR * p.lda + rowBase * ESZ : (int64_t)rowBase * p.lda + (int64_t)kBeg * BKB;
    int64_t bTileOff = TN ? (int64_t)kBeg * KR * p.ldb + colBase * ESZ : (int64_t)colBase * p.ldb + (int64_t)kBeg * BKB;
    if constexpr (WT == 2) {
        if (p.tileGroup) {
            // the rows of a 128-row tile belong to one group; every B operand of the launch is taken from that group's slab
            const int g = p.tileGroup[rowBase / TILE];
            if (g < 0) {
                return;
            }
            bTileOff += (int64_t)g * p.bSlab;
        }
    }
    const uint8_t *gaTile = p.a + aTileOff;
    const uint8_t *gbTile = p.b + bTileOff;
    const uint32_t gaLane = (uint32_t)(lrow * (int)p.lda + lchunk * 16);
    const uint32_t gbLane = (uint32_t)(lrow * (int)p.ldb + lchunk * 16);
    constexpr int LA = BM / (8 * NW);
    constexpr int LB = BN / (8 * NW);
    constexpr int IROWS = !TN ? 8 * NW : TYPE == T_BF16 ? 2 * NW : 4 * NW; // operand rows between two loads of a wave
    const int lastStep = kSteps - 1;
#define RING_LOAD(GT, LD, GL, SBUF, STEP, I0, I1)                                                                                          \
    do {                                                                                                                                   \
        const int st_ = (STEP) < lastStep ? (STEP) : lastStep;                                                                             \
        _Pragma("unroll") for (int i = I0; i < I1; ++i) __builtin_amdgcn_global_load_lds(                                                  \
            TS2_GLB_PTR(GT + ((int64_t)i * IROWS * LD + (int64_t)st_ * (TN ? (int64_t)KR * LD : (int64_t)BKB)) + GL),                      \
            TS2_LDS_PTR(SBUF + (wave + NW * i) * 1024), 16, 0, 0);                                                                         \
    } while (0)
#define RING_LOAD_A(SBUF, STEP, I0, I1) RING_LOAD(gaTile, p.lda, gaLane, SBUF, STEP, I0, I1)
#define RING_LOAD_B(SBUF, STEP, I0, I1) RING_LOAD(gbTile, p.ldb, gbLane, SBUF, STEP, I0, I1)

    TAcc acc[WTM][WTN];
    v16f facc[1][1];
#pragma unroll
    for (int i = 0; i < WTM; ++i) {
#pragma unroll
        for (int j = 0; j < WTN; ++j) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                acc[i][j][e] = 0;
            }
        }
    }
    const int half = lane >> 5;
    const int l32 = lane & 31;
    const int aRow0 = wm * (32 * WTM) + l32;
    const int bRow0 = wn * (32 * WTN) + l32;
    constexpr int NS = TYPE == T_FP8 ? 2 : 4;
    constexpr int ND = (WTM + WTN) * (TN ? (TYPE == T_FP8 ? 4 : 2) : TYPE == T_FP8 ? 2 : 1); // LDS reads per fragment set
    typedef typename std::conditional<TYPE == T_FP8, v8i, v4i>::type TFrag;
    TFrag fa[2][WTM], fb[2][WTN];
    auto loadOne = [&](const uint8_t *base, int row, int sl) -> TFrag {
        if constexpr (TYPE == T_FP8) {
            int ch = sl * 4 + half * 2;
            v4i lo = *(const v4i *)(base + SwizzleOffset(row, ch));
            v4i hi = *(const v4i *)(base + SwizzleOffset(row, ch + 1));
            return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        } else {
            return *(const v4i *)(base + SwizzleOffset(row, sl * 2 + half));
        }
    };
    auto mfma = [&](TFrag a, TFrag b, TAcc c) -> TAcc {
        if constexpr (TYPE == T_I8) {
            return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
        } else if constexpr (TYPE == T_FP8) {
            return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
        } else {
            return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
        }
    };
    // K-major operands: ds_read_b64_tr_b8.  Inside a group of 16 lanes the instruction hands lane j, byte e the byte number j % 8 of
    // the 8 bytes addressed by lane 2 * e + j / 8: with the even lanes pointing at K rows 0..7 of one 8-byte column segment and the odd
    // lanes at the same rows of the next segment, lane j receives column j of those 8 rows - eight consecutive K slots of an MFMA
    // operand whose row is the lane.  Four such reads (K rows 32 * half + 8 * q ..) make the 32 bytes of a 32x32x64 operand.
    // bf16: ds_read_b64_tr_b16 hands lane j, element e the 16-bit value number j % 4 of the 8 bytes addressed by lane 4 * e + j / 4 of
    // its group of 16: lanes 4e .. 4e+3 point at K row e, four tile rows each, and lane j receives tile row j of K rows 0..3; two reads
    // (K rows 8 * half + 4 * r ..) make the eight contraction slots of a 32x32x16 operand.
    int tnA[TN ? WTM : 1], tnB[TN ? WTN : 1];
    if constexpr (TN && TYPE == T_BF16) {
        const int e4 = (lane & 15) >> 2, lanePart = (8 * half + e4) * 512 + 32 * ((lane >> 4) & 1) + 8 * (lane & 3);
#pragma unroll
        for (int i = 0; i < WTM; ++i) {
            tnA[i] = lanePart + (((wm * WTM + i) ^ e4) << 6);
            asm volatile("" : "+v"(tnA[i]));
        }
#pragma unroll
        for (int j = 0; j < WTN; ++j) {
            tnB[j] = lanePart + (((wn * WTN + j) ^ e4) << 6);
            asm volatile("" : "+v"(tnB[j]));
        }
    } else if constexpr (TN) {
        const int e8 = (lane & 15) >> 1, lanePart = (32 * half + e8) * 256 + 16 * ((lane >> 4) & 1) + 8 * (lane & 1);
#pragma unroll
        for (int i = 0; i < WTM; ++i) {
            tnA[i] = lanePart + (((wm * WTM + i) ^ e8) << 5);
            asm volatile("" : "+v"(tnA[i]));
        }
#pragma unroll
        for (int j = 0; j < WTN; ++j) {
            tnB[j] = lanePart + (((wn * WTN + j) ^ e8) << 5);
            asm volatile("" : "+v"(tnB[j]));
        }
    }
    auto loadOneT = [&](const uint8_t *base, int laneOff, int sl) -> TFrag {
        if constexpr (TYPE == T_FP8) {
            typedef int v2i_t __attribute__((ext_vector_type(2)));
            typedef __attribute__((address_space(3))) v2i_t *TTr8;
            const __attribute__((address_space(3))) uint8_t *q = (const __attribute__((address_space(3))) uint8_t *)TS2_LDS_PTR(base) + sl * 64 * 256;
            v2i_t r0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((TTr8)(q + laneOff));
            v2i_t r1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((TTr8)(q + laneOff + 8 * 256));
            v2i_t r2 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((TTr8)(q + laneOff + 16 * 256));
            v2i_t r3 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((TTr8)(q + laneOff + 24 * 256));
            return TFrag{r0[0], r0[1], r1[0], r1[1], r2[0], r2[1], r3[0], r3[1]};
        } else if constexpr (TYPE == T_BF16) {
            typedef short v4s_t __attribute__((ext_vector_type(4)));
            typedef int v2i_t __attribute__((ext_vector_type(2)));
            typedef __attribute__((address_space(3))) v4s_t *TTr16;
            const __attribute__((address_space(3))) uint8_t *q = (const __attribute__((address_space(3))) uint8_t *)TS2_LDS_PTR(base) + sl * 16 * 512;
            v2i_t r0 = __builtin_bit_cast(v2i_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((TTr16)(q + laneOff)));
            v2i_t r1 = __builtin_bit_cast(v2i_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((TTr16)(q + laneOff + 4 * 512)));
            return TFrag{r0[0], r0[1], r1[0], r1[1]};
        } else {
            return TFrag{};
        }
    };
#define LOAD_FRAGS(SET, SA, SB, SL)                                                                                                        \
    do {                                                                                                                                   \
        if constexpr (TN) {                                                                                                                \
            _Pragma("unroll") for (int i = 0; i < WTM; ++i) fa[SET][i] = loadOneT(SA, tnA[i], SL);                                         \
            _Pragma("unroll") for (int j = 0; j < WTN; ++j) fb[SET][j] = loadOneT(SB, tnB[j], SL);                                         \
        } else {                                                                                                                           \
            _Pragma("unroll") for (int i = 0; i < WTM; ++i) fa[SET][i] = loadOne(SA, aRow0 + 32 * i, SL);                                  \
            _Pragma("unroll") for (int j = 0; j < WTN; ++j) fb[SET][j] = loadOne(SB, bRow0 + 32 * j, SL);                                  \
        }                                                                                                                                  \
    } while (0)
#define MFMA_ROWS(SET, I0, I1)                                                                                                             \
    do {                                                                                                                                   \
        _Pragma("unroll") for (int i = I0; i < I1; ++i) _Pragma("unroll") for (int j = 0; j < WTN; ++j) acc[i][j] =                        \
            mfma(SWAPC ? fb[SET][j] : fa[SET][i], SWAPC ? fa[SET][i] : fb[SET][j], acc[i][j]);                                             \
    } while (0)
    // pin the order inside a region: REP groups of (NM MFMAs, NG global loads, NDS LDS reads)
#define INTERLEAVE(REP, NM, NG, NDS)                                                                                                       \
    do {                                                                                                                                   \
        _Pragma("unroll") for (int q = 0; q < REP; ++q)                                                                                    \
        {                                                                                                                                  \
            __builtin_amdgcn_sched_group_barrier(0x008, NM, 0);                                                                            \
            if (NG) __builtin_amdgcn_sched_group_barrier(0x020, NG, 0);                                                                    \
            if (NDS) __builtin_amdgcn_sched_group_barrier(0x100, NDS, 0);                                                                  \
        }                                                                                                                                  \
    } while (0)
    // End of a step: this wave's loads except the newest LA (A of step S+2) have landed and its LDS reads have returned
    // (vmcnt(LA) lgkmcnt(0)), then the workgroup barrier.  Not __syncthreads(): its fence makes the compiler drain every load in
    // flight (vmcnt(0)) before the barrier, which would shorten the lookahead of A to one step.  The empty statements that
    // clobber memory keep the compiler from moving LDS accesses across the barrier.
#define RING_BARRIER()                                                                                                                     \
    do {                                                                                                                                   \
        __builtin_amdgcn_s_waitcnt(0x0070 | LA);                                                                                           \
        asm volatile("" ::: "memory");                                                                                                     \
        __builtin_amdgcn_s_barrier();                                                                                                      \
        asm volatile("" ::: "memory");                                                                                                     \
    } while (0)
    // one K step on stage (CA, CB); (NA1, NB) is the stage of step S+1, NA2 the A stage of step S+2
#define STEP(CA, CB, NA1, NB, NA2, S)                                                                                                      \
    do {                                                                                                                                   \
        /* slice 0: B of step S+1, one load per two MFMAs */                                                                               \
        RING_LOAD_B(NB, (S) + 1, 0, LB);                                                                                                   \
        if constexpr (NS == 2) {                                                                                                           \
            RING_LOAD_A(NA2, (S) + 2, 0, LA);                                                                                              \
        }                                                                                                                                  \
        LOAD_FRAGS(1, CA, CB, 1);                                                                                                          \
        MFMA_ROWS(0, 0, WTM);                                                                                                              \
        if constexpr (NS == 2) {                                                                                                           \
            INTERLEAVE(WTM * WTN, 1, (LA + LB) / (WTM * WTN), ND / (WTM * WTN));                                                           \
        } else {                                                                                                                           \
            INTERLEAVE(8, 2, 1, ND / 8);                                                                                                   \
        }                                                                                                                                  \
        __builtin_amdgcn_sched_barrier(0);                                                                                                 \
        if constexpr (NS == 4) {                                                                                                           \
            RING_LOAD_A(NA2, (S) + 2, 0, LA / 2);                                                                                          \
            LOAD_FRAGS(0, CA, CB, 2);                                                                                                      \
            MFMA_ROWS(1, 0, WTM);                                                                                                          \
            INTERLEAVE(4, 4, 1, ND / 4);                                                                                                   \
            __builtin_amdgcn_sched_barrier(0);                                                                                             \
            RING_LOAD_A(NA2, (S) + 2, LA / 2, LA);                                                                                         \
            LOAD_FRAGS(1, CA, CB, 3);                                                                                                      \
            MFMA_ROWS(0, 0, WTM);                                                                                                          \
            INTERLEAVE(4, 4, 1, ND / 4);                                                                                                   \
            __builtin_amdgcn_sched_barrier(0);                                                                                             \
            MFMA_ROWS(1, 0, WTM / 2);                                                                                                      \
        } else {                                                                                                                           \
            MFMA_ROWS(1, 0, WTM / 2);                                                                                                      \
        }                                                                                                                                  \
        __builtin_amdgcn_sched_barrier(0);                                                                                                 \
        RING_BARRIER(); /* everything but A of step S+2 has landed, in every wave */                                                      \
        LOAD_FRAGS(0, NA1, NB, 0);                                                                                                         \
        __builtin_amdgcn_sched_barrier(0);                                                                                                 \
        MFMA_ROWS(1, WTM / 2, WTM);                                                                                                        \
    } while (0)

    static_assert(LA == 2 * WT && LB == 2 * WT, "the vmcnt immediate of the step barrier is the number of loads of an A stage");
    // several products into the same accumulators: one pass of the pipeline per product (the stage rotation restarts), the fp32 sums
    // rescaled in between so that the epilogue's single factor, the last product's, is right for all of them
    // `units`: the factor the accumulators have to be multiplied with in the end = the factor of the product that ran last.  A product
    // whose factor is zero (an all-zero matrix has scale 0) contributes nothing and is skipped: rescaling the earlier sums to a zero
    // factor would turn them into infinities.
    float units = 0;
    for (int seg = 0; seg < p.nSeg; ++seg) {
    if (seg > 0) {
        // (constant subscripts only: a variable one would move the whole parameter block to private memory)
        gaTile = (seg == 1 ? p.segA[0] : seg == 2 ? p.segA[1] : p.segA[2]) + aTileOff;
        gbTile = (seg == 1 ? p.segB[0] : seg == 2 ? p.segB[1] : p.segB[2]) + bTileOff;
    }
    bool skip = false;
    if constexpr (TYPE != T_I8) {
        if (p.nSeg > 1) {
            float f = seg == 0 ? p.alpha : seg == 1 ? p.segAlpha[0] : seg == 2 ? p.segAlpha[1] : p.segAlpha[2];
            const float *fPtr = seg == 0 ? p.alphaPtr : seg == 1 ? p.segAlphaPtr[0] : seg == 2 ? p.segAlphaPtr[1] : p.segAlphaPtr[2];
            if (fPtr) {
                f *= *fPtr;
            }
            skip = f == 0;
            if (!skip) {
                if (units != 0 && units != f) {
                    const float ratio = units / f;
#pragma unroll
                    for (int i = 0; i < WTM; ++i) {
#pragma unroll
                        for (int j = 0; j < WTN; ++j) {
#pragma unroll
                            for (int e = 0; e < 16; ++e) {
                                acc[i][j][e] *= ratio;
                            }
                        }
                    }
                }
                units = f;
            }
        }
    }
    if (kSteps > 0 && !skip) {
        RING_LOAD_A(sA0, 0, 0, LA);
        RING_LOAD_B(sB0, 0, 0, LB);
        RING_LOAD_A(sA1, 1, 0, LA);
        RING_BARRIER();
        LOAD_FRAGS(0, sA0, sB0, 0);
        int s = 0;
        for (; s + 6 <= kSteps; s += 6) {
            STEP(sA0, sB0, sA1, sB1, sA2, s);
            STEP(sA1, sB1, sA2, sB0, sA0, s + 1);
            STEP(sA2, sB0, sA0, sB1, sA1, s + 2);
            STEP(sA0, sB1, sA1, sB0, sA2, s + 3);
            STEP(sA1, sB0, sA2, sB1, sA0, s + 4);
            STEP(sA2, sB1, sA0, sB0, sA1, s + 5);
        }
        // up to five steps left: the stages continue in the same rotation
        const int rem = kSteps - s;
        // (separate conditionals, not nested ones: every join then has two predecessors and the accumulators stay in place)
        if (rem > 0) {
            STEP(sA0, sB0, sA1, sB1, sA2, s);
        }
        if (rem > 1) {
            STEP(sA1, sB1, sA2, sB0, sA0, s + 1);
        }
        if (rem > 2) {
            STEP(sA2, sB0, sA0, sB1, sA1, s + 2);
        }
        if (rem > 3) {
            STEP(sA0, sB1, sA1, sB0, sA2, s + 3);
        }
        if (rem > 4) {
            STEP(sA1, sB0, sA2, sB1, sA0, s + 4);
        }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70); // the redundant loads of the last steps
    __syncthreads();
    } // products
    if constexpr (TYPE != T_I8) {
        if (p.nSeg > 1) {
            p.alpha = units;
            p.alphaPtr = nullptr;
        }
    }
#undef STEP
#undef RING_BARRIER
#undef INTERLEAVE
#undef LOAD_FRAGS
#undef MFMA_ROWS
#undef RING_LOAD_A
#undef RING_LOAD_B
#undef RING_LOAD
    if constexpr (SWAPC) {
        // every wave stages its rows in a stage array of its own
        uint8_t *waveLds = wave == 0 ? sA0 : wave == 1 ? sA1 : wave == 2 ? sA2 : sB0;
        if constexpr (CT == C_I8PACK) {
            PackEpilogueRows(p, acc, waveLds, rowBase, colBase, wm, wn, lane);
        } else {
            NormEpilogueRows<TYPE, CT == C_BF16NORM, CT == C_F16, WT, WT>(p, acc, waveLds, (float *)sB1, rowBase, colBase, wm, wn, lane);
        }
    } else {
        Epilogue<TYPE, WTM, WTN, CT, EPI, false>(p, acc, facc, sA0, rowBase, colBase, wm, wn, half, l32);
    }
}

// ---------------------------------------------------------------------------------------------------------------------------
// Three stages of both operands for the tiles that leave room for them (256x128: 144 KB): the loads issued during step S are those
// of step S+2, one at a time between the MFMAs, and "all but the newest LA+LB" at the end of a step means step S+1 has landed.  Same
// conventions as GemmNTRing (plain barrier with explicit waits, steps past the end reload the last one, separate static stage
// arrays, three steps per loop iteration).  Carries the k-tile-scaled second accumulator set like GemmNTDirect; WM x WN waves.
template <int TYPE, int WTM, int WTN, int CT, int EPI, bool KT, int WM, int WN>
__global__ void __launch_bounds__(64 * WM * WN, (WM * WN) / 4) GemmNTRing3(GemmP p)
{
    typedef typename AccT<TYPE>::type TAcc;
    constexpr int NW = WM * WN;
    constexpr int BM = 32 * WTM * WM, BN = 32 * WTN * WN;
    __shared__ __attribute__((aligned(1024))) uint8_t sA0[BM * BKB];
    __shared__ __attribute__((aligned(1024))) uint8_t sA1[BM * BKB];
    __shared__ __attribute__((aligned(1024))) uint8_t sA2[BM * BKB];
    __shared__ __attribute__((aligned(1024))) uint8_t sB0[BN * BKB];
    __shared__ __attribute__((aligned(1024))) uint8_t sB1[BN * BKB];
    __shared__ __attribute__((aligned(1024))) uint8_t sB2[BN * BKB];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN;
    const int wn = wave % WN;
    int tm, tn;
    MapTile(blockIdx.x, p.tilesM * p.tilesN, p.tilesM, p.tilesN, &tm, &tn, p.mapGroup ? p.mapGroup : 8);
    const int rowBase = tm * BM;
    const int colBase = tn * BN;
    int kSteps = p.kBytes / BKB;
    int kBeg = 0;
    if (p.splits > 1) {
        int per = (kSteps + p.splits - 1) / p.splits;
        kBeg = blockIdx.y * per;
        kSteps = kSteps - kBeg < per ? kSteps - kBeg : per;
        kSteps = kSteps < 0 ? 0 : kSteps;
        p.c += (int64_t)blockIdx.y * p.splitSlab;
    }
    const int lrow = wave * 8 + (lane >> 3);
    const int lchunk = (lane & 7) ^ ((lrow >> 1) & 7);
    const uint8_t *gaTile = p.a + (int64_t)rowBase * p.lda + (int64_t)kBeg * BKB;
    const uint8_t *gbTile = p.b + (int64_t)colBase * p.ldb + (int64_t)kBeg * BKB;
    const uint32_t gaLane = (uint32_t)(lrow * (int)p.lda + lchunk * 16);
    const uint32_t gbLane = (uint32_t)(lrow * (int)p.ldb + lchunk * 16);
    constexpr int LA = BM / (8 * NW);
    constexpr int LB = BN / (8 * NW);
    constexpr int LT = LA + LB;
    const int lastStep = kSteps - 1;
    // loads I0..I1-1 of the LT loads of a step: the first LA fill the A stage, the others the B stage
#define RING_LOADS(SA, SB, STEP, I0, I1)                                                                                                   \
    do {                                                                                                                                   \
        const int st_ = (STEP) < lastStep ? (STEP) : lastStep;                                                                             \
        _Pragma("unroll") for (int i = I0; i < (I1 < LT ? I1 : LT); ++i)                                                                   \
        {                                                                                                                                  \
            if (i < LA) {                                                                                                                  \
                __builtin_amdgcn_global_load_lds(TS2_GLB_PTR(gaTile + ((int64_t)i * (8 * NW) * p.lda + (int64_t)st_ * BKB) + gaLane),      \
                    TS2_LDS_PTR(SA + (wave + NW * i) * 1024), 16, 0, 0);                                                                   \
            } else {                                                                                                                       \
                __builtin_amdgcn_global_load_lds(TS2_GLB_PTR(gbTile + ((int64_t)(i - LA) * (8 * NW) * p.ldb + (int64_t)st_ * BKB) + gbLane), \
                    TS2_LDS_PTR(SB + (wave + NW * (i - LA)) * 1024), 16, 0, 0);                                                            \
            }                                                                                                                              \
        }                                                                                                                                  \
    } while (0)

    TAcc acc[WTM][WTN];
    v16f facc[KT ? WTM : 1][KT ? WTN : 1];
#pragma unroll
    for (int i = 0; i < WTM; ++i) {
#pragma unroll
        for (int j = 0; j < WTN; ++j) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                acc[i][j][e] = 0;
            }
        }
    }
    if (KT) {
#pragma unroll
        for (int i = 0; i < (KT ? WTM : 1); ++i) {
#pragma unroll
            for (int j = 0; j < (KT ? WTN : 1); ++j) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    facc[i][j][e] = 0;
                }
            }
        }
    }
    const int half = lane >> 5;
    const int l32 = lane & 31;
    const int aRow0 = wm * (32 * WTM) + l32;
    const int bRow0 = wn * (32 * WTN) + l32;
    constexpr int NS = TYPE == T_FP8 ? 2 : 4;
    constexpr int ND = (WTM + WTN) * (TYPE == T_FP8 ? 2 : 1); // ds_read_b128 per fragment set
    constexpr int NM = WTM * WTN;                             // MFMAs per K slice
    constexpr int PER = (LT + NS - 2) / (NS - 1);             // loads issued per K slice (all but the last slice carry loads)
    typedef typename std::conditional<TYPE == T_FP8, v8i, v4i>::type TFrag;
    TFrag fa[2][WTM], fb[2][WTN];
    auto loadOne = [&](const uint8_t *base, int row, int sl) -> TFrag {
        if constexpr (TYPE == T_FP8) {
            int ch = sl * 4 + half * 2;
            v4i lo = *(const v4i *)(base + SwizzleOffset(row, ch));
            v4i hi = *(const v4i *)(base + SwizzleOffset(row, ch + 1));
            return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        } else {
            return *(const v4i *)(base + SwizzleOffset(row, sl * 2 + half));
        }
    };
    auto mfma = [&](TFrag a, TFrag b, TAcc c) -> TAcc {
        if constexpr (TYPE == T_I8) {
            return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
        } else if constexpr (TYPE == T_FP8) {
            return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
        } else {
            return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
        }
    };
#define LOAD_FRAGS(SET, SA, SB, SL)                                                                                                        \
    do {                                                                                                                                   \
        _Pragma("unroll") for (int i = 0; i < WTM; ++i) fa[SET][i] = loadOne(SA, aRow0 + 32 * i, SL);                                      \
        _Pragma("unroll") for (int j = 0; j < WTN; ++j) fb[SET][j] = loadOne(SB, bRow0 + 32 * j, SL);                                      \
    } while (0)
#define MFMA_ROWS(SET, I0, I1)                                                                                                             \
    do {                                                                                                                                   \
        _Pragma("unroll") for (int i = I0; i < I1; ++i) _Pragma("unroll") for (int j = 0; j < WTN; ++j) acc[i][j] =                        \
            mfma(fa[SET][i], fb[SET][j], acc[i][j]);                                                                                       \
    } while (0)
    // PER groups of (MFMAs, one load, LDS reads)
#define INTERLEAVE()                                                                                                                       \
    do {                                                                                                                                   \
        _Pragma("unroll") for (int q = 0; q < PER; ++q)                                                                                    \
        {                                                                                                                                  \
            __builtin_amdgcn_sched_group_barrier(0x008, (NM + PER - 1) / PER, 0);                                                          \
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);                                                                             \
            __builtin_amdgcn_sched_group_barrier(0x100, (ND + PER - 1) / PER, 0);                                                          \
        }                                                                                                                                  \
    } while (0)
#define RING_BARRIER()                                                                                                                     \
    do {                                                                                                                                   \
        __builtin_amdgcn_s_waitcnt(0x0070 | LT); /* vmcnt(LT) lgkmcnt(0): everything but step S+2 has landed */                            \
        asm volatile("" ::: "memory");                                                                                                     \
        __builtin_amdgcn_s_barrier();                                                                                                      \
        asm volatile("" ::: "memory");                                                                                                     \
    } while (0)
    const int tileSteps = KT ? p.kTileBytes / BKB : 0;
    // one K step on stage (CA, CB); (NA, NB) is the stage of step S+1, (FA, FB) the one that receives step S+2
#define STEP(CA, CB, NA, NB, FA, FB, S)                                                                                                    \
    do {                                                                                                                                   \
        _Pragma("unroll") for (int sl = 0; sl < NS - 1; ++sl)                                                                              \
        {                                                                                                                                  \
            RING_LOADS(FA, FB, (S) + 2, sl * PER, (sl + 1) * PER);                                                                         \
            if ((sl & 1) == 0) {                                                                                                           \
                LOAD_FRAGS(1, CA, CB, sl + 1);                                                                                             \
                MFMA_ROWS(0, 0, WTM);                                                                                                      \
            } else {                                                                                                                       \
                LOAD_FRAGS(0, CA, CB, sl + 1);                                                                                             \
                MFMA_ROWS(1, 0, WTM);                                                                                                      \
            }                                                                                                                              \
            INTERLEAVE();                                                                                                                  \
            __builtin_amdgcn_sched_barrier(0);                                                                                             \
        }                                                                                                                                  \
        MFMA_ROWS(1, 0, WTM / 2);                                                                                                          \
        __builtin_amdgcn_sched_barrier(0);                                                                                                 \
        RING_BARRIER();                                                                                                                    \
        LOAD_FRAGS(0, NA, NB, 0);                                                                                                          \
        __builtin_amdgcn_sched_barrier(0);                                                                                                 \
        MFMA_ROWS(1, WTM / 2, WTM);                                                                                                        \
        if (KT) {                                                                                                                          \
            if ((kBeg + (S) + 1) % tileSteps == 0 || (S) + 1 == kSteps) {                                                                  \
                float sc = p.kTileScale[(kBeg + (S)) / tileSteps];                                                                         \
                _Pragma("unroll") for (int i = 0; i < (KT ? WTM : 1); ++i) _Pragma("unroll") for (int j = 0; j < (KT ? WTN : 1); ++j)      \
                    _Pragma("unroll") for (int e = 0; e < 16; ++e)                                                                         \
                {                                                                                                                          \
                    facc[i][j][e] += sc * (float)acc[i][j][e];                                                                             \
                    acc[i][j][e] = 0;                                                                                                      \
                }                                                                                                                          \
            }                                                                                                                              \
        }                                                                                                                                  \
    } while (0)

    static_assert(LT <= 15, "vmcnt immediate");
    if (kSteps > 0) {
        RING_LOADS(sA0, sB0, 0, 0, LT);
        RING_LOADS(sA1, sB1, 1, 0, LT);
        RING_BARRIER();
        LOAD_FRAGS(0, sA0, sB0, 0);
        int s = 0;
        for (; s + 3 <= kSteps; s += 3) {
            STEP(sA0, sB0, sA1, sB1, sA2, sB2, s);
            STEP(sA1, sB1, sA2, sB2, sA0, sB0, s + 1);
            STEP(sA2, sB2, sA0, sB0, sA1, sB1, s + 2);
        }
        const int rem = kSteps - s;
        if (rem > 0) {
            STEP(sA0, sB0, sA1, sB1, sA2, sB2, s);
        }
        if (rem > 1) {
            STEP(sA1, sB1, sA2, sB2, sA0, sB0, s + 1);
        }
    }
#undef STEP
#undef RING_BARRIER
#undef INTERLEAVE
#undef LOAD_FRAGS
#undef MFMA_ROWS
#undef RING_LOADS
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    Epilogue<TYPE, WTM, WTN, CT, EPI, KT>(p, acc, facc, sA0, rowBase, colBase, wm, wn, half, l32);
}

template <int TYPE, int WTM, int WTN, int CT, int EPI, bool KT> int Launch(const GemmP &p, hipStream_t stream)
{
    constexpr int BM = 64 * WTM, BN = 64 * WTN;
    GemmP q = p;
    q.tilesM = (p.m + BM - 1) / BM;
    q.tilesN = (p.n + BN - 1) / BN;
    int nb = q.tilesM * q.tilesN;
    {
        int gy = p.groupOffsets ? p.splitK_groups : (p.splits > 1 ? p.splits : 1);
        // an XCD runs nb/8 consecutive tiles: group the order so that they cover about as many rows of A as of B
        {
            int chunk = (nb % 8) == 0 ? nb / 8 : nb;
            q.mapGroup = p.mapGroup ? p.mapGroup : chunk >= 64 ? 8 : chunk >= 8 ? 4 : 2;
            // A group's rows of A are re-read for every column tile of the group: with many column tiles and a short contraction
            // they stay in the XCD's L2 if they are at most 2 MB (32768 x 8192 x 2048, bf16 result: 554 -> 520 us with groups of 4)
            if (!p.mapGroup && q.mapGroup == 8 && q.tilesN >= 16 && p.kBytes <= 4096 && (int64_t)8 * BM * p.kBytes > (2 << 20)) {
                q.mapGroup = 4;
            }
        }
        if constexpr (WTM == 4 && WTN == 4 && !KT) {
            if (p.kMajor) {
                if constexpr ((TYPE == T_FP8 || TYPE == T_BF16) && (CT == C_F32 || CT == C_I8PACK) && EPI == TS2_EPI_STORE) {
                    if (!p.tileGroup && p.nSeg == 1) {
                        hipLaunchKernelGGL((GemmNTRing<TYPE, CT, EPI, true>), dim3(nb, gy), dim3(256), 0, stream, q);
                        TS2_CHECK_LAUNCH();
                        return TS2_OK;
                    }
                }
                return TS2_ERR_UNSUPPORTED;
            }
            if (!p.tileGroup && !p.noRing) {
                hipLaunchKernelGGL((GemmNTRing<TYPE, CT, EPI>), dim3(nb, gy), dim3(256), 0, stream, q);
                TS2_CHECK_LAUNCH();
                return TS2_OK;
            }
        }
        if constexpr (WTM == 2 && WTN == 2 && !KT && TYPE == T_FP8 && CT != C_I32) {
            if (p.ring128 && !p.kMajor) {
                hipLaunchKernelGGL((GemmNTRing<TYPE, CT, EPI, false, 2>), dim3(nb, gy), dim3(256), 0, stream, q);
                TS2_CHECK_LAUNCH();
                return TS2_OK;
            }
        }
        if (p.nSeg > 1) {
            // several products per launch: the ring kernel, or two products on the 128x128 tile (fp32 / bf16 results)
            if constexpr (WTM == 2 && WTN == 2 && !KT && TYPE != T_I8 && (CT == C_F32 || CT == C_BF16)) {
                if (p.nSeg == 2 && !p.groupOffsets && p.splits <= 1) {
                    hipLaunchKernelGGL((GemmNTDirect<TYPE, WTM, WTN, CT, EPI, KT, 2, 2, true>), dim3(nb, gy), dim3(256), 0, stream, q);
                    TS2_CHECK_LAUNCH();
                    return TS2_OK;
                }
            }
            return TS2_ERR_UNSUPPORTED;
        }
        if (p.kMajor) {
            return TS2_ERR_UNSUPPORTED;
        }
        hipLaunchKernelGGL((GemmNTDirect<TYPE, WTM, WTN, CT, EPI, KT>), dim3(nb, gy), dim3(256), 0, stream, q);
        TS2_CHECK_LAUNCH();
        return TS2_OK;
    }
}

// 256x256 tile with 8 waves (2 x 4, wave tile 128x64): two waves per SIMD hide each other's LDS and barrier stalls
template <int TYPE, int CT, int EPI> int Launch8(const GemmP &p, hipStream_t stream)
{
    GemmP q = p;
    q.tilesM = p.m / 256;
    q.tilesN = p.n / 256;
    hipLaunchKernelGGL((GemmNTDirect<TYPE, 4, 2, CT, EPI, false, 2, 4>), dim3(q.tilesM * q.tilesN, p.groupOffsets ? p.splitK_groups : 1), dim3(512), 0,
        stream, q);
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

template <int TYPE, int WTM, int WTN> int DispatchEpi(const ts2_gemm_args *a, const GemmP &p, hipStream_t stream)
{
    const bool kt = a->kTileScale != nullptr;
    const int epi = a->epilogue;
    if (epi == TS2_EPI_ROW_TILE_MAXNORM) {
        if (a->cType != TS2_I8) {
            return TS2_ERR_UNSUPPORTED;
        }
        if (kt) {
            if constexpr (TYPE == T_I8 && WTM == 2) {
                return Launch<TYPE, WTM, WTN, C_I8PACK, TS2_EPI_STORE, true>(p, stream);
            }
            return TS2_ERR_UNSUPPORTED;
        }
        return Launch<TYPE, WTM, WTN, C_I8PACK, TS2_EPI_STORE, false>(p, stream);
    }
    if (a->cType == TS2_I32) {
        if constexpr (TYPE == T_I8) {
            if (epi == TS2_EPI_STORE && !kt) {
                return Launch<TYPE, WTM, WTN, C_I32, TS2_EPI_STORE, false>(p, stream);
            }
        }
        return TS2_ERR_UNSUPPORTED;
    }
    if (kt) {
        if constexpr (TYPE == T_I8 && WTM == 4 && WTN == 2) {
            if (a->cType == TS2_F32 && epi == TS2_EPI_STORE && (a->tileConfig & 8) && p.splitK <= 1 && !p.groupOffsets) {
                // the same 256x128 tile with eight waves of 64x64: two waves per SIMD, so that one wave's conversion of a finished
                // k-tile (VALU) runs under the other's MFMAs
                GemmP q = p;
                q.tilesM = p.m / 256;
                q.tilesN = (p.n + 127) / 128;
                int nb = q.tilesM * q.tilesN;
                int chunk = (nb % 8) == 0 ? nb / 8 : nb;
                q.mapGroup = p.mapGroup ? p.mapGroup : chunk >= 64 ? 8 : chunk >= 8 ? 4 : 2;
                if (p.noRing) {
                    hipLaunchKernelGGL((GemmNTDirect<TYPE, 2, 2, C_F32, TS2_EPI_STORE, true, 4, 2>), dim3(nb, p.splits > 1 ? p.splits : 1), dim3(512),
                        0, stream, q);
                } else {
                    hipLaunchKernelGGL((GemmNTRing3<TYPE, 2, 2, C_F32, TS2_EPI_STORE, true, 4, 2>), dim3(nb, p.splits > 1 ? p.splits : 1), dim3(512),
                        0, stream, q);
                }
                TS2_CHECK_LAUNCH();
                return TS2_OK;
            }
        }
        if constexpr (TYPE == T_I8 && (WTM == 2 || (WTM == 4 && WTN == 2))) {
            if (a->cType == TS2_F32) {
                return epi == TS2_EPI_ADD ? Launch<TYPE, WTM, WTN, C_F32, TS2_EPI_ADD, true>(p, stream)
                                          : Launch<TYPE, WTM, WTN, C_F32, TS2_EPI_STORE, true>(p, stream);
            }
        }
        return TS2_ERR_UNSUPPORTED;
    }
    if (epi == TS2_EPI_ROW_TILE_NORM) {
        if constexpr (WTN == 4 || (WTM == 2 && WTN == 2 && TYPE != T_I8)) {
            if (a->cType == TS2_BF16 && !kt && p.splitK <= 1) {
                return Launch<TYPE, WTM, WTN, C_BF16NORM, TS2_EPI_STORE, false>(p, stream);
            }
        }
        return TS2_ERR_UNSUPPORTED;
    }
    const bool eight = WTM == 4 && WTN == 4 && (a->tileConfig & 8) && p.splitK <= 1;
    if (a->cType == TS2_F32) {
        if (eight) {
            return epi == TS2_EPI_ADD ? Launch8<TYPE, C_F32, TS2_EPI_ADD>(p, stream) : Launch8<TYPE, C_F32, TS2_EPI_STORE>(p, stream);
        }
        return epi == TS2_EPI_ADD ? Launch<TYPE, WTM, WTN, C_F32, TS2_EPI_ADD, false>(p, stream)
                                  : Launch<TYPE, WTM, WTN, C_F32, TS2_EPI_STORE, false>(p, stream);
    }
    if (a->cType == TS2_F16) {
        if constexpr (WTM == WTN) {
            if (epi == TS2_EPI_STORE && p.splitK <= 1) {
                return Launch<TYPE, WTM, WTN, C_F16, TS2_EPI_STORE, false>(p, stream);
            }
        }
        return TS2_ERR_UNSUPPORTED;
    }
    if (a->cType == TS2_BF16) {
        if (eight) {
            return epi == TS2_EPI_ADD ? Launch8<TYPE, C_BF16, TS2_EPI_ADD>(p, stream) : Launch8<TYPE, C_BF16, TS2_EPI_STORE>(p, stream);
        }
        return epi == TS2_EPI_ADD ? Launch<TYPE, WTM, WTN, C_BF16, TS2_EPI_ADD, false>(p, stream)
                                  : Launch<TYPE, WTM, WTN, C_BF16, TS2_EPI_STORE, false>(p, stream);
    }
    return TS2_ERR_UNSUPPORTED;
}

template <int TYPE> int DispatchTile(const ts2_gemm_args *a, const GemmP &p, hipStream_t stream)
{
    int cfg = a->tileConfig & 3;
    if (cfg == 0) {
        // 256x256 tiles only when they still fill the chip; the k-tile-scaled kernel keeps a second accumulator set and needs 128x128
        long tilesL = (long)(p.m / 256) * (p.n / 256) * (p.splitK > 1 ? p.splitK : 1) * (p.groupOffsets ? p.splitK_groups : 1);
        cfg = (tilesL >= 192 || p.nSeg > 1) ? 1 : 2;
        // A short contraction is mostly its epilogue, which the 256x256 kernel (one workgroup per CU) overlaps with nothing; two or
        // three workgroups of the 128x128 kernels per CU cover each other's.  Measured, e4m3, 65536 x 1024 and 32768 x 2048 results,
        // 256x256 -> 128x128: accumulating into fp32 at K = 128 .. 1024 bytes 147-182 -> 115-150 us, into bf16 215-249 -> 128-175;
        // stored bf16 at K <= 512 55-72 -> 32-53, stored fp32 at K <= 512 equal or better; at K = 1024 stored results are a toss-up.
        if (TYPE == T_FP8 && p.nSeg == 1 && !p.kMajor && !a->kTileScale &&
            (p.kBytes <= 512 || (p.kBytes <= 1024 && a->epilogue == TS2_EPI_ADD))) {
            cfg = 2;
        }
    }
    if (p.kMajor) {
        cfg = 1; // only the 256x256 ring kernel reads contraction-major operands
        if (a->kTileScale || p.tileGroup || (p.m % 256) || (p.n % 256)) {
            return TS2_ERR_UNSUPPORTED;
        }
    }
    // the 256x256 kernel needs full tiles and has no room for the second accumulator set of the k-tile-scaled variant
    if (cfg == 1 && !a->kTileScale && !p.tileGroup && (p.m % 256) == 0 && (p.n % 256) == 0) {
        return DispatchEpi<TYPE, 4, 4>(a, p, stream);
    }
    // 256x128: the large tile that still holds both accumulator sets (int8 with k-tile scales, fp32 result)
    if (cfg == 3) {
        if constexpr (TYPE == T_I8) {
            if (a->kTileScale && a->cType == TS2_F32 && !p.tileGroup && (p.m % 256) == 0) {
                return DispatchEpi<TYPE, 4, 2>(a, p, stream);
            }
        }
        return TS2_ERR_UNSUPPORTED;
    }
    return DispatchEpi<TYPE, 2, 2>(a, p, stream);
}
} // namespace

extern "C" int ts2_gemm_nt(const ts2_gemm_args *a, void *streamPtr)
{
    if (!a || !a->a.ptr || !a->b.ptr || !a->c.ptr) {
        return TS2_ERR_NULL;
    }
    hipStream_t stream = (hipStream_t)streamPtr;
    int esz = a->abType == TS2_BF16 ? 2 : 1;
    if (a->abType != TS2_I8 && a->abType != TS2_E4M3 && a->abType != TS2_BF16) {
        return TS2_ERR_UNSUPPORTED;
    }
    // (the 256x128 kernel, bit 11 of tileConfig, advances 64 bytes of the contraction per step; the others 128)
    if (a->m <= 0 || a->n <= 0 || a->k <= 0 || (a->m % 128) || (a->n % 128) || ((int64_t)a->k * esz) % ((a->tileConfig & 2048) ? 64 : BKB)) {
        return TS2_ERR_SHAPE;
    }
    if (!Aligned16(a->a.ptr, a->a.strideBytes) || !Aligned16(a->b.ptr, a->b.strideBytes) || (((uintptr_t)a->c.ptr) & 3)) {
        return TS2_ERR_ALIGN;
    }
    if (a->kMajor) {
        // rows of A and B are the contraction index: e4m3 or bf16 operands on the 256x256 ring kernel only
        if ((a->abType != TS2_E4M3 && a->abType != TS2_BF16) || (a->m % 256) || (a->n % 256) || a->rowScale || a->kTileScale || a->tileGroup || a->extraSegments ||
            (a->tileConfig & (2 | 4 | 8 | 16)) || (a->splitK > 1 && !a->splitSlabBytes) ||
            !((a->cType == TS2_F32 && a->epilogue == TS2_EPI_STORE) || a->epilogue == TS2_EPI_ROW_TILE_MAXNORM)) {
            return TS2_ERR_UNSUPPORTED;
        }
        if (a->a.y < a->k || a->b.y < a->k || a->a.x < a->m || a->b.x < a->n || a->c.y < a->m || a->c.x < a->n) {
            return TS2_ERR_SHAPE;
        }
    } else if (a->a.y < a->m || a->b.y < a->n || a->a.x < a->k || a->b.x < a->k || a->c.y < a->m || a->c.x < a->n) {
        return TS2_ERR_SHAPE;
    }
    if (a->rowScale && (((uintptr_t)a->rowScale) & 15)) {
        return TS2_ERR_ALIGN; // row scales are fetched four at a time
    }
    if (a->kTileScale && (a->abType != TS2_I8 || a->kTile <= 0 || (a->kTile % 128) || (a->k % a->kTile))) {
        return TS2_ERR_SHAPE;
    }
    if ((a->cType == TS2_BF16 || a->cType == TS2_F16) && (a->c.strideBytes & 3)) {
        return TS2_ERR_ALIGN; // bf16 results are stored two columns at a time
    }
    if ((a->cType == TS2_BF16 || a->cType == TS2_F16 || a->cType == TS2_I8) && (int64_t)128 * a->c.strideBytes >= ((int64_t)1 << 31)) {
        return TS2_ERR_UNSUPPORTED; // the row stores address 128 rows of C from one 32-bit offset
    }
    int splitK = a->splitK > 1 ? a->splitK : 1;
    if (splitK > 1 && !a->splitSlabBytes) {
        return TS2_ERR_UNSUPPORTED; // slices of the contraction are stored, never added atomically
    }
    if (a->tileConfig & 4) {
        return TS2_ERR_UNSUPPORTED; // was: the register-staged loader
    }
    if (a->epilogue == TS2_EPI_ROW_TILE_MAXNORM && (!a->tileScale.ptr || a->tileScale.y < a->n / 128 || a->tileScale.x < a->m)) {
        return TS2_ERR_SHAPE;
    }
    GemmP p;
    p.a = (const uint8_t *)a->a.ptr;
    p.b = (const uint8_t *)a->b.ptr;
    p.c = (uint8_t *)a->c.ptr;
    p.lda = a->a.strideBytes;
    p.ldb = a->b.strideBytes;
    p.ldc = a->epilogue == TS2_EPI_ROW_TILE_MAXNORM ? a->c.strideBytes : a->c.strideBytes;
    p.m = a->m;
    p.n = a->n;
    p.kBytes = a->k * esz;
    p.mLive = a->mLive;
    p.rowScale = a->rowScale;
    p.kTileScale = a->kTileScale;
    p.kTileBytes = a->kTile * esz;
    p.alpha = a->alpha;
    p.alphaPtr = a->alphaPtr;
    p.tileScale = (float *)a->tileScale.ptr;
    p.ldTileScale = a->tileScale.strideBytes / 4;
    p.splitK = splitK;
    p.tilesM = p.tilesN = 0;
    p.tileGroup = a->tileGroup;
    p.bSlab = a->bSlabBytes;
    p.groupOffsets = a->groupOffsets;
    p.cSlab = a->cSlabBytes;
    p.tileScaleSlab = a->tileScaleSlabBytes / 4;
    p.splitK_groups = a->groups;
    p.normalize = a->normalize;
    p.vecScale = a->vecScale;
    p.rope = (const float *)a->rope.ptr;
    p.ldRope = a->rope.strideBytes / 4;
    if (a->epilogue == TS2_EPI_ROW_TILE_NORM) {
        // (the large tile stores rows of 16 bytes per lane through a buffer descriptor over 128 rows)
        if (a->cType != TS2_BF16 || (a->c.strideBytes & 3) || (int64_t)128 * a->c.strideBytes >= ((int64_t)1 << 31)) {
            return TS2_ERR_UNSUPPORTED;
        }
        if ((a->normalize && (!a->tileScale.ptr || a->tileScale.y < a->n / 128 || a->tileScale.x < a->m)) ||
            (a->rope.ptr && (a->rope.y < (a->mLive > 0 ? a->mLive : a->m) || a->rope.x < 128 || (a->rope.strideBytes & 7) || ((uintptr_t)a->rope.ptr & 7)))) {
            return TS2_ERR_SHAPE;
        }
    }
    p.nSeg = 1;
    p.rowsF16 = 0;
    if (a->extraSegments) {
        const bool bigTile = (a->m % 256) == 0 && (a->n % 256) == 0 && (a->tileConfig & 3) <= 1 && !(a->tileConfig & (4 | 8 | 16)) && !a->tileGroup;
        // the 128x128 tile (chosen with tileConfig 2, or implied by tileGroup) takes one further product
        const bool smallTile = a->extraSegments == 1 && ((a->tileConfig & 3) == 2 || a->tileGroup) && !(a->tileConfig & (4 | 8 | 16)) &&
            !a->splitSlabBytes;
        if (a->extraSegments < 0 || a->extraSegments > 3 || !(bigTile || smallTile) || a->abType == TS2_I8 || a->rowScale || a->kTileScale ||
            a->groupOffsets || splitK > 1 || (a->cType != TS2_F32 && a->cType != TS2_BF16) ||
            (a->epilogue != TS2_EPI_STORE && a->epilogue != TS2_EPI_ADD)) {
            return TS2_ERR_UNSUPPORTED;
        }
        for (int i = 0; i < a->extraSegments; ++i) {
            if (!a->segment[i].a || !a->segment[i].b) {
                return TS2_ERR_NULL;
            }
            if ((((uintptr_t)a->segment[i].a) & 15) || (((uintptr_t)a->segment[i].b) & 15)) {
                return TS2_ERR_ALIGN;
            }
            p.segA[i] = (const uint8_t *)a->segment[i].a;
            p.segB[i] = (const uint8_t *)a->segment[i].b;
            p.segAlpha[i] = a->segment[i].alpha;
            p.segAlphaPtr[i] = a->segment[i].alphaPtr;
        }
        p.nSeg = 1 + a->extraSegments;
    }
    p.splits = 1;
    p.splitSlab = 0;
    if (a->splitSlabBytes) {
        // stored (not atomically added) partial products: needs the direct kernel, fp32 results and slices of whole k-tiles
        int kStepsAll = (int)(((int64_t)a->k * esz) / BKB);
        int per = (kStepsAll + splitK - 1) / splitK;
        if (splitK <= 1 || a->cType != TS2_F32 || a->epilogue != TS2_EPI_STORE || a->tileGroup || a->groupOffsets ||
            (a->kTileScale && (per * BKB) % (a->kTile * esz)) || (a->splitSlabBytes & 7)) {
            return TS2_ERR_UNSUPPORTED;
        }
        p.splits = splitK;
        p.splitSlab = a->splitSlabBytes;
        splitK = 1;
        p.splitK = 1;
    }
    p.mapGroup = ((a->tileConfig >> 5) & 3) == 1 ? 8 : ((a->tileConfig >> 5) & 3) == 2 ? 4 : ((a->tileConfig >> 5) & 3) == 3 ? 2 : 0;
    p.gridShrink = (a->tileConfig >> 13) & 3;
    p.noRing = (a->tileConfig & 16) ? 1 : 0; // bit 4: two-stage loop instead of the ring for the 256x256 tile (comparison)
    p.kMajor = a->kMajor ? 1 : 0;
    // The result is read by another kernel later: with a contraction of 1024 bytes or more its stores leave the L2 to the operands
    // (the dense fp8 step: 2.4 ms of 125 per step, all of it from the K = 2048 products; the expert-grouped products at K = 1024:
    // 127 -> 112 us); shorter products are mostly their stores, and inside a layer those measured slower with the hint (K = 512:
    // 167 -> 180 us).  Bits 9 / 10 of tileConfig force one or the other, for comparison.
    p.streamC = (a->tileConfig & 512) ? 0 : (a->tileConfig & 1024) ? 1 : ((int64_t)a->k * esz >= 1024 ? 1 : 0);
    // 128x128 tile, e4m3: the ring pipeline from a contraction of eight steps on (measured on the expert-grouped products: 136 -> 120 us
    // at K = 1024, no gain at K = 512); bit 7 of tileConfig asks for it at any length, bit 4 for the two-stage loop
    p.ring128 = !(a->tileConfig & 16) && ((a->tileConfig & 128) || (int64_t)a->k * esz >= 8 * BKB) ? 1 : 0;
    if (a->groupOffsets && a->groups <= 0) {
        return TS2_ERR_SHAPE;
    }
    {
        // the 256x128 kernel for two workgroups per CU: bit 11 of tileConfig asks for it (TS2_ERR_UNSUPPORTED if it cannot run the call)
        const int type = a->abType == TS2_I8 ? T_I8 : a->abType == TS2_E4M3 ? T_FP8 : T_BF16;
        const int ct = a->epilogue == TS2_EPI_ROW_TILE_NORM      ? C_BF16NORM
                       : a->epilogue == TS2_EPI_ROW_TILE_MAXNORM ? C_I8PACK
                       : a->cType == TS2_F32                     ? C_F32
                       : a->cType == TS2_BF16                    ? C_BF16
                       : a->cType == TS2_F16                     ? C_F16
                       : a->cType == TS2_I32                     ? C_I32
                                                                 : -1;
        const int epi = a->epilogue == TS2_EPI_ADD ? TS2_EPI_ADD : TS2_EPI_STORE;
        if (a->tileConfig & 4096) {
            // bit 12: the persistent kernel whose epilogue runs under the next tile's main loop
            if (ct < 0 || splitK > 1 || (a->tileConfig & (4 | 8 | 16))) {
                return TS2_ERR_UNSUPPORTED;
            }
            if (p.tileGroup) {
                return RunPingGrouped(p, type, ct, epi, stream);
            }
            return RunPing(p, type, ct, epi, stream);
        }
        if (a->tileConfig & 2048) {
            if (ct < 0 || splitK > 1 || (a->tileConfig & (4 | 8 | 16))) {
                return TS2_ERR_UNSUPPORTED;
            }
            return RunTwin(p, type, ct, epi, stream);
        }
        // Automatic choice: products that store their result and whose contraction is short (under 4096 bytes: a workgroup of the
        // 256x256 kernel then spends a third of its time storing and refilling its pipeline) go to the persistent kernel when there
        // are at least two 256x128 tiles per CU.  Measured, e4m3, old -> new: 32768 x 8192 x 2048 normalised 535 -> 470 us, 16-bit 527 ->
        // 482, fp32 546 -> 497; 32768 x 2048 x 2048 fp32 142 -> 127; equal at 4096 bytes and beyond.  Bit 15 of tileConfig keeps the
        // old kernels (comparison).
        static const bool noPersistent = getenv("TS2_GEMM_NO_PERSISTENT") != nullptr; // (comparison runs of whole models)
        // Expert-grouped products with a 16-bit result: the persistent kernel on the exchanged operands (a tile = 256 result columns
        // of one expert x the 128 tokens of a row tile) when the result has 256-column chunks and there are two tiles per CU.
        if (!noPersistent && p.tileGroup && (a->tileConfig & (3 | 4 | 8 | 16 | 128 | 32768)) == 0 && ct >= 0 && splitK <= 1 &&
            (int64_t)(a->m / 128) * (a->n / 256) >= 512 && PingGroupedCanRun(p, type, ct, epi)) {
            return RunPingGrouped(p, type, ct, epi, stream);
        }
        if (!noPersistent && (a->tileConfig & (3 | 4 | 8 | 16 | 32768)) == 0 && ct >= 0 && epi == TS2_EPI_STORE && splitK <= 1 && p.kBytes >= 1024 && p.kBytes < 4096 &&
            (ct == C_F32 || ct == C_BF16 || ct == C_F16 || ct == C_BF16NORM) && (int64_t)(a->m / 256) * (a->n / 128) >= 512 &&
            PingCanRun(p, type, ct, epi)) {
            return RunPing(p, type, ct, epi, stream);
        }
    }
    switch (a->abType) {
    case TS2_I8:
        return DispatchTile<T_I8>(a, p, stream);
    case TS2_E4M3:
        return DispatchTile<T_FP8>(a, p, stream);
    default:
        return DispatchTile<T_BF16>(a, p, stream);
    }
}
