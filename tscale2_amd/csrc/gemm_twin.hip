// NT GEMM kernel for two workgroups per CU:  C[m][n] (op)= scale * sum_k A[m][k] * B[n][k], 8-bit (i8, e4m3) and bf16 operands.
//
// The 256x256 ring kernel (gemm.hip) runs one workgroup per CU with 256 accumulator registers per wave: while a tile's results are
// scaled and stored, and while the next tile's first operands arrive, the matrix cores of that CU idle - a third of the time of a
// product whose contraction is 2048 bytes.  Here a workgroup owns a 256x128 tile with 128 accumulator registers per wave (four waves
// stacked along M, wave tile 64x128 = 2x4 MFMA 32x32 blocks) and at most 256 registers and 72 KB of LDS in all, so that two workgroups
// share a CU and every SIMD holds a wave of each: one workgroup's epilogue and start-up run under the other's main loop, and inside the
// main loop one wave's barrier and LDS waits are filled by the other's MFMAs.  It plays the role of the reference's GEMM cores
// (src/lib/cuda/cuda_i8.cuh:157-320, src/lib/cuda/cuda_matmul.cuh:396-416, src/lib/cuda/sm90_fp8.cuh:171-217) for the products whose
// workgroups are short.
//   * K advances 64 bytes per step through a ring of three stages of both operands (A 16 KB, B 8 KB per stage).  The loads of step
//     S+2 (global -> LDS directly, six per wave) are issued one at a time between the MFMAs of step S; loads complete in order, so
//     "all but the newest six" at the barrier that ends step S means step S+1 has landed.  Steps past the end of K load the last step
//     again into a free stage, so that the loop body has no branches and the count of loads in flight is the same at every barrier.
//   * A stage row is 64 bytes; its four 16-byte chunks are XOR-swizzled by (row / 4) % 4, so that the 16 rows x 16 bytes a quarter
//     wave fetches with ds_read_b128 cover all 64 banks once; a wave-level load deposits 16 rows, the lane choosing the chunk it
//     fetches so that the block lands swizzled.
//   * The wave tile is 128 columns wide = one normalisation tile: the row-owning epilogues (16-bit stores, row-tile normalise + RoPE)
//     work inside a wave.  They stage 32 rows at a time in 8 KB of the wave's own LDS.
//   * The same k order per accumulator as the other kernels (bytes 0..63 of a step by one 32x32x64 MFMA, or two 32x32x32 / four
//     32x32x16 in ascending order): int32 sums are bit-identical, fp32 sums differ only where a stage boundary falls differently,
//     which it does not (128-byte steps are two 64-byte steps in the same order).
#include "gemm_epilogue.h"

using namespace gemmk;

namespace
{
constexpr int TK = 64; // bytes of K per step

__device__ __forceinline__ int Swz64(int row, int chunk)
{
    return row * TK + ((chunk ^ ((row >> 2) & 3)) << 4);
}

template <int TYPE, int CT, int EPI> __global__ void __launch_bounds__(256, 2) GemmNTTwin(GemmP p)
{
    typedef typename AccT<TYPE>::type TAcc;
    constexpr int WTM = 2, WTN = 4, NW = 4, BM = 256, BN = 128;
    // the 16-bit epilogues work on transposed blocks (a lane owns a row): the MFMAs take their operands the other way round
    constexpr bool SWAPC = CT == C_BF16NORM || ((CT == C_BF16 || CT == C_F16) && EPI == TS2_EPI_STORE);
    __shared__ __attribute__((aligned(1024))) uint8_t sA0[BM * TK];
    __shared__ __attribute__((aligned(1024))) uint8_t sA1[BM * TK];
    __shared__ __attribute__((aligned(1024))) uint8_t sA2[BM * TK];
    __shared__ __attribute__((aligned(1024))) uint8_t sB0[BN * TK];
    __shared__ __attribute__((aligned(1024))) uint8_t sB1[BN * TK];
    __shared__ __attribute__((aligned(1024))) uint8_t sB2[BN * TK];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int tm, tn;
    MapTile(blockIdx.x, p.tilesM * p.tilesN, p.tilesM, p.tilesN, &tm, &tn, p.mapGroup ? p.mapGroup : 8);
    const int rowBase = tm * BM;
    const int colBase = tn * BN;
    const int kSteps = p.kBytes / TK;

    // loader: a wave-level load fills 16 stage rows; lane -> (row = lane / 4, slot = lane % 4), and the slot holds chunk
    // slot ^ ((row / 4) % 4) of the row.  Wave w fills the blocks w, w + 4, ..
    const int lrow = lane >> 2;
    const int lchunk = (lane & 3) ^ ((lane >> 4) & 3);
    // Buffer addressing: the tile's first row is the base of a descriptor in scalar registers, the lane adds one 32-bit offset, the
    // 16-row block and the K step a scalar one: a load costs no 64-bit vector arithmetic and keeps no address registers.
    const int64_t aTileOff = (int64_t)rowBase * p.lda, bTileOff = (int64_t)colBase * p.ldb;
    const int lda = (int)p.lda, ldb = (int)p.ldb;
    __amdgpu_buffer_rsrc_t rsrcA = __builtin_amdgcn_make_buffer_rsrc((void *)(p.a + aTileOff), 0, (BM - 1) * lda + p.kBytes, 0x00020000);
    __amdgpu_buffer_rsrc_t rsrcB = __builtin_amdgcn_make_buffer_rsrc((void *)(p.b + bTileOff), 0, (BN - 1) * ldb + p.kBytes, 0x00020000);
    const int gaLane = lrow * lda + lchunk * 16;
    const int gbLane = lrow * ldb + lchunk * 16;
    constexpr int LA = BM / (16 * NW); // 4
    constexpr int LB = BN / (16 * NW); // 2
    constexpr int LT = LA + LB;
    const int lastStep = kSteps - 1;
    // load I of the LT loads of step STEP: the first LA fill the A stage, the others the B stage
#define TWIN_LOAD1(SA, SB, STEP, I)                                                                                                        \
    do {                                                                                                                                   \
        const int st_ = (STEP) < lastStep ? (STEP) : lastStep;                                                                             \
        if ((I) < LA) {                                                                                                                    \
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcA, TS2_LDS_PTR(SA + (wave + NW * (I)) * 1024), 16, gaLane,                        \
                (wave + NW * (I)) * 16 * lda + st_ * TK, 0, 0);                                                                            \
        } else {                                                                                                                           \
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcB, TS2_LDS_PTR(SB + (wave + NW * ((I)-LA)) * 1024), 16, gbLane,                   \
                (wave + NW * ((I)-LA)) * 16 * ldb + st_ * TK, 0, 0);                                                                       \
        }                                                                                                                                  \
    } while (0)
#define TWIN_LOADS(SA, SB, STEP)                                                                                                           \
    do {                                                                                                                                   \
        _Pragma("unroll") for (int i = 0; i < LT; ++i) TWIN_LOAD1(SA, SB, STEP, i);                                                        \
    } while (0)

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
    const int aRow0 = wave * (32 * WTM) + l32;
    const int bRow0 = l32;
    constexpr int NS = TYPE == T_FP8 ? 1 : 2; // K slices per step: 64 bytes (f8f6f4 32x32x64) or 32 bytes (i8 32x32x32, bf16 32x32x16)
    constexpr int ND = (WTM + WTN) * (TYPE == T_FP8 ? 2 : 1); // ds_read_b128 per fragment set
    typedef typename std::conditional<TYPE == T_FP8, v8i, v4i>::type TFrag;
    TFrag fa[NS][WTM], fb[NS][WTN];
    auto loadOne = [&](const uint8_t *base, int row, int sl) -> TFrag {
        if constexpr (TYPE == T_FP8) {
            v4i lo = *(const v4i *)(base + Swz64(row, half * 2));
            v4i hi = *(const v4i *)(base + Swz64(row, half * 2 + 1));
            return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        } else {
            return *(const v4i *)(base + Swz64(row, sl * 2 + half));
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
    // End of a step: this wave's loads except the newest LT (those of step S+2) have landed and its LDS reads have returned, then the
    // workgroup barrier.  A plain s_barrier behind explicit waits: the fence of __syncthreads() would drain every load in flight.
#define TWIN_BARRIER()                                                                                                                     \
    do {                                                                                                                                   \
        __builtin_amdgcn_s_waitcnt(0x0070 | LT);                                                                                           \
        asm volatile("" ::: "memory");                                                                                                     \
        __builtin_amdgcn_s_barrier();                                                                                                      \
        asm volatile("" ::: "memory");                                                                                                     \
    } while (0)
    // One K step.  (CA, CB): the stage of step S, (NA, NB) of step S+1, (FA, FB) receives step S+2.
    // i8 / bf16 (two K slices per step): slice 0 in fragment set 0, slice 1 in set 1, the next step's slice 0 fetched behind the barrier.
#define STEP2(CA, CB, NA, NB, FA, FB, S)                                                                                                   \
    do {                                                                                                                                   \
        TWIN_LOADS(FA, FB, (S) + 2);                                                                                                       \
        LOAD_FRAGS(1, CA, CB, 1);                                                                                                          \
        MFMA_ROWS(0, 0, 2);                                                                                                                \
        INTERLEAVE(6, 1, 1, 1);                                                                                                            \
        __builtin_amdgcn_sched_barrier(0);                                                                                                 \
        MFMA_ROWS(1, 0, 1);                                                                                                                \
        __builtin_amdgcn_sched_barrier(0);                                                                                                 \
        TWIN_BARRIER();                                                                                                                    \
        LOAD_FRAGS(0, NA, NB, 0);                                                                                                          \
        __builtin_amdgcn_sched_barrier(0);                                                                                                 \
        MFMA_ROWS(1, 1, 2);                                                                                                                \
    } while (0)
    // e4m3 (one slice per step, a fragment is 8 registers): ONE fragment set, refilled in place.  The eight MFMAs of a step run
    // (0,0) (0,1) (0,2) (0,3) | barrier | (1,0) (1,1) (1,2) (1,3); fa[0] is free after the fourth, fb[j] after (1,j), fa[1] and fb[3]
    // after the last, and each is fetched from the next stage as soon as it is free, three or four MFMAs (192+ cycles) before its
    // first use.  Two full sets would not fit beside the 128 accumulator registers within the 256 registers of a wave.
    // The MFMAs are volatile asm statements: the order written here is the order issued (as builtins they are pure values that the
    // compiler sinks towards their uses, i.e. into the next step, and then copies accumulators between registers at the loop edges).
#define MF(I, J)                                                                                                                           \
    do {                                                                                                                                   \
        if constexpr (SWAPC) {                                                                                                             \
            asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, %1, %2, %0" : "+v"(acc[I][J]) : "v"(fb[0][J]), "v"(fa[0][I]));                    \
        } else {                                                                                                                           \
            asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, %1, %2, %0" : "+v"(acc[I][J]) : "v"(fa[0][I]), "v"(fb[0][J]));                    \
        }                                                                                                                                  \
        FENCE();                                                                                                                           \
    } while (0)
#define FENCE() __builtin_amdgcn_sched_barrier(0)
#define STEP1(CA, CB, NA, NB, FA, FB, S)                                                                                                   \
    do {                                                                                                                                   \
        MF(0, 0);                                                                                                                          \
        TWIN_LOAD1(FA, FB, (S) + 2, 0);                                                                                                    \
        TWIN_LOAD1(FA, FB, (S) + 2, 1);                                                                                                    \
        FENCE();                                                                                                                           \
        MF(0, 1);                                                                                                                          \
        TWIN_LOAD1(FA, FB, (S) + 2, 2);                                                                                                    \
        TWIN_LOAD1(FA, FB, (S) + 2, 3);                                                                                                    \
        FENCE();                                                                                                                           \
        MF(0, 2);                                                                                                                          \
        TWIN_LOAD1(FA, FB, (S) + 2, 4);                                                                                                    \
        FENCE();                                                                                                                           \
        MF(0, 3);                                                                                                                          \
        TWIN_LOAD1(FA, FB, (S) + 2, 5);                                                                                                    \
        FENCE();                                                                                                                           \
        TWIN_BARRIER();                                                                                                                    \
        fa[0][0] = loadOne(NA, aRow0, 0);                                                                                                  \
        FENCE();                                                                                                                           \
        MF(1, 0);                                                                                                                          \
        fb[0][0] = loadOne(NB, bRow0, 0);                                                                                                  \
        FENCE();                                                                                                                           \
        MF(1, 1);                                                                                                                          \
        fb[0][1] = loadOne(NB, bRow0 + 32, 0);                                                                                             \
        FENCE();                                                                                                                           \
        MF(1, 2);                                                                                                                          \
        fb[0][2] = loadOne(NB, bRow0 + 64, 0);                                                                                             \
        FENCE();                                                                                                                           \
        MF(1, 3);                                                                                                                          \
        fb[0][3] = loadOne(NB, bRow0 + 96, 0);                                                                                             \
        fa[0][1] = loadOne(NA, aRow0 + 32, 0);                                                                                             \
        FENCE();                                                                                                                           \
    } while (0)
#define STEP(CA, CB, NA, NB, FA, FB, S)                                                                                                    \
    do {                                                                                                                                   \
        if constexpr (NS == 1) {                                                                                                           \
            STEP1(CA, CB, NA, NB, FA, FB, S);                                                                                              \
        } else {                                                                                                                           \
            STEP2(CA, CB, NA, NB, FA, FB, S);                                                                                              \
        }                                                                                                                                  \
    } while (0)

    static_assert(LT <= 15, "vmcnt immediate");
    // several products into the same accumulators: one pass of the pipeline per product, the fp32 sums rescaled in between so that the
    // epilogue's single factor, the last product's, is right for all of them.  A product whose factor is zero is skipped.
    float units = 0;
    for (int seg = 0; seg < p.nSeg; ++seg) {
        if (seg > 0) {
            rsrcA = __builtin_amdgcn_make_buffer_rsrc((void *)((seg == 1 ? p.segA[0] : seg == 2 ? p.segA[1] : p.segA[2]) + aTileOff), 0,
                (BM - 1) * lda + p.kBytes, 0x00020000);
            rsrcB = __builtin_amdgcn_make_buffer_rsrc((void *)((seg == 1 ? p.segB[0] : seg == 2 ? p.segB[1] : p.segB[2]) + bTileOff), 0,
                (BN - 1) * ldb + p.kBytes, 0x00020000);
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
            TWIN_LOADS(sA0, sB0, 0);
            TWIN_LOADS(sA1, sB1, 1);
            TWIN_BARRIER();
            LOAD_FRAGS(0, sA0, sB0, 0);
            int s = 0;
            for (; s + 3 <= kSteps; s += 3) {
                STEP(sA0, sB0, sA1, sB1, sA2, sB2, s);
                STEP(sA1, sB1, sA2, sB2, sA0, sB0, s + 1);
                STEP(sA2, sB2, sA0, sB0, sA1, sB1, s + 2);
            }
            // up to two steps left, in the same rotation (separate conditionals, not nested ones: every join then has two predecessors
            // and the accumulators stay in place)
            const int rem = kSteps - s;
            if (rem > 0) {
                STEP(sA0, sB0, sA1, sB1, sA2, sB2, s);
            }
            if (rem > 1) {
                STEP(sA1, sB1, sA2, sB2, sA0, sB0, s + 1);
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0F70); // the redundant loads of the last steps
        if constexpr (NS == 1) {
            // the compiler does not see the MFMAs inside the asm statements: the 18 wait states between the last one and the first
            // read of its result are spelled out
            asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
        }
        __syncthreads();
    } // products
    if constexpr (TYPE != T_I8) {
        if (p.nSeg > 1) {
            p.alpha = units;
            p.alphaPtr = nullptr;
        }
    }
#undef STEP
#undef STEP1
#undef STEP2
#undef MF
#undef FENCE
#undef TWIN_BARRIER
#undef INTERLEAVE
#undef LOAD_FRAGS
#undef MFMA_ROWS
#undef TWIN_LOADS
#undef TWIN_LOAD1
    if constexpr (SWAPC) {
        // every wave stages 32 of its rows at a time in 8 KB of a stage array of its own
        uint8_t *waveLds = wave == 0 ? sA0 : wave == 1 ? sA1 : wave == 2 ? sA2 : sB0;
        NormEpilogueRows<TYPE, CT == C_BF16NORM, CT == C_F16, WTM, WTN, true>(p, acc, waveLds, (float *)sB1, rowBase, colBase, wave, 0, lane);
    } else {
        Epilogue<TYPE, WTM, WTN, CT, EPI, false>(p, acc, facc, sA0, rowBase, colBase, wave, 0, half, l32);
    }
}

template <int TYPE, int CT, int EPI> int LaunchTwin(const GemmP &p, hipStream_t stream)
{
    GemmP q = p;
    q.tilesM = p.m / 256;
    q.tilesN = p.n / 128;
    const int nb = q.tilesM * q.tilesN;
    if (!p.mapGroup) {
        // an XCD runs nb/8 consecutive tiles: group the order so that they cover about as many bytes of A as of B
        const int chunk = (nb % 8) == 0 ? nb / 8 : nb;
        q.mapGroup = chunk >= 128 ? 8 : chunk >= 16 ? 4 : 2;
    }
    hipLaunchKernelGGL((GemmNTTwin<TYPE, CT, EPI>), dim3(nb), dim3(256), 0, stream, q);
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

template <int TYPE> int DispatchTwin(const GemmP &p, int ct, int epi, hipStream_t stream)
{
    if (ct == C_F32) {
        return epi == TS2_EPI_ADD ? LaunchTwin<TYPE, C_F32, TS2_EPI_ADD>(p, stream) : LaunchTwin<TYPE, C_F32, TS2_EPI_STORE>(p, stream);
    }
    if (ct == C_BF16) {
        return epi == TS2_EPI_ADD ? LaunchTwin<TYPE, C_BF16, TS2_EPI_ADD>(p, stream) : LaunchTwin<TYPE, C_BF16, TS2_EPI_STORE>(p, stream);
    }
    if (epi != TS2_EPI_STORE) {
        return TS2_ERR_UNSUPPORTED;
    }
    if (ct == C_BF16NORM) {
        return LaunchTwin<TYPE, C_BF16NORM, TS2_EPI_STORE>(p, stream);
    }
    if (ct == C_F16) {
        return LaunchTwin<TYPE, C_F16, TS2_EPI_STORE>(p, stream);
    }
    if constexpr (TYPE == T_I8) {
        if (ct == C_I32) {
            return LaunchTwin<TYPE, C_I32, TS2_EPI_STORE>(p, stream);
        }
    }
    return TS2_ERR_UNSUPPORTED;
}
} // namespace

namespace gemmk
{
bool TwinCanRun(const GemmP &p, int type, int ct, int epi)
{
    if (p.m % 256 || p.n % 128 || p.kBytes % TK || p.kBytes < TK) {
        return false;
    }
    if (p.tileGroup || p.groupOffsets || p.kTileScale || p.kMajor || p.splitK > 1 || p.splits > 1) {
        return false;
    }
    if (ct == C_I8PACK || (ct == C_I32 && type != T_I8)) {
        return false;
    }
    if (p.nSeg > 1 && (type == T_I8 || !(ct == C_F32 || ct == C_BF16))) {
        return false;
    }
    return true;
}

int RunTwin(const GemmP &p, int type, int ct, int epi, hipStream_t stream)
{
    if (!TwinCanRun(p, type, ct, epi)) {
        return TS2_ERR_UNSUPPORTED;
    }
    switch (type) {
    case T_I8:
        return DispatchTwin<T_I8>(p, ct, epi, stream);
    case T_FP8:
        return DispatchTwin<T_FP8>(p, ct, epi, stream);
    default:
        return DispatchTwin<T_BF16>(p, ct, epi, stream);
    }
}
} // namespace gemmk
