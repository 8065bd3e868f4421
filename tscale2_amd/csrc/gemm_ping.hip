// Persistent NT GEMM whose epilogue runs under the next tile's main loop:  C[m][n] (op)= scale * sum_k A[m][k] * B[n][k]
//
// One workgroup of eight waves per CU walks a list of 256x128 tiles.  The waves form two groups of four (one wave of each group on
// every SIMD); a group owns every other tile of the list.  While group X multiplies tile t (wave tile 64x128 = 2x4 MFMA 32x32 blocks,
// 128 accumulator registers), group Y scales and stores tile t-1 from its registers and clears them; at the end of the tile the
// groups change roles.  The operand stages form ONE ring that both groups read in turn: three stages of 256 rows of A and 128 rows of
// B, 128 contraction bytes per row (48 KB each, the same swizzled layout and 128-byte global lines as the 256x256 ring kernel of
// gemm.hip).  The loads run two steps ahead of the MFMAs straight through the tile boundaries, so that the pipeline is never drained or
// refilled between tiles, and the matrix cores of a CU idle neither while results are stored nor while first operands arrive - which
// costs the one-workgroup-per-CU kernel a third of the time of a product with a 2048-byte contraction.
// It plays the role of the reference's GEMM cores (src/lib/cuda/cuda_i8.cuh:157-320, src/lib/cuda/cuda_matmul.cuh:396-416,
// src/lib/cuda/sm90_fp8.cuh:171-217).
//
//   * Time is cut into slots of one 128-byte contraction step; every slot ends with a workgroup barrier that all eight waves reach.
//     The group that multiplies issues the loads of step S+2 (twelve wave-level loads per wave, global -> LDS directly) between its
//     MFMAs; "all but the newest twelve" before the barrier means step S+1 has landed.  The other group does one piece of its epilogue
//     (one 32x32 block of its wave tile) per slot and then only keeps the barrier count.
//   * The loads are asm statements (the compiler then inserts no waits of its own between them and the LDS reads, and the stage can be
//     chosen at run time); the LDS reads are ordinary loads, so the compiler tracks their arrival; the MFMAs are asm statements so
//     that they are issued in the order written (as builtins they are pure values which the compiler sinks towards their uses).
//   * One fragment set, refilled in place: of the eight MFMAs of a 64-byte slice fa[0] is free after the fourth, fb[j] after (1,j),
//     and each is fetched again - from the next slice, behind the barrier from the next stage - as soon as it is free.
//   * Same contraction order per accumulator as every other kernel of the library, so results are bit-identical to theirs.
//   * Expert-grouped products (the reference's TMoeMatMulKernelCall, src/gpt/compute/moe_matmul.cuh:47-120) run on the same schedule
//     with the operands exchanged, see GRP below.
#include "gemm_epilogue.h"

using namespace gemmk;

namespace
{
constexpr int PK = 128;                  // contraction bytes per step
constexpr int PBM = 256, PBN = 128;      // tile of a group
constexpr int PSTAGE = (PBM + PBN) * PK; // 48 KB
constexpr int PLDS = 3 * PSTAGE;

typedef __attribute__((address_space(3))) uint8_t *TLds;

struct PingP {
    GemmP g;
    int nTiles;
};

// descriptor of rows [row0, row0 + rows) of an operand, in scalar registers
__device__ __forceinline__ v4i MakeRsrc(const uint8_t *base, int64_t off, int bytes)
{
    const uint64_t a = (uint64_t)(uintptr_t)(base + off);
    v4i r;
    r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
    r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32) & 0xffff);
    r[2] = __builtin_amdgcn_readfirstlane(bytes);
    r[3] = 0x00020000;
    return r;
}

// GRP (expert-grouped products, e4m3, 16-bit result): the roles of the operands are exchanged.  The 256-row side of a tile holds rows
// of the weight slab of the tile's expert (p.a = the slabs, p.bSlab apart), the 128-row side the 128 tokens of one row tile of the
// expert-ordered activations (p.b), whose expert p.tileGroup names (-1: nothing is stored).  A block of accumulators is then C^T:
// a lane owns a token and four consecutive result columns per register quad, and the wave's 64 columns of 32 tokens leave as whole
// 128-byte row segments through 4 KB of the wave's own LDS, one token block per slot.  With the normalising epilogue a token's 128-column
// tile spans two waves (64 columns each): in a first piece every wave leaves its sums of squares in its partner's LDS area, the slot
// barrier separates that from the partner reading them, and the four token blocks follow.  The last tile of a workgroup has no slot
// barriers left, so there the group that is already done keeps one barrier for the other's exchange.
template <int TYPE, int CT, int EPI, bool GRP = false> __global__ void __launch_bounds__(512, 2) GemmNTPing(PingP pp)
{
    typedef typename AccT<TYPE>::type TAcc;
    const GemmP &p = pp.g;
    constexpr int WTM = 2, WTN = 4;
    // the normalising epilogue works on transposed blocks (a lane owns a row): the MFMAs take their operands the other way round
    constexpr bool SWAPC = CT == C_BF16NORM && !GRP;
    __shared__ __attribute__((aligned(1024))) uint8_t lds[PLDS];
    static_assert(!GRP || ((CT == C_BF16 || CT == C_F16 || CT == C_BF16NORM) && EPI == TS2_EPI_STORE && TYPE == T_FP8), "grouped: e4m3 operands, 16-bit result");
    __shared__ __attribute__((aligned(1024))) uint8_t ldsEpi[CT == C_BF16NORM || GRP ? 16384 : 16]; // 4 KB per wave of the storing group

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int group = wave >> 2; // waves w and w + 4 share a SIMD
    const int gw = wave & 3;
    const int half = lane >> 5, l32 = lane & 31;
    // grouped products may add a second product of the same shapes into the same accumulators (p.nSeg == 2: operands segA[0], segB[0]):
    // its steps follow the first product's, and at the seam the accumulators are brought to the second product's factor, which is the
    // one the epilogue applies - the same arithmetic as the two-product form of the 128x128 kernel.  A second factor of zero (the scale
    // of an all-zero matrix) leaves the first product alone.
    const int kSlots1 = p.kBytes / PK;
    bool twoProducts = false;
    float seamRatio = 1.f, unitsOfSum = 0.f;
    if constexpr (GRP) {
        if (p.nSeg == 2) {
            float cur = p.alpha, nxt = p.segAlpha[0];
            if (p.alphaPtr) {
                cur *= *p.alphaPtr;
            }
            if (p.segAlphaPtr[0]) {
                nxt *= *p.segAlphaPtr[0];
            }
            unitsOfSum = cur;
            if (nxt != 0) {
                twoProducts = true;
                unitsOfSum = nxt;
                seamRatio = cur / nxt;
            }
        }
    }
    const int kSlots = twoProducts ? 2 * kSlots1 : kSlots1;
    const int myTiles = ((int)blockIdx.x < pp.nTiles) ? (pp.nTiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x : 0;
    const unsigned ldsBase = (unsigned)(uintptr_t)(TLds)lds;
    const int lda = (int)p.lda, ldb = (int)p.ldb;

    // ---- loader.  A wave-level load fills 8 stage rows of 128 bytes; lane -> (row = lane / 8, slot = lane % 8), the slot holds chunk
    // slot ^ ((row / 2) % 8) of the row.  Wave gw of the multiplying group fills the blocks gw, gw + 4, .. (all of one parity, so the
    // chunk is fixed): 8 of A, 4 of B.
    const int lrow = gw * 8 + (lane >> 3);
    const int lchunk = (lane & 7) ^ ((lrow >> 1) & 7);
    const int gaLane = (lane >> 3) * lda + lchunk * 16;
    const int gbLane = (lane >> 3) * ldb + lchunk * 16;
    // tile number i of this workgroup -> first row / column
    auto tileOrigin = [&](int i, int *rowBase, int *colBase) {
        int tm, tn;
        MapTile((int)blockIdx.x + i * (int)gridDim.x, pp.nTiles, p.tilesM, p.tilesN, &tm, &tn, p.mapGroup ? p.mapGroup : 8);
        *rowBase = tm * PBM;
        *colBase = tn * PBN;
    };
    auto tileRsrcOf = [&](const uint8_t *baseA, const uint8_t *baseB, int i, v4i *ra, v4i *rb) {
        int rowBase, colBase;
        tileOrigin(i < myTiles ? i : myTiles - 1, &rowBase, &colBase);
        int64_t slab = 0;
        if constexpr (GRP) {
            const int g = p.tileGroup[colBase / PBN];
            slab = g > 0 ? g * p.bSlab : 0; // (a tile without an expert multiplies the first slab and stores nothing)
        }
        *ra = MakeRsrc(baseA, slab + (int64_t)rowBase * p.lda, (PBM - 1) * lda + p.kBytes);
        *rb = MakeRsrc(baseB, (int64_t)colBase * p.ldb, (PBN - 1) * ldb + p.kBytes);
    };
    auto tileRsrc = [&](int i, v4i *ra, v4i *rb) { tileRsrcOf(p.a, p.b, i, ra, rb); };
#define PING_LOAD(M0VAL, VOFF, RSRC, SOFF)                                                                                                 \
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" ::"s"(M0VAL), "v"(VOFF), "s"(RSRC), "s"(SOFF) : "memory")
    // load number I (0..11) of a step: the first 8 are A blocks gw + 4 * I, the others B blocks
#define PING_LOAD1(STOFF, RA, RB, KOFF, I)                                                                                                 \
    do {                                                                                                                                   \
        if ((I) < 8) {                                                                                                                     \
            PING_LOAD(ldsBase + (STOFF) + (gw + 4 * (I)) * 1024, gaLane, RA, (gw + 4 * (I)) * 8 * lda + (KOFF));                           \
        } else {                                                                                                                           \
            PING_LOAD(ldsBase + (STOFF) + PBM * PK + (gw + 4 * ((I)-8)) * 1024, gbLane, RB, (gw + 4 * ((I)-8)) * 8 * ldb + (KOFF));        \
        }                                                                                                                                  \
    } while (0)

    // ---- operand fragments: row r of a stage at r * 128, chunk c at slot c ^ ((r / 2) % 8)
    typedef typename std::conditional<TYPE == T_FP8, v8i, v4i>::type TFrag;
    constexpr int NS = TYPE == T_FP8 ? 2 : 4; // slices of a step: 64 bytes (f8f6f4 32x32x64) or 32 (i8 32x32x32, bf16 32x32x16)
    const int sw = (l32 >> 1) & 7;
    const int aLane = (gw * 64 + l32) * PK, bLane = PBM * PK + l32 * PK;
    auto frag = [&](int stOff, int laneBase, int blk, int sl) -> TFrag {
        const uint8_t *row = lds + stOff + laneBase + blk * (32 * PK);
        if constexpr (TYPE == T_FP8) {
            const int c = sl * 4 + half * 2;
            v4i lo = *(const v4i *)(row + ((c ^ sw) << 4));
            v4i hi = *(const v4i *)(row + (((c + 1) ^ sw) << 4));
            return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        } else {
            return *(const v4i *)(row + (((sl * 2 + half) ^ sw) << 4));
        }
    };
    TAcc acc[WTM][WTN];
    TFrag fa[WTM], fb[WTN];
#define FENCE() __builtin_amdgcn_sched_barrier(0)
#define MF(I, J)                                                                                                                           \
    do {                                                                                                                                   \
        if constexpr (TYPE == T_FP8) {                                                                                                     \
            if constexpr (SWAPC) {                                                                                                         \
                asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, %1, %2, %0" : "+v"(acc[I][J]) : "v"(fb[J]), "v"(fa[I]));                      \
            } else {                                                                                                                       \
                asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, %1, %2, %0" : "+v"(acc[I][J]) : "v"(fa[I]), "v"(fb[J]));                      \
            }                                                                                                                              \
        } else if constexpr (TYPE == T_I8) {                                                                                               \
            if constexpr (SWAPC) {                                                                                                         \
                asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(acc[I][J]) : "v"(fb[J]), "v"(fa[I]));                          \
            } else {                                                                                                                       \
                asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(acc[I][J]) : "v"(fa[I]), "v"(fb[J]));                          \
            }                                                                                                                              \
        } else {                                                                                                                           \
            if constexpr (SWAPC) {                                                                                                         \
                asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[I][J]) : "v"(fb[J]), "v"(fa[I]));                        \
            } else {                                                                                                                       \
                asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[I][J]) : "v"(fa[I]), "v"(fb[J]));                        \
            }                                                                                                                              \
        }                                                                                                                                  \
        FENCE();                                                                                                                           \
    } while (0)
#define ZERO_ACC()                                                                                                                         \
    do {                                                                                                                                   \
        _Pragma("unroll") for (int i = 0; i < WTM; ++i) _Pragma("unroll") for (int j = 0; j < WTN; ++j) _Pragma("unroll") for (int e = 0;  \
                                                                                                                             e < 16; ++e)  \
            acc[i][j][e] = 0;                                                                                                              \
    } while (0)
    // the barrier that ends a slot
#define SLOT_BARRIER_MUL()                                                                                                                 \
    do {                                                                                                                                   \
        asm volatile("s_waitcnt vmcnt(12) lgkmcnt(0)\n\ts_barrier" ::: "memory");                                                          \
    } while (0)
#define SLOT_BARRIER() asm volatile("s_barrier" ::: "memory")

    // One slot of the multiplying group: slices 0 .. NS-1 of the step in stage stC; the loads of step S+2 (stage stL, descriptors and
    // contraction offset of that step) go out one behind each of the first MFMAs; behind the barrier the fragments of step S+1's first
    // slice are fetched from stage stN unless LAST (the next step is the other group's).
    // MFMAs per load: e4m3 16 MFMAs per slot, i8 / bf16 32
    constexpr int MPL = TYPE == T_FP8 ? 1 : 2;
#define SLICE(Q, STC, STN, STL, RA, RB, KOFF, LAST)                                                                                        \
    do {                                                                                                                                   \
        constexpr bool lastSlice_ = (Q) == NS - 1;                                                                                         \
        constexpr int m0_ = (Q)*8;                                                                                                         \
        MF(0, 0);                                                                                                                          \
        if ((m0_ + 0) % MPL == 0 && (m0_ + 0) / MPL < 12) { PING_LOAD1(STL, RA, RB, KOFF, (m0_ + 0) / MPL); FENCE(); }                     \
        MF(0, 1);                                                                                                                          \
        if ((m0_ + 1) % MPL == 0 && (m0_ + 1) / MPL < 12) { PING_LOAD1(STL, RA, RB, KOFF, (m0_ + 1) / MPL); FENCE(); }                     \
        MF(0, 2);                                                                                                                          \
        if ((m0_ + 2) % MPL == 0 && (m0_ + 2) / MPL < 12) { PING_LOAD1(STL, RA, RB, KOFF, (m0_ + 2) / MPL); FENCE(); }                     \
        MF(0, 3);                                                                                                                          \
        if ((m0_ + 3) % MPL == 0 && (m0_ + 3) / MPL < 12) { PING_LOAD1(STL, RA, RB, KOFF, (m0_ + 3) / MPL); FENCE(); }                     \
        if (lastSlice_) {                                                                                                                  \
            SLOT_BARRIER_MUL();                                                                                                            \
        }                                                                                                                                  \
        if (!(lastSlice_ && (LAST))) {                                                                                                     \
            fa[0] = frag(lastSlice_ ? (STN) : (STC), aLane, 0, lastSlice_ ? 0 : (Q) + 1);                                                  \
            FENCE();                                                                                                                       \
        }                                                                                                                                  \
        MF(1, 0);                                                                                                                          \
        if ((m0_ + 4) % MPL == 0 && (m0_ + 4) / MPL < 12) { PING_LOAD1(STL, RA, RB, KOFF, (m0_ + 4) / MPL); FENCE(); }                     \
        if (!(lastSlice_ && (LAST))) {                                                                                                     \
            fb[0] = frag(lastSlice_ ? (STN) : (STC), bLane, 0, lastSlice_ ? 0 : (Q) + 1);                                                  \
            FENCE();                                                                                                                       \
        }                                                                                                                                  \
        MF(1, 1);                                                                                                                          \
        if ((m0_ + 5) % MPL == 0 && (m0_ + 5) / MPL < 12) { PING_LOAD1(STL, RA, RB, KOFF, (m0_ + 5) / MPL); FENCE(); }                     \
        if (!(lastSlice_ && (LAST))) {                                                                                                     \
            fb[1] = frag(lastSlice_ ? (STN) : (STC), bLane, 1, lastSlice_ ? 0 : (Q) + 1);                                                  \
            FENCE();                                                                                                                       \
        }                                                                                                                                  \
        MF(1, 2);                                                                                                                          \
        if ((m0_ + 6) % MPL == 0 && (m0_ + 6) / MPL < 12) { PING_LOAD1(STL, RA, RB, KOFF, (m0_ + 6) / MPL); FENCE(); }                     \
        if (!(lastSlice_ && (LAST))) {                                                                                                     \
            fb[2] = frag(lastSlice_ ? (STN) : (STC), bLane, 2, lastSlice_ ? 0 : (Q) + 1);                                                  \
            FENCE();                                                                                                                       \
        }                                                                                                                                  \
        MF(1, 3);                                                                                                                          \
        if ((m0_ + 7) % MPL == 0 && (m0_ + 7) / MPL < 12) { PING_LOAD1(STL, RA, RB, KOFF, (m0_ + 7) / MPL); FENCE(); }                     \
        if (!(lastSlice_ && (LAST))) {                                                                                                     \
            fb[3] = frag(lastSlice_ ? (STN) : (STC), bLane, 3, lastSlice_ ? 0 : (Q) + 1);                                                  \
            fa[1] = frag(lastSlice_ ? (STN) : (STC), aLane, 1, lastSlice_ ? 0 : (Q) + 1);                                                  \
            FENCE();                                                                                                                       \
        }                                                                                                                                  \
    } while (0)
#define SLOT(STC, STN, STL, RA, RB, KOFF, LAST)                                                                                            \
    do {                                                                                                                                   \
        SLICE(0, STC, STN, STL, RA, RB, KOFF, LAST);                                                                                       \
        SLICE(1, STC, STN, STL, RA, RB, KOFF, LAST);                                                                                       \
        if constexpr (NS == 4) {                                                                                                           \
            SLICE(2, STC, STN, STL, RA, RB, KOFF, LAST);                                                                                   \
            SLICE(3, STC, STN, STL, RA, RB, KOFF, LAST);                                                                                   \
        }                                                                                                                                  \
    } while (0)

    // ---- epilogue pieces of the storing group: block (i, j) of the wave tile, lane = column, registers walk down the rows
    float scale = p.alpha;
    if (p.alphaPtr) {
        scale *= *p.alphaPtr;
    }
    if constexpr (GRP) {
        if (p.nSeg == 2) {
            scale = unitsOfSum;
        }
    }
    const int mLive = p.mLive > 0 ? p.mLive : GRP ? p.n : p.m;
    // old values of block (i, j) for the accumulating epilogue: fetched one piece ahead
    auto loadOld = [&](auto iTag, auto jTag, int rowBase, int colBase, float (&old)[16]) {
        constexpr int i = decltype(iTag)::value, j = decltype(jTag)::value;
        const int firstRow = rowBase + gw * 64;
        const int col = colBase + j * 32 + l32;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int row = firstRow + i * 32 + (e >> 2) * 8 + half * 4 + (e & 3);
            const uint8_t *src = p.c + (int64_t)row * p.ldc;
            if (CT == C_F32) {
                old[e] = row < mLive ? __builtin_nontemporal_load((const float *)src + col) : 0.f;
            } else {
                old[e] = row < mLive ? Bf16ToFloat(((const bf16_t *)src)[col]) : 0.f;
            }
        }
    };
    auto storeBlock = [&](auto iTag, auto jTag, int rowBase, int colBase, const float (&old)[16]) {
        constexpr int i = decltype(iTag)::value, j = decltype(jTag)::value;
        const int firstRow = rowBase + gw * 64; // of the wave tile
        const int col = colBase + j * 32 + l32;
        float v[16];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            float4 r = make_float4(1.f, 1.f, 1.f, 1.f);
            if (p.rowScale) {
                r = *(const float4 *)(p.rowScale + firstRow + i * 32 + q * 8 + half * 4);
            }
            v[q * 4 + 0] = (float)acc[i][j][q * 4 + 0] * (scale * r.x);
            v[q * 4 + 1] = (float)acc[i][j][q * 4 + 1] * (scale * r.y);
            v[q * 4 + 2] = (float)acc[i][j][q * 4 + 2] * (scale * r.z);
            v[q * 4 + 3] = (float)acc[i][j][q * 4 + 3] * (scale * r.w);
        }
        auto rowOf = [&](int e) { return firstRow + i * 32 + (e >> 2) * 8 + half * 4 + (e & 3); };
        const bool allLive = firstRow + i * 32 + 32 <= mLive && (int64_t)64 * p.ldc < ((int64_t)1 << 31);
        if constexpr (CT == C_I32) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                ((int *)(p.c + (int64_t)rowOf(e) * p.ldc))[col] = (int)acc[i][j][e];
            }
        } else if constexpr (EPI == TS2_EPI_ADD) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                if (rowOf(e) < mLive) {
                    uint8_t *dst = p.c + (int64_t)rowOf(e) * p.ldc;
                    if (CT == C_F32) {
                        __builtin_nontemporal_store(old[e] + v[e], (float *)dst + col);
                    } else {
                        ((bf16_t *)dst)[col] = FloatToBf16(old[e] + v[e]);
                    }
                }
            }
        } else if (allLive) {
            const TWaveStore w = MakeWaveStore<WTM>(p.c, p.ldc, firstRow, colBase + l32, CT == C_F32 ? 4 : 2, half, l32);
            if constexpr (CT == C_F32) {
                if (p.streamC) {
                    StoreBlock32Buf<2>(w, i, j * 128, v);
                } else {
                    StoreBlock32Buf<0>(w, i, j * 128, v);
                }
            } else {
                if (p.streamC) {
                    StoreBlock16Buf<CT == C_F16, 2>(w, i, j * 64, v);
                } else {
                    StoreBlock16Buf<CT == C_F16, 0>(w, i, j * 64, v);
                }
            }
        } else {
            if constexpr (CT == C_F32) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    ((float *)(p.c + (int64_t)rowOf(e) * p.ldc))[col] = rowOf(e) < mLive ? v[e] : 0.f;
                }
            } else {
                StoreBlockBf16<CT == C_F16>(p.c, p.ldc, col, l32, mLive, v, rowOf);
            }
        }
    };
    // The normalising epilogue (TStoreRowTileNormalize / TStoreRowTileNormalizeRope): a lane owns row l32 of block row i.  The first
    // piece of a block row normalises, rotates and packs the row's 128 columns (pk) and sends columns 0..63 on their way, the second
    // piece columns 64..127: the rows are staged in 4 KB of the wave's own LDS (128 bytes per row, 8-byte granules XOR-swizzled by the
    // row pair) and leave as 16-byte stores of whole 128-byte row segments, eight lanes per row.
    uint8_t *waveEpi = ldsEpi + (CT == C_BF16NORM || GRP ? gw * 4096 : 0);
    auto normPack = [&](auto iTag, int rowBase, int colBase, uint2 (&pk)[4][4]) {
        constexpr int i = decltype(iTag)::value;
        const int row = rowBase + gw * 64 + i * 32 + l32;
        const bool live = row < mLive;
        float rs = scale;
        if (p.rowScale) {
            rs *= p.rowScale[row];
        }
        float v[4][16];
        NormRowValues<true, 4>(p, acc[i], row, live, rs, colBase / TILE, 0, half, true, 0.f, v);
        if (__builtin_amdgcn_readfirstlane(p.rowsF16)) { // (a branch, not 32 selects)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    pk[j][q] = make_uint2(PackF16x2(v[j][4 * q], v[j][4 * q + 1]), PackF16x2(v[j][4 * q + 2], v[j][4 * q + 3]));
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    pk[j][q] = make_uint2(PackBf16x2(v[j][4 * q], v[j][4 * q + 1]), PackBf16x2(v[j][4 * q + 2], v[j][4 * q + 3]));
                }
            }
        }
    };
    auto normFlush = [&](auto iTag, auto hTag, int rowBase, int colBase, const uint2 (&pk)[4][4]) {
        constexpr int i = decltype(iTag)::value, h = decltype(hTag)::value;
        typedef unsigned v4u_t __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int g = (jj * 8 + q * 2 + half) ^ (((l32 >> 1) & 7) << 1);
                *(uint2 *)(waveEpi + l32 * 128 + g * 8) = pk[h * 2 + jj][q];
            }
        }
        const int firstRow = rowBase + gw * 64;
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(p.c + (int64_t)firstRow * p.ldc), 0, (int)(64 * p.ldc), 0x00020000);
        const int ldc = (int)p.ldc;
        const int t8 = lane & 7, rsub = lane >> 3;
        const int laneOff = rsub * ldc + (colBase + h * 64) * 2 + t8 * 16;
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int r = it * 8 + rsub;
            const int g = (2 * t8) ^ (((r >> 1) & 7) << 1);
            const uint4 d = *(const uint4 *)(waveEpi + r * 128 + g * 8);
            const int so = (i * 32 + it * 8) * ldc;
            if (p.streamC) {
                __builtin_amdgcn_raw_buffer_store_b128((v4u_t){d.x, d.y, d.z, d.w}, rsrc, laneOff, so, 2);
            } else {
                __builtin_amdgcn_raw_buffer_store_b128((v4u_t){d.x, d.y, d.z, d.w}, rsrc, laneOff, so, 0);
            }
        }
    };
    // grouped products: token block j of the tile (32 tokens x the wave's 64 result columns); rowBase = first result column of the tile,
    // colBase = its first token
    // sums of squares of this wave's 64 columns for the tokens of the tile (lane = token l32 of block j; both half waves get the sum)
    auto grpSums = [&](int colBase, float (&own)[4]) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int token = colBase + j * 32 + l32;
            const bool live = token < mLive;
            float rs = scale;
            if (p.rowScale) {
                rs *= p.rowScale[token];
            }
            float sum = 0;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const float x = live ? (float)acc[i][j][e] * rs : 0.f;
                    sum += x * x;
                }
            }
            float a, b;
            LaneSwap32(sum, &a, &b);
            own[j] = a + b;
        }
    };
    auto grpFlush = [&](auto jTag, int rowBase, int colBase, float tileSum2) {
        constexpr int j = decltype(jTag)::value;
        typedef unsigned v4u_t __attribute__((ext_vector_type(4)));
        const int token = colBase + j * 32 + l32;
        const bool live = token < mLive;
        float rs = scale;
        if (p.rowScale) {
            rs *= p.rowScale[token];
        }
        float v[2][16];
        if constexpr (CT == C_BF16NORM) {
            TAcc two[2] = {acc[0][j], acc[1][j]};
            NormRowValues<true, 2>(p, two, token, live, rs, (rowBase + gw * 64) / TILE, (gw & 1) * 64, half, (gw & 1) == 0, tileSum2, v);
        } else {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    v[i][e] = live ? (float)acc[i][j][e] * rs : 0.f;
                }
            }
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float v0 = v[i][4 * q], v1 = v[i][4 * q + 1], v2 = v[i][4 * q + 2], v3 = v[i][4 * q + 3];
                const int g = (i * 8 + q * 2 + half) ^ (((l32 >> 1) & 7) << 1);
                *(uint2 *)(waveEpi + l32 * 128 + g * 8) =
                    CT == C_F16 ? make_uint2(PackF16x2(v0, v1), PackF16x2(v2, v3)) : make_uint2(PackBf16x2(v0, v1), PackBf16x2(v2, v3));
            }
        }
        const int firstToken = colBase + j * 32;
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(p.c + (int64_t)firstToken * p.ldc), 0, (int)(32 * p.ldc), 0x00020000);
        const int ldc = (int)p.ldc;
        const int t8 = lane & 7, rsub = lane >> 3;
        const int laneOff = rsub * ldc + (rowBase + gw * 64) * 2 + t8 * 16;
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int r = it * 8 + rsub;
            const int g = (2 * t8) ^ (((r >> 1) & 7) << 1);
            const uint4 d = *(const uint4 *)(waveEpi + r * 128 + g * 8);
            const int so = it * 8 * ldc;
            if (p.streamC) {
                __builtin_amdgcn_raw_buffer_store_b128((v4u_t){d.x, d.y, d.z, d.w}, rsrc, laneOff, so, 2);
            } else {
                __builtin_amdgcn_raw_buffer_store_b128((v4u_t){d.x, d.y, d.z, d.w}, rsrc, laneOff, so, 0);
            }
        }
    };
    // the whole epilogue of tile number t of this workgroup, one block per slot; nBarriers slot barriers are kept in all
    auto epiloguePhase = [&](int t, int nBarriers) {
        int rowBase, colBase;
        tileOrigin(t, &rowBase, &colBase);
        // the compiler does not see the MFMAs inside the asm statements: the wait states between the last one and the first read of a
        // result are spelled out
        asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
        FENCE(); // (no accumulator is read above this line)
        int done = 0;
#define END_PIECE()                                                                                                                        \
    do {                                                                                                                                   \
        if (done < nBarriers) {                                                                                                            \
            SLOT_BARRIER();                                                                                                                \
            ++done;                                                                                                                        \
        }                                                                                                                                  \
    } while (0)
        // (the first piece waits for the loads this group issued in its last two slots as the multiplying group)
#define WAIT_OWN_LOADS() asm volatile("s_waitcnt vmcnt(0)" ::: "memory")
        if constexpr (GRP) {
            const bool hasExpert = p.tileGroup[colBase / PBN] >= 0;
            float tileSum2[4] = {0.f, 0.f, 0.f, 0.f};
            if constexpr (CT == C_BF16NORM) {
                float own[4];
                grpSums(colBase, own);
                WAIT_OWN_LOADS();
                float *mine = (float *)waveEpi, *theirs = (float *)(ldsEpi + (gw ^ 1) * 4096);
                if (half == 0) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        theirs[j * 32 + l32] = own[j];
                    }
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                END_PIECE();
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    tileSum2[j] = own[j] + mine[j * 32 + l32];
                }
            }
#define GPIECE(J)                                                                                                                          \
    do {                                                                                                                                   \
        if ((J) == 0 && CT != C_BF16NORM) {                                                                                                \
            WAIT_OWN_LOADS();                                                                                                              \
        }                                                                                                                                  \
        if (hasExpert) {                                                                                                                   \
            grpFlush(std::integral_constant<int, J>(), rowBase, colBase, tileSum2[J]);                                                     \
        }                                                                                                                                  \
        END_PIECE();                                                                                                                       \
    } while (0)
            GPIECE(0);
            GPIECE(1);
            GPIECE(2);
            GPIECE(3);
#undef GPIECE
        } else if constexpr (CT == C_BF16NORM) {
            uint2 pk[4][4];
#define NPIECE(I)                                                                                                                          \
    do {                                                                                                                                   \
        normPack(std::integral_constant<int, I>(), rowBase, colBase, pk);                                                                  \
        if ((I) == 0) {                                                                                                                    \
            WAIT_OWN_LOADS();                                                                                                              \
        }                                                                                                                                  \
        normFlush(std::integral_constant<int, I>(), std::integral_constant<int, 0>(), rowBase, colBase, pk);                               \
        END_PIECE();                                                                                                                       \
        normFlush(std::integral_constant<int, I>(), std::integral_constant<int, 1>(), rowBase, colBase, pk);                               \
        END_PIECE();                                                                                                                       \
    } while (0)
            NPIECE(0);
            NPIECE(1);
#undef NPIECE
        } else {
            // accumulating epilogue: the old values of a block are fetched one piece ahead of their use.  (Deeper prefetch does not fit
            // beside the accumulators; products that accumulate are left to the 256x256 kernel by the dispatcher.)
            float oldA[16], oldB[16];
            if constexpr (EPI == TS2_EPI_ADD && CT != C_I32) {
                loadOld(std::integral_constant<int, 0>(), std::integral_constant<int, 0>(), rowBase, colBase, oldA);
            }
            // piece (I, J); (NI, NJ) is the next one (NI < 0: none)
#define PIECE(I, J, NI, NJ, OLD, NEXTOLD)                                                                                                  \
    do {                                                                                                                                   \
        if ((I) == 0 && (J) == 0) {                                                                                                        \
            WAIT_OWN_LOADS();                                                                                                              \
        }                                                                                                                                  \
        if constexpr (EPI == TS2_EPI_ADD && CT != C_I32) {                                                                                 \
            if ((NI) >= 0) {                                                                                                               \
                loadOld(std::integral_constant < int, (NI) < 0 ? 0 : (NI) > (), std::integral_constant<int, NJ>(), rowBase, colBase, NEXTOLD); \
            }                                                                                                                              \
        }                                                                                                                                  \
        storeBlock(std::integral_constant<int, I>(), std::integral_constant<int, J>(), rowBase, colBase, OLD);                             \
        END_PIECE();                                                                                                                       \
    } while (0)
            PIECE(0, 0, 0, 1, oldA, oldB);
            PIECE(0, 1, 0, 2, oldB, oldA);
            PIECE(0, 2, 0, 3, oldA, oldB);
            PIECE(0, 3, 1, 0, oldB, oldA);
            PIECE(1, 0, 1, 1, oldA, oldB);
            PIECE(1, 1, 1, 2, oldB, oldA);
            PIECE(1, 2, 1, 3, oldA, oldB);
            PIECE(1, 3, -1, 0, oldB, oldA);
#undef PIECE
        }
#undef WAIT_OWN_LOADS
#undef END_PIECE
        for (; done < nBarriers; ++done) {
            SLOT_BARRIER();
        }
    };

    // ---- the tile list.  Phase i (kSlots slots): group i % 2 multiplies tile i while the other group stores tile i - 1.  Each group
    // runs its own plain loop "multiply my tile, store it during the next phase": the accumulators are cleared at the start of a
    // tile and dead after its epilogue, so nothing but addresses is carried around the loop.
#define ROTATE(N)                                                                                                                          \
    do {                                                                                                                                   \
        if ((N) == 1) {                                                                                                                    \
            const int x_ = stC;                                                                                                            \
            stC = stN;                                                                                                                     \
            stN = stL;                                                                                                                     \
            stL = x_;                                                                                                                      \
        } else if ((N) == 2) {                                                                                                             \
            const int x_ = stL;                                                                                                            \
            stL = stN;                                                                                                                     \
            stN = stC;                                                                                                                     \
            stC = x_;                                                                                                                      \
        }                                                                                                                                  \
    } while (0)
    if (myTiles > 0) {
        int stC = 0, stN = PSTAGE, stL = 2 * PSTAGE; // stages of step S, S+1, S+2
        v4i ra, rb, na, nb;
        if (group == 0) {
            tileRsrc(0, &ra, &rb);
#pragma unroll
            for (int i = 0; i < 12; ++i) {
                PING_LOAD1(stC, ra, rb, 0, i);
            }
#pragma unroll
            for (int i = 0; i < 12; ++i) {
                PING_LOAD1(stN, ra, rb, PK, i);
            }
            SLOT_BARRIER_MUL();
        } else {
            SLOT_BARRIER();
            // phase 0 belongs to the other group
            for (int s = 0; s < kSlots; ++s) {
                SLOT_BARRIER();
            }
            ROTATE(kSlots % 3);
        }
        for (int t = group; t < myTiles; t += 2) {
            // ---- phase t: multiply tile t
            ZERO_ACC();
            // fragments of the first slice (the stage landed before the last barrier)
            fa[0] = frag(stC, aLane, 0, 0);
            fa[1] = frag(stC, aLane, 1, 0);
#pragma unroll
            for (int j = 0; j < WTN; ++j) {
                fb[j] = frag(stC, bLane, j, 0);
            }
            FENCE();
            tileRsrc(t, &ra, &rb);
            tileRsrc(t + 1, &na, &nb);
            v4i ra2 = ra, rb2 = rb; // second product of a grouped sum
            if constexpr (GRP) {
                if (twoProducts) {
                    tileRsrcOf(p.segA[0], p.segB[0], t, &ra2, &rb2);
                }
            }
            for (int s = 0; s < kSlots - 1; ++s) {
                // step s + 2 of this tile, or step s + 2 - kSlots of the next one (of the last tile again when there is none: harmless,
                // and the count of loads in flight stays the same)
                const bool wrap = s + 2 >= kSlots;
                const bool second = GRP && !wrap && s + 2 >= kSlots1;
                const v4i la = wrap ? na : second ? ra2 : ra, lb = wrap ? nb : second ? rb2 : rb;
                const int kOff = (wrap ? s + 2 - kSlots : second ? s + 2 - kSlots1 : s + 2) * PK;
                SLOT(stC, stN, stL, la, lb, kOff, false);
                ROTATE(1);
                if constexpr (GRP) {
                    if (twoProducts && s == kSlots1 - 1) {
                        // the seam: the first product's sums in units of the second's factor (wait states of the last MFMAs spelled out)
                        FENCE();
                        asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
                        FENCE();
#pragma unroll
                        for (int i = 0; i < WTM; ++i) {
#pragma unroll
                            for (int j = 0; j < WTN; ++j) {
#pragma unroll
                                for (int e = 0; e < 16; ++e) {
                                    acc[i][j][e] *= seamRatio;
                                }
                            }
                        }
                        FENCE();
                        asm volatile("s_nop 4" ::: "memory");
                        FENCE();
                    }
                }
            }
            SLOT(stC, stN, stL, na, nb, PK, true); // loads step kSlots + 1 = step 1 of the next tile
            ROTATE(1);
            // ---- phase t + 1: store tile t, under the other group's tile if there is one
            const bool more = t + 1 < myTiles;
            epiloguePhase(t, more ? kSlots : (GRP && CT == C_BF16NORM) ? 1 : 0);
            if (more) {
                ROTATE(kSlots % 3);
            }
        }
        if constexpr (GRP && CT == C_BF16NORM) {
            if (((myTiles - 1) & 1) != group) {
                SLOT_BARRIER(); // the other group's last epilogue exchanges its sums across this barrier
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
#undef ROTATE
#undef SLOT
#undef SLICE
#undef SLOT_BARRIER
#undef SLOT_BARRIER_MUL
#undef ZERO_ACC
#undef MF
#undef FENCE
#undef PING_LOAD1
#undef PING_LOAD
}

template <int TYPE, int CT, int EPI, bool GRP = false> int LaunchPing(const GemmP &p, hipStream_t stream)
{
    PingP q;
    q.g = p;
    q.g.tilesM = p.m / PBM;
    q.g.tilesN = p.n / PBN;
    q.nTiles = q.g.tilesM * q.g.tilesN;
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            return TS2_ERR_LAUNCH;
        }
        cus = n;
    }
    int grid = cus >> (2 * p.gridShrink);
    if (grid < 8) {
        grid = 8;
    }
    if (grid % 8) {
        grid -= grid % 8; // the tile order assumes workgroup ids dealt round-robin to 8 XCDs
    }
    if (grid > q.nTiles) {
        grid = q.nTiles;
    }
    if (!p.mapGroup) {
        const int chunk = (grid % 8) == 0 ? grid / 8 : grid;
        q.g.mapGroup = chunk >= 128 ? 8 : chunk >= 16 ? 4 : 2;
    }
    hipLaunchKernelGGL((GemmNTPing<TYPE, CT, EPI, GRP>), dim3(grid), dim3(512), 0, stream, q);
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

template <int TYPE> int DispatchPing(const GemmP &p, int ct, int epi, hipStream_t stream)
{
    if (ct == C_F32) {
        return epi == TS2_EPI_ADD ? LaunchPing<TYPE, C_F32, TS2_EPI_ADD>(p, stream) : LaunchPing<TYPE, C_F32, TS2_EPI_STORE>(p, stream);
    }
    // Stored 16-bit results leave through the row-owning epilogue of the normalising kernel with its normalisation and rotation off
    // (whole 128-byte row segments as 16-byte stores instead of 4-byte stores of column pairs: e4m3 32768 x 8192 x 2048 453 -> 428 us,
    // the half-precision logits 2800 -> 2655) when the result's rows allow its 16-byte stores; same values.
    if ((ct == C_BF16 || ct == C_F16) && epi == TS2_EPI_STORE && (((uintptr_t)p.c | (uintptr_t)p.ldc) & 15) == 0 &&
        (int64_t)64 * p.ldc < ((int64_t)1 << 31)) {
        GemmP q = p;
        q.normalize = 0;
        q.rope = nullptr;
        q.rowsF16 = ct == C_F16;
        return LaunchPing<TYPE, C_BF16NORM, TS2_EPI_STORE>(q, stream);
    }
    if (ct == C_BF16) {
        return epi == TS2_EPI_ADD ? LaunchPing<TYPE, C_BF16, TS2_EPI_ADD>(p, stream) : LaunchPing<TYPE, C_BF16, TS2_EPI_STORE>(p, stream);
    }
    if (epi != TS2_EPI_STORE) {
        return TS2_ERR_UNSUPPORTED;
    }
    if (ct == C_F16) {
        return LaunchPing<TYPE, C_F16, TS2_EPI_STORE>(p, stream);
    }
    if (ct == C_BF16NORM) {
        return LaunchPing<TYPE, C_BF16NORM, TS2_EPI_STORE>(p, stream);
    }
    if constexpr (TYPE == T_I8) {
        if (ct == C_I32) {
            return LaunchPing<TYPE, C_I32, TS2_EPI_STORE>(p, stream);
        }
    }
    return TS2_ERR_UNSUPPORTED;
}
} // namespace

namespace gemmk
{
bool PingCanRun(const GemmP &p, int type, int ct, int epi)
{
    if (p.m % PBM || p.n % PBN || p.kBytes % PK || p.kBytes < 8 * PK) {
        return false; // (a tile's epilogue is eight pieces, one per slot of the next tile)
    }
    if (p.tileGroup || p.groupOffsets || p.kTileScale || p.kMajor || p.splitK > 1 || p.splits > 1 || p.nSeg > 1) {
        return false;
    }
    if (ct == C_I8PACK || (ct == C_I32 && type != T_I8)) {
        return false;
    }
    if (ct == C_BF16NORM && ((((uintptr_t)p.c | (uintptr_t)p.ldc) & 15) || (int64_t)64 * p.ldc >= ((int64_t)1 << 31))) {
        return false; // the normalised rows leave as 16-byte stores addressed from one 32-bit offset
    }
    if ((int64_t)(PBM - 1) * p.lda + p.kBytes >= ((int64_t)1 << 31) || (int64_t)(PBN - 1) * p.ldb + p.kBytes >= ((int64_t)1 << 31)) {
        return false; // a tile's rows are addressed from one 32-bit offset
    }
    return true;
}

// expert-grouped product C[m][n] = A[m][k] * B_g[n][k] with g = tileGroup[row / 128]: the persistent kernel on the exchanged operands
bool PingGroupedCanRun(const GemmP &p, int type, int ct, int epi)
{
    if (!p.tileGroup || type != T_FP8 || (ct != C_BF16 && ct != C_F16 && ct != C_BF16NORM) || epi != TS2_EPI_STORE || (ct == C_BF16NORM && p.nSeg > 1)) {
        return false;
    }
    if (p.m % PBN || p.n % PBM || p.kBytes % PK || p.kBytes < 4 * PK) {
        return false; // (a tile's epilogue is four pieces, one per slot of the next tile)
    }
    if (p.groupOffsets || p.kTileScale || p.kMajor || p.splitK > 1 || p.splits > 1 || p.nSeg > 2) {
        return false;
    }
    if ((((uintptr_t)p.c | (uintptr_t)p.ldc) & 15) || (int64_t)32 * p.ldc >= ((int64_t)1 << 31)) {
        return false;
    }
    if ((int64_t)(PBM - 1) * p.ldb + p.kBytes >= ((int64_t)1 << 31) || (int64_t)(PBN - 1) * p.lda + p.kBytes >= ((int64_t)1 << 31)) {
        return false;
    }
    return true;
}

int RunPingGrouped(const GemmP &p, int type, int ct, int epi, hipStream_t stream)
{
    if (!PingGroupedCanRun(p, type, ct, epi)) {
        return TS2_ERR_UNSUPPORTED;
    }
    GemmP q = p;
    q.a = p.b;
    q.lda = p.ldb;
    q.b = p.a;
    q.ldb = p.lda;
    q.m = p.n;
    q.n = p.m;
    q.mLive = p.mLive > 0 ? p.mLive : p.m;
    q.segA[0] = p.segB[0];
    q.segB[0] = p.segA[0];
    return ct == C_F16        ? LaunchPing<T_FP8, C_F16, TS2_EPI_STORE, true>(q, stream)
           : ct == C_BF16NORM ? LaunchPing<T_FP8, C_BF16NORM, TS2_EPI_STORE, true>(q, stream)
                              : LaunchPing<T_FP8, C_BF16, TS2_EPI_STORE, true>(q, stream);
}

int RunPing(const GemmP &p, int type, int ct, int epi, hipStream_t stream)
{
    if (!PingCanRun(p, type, ct, epi)) {
        return TS2_ERR_UNSUPPORTED;
    }
    switch (type) {
    case T_I8:
        return DispatchPing<T_I8>(p, ct, epi, stream);
    case T_FP8:
        return DispatchPing<T_FP8>(p, ct, epi, stream);
    default:
        return DispatchPing<T_BF16>(p, ct, epi, stream);
    }
}
} // namespace gemmk
