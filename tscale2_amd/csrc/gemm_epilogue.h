// Parameter block, tile order and the fused epilogues shared by the GEMM kernels (gemm.hip, gemm_twin.hip).
#pragma once
#include "common.h"
#include <type_traits>

#define TS2_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))
#define TS2_GLB_PTR(p) ((const __attribute__((address_space(1))) void *)(p))

namespace gemmk
{
struct GemmP {
    const uint8_t *a;
    const uint8_t *b;
    uint8_t *c;
    int64_t lda, ldb, ldc; // bytes
    int m, n, kBytes;      // kBytes = K * sizeof(element)
    int mLive;
    const float *rowScale;
    const float *kTileScale;
    int kTileBytes;
    float alpha;
    const float *alphaPtr;
    float *tileScale;
    int64_t ldTileScale; // floats
    int splitK;
    int tilesM, tilesN;
    // expert-grouped modes (MoE)
    const int *tileGroup;    // [m/128]: group of each 128-row tile of A/C, -1 = skip; B slab = b + group * bSlab
    int64_t bSlab;           // bytes
    const int *groupOffsets; // [groups+1] contraction row ranges (multiples of 128); blockIdx.y = group
    int64_t cSlab;           // bytes between the C blocks of consecutive groups
    int64_t tileScaleSlab;   // floats
    int splitK_groups;       // number of groups when groupOffsets is set
    int noRing;              // 1: keep the two-stage loop for the 256x256 tile (comparison)
    int kMajor;              // 1: A is [k][m], B is [k][n] (fp8, ring kernel): operands are transposed by the LDS reads
    int streamC;             // results stored with the non-temporal hint
    int ring128;             // 128x128 tile: the ring pipeline (two workgroups per CU) instead of the two-stage loop
    int mapGroup;            // M tiles per group of the tile order (an XCD's share of the tiles should be about square)
    int gridShrink;          // persistent kernel: workgroups = CUs >> (2 * gridShrink) (tests: many tiles per workgroup on small products)
    int splits;              // >1 with splitSlab: blockIdx.y = slice of the contraction, partial product stored to c + y * splitSlab
    int64_t splitSlab;       // bytes
    // row-tile normalise / rope epilogue (C_BF16NORM)
    int normalize;
    float vecScale;
    const float *rope; // [m][128] (cos, sin) pairs, may be null
    int64_t ldRope;    // floats
    // further products added into the same accumulators (ring kernel): product i+1 = segA[i] * segB[i]^T * segAlpha[i] * *segAlphaPtr[i]
    int nSeg; // 1 + number of further products
    const uint8_t *segA[3], *segB[3];
    float segAlpha[3];
    const float *segAlphaPtr[3];
    int rowsF16; // persistent kernel, row-owning epilogue: the 16-bit rows are IEEE half instead of bf16
};

enum { T_I8 = 0, T_FP8 = 1, T_BF16 = 2 };
enum { C_F32 = 0, C_BF16 = 1, C_I32 = 2, C_I8PACK = 3, C_BF16NORM = 4, C_F16 = 5 };

constexpr int BKB = 128; // bytes of K per step

template <int TYPE> struct AccT {
    typedef v16f type;
};
template <> struct AccT<T_I8> {
    typedef v16i type;
};

__device__ __forceinline__ int SwizzleOffset(int row, int chunk)
{
    return row * BKB + ((chunk ^ ((row >> 1) & 7)) << 4);
}

// tile id -> (tileM, tileN): XCD-aware, then grouped along M
__device__ __forceinline__ void MapTile(int bid, int nb, int tilesM, int tilesN, int *tm, int *tn, int GROUP = 8)
{
    int id = bid;
    if ((nb & 7) == 0) {
        id = (bid & 7) * (nb >> 3) + (bid >> 3);
    }
    int perGroup = GROUP * tilesN;
    int g = id / perGroup;
    int first = g * GROUP;
    int gsz = tilesM - first < GROUP ? tilesM - first : GROUP;
    int r = id - g * perGroup;
    *tm = first + r % gsz;
    *tn = r / gsz;
}

// bf16 store of one 32x32 block held as v[e] (lane = column, e -> row): neighbouring lanes swap one value so that even lanes store
// columns (c, c+1) of the even row of a row pair and odd lanes those of the odd row: 4-byte stores instead of 2-byte ones.
// rowOf(e) gives the global row; rows >= mLive are written as zeros.
template <bool F16 = false, class TRow>
__device__ __forceinline__ void StoreBlockBf16(uint8_t *c, int64_t ldc, int col, int l32, int mLive, const float (&v)[16], TRow rowOf)
{
    const bool odd = l32 & 1;
#pragma unroll
    for (int e = 0; e < 16; e += 2) {
        // rows e and e+1 are consecutive rows of the block (e%4 = 0,1 or 2,3)
        float give = odd ? v[e] : v[e + 1];
        float got = LaneXor1(give);
        float lo = odd ? got : v[e];
        float hi = odd ? v[e + 1] : got;
        int row = rowOf(odd ? e + 1 : e);
        uint32_t packed = row < mLive ? (F16 ? PackF16x2(lo, hi) : PackBf16x2(lo, hi)) : 0u;
        *(uint32_t *)(c + (int64_t)row * ldc + (int64_t)(col & ~1) * 2) = packed;
    }
}

// The same store for a block whose 32 rows all lie below mLive, through a buffer descriptor that starts at the wave tile's first row:
// the lane's part of the address (its column pair, and the row it owns inside a group of eight) is one register for the whole
// epilogue and the block's part goes in as the scalar offset, so a store costs no vector arithmetic for its address.  The pair is
// made from the lane's own packed (row e, row e+1) values and the neighbour's by one byte permute instead of three selects.
struct TWaveStore {
    __amdgpu_buffer_rsrc_t rsrc;
    int laneOff;   // bytes: (row owned inside a group of eight) * ldc + column part
    uint32_t sel;  // byte selector of the pair permute (16-bit results)
    int ldc;
};

template <int WTM> __device__ __forceinline__ TWaveStore MakeWaveStore(uint8_t *c, int64_t ldc, int firstRow, int col, int elemBytes, int half, int l32)
{
    TWaveStore w;
    w.rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(c + (int64_t)firstRow * ldc), 0, (int)(32 * WTM * ldc), 0x00020000);
    const bool odd = l32 & 1;
    w.ldc = (int)ldc;
    if (elemBytes == 2) {
        w.laneOff = (half * 4 + (odd ? 1 : 0)) * (int)ldc + (col & ~1) * 2;
    } else {
        w.laneOff = (half * 4) * (int)ldc + col * 4;
    }
    w.sel = odd ? 0x07060302u : 0x01000504u;
    return w;
}

// v[e]: the 16 values of the lane's column in block row `blockRow` of the wave tile, block column offset colBytes
template <bool F16, int AUX> __device__ __forceinline__ void StoreBlock16Buf(const TWaveStore &w, int blockRow, int colBytes, const float (&v)[16])
{
#pragma unroll
    for (int e = 0; e < 16; e += 2) {
        const uint32_t own = F16 ? PackF16x2(v[e], v[e + 1]) : PackBf16x2(v[e], v[e + 1]);
        const uint32_t other = (uint32_t)LaneDpp<DPP_XOR1>((int)own);
        // even lanes: (own row e, neighbour's row e) = columns (c, c+1) of row e; odd lanes: (neighbour's row e+1, own row e+1)
        const uint32_t packed = __builtin_amdgcn_perm(own, other, w.sel);
        const int rowInTile = blockRow * 32 + (e >> 2) * 8 + (e & 2);
        __builtin_amdgcn_raw_buffer_store_b32(packed, w.rsrc, w.laneOff, rowInTile * w.ldc + colBytes, AUX);
    }
}

template <int AUX> __device__ __forceinline__ void StoreBlock32Buf(const TWaveStore &w, int blockRow, int colBytes, const float (&v)[16])
{
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        const int rowInTile = blockRow * 32 + (e >> 2) * 8 + (e & 3);
        __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v[e]), w.rsrc, w.laneOff, rowInTile * w.ldc + colBytes, AUX);
    }
}

template <int TYPE, int WTM, int WTN, int CT, int EPI, bool KT, class TAcc, class TFAcc>
__device__ __forceinline__ void Epilogue(const GemmP &p, TAcc (&acc)[WTM][WTN], TFAcc &facc, uint8_t *lds, int rowBase, int colBase, int wm, int wn,
    int half, int l32)
{
    // ---- epilogue.  MFMA 32x32 result: lane holds column l32, rows (e/4)*8 + half*4 + e%4
    float scale = p.alpha;
    if (p.alphaPtr) {
        scale *= *p.alphaPtr;
    }
    const int mLive = p.mLive > 0 ? p.mLive : p.m;
    auto accVal = [&](int i, int j, int e) -> float {
        if constexpr (KT) {
            return facc[i][j][e];
        } else {
            return (float)acc[i][j][e];
        }
    };
    auto rowLocal = [&](int i, int e) { return wm * (32 * WTM) + i * 32 + (e >> 2) * 8 + half * 4 + (e & 3); };
    // scale of every row of the wave's tile, fetched up front (four consecutive rows per load): one dependent load per row inside
    // the store loops cost the row-scaled product about 10 us per launch
    float rsAll[WTM][16];
#pragma unroll
    for (int i = 0; i < WTM; ++i) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            float4 r = make_float4(1.f, 1.f, 1.f, 1.f);
            if (p.rowScale) {
                r = *(const float4 *)(p.rowScale + rowBase + rowLocal(i, q * 4));
            }
            rsAll[i][q * 4 + 0] = scale * r.x;
            rsAll[i][q * 4 + 1] = scale * r.y;
            rsAll[i][q * 4 + 2] = scale * r.z;
            rsAll[i][q * 4 + 3] = scale * r.w;
        }
    }

    if constexpr (CT == C_BF16NORM) {
        // TStoreRowTileNormalize / TStoreRowTileNormalizeRope (src/lib/cuda/cuda_matmul.cuh:495-525, src/gpt/compute/gpu_rope.cuh:25-60):
        // per row and 128-column tile v = acc*scale; scale_t = rms(v)*vecScale, v /= scale_t; rotate (even, odd) column pairs by the
        // row's (cos, sin) table; bf16.  The wave's 128 columns (WTN == 4) are exactly one tile, so the reduction stays inside the
        // 32-lane group.
        // With the 64-column wave tile (WTN == 2) a tile's columns lie in the two waves along N: they exchange their halves of every
        // row's sum through LDS, which the main loop no longer uses, and add them in the same order.
        static_assert(WTN == 4 || WTN == 2 || CT != C_BF16NORM, "the normalising epilogue needs a wave tile of 64 or 128 columns");
        const int tile = (colBase + wn * (32 * WTN)) / TILE;
        const int colInTile = (wn * (32 * WTN)) & (TILE - 1);
        // all rows of the wave tile live: the stores with scalar addressing
        const int firstRow = rowBase + wm * (32 * WTM);
        const bool wholeTileLive = firstRow + 32 * WTM <= mLive && (int64_t)32 * WTM * p.ldc < ((int64_t)1 << 31);
        const TWaveStore waveStore = MakeWaveStore<WTM>(p.c, p.ldc, firstRow, colBase + wn * (32 * WTN) + l32, 2, half, l32);
        float *xch = (float *)lds;
        // sums of squares of the 16 rows of block row i over the wave's columns
        auto blockRowSum2 = [&](int i, float (&out)[WTN][16], float (&sum2)[16]) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                float rs = rsAll[i][e];
                sum2[e] = 0;
#pragma unroll
                for (int j = 0; j < WTN; ++j) {
                    out[j][e] = accVal(i, j, e) * rs;
                    sum2[e] += out[j][e] * out[j][e];
                }
            }
            if (p.normalize) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    sum2[e] += LaneDpp<DPP_XOR1>(sum2[e]);
                }
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    sum2[e] += LaneDpp<DPP_XOR2>(sum2[e]);
                }
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    sum2[e] += LaneDpp<DPP_HALF_MIRROR>(sum2[e]);
                }
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    sum2[e] += LaneDpp<DPP_MIRROR>(sum2[e]);
                }
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    float a, b;
                    LaneSwap16(sum2[e], &a, &b);
                    sum2[e] = a + b;
                }
            }
        };
        if (WTN == 2 && p.normalize) {
#pragma unroll
            for (int i = 0; i < WTM; ++i) {
                float out[WTN][16];
                float sum2[16];
                blockRowSum2(i, out, sum2);
                if (l32 == 0) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        xch[rowLocal(i, e) * 2 + wn] = sum2[e];
                    }
                }
            }
            __syncthreads();
        }
#pragma unroll
        for (int i = 0; i < WTM; ++i) {
            // phase by phase over the 16 rows of the block row, so that the cross-lane steps and the loads of the rope table of
            // different rows are independent instructions in flight together
            float out[WTN][16];
            float sum2[16];
            blockRowSum2(i, out, sum2);
            if (p.normalize) {
                if (WTN == 2) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int rl = rowLocal(i, e);
                        sum2[e] = xch[rl * 2] + xch[rl * 2 + 1];
                    }
                }
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int row = rowBase + rowLocal(i, e);
                    float discr = 0;
                    if (sum2[e] > 0 && row < mLive) {
                        // hardware square root and reciprocal (1 ulp each): every lane of the group repeats this per row, and the
                        // correctly rounded sequences were most of the epilogue's instructions
                        discr = __builtin_amdgcn_sqrtf(sum2[e] * (1.f / TILE)) * p.vecScale;
                        float inv = __builtin_amdgcn_rcpf(discr);
#pragma unroll
                        for (int j = 0; j < WTN; ++j) {
                            out[j][e] *= inv;
                        }
                    }
                    if (l32 == 0 && (WTN == 4 || wn == 0)) {
                        p.tileScale[(int64_t)tile * p.ldTileScale + row] = discr;
                    }
                }
            }
            if (p.rope) {
#pragma unroll
                for (int eq = 0; eq < 4; ++eq) {
                    float2 cs[4][WTN];
#pragma unroll
                    for (int ee = 0; ee < 4; ++ee) {
                        const int row = rowBase + rowLocal(i, eq * 4 + ee);
#pragma unroll
                        for (int j = 0; j < WTN; ++j) {
                            cs[ee][j] = *(const float2 *)(p.rope + (int64_t)row * p.ldRope + ((colInTile + j * 32 + l32) & ~1));
                        }
                    }
#pragma unroll
                    for (int ee = 0; ee < 4; ++ee) {
                        const int e = eq * 4 + ee;
#pragma unroll
                        for (int j = 0; j < WTN; ++j) {
                            float own = out[j][e];
                            float other = LaneXor1(own);
                            out[j][e] = (l32 & 1) ? other * cs[ee][j].y + own * cs[ee][j].x : own * cs[ee][j].x - other * cs[ee][j].y;
                        }
                    }
                }
            }
            if (wholeTileLive) {
#pragma unroll
                for (int j = 0; j < WTN; ++j) {
                    if (p.streamC) {
                        StoreBlock16Buf<false, 2>(waveStore, i, j * 64, out[j]);
                    } else {
                        StoreBlock16Buf<false, 0>(waveStore, i, j * 64, out[j]);
                    }
                }
            } else {
#pragma unroll
                for (int j = 0; j < WTN; ++j) {
                    StoreBlockBf16(p.c, p.ldc, colBase + wn * (32 * WTN) + j * 32 + l32, l32, mLive, out[j],
                        [&](int e) { return rowBase + rowLocal(i, e); });
                }
            }
        }
    } else if constexpr (CT == C_I8PACK) {
        // TStoreRowTileMaxNormalize (src/lib/cuda/cuda_matmul.cuh:530-559): per row and 128 columns scale = maxabs/127, bytes =
        // sat_i8(rne(v/scale)), TileScale[tile][row] = scale.  A 128-column tile is 4 MFMA blocks: inside one wave when WTN == 4,
        // shared by the two waves along N when WTN == 2 (row maxima exchanged through LDS, which the main loop no longer uses).
        float *xch = (float *)lds;
        // row maxima of a block row, all 16 rows a step at a time (independent cross-lane instructions)
        auto blockRowMax = [&](int i, float (&mx)[16]) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                mx[e] = 0;
#pragma unroll
                for (int j = 0; j < WTN; ++j) {
                    mx[e] = fmaxf(mx[e], fabsf(accVal(i, j, e)));
                }
            }
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                mx[e] = fmaxf(mx[e], LaneDpp<DPP_XOR1>(mx[e]));
            }
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                mx[e] = fmaxf(mx[e], LaneDpp<DPP_XOR2>(mx[e]));
            }
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                mx[e] = fmaxf(mx[e], LaneDpp<DPP_HALF_MIRROR>(mx[e]));
            }
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                mx[e] = fmaxf(mx[e], LaneDpp<DPP_MIRROR>(mx[e]));
            }
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                float a, b;
                LaneSwap16(mx[e], &a, &b);
                mx[e] = fmaxf(a, b);
            }
        };
        if (WTN == 2) {
#pragma unroll
            for (int i = 0; i < WTM; ++i) {
                float mx[16];
                blockRowMax(i, mx);
                if (l32 == 0) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        xch[rowLocal(i, e) * 2 + wn] = mx[e];
                    }
                }
            }
            __syncthreads();
        }
#pragma unroll
        for (int i = 0; i < WTM; ++i) {
            float mxs[16];
            if (WTN == 2) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int rl = rowLocal(i, e);
                    mxs[e] = fmaxf(xch[rl * 2], xch[rl * 2 + 1]);
                }
            } else {
                blockRowMax(i, mxs);
            }
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int rl = rowLocal(i, e);
                const int row = rowBase + rl;
                float rs = rsAll[i][e];
                float mx = mxs[e] * fabsf(rs);
                float discr = 0, mult = 0;
                if (mx > 0 && row < mLive) {
                    discr = mx / 127;
                    mult = 1 / discr;
                }
                float sgnScale = rs;
#pragma unroll
                for (int j = 0; j < WTN; ++j) {
                    int col = colBase + wn * (32 * WTN) + j * 32 + l32;
                    ((int8_t *)p.c)[(int64_t)row * p.ldc + col] = (int8_t)CvtToI8(accVal(i, j, e) * sgnScale * mult);
                }
                if (l32 == 0 && (WTN == 4 || wn == 0)) {
                    int tile = (colBase + wn * (32 * WTN)) / TILE;
                    p.tileScale[(int64_t)tile * p.ldTileScale + row] = discr;
                }
            }
        }
    } else {
        if constexpr (EPI == TS2_EPI_ADD && (CT == C_F32 || CT == C_BF16)) {
            if (p.splitK <= 1) {
                // C += product: the old values of eight rows (two e-quads) across the wave's width are one batch of loads, and the
                // batch after the one being added and stored is already in flight, so the read latency of C is paid once per tile
                constexpr int NCH = WTM * 2;
                float old[2][8][WTN];
                auto rowOf = [&](int ch, int r) { return rowBase + rowLocal(ch >> 1, (ch & 1) * 8 + r); };
                auto fetch = [&](int ch, float (&o)[8][WTN]) {
#pragma unroll
                    for (int r = 0; r < 8; ++r) {
                        const int row = rowOf(ch, r);
                        const uint8_t *src = p.c + (int64_t)row * p.ldc;
#pragma unroll
                        for (int j = 0; j < WTN; ++j) {
                            const int col = colBase + wn * (32 * WTN) + j * 32 + l32;
                            if (CT == C_F32) {
                                o[r][j] = row < mLive ? __builtin_nontemporal_load((const float *)src + col) : 0.f;
                            } else {
                                o[r][j] = row < mLive ? Bf16ToFloat(((const bf16_t *)src)[col]) : 0.f;
                            }
                        }
                    }
                };
                fetch(0, old[0]);
#pragma unroll
                for (int ch = 0; ch < NCH; ++ch) {
                    if (ch + 1 < NCH) {
                        fetch(ch + 1, old[(ch + 1) & 1]);
                    }
#pragma unroll
                    for (int r = 0; r < 8; ++r) {
                        const int row = rowOf(ch, r);
                        if (row < mLive) {
                            uint8_t *dst = p.c + (int64_t)row * p.ldc;
                            const float rs = rsAll[ch >> 1][(ch & 1) * 8 + r];
#pragma unroll
                            for (int j = 0; j < WTN; ++j) {
                                const int col = colBase + wn * (32 * WTN) + j * 32 + l32;
                                float v = old[ch & 1][r][j] + accVal(ch >> 1, j, (ch & 1) * 8 + r) * rs;
                                if constexpr (CT == C_F32) {
                                    __builtin_nontemporal_store(v, (float *)dst + col);
                                } else {
                                    ((bf16_t *)dst)[col] = FloatToBf16(v);
                                }
                            }
                        }
                    }
                }
                return;
            }
        }
        if constexpr ((CT == C_BF16 || CT == C_F16 || CT == C_F32) && EPI == TS2_EPI_STORE) {
            // every row of the wave tile is live, no atomics, rows within the descriptor's reach: the stores with scalar addressing
            const int firstRow = rowBase + wm * (32 * WTM);
            if (p.splitK <= 1 && firstRow + 32 * WTM <= mLive && (int64_t)32 * WTM * p.ldc < ((int64_t)1 << 31)) {
                const TWaveStore w = MakeWaveStore<WTM>(p.c, p.ldc, firstRow, colBase + wn * (32 * WTN) + l32, CT == C_F32 ? 4 : 2, half, l32);
#pragma unroll
                for (int i = 0; i < WTM; ++i) {
#pragma unroll
                    for (int j = 0; j < WTN; ++j) {
                        float v[16];
#pragma unroll
                        for (int e = 0; e < 16; ++e) {
                            v[e] = accVal(i, j, e) * rsAll[i][e];
                        }
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
                    }
                }
                return;
            }
        }
        // four consecutive rows (one e-quad) across the wave's whole width at a time: a row's WTN 128-byte segments are written back
        // to back, and for the accumulate epilogues the 4 x WTN old values are all fetched before the first store
#pragma unroll
        for (int i = 0; i < WTM; ++i) {
            if constexpr ((CT == C_BF16 || CT == C_F16) && EPI == TS2_EPI_STORE) {
#pragma unroll
                for (int j = 0; j < WTN; ++j) {
                    const int col = colBase + wn * (32 * WTN) + j * 32 + l32;
                    float v[16];
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        v[e] = accVal(i, j, e) * rsAll[i][e];
                    }
                    StoreBlockBf16<CT == C_F16>(p.c, p.ldc, col, l32, mLive, v, [&](int e) { return rowBase + rowLocal(i, e); });
                }
            } else {
#pragma unroll
                for (int eq = 0; eq < 4; ++eq) {
                    float old[4][WTN];
                    if (EPI == TS2_EPI_ADD && p.splitK <= 1 && (CT == C_F32 || CT == C_BF16)) {
#pragma unroll
                        for (int ee = 0; ee < 4; ++ee) {
                            const int row = rowBase + rowLocal(i, eq * 4 + ee);
                            const uint8_t *src = p.c + (int64_t)row * p.ldc;
#pragma unroll
                            for (int j = 0; j < WTN; ++j) {
                                const int col = colBase + wn * (32 * WTN) + j * 32 + l32;
                                if (CT == C_F32) {
                                    old[ee][j] = row < mLive ? ((const float *)src)[col] : 0.f;
                                } else {
                                    old[ee][j] = row < mLive ? Bf16ToFloat(((const bf16_t *)src)[col]) : 0.f;
                                }
                            }
                        }
                    }
#pragma unroll
                    for (int ee = 0; ee < 4; ++ee) {
                        const int e = eq * 4 + ee;
                        const int row = rowBase + rowLocal(i, e);
                        const bool live = row < mLive;
                        uint8_t *dst = p.c + (int64_t)row * p.ldc;
                        float rs = rsAll[i][e];
#pragma unroll
                        for (int j = 0; j < WTN; ++j) {
                            const int col = colBase + wn * (32 * WTN) + j * 32 + l32;
                            if constexpr (CT == C_I32) {
                                if constexpr (TYPE == T_I8) {
                                    ((int *)dst)[col] = acc[i][j][e];
                                }
                            } else {
                                float v = live ? accVal(i, j, e) * rs : 0.f;
                                if constexpr (CT == C_F32) {
                                    float *d = (float *)dst + col;
                                    if (EPI == TS2_EPI_ADD) {
                                        if (live) {
                                            *d = old[ee][j] + v;
                                        }
                                    } else {
                                        *d = v;
                                    }
                                } else if constexpr (CT == C_BF16) {
                                    bf16_t *d = (bf16_t *)dst + col;
                                    if (live) {
                                        *d = FloatToBf16(old[ee][j] + v);
                                    }
                                }
                            }
                        }
                    }
                }
            }
        }
    }
}

// One row of a block row held by a lane that owns the row (registers walk along the columns: v[j][e] is column j * 32 + (e / 4) * 8 +
// half * 4 + e % 4 of the wave's WT * 32 columns): scaled, normalised by the rms of the row's 128-column tile (TStoreRowTileNormalize,
// src/lib/cuda/cuda_matmul.cuh:495-525) and rotated by the row's (cos, sin) table (src/gpt/compute/gpu_rope.cuh:25-60).  WT = 2: the
// tile's sum of squares comes in (two waves share a tile).  ropeCol0: first column of the wave inside the 128-wide head.
template <bool NORM, int WT, class TAcc>
__device__ __forceinline__ void NormRowValues(const GemmP &p, TAcc (&accRow)[WT], int row, bool live, float rs, int tile, int ropeCol0, int half,
    bool writeScale, float tileSum2, float (&v)[WT][16])
{
    float sum2 = 0;
#pragma unroll
    for (int j = 0; j < WT; ++j) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            v[j][e] = live ? (float)accRow[j][e] * rs : 0.f;
            sum2 += v[j][e] * v[j][e];
        }
    }
    if (NORM && p.normalize) {
        if constexpr (WT == 2) {
            sum2 = tileSum2;
        } else {
            float a, b;
            LaneSwap32(sum2, &a, &b);
            sum2 = a + b;
        }
        float discr = 0;
        if (sum2 > 0) {
            discr = __builtin_amdgcn_sqrtf(sum2 * (1.f / TILE)) * p.vecScale;
            const float inv = __builtin_amdgcn_rcpf(discr);
#pragma unroll
            for (int j = 0; j < WT; ++j) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    v[j][e] *= inv;
                }
            }
        }
        if (half == 0 && writeScale) {
            p.tileScale[(int64_t)tile * p.ldTileScale + row] = discr;
        }
    }
    if (NORM && p.rope && live) {
        const float *ropeRow = p.rope + (int64_t)row * p.ldRope;
#pragma unroll
        for (int j = 0; j < WT; ++j) {
#pragma unroll
            for (int e = 0; e < 16; e += 2) {
                const float2 cs = *(const float2 *)(ropeRow + ropeCol0 + j * 32 + (e >> 2) * 8 + half * 4 + (e & 3));
                const float x = v[j][e], y = v[j][e + 1];
                v[j][e] = x * cs.x - y * cs.y;
                v[j][e + 1] = y * cs.x + x * cs.y;
            }
        }
    }
}

// The normalising epilogue (TStoreRowTileNormalize / TStoreRowTileNormalizeRope) of the 256x256 ring kernel on accumulators that the
// MFMAs produced transposed (operands swapped: a block holds C^T, so a lane owns one ROW of the block and its registers walk along the
// columns, four consecutive ones per e-quad).  The sum of squares of a row's 128-column tile is then 64 in-lane terms plus one swap
// with the other half wave, one square root and reciprocal per lane and block row, the rotated pairs of RoPE sit in one lane - against
// five cross-lane steps for each of the 16 rows of a block row, and 16 square roots per lane, in the lane = column layout.  The bf16
// rows go through the wave's own 32 KB of LDS (free after the main loop; 8-byte granules XOR-swizzled by the row so that the 32 rows
// of a store hit different banks) and leave as 16-byte stores of whole 256-byte row segments.
// NORM false: the plain 16-bit store (TStoreScaled) through the same staging; F16: IEEE half instead of bf16.
// WT = 2: the same for the 64x64 wave tile of the 128x128 kernels: rows of 128 bytes, 8 KB of the wave's stage array, eight lanes per
// row on the way out.  A 128-column tile spans the two waves of a row there: each leaves its 64-column sums of squares in xchg (LDS,
// 4 x 64 floats outside the staged rows) and adds its neighbour's after one workgroup barrier.
// BLOCKWISE: one block row (32 rows) is staged and stored at a time, so a wave needs 32 x RB bytes of LDS instead of its whole tile.
template <int TYPE, bool NORM, bool F16, int WTM, int WTN, bool BLOCKWISE = false, class TAcc>
__device__ __forceinline__ void NormEpilogueRows(const GemmP &p, TAcc (&acc)[WTM][WTN], uint8_t *waveLds, float *xchg, int rowBase, int colBase,
    int wm, int wn, int lane)
{
    static_assert(WTN == 4 || (WTN == 2 && WTM == 2), "wave tiles of 128 columns (any height) or 64 x 64");
    constexpr int RWM = 32 * WTM, RW = 32 * WTN; // rows and columns of the wave tile
    constexpr int RB = RW * 2;                  // bytes of a staged row
    constexpr int WT = WTN;
    constexpr int SWZ = WT == 4 ? 15 : 7;       // rows that differ in these bits (WT = 2: of r / 2) take different granule pairs
    constexpr int SWS = WT == 4 ? 0 : 1;
    const int half = lane >> 5, l32 = lane & 31;
    float scale = p.alpha;
    if (p.alphaPtr) {
        scale *= *p.alphaPtr;
    }
    const int mLive = p.mLive > 0 ? p.mLive : p.m;
    const int tile = (colBase + wn * RW) / TILE;
    const int firstRow = rowBase + wm * RWM;
    float tileSum2[WTM];
    if constexpr (NORM && WT == 2) {
        if (p.normalize) { // (uniform over the workgroup)
            const int wave = wm * 2 + wn;
#pragma unroll
            for (int i = 0; i < WTM; ++i) {
                const bool live = firstRow + i * 32 + l32 < mLive;
                float rs = scale;
                if (p.rowScale) {
                    rs *= p.rowScale[firstRow + i * 32 + l32];
                }
                float own = 0;
#pragma unroll
                for (int j = 0; j < WT; ++j) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const float x = live ? (float)acc[i][j][e] * rs : 0.f;
                        own += x * x;
                    }
                }
                float a, b;
                LaneSwap32(own, &a, &b);
                tileSum2[i] = a + b;
                if (half == 0) {
                    xchg[wave * 64 + i * 32 + l32] = tileSum2[i];
                }
            }
            __syncthreads();
#pragma unroll
            for (int i = 0; i < WTM; ++i) {
                tileSum2[i] += xchg[(wave ^ 1) * 64 + i * 32 + l32];
            }
        }
    }
    // rows back out: LPR lanes take one row's bytes, 64 / LPR rows per store instruction
    typedef unsigned v4u_t __attribute__((ext_vector_type(4)));
    constexpr int LPR = RB / 16, RPI = 64 / LPR;
    const int t = lane % LPR, rsub = lane / LPR;
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(p.c + (int64_t)firstRow * p.ldc), 0, (int)(RWM * p.ldc), 0x00020000);
    const int ldc = (int)p.ldc;
    const int laneOff = rsub * ldc + (colBase + wn * RW) * 2 + t * 16;
    const bool aligned16 = (((uintptr_t)p.c | (uintptr_t)p.ldc) & 15) == 0;
    // staged rows 0 .. nRows-1 of the LDS area are rows rowOff .. of the wave tile
    auto flushRows = [&](int rowOff, auto nRowsTag) {
        constexpr int nRows = decltype(nRowsTag)::value;
#pragma unroll
        for (int it = 0; it < nRows / RPI; ++it) {
            const int r = it * RPI + rsub;
            const int g = (2 * t) ^ (((r >> SWS) & SWZ) << 1);
            const uint4 d = *(const uint4 *)(waveLds + r * RB + g * 8);
            const int so = (rowOff + it * RPI) * ldc;
            if (!aligned16) {
                // (a result whose rows do not start on 16 bytes: the same data in 4-byte stores)
                __builtin_amdgcn_raw_buffer_store_b32(d.x, rsrc, laneOff, so, 0);
                __builtin_amdgcn_raw_buffer_store_b32(d.y, rsrc, laneOff, so + 4, 0);
                __builtin_amdgcn_raw_buffer_store_b32(d.z, rsrc, laneOff, so + 8, 0);
                __builtin_amdgcn_raw_buffer_store_b32(d.w, rsrc, laneOff, so + 12, 0);
            } else if (p.streamC) {
                __builtin_amdgcn_raw_buffer_store_b128((v4u_t){d.x, d.y, d.z, d.w}, rsrc, laneOff, so, 2);
            } else {
                __builtin_amdgcn_raw_buffer_store_b128((v4u_t){d.x, d.y, d.z, d.w}, rsrc, laneOff, so, 0);
            }
        }
    };
#pragma unroll
    for (int i = 0; i < WTM; ++i) {
        const int r = i * 32 + l32; // row inside the wave tile
        const int rl = BLOCKWISE ? l32 : r; // its staged row
        const int row = firstRow + r;
        const bool live = row < mLive;
        float rs = scale;
        if (p.rowScale) {
            rs *= p.rowScale[row];
        }
        float v[WT][16];
        NormRowValues<NORM, WT>(p, acc[i], row, live, rs, tile, WT == 2 ? wn * RW : 0, half, WT == 4 || wn == 0, WT == 2 ? tileSum2[i] : 0.f, v);
#pragma unroll
        for (int j = 0; j < WT; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int g = (j * 8 + q * 2 + half) ^ (((rl >> SWS) & SWZ) << 1); // 8-byte granule of the row, swizzled
                *(uint2 *)(waveLds + rl * RB + g * 8) = F16 ? make_uint2(PackF16x2(v[j][4 * q], v[j][4 * q + 1]), PackF16x2(v[j][4 * q + 2], v[j][4 * q + 3]))
                                                           : make_uint2(PackBf16x2(v[j][4 * q], v[j][4 * q + 1]), PackBf16x2(v[j][4 * q + 2], v[j][4 * q + 3]));
            }
        }
        if constexpr (BLOCKWISE) {
            flushRows(i * 32, std::integral_constant<int, 32>());
        }
    }
    if constexpr (!BLOCKWISE) {
        flushRows(0, std::integral_constant<int, RWM>());
    }
}

// The packed-delta epilogue (TStoreRowTileMaxNormalize, src/lib/cuda/cuda_matmul.cuh:530-559) of the 256x256 ring kernel in the same
// row-owning form: the largest magnitude of a row's 128-column tile is 64 in-lane terms and one swap with the other half wave, four
// consecutive columns are one 32-bit word of bytes, the 128-byte rows are staged in the wave's own LDS (words XOR-swizzled in groups
// of four by the row) and leave as 16-byte stores, eight lanes per row; a tile's scales are 32 consecutive floats per store.  Same
// arithmetic, element for element, as the lane = column form (maximum of |acc| times |scale|, /127, reciprocal, (acc * scale) * mult).
template <class TAcc>
__device__ __forceinline__ void PackEpilogueRows(const GemmP &p, TAcc (&acc)[4][4], uint8_t *waveLds, int rowBase, int colBase, int wm, int wn, int lane)
{
    const int half = lane >> 5, l32 = lane & 31;
    float scale = p.alpha;
    if (p.alphaPtr) {
        scale *= *p.alphaPtr;
    }
    const int mLive = p.mLive > 0 ? p.mLive : p.m;
    const int tile = (colBase + wn * 128) / TILE;
    const int firstRow = rowBase + wm * 128;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = i * 32 + l32; // row inside the wave tile
        const int row = firstRow + r;
        float rs = scale;
        if (p.rowScale) {
            rs *= p.rowScale[row];
        }
        float mx = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                mx = fmaxf(mx, fabsf((float)acc[i][j][e]));
            }
        }
        float a, b;
        LaneSwap32(mx, &a, &b);
        mx = fmaxf(a, b) * fabsf(rs);
        float discr = 0, mult = 0;
        if (mx > 0 && row < mLive) {
            discr = mx / 127;
            mult = 1 / discr;
        }
        if (half == 0) {
            p.tileScale[(int64_t)tile * p.ldTileScale + row] = discr;
        }
        const int swz = ((r >> 1) & 7) << 2;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                uint32_t w = 0;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    w |= (uint32_t)(CvtToI8((float)acc[i][j][4 * q + c] * rs * mult) & 0xff) << (8 * c);
                }
                *(uint32_t *)(waveLds + r * 128 + (((j * 8 + q * 2 + half) ^ swz) << 2)) = w;
            }
        }
    }
    typedef unsigned v4u_t __attribute__((ext_vector_type(4)));
    const int t = lane & 7, rsub = lane >> 3;
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(p.c + (int64_t)firstRow * p.ldc), 0, (int)(128 * p.ldc), 0x00020000);
    const int ldc = (int)p.ldc;
    const int laneOff = rsub * ldc + colBase + wn * 128 + t * 16;
    const int alignBits = (int)(((uintptr_t)p.c | (uintptr_t)p.ldc) & 15);
#pragma unroll
    for (int it = 0; it < 16; ++it) {
        const int r = it * 8 + rsub;
        const uint4 d = *(const uint4 *)(waveLds + r * 128 + (((4 * t) ^ (((r >> 1) & 7) << 2)) << 2));
        if (alignBits == 0) {
            if (p.streamC) {
                __builtin_amdgcn_raw_buffer_store_b128((v4u_t){d.x, d.y, d.z, d.w}, rsrc, laneOff, it * 8 * ldc, 2);
            } else {
                __builtin_amdgcn_raw_buffer_store_b128((v4u_t){d.x, d.y, d.z, d.w}, rsrc, laneOff, it * 8 * ldc, 0);
            }
        } else if ((alignBits & 3) == 0) {
            __builtin_amdgcn_raw_buffer_store_b32(d.x, rsrc, laneOff, it * 8 * ldc, 0);
            __builtin_amdgcn_raw_buffer_store_b32(d.y, rsrc, laneOff, it * 8 * ldc + 4, 0);
            __builtin_amdgcn_raw_buffer_store_b32(d.z, rsrc, laneOff, it * 8 * ldc + 8, 0);
            __builtin_amdgcn_raw_buffer_store_b32(d.w, rsrc, laneOff, it * 8 * ldc + 12, 0);
        } else {
            // (rows that start off the 4-byte grid: byte stores)
            const uint32_t w[4] = {d.x, d.y, d.z, d.w};
            uint8_t *dst = p.c + (int64_t)(firstRow + r) * p.ldc + colBase + wn * 128 + t * 16;
#pragma unroll
            for (int c = 0; c < 16; ++c) {
                dst[c] = (uint8_t)(w[c >> 2] >> (8 * (c & 3)));
            }
        }
    }
}

// The 256x128 kernel for two workgroups per CU (gemm_twin.hip): type T_*, ct C_*, epi TS2_EPI_STORE / TS2_EPI_ADD
bool TwinCanRun(const GemmP &p, int type, int ct, int epi);
int RunTwin(const GemmP &p, int type, int ct, int epi, hipStream_t stream);
// The persistent eight-wave kernel whose epilogue runs under the next tile's main loop (gemm_ping.hip)
bool PingCanRun(const GemmP &p, int type, int ct, int epi);
int RunPing(const GemmP &p, int type, int ct, int epi, hipStream_t stream);
bool PingGroupedCanRun(const GemmP &p, int type, int ct, int epi);
int RunPingGrouped(const GemmP &p, int type, int ct, int epi, hipStream_t stream);
} // namespace gemmk
