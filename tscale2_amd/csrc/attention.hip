// Base-2 "sink" attention of the reference (forward, dQ, dK/dV) on gfx950 bf16 MFMA, head dimension 128.
//
// Math (src/gpt/compute/layer_att_reference.h:47-211): for query row q and every key row t of its span [start[q], finish[q]]
//   dp = <q,k_t> * attDotScale - slope * (q - t);  m = max(0, max dp);  S = 2^-m + sum_t 2^(dp-m)   (a zero vector of weight 1)
//   out = sum_t w_t v_t,  w_t = 2^(dp-m)/S;  stats L = m + log2 S  (SumWeightLog of src/gpt/compute/gpu_att_fp16.cu:192-205)
//   dDot = w_t (<dO_q, v_t> - dScale_q) attDotScale ln2;  dq += dDot k_t;  dk_t += dDot q;  dv_t += w_t dO_q
//
// Design for CDNA4 (replaces Fp16Att / Fp16AttGradQ / Fp16AttGradKV, src/gpt/compute/gpu_att_fp16.cuh:60-358, whose 16-key
// mma.sync tiling does not map to MFMA):
//   * a wave owns 32 rows (queries in the forward and dQ kernels, keys in the dK/dV kernel); the other side streams through LDS in
//     64-row tiles and is consumed 32 rows at a time.  Every product is a v_mfma_f32_32x32x16_bf16 whose N index (the lane) is the
//     wave's own row, so all softmax statistics are per lane and the running rescale of the accumulators needs no cross-lane traffic:
//         S^T = K Q^T,  O^T += V^T P^T,  dP^T = V dO^T,  dQ^T += K^T dS^T      (lane = query)
//         S = Q K^T,  dP = dO V^T,  dV^T += dO^T P,  dK^T += Q^T dS             (lane = key)
//     The probability / score-gradient blocks never leave registers: an MFMA result block, rounded to bf16, is the B operand of the
//     next product (the contraction index order of an MFMA is free as long as A and B agree).
//   * the streamed tiles go global -> LDS with buffer_load_dwordx4 ... lds into two buffers used in turn: no staging registers, no
//     ds_write, one barrier per tile.  Rows are unpadded; the 16-byte chunks of a row are XOR-swizzled by
//     Swz(row) = 4 * (row % 4) + (row / 4) % 4, which makes both kinds of operand fetch bank-conflict free:
//       - row-major fragments (contraction over d): ds_read_b128, 16 consecutive rows at one chunk column -> 16 different chunks;
//       - transposed fragments (contraction over the tile's rows): ds_read_b64_tr_b16 straight from the row-major tile.  Inside each
//         group of 16 lanes the instruction hands lane j, element e the 16-bit value number j % 4 of the 8 bytes addressed by lane
//         4 * e + j / 4; with lane i pointing at row i / 4, columns 4 * (i % 4) .. + 3 of a 4 x 16 block, lane j receives column j
//         of rows 0..3: four contraction slots of an MFMA A operand.  A half wave touches 4 rows x 64 bytes, which the swizzle
//         spreads over all 64 banks.
//   * the wave's own rows (the B operands of the products that contract over d) stay in registers for the whole kernel, so every
//     MFMA costs one 1 KB operand fetch from LDS.  With that every kernel fits 256 registers and 64-70 KB of LDS: two workgroups share
//     a CU (the exponentials and conversions of one run between the products of the other), where one wave per SIMD waits out every
//     LDS and MFMA latency itself.  The dK/dV kernel gets there by giving dK and dV to different waves, which hand P over in LDS.
//   * the register budget shapes the control flow: blocks of 32 rows that a wave does not see are skipped by loops of no trips, not
//     by branches (the join after a branch makes the compiler copy the 64 accumulator registers); the two tile buffers are two
//     copies of the code in one loop body (an operand fetch names its LDS array, so it never waits for the loads in flight into the
//     other array); values needed once per tile (lane offsets of the loads, the statistics pass) are recomputed from a lane index
//     obtained on the spot instead of living across the loop.
//   * workgroup ids are remapped so that an XCD works on consecutive blocks of one head, whose streamed rows overlap in its L2.
//   * spans are one inclusive key range per query (every causal window / document-start pattern of
//     src/gpt/att/sliding_window.cpp:111-118,226-240); masking is one unsigned compare per element, blocks outside a wave's range are
//     skipped, tiles outside the workgroup's range are never loaded; kernels are specialised on whether there is a slope.
#include "common.h"
#include <type_traits>

namespace
{
constexpr int HD = 128;          // Q_DIM = TT_DIM (src/gpt/compute/cfg_precision.h:79-80)
constexpr int WROWS = 32;        // rows owned by one wave
constexpr int BROWS = 128;       // rows owned by one workgroup of the forward and dQ kernels, and of a reverse range
constexpr int KVROWS = 64;       // key rows owned by one workgroup of the dK/dV kernel
constexpr int TR = 64;           // rows of a streamed tile
constexpr int ROWB = HD * 2;     // bytes of a tile row
constexpr int TILE_BYTES = TR * ROWB;
constexpr float LN2 = 0.693147f; // LOG2 of src/gpt/model_params/model_dim.h:16
#define TS2_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))
#define TS2_GLB_PTR(p) ((const __attribute__((address_space(1))) void *)(p))

struct AttP {
    const uint8_t *q, *k, *v, *dO; // bf16 [lenRound][heads*128]
    int64_t ldq, ldk, ldv, lddo;
    const int *spanStart, *spanFinish;
    const int *revLo, *revHi; // per 128-key block: range of query rows that reach it
    float attDotScale, slope;
    float *sumWeightLog; // [heads][ldStat]
    const float *dScale;
    int64_t ldStat;
    uint8_t *out0, *out1; // forward: valLookup; dQ kernel: dQ; dK/dV kernel: dK, dV
    int64_t ldo0, ldo1;
    int lenRound;
    // score gradients handed from the dK/dV kernel to the dQ kernel (optional): per query row the number of its 32-query block's first
    // block of dS (dsBase[lenRound] = blocks per head), the blocks themselves (2 KB each), and how many of them the array holds
    const int *dsBase;
    uint8_t *ds;
    int64_t dsCap;
};

constexpr int DS_BLOCK_BYTES = 32 * 32 * 2; // a 32 x 32 block of dS in bf16

// result registers 8*s .. 8*s+7 of a 32x32 block -> bf16 B operand whose slots match FragTr's row order
__device__ __forceinline__ v8bf PackB(const float *x, int s)
{
    v4i r;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        r[w] = (int)PackBf16x2(x[8 * s + 2 * w], x[8 * s + 2 * w + 1]);
    }
    return __builtin_bit_cast(v8bf, r);
}

// row index inside a 32x32 MFMA result block held in register e by a lane of the given half
__device__ __forceinline__ int BlkRow(int e, int half)
{
    return (e >> 2) * 8 + half * 4 + (e & 3);
}

template <bool F32> __device__ __forceinline__ void Store4Out(uint8_t *p, float a, float b, float c, float d)
{
    if (F32) {
        *(float4 *)p = make_float4(a, b, c, d);
    } else {
        *(uint2 *)p = make_uint2(PackBf16x2(a, b), PackBf16x2(c, d));
    }
}

// accumulators acc[db][e] hold X^T[d][own row]; write X[row][d]
template <bool F32> __device__ __forceinline__ void StoreOwnRows(uint8_t *out, int64_t ld, int col0, v16f *acc, float mult, int l32, int half)
{
    constexpr int ES = F32 ? 4 : 2;
#pragma unroll
    for (int db = 0; db < 4; ++db) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            int d = db * 32 + g * 8 + half * 4;
            Store4Out<F32>(out + (int64_t)l32 * ld + (int64_t)(col0 + d) * ES, acc[db][4 * g] * mult, acc[db][4 * g + 1] * mult,
                acc[db][4 * g + 2] * mult, acc[db][4 * g + 3] * mult);
        }
    }
}

// key range of the workgroup's query rows: min start / max finish over rows with a non-empty span
__device__ __forceinline__ void BlockKeyRange(int start, int finish, int tid, int *lo, int *hi, int *red)
{
    int s = finish >= start ? start : 0x7fffffff;
    int f = finish >= start ? finish : -1;
    s = WaveMinInt(s);
    f = WaveMaxInt(f);
    if ((tid & 63) == 0) {
        red[(tid >> 6) * 2] = s;
        red[(tid >> 6) * 2 + 1] = f;
    }
    __syncthreads();
    *lo = min(min(red[0], red[2]), min(red[4], red[6]));
    *hi = max(max(red[1], red[3]), max(red[5], red[7]));
}

// span of the lane's own row in a form that needs one unsigned compare per key, plus the wave-wide bounds that tell whether a tile
// is seen completely, partly or not at all by the 32 rows of the wave
struct TRowSpan {
    int start;     // 0x7fffffff for an empty span
    unsigned len;  // finish - start (0 for an empty span, whose start makes every compare fail)
    int waveMaxStart, waveMinFinish, waveMinStart, waveMaxFinish;
};

__device__ __forceinline__ TRowSpan MakeRowSpan(int start, int finish)
{
    TRowSpan r;
    bool some = finish >= start;
    r.start = some ? start : 0x7fffffff;
    r.len = some ? (unsigned)(finish - start) : 0u;
    int a = r.start, b = some ? finish : -1, c = r.start, d = b;
    a = WaveMaxInt(a);
    b = WaveMinInt(b);
    c = WaveMinInt(c);
    d = WaveMaxInt(d);
    // the same in every lane: held as scalars, so that the tests on them are uniform branches
    r.waveMaxStart = __builtin_amdgcn_readfirstlane(a);
    r.waveMinFinish = __builtin_amdgcn_readfirstlane(b);
    r.waveMinStart = __builtin_amdgcn_readfirstlane(c);
    r.waveMaxFinish = __builtin_amdgcn_readfirstlane(d);
    return r;
}

// reverse ranges: for every 128-key block the first and last query row whose span touches it
__global__ void RevInit(int *revLo, int *revHi, int n)
{
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        revLo[i] = 0x7fffffff;
        revHi[i] = -1;
    }
}

// a wave takes 64 consecutive queries and issues one atomic pair per key block that any of them reaches (the queries of a wave reach
// much the same blocks: one atomic per query and block made the few hundred block entries the bottleneck)
__global__ void RevBuild(const int *spanStart, const int *spanFinish, int len, int *revLo, int *revHi)
{
    const int q = blockIdx.x * blockDim.x + threadIdx.x;
    int s = 0, f = -1;
    if (q < len) {
        s = spanStart[q];
        f = spanFinish[q];
    }
    const bool some = f >= s;
    const int bLo = some ? s / BROWS : 0x7fffffff, bHi = some ? f / BROWS : -1;
    const int wLo = __builtin_amdgcn_readfirstlane(WaveMinInt(bLo)), wHi = __builtin_amdgcn_readfirstlane(WaveMaxInt(bHi));
    for (int b = wLo; b <= wHi; ++b) {
        const bool touch = some && b >= bLo && b <= bHi;
        const int qMin = WaveMinInt(touch ? q : 0x7fffffff), qMax = WaveMaxInt(touch ? q : -1);
        if ((threadIdx.x & 63) == 0 && qMax >= 0) {
            atomicMin(&revLo[b], qMin);
            atomicMax(&revHi[b], qMax);
        }
    }
}

typedef short v4s16 __attribute__((ext_vector_type(4)));

// chunk swizzle of a tile row (16 chunks of 16 bytes): a bijection of row % 16 whose upper two bits are row % 4
__device__ __forceinline__ int Swz(int row)
{
    return ((row & 3) << 2) | ((row >> 2) & 3);
}

// the lane index, computed where it is asked for (the volatile asm keeps the computation, and everything derived from it, from
// being moved out of a loop and held in registers across it)
__device__ __forceinline__ int FreshLaneId()
{
    int lane;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane));
    return lane;
}

// Direct tile load: a wave-level load fills 4 consecutive tile rows (1 KB); wave w issues the loads of row groups w, w + 4, w + 8,
// w + 12, whose Swz depends on the lane and on w only.  Buffer addressing: the tile's first row is the base of a descriptor held
// in scalar registers, a lane adds one 32-bit offset and the row group a scalar one, so a load costs no 64-bit vector arithmetic and
// no address registers outlive it (the lane index is obtained on the spot for the same reason).  Reads past the 64 rows of the
// descriptor would return zeros instead of touching memory.
__device__ __forceinline__ void LoadTileDirect(uint8_t *tile, const uint8_t *g, int64_t ld, int wave)
{
    const int lane = FreshLaneId();
    const int lrow = lane >> 4;
    const int chunk = (lane & 15) ^ ((lrow << 2) | wave);
    const int laneOff = lrow * (int)ld + chunk * 16;
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)g, 0, TR * (int)ld, 0x00020000);
#pragma unroll
    for (int i = 0; i < TR / 16; ++i) {
        const int u = wave + 4 * i;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, TS2_LDS_PTR(tile + u * 1024), 16, laneOff, 4 * u * (int)ld, 0, 0);
    }
}

// Operand fetches take (tile, compile-time offset) + a per-lane byte offset that is computed once per kernel and made opaque to the
// optimiser: the tile address and the constant part then fold into the instruction's offset field, and a kernel keeps ten address
// registers for all of its fetches instead of one per (buffer, block, step).
typedef const __attribute__((address_space(3))) uint8_t *TLdsBytes;

struct TFragLane {
    int row[4];   // FragRow, ds = 0..3: l32 * ROWB + (((2 * ds) ^ Swz(l32) ^ half) << 4)
    int rowHi;    // ds = 4..7 flips bit 3 of the chunk: row[ds - 4] + rowHi, rowHi = +-128
    int trLo[4];  // FragTr, slots 0..3 of column block db
    int trHi;     // slots 4..7 (8 rows further down, chunk ^ 2): trLo[db] + trHi
};

__device__ __forceinline__ TFragLane MakeFragLane(int lane)
{
    const int l32 = lane & 31, half = lane >> 5;
    const int swzLane = Swz(l32) ^ half;
    TFragLane f;
#pragma unroll
    for (int ds = 0; ds < 4; ++ds) {
        f.row[ds] = l32 * ROWB + (((2 * ds) ^ swzLane) << 4);
        asm volatile("" : "+v"(f.row[ds]));
    }
    f.rowHi = (swzLane & 8) ? -128 : 128;
    asm volatile("" : "+v"(f.rowHi));
    // transposed fetch: inside a group of 16 lanes, lane i points at row i / 4, columns 4 * (i % 4) .. + 3 of the group's 4 x 16 block;
    // the two groups of a half wave sit side by side (32 columns), the halves of the wave 4 rows apart
    const int g = lane >> 4, i = lane & 15, h = g >> 1, dsub = g & 1, r = i >> 2, c4 = i & 3;
    const int base = (4 * h + r) * ROWB + 8 * (c4 & 1);
    const int cl = (2 * dsub + (c4 >> 1)) ^ h;
#pragma unroll
    for (int db = 0; db < 4; ++db) {
        const int blk = (db ^ r) << 2;
        f.trLo[db] = base + ((blk | cl) << 4);
        asm volatile("" : "+v"(f.trLo[db]));
    }
    f.trHi = 8 * ROWB + (((cl ^ 2) - cl) << 4);
    asm volatile("" : "+v"(f.trHi));
    return f;
}

// A operand, contraction over d: lane row = rb * 32 + l32, d = ds * 16 + half * 8 .. + 7
__device__ __forceinline__ v8bf FragRow(const uint8_t *tile, int rb, int ds, const TFragLane &f)
{
    TLdsBytes b = (TLdsBytes)TS2_LDS_PTR(tile) + rb * 32 * ROWB;
    const int off = ds < 4 ? f.row[ds] : f.row[ds - 4] + f.rowHi;
    return __builtin_bit_cast(v8bf, *(const __attribute__((address_space(3))) v4i *)(b + off));
}

// A operand, contraction over tile rows: lane row = d = db * 32 + l32; slots = tile rows rb * 32 + 16 * ks + 4 * half + {0..3} and + 8
__device__ __forceinline__ v8bf FragTr(const uint8_t *tile, int rb, int ks, int db, const TFragLane &f)
{
    typedef __attribute__((address_space(3))) v4s16 *TTrPtr;
    TLdsBytes b = (TLdsBytes)TS2_LDS_PTR(tile) + (rb * 32 + 16 * ks) * ROWB;
    v4s16 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TTrPtr)(b + f.trLo[db]));
    v4s16 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TTrPtr)(b + (f.trLo[db] + f.trHi)));
    typedef short v8s16 __attribute__((ext_vector_type(8)));
    v8s16 r = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(v8bf, r);
}

// the wave's own rows as B operands: lane row = l32, d = ds * 16 + half * 8 .. + 7
__device__ __forceinline__ void LoadOwnFrags(v8bf (&f)[8], const uint8_t *g, int64_t ld, int l32, int half)
{
#pragma unroll
    for (int ds = 0; ds < 8; ++ds) {
        f[ds] = __builtin_bit_cast(v8bf, *(const v4i *)(g + (int64_t)l32 * ld + (ds * 16 + half * 8) * 2));
    }
}

// workgroup ids are handed to the 8 XCDs in turn: remap them so that an XCD works on consecutive blocks of one head (the rows they
// stream overlap, and so stay in that XCD's L2)
__device__ __forceinline__ void MapAttBlock(int *blk, int *head)
{
    const int nbx = gridDim.x, nb = nbx * gridDim.y, bid = blockIdx.x + blockIdx.y * nbx;
    const int id = (nb & 7) == 0 ? (bid & 7) * (nb >> 3) + (bid >> 3) : bid;
    *head = id / nbx;
    *blk = id - *head * nbx;
}

// forward: grid (lenRound/128, heads); a wave owns 32 query rows
template <bool ALIBI> __global__ void __launch_bounds__(256, 2) AttForward(AttP p)
{
    __shared__ __attribute__((aligned(1024))) uint8_t kT0[TILE_BYTES], kT1[TILE_BYTES], vT0[TILE_BYTES], vT1[TILE_BYTES];
    __shared__ int red[8];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), l32 = lane & 31, half = lane >> 5;
    int blk, head;
    MapAttBlock(&blk, &head);
    // later query blocks of a causal sequence see more keys: they start first so that the short ones fill the tail of the launch
    const int myRow = (gridDim.x - 1 - blk) * BROWS + wave * WROWS + l32;
    const int64_t hoff = (int64_t)head * HD * 2;
    const int start = p.spanStart[myRow], finish = p.spanFinish[myRow];
    int kLo, kHi;
    BlockKeyRange(start, finish, tid, &kLo, &kHi, red);
    kLo = __builtin_amdgcn_readfirstlane(kLo);
    kHi = __builtin_amdgcn_readfirstlane(kHi);
    const int tFirst = kHi >= kLo ? (kLo / TR) * TR : 1;
    const uint8_t *gk = p.k + hoff, *gv = p.v + hoff;
    if (tFirst <= kHi) {
        LoadTileDirect(kT0, gk + (int64_t)tFirst * p.ldk, p.ldk, wave);
        LoadTileDirect(vT0, gv + (int64_t)tFirst * p.ldv, p.ldv, wave);
    }
    v8bf qf[8];
    LoadOwnFrags(qf, p.q + (int64_t)(myRow - l32) * p.ldq + hoff, p.ldq, l32, half);
    const TRowSpan sp = MakeRowSpan(start, finish);
    const TFragLane fl = MakeFragLane(lane);
    float zero = 0; // opaque, as in AttGradQ
    asm volatile("" : "+v"(zero));
    v16f oacc[4];
#pragma unroll
    for (int db = 0; db < 4; ++db) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            oacc[db][e] = zero;
        }
    }
    float m = 0, sum = 1; // the sink: a zero vector with weight 2^-m
    auto tile = [&](const uint8_t *kt, const uint8_t *vt, int t0) __attribute__((always_inline)) {
#pragma unroll
        for (int kb = 0; kb < TR / 32; ++kb) {
            const int k0 = t0 + kb * 32;
            const uint8_t *kt2 = kt + kb * 32 * ROWB, *vt2 = vt + kb * 32 * ROWB;
            int trips = __builtin_amdgcn_readfirstlane((int)!(k0 > sp.waveMaxFinish || k0 + 31 < sp.waveMinStart)); // (see AttGradQ)
            asm volatile("" : "+s"(trips));
#pragma unroll 1
            for (int trip = 0; trip < trips; ++trip) {
                v16f s;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    s[e] = 0;
                }
                // phase 1: S^T = K Q^T, operands three steps ahead (one product per step)
                v8bf fk[4];
#pragma unroll
                for (int ds = 0; ds < 3; ++ds) {
                    fk[ds] = FragRow(kt2, 0, ds, fl);
                }
#pragma unroll
                for (int ds = 0; ds < 8; ++ds) {
                    if (ds + 3 < 8) {
                        fk[(ds + 3) & 3] = FragRow(kt2, 0, ds + 3, fl);
                    }
                    s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fk[ds & 3], qf[ds], s, 0, 0, 0);
                }
                // the first operands of phase 3 are requested before the arithmetic of phase 2, which covers their latency
                v8bf ft[3];
                ft[0] = FragTr(vt2, 0, 0, 0, fl);
                ft[1] = FragTr(vt2, 0, 0, 1, fl);
                __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
#pragma unroll
                for (int ds = 0; ds < 5; ++ds) {
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                }
                __builtin_amdgcn_sched_group_barrier(0x008, 3, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
                // phase 2: running maximum and weights of the block's 32 keys.  logit = s * scale - slope * (row - key)
                float sv[16];
                float mx = m;
                const float kc = ALIBI ? p.slope * (float)(k0 + half * 4 - myRow) : 0.f;
                const bool full = k0 >= sp.waveMaxStart && k0 + 31 <= sp.waveMinFinish;
                if (full) { // every row of the wave sees every key of the block: no span tests
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        sv[e] = ALIBI ? fmaf(s[e], p.attDotScale, fmaf(p.slope, (float)BlkRow(e, 0), kc)) : s[e] * p.attDotScale;
                        mx = fmaxf(mx, sv[e]);
                    }
                } else {
                    const int rel0 = k0 + half * 4 - sp.start;
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const float x = ALIBI ? fmaf(s[e], p.attDotScale, fmaf(p.slope, (float)BlkRow(e, 0), kc)) : s[e] * p.attDotScale;
                        sv[e] = (unsigned)(rel0 + BlkRow(e, 0)) <= sp.len ? x : -INFINITY;
                        mx = fmaxf(mx, sv[e]);
                    }
                }
                {
                    float lo, hi;
                    LaneSwap32(mx, &lo, &hi);
                    mx = fmaxf(lo, hi);
                }
                const float alpha = __builtin_amdgcn_exp2f(m - mx);
                int rescale = __builtin_amdgcn_readfirstlane((int)(__any(mx != m) != 0));
                asm volatile("" : "+s"(rescale));
                m = mx;
                float ps = 0;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    sv[e] = __builtin_amdgcn_exp2f(sv[e] - m); // exp2(-inf) = 0 for masked keys
                    ps += sv[e];
                }
                {
                    float lo, hi;
                    LaneSwap32(ps, &lo, &hi);
                    ps = lo + hi;
                }
                sum = sum * alpha + ps;
                // the maximum of no row moved in most blocks; the rescaling is a loop of no trips then (not a branch, see AttGradQ)
#pragma unroll 1
                for (int r = 0; r < rescale; ++r) {
#pragma unroll
                    for (int db = 0; db < 4; ++db) {
#pragma unroll
                        for (int e = 0; e < 16; ++e) {
                            oacc[db][e] *= alpha;
                        }
                    }
                }
                const v8bf pb[2] = {PackB(sv, 0), PackB(sv, 1)};
                // phase 3: O^T += V^T P^T, operands two products ahead
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    if (i + 2 < 8) {
                        ft[(i + 2) % 3] = FragTr(vt2, 0, (i + 2) >> 2, (i + 2) & 3, fl);
                    }
                    oacc[i & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ft[i % 3], pb[i >> 2], oacc[i & 3], 0, 0, 0);
                }
#pragma unroll
                for (int i = 0; i < 6; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                }
                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            }
        }
    };
    // two tiles per trip, one per buffer, in straight-line code (see AttGradQ)
    for (int t0 = tFirst; t0 <= kHi;) {
        __builtin_amdgcn_s_waitcnt(0x0f70); // vmcnt(0): the tile of this step has landed
        __syncthreads();                    // ... for every wave, and every wave is done with the other buffer
        if (t0 + TR <= kHi) {
            LoadTileDirect(kT1, gk + (int64_t)(t0 + TR) * p.ldk, p.ldk, wave);
            LoadTileDirect(vT1, gv + (int64_t)(t0 + TR) * p.ldv, p.ldv, wave);
        }
        tile(kT0, vT0, t0);
        t0 += TR;
        if (t0 > kHi) {
            break;
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
        if (t0 + TR <= kHi) {
            LoadTileDirect(kT0, gk + (int64_t)(t0 + TR) * p.ldk, p.ldk, wave);
            LoadTileDirect(vT0, gv + (int64_t)(t0 + TR) * p.ldv, p.ldv, wave);
        }
        tile(kT1, vT1, t0);
        t0 += TR;
    }
    StoreOwnRows<false>(p.out0 + (int64_t)(myRow - l32) * p.ldo0, p.ldo0, head * HD, oacc, 1 / sum, l32, half);
    if (half == 0) {
        p.sumWeightLog[(int64_t)head * p.ldStat + myRow] = m + log2f(sum);
    }
}

// dQ: grid (lenRound/128, heads); a wave owns 32 query rows
template <bool F32, bool ALIBI> __global__ void __launch_bounds__(256, 2) AttGradQ(AttP p)
{
    __shared__ __attribute__((aligned(1024))) uint8_t kT0[TILE_BYTES], kT1[TILE_BYTES], vT0[TILE_BYTES], vT1[TILE_BYTES];
    __shared__ int red[8];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), l32 = lane & 31, half = lane >> 5;
    int blk, head;
    MapAttBlock(&blk, &head);
    // later query blocks of a causal sequence see more keys: they start first so that the short ones fill the tail of the launch
    const int myRow = (gridDim.x - 1 - blk) * BROWS + wave * WROWS + l32;
    const int64_t hoff = (int64_t)head * HD * 2;
    const int start = p.spanStart[myRow], finish = p.spanFinish[myRow];
    int kLo, kHi;
    BlockKeyRange(start, finish, tid, &kLo, &kHi, red);
    kLo = __builtin_amdgcn_readfirstlane(kLo);
    kHi = __builtin_amdgcn_readfirstlane(kHi);
    const int tFirst = kHi >= kLo ? (kLo / TR) * TR : 1;
    const uint8_t *gk = p.k + hoff, *gv = p.v + hoff;
    if (tFirst <= kHi) {
        LoadTileDirect(kT0, gk + (int64_t)tFirst * p.ldk, p.ldk, wave);
        LoadTileDirect(vT0, gv + (int64_t)tFirst * p.ldv, p.ldv, wave);
    }
    v8bf qf[8], of[8];
    LoadOwnFrags(qf, p.q + (int64_t)(myRow - l32) * p.ldq + hoff, p.ldq, l32, half);
    LoadOwnFrags(of, p.dO + (int64_t)(myRow - l32) * p.lddo + hoff, p.lddo, l32, half);
    const float L = p.sumWeightLog[(int64_t)head * p.ldStat + myRow];
    const float gmul = p.attDotScale * LN2;
    const float negDScale = -p.dScale[(int64_t)head * p.ldStat + myRow] * gmul;
    const TRowSpan sp = MakeRowSpan(start, finish);
    const TFragLane fl = MakeFragLane(lane);
    // cleared from a register the optimiser cannot see through: a constant zero vector would be kept alive across the tile loop as the
    // source of every other zero in the kernel, sixteen registers wide
    float zero = 0;
    asm volatile("" : "+v"(zero));
    v16f acc[4];
#pragma unroll
    for (int db = 0; db < 4; ++db) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            acc[db][e] = zero;
        }
    }
    // one 64-key tile: the 32-key blocks that some row of the wave sees (a run of blocks, wave-uniform bounds)
    auto tile = [&](const uint8_t *kt, const uint8_t *vt, int t0) __attribute__((always_inline)) {
#pragma unroll
        for (int kb = 0; kb < TR / 32; ++kb) {
            const int k0 = t0 + kb * 32;
            const uint8_t *kt2 = kt + kb * 32 * ROWB, *vt2 = vt + kb * 32 * ROWB;
            // A block is skipped by a loop of no trips rather than by a branch around it: the accumulators are then values carried by
            // a loop, which stay in their registers, where the join after a branch made the compiler copy all 64 of them.  The trip
            // count is opaque to the optimiser, or it would turn the loop back into that branch.
            int trips = __builtin_amdgcn_readfirstlane((int)!(k0 > sp.waveMaxFinish || k0 + 31 < sp.waveMinStart));
            asm volatile("" : "+s"(trips));
#pragma unroll 1
            for (int trip = 0; trip < trips; ++trip) {
            v16f s, dp;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                s[e] = 0;
                dp[e] = 0;
            }
            // phase 1: S^T = K Q^T and dP^T = V dO^T; the operands of step ds + 1 are requested before the products of step ds.
            // The wave raises its issue priority for its two MFMA phases: the SIMD's other wave then fills the gaps between this one's
            // products with its arithmetic instead of delaying them (3 % on this kernel; the same in the forward and the dK/dV
            // kernels measured nothing and a loss, and is not used there).
            v8bf fk[2], fv[2];
            fk[0] = FragRow(kt2, 0, 0, fl);
            fv[0] = FragRow(vt2, 0, 0, fl);
            __builtin_amdgcn_s_setprio(1);
#pragma unroll
            for (int ds = 0; ds < 8; ++ds) {
                if (ds + 1 < 8) {
                    fk[(ds + 1) & 1] = FragRow(kt2, 0, ds + 1, fl);
                    fv[(ds + 1) & 1] = FragRow(vt2, 0, ds + 1, fl);
                }
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fk[ds & 1], qf[ds], s, 0, 0, 0);
                dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fv[ds & 1], of[ds], dp, 0, 0, 0);
            }
            // the first operands of phase 3 are requested before the arithmetic of phase 2, which covers their latency
            v8bf ft[3];
            ft[0] = FragTr(kt2, 0, 0, 0, fl);
            ft[1] = FragTr(kt2, 0, 0, 1, fl);
            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
            for (int ds = 0; ds < 7; ++ds) {
                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
            __builtin_amdgcn_s_setprio(0);
            // phase 2: dS = w (dP - dScale) attDotScale ln2, w = 2^(logit - L): three instructions and the exponential per element
            // (without a slope the position term drops out of the logit)
            const float kc = ALIBI ? p.slope * (float)(k0 + half * 4 - myRow) - L : -L;
            const int rel0 = k0 + half * 4 - sp.start;
            const bool full = k0 >= sp.waveMaxStart && k0 + 31 <= sp.waveMinFinish;
            float dsv[16];
            if (full) { // every row of the wave sees every key of the block: no span tests
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    float x = fmaf(s[e], p.attDotScale, ALIBI ? fmaf(p.slope, (float)BlkRow(e, 0), kc) : kc);
                    float w = __builtin_amdgcn_exp2f(x);
                    dsv[e] = w * fmaf(dp[e], gmul, negDScale);
                }
            } else {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    float x = fmaf(s[e], p.attDotScale, ALIBI ? fmaf(p.slope, (float)BlkRow(e, 0), kc) : kc);
                    float w = __builtin_amdgcn_exp2f(x);
                    w = (unsigned)(rel0 + BlkRow(e, 0)) <= sp.len ? w : 0.f;
                    dsv[e] = w * fmaf(dp[e], gmul, negDScale);
                }
            }
            const v8bf sb[2] = {PackB(dsv, 0), PackB(dsv, 1)};
            __builtin_amdgcn_s_setprio(1);
            // phase 3: dQ^T += K^T dS^T, operands two products ahead
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                if (i + 2 < 8) {
                    ft[(i + 2) % 3] = FragTr(kt2, 0, (i + 2) >> 2, (i + 2) & 3, fl);
                }
                acc[i & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ft[i % 3], sb[i >> 2], acc[i & 3], 0, 0, 0);
            }
#pragma unroll
            for (int i = 0; i < 6; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            __builtin_amdgcn_s_setprio(0);
            }
        }
    };
    // two tiles per trip, one per buffer, in straight-line code: the accumulators live in one set of registers throughout, and the
    // operand reads of one buffer are known not to touch the buffer that the loads in flight fill
    for (int t0 = tFirst; t0 <= kHi;) {
        __builtin_amdgcn_s_waitcnt(0x0f70); // vmcnt(0): the tile of this step has landed
        __syncthreads();                    // ... for every wave, and every wave is done with the other buffer
        if (t0 + TR <= kHi) {
            LoadTileDirect(kT1, gk + (int64_t)(t0 + TR) * p.ldk, p.ldk, wave);
            LoadTileDirect(vT1, gv + (int64_t)(t0 + TR) * p.ldv, p.ldv, wave);
        }
        tile(kT0, vT0, t0);
        t0 += TR;
        if (t0 > kHi) {
            break;
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
        if (t0 + TR <= kHi) {
            LoadTileDirect(kT0, gk + (int64_t)(t0 + TR) * p.ldk, p.ldk, wave);
            LoadTileDirect(vT0, gv + (int64_t)(t0 + TR) * p.ldv, p.ldv, wave);
        }
        tile(kT1, vT1, t0);
        t0 += TR;
    }
    StoreOwnRows<F32>(p.out0 + (int64_t)(myRow - l32) * p.ldo0, p.ldo0, head * HD, acc, 1.f, l32, half);
}

__device__ __forceinline__ int Half32MaxInt(int v)
{
    v = max(v, LaneDpp<DPP_XOR1>(v));
    v = max(v, LaneDpp<DPP_XOR2>(v));
    v = max(v, LaneDpp<DPP_HALF_MIRROR>(v));
    v = max(v, LaneDpp<DPP_MIRROR>(v));
    int a, b;
    LaneSwap16(v, &a, &b);
    return max(a, b);
}

// dK, dV: grid (lenRound/64, heads).  The workgroup owns 64 key rows and streams the query rows that reach them; its four waves are
// two key blocks x two roles.  Both accumulators of a key block in one wave would need 128 registers and leave room for one wave per
// SIMD only; split over two waves, the kernel runs two workgroups per CU, and the two waves share the four products evenly: the dV
// wave forms S = Q K^T and the probabilities P and accumulates dV^T += dO^T P; the dK wave forms dP = dO V^T, takes P from the dV wave
// through LDS (fp32, the very values it would have computed itself), forms dS and accumulates dK^T += Q^T dS.
//
// Hand-over of a 32 x 32 block of P (4 KB per key block, one slot): two counters in LDS per key block, `ready` = number of blocks
// written by the dV wave, `taken` = number of blocks read by the dK wave.  The dV wave writes block n after taken >= n - 1 and then
// sets ready = n; the dK wave reads block n after ready >= n and then sets taken = n.  A wave's LDS operations complete in the order
// it issues them, so a counter is never seen before the data it covers.  Both waves of a pair skip the same blocks (the test
// depends on the pair's keys and the tile's bounds only), so they count the same blocks; neither wait depends on anything the
// waiting wave still has to do, and the tile barrier is reached by both after the same blocks.  The waits are bounded all the same:
// a wave whose wait runs out stops waiting for the rest of the launch (its results are then wrong, which the tests would show,
// but every wave finishes).
__device__ __forceinline__ void WaitCounter(int ldsAddr, int want, int &waiting)
{
    if (waiting) {
        int spins = 1 << 15;
#pragma unroll 1
        for (;;) {
            int v;
            asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(ldsAddr) : "memory");
            if (__builtin_amdgcn_readfirstlane(v) >= want) {
                break;
            }
            if (--spins == 0) {
                waiting = 0;
                break;
            }
            __builtin_amdgcn_s_sleep(1);
        }
    }
}

__device__ __forceinline__ void SetCounter(int ldsAddr, int value)
{
    asm volatile("ds_write_b32 %0, %1" : : "v"(ldsAddr), "v"(value) : "memory");
}

template <bool F32, bool ALIBI, bool DS> __global__ void __launch_bounds__(256, 2) AttGradKV(AttP p)
{
    __shared__ __attribute__((aligned(16))) float pBlock[2][4][64][4]; // [key block][quarter][lane][4 values]: P of the block in hand
    __shared__ int pCount[2][2];                                          // [key block][ready, taken]
    __shared__ __attribute__((aligned(1024))) uint8_t qT0[TILE_BYTES], qT1[TILE_BYTES], oT0[TILE_BYTES], oT1[TILE_BYTES];
    // [slot][L, dScale, span start, span finish, first dS block of the query's block][query], as loaded
    __shared__ __attribute__((aligned(16))) float rawStat[2][DS ? 5 : 4][TR];
    // [slot][-L - slope * (q - keyBase), -dScale * attDotScale * ln2, span start (0x7fffffff if empty), span length][query]: one array,
    // one address register
    __shared__ __attribute__((aligned(16))) float st[2][4][TR];
    __shared__ int stT[2][2][5]; // [slot][32-query block]: bounds over the block's queries, first dS block
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), l32 = lane & 31, half = lane >> 5;
    int block, head;
    MapAttBlock(&block, &head);
    // co-resident workgroups get opposite role orders, so that a SIMD is not handed two waves of the longer role
    const int rolePar = ((blockIdx.x + blockIdx.y * gridDim.x) >> 8) & 1;
    const int role = (wave ^ rolePar) & 1; // 0: dV, 1: dK
    // the wave that fetches and digests the per-query statistics of the coming tiles: the dK wave of the first key block, which
    // spends part of every block waiting for P anyway
    const int statWave = 1 ^ rolePar;
    const int keyBase = block * KVROWS;
    const int myRow = keyBase + (wave >> 1) * WROWS + l32; // my key
    const int64_t hoff = (int64_t)head * HD * 2;
    const int qLo = p.revLo[block >> 1], qHi = p.revHi[block >> 1];
    const int tFirst = qHi >= qLo ? (qLo / TR) * TR : 1;
    const uint8_t *gq = p.q + hoff, *go = p.dO + hoff;
    if (tid < 4) {
        (&pCount[0][0])[tid] = 0; // visible to every wave after the first tile's barrier
    }
    auto loadStats = [&](int t0, int slot) __attribute__((always_inline)) {
        if (wave == statWave) {
            const int lane = FreshLaneId();
            const int64_t so = (int64_t)head * p.ldStat + t0 + lane;
            __builtin_amdgcn_global_load_lds(TS2_GLB_PTR(p.sumWeightLog + so), TS2_LDS_PTR(&rawStat[slot][0][0]), 4, 0, 0);
            __builtin_amdgcn_global_load_lds(TS2_GLB_PTR(p.dScale + so), TS2_LDS_PTR(&rawStat[slot][1][0]), 4, 0, 0);
            __builtin_amdgcn_global_load_lds(TS2_GLB_PTR(p.spanStart + t0 + lane), TS2_LDS_PTR(&rawStat[slot][2][0]), 4, 0, 0);
            __builtin_amdgcn_global_load_lds(TS2_GLB_PTR(p.spanFinish + t0 + lane), TS2_LDS_PTR(&rawStat[slot][3][0]), 4, 0, 0);
            if constexpr (DS) {
                __builtin_amdgcn_global_load_lds(TS2_GLB_PTR(p.dsBase + t0 + lane), TS2_LDS_PTR(&rawStat[slot][DS ? 4 : 0][0]), 4, 0, 0);
            }
        }
    };
    // the statistics wave: raw statistics of the tile at t0 (slot) -> the form the products use
    auto digestStats = [&](int t0, int slot) __attribute__((always_inline)) {
        if (wave == statWave) {
            // the lane index is computed afresh: a value kept from the kernel's start would hold registers (or be spilled) across the
            // tile loop for the sake of these few instructions
            const int lane = FreshLaneId(), l32 = lane & 31, half = lane >> 5;
            const float rawL = rawStat[slot][0][lane];
            int preS = __float_as_int(rawStat[slot][2][lane]), preF = __float_as_int(rawStat[slot][3][lane]);
            const bool some = preF >= preS;
            preS = some ? preS : 0x7fffffff;
            preF = some ? preF : -1;
            float *dst = &st[slot][0][lane];
            dst[0] = -rawL - p.slope * (float)(t0 + lane - keyBase);
            dst[TR] = -rawStat[slot][1][lane] * (p.attDotScale * LN2);
            dst[2 * TR] = __int_as_float(preS);
            dst[3 * TR] = __int_as_float(some ? preF - preS : 0);
            const int a = Half32MaxInt(preS), b = -Half32MaxInt(-preF), c = -Half32MaxInt(-preS), d = Half32MaxInt(preF);
            if (l32 == 0) {
                stT[slot][half][0] = a; // latest span start of the block's queries
                stT[slot][half][1] = b; // earliest finish
                stT[slot][half][2] = c; // earliest start
                stT[slot][half][3] = d; // latest finish
                if constexpr (DS) {
                    stT[slot][half][4] = __float_as_int(rawStat[slot][DS ? 4 : 0][lane]);
                }
            }
        }
    };
    if (tFirst <= qHi) {
        loadStats(tFirst, 0);
        if (tFirst + TR <= qHi) {
            loadStats(tFirst + TR, 1);
        }
        LoadTileDirect(qT0, gq + (int64_t)tFirst * p.ldq, p.ldq, wave);
        LoadTileDirect(oT0, go + (int64_t)tFirst * p.lddo, p.lddo, wave);
    }
    const float gmul = p.attDotScale * LN2;
    const TFragLane fl = MakeFragLane(lane);
    const int kw0 = __builtin_amdgcn_readfirstlane(myRow - l32); // first key of this wave
    const float ck = p.slope * (float)(myRow - keyBase);
    const int64_t dsHead = DS ? (int64_t)head * p.dsBase[p.lenRound] : 0; // first dS block of this head
    // the whole tile loop once per role, as separate code: no value of one role's path meets a value of the other's, and every
    // operand fetch names the LDS array it reads (a fetch through a selected pointer would have to wait for the loads in flight)
    auto run = [&](auto roleTag) __attribute__((always_inline)) {
        constexpr int ROLE = decltype(roleTag)::value;
        v8bf own[8]; // the wave's keys as B operands: K for S (dV wave), V for dP (dK wave)
        if constexpr (ROLE) {
            LoadOwnFrags(own, p.v + (int64_t)(myRow - l32) * p.ldv + hoff, p.ldv, l32, half);
        } else {
            LoadOwnFrags(own, p.k + (int64_t)(myRow - l32) * p.ldk + hoff, p.ldk, l32, half);
        }
        float zero = 0; // opaque, as in AttGradQ
        asm volatile("" : "+v"(zero));
        v16f acc[4];
#pragma unroll
        for (int db = 0; db < 4; ++db) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                acc[db][e] = zero;
            }
        }
        // LDS addresses of the pair's block of P (this lane's 16 bytes of quarter 0) and of its two counters
        v4f *const pMine = (v4f *)&pBlock[wave >> 1][0][lane][0]; // named through the array: known not to be a tile with loads in flight
        const int readyAddr = (int)(uintptr_t)TS2_LDS_PTR(&pCount[wave >> 1][0]), takenAddr = readyAddr + 4;
        int blockNo = 0, waiting = 1;
        asm volatile("" : "+s"(waiting));
        if (tFirst <= qHi) {
            __builtin_amdgcn_s_waitcnt(0x0f70);
            digestStats(tFirst, 0);
        }
        // ---- pieces of a 32 x 32 block --------------------------------------------------------------------------------------------
        // first product: S = Q K^T (dV wave) or dP = dO V^T (dK wave), operands three steps ahead
        auto firstProduct = [&](v16f &x, const uint8_t *rt) __attribute__((always_inline)) {
            v8bf fr[4];
#pragma unroll
            for (int ds = 0; ds < 3; ++ds) {
                fr[ds] = FragRow(rt, 0, ds, fl);
            }
#pragma unroll
            for (int ds = 0; ds < 8; ++ds) {
                if (ds + 3 < 8) {
                    fr[(ds + 3) & 3] = FragRow(rt, 0, ds + 3, fl);
                }
                x = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[ds & 3], own[ds], x, 0, 0, 0);
            }
        };
        // dV wave: P from S and the per-query statistics of the tile
        auto probabilities = [&](const v16f &x, float (&wv)[16], int slot, int qb, auto fullTag) __attribute__((always_inline)) {
            constexpr bool full = decltype(fullTag)::value; // every query of the block sees every key of the wave: no span tests
            const float *ps = &st[slot][0][qb * 32 + half * 4];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const float4 L4 = *(const float4 *)(ps + g * 8);
                const float Ls[4] = {L4.x, L4.y, L4.z, L4.w};
                int Ss[4] = {0, 0, 0, 0};
                unsigned Ns[4] = {0, 0, 0, 0};
                if (!full) {
                    const int4 S4 = *(const int4 *)(ps + 2 * TR + g * 8);
                    const int4 N4 = *(const int4 *)(ps + 3 * TR + g * 8);
                    Ss[0] = S4.x; Ss[1] = S4.y; Ss[2] = S4.z; Ss[3] = S4.w;
                    Ns[0] = (unsigned)N4.x; Ns[1] = (unsigned)N4.y; Ns[2] = (unsigned)N4.z; Ns[3] = (unsigned)N4.w;
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int e = g * 4 + j;
                    float w = __builtin_amdgcn_exp2f(fmaf(x[e], p.attDotScale, ALIBI ? Ls[j] + ck : Ls[j]));
                    if (!full) {
                        w = (unsigned)(myRow - Ss[j]) <= Ns[j] ? w : 0.f;
                    }
                    wv[e] = w;
                }
            }
        };
        // pins values to the point of the call: without it the compiler sinks the arithmetic that makes them past the wait loops of the
        // hand-over, to just before their first use, and nothing is left to issue between the products
        auto pin16 = [&](float (&v)[16]) __attribute__((always_inline)) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                asm volatile("" : "+v"(v[4 * g]), "+v"(v[4 * g + 1]), "+v"(v[4 * g + 2]), "+v"(v[4 * g + 3]));
            }
        };
        // dV wave: hand block number n over once block n - 1 has been taken
        auto giveP = [&](const float (&wv)[16], int n) __attribute__((always_inline)) {
            WaitCounter(takenAddr, n - 1, waiting);
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                pMine[g * 64] = v4f{wv[4 * g], wv[4 * g + 1], wv[4 * g + 2], wv[4 * g + 3]};
            }
            SetCounter(readyAddr, n);
        };
        // dK wave: take block number n and form dS = P (dP attDotScale ln2 - dScale attDotScale ln2); the factor that does not need P
        // is formed before the wait
        auto takeP = [&](const v16f &x, float (&wv)[16], int slot, int qb, int n) __attribute__((always_inline)) {
            const float *ps = &st[slot][1][qb * 32 + half * 4];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const float4 D4 = *(const float4 *)(ps + g * 8);
                wv[4 * g] = fmaf(x[4 * g], gmul, D4.x);
                wv[4 * g + 1] = fmaf(x[4 * g + 1], gmul, D4.y);
                wv[4 * g + 2] = fmaf(x[4 * g + 2], gmul, D4.z);
                wv[4 * g + 3] = fmaf(x[4 * g + 3], gmul, D4.w);
            }
            pin16(wv);
            WaitCounter(readyAddr, n, waiting);
            v4f pw[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                pw[g] = pMine[g * 64];
            }
            SetCounter(takenAddr, n); // issued after the reads, so carried out after them
#pragma unroll
            for (int g = 0; g < 4; ++g) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    wv[4 * g + j] *= pw[g][j];
                }
            }
        };
        // dK wave: the block of dS goes to the dQ kernel, transposed on the way.  Here a lane is a key and its registers walk over the
        // queries; the dQ kernel's lanes are queries.  The operand pair the wave is about to multiply with, taken as the A operand of
        // two more MFMAs against the matching slices of the identity, comes back as dS^T with lane = query, registers = keys in the
        // order of the other kernel's operand fetches (exact: every sum has one term, and the values are bf16 already).  Block
        // number first(query block) + (this key block - first key block the query block sees); a lane's two operands of 16 bytes sit at
        // lane * 16 and 1024 + lane * 16: a wave writes, and the dQ kernel's wave reads, 1 KB contiguous per instruction.
        v8bf idB[2];
        if constexpr (DS && ROLE == 1) {
#pragma unroll
            for (int sl = 0; sl < 2; ++sl) {
                v4i r;
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    // slot j of operand sl in a lane of half h stands for query 16 sl + (j >> 2) * 8 + 4 h + (j & 3)
                    const int qa = 16 * sl + ((2 * w) >> 2) * 8 + 4 * half + ((2 * w) & 3), qb2 = qa + 1;
                    r[w] = (qa == l32 ? 0x3f80 : 0) | (qb2 == l32 ? 0x3f800000 : 0);
                }
                idB[sl] = __builtin_bit_cast(v8bf, r);
            }
        }
        auto giveDs = [&](const v8bf (&wb)[2], int slot, int qb) __attribute__((always_inline)) {
            if constexpr (DS && ROLE == 1) {
                const int first = __builtin_amdgcn_readfirstlane(stT[slot][qb][4]);
                const int startMin = __builtin_amdgcn_readfirstlane(stT[slot][qb][2]);
                const int64_t id = dsHead + first + ((kw0 >> 5) - (startMin >> 5));
                v16f tr;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    tr[e] = 0;
                }
                tr = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wb[0], idB[0], tr, 0, 0, 0);
                tr = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wb[1], idB[1], tr, 0, 0, 0);
                float tv[16];
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    tv[e] = tr[e];
                }
                const v8bf o0 = PackB(tv, 0), o1 = PackB(tv, 1);
                if (id >= 0 && id < p.dsCap) {
                    uint8_t *dst = p.ds + id * DS_BLOCK_BYTES + lane * 16;
                    *(v4i *)dst = __builtin_bit_cast(v4i, o0);
                    *(v4i *)(dst + 1024) = __builtin_bit_cast(v4i, o1);
                }
            }
        };
        // second product: dV^T += dO^T P or dK^T += Q^T dS, operands four products ahead; the first four are requested by the caller
        // (before the arithmetic that makes wb) with secondOperands
        auto secondOperands = [&](v8bf (&ft)[5], const uint8_t *tt) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                ft[i] = FragTr(tt, 0, i >> 2, i & 3, fl);
            }
        };
        auto secondProduct = [&](v8bf (&ft)[5], const uint8_t *tt, const v8bf (&wb)[2]) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                if (i + 4 < 8) {
                    ft[(i + 4) % 5] = FragTr(tt, 0, (i + 4) >> 2, (i + 4) & 3, fl);
                }
                acc[i & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ft[i % 5], wb[i >> 2], acc[i & 3], 0, 0, 0);
            }
        };
        // one 64-query tile: the 32-query blocks of which some query sees a key of this wave.  When both blocks are seen (the usual
        // case away from the edges of a span) they are worked on together, so that the wave always has instructions of one block
        // to issue while it waits for a result of the other: both first products, then the arithmetic of block 0 between the
        // products... (two waves per SIMD alone do not cover the latencies of a chain of dependent steps).
        auto tile = [&](const uint8_t *qt, const uint8_t *ot, int slot) __attribute__((always_inline)) {
            int bounds[2][4];
#pragma unroll
            for (int qb = 0; qb < 2; ++qb) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    bounds[qb][j] = __builtin_amdgcn_readfirstlane(stT[slot][qb][j]);
                }
            }
            const bool seen0 = !(bounds[0][3] < kw0 || bounds[0][2] > kw0 + 31), seen1 = !(bounds[1][3] < kw0 || bounds[1][2] > kw0 + 31);
            const bool full0 = bounds[0][0] <= kw0 && bounds[0][1] >= kw0 + 31, full1 = bounds[1][0] <= kw0 && bounds[1][1] >= kw0 + 31;
            const uint8_t *rtile = ROLE ? ot : qt; // the tile the first product reads by rows: dO for dP, Q for S
            const uint8_t *ttile = ROLE ? qt : ot; // the tile whose transpose the second product takes: Q^T for dK, dO^T for dV
            // skipped by loops of no trips, not by branches (see AttGradQ)
            const bool pair = seen0 && seen1 && full0 && full1;
            int pairTrips = __builtin_amdgcn_readfirstlane((int)pair);
            asm volatile("" : "+s"(pairTrips));
#pragma unroll 1
            for (int trip = 0; trip < pairTrips; ++trip) {
                const int n0 = blockNo + 1, n1 = blockNo + 2;
                blockNo += 2;
                v16f x0, x1;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    x0[e] = 0;
                    x1[e] = 0;
                }
                v8bf ft[5];
                float wv[16];
                firstProduct(x0, rtile);
                firstProduct(x1, rtile + 32 * ROWB);
                secondOperands(ft, ttile);
                if constexpr (ROLE == 0) {
                    float wv1[16];
                    probabilities(x0, wv, slot, 0, std::true_type{});
                    // the second first-product runs with the arithmetic of block 0 between its MFMAs
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    }
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                        __builtin_amdgcn_sched_group_barrier(0x002, 7, 0);
                    }
                    pin16(wv);
                    giveP(wv, n0);
                    const v8bf wb0[2] = {PackB(wv, 0), PackB(wv, 1)};
                    probabilities(x1, wv1, slot, 1, std::true_type{});
                    secondProduct(ft, ttile, wb0);
                    // ... and the arithmetic of block 1 between the MFMAs of block 0's second product
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                        __builtin_amdgcn_sched_group_barrier(0x002, 7, 0);
                    }
                    secondOperands(ft, ttile + 32 * ROWB);
                    pin16(wv1);
                    giveP(wv1, n1);
                    const v8bf wb1[2] = {PackB(wv1, 0), PackB(wv1, 1)};
                    secondProduct(ft, ttile + 32 * ROWB, wb1);
                } else {
                    takeP(x0, wv, slot, 0, n0);
                    const v8bf wb0[2] = {PackB(wv, 0), PackB(wv, 1)};
                    giveDs(wb0, slot, 0);
                    secondProduct(ft, ttile, wb0);
                    secondOperands(ft, ttile + 32 * ROWB);
                    takeP(x1, wv, slot, 1, n1);
                    const v8bf wb1[2] = {PackB(wv, 0), PackB(wv, 1)};
                    giveDs(wb1, slot, 1);
                    secondProduct(ft, ttile + 32 * ROWB, wb1);
                }
            }
#pragma unroll
            for (int qb = 0; qb < TR / 32; ++qb) {
                const bool full = qb ? full1 : full0;
                int trips = __builtin_amdgcn_readfirstlane((int)((qb ? seen1 : seen0) && !pair));
                asm volatile("" : "+s"(trips));
#pragma unroll 1
                for (int trip = 0; trip < trips; ++trip) {
                    ++blockNo;
                    v16f x;
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        x[e] = 0;
                    }
                    v8bf ft[5];
                    float wv[16];
                    firstProduct(x, rtile + qb * 32 * ROWB);
                    secondOperands(ft, ttile + qb * 32 * ROWB);
                    if constexpr (ROLE == 0) {
                        if (full) {
                            probabilities(x, wv, slot, qb, std::true_type{});
                        } else {
                            probabilities(x, wv, slot, qb, std::false_type{});
                        }
                        giveP(wv, blockNo);
                    } else {
                        takeP(x, wv, slot, qb, blockNo);
                    }
                    const v8bf wb[2] = {PackB(wv, 0), PackB(wv, 1)};
                    if constexpr (ROLE == 1) {
                        giveDs(wb, slot, qb);
                    }
                    secondProduct(ft, ttile + qb * 32 * ROWB, wb);
                }
            }
        };
        // two tiles per trip, one per buffer, in straight-line code (as in AttGradQ).  The raw statistics of the next tile are digested
        // before any new load is in flight, so that their reads wait for nothing.
        for (int t0 = tFirst; t0 <= qHi;) {
            __builtin_amdgcn_s_waitcnt(0x0f70); // vmcnt(0): the tile of this step and the raw statistics of the next have landed
            __syncthreads();                    // ... for every wave; every wave is done with the other buffers; st*[0] is visible
            if (t0 + TR <= qHi) {
                digestStats(t0 + TR, 1);
                LoadTileDirect(qT1, gq + (int64_t)(t0 + TR) * p.ldq, p.ldq, wave);
                LoadTileDirect(oT1, go + (int64_t)(t0 + TR) * p.lddo, p.lddo, wave);
            }
            if (t0 + 2 * TR <= qHi) {
                loadStats(t0 + 2 * TR, 0); // the slot of this step's raw statistics, digested one step ago
            }
            tile(qT0, oT0, 0);
            t0 += TR;
            if (t0 > qHi) {
                break;
            }
            __builtin_amdgcn_s_waitcnt(0x0f70);
            __syncthreads();
            if (t0 + TR <= qHi) {
                digestStats(t0 + TR, 0);
                LoadTileDirect(qT0, gq + (int64_t)(t0 + TR) * p.ldq, p.ldq, wave);
                LoadTileDirect(oT0, go + (int64_t)(t0 + TR) * p.lddo, p.lddo, wave);
            }
            if (t0 + 2 * TR <= qHi) {
                loadStats(t0 + 2 * TR, 1);
            }
            tile(qT1, oT1, 1);
            t0 += TR;
        }
        uint8_t *out = ROLE ? p.out0 : p.out1;
        const int64_t ldo = ROLE ? p.ldo0 : p.ldo1;
        StoreOwnRows<F32>(out + (int64_t)(myRow - l32) * ldo, ldo, head * HD, acc, 1.f, l32, half);
    };
    if (role) {
        run(std::integral_constant<int, 1>{});
    } else {
        run(std::integral_constant<int, 0>{});
    }
}

// dQ from the score gradients the dK/dV kernel left behind: dQ^T += K^T dS^T, one product per block, no statistics, no exponentials.
// grid (lenRound/128, heads); a wave owns 32 query rows (as in AttGradQ) and streams the key tiles its rows reach through LDS.  Its blocks
// of dS arrive transposed and in operand order (see giveDs), one after the other in memory: 32 bytes per lane and block straight into
// registers.  The kernel is a stream of loads with 16 MFMAs per tile and wave, so everything is requested two tiles ahead: three
// K buffers in LDS, three sets of dS registers, used in turn (three copies of the tile code per trip).  Every trip issues the same
// number of loads - past the end of the range they re-read the last tile, and a block the wave does not see is replaced by block 0 -
// so that "all but the newest eight" (vmcnt) at the top of a trip means that the tile and the blocks of this trip have landed.
template <bool F32> __global__ void __launch_bounds__(256, 3) AttGradQFromDs(AttP p)
{
    __shared__ __attribute__((aligned(1024))) uint8_t kT0[TILE_BYTES], kT1[TILE_BYTES], kT2[TILE_BYTES];
    __shared__ int red[8];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), l32 = lane & 31;
    int blk, head;
    MapAttBlock(&blk, &head);
    const int myRow = (gridDim.x - 1 - blk) * BROWS + wave * WROWS + l32; // long blocks first, as in AttGradQ
    const int64_t hoff = (int64_t)head * HD * 2;
    const int start = p.spanStart[myRow], finish = p.spanFinish[myRow];
    int kLo, kHi;
    BlockKeyRange(start, finish, tid, &kLo, &kHi, red);
    kLo = __builtin_amdgcn_readfirstlane(kLo);
    kHi = __builtin_amdgcn_readfirstlane(kHi);
    if (kHi < kLo) { // no row of the workgroup has a span (wave-uniform, before any barrier of the loop)
        v16f none[4];
#pragma unroll
        for (int db = 0; db < 4; ++db) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                none[db][e] = 0;
            }
        }
        StoreOwnRows<F32>(p.out0 + (int64_t)(myRow - l32) * p.ldo0, p.ldo0, head * HD, none, 1.f, l32, lane >> 5);
        return;
    }
    const int tFirst = (kLo / TR) * TR, tLast = (kHi / TR) * TR;
    const uint8_t *gk = p.k + hoff;
    const TRowSpan sp = MakeRowSpan(start, finish);
    // this wave's blocks of dS: number first + (key block - first key block the wave's rows see), per head
    const int64_t dsFirst = (int64_t)head * p.dsBase[p.lenRound] + __builtin_amdgcn_readfirstlane(p.dsBase[myRow]) - (sp.waveMinStart >> 5);
    const uint8_t *dsLane = p.ds + lane * 16;
    // requests for the tile at t0 (clamped to the last tile): its K rows, then the wave's two blocks of dS (block 0 for one it does not use)
    auto request = [&](uint8_t *kt, v4i (&sb)[2][2], int t0) __attribute__((always_inline)) {
        const int tt = t0 <= tLast ? t0 : tLast;
        LoadTileDirect(kt, gk + (int64_t)tt * p.ldk, p.ldk, wave);
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            const int k0 = tt + kb * 32;
            int64_t id = dsFirst + (k0 >> 5);
            if (k0 > sp.waveMaxFinish || k0 + 31 < sp.waveMinStart || id < 0 || id >= p.dsCap) {
                id = 0;
            }
            sb[kb][0] = *(const v4i *)(dsLane + id * DS_BLOCK_BYTES);
            sb[kb][1] = *(const v4i *)(dsLane + id * DS_BLOCK_BYTES + 1024);
        }
    };
    v4i sb0[2][2], sb1[2][2], sb2[2][2];
    request(kT0, sb0, tFirst);
    request(kT1, sb1, tFirst + TR);
    const TFragLane fl = MakeFragLane(lane);
    float zero = 0; // opaque, as in AttGradQ
    asm volatile("" : "+v"(zero));
    v16f acc[4];
#pragma unroll
    for (int db = 0; db < 4; ++db) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            acc[db][e] = zero;
        }
    }
    auto tile = [&](const uint8_t *kt, const v4i (&sb)[2][2], int t0) __attribute__((always_inline)) {
#pragma unroll
        for (int kb = 0; kb < TR / 32; ++kb) {
            const int k0 = t0 + kb * 32;
            const uint8_t *kt2 = kt + kb * 32 * ROWB;
            int trips = __builtin_amdgcn_readfirstlane((int)!(k0 > sp.waveMaxFinish || k0 + 31 < sp.waveMinStart)); // (see AttGradQ)
            asm volatile("" : "+s"(trips));
#pragma unroll 1
            for (int trip = 0; trip < trips; ++trip) {
                const v8bf b[2] = {__builtin_bit_cast(v8bf, sb[kb][0]), __builtin_bit_cast(v8bf, sb[kb][1])};
                v8bf ft[5];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    ft[i] = FragTr(kt2, 0, i >> 2, i & 3, fl);
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    if (i + 4 < 8) {
                        ft[(i + 4) % 5] = FragTr(kt2, 0, (i + 4) >> 2, (i + 4) & 3, fl);
                    }
                    acc[i & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ft[i % 5], b[i >> 2], acc[i & 3], 0, 0, 0);
                }
            }
        }
    };
    // per trip: the loads of this tile have landed (all but the eight of the next one), for every wave; request the tile after next
    // into the buffer every wave has just left; multiply
#define DQ_TRIP(KC, SC, KN, SN)                                                                                                            \
    __builtin_amdgcn_s_waitcnt(0x0f78); /* vmcnt(8) */                                                                                     \
    __syncthreads();                                                                                                                       \
    request(KN, SN, t0 + 2 * TR);                                                                                                          \
    tile(KC, SC, t0);                                                                                                                      \
    t0 += TR;                                                                                                                              \
    if (t0 > kHi) {                                                                                                                        \
        break;                                                                                                                             \
    }
    for (int t0 = tFirst;;) {
        DQ_TRIP(kT0, sb0, kT2, sb2)
        DQ_TRIP(kT1, sb1, kT0, sb0)
        DQ_TRIP(kT2, sb2, kT1, sb1)
    }
#undef DQ_TRIP
    __builtin_amdgcn_s_waitcnt(0x0f70); // the requests past the end land before the workgroup's LDS is given up
    StoreOwnRows<F32>(p.out0 + (int64_t)(myRow - l32) * p.ldo0, p.ldo0, head * HD, acc, 1.f, l32, lane >> 5);
}

// dsBase[q] = number of the first block of dS of q's 32-query block, numbering the blocks (query block, key block it sees) in the
// order of the query blocks; dsBase[lenRound] = their count.  A query block sees the key blocks from (earliest span start) / 32 to
// (latest span finish) / 32 of its rows with a span.  One workgroup; a thread takes a run of query blocks.
__global__ void __launch_bounds__(1024) DsIndexBuild(const int *spanStart, const int *spanFinish, int lenRound, int *dsBase)
{
    __shared__ int part[1024];
    const int nqb = lenRound / 32, tid = threadIdx.x;
    const int per = (nqb + 1023) / 1024, q0 = tid * per, q1 = min(nqb, q0 + per);
    auto count = [&](int qb) {
        int lo = 0x7fffffff, hi = -1;
        for (int i = 0; i < 32; ++i) {
            const int s = spanStart[qb * 32 + i], f = spanFinish[qb * 32 + i];
            if (f >= s) {
                lo = min(lo, s);
                hi = max(hi, f);
            }
        }
        return hi >= lo ? (hi >> 5) - (lo >> 5) + 1 : 0;
    };
    int sum = 0;
    for (int qb = q0; qb < q1; ++qb) {
        sum += count(qb);
    }
    part[tid] = sum;
    __syncthreads();
    for (int d = 1; d < 1024; d *= 2) { // inclusive scan
        const int v = tid >= d ? part[tid - d] : 0;
        __syncthreads();
        part[tid] += v;
        __syncthreads();
    }
    int run = part[tid] - sum;
    for (int qb = q0; qb < q1; ++qb) {
        for (int i = 0; i < 32; ++i) {
            dsBase[qb * 32 + i] = run;
        }
        run += count(qb);
    }
    if (tid == 1023) {
        dsBase[lenRound] = part[1023];
    }
}

bool ActOk(const ts2_mat *m, int rows, int cols)
{
    // the tile loads address a row group of a tile with 32-bit offsets (64 rows of one stride)
    return m && m->ptr && m->y >= rows && m->x >= cols && Aligned16(m->ptr, m->strideBytes) && m->strideBytes > 0 && m->strideBytes < (1 << 24);
}

} // namespace

extern "C" int ts2_att_build_rev(int32_t len, int32_t lenRound, const int32_t *spanStart, const int32_t *spanFinish, int32_t *revLo, int32_t *revHi,
    void *stream)
{
    if (!spanStart || !spanFinish || !revLo || !revHi) {
        return TS2_ERR_NULL;
    }
    if (lenRound % BROWS || len > lenRound) {
        return TS2_ERR_SHAPE;
    }
    int n = lenRound / BROWS;
    hipLaunchKernelGGL(RevInit, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream, revLo, revHi, n);
    TS2_CHECK_LAUNCH();
    hipLaunchKernelGGL(RevBuild, dim3((len + 255) / 256), dim3(256), 0, (hipStream_t)stream, spanStart, spanFinish, len, revLo, revHi);
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_att_forward(const ts2_att_args *a, void *stream)
{
    if (!a || !a->spanStart || !a->spanFinish || !a->sumWeightLog.ptr) {
        return TS2_ERR_NULL;
    }
    int cols = a->heads * HD;
    if (a->lenRound % BROWS || a->heads <= 0 || !ActOk(&a->q, a->lenRound, cols) || !ActOk(&a->k, a->lenRound, cols) ||
        !ActOk(&a->v, a->lenRound, cols) || !ActOk(&a->valLookup, a->lenRound, cols) || a->sumWeightLog.y < a->heads ||
        a->sumWeightLog.x < a->lenRound) {
        return TS2_ERR_SHAPE;
    }
    AttP p = {};
    p.q = (const uint8_t *)a->q.ptr;
    p.k = (const uint8_t *)a->k.ptr;
    p.v = (const uint8_t *)a->v.ptr;
    p.ldq = a->q.strideBytes;
    p.ldk = a->k.strideBytes;
    p.ldv = a->v.strideBytes;
    p.spanStart = a->spanStart;
    p.spanFinish = a->spanFinish;
    p.attDotScale = a->attDotScale;
    p.slope = a->alibiSlope;
    p.sumWeightLog = (float *)a->sumWeightLog.ptr;
    p.ldStat = a->sumWeightLog.strideBytes / 4;
    p.out0 = (uint8_t *)a->valLookup.ptr;
    p.ldo0 = a->valLookup.strideBytes;
    p.lenRound = a->lenRound;
    // the kernels without a slope leave the position term out of every logit; all LDS is static (two workgroups per CU)
    auto kernel = a->alibiSlope != 0 ? AttForward<true> : AttForward<false>;
    hipLaunchKernelGGL(kernel, dim3(a->lenRound / BROWS, a->heads), dim3(256), 0, (hipStream_t)stream, p);
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int ts2_att_build_ds_index(int32_t lenRound, const int32_t *spanStart, const int32_t *spanFinish, int32_t *dsBase, void *stream)
{
    if (!spanStart || !spanFinish || !dsBase) {
        return TS2_ERR_NULL;
    }
    if (lenRound <= 0 || lenRound % BROWS) {
        return TS2_ERR_SHAPE;
    }
    hipLaunchKernelGGL(DsIndexBuild, dim3(1), dim3(1024), 0, (hipStream_t)stream, spanStart, spanFinish, lenRound, dsBase);
    TS2_CHECK_LAUNCH();
    return TS2_OK;
}

extern "C" int64_t ts2_att_ds_blocks(int32_t lenRound, const int32_t *spanStartHost, const int32_t *spanFinishHost)
{
    if (!spanStartHost || !spanFinishHost || lenRound <= 0 || lenRound % 32) {
        return TS2_ERR_SHAPE;
    }
    int64_t total = 0;
    for (int qb = 0; qb < lenRound / 32; ++qb) {
        int lo = 0x7fffffff, hi = -1;
        for (int i = 0; i < 32; ++i) {
            const int s = spanStartHost[qb * 32 + i], f = spanFinishHost[qb * 32 + i];
            if (f >= s) {
                lo = s < lo ? s : lo;
                hi = f > hi ? f : hi;
            }
        }
        total += hi >= lo ? (hi >> 5) - (lo >> 5) + 1 : 0;
    }
    return total;
}

extern "C" int ts2_att_backward(const ts2_att_grad_args *a, void *stream)
{
    if (!a || !a->spanStart || !a->spanFinish || !a->revLo || !a->revHi || !a->sumWeightLog.ptr || !a->dScale.ptr) {
        return TS2_ERR_NULL;
    }
    int cols = a->heads * HD;
    bool f32 = a->gradType == TS2_F32;
    if (!f32 && a->gradType != TS2_BF16) {
        return TS2_ERR_UNSUPPORTED;
    }
    if (a->lenRound % BROWS || a->heads <= 0 || !ActOk(&a->q, a->lenRound, cols) || !ActOk(&a->k, a->lenRound, cols) ||
        !ActOk(&a->v, a->lenRound, cols) || !ActOk(&a->dValLookup, a->lenRound, cols) || !ActOk(&a->dQ, a->lenRound, cols) ||
        !ActOk(&a->dK, a->lenRound, cols) || !ActOk(&a->dV, a->lenRound, cols) || a->sumWeightLog.y < a->heads ||
        a->sumWeightLog.x < a->lenRound || a->dScale.y < a->heads || a->dScale.x < a->lenRound ||
        a->dScale.strideBytes != a->sumWeightLog.strideBytes) {
        return TS2_ERR_SHAPE;
    }
    AttP p = {};
    p.q = (const uint8_t *)a->q.ptr;
    p.k = (const uint8_t *)a->k.ptr;
    p.v = (const uint8_t *)a->v.ptr;
    p.dO = (const uint8_t *)a->dValLookup.ptr;
    p.ldq = a->q.strideBytes;
    p.ldk = a->k.strideBytes;
    p.ldv = a->v.strideBytes;
    p.lddo = a->dValLookup.strideBytes;
    p.spanStart = a->spanStart;
    p.spanFinish = a->spanFinish;
    p.revLo = a->revLo;
    p.revHi = a->revHi;
    p.attDotScale = a->attDotScale;
    p.slope = a->alibiSlope;
    p.sumWeightLog = (float *)a->sumWeightLog.ptr;
    p.dScale = (const float *)a->dScale.ptr;
    p.ldStat = a->sumWeightLog.strideBytes / 4;
    p.lenRound = a->lenRound;
    const bool alibi = a->alibiSlope != 0; // the kernels without a slope leave the position term out of every logit
    // with a dS array the dK/dV kernel leaves its score gradients behind and dQ is one product over them (both must run: which == 3)
    const bool viaDs = a->which == 3 && a->dsBase && a->dsScratch && a->dsCapacityBlocks > 0;
    if (viaDs) {
        if (((uintptr_t)a->dsScratch & 15) != 0) {
            return TS2_ERR_ALIGN;
        }
        p.dsBase = a->dsBase;
        p.ds = (uint8_t *)a->dsScratch;
        p.dsCap = a->dsCapacityBlocks;
    }
    if ((a->which & 1) && !viaDs) {
        p.out0 = (uint8_t *)a->dQ.ptr;
        p.ldo0 = a->dQ.strideBytes;
        auto kernel = f32 ? (alibi ? AttGradQ<true, true> : AttGradQ<true, false>) : (alibi ? AttGradQ<false, true> : AttGradQ<false, false>);
        hipLaunchKernelGGL(kernel, dim3(a->lenRound / BROWS, a->heads), dim3(256), 0, (hipStream_t)stream, p);
        TS2_CHECK_LAUNCH();
    }
    if (a->which & 2) {
        p.out0 = (uint8_t *)a->dK.ptr;
        p.ldo0 = a->dK.strideBytes;
        p.out1 = (uint8_t *)a->dV.ptr;
        p.ldo1 = a->dV.strideBytes;
        auto kernel = f32 ? (alibi ? AttGradKV<true, true, false> : AttGradKV<true, false, false>)
                          : (alibi ? AttGradKV<false, true, false> : AttGradKV<false, false, false>);
        if (viaDs) {
            kernel = f32 ? (alibi ? AttGradKV<true, true, true> : AttGradKV<true, false, true>)
                         : (alibi ? AttGradKV<false, true, true> : AttGradKV<false, false, true>);
        }
        hipLaunchKernelGGL(kernel, dim3(a->lenRound / KVROWS, a->heads), dim3(256), 0, (hipStream_t)stream, p);
        TS2_CHECK_LAUNCH();
    }
    if (viaDs) {
        p.out0 = (uint8_t *)a->dQ.ptr;
        p.ldo0 = a->dQ.strideBytes;
        hipLaunchKernelGGL(f32 ? AttGradQFromDs<true> : AttGradQFromDs<false>, dim3(a->lenRound / BROWS, a->heads), dim3(256), 0, (hipStream_t)stream, p);
        TS2_CHECK_LAUNCH();
    }
    return TS2_OK;
}
