/*
 * ts2_abi.h — C ABI of the MI355X (gfx950) backward path for the TScale2 transformer trainer.
 *
 * Every entry point replaces one operator (or kernel launch) of the reference's src/gpt operator surface; the reference
 * interface it stands for is cited as path:line under the reference tree.  Conventions follow the reference:
 *   - 2-D device arrays are row-major [y][x] with a byte stride (TCuda2DPtr, src/lib/cuda/cuda_arrays.h:217-253);
 *   - activations are [token][feature], weights are [out][in], "len" is the number of live token rows;
 *   - the caller owns every buffer, nothing is allocated or retained by the library, all work is enqueued on the
 *     caller's stream (a hipStream_t passed as void*) and the call returns without synchronising;
 *   - device-resident scalars (weight scale, gradient scale) are passed as float* so no host sync is needed
 *     (TCudaPOD<float>, src/lib/cuda/cuda_arrays.h:54-93).
 * Errors: the reference aborts (Y_VERIFY, src/util/pch.h:113); here every function returns 0 on success and a negative
 * TS2_ERR_* code on invalid shapes/alignment/unsupported combinations, and never aborts.
 */
#ifndef TS2_ABI_H
#define TS2_ABI_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TS2_OK 0
#define TS2_ERR_SHAPE (-1)       /* dimension not a multiple of the required tile, or size mismatch */
#define TS2_ERR_ALIGN (-2)       /* pointer or stride not 16-byte aligned */
#define TS2_ERR_UNSUPPORTED (-3) /* dtype / epilogue combination not implemented */
#define TS2_ERR_NULL (-4)        /* required pointer missing */
#define TS2_ERR_LAUNCH (-5)      /* the HIP runtime refused the launch */

/* element types (TFastModelFloat / TNormStateFloat / TFastGradientFloat choices, src/gpt/compute/cfg_precision.h:20-46) */
enum ts2_dtype {
    TS2_I8 = 0,
    TS2_E4M3 = 1, /* OCP e4m3fn, the format of src/util/fp8.h:4-21 */
    TS2_BF16 = 2, /* 16-bit activations; the reference uses IEEE half here */
    TS2_F32 = 3,
    TS2_I32 = 4,
    TS2_F16 = 5 /* IEEE half: result type of ts2_gemm_nt / ts2_matmul_forward only (the final layer's logits, as in the reference) */
};

/* row-major 2-D view: TCuda2DPtr<T>{Data, StrideInBytes} + debug sizes, src/lib/cuda/cuda_arrays.h:217-253 */
typedef struct ts2_mat {
    void *ptr;
    int64_t strideBytes;
    int32_t x; /* columns (elements) */
    int32_t y; /* rows */
} ts2_mat;

/* GEMM epilogues = the reference's "store functors", src/lib/cuda/cuda_matmul.cuh:420-559 */
enum ts2_epilogue {
    TS2_EPI_STORE = 0,           /* TStore / TStoreScaled        :440-451,467-477 */
    TS2_EPI_ADD = 1,             /* TStoreAdd / TStoreAddScaled  :455-463,481-490 */
    TS2_EPI_ROW_TILE_MAXNORM = 2, /* TStoreRowTileMaxNormalize    :530-559  packed delta: i8 + TileScale[n/128][m] */
    /* TStoreRowTileNormalize :495-525 and TStoreRowTileNormalizeRope (src/gpt/compute/gpu_rope.cuh:25-60): cType TS2_BF16;
     * v = alpha*acc; if normalize: tileScale[n/128][m] = rms over each 128-column tile * vecScale (0 for zero tiles), v /= it;
     * if rope.ptr: rotate (even, odd) column pairs of each 128-wide head by the row's (cos, sin) table fp32 [m][128].
     * Carried by the 256x256-tile kernel (m, n multiples of 256 and (m/256)*(n/256) >= 192, or tileConfig 1) and, for TS2_E4M3 and
     * TS2_BF16 operands, by the 128x128-tile kernel (tileConfig 2, or implied by tileGroup: the expert-grouped expand product,
     * MatmulExpand.Forward<TStoreRowTileNormalize>, src/gpt/compute/layer_moe.cu:160-162); else TS2_ERR_UNSUPPORTED and the caller
     * runs ts2_row_tile_normalize_rope on a plain product. */
    TS2_EPI_ROW_TILE_NORM = 3
};

/*
 * C[m][n] (op)= alpha * (*alphaPtr) * rowScale[m] * sum_k A[m][k] * B[n][k]
 * Both operands K-contiguous — the contract of every GEMM core of the reference:
 *   Int8MatMulKernel / Int8MatMulKernelRowScale / Int8MatMulYScaleKernel  src/lib/cuda/cuda_i8.cuh:157-320
 *   GenericMatMulKernel (fp8, fp16)                                        src/lib/cuda/cuda_matmul.cuh:396-416
 * abType: TS2_I8 (int32 accumulate, exact), TS2_E4M3 or TS2_BF16 (fp32 accumulate).
 * cType : TS2_F32, TS2_BF16, TS2_F16 (TS2_EPI_STORE only), TS2_I32 (raw accumulator, TS2_I8 inputs and TS2_EPI_STORE only) or TS2_I8
 *         (ROW_TILE_MAXNORM).
 *         16-bit and TS2_I8 results: 128 rows of C within 2 GiB (row stride below 16 MiB), else TS2_ERR_UNSUPPORTED; 16-bit rows
 *         4-byte aligned.
 * rowScale  (optional, [m], 16-byte aligned): per-row scale of A applied to the accumulator before the epilogue (the dX kernel).
 * kTileScale (optional, [k/kTile], TS2_I8 only): one scale per kTile contraction rows; each tile's int32 sum is exact and
 *             tiles are added in fp32 in tile order (the dW kernel).  kTile must be a multiple of 128.
 * splitK    : >1 cuts the contraction into that many slices, each STORED to its own slab of C (splitSlabBytes, below; required:
 *             partial sums are never added atomically, every result of the library is deterministic).
 * Requirements: k a multiple of 128 (8-bit) or 64 (bf16); m, n multiples of 128; 16-byte aligned rows.
 * Rows >= mLive of C are written as zeros when mLive < m (producers keep pad rows zero, src/lib/cuda/cuda_matmul.cuh:10).
 */
typedef struct ts2_gemm_args {
    ts2_mat a, b, c;
    int32_t abType, cType;
    int32_t m, n, k;
    int32_t mLive; /* 0 = all rows live */
    const float *rowScale;
    const float *kTileScale;
    int32_t kTile;
    float alpha;
    const float *alphaPtr;
    int32_t epilogue;
    ts2_mat tileScale; /* ROW_TILE_MAXNORM: fp32 [n/128][m] */
    int32_t splitK;
    /* bits 0-1: 0 = choose (256x256 when m, n are multiples of 256 and there are 192 tiles or more, except for TS2_E4M3 products with
     * k <= 512, or k <= 1024 and TS2_EPI_ADD, which are mostly their epilogue and run on 128x128); 1 = 256x256 workgroup tile;
     * 2 = 128x128; 3 = 256x128 (int8 with kTileScale, fp32 result).
     * Comparison switches, all off in normal use: bit 2 (4) unused (TS2_ERR_UNSUPPORTED); bit 3 (8) eight waves per workgroup (256x256
     * store/accumulate results; with tile 3: the form BackpropDelta launches); bit 4 (16) two LDS stages instead of the ring on the
     * 256x256 tile (and on the 128x128 tile with TS2_E4M3 operands, which takes the ring from k = 1024 on); bits 5-6 tile-order
     * group 8 / 4 / 2 instead of the automatic choice; bit 7 (128) the ring on the 128x128 tile at any k; bits 9 / 10 (512 / 1024)
     * plain / non-temporal stores of C instead of the choice by k; bit 11 (2048) the 256x128 kernel with 64-byte steps for two
     * workgroups per CU (k a multiple of 64 bytes); bit 12 (4096) the persistent eight-wave kernel whose epilogue runs under the next
     * tile's main loop (m % 256 = 0, k >= 1024 bytes; fp32 / 16-bit / raw int32 results, store or accumulate), bits 13-14 its
     * workgroup count as CUs >> 2, 4, 6 (tests).  Bits 11 and 12 return TS2_ERR_UNSUPPORTED for calls their kernel cannot run.  With
     * bits 0-4 clear the persistent kernel is also chosen automatically for stored results with 1024 <= k bytes < 4096 and at least
     * 512 tiles of 256x128; bit 15 (32768) switches that off.  The same kernel, on exchanged operands, takes tileGroup products
     * of TS2_E4M3 operands with a 16-bit stored result (plain or ROW_TILE_NORM; also with one further product) when n % 256 = 0,
     * k >= 512 bytes, c and its stride are multiples of 16 bytes and (m/128)*(n/256) >= 512 - or when bit 12 asks for it;
     * results are bit-identical to the 128x128 kernels'. */
    int32_t tileConfig;
    /* Expert-grouped products (TMoeMatMulKernelCall / TMoeDeltaMatMulKernelCall, src/gpt/compute/moe_matmul.cuh:47-215):
     * tileGroup [m/128] (device): rows of A and C are grouped by expert in 128-row tiles; tile i multiplies the B slab
     *           b + tileGroup[i]*bSlabBytes (n rows each); tiles with group -1 are skipped (XpTileExpertId).
     * groupOffsets [groups+1] (device): delta mode, one product per group g over contraction rows
     *           groupOffsets[g] .. groupOffsets[g+1] (multiples of 128; ExpertOffset), written to c + g*cSlabBytes and, for
     *           ROW_TILE_MAXNORM, tileScale + g*tileScaleSlabBytes. */
    const int32_t *tileGroup;
    int64_t bSlabBytes;
    const int32_t *groupOffsets;
    int32_t groups;
    int64_t cSlabBytes;
    int64_t tileScaleSlabBytes;
    /* splitK > 1 with splitSlabBytes != 0: slice i of the contraction is STORED to c + i*splitSlabBytes (fp32, TS2_EPI_STORE; slices
     * are whole k-tiles): deterministic, the caller sums the slices (ts2_pack_delta does).  splitK > 1 without it is refused. */
    int64_t splitSlabBytes;
    /* TS2_EPI_ROW_TILE_NORM */
    int32_t normalize;
    float vecScale;
    ts2_mat rope;
    /* extraSegments > 0 (at most 3): C (+)= sum over the 1 + extraSegments products alpha_i * (*alphaPtr_i) * A_i * B_i^T with the same
     * m, n, k, operand type and operand strides; a, b, alpha, alphaPtr above describe product 0, segment[i-1] product i.  One launch
     * and one pass over C instead of one read-modify-write of C per product: the gradient of a layer input that feeds several
     * matrices (Backprop of Q, K, V and gate in src/gpt/compute/layer_att.cu:236-260 adds four products into the same array).
     * 256x256-tile kernel (m, n multiples of 256), or one further product on the 128x128 tile (tileConfig 2, or with tileGroup: the
     * expert-grouped dX of wide and gate, src/gpt/compute/layer_moe.cu:236-250, where every B_i takes the tile's slab); TS2_E4M3 or
     * TS2_BF16 operands, fp32 or bf16 C, TS2_EPI_STORE or TS2_EPI_ADD, no rowScale, kTileScale, groupOffsets or splitK; the fp32 sums
     * of the products are rescaled in registers between products. */
    int32_t extraSegments;
    struct {
        const void *a;
        const void *b;
        float alpha;
        const float *alphaPtr;
    } segment[3];
    /* kMajor != 0: A is [k][m] and B is [k][n] - the rows of both operands are the contraction index, C[i][j] = sum_k A[k][i] * B[k][j].
     * The form a delta product dW = dY^T X takes on the untransposed activations ([token][feature], src/gpt/compute/matmul_fwdbwd.cuh:314-391
     * transposes both first; the final layer's Fp16MatMul<1, 1, TStoreDelta>, src/gpt/compute/gpu_final.cuh:265, reads both transposed):
     * the operands are transposed by the LDS reads of the kernel instead.  TS2_E4M3 or TS2_BF16 operands, m and n multiples
     * of 256 (the 256x256 kernel; with tileConfig 0 the caller must make sure that (m/256)*(n/256)*slices >= 192 or pass tileConfig 1),
     * fp32 TS2_EPI_STORE results (also as stored slices, splitSlabBytes) or TS2_EPI_ROW_TILE_MAXNORM; nothing else. */
    int32_t kMajor;
} ts2_gemm_args;

int ts2_gemm_nt(const ts2_gemm_args *args, void *stream);


/* ------------------------------------------------------------------------------------------------------------------------
 * Bandwidth-bound fused kernels.  All 2-D operands are [row = token][feature]; feature counts are multiples of 128; per-tile
 * scale arrays are fp32 [feature/128][row] like the reference's (TFragmentStates::StateScale, layer_cuda_base.cuh:125-149).
 * "len" = live rows, "lenRound" = rows including padding (multiple of 128) where a kernel also clears the pad rows. */

/* LayerNormalizeStateVecs, src/gpt/compute/gpu_layer_norm.cuh:6-32: per 128-tile scale = sqrt(sum2/128)*vecScale,
 * normState = state/scale as normType (TS2_I8 | TS2_E4M3 | TS2_BF16), scale 0 and zero data for zero tiles and rows >= len. */
int ts2_layer_normalize_state_vecs(const ts2_mat *state, int32_t stateType, int32_t len, int32_t lenRound, float vecScale,
    const ts2_mat *normState, int32_t normType, const ts2_mat *normStateScale, void *stream);

/* BackpropLayerNormalize, src/gpt/compute/gpu_layer_norm.cuh:89-115: g = dNormState * (*combinerScale) * (*gradScale); tile-norm
 * backward against normState*stateScale; stateGrad += g (fp32, in place); stateGradFast = stateGrad * (*gradMult) as fastType
 * (TS2_BF16 | TS2_E4M3); atomic max of |stateGrad| into *nextLayerGradMaxNorm.  Scalar pointers may be NULL (= 1). */
int ts2_backprop_layer_normalize(const ts2_mat *normState, int32_t normType, const ts2_mat *stateScale, const ts2_mat *dNormState,
    const float *combinerScale, const float *gradScale, const float *gradMult, const ts2_mat *stateGrad, const ts2_mat *stateGradFast,
    int32_t fastType, float *nextLayerGradMaxNorm, int32_t len, void *stream);

/* BackpropFinalNormalize, src/gpt/compute/gpu_layer_norm.cuh:119-146: same without the residual add; rows >= len are cleared. */
int ts2_backprop_final_normalize(int32_t len, int32_t lenRound, const ts2_mat *normState, int32_t normType, const ts2_mat *stateScale,
    const ts2_mat *dNormState, const ts2_mat *stateGrad, const ts2_mat *stateGradFast, int32_t fastType, float *nextLayerGradMaxNorm,
    void *stream);

/* ScaleGrad + ComputeGradMult, src/gpt/compute/gpu_grad_scale.cuh:33-62: gradMult = 2^floor(log2(128 / *gradMaxNorm)) (1 if the
 * max is 0); when it differs from *prevGradMult rewrite gradFast = grad * gradMult; publishes *gradScaleOut = 1/gradMult and
 * *gradMultOut = gradMult. */
int ts2_scale_grad(const float *gradMaxNorm, const float *prevGradMult, const ts2_mat *grad, const ts2_mat *gradFast, int32_t fastType,
    int32_t len, float *gradScaleOut, float *gradMultOut, void *stream);

/* MatrixLoLU, src/gpt/compute/gpu_lolu.cuh:41-69: res = vals * sigmoid(2*gate) * resMult as resType; rows in [len, lenRound) zero.
 * gate and vals are TS2_BF16. */
int ts2_matrix_lolu(int32_t len, int32_t lenRound, const ts2_mat *gate, const ts2_mat *vals, float resMult, const ts2_mat *res,
    int32_t resType, void *stream);

/* BackpropRowTileNormalizeLoLU, src/gpt/compute/gpu_lolu.cuh:107-137 (FFN): vals*valsScale is the normalised "wide"; gradGate =
 * grad*vals*m(1-m)*2, gradVals = tile-norm backward of (grad*m) against vals*valsSrcTileScale; outputs as gradOutType. */
int ts2_backprop_row_tile_normalize_lolu(int32_t len, int32_t lenRound, const ts2_mat *gate, const ts2_mat *vals, float valsScale,
    const ts2_mat *valsSrcTileScale, const ts2_mat *grad, int32_t gradType, const ts2_mat *gradGate, const ts2_mat *gradVals,
    int32_t gradOutType, void *stream);

/* The same for TS2_BF16 gradients and TS2_E4M3 results, leaving also the transposed copies gradGateT, gradValsT [dim][lenRound] that
 * the delta products of the two matrices contract over (the reference's producers can save a transposed copy the same way: saveTransposed
 * of ComputeRG, src/gpt/compute/layer_moe.cu:117, and the transposing MoeGroupSamples, moe_kernels.cuh:89-143).  BackpropDelta is then
 * called with gradT pointing at the copy and gradTValid set.  lenRound must be a multiple of 128. */
int ts2_backprop_row_tile_normalize_lolu_t(int32_t len, int32_t lenRound, const ts2_mat *gate, const ts2_mat *vals, float valsScale,
    const ts2_mat *valsSrcTileScale, const ts2_mat *grad, const ts2_mat *gradGate, const ts2_mat *gradVals, const ts2_mat *gradGateT,
    const ts2_mat *gradValsT, void *stream);

/* BackpropLoLUdScale, src/gpt/compute/gpu_lolu.cuh:141-173 (attention): gate backward plus dScale[head][t] = <vals*valsScale,
 * gradVals> per 128-wide head. */
int ts2_backprop_lolu_dscale(int32_t len, int32_t lenRound, const ts2_mat *gate, const ts2_mat *vals, float valsScale, const ts2_mat *grad,
    int32_t gradType, const ts2_mat *gradGate, int32_t gradGateType, const ts2_mat *gradVals, int32_t gradValsType, const ts2_mat *dScale,
    void *stream);

/* NormalizeVecsRowMaxKernel, src/gpt/compute/row_scale.cuh:12-43, deterministic (the reference adds a random dither before rounding):
 * per row scale = maxabs/127, dst = sat_i8(rne(src/scale)); optional colScale[x] multiplies the source first; rows >= len cleared. */
int ts2_normalize_vecs_row_max(int32_t len, int32_t lenRound, const ts2_mat *src, int32_t srcType, const float *colScale,
    const ts2_mat *dst, float *rowScale, void *stream);

/* the same, also writing rowAbsMax[t] = abs-max of row t before the column scales (NULL: not wanted); ts2_tile_max_from_rows turns
 * those into the k-tile maxima tileMax[t/kTile] = max_t rowAbsMax[t]*|rowMult[t]| without another pass over the matrix */
int ts2_normalize_vecs_row_max2(int32_t len, int32_t lenRound, const ts2_mat *src, int32_t srcType, const float *colScale,
    const ts2_mat *dst, float *rowScale, float *rowAbsMax, void *stream);
int ts2_tile_max_from_rows(int32_t len, const float *rowAbsMax, const float *rowMult, int32_t kTile, float *tileMax, void *stream);

/* the same with the reference's dither (src/gpt/compute/row_scale.cuh:32-35 adds uniform noise in (-0.5, 0.5) before it rounds, which
 * makes the int8 gradient unbiased): ditherSeed != 0 quantises dst = sat_i8(rne(fma(src, 1/scale, u))) with
 * u(t, x) = (byte (x % 4) of H(ditherSeed, t, x / 4) - 127.5) / 256, H(s, r, c) = lowbias32(s ^ r * 0x9E3779B1 ^ c * 0x85EBCA6B),
 * lowbias32(h): h ^= h >> 16; h *= 0x7FEB352D; h ^= h >> 15; h *= 0x846CA68B; h ^= h >> 16 - the reference draws its noise from an LCG
 * seeded with the row's own bits; this stream is the library's own, the property (E[dst * scale] = src) is the reference's.
 * ditherSeed 0 = ts2_normalize_vecs_row_max2. */
int ts2_normalize_vecs_row_max_dither(int32_t len, int32_t lenRound, const ts2_mat *src, int32_t srcType, const float *colScale,
    const ts2_mat *dst, float *rowScale, float *rowAbsMax, uint32_t ditherSeed, void *stream);

/* HistSortFloatsStableKernel, src/lib/cuda/cuda_sort.cu:115-186 (SortPositiveFloatsApproxStable as BackpropMulti calls it on the row
 * scales of the gradient, src/gpt/compute/matmul_fwdbwd.cuh:325): order[0..len) = the rows sorted ascending by the top 13 bits (sign,
 * exponent, four mantissa bits) of key[t] = rowAbsMax[t] * |rowMult[t]| (rowMult optional); rows that share those bits come in
 * descending row order, as in the reference (whose own test holds the hash of that order).  len < 500: the exact order the reference
 * takes there (PerformRegularSort, cuda_sort.cu:50-60,117-120): ascending by the whole key, equal keys in ascending row order.
 * Deterministic.  tmp: len ints of scratch. */
int ts2_sort_rows_by_scale(int32_t len, const float *rowAbsMax, const float *rowMult, int32_t *order, int32_t *tmp, void *stream);

/* Per-k-tile abs-max of a [len][dim] matrix (optionally times rowMult[t]): tileMax[t/kTile] = max |src|, the first half of
 * ShuffleMaxScaleTransposeKernel (src/gpt/compute/matmul_fwdbwd.cuh:209-231) without the sort.  tileMax must be zeroed by the
 * caller or with clear=1. */
int ts2_tile_absmax(int32_t len, const ts2_mat *src, int32_t srcType, const float *rowMult, int32_t kTile, float *tileMax, int32_t clear,
    void *stream);

/* Quantise + transpose: dst[x][t] = cvt(src[t][x] * rowMult[t] * mult(t)) for t < len, 0 for len <= t < lenRound.
 * dstType TS2_I8: mult = 127/tileMax[t/kTile] and tileScale[t/kTile] = tileMax/127 (1 when the tile is all zero) is written;
 * dstType equal to srcType (1-byte types): pure byte transpose (TransposeI8Matrix, src/lib/cuda/cuda_i8.cuh:14-71;
 * ShuffleTransposeKernel / ShuffleMaxScaleTransposeKernel, src/gpt/compute/matmul_fwdbwd.cuh:169-280).
 * rowIndex (optional, [lenRound], -1 = zero row) gathers source rows first (MoeGroupSamples, moe_kernels.cuh:89-143). */
int ts2_transpose_quant(int32_t len, int32_t lenRound, const ts2_mat *src, int32_t srcType, const float *rowMult, const float *tileMax,
    int32_t kTile, const int32_t *rowIndex, const ts2_mat *dstT, int32_t dstType, float *tileScale, void *stream);
/* the same with the dither of ts2_normalize_vecs_row_max_dither in the requantisation (dstType TS2_I8): the noise of element (t, x) is
 * u(t, x) with t the position in dstT's rows (after the gather through rowIndex), x the source column. */
int ts2_transpose_quant_dither(int32_t len, int32_t lenRound, const ts2_mat *src, int32_t srcType, const float *rowMult, const float *tileMax,
    int32_t kTile, const int32_t *rowIndex, const ts2_mat *dstT, int32_t dstType, float *tileScale, uint32_t ditherSeed, void *stream);

/* Compress (src/gpt/matrix/delta.cpp:155-179) of a sum of fp32 partial products: delta = packed(alpha * (*alphaPtr) * sum_i partial_i),
 * partial_i = fp32 [rows][cols] at partial->ptr + i*slabBytes; the same arithmetic as TS2_EPI_ROW_TILE_MAXNORM.  Used with the stored
 * split-K products of ts2_gemm_nt (splitSlabBytes). */
int ts2_pack_delta(const ts2_mat *partial, int32_t splits, int64_t slabBytes, int32_t rows, int32_t cols, float alpha, const float *alphaPtr,
    const ts2_mat *delta, const ts2_mat *deltaTileScale, void *stream);

/* ------------------------------------------------------------------------------------------------------------------------
 * Linear-layer backward operator = TMatMulBuffers::{BackpropMulti, BackpropDelta} + Backprop()
 * (src/gpt/compute/layer_cuda_base.cuh:153-250) over TInt8MatMulBwdBuffers / TFp8MatMulBwdBuffers
 * (src/gpt/compute/matmul_fwdbwd.cuh:108-163,283-391).  mode = TS2_I8 or TS2_E4M3 (BWD_MATMUL_TYPE, cfg_precision.h:20-35).
 *
 * Scratch is caller-owned, like the reference's pool-allocated members; every buffer the mode does not use may be empty:
 *   grad8 [lenRound][gradDim] i8 + grad8RowScale [lenRound]   (I8: Grad8, Grad8RowScale)
 *   gradT [gradDim][lenRound] 8-bit                             (I8: Grad8T; E4M3: GradE5T)
 *   srcT  [srcDim][lenRound] 8-bit                              (I8: Src8T;  E4M3: SrcE4T)
 *   tileMax, tileScale [lenRound/kTile] fp32                    (I8: SortedTileScale)
 *   transformT [srcDim][gradDim] 8-bit                          (TransformT)
 * Differences from the reference, by design: the dither of the int8 quantisers is optional and drawn from the library's own
 * counter-based stream (ditherSeed), the sort of the rows is optional (sortRows; without it each kTile consecutive tokens share the
 * delta GEMM's scale) and exact int32 sums per k-tile added in fp32. */
typedef struct ts2_matmul_bwd_buffers {
    ts2_mat grad8;
    float *grad8RowScale;
    ts2_mat gradT;
    ts2_mat srcT;
    float *tileMax;
    float *tileScale;
    ts2_mat transformT;
    /* optional: fp32 [splits*gradDim][srcDim].  When present (ptr != NULL, splits > 1) BackpropDelta runs the product as `splits`
     * deterministic slices of the token axis on the large tile and packs their sum (ts2_pack_delta): faster when gradDim x srcDim
     * has too few tiles to fill the device; the fp32 sum is then associated per slice (slices are whole k-tiles). */
    ts2_mat partial;
    int32_t splits;
    /* optional (I8): [lenRound] abs-max of every row of the gradient, written by BackpropMulti.  BackpropDelta reads it instead of
     * scanning the gradient again when gradRowAbsMaxValid != 0: the caller sets that when both calls get the same gradient tensor. */
    float *gradRowAbsMax;
    int32_t gradRowAbsMaxValid;
    /* != 0: srcT already holds the transpose of the `src` given to BackpropDelta (an earlier BackpropDelta call with the same buffers
     * and the same source tensor left it there, as for the matrices of one layer that share their input); the transpose is skipped. */
    int32_t srcTValid;
    /* != 0 (E4M3): gradT already holds the transpose of the `grad` given to BackpropDelta (its producer wrote it, e.g.
     * ts2_backprop_row_tile_normalize_lolu_t); the transpose is skipped. */
    int32_t gradTValid;
    /* != 0: transformT already holds the transpose of the `transformFast` given to BackpropMulti (the matrix has not changed since an
     * earlier call left it there: weights change once per optimiser step, not per micro-batch); the transpose is skipped. */
    int32_t transformTValid;
    /* optional (I8): sortRows != 0 makes BackpropDelta contract over the rows in the order of ts2_sort_rows_by_scale (key = the gradient
     * row's abs-max times |srcRowScale|), as the reference does (ShuffleMaxScaleTransposeKernel / ShuffleTransposeKernel gather the rows
     * through the sorted list, matmul_fwdbwd.cuh:169-280): the rows of a k-tile then have like magnitudes and their common scale wastes
     * few bits.  Needs gradRowAbsMax (valid) and rowOrder / rowOrderTmp [lenRound]; srcTValid is ignored (the source is gathered in this
     * matrix's own order).  The delta itself does not depend on the order of the rows beyond the quantisation. */
    int32_t *rowOrder;
    int32_t *rowOrderTmp;
    int32_t sortRows;
    /* != 0 (E4M3): rows len .. lenRound of the `src` and `grad` given to BackpropDelta hold zeros (the producers of this library leave
     * them so, like the reference's, src/lib/cuda/cuda_matmul.cuh:10).  With srcDim and gradDim on the 256 grid the delta product then
     * reads both operands as they are - contraction-major, ts2_gemm_args.kMajor - and neither is transposed: gradT, srcT and their
     * Valid flags are not used.  The result is bit-identical to the transposing sequence. */
    int32_t padRowsZero;
    /* != 0 (I8): BackpropMulti and BackpropDelta quantise the gradient with the dither of ts2_normalize_vecs_row_max_dither /
     * ts2_transpose_quant_dither under this seed (unbiased int8 gradients, as the reference's NormalizeVecsRowMaxWithNoise gives); 0 rounds
     * to nearest.  A caller varies the seed from matrix to matrix and from step to step. */
    uint32_t ditherSeed;
} ts2_matmul_bwd_buffers;

/* Bytes of every scratch member of ts2_matmul_bwd_buffers for one matrix, the sizes TInt8MatMulBwdBuffers / TFp8MatMulBwdBuffers allocate
 * from the reference's pools (src/gpt/compute/matmul_fwdbwd.cuh:108-125,283-311): out[0] grad8, [1] grad8RowScale, [2] gradT, [3] srcT,
 * [4] tileMax, [5] tileScale, [6] transformT, [7] partial (splits slices), [8] gradRowAbsMax; members the mode does not use are 0.
 * Rows are dense (stride = row bytes).  Returns TS2_ERR_SHAPE for sizes the operator refuses. */
int ts2_matmul_bwd_scratch_bytes(int32_t mode, int32_t lenRound, int32_t srcDim, int32_t gradDim, int32_t kTile, int32_t splits, int64_t out[9]);

/* BackpropMulti (prep of dX): I8: quantise grad (TS2_BF16 | TS2_F32, optionally times gradColScale[gradDim]) per row to
 * grad8/grad8RowScale and transpose the weight; E4M3: transpose the weight.  transformFast is [gradDim][srcDim]. */
int ts2_matmul_backprop_multi(int32_t mode, int32_t len, int32_t lenRound, int32_t srcDim, int32_t gradDim, const ts2_mat *transformFast,
    const ts2_mat *grad, int32_t gradType, const float *gradColScale, const ts2_matmul_bwd_buffers *buf, void *stream);

/* Backprop(): srcGrad[len][srcDim] (+)= alpha * (*alphaPtr) * grad * W.  I8 reads grad8/grad8RowScale from buf; E4M3 reads grad
 * (e4m3 [lenRound][gradDim]) directly.  srcGradType TS2_F32 | TS2_BF16; add != 0 accumulates (multi-source sum). */
int ts2_matmul_backprop(int32_t mode, int32_t len, int32_t lenRound, int32_t srcDim, int32_t gradDim, const ts2_mat *grad,
    const ts2_matmul_bwd_buffers *buf, float alpha, const float *alphaPtr, const ts2_mat *srcGrad, int32_t srcGradType, int32_t add,
    void *stream);

/* Backprop() of `count` (2..4) matrices that share their input (Q, K, V and gate of an attention layer,
 * src/gpt/compute/layer_att.cu:236-260; wide and gate of an FFN layer, layer_ffn.cu): srcGrad (+)= sum_i alpha[i] * (*alphaPtr[i]) *
 * grad[i] * W_i, where the reference adds one product after the other into the same array.  Every bufs[i] must have been prepared by
 * ts2_matmul_backprop_multi for its matrix; all matrices are [gradDim][srcDim].  TS2_E4M3 with srcDim and lenRound multiples of 256
 * runs as one launch (one pass over srcGrad); otherwise the products are launched one after the other as the reference does. */
int ts2_matmul_backprop_group(int32_t mode, int32_t len, int32_t lenRound, int32_t srcDim, int32_t gradDim, int32_t count,
    const ts2_mat *const *grad, const ts2_matmul_bwd_buffers *const *bufs, const float *alpha, const float *const *alphaPtr,
    const ts2_mat *srcGrad, int32_t srcGradType, int32_t add, void *stream);

/* BackpropDelta: delta[gradDim][srcDim] = alpha * (*gradScale) * sum_t grad[t][k]*src[t][x] as the packed delta (i8 + tileScale
 * [srcDim/128][gradDim], TCudaPackedDeltaMatrix, src/gpt/matrix/delta_cuda.h:9-38).  src is the 8-bit layer input
 * [lenRound][srcDim]; I8: grad (TS2_BF16 | TS2_F32) is requantised per kTile rows (times srcRowScale[t] if given);
 * E4M3: grad is e4m3 and only transposed. */
int ts2_matmul_backprop_delta(int32_t mode, int32_t len, int32_t lenRound, int32_t srcDim, int32_t gradDim, const ts2_mat *src,
    const float *srcRowScale, const ts2_mat *grad, int32_t gradType, float alpha, const float *gradScale, int32_t kTile,
    const ts2_matmul_bwd_buffers *buf, const ts2_mat *delta, const ts2_mat *deltaTileScale, void *stream);

/* Forward product of the same operator, TMatMulBuffers::Forward<TStoreScaled> (layer_cuda_base.cuh:183-193):
 * res[len][dstDim] = alpha * (*alphaPtr) * src * W^T, src and W 8-bit of the same type, resType TS2_F32 | TS2_BF16. */
int ts2_matmul_forward(int32_t mode, int32_t len, int32_t lenRound, int32_t srcDim, int32_t dstDim, const ts2_mat *src,
    const ts2_mat *transformFast, float alpha, const float *alphaPtr, const ts2_mat *res, int32_t resType, int32_t add, void *stream);

/* Forward<TStoreRowTileNormalize> / Forward<TStoreRowTileNormalizeRope> of the same operator (store functors of
 * src/lib/cuda/cuda_matmul.cuh:495-525 and src/gpt/compute/gpu_rope.cuh:25-60): res (TS2_BF16) = rope(normalise(alpha * (*alphaPtr) *
 * src * W^T)), tileScale fp32 [dstDim/128][lenRound] when normalize.  Fused into the product's epilogue where the 256x256-tile kernel
 * applies (lenRound, dstDim multiples of 256, at least 192 tiles); otherwise the product goes to `raw` (fp32 [lenRound][dstDim]
 * scratch) and ts2_row_tile_normalize_rope finishes it. */
int ts2_matmul_forward_norm_rope(int32_t mode, int32_t len, int32_t lenRound, int32_t srcDim, int32_t dstDim, const ts2_mat *src,
    const ts2_mat *transformFast, float alpha, const float *alphaPtr, int32_t normalize, float vecScale, const ts2_mat *ropeBuf,
    const ts2_mat *res, const ts2_mat *tileScale, const ts2_mat *raw, void *stream);

/* ------------------------------------------------------------------------------------------------------------------------
 * Attention (head dimension 128 = Q_DIM = TT_DIM, src/gpt/compute/cfg_precision.h:79-80).  q, k, v, valLookup, dValLookup are
 * TS2_BF16 [lenRound][heads*128]; q and k already rotated (RoPE) and q, v head-normalised, as the reference stores them
 * (src/gpt/compute/layer_att.cu:108-143).  Spans: query row t attends key rows spanStart[t] .. spanFinish[t] inclusive
 * (finish < start = nothing); both arrays have lenRound entries and pad rows must be empty.  This covers every causal attention
 * type of src/gpt/att/sliding_window.cpp:111-118,226-240 (one span per row); the reference's general span groups
 * (TAttentionSpanGroup, src/gpt/att/att.h:86-121) are only needed by its cross-batch attention, which is out of scope.
 * logit = <q,k> * attDotScale - alibiSlope * (query row - key row); softmax base 2 with the implicit zero "sink" vector.
 * Stats: sumWeightLog fp32 [heads][lenRound] = max + log2(sum), dScale fp32 [heads][lenRound] (same stride).
 * Rows >= len of q/k/v/dValLookup must be finite (producers write zeros). */
typedef struct ts2_att_args {
    int32_t len, lenRound, heads;
    ts2_mat q, k, v;
    const int32_t *spanStart, *spanFinish;
    float attDotScale, alibiSlope;
    ts2_mat valLookup;    /* out */
    ts2_mat sumWeightLog; /* out */
} ts2_att_args;

/* Fp16Att, src/gpt/compute/gpu_att_fp16.cu:41-215 */
int ts2_att_forward(const ts2_att_args *args, void *stream);

typedef struct ts2_att_grad_args {
    int32_t len, lenRound, heads;
    ts2_mat q, k, v, dValLookup;
    const int32_t *spanStart, *spanFinish;
    const int32_t *revLo, *revHi; /* [lenRound/128] from ts2_att_build_rev */
    float attDotScale, alibiSlope;
    ts2_mat sumWeightLog, dScale; /* in */
    ts2_mat dQ, dK, dV;           /* out, gradType = TS2_BF16 | TS2_F32 */
    int32_t gradType;
    int32_t which; /* bit 0: dQ (Fp16AttGradQ), bit 1: dK and dV (Fp16AttGradKV) */
    /* optional, all three or none, used when which == 3: the score gradients dS leave the dK/dV kernel as 32 x 32 bf16 blocks (2 KB
     * each) in dsScratch and dQ is a single product over them instead of a second evaluation of S and dP (5 products per backward
     * instead of 7).  dsBase: [lenRound + 1] from ts2_att_build_ds_index on the same spans; dsScratch: 16-byte aligned,
     * dsCapacityBlocks blocks of 2048 bytes, at least heads * ts2_att_ds_blocks(spans) (blocks beyond the capacity are dropped:
     * wrong gradients for those rows, no access outside the array).  Without them the kernels of the two bits run independently. */
    const int32_t *dsBase;
    void *dsScratch;
    int64_t dsCapacityBlocks;
} ts2_att_grad_args;

/* Fp16AttGradQ + Fp16AttGradKV, src/gpt/compute/gpu_att_fp16.cuh:60-358 (their norm/rope epilogues are
 * ts2_backprop_row_tile_normalize_rope below) */
int ts2_att_backward(const ts2_att_grad_args *args, void *stream);

/* Transposed span graph reduced to what the dK/dV kernel needs: per block of 128 key rows the first and last query row whose
 * span touches it (replaces TransposeAttention + GroupAttention on the host, src/gpt/att/att.cpp:25-55, att.h:125-211). */
int ts2_att_build_rev(int32_t len, int32_t lenRound, const int32_t *spanStart, const int32_t *spanFinish, int32_t *revLo, int32_t *revHi,
    void *stream);
/* Numbering of the blocks of score gradients that ts2_att_backward can hand from its dK/dV kernel to its dQ kernel (no counterpart in
 * the reference, whose two kernels each evaluate the scores): a block exists for every (32-query block, 32-key block) pair such that
 * the key block lies between the earliest span start and the latest span finish of the query block's rows.  dsBase[q] = number of
 * the first block of q's query block, dsBase[lenRound] = blocks per head; device arrays, spans of lenRound rows (empty: finish <
 * start).  ts2_att_ds_blocks counts the blocks per head on the host from host copies of the same spans (to size the array). */
int ts2_att_build_ds_index(int32_t lenRound, const int32_t *spanStart, const int32_t *spanFinish, int32_t *dsBase, void *stream);
int64_t ts2_att_ds_blocks(int32_t lenRound, const int32_t *spanStartHost, const int32_t *spanFinishHost);

/* TStoreRowTileNormalize / TStoreRowTileNormalizeRope as a stand-alone pass (src/lib/cuda/cuda_matmul.cuh:495-525,
 * src/gpt/compute/gpu_rope.cuh:25-60): per row and 128-wide head: v = src*srcMult; if normalize: scale = rms(v)*vecScale
 * (stored in tileScale[head][row], 0 for zero tiles) and v /= scale; if ropeBuf (fp32 [lenRound][128] = cos,sin pairs of
 * src/gpt/att/rope.cpp:14-22): rotate pairs by +1; store as TS2_BF16; rows in [len, lenRound) are cleared. */
int ts2_row_tile_normalize_rope(int32_t len, int32_t lenRound, const ts2_mat *src, int32_t srcType, float srcMult, int32_t normalize,
    float vecScale, const ts2_mat *ropeBuf, const ts2_mat *dst, const ts2_mat *tileScale, void *stream);

/* TStoreAttBackNormalizeRope / TStoreAttBackNormalize / TStoreAttBackRope, src/gpt/compute/gpu_att_utils.cuh:280-352: per row
 * and head: g = grad*gradMult; if srcNorm: tile-norm backward against srcNorm*srcTileScale (the stored normalised, rotated
 * vector); if ropeBuf: rotate pairs by -1; store as dstType (TS2_BF16 | TS2_E4M3 | TS2_F32); rows in [len, lenRound) cleared. */
int ts2_backprop_row_tile_normalize_rope(int32_t len, int32_t lenRound, const ts2_mat *grad, int32_t gradType, float gradMult,
    const ts2_mat *srcNorm, const ts2_mat *srcTileScale, const ts2_mat *ropeBuf, const ts2_mat *dst, int32_t dstType, void *stream);

/* ------------------------------------------------------------------------------------------------------------------------
 * Mixture of experts (src/gpt/compute/layer_moe.cu, moe_kernels.cu, moe_kernels.cuh).  Tables, all device-resident and
 * caller-owned, named as in the reference (layer_moe.cu:82-89):
 *   sampleExpertIds / sampleExpertWeights / sampleExpertOffset [len*selected]   per (token, slot)
 *   expertOffset [experts+2]   first grouped row of each expert (multiples of 128); [experts] = rows in use; [experts+1] = lenMoe
 *   xpTileExpertId [lenMoe/128]   expert of each 128-row tile, -1 for the unused tail
 *   xpSampleId [lenMoe] token of each grouped row (-1 = padding), xpSampleWeight [lenMoe] its routing weight
 * lenMoe is the capacity of the grouped buffers: at least len*selected + 128*experts, a multiple of 128. */
typedef struct ts2_moe_tables {
    int32_t *sampleExpertIds;
    float *sampleExpertWeights;
    int32_t *sampleExpertOffset;
    int32_t *expertOffset;
    int32_t *xpTileExpertId;
    int32_t *xpSampleId;
    float *xpSampleWeight;
    int32_t *blockCounts; /* scratch: [ceil(len*selected/256)][experts] */
} ts2_moe_tables;

/* MoeCalcSampleExpertLists + GroupPerExpertLists + InitXpTables + FillXpTables (moe_kernels.cu:54-225): top-`selected` logits
 * per token (ties: lowest index), w = exp((s - max)/2) scaled so that sum w^2 = experts; grouped rows are ordered by
 * (expert, token, slot) — deterministic, where the reference's order within an expert depends on atomics.
 * select: TS2_BF16 | TS2_F32 [len][>= experts]. */
int ts2_moe_route(int32_t len, int32_t lenMoe, int32_t experts, int32_t selected, const ts2_mat *select, int32_t selectType,
    const ts2_moe_tables *tables, void *stream);

/* ts2_moe_route for callers that cannot allocate and have no workspace to hand over (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same tables and same results as ts2_moe_route; the
 * counting sort's scratch (tables->blockCounts there, ignored here and may be NULL) is a fixed device array inside the library:
 * TS2_MOE_ROUTE_STATIC_INTS ints (512 KiB) held by every GPU the library runs on until the process ends.  A call needs
 * ceil(len*selected/256) * experts <= TS2_MOE_ROUTE_STATIC_INTS (e.g. 65536 tokens, top-2, 64 experts: 32768) and returns TS2_ERR_SHAPE
 * beyond that.  The call allocates and frees nothing.  All calls on one GPU share that GPU's array: calls that may overlap on one GPU
 * (different streams, different host threads) race and must be ordered by the caller.
 * The first call on a device also resolves the array's address there and sets a kernel's LDS attribute; neither is a stream
 * operation and neither belongs under stream capture.  ts2_device_info (and with it ts2_model_create) does both for the current
 * device: call one of them, or make one eager call of this entry point, on each device before a capture that contains it. */
#define TS2_MOE_ROUTE_STATIC_INTS 131072
int ts2_moe_route_static(int32_t len, int32_t lenMoe, int32_t experts, int32_t selected, const ts2_mat *select, int32_t selectType,
    const ts2_moe_tables *tables, void *stream);

/* MoeGroupSamples (moe_kernels.cuh:89-143): dst[row] = src[xpSampleId[row]] (zeros for padding) for row < lenMoe; elemSize 1 or 2
 * bytes.  The transposed copy the reference can emit is ts2_transpose_quant with rowIndex = xpSampleId. */
int ts2_moe_group_samples(int32_t lenMoe, int32_t elemSize, const ts2_mat *src, const int32_t *xpSampleId, const ts2_mat *dst, void *stream);

/* MatrixLoLUmoe (moe_kernels.cuh:15-44): res = vals * sigmoid(2*gate) * xpSampleWeight[row] * resMult over grouped rows */
int ts2_matrix_lolu_moe(int32_t lenMoe, const float *xpSampleWeight, const ts2_mat *gate, const ts2_mat *vals, float resMult,
    const ts2_mat *res, int32_t resType, void *stream);

/* BackpropRowTileNormalizeLoLUmoe (moe_kernels.cu:229-302): the FFN gate/norm backward over grouped rows, with the routing
 * weight folded in and dExpertWeight[row] = sum_x grad*vals*sigmoid(2 gate) */
int ts2_backprop_row_tile_normalize_lolu_moe(int32_t lenMoe, const float *xpSampleWeight, const ts2_mat *gate, const ts2_mat *vals,
    float valsScale, const ts2_mat *valsSrcTileScale, const ts2_mat *grad, int32_t gradType, float gradMult, const ts2_mat *gradGate,
    const ts2_mat *gradVals, int32_t gradOutType, float *dExpertWeight, void *stream);

/* BackpropMoeKernel (moe_kernels.cu:306-355): routing backward per token -> dMoeSelect [lenRound][dMoe->x] (TS2_F32 | TS2_BF16 | TS2_E4M3), columns
 * >= experts and rows >= len cleared */
int ts2_backprop_moe(int32_t len, int32_t lenRound, int32_t experts, int32_t selected, const ts2_moe_tables *tables,
    const float *dExpertWeight, const ts2_mat *dMoe, int32_t dMoeType, void *stream);

/* CombineExperts (moe_kernels.cuh:146-177): res[t] (op)= alpha * (*alphaPtr) * sum over the token's `selected` grouped rows of
 * src; src TS2_BF16 | TS2_F32 [lenMoe][dim], res TS2_F32 [len][dim]; add != 0 accumulates (TStoreAdd) */
int ts2_combine_experts(int32_t len, int32_t selected, const ts2_mat *src, int32_t srcType, const ts2_moe_tables *tables, float alpha,
    const float *alphaPtr, const ts2_mat *res, int32_t add, void *stream);

/* Batched byte transpose: batch slabs of [rows][cols] -> [cols][rows] (MoeTransposeI8Kernel, src/gpt/compute/moe_matmul.cu:9-19);
 * rows and cols multiples of 128 */
int ts2_transpose_u8_batched(int32_t batch, int32_t rows, int32_t cols, const void *src, int64_t srcStride, int64_t srcSlabBytes, void *dst,
    int64_t dstStride, int64_t dstSlabBytes, void *stream);

/* ------------------------------------------------------------------------------------------------------------------------
 * Optimiser apply on the device (src/gpt/matrix/agpu_cuda.cuh, agpu_cuda.cu; CPU twin THostModelMatrix::AddDelta,
 * src/gpt/matrix/host_matrix.cpp:112-145): packed delta -> row-normalised moving average -> fp32 master weights -> fast weights.
 * Matrices are [ySize = out][xSize = in], xSize a multiple of 128; every array is device-resident and caller-owned. */

/* TAddGradientKernelParams (agpu_cuda.cuh:19-27), device-resident like the reference's CudaAGParams so that a captured sequence of launches
 * follows a changing learning rate; stepMult = TTrainingStep::Rate (src/gpt/train_config/train_step.h:4-27). */
typedef struct ts2_add_gradient_params {
    float dispDecay, beta1, weight0, weight1, l2Reg, stepMult;
} ts2_add_gradient_params;

/* UnpackDeltaKernel<ADD_TO_TARGET>, agpu_cuda.cuh:35-49: dst[y][x] (+)= delta[y][x] * tileScale[x/128][y] */
int ts2_unpack_delta(int32_t xSize, int32_t ySize, const ts2_mat *delta, const ts2_mat *tileScale, const ts2_mat *dst, int32_t addToTarget,
    void *stream);
/* MatrixRowSum2Kernel, agpu_cuda.cu:33-52: sum2arr[y] = sum_x matr[y][x]^2 */
int ts2_matrix_row_sum2(int32_t xSize, int32_t ySize, const ts2_mat *matr, float *sum2arr, void *stream);
/* the same row sums taken from a packed delta without expanding it (UnpackDeltaKernel<0> + MatrixRowSum2Kernel in one pass over the bytes) */
int ts2_packed_delta_row_sum2(int32_t xSize, int32_t ySize, const ts2_mat *delta, const ts2_mat *tileScale, float *sum2arr, void *stream);
/* UpdateGlobalRowDisp, agpu_cuda.cu:60-109: sumWeight = sumWeight * dispDecay + 1; per block of ySize / rowDispSize rows
 * rowDisp = rowDisp * dispDecay + mean square of the block's delta; rowScale[y] = 1 / sqrt(rowDisp / sumWeight) (0 when that is 0) */
int ts2_update_global_row_disp(int32_t xSize, int32_t ySize, int32_t rowDispSize, const float *deltaSum2arr, const ts2_add_gradient_params *params,
    float *sumWeight, float *rowDisp, float *rowScale, void *stream);
/* AddGradientKernel, agpu_cuda.cu:112-139: d = grad * rowScale[y]; avgGrad = avgGrad * beta1 + d * (1 - beta1);
 * weights = weights * (1 - step * l2Reg) + (avgGrad * weight1 + d * weight0) * step with step = stepMult * sqrt(*sparsity);
 * weightsRowSum2[y] = sum_x weights[y][x]^2 */
int ts2_add_gradient(int32_t xSize, int32_t ySize, const ts2_mat *grad, const ts2_add_gradient_params *params, const float *rowScale,
    const float *sparsity, const ts2_mat *avgGrad, const ts2_mat *weights, float *weightsRowSum2, void *stream);
/* ConvertMatrixKernel, agpu_cuda.cuh:65-101: *matrixScale = sko = sqrt(sum(sum2arr[0..totalYSize)) / (totalXSize * totalYSize));
 * fast = cvt(weights * 32 / sko) as fastType (TS2_I8 | TS2_E4M3 | TS2_BF16), all zero for a zero matrix; rows ySize .. yBufSize cleared.
 * convertMult: one float of scratch. */
int ts2_convert_matrix(int32_t xSize, int32_t ySize, int32_t yBufSize, int32_t totalXSize, int32_t totalYSize, const ts2_mat *weights,
    const float *sum2arr, const ts2_mat *fast, int32_t fastType, float *matrixScale, float *convertMult, void *stream);

/* device state of one matrix = the members of TAgpuCudaModelMatrix (agpu_cuda.cuh:343-360,431-470) on one device */
typedef struct ts2_opt_matrix {
    int32_t xSize, ySize, yBufSize; /* yBufSize: rows of `fast` (ySize rounded up to 128) */
    int32_t rowDispSize;            /* divides ySize: rows per dispersion estimate = ySize / rowDispSize (GetRowDispSize) */
    ts2_mat weights, avgGrad;       /* fp32 [ySize][xSize]: Weights, AvgGrad */
    ts2_mat grad;                   /* fp32 [ySize][xSize]: Grad, the accumulator over micro-batches; may be empty when every delta is
                                       applied at once (TS2_BM_GRAD_APPLY without TS2_BM_GRAD_ADD) */
    float *gradRowSum2, *weightsRowSum2, *rowScale; /* [ySize] */
    float *rowDisp;                 /* [rowDispSize] */
    float *sumWeight, *sparsity;    /* [1] each */
    ts2_mat fast;                   /* FastDevice [yBufSize][xSize] of fastType */
    int32_t fastType;
    float *matrixScale;             /* [1]: MatrixScale (GetScale) */
    float *convertMult;             /* [1] scratch */
} ts2_opt_matrix;

enum { TS2_BM_GRAD_ADD = 1, TS2_BM_GRAD_APPLY = 2 }; /* EBackpropMode bits, src/gpt/matrix/base_cuda.cuh */

/* TAgpuCudaModelMatrix::Convert, agpu_cuda.cuh:412-428 (after the master weights were set: CopyToDevice) */
int ts2_opt_convert(const ts2_opt_matrix *m, void *stream);
/* TAgpuCudaModelMatrix::AddDelta(TCudaPackedDeltaMatrix&, bm) with ApplyGradientImpl, agpu_cuda.cuh:484-590, on one device (its
 * all-reduces over devices drop out): backpropMode = TS2_BM_GRAD_ADD adds the delta to `grad`, otherwise it replaces it;
 * TS2_BM_GRAD_APPLY then updates the dispersion estimates, the moving average, the weights and the fast weights.  APPLY without ADD
 * reads the packed bytes directly: `grad` is neither read nor written and may be an empty ts2_mat.  The reference leaves the unpacked
 * delta in Grad on that path too (UnpackDeltaKernel<0>, agpu_cuda.cuh:579-585); here `grad` holds valid data only after a call with
 * TS2_BM_GRAD_ADD or one without TS2_BM_GRAD_APPLY, so a caller that reads it, or mixes this call with ts2_unpack_delta /
 * ts2_add_gradient on the same state, must use one of those. */
int ts2_opt_add_delta(const ts2_opt_matrix *m, const ts2_mat *delta, const ts2_mat *tileScale, int32_t backpropMode,
    const ts2_add_gradient_params *params, void *stream);

/* ------------------------------------------------------------------------------------------------------------------------
 * Layer stack and one-GPU step driver: the counterpart of TCudaLayerBase::{AddForward, AddBackward}
 * (src/gpt/compute/layer_cuda_base.cuh:290-294) and of the executor's forward/backprop graphs
 * (src/gpt/compute/gpu_transformer.cu:260-471; IModelImpl::Backprop, src/gpt/compute/model.h:60-67).
 * The model object owns its device memory (allocated once at creation, like the reference's pools); the per-step entry points
 * allocate nothing.  Weights are handed over already quantised (fast bytes + matrix scale), exactly what the reference's
 * ICudaModelMatrixBase<T>::GetFast/GetScale expose (src/gpt/matrix/base_cuda.cuh:19-43). */
typedef struct ts2_model ts2_model;

enum { TS2_LT_ATT = 0, TS2_LT_FFN = 2, TS2_LT_MOE = 3 }; /* ELayerType, src/gpt/model_params/model_dim.h:57-62 */
#define TS2_LAYER_EMBED (-1)
#define TS2_LAYER_FINAL (-2)

typedef struct ts2_model_config {
    int32_t mode; /* TS2_I8: i8 weights/states, bf16 fast gradients; TS2_E4M3: e4m3 weights/states/fast gradients */
    int32_t dim, headCount, ffnDim, expertDim, expertCount, moeSelected; /* TModelDims, model_dim.h:118-141 (head dim 128) */
    int32_t depth;                                                       /* number of layers */
    const int32_t *layerType;                                            /* [depth] TS2_LT_* */
    const int32_t *layerAttId;                                           /* [depth] attention type of attention layers */
    const float *layerSlope;                                             /* [depth] ALiBi slope */
    int32_t attTypeCount;
    int32_t vocab, labelCount, maxLen;
    int32_t kTile; /* rows sharing one scale in the int8 delta GEMM (0 = 512) */
    /* 0: every FFN and attention layer keeps what its forward pass computed for its backward pass when that fits into half of the
     * free device memory; 1: the backward recomputes it, as the reference's AddBackward does (layer_ffn.cu:83-113, layer_att.cu:160-226) */
    int32_t recompute;
    /* != 0 (TS2_I8 models): the int8 quantisers of every linear backward dither (ts2_matmul_bwd_buffers.ditherSeed), each call under a
     * seed of its own derived from this one and a call counter; 0: round to nearest */
    uint32_t ditherSeed;
} ts2_model_config;

/* Host helpers for setting a model up (no device work).
 * ts2_model_schedule: the layer list a model depth stands for - InitAlibi, src/gpt/model_params/model_dim.cpp:82-158 (the ALIBI_V3
 *   branch every model string of the reference selects): attention types {1, 64, wideWindow} (depth 1: the single-attention profiling
 *   case), layers as (type, attention type, ALiBi slope).  moeExpertCount > 0 makes the MLPs behind the first groups MoE layers.
 *   Returns the number of layers written (<= maxLayers, else TS2_ERR_SHAPE); attWidth must hold 3 entries.
 * ts2_fill_rope_buf: the (cos, sin) table fp32 [ropeLen][width] of FillRopeBuf, src/gpt/att/rope.cpp:4-38 (theta 5e5), host memory. */
int ts2_model_schedule(int32_t depth, int32_t moeExpertCount, int32_t wideWindow, int32_t maxLayers, int32_t *layerType, int32_t *layerAttId,
    float *layerSlope, int32_t *attWidth, int32_t *attTypeCount);
int ts2_fill_rope_buf(float *buf, int32_t width, int32_t ropeLen);

ts2_model *ts2_model_create(const ts2_model_config *cfg);
void ts2_model_destroy(ts2_model *m);
/* matrixId: MP_ATT_{Q,K,V,GATE,COMBINER} = 0..4, MP_FFN_{EXPAND,GATE,CONTRACT} = 0..2, MP_MOE_{EXPAND,GATE,CONTRACT,SELECT} = 0..3
 * (model_dim.h:65-80); fastHost is [rows][cols] bytes of the model's 8-bit type, scale the matrix scale. */
int ts2_model_set_matrix(ts2_model *m, int32_t layer, int32_t matrixId, const void *fastHost, int32_t rows, int32_t cols, float scale);
int ts2_model_set_bias(ts2_model *m, const float *biasHost);
/* Optimiser state of the step driver (optional).  ts2_model_set_master gives a matrix fp32 master weights [rows][cols] (rows without the
 * tile padding), a dispersion granularity (rowDispSize = rows: per row, 1: per matrix; SetSizesPerRowDisp / SetSizesPerMatrixDisp,
 * src/gpt/model_params/model_matrix.h:116-127) and its sparsity factor, and derives the fast weights and the matrix scale from them on the
 * device (CopyToDevice + Convert, src/gpt/matrix/agpu_cuda.cuh:412-428,473-482).  ts2_model_apply_deltas runs one optimiser step
 * (ts2_opt_add_delta with TS2_BM_GRAD_APPLY) over every such matrix with the deltas of the last ts2_model_backprop; matrices without
 * master weights keep theirs.  paramsHost is a host struct.  ts2_model_get_master / ts2_model_get_matrix read weights back. */
int ts2_model_set_master(ts2_model *m, int32_t layer, int32_t matrixId, const float *weightsHost, int32_t rows, int32_t cols, int32_t rowDispSize,
    float sparsity);
int ts2_model_apply_deltas(ts2_model *m, const ts2_add_gradient_params *paramsHost, void *stream);
int ts2_model_get_master(ts2_model *m, int32_t layer, int32_t matrixId, float *hostOut, int32_t rows, int32_t cols);
int ts2_model_get_matrix(ts2_model *m, int32_t layer, int32_t matrixId, void *fastHostOut, int32_t rows, int32_t cols, float *scaleOut);
/* nodes of one batch (TBatchNodes, src/gpt/att/nodes_batch.h:42-57): label CSR, target token per row (-1 = none), one span per
 * row and attention type, RoPE table [len][128]; host arrays */
int ts2_model_set_batch(ts2_model *m, int32_t len, const int32_t *labelPtr, const uint32_t *labels, const int32_t *targetPerRow,
    const int32_t *const *spanStart, const int32_t *const *spanFinish, const float *ropeBuf, void *stream);
/* The checks ts2_model_set_batch makes before it copies anything, as a host-only function (no device access): label CSR monotone from 0
 * and within labelCap, label ids (low 31 bits; bit 31 is the sign of the embedding term, src/gpt/compute/cpu_transformer.cpp:76-100) below
 * labelCount, -1 <= target < vocab, and for every attention type and row 0 <= start <= len and -1 <= finish < len (finish < start = empty).  The
 * reference trusts its own node builder (InitLabelData, src/gpt/att/sliding_window.cpp:269-306); a caller-supplied batch that breaks one
 * of these would be an out-of-bounds access on the device, so it is refused with TS2_ERR_SHAPE / TS2_ERR_NULL instead.
 * ts2_model_set_batch, ts2_model_set_matrix and ts2_model_set_bias copy with blocking copies on the null stream; set_batch waits for
 * `stream` first, so a step still running there cannot see a half-written batch. */
int ts2_validate_batch(int32_t len, int32_t labelCap, int32_t labelCount, int32_t vocab, int32_t attTypeCount, const int32_t *labelPtr,
    const uint32_t *labels, const int32_t *targetPerRow, const int32_t *const *spanStart, const int32_t *const *spanFinish);
int ts2_model_forward(ts2_model *m, void *stream);  /* states + predictions ("prediction" array holds probabilities) */
int ts2_model_backprop(ts2_model *m, void *stream); /* forward, loss gradient, backward through all layers, every delta */
/* one layer in isolation on the model's buffers ("state" in, "state" out / "stateGrad" in-out) */
int ts2_layer_forward(ts2_model *m, int32_t layer, void *stream);
int ts2_layer_backward(ts2_model *m, int32_t layer, void *stream);
/* dequantised delta of a matrix into hostOut [rows][cols] (synchronises the device) */
int ts2_model_get_delta(ts2_model *m, int32_t layer, int32_t matrixId, float *hostOut, int32_t rows, int32_t cols);
/* device view of an internal array: "state", "stateGrad", "stateGradFast", "dNormState", "prediction", "normState"[i], "stateScale"[i],
 * "expertOffset" (TS2_I32 [1][experts+2], MoE models: the routing of the last MoE layer that ran), "gradMaxNorm" (fp32 [1][depth+2]: the
 * running maxima of |stateGrad|; ts2_layer_backward derives its gradient multiplier from element 0, which a caller that sets stateGrad
 * itself must set to its abs-max), "finalGrad" (bf16 [lenRound][vocab]: the soft-max gradient of the last ts2_model_backprop).
 * For tests that compare a layer's interior: "act.a0".."act.a3", "act.scale0", "act.scale1", "act.rg", "act.val", "act.swl" with index =
 * layer: what that layer keeps from its forward pass (FFN: wide, gate, wide's tile scales, rg; attention: q, gate, k, v, q's and v's
 * scales, the attention output - overwritten with dQ by the layer's backward -, vlg, the soft-max statistics); "scratch.g0".."scratch.g3",
 * "scratch.f0".."scratch.f3", "scratch.dscale" with index = number of columns: the gradient scratch of the layer backward that ran last
 * (bf16: drg / dvlg, dVal, dK, dV; fast-gradient type: dwide / dq, dgate, dk, dv). */
int ts2_model_array(ts2_model *m, const char *name, int32_t index, ts2_mat *out, int32_t *type);
/* host copy of the same arrays, rows packed ([y][x] elements); synchronises the device */
int ts2_model_read(ts2_model *m, const char *name, int32_t index, void *hostOut, int64_t hostBytes);
int ts2_model_scalars(ts2_model *m, float *lossSumHost, int32_t *lenRound, int32_t *lenMoe);

/* ------------------------------------------------------------------------------------------------------------------------
 * Checkpoint and weight-exchange formats (host side; no device work).
 * ts2_checkpoint_parse reads the bytes of a TModelParams as the reference's SAVELOAD writes them (src/gpt/model_params/model_params.h:7-18,
 * model_matrix.h:61-70, model_dim.h:118-178 through src/util/bin_saver.h) and returns NULL when they do not parse exactly;
 * ts2_checkpoint_write produces the same bytes again (returns the byte count, also when out is NULL or cap too small: nothing beyond
 * cap is written).  Matrices: layer = -1 addresses the model-level ones (0 = embedding MP_MODEL_EMBED, 1 = final MP_MODEL_FINAL,
 * model_dim.h:84-86), otherwise a layer's in the order of EnumLayerMatrices (model_dim.h:225-262).  The views point into the
 * checkpoint object and live as long as it does; weights / avgGrad are [ySize][xSize] floats (Matr, Grad1), rowDispSize is 1 or ySize. */
typedef struct ts2_checkpoint ts2_checkpoint;
typedef struct ts2_checkpoint_info {
    int32_t dim, qDim, ttDim, expertDim, headCount, ffnTiles, moeExpertCount, moeSelected, kvRep, depth; /* TModelDims */
    int64_t labelCount, inputTokenCount, outputTokenCount;
    int32_t attTypeCount, layerCount;
    uint64_t flags, docStartToken;
    int64_t fragLen;
    int32_t biasCount;
    const float *bias;
} ts2_checkpoint_info;
typedef struct ts2_checkpoint_matrix_view {
    int32_t xSize, ySize;
    const float *weights, *avgGrad;
    float sumWeight;
    const float *rowDisp;
    int32_t rowDispSize;
    float sparsity;
} ts2_checkpoint_matrix_view;
ts2_checkpoint *ts2_checkpoint_parse(const void *bytes, int64_t size);
void ts2_checkpoint_free(ts2_checkpoint *c);
int64_t ts2_checkpoint_write(const ts2_checkpoint *c, void *out, int64_t cap);
int ts2_checkpoint_get_info(const ts2_checkpoint *c, ts2_checkpoint_info *out);
int ts2_checkpoint_att_type(const ts2_checkpoint *c, int32_t id, int32_t *width, int32_t *type);
int ts2_checkpoint_layer(const ts2_checkpoint *c, int32_t layer, int32_t *layerType, float *alibiSlope, int32_t *attTypeId, int32_t *matrixCount);
int ts2_checkpoint_matrix(const ts2_checkpoint *c, int32_t layer, int32_t matrixId, ts2_checkpoint_matrix_view *out);
/* PackMatrix / AddPackedMatrix, src/gpt/model_params/model_matrix.cpp:6-58: the fp16-row format in which weights travel between
 * workers: per row a float rms, then (unless it is 0) xSize IEEE halves of row / rms; xSize a multiple of 16.
 * ts2_pack_matrix_fp16 returns the byte count (also when out is NULL or cap too small); ts2_add_packed_matrix_fp16 adds scale * matrix. */
int64_t ts2_pack_matrix_fp16(const float *matr, int32_t xSize, int32_t ySize, void *out, int64_t cap);
int ts2_add_packed_matrix_fp16(float *matr, int32_t xSize, int32_t ySize, const void *in, int64_t size, float scale);

/* CU count and nominal clock of the current device.  Also the library's per-device set-up call: it resolves what
 * ts2_moe_route_static would otherwise resolve on its first call on this device (see there). */
int ts2_device_info(int *cuCount, int *clockMHz);

const char *ts2_version(void);

#ifdef __cplusplus
}
#endif
#endif
