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
    TS2_I32 = 4
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
    TS2_EPI_ROW_TILE_MAXNORM = 2 /* TStoreRowTileMaxNormalize    :530-559  packed delta: i8 + TileScale[n/128][m] */
};

/*
 * C[m][n] (op)= alpha * (*alphaPtr) * rowScale[m] * sum_k A[m][k] * B[n][k]
 * Both operands K-contiguous — the contract of every GEMM core of the reference:
 *   Int8MatMulKernel / Int8MatMulKernelRowScale / Int8MatMulYScaleKernel  src/lib/cuda/cuda_i8.cuh:157-320
 *   GenericMatMulKernel (fp8, fp16)                                        src/lib/cuda/cuda_matmul.cuh:396-416
 * abType: TS2_I8 (int32 accumulate, exact), TS2_E4M3 or TS2_BF16 (fp32 accumulate).
 * cType : TS2_F32, TS2_BF16, TS2_I32 (raw accumulator, TS2_I8 inputs and TS2_EPI_STORE only) or TS2_I8 (ROW_TILE_MAXNORM).
 * rowScale  (optional, [m])  : per-row scale of A applied to the accumulator before the epilogue (the dX kernel).
 * kTileScale (optional, [k/kTile], TS2_I8 only): one scale per kTile contraction rows; each tile's int32 sum is exact and
 *             tiles are added in fp32 in tile order (the dW kernel).  kTile must be a multiple of 128.
 * splitK    : >1 splits the contraction over workgroups; partial sums are added with fp32 atomics (TS2_EPI_ADD semantics on a
 *             C the caller has zeroed, or TS2_EPI_STORE with the library zero-filling first).  1 = deterministic.
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
    int32_t tileConfig; /* 0 = choose; 1 = 256x256 workgroup tile; 2 = 128x128 */
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

/* BackpropLoLUdScale, src/gpt/compute/gpu_lolu.cuh:141-173 (attention): gate backward plus dScale[head][t] = <vals*valsScale,
 * gradVals> per 128-wide head. */
int ts2_backprop_lolu_dscale(int32_t len, int32_t lenRound, const ts2_mat *gate, const ts2_mat *vals, float valsScale, const ts2_mat *grad,
    int32_t gradType, const ts2_mat *gradGate, int32_t gradGateType, const ts2_mat *gradVals, int32_t gradValsType, const ts2_mat *dScale,
    void *stream);

/* NormalizeVecsRowMaxKernel, src/gpt/compute/row_scale.cuh:12-43, deterministic (the reference adds a random dither before rounding):
 * per row scale = maxabs/127, dst = sat_i8(rne(src/scale)); optional colScale[x] multiplies the source first; rows >= len cleared. */
int ts2_normalize_vecs_row_max(int32_t len, int32_t lenRound, const ts2_mat *src, int32_t srcType, const float *colScale,
    const ts2_mat *dst, float *rowScale, void *stream);

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
 * Differences from the reference, by design: no random dither in the int8 quantisers, no sort of the rows (each kTile
 * consecutive tokens share the delta GEMM's scale) and exact int32 sums per k-tile added in fp32. */
typedef struct ts2_matmul_bwd_buffers {
    ts2_mat grad8;
    float *grad8RowScale;
    ts2_mat gradT;
    ts2_mat srcT;
    float *tileMax;
    float *tileScale;
    ts2_mat transformT;
} ts2_matmul_bwd_buffers;

/* BackpropMulti (prep of dX): I8: quantise grad (TS2_BF16 | TS2_F32, optionally times gradColScale[gradDim]) per row to
 * grad8/grad8RowScale and transpose the weight; E4M3: transpose the weight.  transformFast is [gradDim][srcDim]. */
int ts2_matmul_backprop_multi(int32_t mode, int32_t len, int32_t lenRound, int32_t srcDim, int32_t gradDim, const ts2_mat *transformFast,
    const ts2_mat *grad, int32_t gradType, const float *gradColScale, const ts2_matmul_bwd_buffers *buf, void *stream);

/* Backprop(): srcGrad[len][srcDim] (+)= alpha * (*alphaPtr) * grad * W.  I8 reads grad8/grad8RowScale from buf; E4M3 reads grad
 * (e4m3 [lenRound][gradDim]) directly.  srcGradType TS2_F32 | TS2_BF16; add != 0 accumulates (multi-source sum). */
int ts2_matmul_backprop(int32_t mode, int32_t len, int32_t lenRound, int32_t srcDim, int32_t gradDim, const ts2_mat *grad,
    const ts2_matmul_bwd_buffers *buf, float alpha, const float *alphaPtr, const ts2_mat *srcGrad, int32_t srcGradType, int32_t add,
    void *stream);

/* BackpropDelta: delta[gradDim][srcDim] = (*gradScale) * sum_t grad[t][k]*src[t][x] as the packed delta (i8 + tileScale
 * [srcDim/128][gradDim], TCudaPackedDeltaMatrix, src/gpt/matrix/delta_cuda.h:9-38).  src is the 8-bit layer input
 * [lenRound][srcDim]; I8: grad (TS2_BF16 | TS2_F32) is requantised per kTile rows (times srcRowScale[t] if given);
 * E4M3: grad is e4m3 and only transposed. */
int ts2_matmul_backprop_delta(int32_t mode, int32_t len, int32_t lenRound, int32_t srcDim, int32_t gradDim, const ts2_mat *src,
    const float *srcRowScale, const ts2_mat *grad, int32_t gradType, const float *gradScale, int32_t kTile,
    const ts2_matmul_bwd_buffers *buf, const ts2_mat *delta, const ts2_mat *deltaTileScale, void *stream);

/* Forward product of the same operator, TMatMulBuffers::Forward<TStoreScaled> (layer_cuda_base.cuh:183-193):
 * res[len][dstDim] = alpha * (*alphaPtr) * src * W^T, src and W 8-bit of the same type, resType TS2_F32 | TS2_BF16. */
int ts2_matmul_forward(int32_t mode, int32_t len, int32_t lenRound, int32_t srcDim, int32_t dstDim, const ts2_mat *src,
    const ts2_mat *transformFast, float alpha, const float *alphaPtr, const ts2_mat *res, int32_t resType, int32_t add, void *stream);

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
} ts2_att_grad_args;

/* Fp16AttGradQ + Fp16AttGradKV, src/gpt/compute/gpu_att_fp16.cuh:60-358 (their norm/rope epilogues are
 * ts2_backprop_row_tile_normalize_rope below) */
int ts2_att_backward(const ts2_att_grad_args *args, void *stream);

/* Transposed span graph reduced to what the dK/dV kernel needs: per block of 128 key rows the first and last query row whose
 * span touches it (replaces TransposeAttention + GroupAttention on the host, src/gpt/att/att.cpp:25-55, att.h:125-211). */
int ts2_att_build_rev(int32_t len, int32_t lenRound, const int32_t *spanStart, const int32_t *spanFinish, int32_t *revLo, int32_t *revHi,
    void *stream);

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

/* peak dense MFMA rate the library prices its kernels against, in T(FL)OP/s, and the CU count it tiles for */
int ts2_device_info(int *cuCount, int *clockMHz);
const char *ts2_version(void);

#ifdef __cplusplus
}
#endif
#endif
