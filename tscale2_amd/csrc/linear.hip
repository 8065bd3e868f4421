// Linear-layer backward operator: the call sequences of TMatMulBuffers (src/gpt/compute/layer_cuda_base.cuh:153-250) expressed
// over the kernels of this library.  Host code only; every step is enqueued on the caller's stream.
#include "common.h"
#include "internal.h"

namespace
{
bool Is8(int mode)
{
    return mode == TS2_I8 || mode == TS2_E4M3;
}
} // namespace

extern "C" int ts2_matmul_bwd_scratch_bytes(int32_t mode, int32_t lenRound, int32_t srcDim, int32_t gradDim, int32_t kTile, int32_t splits,
    int64_t out[9])
{
    if (!out) {
        return TS2_ERR_NULL;
    }
    if (!Is8(mode)) {
        return TS2_ERR_UNSUPPORTED;
    }
    if (kTile <= 0) {
        kTile = 512;
    }
    if (srcDim <= 0 || gradDim <= 0 || lenRound <= 0 || srcDim % 128 || gradDim % 128 || lenRound % 128 || kTile % 128 || splits < 0 ||
        (mode == TS2_I8 && lenRound % kTile)) {
        return TS2_ERR_SHAPE;
    }
    const int64_t L = lenRound, S = srcDim, G = gradDim, nTiles = (L + kTile - 1) / kTile;
    const bool i8 = mode == TS2_I8;
    out[0] = i8 ? L * G : 0;         // grad8
    out[1] = i8 ? L * 4 : 0;         // grad8RowScale
    out[2] = G * L;                  // gradT
    out[3] = S * L;                  // srcT
    out[4] = i8 ? nTiles * 4 : 0;    // tileMax
    out[5] = i8 ? nTiles * 4 : 0;    // tileScale
    out[6] = S * G;                  // transformT
    out[7] = splits > 1 ? (int64_t)splits * G * S * 4 : 0; // partial
    out[8] = i8 ? L * 4 : 0;         // gradRowAbsMax (optional)
    return TS2_OK;
}

extern "C" int ts2_matmul_backprop_multi(int32_t mode, int32_t len, int32_t lenRound, int32_t srcDim, int32_t gradDim,
    const ts2_mat *transformFast, const ts2_mat *grad, int32_t gradType, const float *gradColScale, const ts2_matmul_bwd_buffers *buf, void *stream)
{
    if (!transformFast || !buf) {
        return TS2_ERR_NULL;
    }
    if (!Is8(mode)) {
        return TS2_ERR_UNSUPPORTED;
    }
    if (srcDim % 128 || gradDim % 128 || lenRound % 128 || len > lenRound) {
        return TS2_ERR_SHAPE;
    }
    if (mode == TS2_I8) {
        if (!grad || !buf->grad8RowScale) {
            return TS2_ERR_NULL;
        }
        int rc = ts2_normalize_vecs_row_max_dither(len, lenRound, grad, gradType, gradColScale, &buf->grad8, buf->grad8RowScale, buf->gradRowAbsMax,
            buf->ditherSeed, stream);
        if (rc) {
            return rc;
        }
    }
    // W [gradDim][srcDim] -> W^T [srcDim][gradDim] so that the dX GEMM contracts over contiguous bytes
    if (buf->transformTValid) {
        return TS2_OK;
    }
    return ts2_transpose_quant(gradDim, gradDim, transformFast, mode, nullptr, nullptr, 0, nullptr, &buf->transformT, mode, nullptr, stream);
}

extern "C" int ts2_matmul_backprop(int32_t mode, int32_t len, int32_t lenRound, int32_t srcDim, int32_t gradDim, const ts2_mat *grad,
    const ts2_matmul_bwd_buffers *buf, float alpha, const float *alphaPtr, const ts2_mat *srcGrad, int32_t srcGradType, int32_t add, void *stream)
{
    if (!buf || !srcGrad) {
        return TS2_ERR_NULL;
    }
    if (!Is8(mode)) {
        return TS2_ERR_UNSUPPORTED;
    }
    ts2_gemm_args g = {};
    if (mode == TS2_I8) {
        g.a = buf->grad8;
        g.rowScale = buf->grad8RowScale;
    } else {
        if (!grad) {
            return TS2_ERR_NULL;
        }
        g.a = *grad;
    }
    g.b = buf->transformT;
    g.c = *srcGrad;
    g.abType = mode;
    g.cType = srcGradType;
    g.m = lenRound;
    g.n = srcDim;
    g.k = gradDim;
    g.mLive = len;
    g.alpha = alpha;
    g.alphaPtr = alphaPtr;
    g.epilogue = add ? TS2_EPI_ADD : TS2_EPI_STORE;
    g.splitK = 1;
    return ts2_gemm_nt(&g, stream);
}

extern "C" int ts2_matmul_backprop_group(int32_t mode, int32_t len, int32_t lenRound, int32_t srcDim, int32_t gradDim, int32_t count,
    const ts2_mat *const *grad, const ts2_matmul_bwd_buffers *const *bufs, const float *alpha, const float *const *alphaPtr,
    const ts2_mat *srcGrad, int32_t srcGradType, int32_t add, void *stream)
{
    if (!grad || !bufs || !alpha || !srcGrad || count < 1 || count > 4) {
        return TS2_ERR_NULL;
    }
    for (int i = 0; i < count; ++i) {
        if (!bufs[i] || (mode != TS2_I8 && !grad[i])) {
            return TS2_ERR_NULL;
        }
    }
    bool one = mode == TS2_E4M3 && count > 1 && (lenRound % 256) == 0 && (srcDim % 256) == 0 && (srcGradType == TS2_F32 || srcGradType == TS2_BF16);
    for (int i = 1; i < count && one; ++i) {
        one = grad[i]->strideBytes == grad[0]->strideBytes && bufs[i]->transformT.strideBytes == bufs[0]->transformT.strideBytes;
    }
    if (!one) {
        for (int i = 0; i < count; ++i) {
            int rc = ts2_matmul_backprop(mode, len, lenRound, srcDim, gradDim, grad[i], bufs[i], alpha[i], alphaPtr ? alphaPtr[i] : nullptr, srcGrad,
                srcGradType, add || i > 0, stream);
            if (rc) {
                return rc;
            }
        }
        return TS2_OK;
    }
    ts2_gemm_args g = {};
    g.a = *grad[0];
    g.b = bufs[0]->transformT;
    g.c = *srcGrad;
    g.abType = mode;
    g.cType = srcGradType;
    g.m = lenRound;
    g.n = srcDim;
    g.k = gradDim;
    g.mLive = len;
    g.alpha = alpha[0];
    g.alphaPtr = alphaPtr ? alphaPtr[0] : nullptr;
    g.epilogue = add ? TS2_EPI_ADD : TS2_EPI_STORE;
    g.splitK = 1;
    g.extraSegments = count - 1;
    for (int i = 1; i < count; ++i) {
        g.segment[i - 1].a = grad[i]->ptr;
        g.segment[i - 1].b = bufs[i]->transformT.ptr;
        g.segment[i - 1].alpha = alpha[i];
        g.segment[i - 1].alphaPtr = alphaPtr ? alphaPtr[i] : nullptr;
    }
    return ts2_gemm_nt(&g, stream);
}

extern "C" int ts2_matmul_backprop_delta(int32_t mode, int32_t len, int32_t lenRound, int32_t srcDim, int32_t gradDim, const ts2_mat *src,
    const float *srcRowScale, const ts2_mat *grad, int32_t gradType, float alpha, const float *gradScale, int32_t kTile, const ts2_matmul_bwd_buffers *buf,
    const ts2_mat *delta, const ts2_mat *deltaTileScale, void *stream)
{
    if (!buf || !src || !grad || !delta || !deltaTileScale) {
        return TS2_ERR_NULL;
    }
    if (!Is8(mode)) {
        return TS2_ERR_UNSUPPORTED;
    }
    int rc;
    bool kMajor = false;
    ts2_gemm_args g = {};
    if (mode == TS2_I8) {
        if (kTile <= 0 || kTile % 128 || lenRound % kTile || !buf->tileMax || !buf->tileScale) {
            return TS2_ERR_SHAPE;
        }
        if (buf->sortRows) {
            // the reference's order: rows sorted by their scale, gathered through the sorted list by both transposing passes
            if (!buf->gradRowAbsMax || !buf->gradRowAbsMaxValid || !buf->rowOrder || !buf->rowOrderTmp) {
                return TS2_ERR_NULL;
            }
            rc = ts2_sort_rows_by_scale(len, buf->gradRowAbsMax, srcRowScale, buf->rowOrder, buf->rowOrderTmp, stream);
            if (rc) {
                return rc;
            }
            rc = Ts2TransposeQuantRows(len, lenRound, grad, gradType, srcRowScale, nullptr, buf->gradRowAbsMax, kTile, buf->rowOrder, &buf->gradT,
                TS2_I8, buf->tileScale, stream, buf->ditherSeed);
        } else if (buf->gradRowAbsMax && buf->gradRowAbsMaxValid) {
            // the k-tile maxima follow from the row maxima of the dX pass: the transposing quantiser forms them itself
            rc = Ts2TransposeQuantRows(len, lenRound, grad, gradType, srcRowScale, nullptr, buf->gradRowAbsMax, kTile, nullptr, &buf->gradT, TS2_I8,
                buf->tileScale, stream, buf->ditherSeed);
        } else {
            rc = ts2_tile_absmax(len, grad, gradType, srcRowScale, kTile, buf->tileMax, 1, stream);
            if (rc) {
                return rc;
            }
            rc = ts2_transpose_quant_dither(len, lenRound, grad, gradType, srcRowScale, buf->tileMax, kTile, nullptr, &buf->gradT, TS2_I8, buf->tileScale,
                buf->ditherSeed, stream);
        }
        if (rc) {
            return rc;
        }
        g.kTileScale = buf->tileScale;
        g.kTile = kTile;
    } else {
        if (gradType != TS2_E4M3) {
            return TS2_ERR_UNSUPPORTED;
        }
        // both operands as they lie in memory, [token][feature]: the kernel's LDS reads do the transposing
        kMajor = (len == lenRound || buf->padRowsZero) && (gradDim % 256) == 0 && (srcDim % 256) == 0 && grad->y >= lenRound && src->y >= lenRound;
        if (!kMajor && !buf->gradTValid) {
            rc = ts2_transpose_quant(len, lenRound, grad, TS2_E4M3, nullptr, nullptr, 0, nullptr, &buf->gradT, TS2_E4M3, nullptr, stream);
            if (rc) {
                return rc;
            }
        }
    }
    const int *rowOrder = (mode == TS2_I8 && buf->sortRows) ? buf->rowOrder : nullptr;
    if (!kMajor && (!buf->srcTValid || rowOrder)) {
        rc = ts2_transpose_quant(len, lenRound, src, mode, nullptr, nullptr, 0, rowOrder, &buf->srcT, mode, nullptr, stream);
        if (rc) {
            return rc;
        }
    }
    g.a = kMajor ? *grad : buf->gradT;
    g.b = kMajor ? *src : buf->srcT;
    g.kMajor = kMajor ? 1 : 0;
    g.abType = mode;
    g.m = gradDim;
    g.n = srcDim;
    g.k = lenRound;
    const int splits = buf->partial.ptr ? buf->splits : 1;
    if (splits > 1) {
        // few output tiles: slices of the token axis as separate stored products on the large tile, then pack their sum
        int esz = 1;
        int64_t sliceBytes = ((int64_t)lenRound * esz / 128 + splits - 1) / splits * 128;
        bool ok = buf->partial.y >= splits * gradDim && buf->partial.x >= srcDim && (mode != TS2_I8 || sliceBytes % kTile == 0);
        if (!ok) {
            return TS2_ERR_SHAPE;
        }
        g.c = buf->partial;
        g.c.y = gradDim;
        g.cType = TS2_F32;
        g.alpha = 1.f;
        g.epilogue = TS2_EPI_STORE;
        g.splitK = splits;
        g.splitSlabBytes = (int64_t)gradDim * buf->partial.strideBytes;
        // int8: 256x128 tile with eight waves (the k-tile conversions of one wave run under the other's MFMAs)
        g.tileConfig = mode == TS2_I8 ? ((gradDim % 256) == 0 ? (3 | 8) : 2) : (((gradDim % 256) == 0 && (srcDim % 256) == 0) ? 1 : 2);
        rc = ts2_gemm_nt(&g, stream);
        if (rc) {
            return rc;
        }
        return ts2_pack_delta(&buf->partial, splits, g.splitSlabBytes, gradDim, srcDim, alpha, gradScale, delta, deltaTileScale, stream);
    }
    g.c = *delta;
    g.cType = TS2_I8;
    g.alpha = alpha;
    g.alphaPtr = gradScale;
    g.epilogue = TS2_EPI_ROW_TILE_MAXNORM;
    g.tileScale = *deltaTileScale;
    g.splitK = 1;
    return ts2_gemm_nt(&g, stream);
}

extern "C" int ts2_matmul_forward(int32_t mode, int32_t len, int32_t lenRound, int32_t srcDim, int32_t dstDim, const ts2_mat *src,
    const ts2_mat *transformFast, float alpha, const float *alphaPtr, const ts2_mat *res, int32_t resType, int32_t add, void *stream)
{
    if (!src || !transformFast || !res) {
        return TS2_ERR_NULL;
    }
    ts2_gemm_args g = {};
    g.a = *src;
    g.b = *transformFast;
    g.c = *res;
    g.abType = mode;
    g.cType = resType;
    g.m = lenRound;
    g.n = dstDim;
    g.k = srcDim;
    g.mLive = len;
    g.alpha = alpha;
    g.alphaPtr = alphaPtr;
    g.epilogue = add ? TS2_EPI_ADD : TS2_EPI_STORE;
    g.splitK = 1;
    return ts2_gemm_nt(&g, stream);
}

// Forward<TStoreRowTileNormalize> / Forward<TStoreRowTileNormalizeRope> of the same operator (layer_cuda_base.cuh:183-193 with the store
// functors of cuda_matmul.cuh:495-525 and gpu_rope.cuh:25-60): res = rope(normalise(alpha * (*alphaPtr) * src * W^T)) as bf16 plus the
// per-tile scales.  The product carries the epilogue itself where the 256x256-tile kernel applies; otherwise it is stored in fp32 into
// `raw` (caller scratch [lenRound][dstDim], may be null only when the fused form applies) and finished by the stand-alone pass.
extern "C" int ts2_matmul_forward_norm_rope(int32_t mode, int32_t len, int32_t lenRound, int32_t srcDim, int32_t dstDim, const ts2_mat *src,
    const ts2_mat *transformFast, float alpha, const float *alphaPtr, int32_t normalize, float vecScale, const ts2_mat *ropeBuf,
    const ts2_mat *res, const ts2_mat *tileScale, const ts2_mat *raw, void *stream)
{
    if (!src || !transformFast || !res || (normalize && !tileScale)) {
        return TS2_ERR_NULL;
    }
    ts2_gemm_args g = {};
    g.a = *src;
    g.b = *transformFast;
    g.abType = mode;
    g.m = lenRound;
    g.n = dstDim;
    g.k = srcDim;
    g.mLive = len;
    g.alpha = alpha;
    g.alphaPtr = alphaPtr;
    g.splitK = 1;
    const bool fused = lenRound % 256 == 0 && dstDim % 256 == 0 && (int64_t)(lenRound / 256) * (dstDim / 256) >= 192;
    if (fused) {
        g.c = *res;
        g.cType = TS2_BF16;
        g.epilogue = TS2_EPI_ROW_TILE_NORM;
        g.normalize = normalize;
        g.vecScale = vecScale;
        if (ropeBuf) {
            g.rope = *ropeBuf;
        }
        if (normalize) {
            g.tileScale = *tileScale;
        }
        return ts2_gemm_nt(&g, stream);
    }
    if (!raw) {
        return TS2_ERR_NULL;
    }
    g.c = *raw;
    g.cType = TS2_F32;
    g.epilogue = TS2_EPI_STORE;
    int rc = ts2_gemm_nt(&g, stream);
    if (rc != TS2_OK) {
        return rc;
    }
    return ts2_row_tile_normalize_rope(len, lenRound, raw, TS2_F32, 1.f, normalize, vecScale, ropeBuf, res, tileScale, stream);
}
