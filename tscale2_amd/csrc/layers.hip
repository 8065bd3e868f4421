// Layer orchestration and the one-GPU step driver: the call order of the reference's CUDA layers and executor
//   TCudaFFLayer::AddForward/AddBackward     src/gpt/compute/layer_ffn.cu:56-113
//   TCudaAttLayer::AddForward/AddBackward    src/gpt/compute/layer_att.cu:108-226
//   TCudaMoELayer::AddForward/AddBackward    src/gpt/compute/layer_moe.cu:117-272
//   AddForwardGraph / CreateBackpropGraph    src/gpt/compute/gpu_transformer.cu:260-471
// expressed over the C ABI of this library.  Host code only.  Unlike the reference's CUDA path, which drops constant factors
// (matrix scales, 1/24 storage scales) because its optimiser normalises every delta, this driver keeps every factor of the CPU
// path (src/gpt/compute/cpu_transformer.cpp, layer_*.cu CPU classes), so its deltas are directly comparable with the CPU oracle.
#include "common.h"
#include "internal.h"
#include <math.h>
#include <string.h>
#include <vector>

namespace
{
constexpr float VEC = 1 / 24.0f;    // STATE/Q/K/V/FFN/MOE_VEC_SCALE, src/gpt/compute/cfg_precision.h:72-77
constexpr float DISCR = 1 / 32.0f;  // MODEL_DISCR_SCALE, src/gpt/model_params/model_dim.h:9
constexpr float LN2F = 0.693147f;   // LOG2, model_dim.h:16

inline float Dot(int dim)
{
    return sqrtf(1.0f / dim);
}

// pitched host<->device copy as plain 1-D copies (one when both sides are dense, else one per row)
hipError_t Copy2D(void *dst, size_t dpitch, const void *src, size_t spitch, size_t width, size_t height, hipMemcpyKind kind)
{
    if (dpitch == width && spitch == width) {
        return hipMemcpy(dst, src, width * height, kind);
    }
    for (size_t y = 0; y < height; ++y) {
        hipError_t e = hipMemcpy((uint8_t *)dst + y * dpitch, (const uint8_t *)src + y * spitch, width, kind);
        if (e != hipSuccess) {
            return e;
        }
    }
    return hipSuccess;
}

int ElemSz(int type)
{
    return (type == TS2_F32 || type == TS2_I32) ? 4 : ((type == TS2_BF16 || type == TS2_F16) ? 2 : 1);
}

struct Arr {
    ts2_mat m = {nullptr, 0, 0, 0};
    int type = 0;
    const ts2_mat *P() const { return &m; }
};

#define CK(x)                                                                                                                              \
    do {                                                                                                                                   \
        int rc_ = (x);                                                                                                                     \
        if (rc_ != 0)                                                                                                                      \
            return rc_;                                                                                                                    \
    } while (0)

struct TMatrix {
    Arr fast;           // [dst][src] 8-bit ([slabs*dst][src] for expert matrices)
    Arr fastT;          // [src][dst]: the transpose the dX products contract over, kept until the matrix is set again (not for slabs)
    bool fastTValid = false;
    float *scale = 0;   // device: matrix scale (rms of the fp32 master weights)
    Arr delta;          // i8 packed delta, same shape
    Arr deltaTileScale; // fp32 [src/128][rows]
    int srcDim = 0, dstDim = 0, slabs = 1;
    // optimiser state (master weights, moving average, dispersion estimates), present once ts2_model_set_master has been called
    ts2_opt_matrix opt = {};
    Arr optWeights, optAvgGrad;
    bool hasOpt = false;
    int optRows = 0; // rows of the master matrix (the model's rows without tile padding)
};

struct TActs;
struct TLayer {
    int type = 0;
    float slope = 0;
    int attId = 0;
    TMatrix w[5];
    TActs *acts = nullptr;
    // fp8 attention layers: the packed deltas of Q, K, V and gate are row blocks of one [4Q][dim] array (and column blocks of one
    // tile-scale array), so that one delta product over the four stacked transposed gradients fills them all
    TMatrix qkvg;
    bool fusedDelta = false;
};

enum { LT_ATT = 0, LT_FFN = 2, LT_MOE = 3 };

// What a layer's forward pass leaves behind for its backward pass.  The reference recomputes all of it inside AddBackward (its
// Fwd/Bwd pools are shared between layers, layer_cuda_base.cuh:101-121); with 288 GB of HBM every FFN and attention layer keeps its own
// set (about 1.35 GB per FFN layer and 0.75 GB per attention layer at dim 2048, ffn 8192, 32768 tokens) and the backward starts
// from it.  One shared set (recompute mode) serves all layers otherwise.
struct TActs {
    Arr a16[4]; // bf16: wide/q, gate, k, v
    Arr tsc[2]; // fp32 tile scales: wide/q, v
    Arr rg8;    // 8-bit rg / vlg
    Arr val16;  // bf16 attention output (its storage is reused for dQ by the backward)
    Arr swl;    // fp32 [heads][R] softmax statistics
    bool valid = false;
};
} // namespace

struct ts2_model {
    ts2_model_config cfg;
    std::vector<int> layerType, layerAttId;
    std::vector<float> layerSlope;
    std::vector<TLayer> layers;
    std::vector<void *> allocs;
    int mode = TS2_I8, fastGradType = TS2_BF16;
    int R = 0; // lenRound capacity
    int VP = 0; // vocabulary rows of the final matrix and columns of the logits as allocated: a large vocabulary is padded with zero
                // rows to a multiple of 256 so that its three products run on the 256x256 tile
    int len = 0;
    int lenMoe = 0;
    int kTile = 512;
    // model
    TMatrix embed, finalW;
    float *bias = 0;
    ts2_add_gradient_params *optParams = 0; // device copy of the optimiser step parameters
    // batch
    int *labelPtr = 0;
    uint32_t *labels = 0;
    int labelCap = 0;
    int *target = 0;
    std::vector<int *> spanStart, spanFinish, revLo, revHi;
    Arr rope;
    // states
    Arr state, stateGrad, stateGradFast, dNormState;
    std::vector<Arr> normState, stateScale;
    float *gradMaxNorm = 0, *gradScale = 0, *gradMult = 0, *lossSum = 0;
    // layer scratch (shared by all layers: one layer runs at a time)
    Arr raw;                                 // fp32 [R'][maxW]
    TActs shared;                            // the one activation set of recompute mode (and of MoE layers)
    std::vector<TActs> acts;                 // per layer; entries of kept layers own storage, the others alias `shared`
    bool keep = false;      // FFN and attention layers own activation sets
    bool useKept = false;   // inside ModelBackprop: the backward of a layer starts from what its forward left
    int sharedOwner = -1;   // the MoE layer whose forward filled the shared set, its gathered input and the routing tables last
    Arr g32;                                 // fp32 [R'][maxW] gradient scratch (drg / dvlg)
    Arr gf[4];                               // fast-gradient type [R'][maxW]: dwide/dq, dgate, dk, dv
    Arr g16[4];                              // bf16 [R'][maxW]: -, dVal, dK, dV
    Arr dScale;                              // fp32 [heads][R]
    // MoE
    ts2_moe_tables moe = {};
    Arr normMoe, sgMoe, moeSel, dMoeSel;     // grouped 8-bit input / gradient, select logits fp32, their gradient
    float *dExpertWeight = 0;
    // final layer
    Arr logits, gradV, gradVT, fnT, wfT;
    Arr logits16;                            // IEEE-half logits of the backward pass (the fp32 ones serve ts2_model_forward)
    // linear backward scratch
    uint8_t *sGrad8 = 0, *sGradT = 0, *sSrcT = 0, *sWT = 0;
    uint8_t *sGradTa = 0, *sGradTb = 0; // transposed gradients written by their producer (fp8 FFN backward)
    float *sPartial = 0;                     // fp32 slices of a delta product with few output tiles
    size_t sPartialFloats = 0;
    float *sRowScale = 0, *sTileMax = 0, *sTileScale = 0;
    uint32_t ditherCalls = 0; // uses of the linear operator so far (seeds of the int8 dither)
    int maxW = 0, RP = 0; // RP = rows of the row-indexed scratch (max(R, lenMoe))
    int cuCount = 256;

    void *Dev(size_t bytes)
    {
        void *p = nullptr;
        if (hipMalloc(&p, bytes ? bytes : 16) != hipSuccess) {
            return nullptr;
        }
        allocs.push_back(p);
        if (hipMemset(p, 0, bytes ? bytes : 16) != hipSuccess) {
            return nullptr;
        }
        return p;
    }
    bool Alloc(Arr *a, int rows, int cols, int type)
    {
        a->type = type;
        int64_t stride = ((int64_t)cols * ElemSz(type) + 255) / 256 * 256;
        a->m.ptr = Dev((size_t)stride * rows);
        a->m.strideBytes = stride;
        a->m.x = cols;
        a->m.y = rows;
        return a->m.ptr != nullptr;
    }
    ~ts2_model()
    {
        for (void *p : allocs) {
            (void)hipFree(p);
        }
    }
};

namespace
{
// view of the first rows x cols of an array (same storage)
Arr View(const Arr &a, int rows, int cols)
{
    Arr r = a;
    r.m.x = cols;
    r.m.y = rows;
    return r;
}

Arr Flat(void *p, int rows, int cols, int type)
{
    Arr r;
    r.type = type;
    r.m.ptr = p;
    r.m.strideBytes = (int64_t)cols * ElemSz(type);
    r.m.x = cols;
    r.m.y = rows;
    return r;
}

ts2_matmul_bwd_buffers Scratch(ts2_model *M, int rows, int srcDim, int gradDim)
{
    ts2_matmul_bwd_buffers b = {};
    b.grad8 = Flat(M->sGrad8, rows, gradDim, TS2_I8).m;
    b.grad8RowScale = M->sRowScale;
    b.gradT = Flat(M->sGradT, gradDim, rows, M->mode).m;
    b.srcT = Flat(M->sSrcT, srcDim, rows, M->mode).m;
    b.tileMax = M->sTileMax;
    b.tileScale = M->sTileScale;
    b.transformT = Flat(M->sWT, srcDim, gradDim, M->mode).m;
    if (M->cfg.ditherSeed) {
        // every use of the operator draws its own noise: the call counter runs on from step to step
        uint32_t h = M->cfg.ditherSeed + 0x9E3779B9u * ++M->ditherCalls;
        h ^= h >> 15;
        h *= 0x2C1B3C6Du;
        h ^= h >> 12;
        b.ditherSeed = h | 1u;
    }
    return b;
}

// res (+)= alpha [* scale] * src8 * W^T
int Forward(ts2_model *M, TMatrix &W, const Arr &src8, float alpha, bool useScale, const Arr &res, bool add, void *s)
{
    return ts2_matmul_forward(M->mode, M->len, M->R, W.srcDim, W.dstDim, src8.P(), W.fast.P(), alpha, useScale ? W.scale : nullptr, res.P(),
        res.type, add, s);
}

// dst16 = rope(normalise(alpha [* scale] * src8 * W^T)), tile scales to tileScale (fused into the product where the big tile applies)
int ForwardNormRope(ts2_model *M, TMatrix &W, const Arr &src8, float alpha, bool useScale, bool normalize, float vecScale, const Arr *rope,
    const Arr &dst16, const Arr *tileScale, void *s)
{
    Arr raw = View(M->raw, M->R, W.dstDim);
    return ts2_matmul_forward_norm_rope(M->mode, M->len, M->R, W.srcDim, W.dstDim, src8.P(), W.fast.P(), alpha, useScale ? W.scale : nullptr,
        normalize, vecScale, rope ? rope->P() : nullptr, dst16.P(), tileScale ? tileScale->P() : nullptr, raw.P(), s);
}

// srcGrad (+)= alpha [* scale] * gradFast * W   (TMatMulBuffers::BackpropMulti + Backprop)
int BackpropDX(ts2_model *M, TMatrix &W, const Arr &gradFast, float alpha, bool useScale, const Arr &srcGrad, bool add, void *s)
{
    ts2_matmul_bwd_buffers b = Scratch(M, M->R, W.srcDim, W.dstDim);
    if (W.fastT.m.ptr) {
        b.transformT = W.fastT.m;
        b.transformTValid = W.fastTValid;
    }
    CK(ts2_matmul_backprop_multi(M->mode, M->len, M->R, W.srcDim, W.dstDim, W.fast.P(), gradFast.P(), gradFast.type, nullptr, &b, s));
    W.fastTValid = W.fastT.m.ptr != nullptr;
    return ts2_matmul_backprop(M->mode, M->len, M->R, W.srcDim, W.dstDim, gradFast.P(), &b, alpha, useScale ? W.scale : nullptr, srcGrad.P(),
        srcGrad.type, add, s);
}

// srcGrad (+)= sum_i alpha [* scale_i] * grad_i * W_i for the matrices of a layer that share their input: every weight is transposed
// into its own part of the transpose scratch, then one grouped Backprop
int BackpropDXGroup(ts2_model *M, int count, TMatrix *const *W, const Arr *const *grad, float alpha, const bool *useScale, const Arr &srcGrad,
    bool add, void *s)
{
    ts2_matmul_bwd_buffers b[4];
    const ts2_matmul_bwd_buffers *bp[4];
    const ts2_mat *gp[4];
    float al[4];
    const float *ap[4];
    const int srcDim = W[0]->srcDim, dstDim = W[0]->dstDim;
    if (M->mode != TS2_E4M3) {
        // int8: the row-quantised gradient lives in the one shared scratch, so the products go one after the other
        for (int i = 0; i < count; ++i) {
            CK(BackpropDX(M, *W[i], *grad[i], alpha, useScale[i], srcGrad, add || i > 0, s));
        }
        return 0;
    }
    for (int i = 0; i < count; ++i) {
        if (W[i]->srcDim != srcDim || W[i]->dstDim != dstDim) {
            return TS2_ERR_SHAPE;
        }
        if ((size_t)(i + 1) * srcDim * dstDim > (size_t)4 * M->maxW * M->maxW) {
            return TS2_ERR_SHAPE;
        }
        b[i] = Scratch(M, M->R, srcDim, dstDim);
        b[i].transformT = Flat(M->sWT + (size_t)i * srcDim * dstDim, srcDim, dstDim, M->mode).m;
        if (W[i]->fastT.m.ptr) {
            b[i].transformT = W[i]->fastT.m;
            b[i].transformTValid = W[i]->fastTValid;
        }
        CK(ts2_matmul_backprop_multi(M->mode, M->len, M->R, srcDim, dstDim, W[i]->fast.P(), grad[i]->P(), grad[i]->type, nullptr, &b[i], s));
        W[i]->fastTValid = W[i]->fastT.m.ptr != nullptr;
        bp[i] = &b[i];
        gp[i] = grad[i]->P();
        al[i] = alpha;
        ap[i] = useScale[i] ? W[i]->scale : nullptr;
    }
    return ts2_matmul_backprop_group(M->mode, M->len, M->R, srcDim, dstDim, count, gp, bp, al, ap, srcGrad.P(), srcGrad.type, add, s);
}

// slices of the token axis for a delta product [dstDim x srcDim]: enough to give every CU a 256x256 tile, each slice a whole number of
// k-tiles and at least 4096 tokens long
int DeltaSplits(ts2_model *M, int srcDim, int dstDim)
{
    if (M->mode != TS2_E4M3) {
        return 1;
    }
    if ((srcDim % 256) || (dstDim % 256)) {
        // 128x128 tiles (the select matrix of a MoE layer: 128 x dim): two workgroups per CU, slices of at least 2048 tokens
        int tiles = (srcDim / 128) * (dstDim / 128), splits = 1;
        while (splits < 32 && tiles * splits < 512 && M->R % (splits * 2 * 128) == 0 && M->R / (splits * 2) >= 2048) {
            splits *= 2;
        }
        return splits;
    }
    int tiles = (srcDim / 256) * (dstDim / 256);
    if (tiles >= 192) {
        return 1;
    }
    int splits = 1;
    while (splits < 8 && tiles * splits < 192 && M->R % (splits * 2 * 128) == 0 && M->R / (splits * 2) >= 4096) {
        splits *= 2;
    }
    return splits;
}

// fp8 operands, whole 128-row groups, both widths on the 256 grid: the delta product contracts over the rows of gradient and source as
// they lie in memory (ts2_gemm_args.kMajor), so nobody has to leave or make a transpose of either
bool DeltaReadsRows(ts2_model *M, int srcDim, int dstDim)
{
    return M->mode == TS2_E4M3 && M->fastGradType == TS2_E4M3 && M->len == M->R && (srcDim % 256) == 0 && (dstDim % 256) == 0;
}

// columns [k * cols, (k + 1) * cols) of a
Arr ColBlock(const Arr &a, int k, int cols)
{
    Arr r = a;
    r.m.ptr = (uint8_t *)a.m.ptr + (size_t)k * cols * ElemSz(a.type);
    r.m.x = cols;
    return r;
}

// delta = alpha * gradScale * gradFast^T * src8   (TMatMulBuffers::BackpropDelta)
int BackpropDelta(ts2_model *M, TMatrix &W, const Arr &src8, const Arr &gradFast, float alpha, const float *gradScale, void *s,
    bool sameSrcAsLastCall = false, const Arr *gradTReady = nullptr)
{
    ts2_matmul_bwd_buffers b = Scratch(M, M->R, W.srcDim, W.dstDim);
    b.srcTValid = sameSrcAsLastCall; // the matrices of a layer that share their input transpose it once
    if (gradTReady) { // the producer of the gradient left its transpose
        b.gradT = gradTReady->m;
        b.gradTValid = 1;
    }
    // a delta with fewer large tiles than the chip has CUs runs as slices of the token axis on the large tile, packed afterwards
    int splits = DeltaSplits(M, W.srcDim, W.dstDim);
    if (splits > 1 && (size_t)splits * W.dstDim * W.srcDim <= M->sPartialFloats) {
        b.partial = Flat(M->sPartial, splits * W.dstDim, W.srcDim, TS2_F32).m;
        b.splits = splits;
    }
    return ts2_matmul_backprop_delta(M->mode, M->len, M->R, W.srcDim, W.dstDim, src8.P(), nullptr, gradFast.P(), gradFast.type, alpha, gradScale,
        M->kTile, &b, W.delta.P(), W.deltaTileScale.P(), s);
}

// ---------------------------------------------------------------------------------------------------------------------------
// FFN: src/gpt/compute/layer_ffn.cu:56-113 (CUDA order) with the CPU path's factors (layer_ffn.cu:190-248)
int FfnComputeRG(ts2_model *M, TLayer &L, const Arr &norm8, void *s)
{
    int D = M->cfg.dim, F = M->cfg.ffnDim, len = M->len, R = M->R;
    TActs &A = *L.acts;
    Arr wideRaw = View(M->raw, R, F), wide16 = View(A.a16[0], R, F), gate16 = View(A.a16[1], R, F), wideScale = View(A.tsc[0], F / 128, R);
    Arr rg8 = View(A.rg8, R, F);
    // wide = MulForward(n, We) in true units, then per-tile normalisation to 1/24 units + tile scale
    CK(ForwardNormRope(M, L.w[0], norm8, VEC * DISCR * Dot(D), true, true, VEC, nullptr, wide16, &wideScale, s));
    // gate uses the matrix without its scale (GetDataNoScale)
    CK(Forward(M, L.w[1], norm8, VEC * DISCR * Dot(D), false, gate16, false, s));
    return ts2_matrix_lolu(len, R, gate16.P(), wide16.P(), 1.f, rg8.P(), M->mode, s);
}

int FfnForward(ts2_model *M, TLayer &L, const Arr &norm8, void *s)
{
    int F = M->cfg.ffnDim;
    CK(FfnComputeRG(M, L, norm8, s));
    return Forward(M, L.w[2], View(L.acts->rg8, M->R, F), VEC * DISCR * Dot(F), true, M->state, true, s);
}

int FfnBackward(ts2_model *M, TLayer &L, const Arr &norm8, const float *gradScale, void *s)
{
    int D = M->cfg.dim, F = M->cfg.ffnDim, len = M->len, R = M->R;
    TActs &A = *L.acts;
    Arr wide16 = View(A.a16[0], R, F), gate16 = View(A.a16[1], R, F), wideScale = View(A.tsc[0], F / 128, R), rg8 = View(A.rg8, R, F);
    // drg travels in bf16 (the reference uses half here): its consumer rounds to the 8-bit gradient type anyway
    Arr drg = View(M->g16[0], R, F), dwide = View(M->gf[0], R, F), dgate = View(M->gf[1], R, F);
    if (!(M->useKept && A.valid)) {
        CK(FfnComputeRG(M, L, norm8, s));
    }
    // contract backward
    CK(BackpropDX(M, L.w[2], M->stateGradFast, DISCR * Dot(F), true, drg, false, s));
    // fp8: the gate/norm backward also writes the transposed gradients that the two delta products contract over
    const bool fusedT = !DeltaReadsRows(M, D, F) && M->mode == TS2_E4M3 && M->fastGradType == TS2_E4M3 && M->sGradTa && (R % 128) == 0;
    Arr dwideT = Flat(M->sGradTa, F, R, TS2_E4M3), dgateT = Flat(M->sGradTb, F, R, TS2_E4M3);
    if (fusedT) {
        CK(ts2_backprop_row_tile_normalize_lolu_t(len, R, gate16.P(), wide16.P(), VEC, wideScale.P(), drg.P(), dgate.P(), dwide.P(), dgateT.P(),
            dwideT.P(), s));
    } else {
        CK(ts2_backprop_row_tile_normalize_lolu(len, R, gate16.P(), wide16.P(), VEC, wideScale.P(), drg.P(), TS2_BF16, dgate.P(), dwide.P(),
            M->fastGradType, s));
    }
    {
        TMatrix *const ws[2] = {&L.w[0], &L.w[1]};
        const Arr *const gs[2] = {&dwide, &dgate};
        const bool us[2] = {true, false};
        CK(BackpropDXGroup(M, 2, ws, gs, DISCR * Dot(D), us, M->dNormState, false, s));
    }
    // deltas (sources are stored in 1/24 units)
    CK(BackpropDelta(M, L.w[2], rg8, M->stateGradFast, VEC, gradScale, s));
    CK(BackpropDelta(M, L.w[0], norm8, dwide, VEC, gradScale, s, false, fusedT ? &dwideT : nullptr));
    return BackpropDelta(M, L.w[1], norm8, dgate, VEC, gradScale, s, true, fusedT ? &dgateT : nullptr);
}

// ---------------------------------------------------------------------------------------------------------------------------
// attention: src/gpt/compute/layer_att.cu:108-226 with the CPU path's factors (layer_att.cu:368-482)
float AttDotScale()
{
    return Dot(128) * (0.5f / LN2F); // CalcDotScale(QDim) * CalcAttentionMult(), layer_att_reference.h:29-32
}

int AttComputeVLG(ts2_model *M, TLayer &L, const Arr &norm8, void *s)
{
    int D = M->cfg.dim, H = M->cfg.headCount, Q = H * 128, len = M->len, R = M->R;
    TActs &A = *L.acts;
    Arr raw = View(M->raw, R, Q), q16 = View(A.a16[0], R, Q), gate16 = View(A.a16[1], R, Q), k16 = View(A.a16[2], R, Q), v16 = View(A.a16[3], R, Q);
    Arr qScale = View(A.tsc[0], H, R), vScale = View(A.tsc[1], H, R), val16 = View(A.val16, R, Q), vlg8 = View(A.rg8, R, Q);
    float a = VEC * DISCR * Dot(D);
    CK(ForwardNormRope(M, L.w[0], norm8, a, true, true, 1.f, &M->rope, q16, &qScale, s));
    CK(ForwardNormRope(M, L.w[1], norm8, a, true, false, 1.f, &M->rope, k16, nullptr, s));
    CK(ForwardNormRope(M, L.w[2], norm8, a, true, true, 1.f, nullptr, v16, &vScale, s));
    CK(Forward(M, L.w[3], norm8, a, false, gate16, false, s));
    ts2_att_args at = {};
    at.len = len;
    at.lenRound = R;
    at.heads = H;
    at.q = q16.m;
    at.k = k16.m;
    at.v = v16.m;
    at.spanStart = M->spanStart[L.attId];
    at.spanFinish = M->spanFinish[L.attId];
    at.attDotScale = AttDotScale();
    at.alibiSlope = L.slope;
    at.valLookup = val16.m;
    at.sumWeightLog = A.swl.m;
    CK(ts2_att_forward(&at, s));
    // VLG = sigmoid(2 gate) * val in 1/24 units
    return ts2_matrix_lolu(len, R, gate16.P(), val16.P(), 24.f, vlg8.P(), M->mode, s);
}

int AttForward(ts2_model *M, TLayer &L, const Arr &norm8, void *s)
{
    int TT = M->cfg.headCount * 128;
    CK(AttComputeVLG(M, L, norm8, s));
    return Forward(M, L.w[4], View(L.acts->rg8, M->R, TT), VEC * DISCR * Dot(TT), true, M->state, true, s);
}

int AttBackward(ts2_model *M, TLayer &L, const Arr &norm8, const float *gradScale, void *s)
{
    int D = M->cfg.dim, H = M->cfg.headCount, Q = H * 128, len = M->len, R = M->R;
    TActs &A = *L.acts;
    Arr q16 = View(A.a16[0], R, Q), gate16 = View(A.a16[1], R, Q), k16 = View(A.a16[2], R, Q), v16 = View(A.a16[3], R, Q);
    Arr qScale = View(A.tsc[0], H, R), vScale = View(A.tsc[1], H, R), val16 = View(A.val16, R, Q), vlg8 = View(A.rg8, R, Q);
    Arr dvlg = View(M->g16[0], R, Q), dGate = View(M->gf[1], R, Q), dVal16 = View(M->g16[1], R, Q);
    // one delta product for the four matrices that read the layer input, contracting over rows: their gradients are written side by side
    // as column blocks of one [R][4Q] array (the transpose scratch, which nothing else uses then)
    const bool stacked = L.fusedDelta && DeltaReadsRows(M, D, 4 * Q);
    Arr gStack = Flat(M->sGradT, R, 4 * Q, M->fastGradType);
    if (stacked) {
        dGate = ColBlock(gStack, 3, Q);
    }
    if (!(M->useKept && A.valid)) {
        CK(AttComputeVLG(M, L, norm8, s));
    }
    A.valid = false; // the backward reuses val16's storage for dQ
    // combiner backward
    CK(BackpropDX(M, L.w[4], M->stateGradFast, DISCR * Dot(Q), true, dvlg, false, s));
    CK(BackpropDelta(M, L.w[4], vlg8, M->stateGradFast, VEC, gradScale, s));
    // gate backward + dScale
    CK(ts2_backprop_lolu_dscale(len, R, gate16.P(), val16.P(), 1.f, dvlg.P(), TS2_BF16, dGate.P(), M->fastGradType, dVal16.P(), TS2_BF16,
        M->dScale.P(), s));
    // attention backward (dQ, dK, dV in bf16; val16's buffer is reused for dQ once dScale is known)
    Arr dQ = View(A.val16, R, Q), dK = View(M->g16[2], R, Q), dV = View(M->g16[3], R, Q);
    ts2_att_grad_args ag = {};
    ag.len = len;
    ag.lenRound = R;
    ag.heads = H;
    ag.q = q16.m;
    ag.k = k16.m;
    ag.v = v16.m;
    ag.dValLookup = dVal16.m;
    ag.spanStart = M->spanStart[L.attId];
    ag.spanFinish = M->spanFinish[L.attId];
    ag.revLo = M->revLo[L.attId];
    ag.revHi = M->revHi[L.attId];
    ag.attDotScale = AttDotScale();
    ag.alibiSlope = L.slope;
    ag.sumWeightLog = A.swl.m;
    ag.dScale = M->dScale.m;
    ag.dQ = dQ.m;
    ag.dK = dK.m;
    ag.dV = dV.m;
    ag.gradType = TS2_BF16;
    ag.which = 3;
    CK(ts2_att_backward(&ag, s));
    // epilogues: norm backward against the stored rotated vector, then inverse rope (TStoreAttBack*, gpu_att_utils.cuh:280-352)
    Arr dQf = View(M->gf[0], R, Q), dKf = View(M->gf[2], R, Q), dVf = View(M->gf[3], R, Q);
    if (stacked) {
        dQf = ColBlock(gStack, 0, Q);
        dKf = ColBlock(gStack, 1, Q);
        dVf = ColBlock(gStack, 2, Q);
    }
    CK(ts2_backprop_row_tile_normalize_rope(len, R, dQ.P(), TS2_BF16, 1.f, q16.P(), qScale.P(), M->rope.P(), dQf.P(), M->fastGradType, s));
    CK(ts2_backprop_row_tile_normalize_rope(len, R, dK.P(), TS2_BF16, 1.f, nullptr, nullptr, M->rope.P(), dKf.P(), M->fastGradType, s));
    CK(ts2_backprop_row_tile_normalize_rope(len, R, dV.P(), TS2_BF16, 1.f, v16.P(), vScale.P(), nullptr, dVf.P(), M->fastGradType, s));
    float a = DISCR * Dot(D);
    {
        TMatrix *const ws[4] = {&L.w[0], &L.w[1], &L.w[2], &L.w[3]};
        const Arr *const gs[4] = {&dQf, &dKf, &dVf, &dGate};
        const bool us[4] = {true, true, true, false};
        CK(BackpropDXGroup(M, 4, ws, gs, a, us, M->dNormState, false, s));
    }
    if (stacked) {
        return BackpropDelta(M, L.qkvg, norm8, gStack, VEC, gradScale, s);
    }
    if (L.fusedDelta) {
        // the four transposed gradients stacked as row blocks of one [4Q][R] array, then one delta product [4Q x D]: 256 large tiles
        // instead of four products of 64 that each need token-axis slices and a pack pass
        Arr gT = Flat(M->sGradT, 4 * Q, R, M->mode);
        const Arr *const gs4[4] = {&dQf, &dKf, &dVf, &dGate};
        for (int k = 0; k < 4; ++k) {
            Arr blk = gT;
            blk.m.ptr = (uint8_t *)gT.m.ptr + (size_t)k * Q * gT.m.strideBytes;
            blk.m.y = Q;
            CK(ts2_transpose_quant(len, R, gs4[k]->P(), M->mode, nullptr, nullptr, 0, nullptr, blk.P(), M->mode, nullptr, s));
        }
        return BackpropDelta(M, L.qkvg, norm8, dQf, VEC, gradScale, s, false, &gT);
    }
    CK(BackpropDelta(M, L.w[0], norm8, dQf, VEC, gradScale, s));
    CK(BackpropDelta(M, L.w[1], norm8, dKf, VEC, gradScale, s, true));
    CK(BackpropDelta(M, L.w[2], norm8, dVf, VEC, gradScale, s, true));
    return BackpropDelta(M, L.w[3], norm8, dGate, VEC, gradScale, s, true);
}

// ---------------------------------------------------------------------------------------------------------------------------
// MoE: src/gpt/compute/layer_moe.cu:117-272 with the CPU path's factors (layer_moe.cu:458-537).  fp8 operands only.
int GroupedGemm(ts2_model *M, const Arr &a, const Arr &bSlabs, int slabRows, int n, int k, const Arr &c, float alpha, const float *alphaPtr, bool add,
    void *s, const Arr *a2 = nullptr, const Arr *bSlabs2 = nullptr, const float *alphaPtr2 = nullptr, const Arr *normTileScale = nullptr,
    float normVecScale = 1.f)
{
    ts2_gemm_args g = {};
    g.a = a.m;
    g.b = bSlabs.m;
    g.b.y = slabRows; // one slab; the kernel offsets by the tile's expert
    g.c = c.m;
    g.abType = a.type;
    g.cType = c.type;
    g.m = M->lenMoe;
    g.n = n;
    g.k = k;
    g.alpha = alpha;
    g.alphaPtr = alphaPtr;
    g.epilogue = add ? TS2_EPI_ADD : TS2_EPI_STORE;
    g.splitK = 1;
    g.tileGroup = M->moe.xpTileExpertId;
    g.bSlabBytes = (int64_t)slabRows * bSlabs.m.strideBytes;
    if (normTileScale) { // Forward<TStoreRowTileNormalize>: the product leaves normalised 16-bit rows and their tile scales
        g.epilogue = TS2_EPI_ROW_TILE_NORM;
        g.normalize = 1;
        g.vecScale = normVecScale;
        g.tileScale = normTileScale->m;
    }
    if (a2) { // a second product with the same shapes and strides into the same result (its factor: alpha * *alphaPtr2)
        if (a2->m.strideBytes != a.m.strideBytes || bSlabs2->m.strideBytes != bSlabs.m.strideBytes) {
            return TS2_ERR_SHAPE;
        }
        g.extraSegments = 1;
        g.segment[0].a = a2->m.ptr;
        g.segment[0].b = bSlabs2->m.ptr;
        g.segment[0].alpha = alpha;
        g.segment[0].alphaPtr = alphaPtr2;
    }
    return ts2_gemm_nt(&g, s);
}

// per-expert delta: delta_e[gradDim][srcDim] = alpha * gradScale * sum over the expert's rows of grad^T src
int GroupedDelta(ts2_model *M, TMatrix &W, const Arr &src8, const Arr &gradFast, float alpha, const float *gradScale, void *s,
    bool sameSrcAsLastCall = false)
{
    int E = M->cfg.expertCount, rows = M->lenMoe;
    ts2_gemm_args g = {};
    if (M->fastGradType == TS2_E4M3 && (W.srcDim % 256) == 0 && (W.dstDim % 256) == 0) {
        // every row of the expert-ordered arrays is written (pad rows of an expert's group hold zeros): contract over them as they lie
        g.a = gradFast.m;
        g.b = src8.m;
        g.kMajor = 1;
        g.tileConfig = 1;
    } else {
        Arr gradT = Flat(M->sGradT, W.dstDim, rows, M->mode), srcT = Flat(M->sSrcT, W.srcDim, rows, M->mode);
        CK(ts2_transpose_quant(rows, rows, gradFast.P(), M->mode, nullptr, nullptr, 0, nullptr, gradT.P(), M->mode, nullptr, s));
        if (!sameSrcAsLastCall) { // (the expand and gate matrices share their source: one transpose)
            CK(ts2_transpose_quant(rows, rows, src8.P(), M->mode, nullptr, nullptr, 0, nullptr, srcT.P(), M->mode, nullptr, s));
        }
        g.a = gradT.m;
        g.b = srcT.m;
    }
    g.c = W.delta.m;
    g.c.y = W.dstDim;
    g.abType = M->mode;
    g.cType = TS2_I8;
    g.m = W.dstDim;
    g.n = W.srcDim;
    g.k = rows;
    g.alpha = alpha;
    g.alphaPtr = gradScale;
    g.epilogue = TS2_EPI_ROW_TILE_MAXNORM;
    g.tileScale = W.deltaTileScale.m;
    g.tileScale.x = W.dstDim;
    g.splitK = 1;
    g.groupOffsets = M->moe.expertOffset;
    g.groups = E;
    g.cSlabBytes = (int64_t)W.dstDim * W.delta.m.strideBytes;
    g.tileScaleSlabBytes = (int64_t)W.dstDim * 4; // tileScale rows are [src/128][E*dst]: slab e starts at column e*dst
    return ts2_gemm_nt(&g, s);
}

int MoeComputeRG(ts2_model *M, TLayer &L, const Arr &norm8, void *s)
{
    int D = M->cfg.dim, X = M->cfg.expertDim, E = M->cfg.expertCount, K = M->cfg.moeSelected, len = M->len, R = M->R, RM = M->lenMoe;
    float a = VEC * DISCR * Dot(D);
    // select logits (matrix without scale), routing tables, gather of the layer input into expert order
    CK(Forward(M, L.w[3], norm8, a, false, M->moeSel, false, s));
    CK(ts2_moe_route(len, RM, E, K, M->moeSel.P(), TS2_F32, &M->moe, s));
    CK(ts2_moe_group_samples(RM, 1, norm8.P(), M->moe.xpSampleId, M->normMoe.P(), s));
    TActs &A = M->shared;
    Arr wide16 = View(A.a16[0], RM, X), gate16 = View(A.a16[1], RM, X), wideScale = View(A.tsc[0], X / 128, RM);
    Arr rg8 = View(A.rg8, RM, X);
    CK(GroupedGemm(M, M->normMoe, L.w[0].fast, X, X, D, wide16, a, L.w[0].scale, false, s, nullptr, nullptr, nullptr, &wideScale, VEC));
    CK(GroupedGemm(M, M->normMoe, L.w[1].fast, X, X, D, gate16, a, nullptr, false, s));
    return ts2_matrix_lolu_moe(RM, M->moe.xpSampleWeight, gate16.P(), wide16.P(), 1.f, rg8.P(), M->mode, s);
}

int MoeForward(ts2_model *M, TLayer &L, const Arr &norm8, void *s)
{
    int D = M->cfg.dim, X = M->cfg.expertDim, E = M->cfg.expertCount, RM = M->lenMoe;
    CK(MoeComputeRG(M, L, norm8, s));
    // the experts' results travel in 16 bits (the reference's ContractResult is half, layer_moe.cu:33)
    Arr contract = View(M->g16[0], RM, D);
    CK(GroupedGemm(M, View(M->shared.rg8, RM, X), L.w[2].fast, D, D, X, contract, VEC * DISCR * Dot(E * X), L.w[2].scale, false, s));
    return ts2_combine_experts(M->len, M->cfg.moeSelected, contract.P(), TS2_BF16, &M->moe, 1.f, nullptr, M->state.P(), 1, s);
}

int MoeBackward(ts2_model *M, TLayer &L, const Arr &norm8, const float *gradScale, bool kept, void *s)
{
    int D = M->cfg.dim, X = M->cfg.expertDim, E = M->cfg.expertCount, K = M->cfg.moeSelected, len = M->len, R = M->R, RM = M->lenMoe;
    if (!kept) {
        CK(MoeComputeRG(M, L, norm8, s));
    }
    TActs &A = M->shared;
    Arr wide16 = View(A.a16[0], RM, X), gate16 = View(A.a16[1], RM, X), wideScale = View(A.tsc[0], X / 128, RM), rg8 = View(A.rg8, RM, X);
    // state gradient into expert order
    CK(ts2_moe_group_samples(RM, 1, M->stateGradFast.P(), M->moe.xpSampleId, M->sgMoe.P(), s));
    // contract backward: dRG[row][x] = sum_d sg[row][d] Wc_e[d][x]: needs Wc_e^T = [X][D] per expert
    // (the experts' transposed matrices are kept from one backward to the next like the dense layers', and redone when a matrix is set
    // or updated)
    auto keptT = [&](TMatrix &W, int rows, int cols) -> int { // slabs of [rows][cols] -> [cols][rows]
        if (!W.fastTValid) {
            CK(ts2_transpose_u8_batched(E, rows, cols, W.fast.m.ptr, W.fast.m.strideBytes, (int64_t)rows * W.fast.m.strideBytes, W.fastT.m.ptr,
                W.fastT.m.strideBytes, (int64_t)cols * W.fastT.m.strideBytes, s));
            W.fastTValid = true;
        }
        return 0;
    };
    CK(keptT(L.w[2], D, X));
    Arr wcT = L.w[2].fastT;
    Arr drg = View(M->g16[0], RM, X); // 16 bits like the reference's DRG and StateGradFull (layer_moe.cu:35,46)
    CK(GroupedGemm(M, M->sgMoe, wcT, X, X, D, drg, DISCR * Dot(E * X), L.w[2].scale, false, s));
    Arr dwide = View(M->gf[0], RM, X), dgate = View(M->gf[1], RM, X);
    CK(ts2_backprop_row_tile_normalize_lolu_moe(RM, M->moe.xpSampleWeight, gate16.P(), wide16.P(), VEC, wideScale.P(), drg.P(), TS2_BF16, 1.f,
        dgate.P(), dwide.P(), M->fastGradType, M->dExpertWeight, s));
    // dExpertWeight was computed against rg in 1/24 units of nothing: vals*valsScale is the true normalised wide, so it is in true
    // (scaled-gradient) units already
    CK(ts2_backprop_moe(len, R, E, K, &M->moe, M->dExpertWeight, M->dMoeSel.P(), M->fastGradType, s));
    // expand + gate backward into grouped rows, then back to token order
    Arr sgFull = View(M->g16[1], RM, D);
    CK(keptT(L.w[0], X, D));
    CK(keptT(L.w[1], X, D));
    // both products in one launch (one pass over the result)
    Arr weT = L.w[0].fastT, wgT = L.w[1].fastT;
    CK(GroupedGemm(M, dwide, weT, D, D, X, sgFull, DISCR * Dot(D), L.w[0].scale, false, s, &dgate, &wgT, nullptr));
    CK(ts2_combine_experts(len, K, sgFull.P(), TS2_BF16, &M->moe, 1.f, nullptr, M->dNormState.P(), 0, s));
    // select matrix: dNormState += dMoe * Wsel / sqrt(D) and its delta through the same 8-bit operator as every other matrix (the
    // reference uses its fp16 kernels here, MatmulSelect.BackpropFp16, layer_moe.cu:264); rows >= experts of the matrix are zero
    CK(BackpropDX(M, L.w[3], M->dMoeSel, DISCR * Dot(D), false, M->dNormState, true, s));
    CK(BackpropDelta(M, L.w[3], norm8, M->dMoeSel, VEC, gradScale, s));
    // expert deltas
    CK(GroupedDelta(M, L.w[2], rg8, M->sgMoe, VEC, gradScale, s));
    CK(GroupedDelta(M, L.w[0], M->normMoe, dwide, VEC, gradScale, s));
    return GroupedDelta(M, L.w[1], M->normMoe, dgate, VEC, gradScale, s, true);
}
} // namespace

// ---------------------------------------------------------------------------------------------------------------------------
// step driver
namespace
{
int InitMatrix(ts2_model *M, TMatrix *W, int srcDim, int dstDim, int slabs, bool keepT = true)
{
    W->srcDim = srcDim;
    W->dstDim = dstDim;
    W->slabs = slabs;
    if (!M->Alloc(&W->fast, dstDim * slabs, srcDim, M->mode) || !M->Alloc(&W->delta, dstDim * slabs, srcDim, TS2_I8) ||
        !M->Alloc(&W->deltaTileScale, srcDim / 128, dstDim * slabs, TS2_F32)) {
        return TS2_ERR_LAUNCH;
    }
    // the transposed copy the dX products contract over, kept while the weights do not change (expert matrices: slab by slab)
    if (keepT && !M->Alloc(&W->fastT, srcDim * slabs, dstDim, M->mode)) {
        return TS2_ERR_LAUNCH;
    }
    W->scale = (float *)M->Dev(4);
    return W->scale ? 0 : TS2_ERR_LAUNCH;
}

int RoundUp(int x, int m)
{
    return (x + m - 1) / m * m;
}

int LayerForward(ts2_model *M, int d, void *s)
{
    TLayer &L = M->layers[d];
    const Arr &n8 = M->normState[d];
    if (L.type == LT_FFN) {
        CK(FfnForward(M, L, n8, s));
    } else if (L.type == LT_ATT) {
        CK(AttForward(M, L, n8, s));
    } else if (L.type == LT_MOE) {
        // MoE layers work in the shared set; in keep mode nothing else touches it (nor the routing tables and the gathered input), so
        // what the last MoE layer's forward left is still there when its backward runs
        CK(MoeForward(M, L, n8, s));
        M->shared.valid = M->keep;
        M->sharedOwner = d;
        return 0;
    } else {
        return TS2_ERR_UNSUPPORTED;
    }
    L.acts->valid = L.acts != &M->shared; // a set of its own still holds this layer's activations when its backward runs
    return 0;
}

int LayerBackward(ts2_model *M, int d, const float *gradScale, void *s)
{
    TLayer &L = M->layers[d];
    const Arr &n8 = M->normState[d];
    if (L.type == LT_FFN) {
        return FfnBackward(M, L, n8, gradScale, s);
    } else if (L.type == LT_ATT) {
        return AttBackward(M, L, n8, gradScale, s);
    } else if (L.type == LT_MOE) {
        const bool kept = M->useKept && M->shared.valid && M->sharedOwner == d;
        M->shared.valid = false;
        return MoeBackward(M, L, n8, gradScale, kept, s);
    }
    return TS2_ERR_UNSUPPORTED;
}

// AddForwardGraph, src/gpt/compute/gpu_transformer.cu:260-309
int ModelForward(ts2_model *M, void *s)
{
    int D = M->cfg.dim, depth = (int)M->layers.size();
    CK(Ts2EmbedForward(M->len, M->R, D, M->labelPtr, M->labels, M->embed.fast.P(), M->mode, DISCR, M->embed.scale, M->state.P(), s));
    CK(ts2_layer_normalize_state_vecs(M->state.P(), TS2_F32, M->len, M->R, VEC, M->normState[0].P(), M->mode, M->stateScale[0].P(), s));
    for (int d = 0; d < depth; ++d) {
        CK(LayerForward(M, d, s));
        CK(ts2_layer_normalize_state_vecs(M->state.P(), TS2_F32, M->len, M->R, VEC, M->normState[d + 1].P(), M->mode, M->stateScale[d + 1].P(), s));
    }
    return 0;
}

// final layer: src/gpt/compute/gpu_final.cuh:223-296 / cpu_transformer.cpp:119-172
int FinalLogits(ts2_model *M, const Arr &logits, void *s)
{
    int D = M->cfg.dim, depth = (int)M->layers.size();
    return Forward(M, M->finalW, M->normState[depth], VEC * DISCR * Dot(D) / LN2F, true, logits, false, s);
}

int FinalBackward(ts2_model *M, void *s)
{
    int D = M->cfg.dim, V = M->cfg.vocab, VP = M->VP, depth = (int)M->layers.size(), R = M->R;
    // logits in IEEE half like the reference's logit window: a third of the traffic of fp32 logits written once and read twice
    CK(FinalLogits(M, M->logits16, s));
    CK(Ts2ZeroRows(Flat(M->lossSum, 1, 1, TS2_F32).P(), 1, 4, s));
    CK(Ts2FinalSoftmaxGradHalf(R, V, M->logits16.P(), M->bias, M->target, 1.f, M->gradV.P(), M->lossSum, s));
    // dfn = grad * Wf / sqrt(D): bf16 product, the 8-bit weights converted exactly
    // (columns V..VP of the logits are products with zero rows, the same columns of the gradient stay zero: the softmax pass covers V)
    if (!M->finalW.fastTValid) { // kept until the matrix is set or updated, like the layer matrices' transposes
        CK(Ts2TransposeToBf16(VP, VP, D, M->finalW.fast.P(), M->mode, M->wfT.P(), s));
        M->finalW.fastTValid = true;
    }
    ts2_gemm_args g = {};
    g.a = M->gradV.m;
    g.b = M->wfT.m;
    g.c = M->dNormState.m;
    g.abType = TS2_BF16;
    g.cType = TS2_F32;
    g.m = R;
    g.n = D;
    g.k = VP;
    g.mLive = M->len;
    g.alpha = DISCR * Dot(D);
    g.alphaPtr = M->finalW.scale;
    g.epilogue = TS2_EPI_STORE;
    g.splitK = 1;
    CK(ts2_gemm_nt(&g, s));
    // delta_final[v][d] = sum_t grad[t][v] * fn[t][d]
    ts2_gemm_args h = {};
    if (M->len == R && (VP % 256) == 0 && (D % 256) == 0) {
        // whole row groups: the product contracts over the rows of the gradient and of the final state as they lie
        // (Fp16MatMul<1, 1, TStoreDelta>, gpu_final.cuh:265); the 8-bit state only changes its type
        Arr fn16 = Flat(M->fnT.m.ptr, R, D, TS2_BF16);
        CK(Ts2RowsToBf16(M->len, R, D, M->normState[depth].P(), M->mode, fn16.P(), s));
        h.a = M->gradV.m;
        h.b = fn16.m;
        h.kMajor = 1;
        h.tileConfig = 1;
    } else {
        CK(Ts2TransposeToBf16(M->len, R, VP, M->gradV.P(), TS2_BF16, M->gradVT.P(), s));
        CK(Ts2TransposeToBf16(M->len, R, D, M->normState[depth].P(), M->mode, M->fnT.P(), s));
        h.a = M->gradVT.m;
        h.b = M->fnT.m;
    }
    h.c = M->finalW.delta.m;
    h.abType = TS2_BF16;
    h.cType = TS2_I8;
    h.m = VP;
    h.n = D;
    h.k = R;
    h.alpha = VEC;
    h.epilogue = TS2_EPI_ROW_TILE_MAXNORM;
    h.tileScale = M->finalW.deltaTileScale.m;
    h.splitK = 1;
    // One workgroup per CU at a time: the 256-row groups of the vocabulary beyond the last full round of the chip would take a round of
    // their own at a fraction of the CUs.  They run as slices of the token axis instead (stored fp32 products, packed afterwards).
    const int tilesM = VP / 256, tilesN = D / 256, cus = M->cuCount;
    const int rowsPerRound = tilesN > 0 && cus % tilesN == 0 ? cus / tilesN : 0;
    const int tailRows = h.kMajor && rowsPerRound > 0 && tilesM > rowsPerRound ? tilesM % rowsPerRound : 0;
    int tailSplits = tailRows > 0 ? cus / (tailRows * tilesN) : 0;
    tailSplits = tailSplits > 8 ? 8 : tailSplits;
    if (tailSplits >= 2 && R / tailSplits >= 2048 && (size_t)tailSplits * tailRows * 256 * D <= M->sPartialFloats) {
        const int mainM = (tilesM - tailRows) * 256, tailM = tailRows * 256;
        h.m = mainM;
        CK(ts2_gemm_nt(&h, s));
        ts2_gemm_args t = h;
        t.a.ptr = (uint8_t *)h.a.ptr + (size_t)mainM * 2; // columns mainM.. of the gradient [token][vocabulary]
        t.a.x = tailM;
        t.m = tailM;
        Arr part = Flat(M->sPartial, tailSplits * tailM, D, TS2_F32);
        t.c = part.m;
        t.c.y = tailM;
        t.cType = TS2_F32;
        t.alpha = 1.f;
        t.epilogue = TS2_EPI_STORE;
        t.tileScale = ts2_mat{};
        t.splitK = tailSplits;
        t.splitSlabBytes = (int64_t)tailM * part.m.strideBytes;
        CK(ts2_gemm_nt(&t, s));
        ts2_mat dTail = M->finalW.delta.m, sTail = M->finalW.deltaTileScale.m;
        dTail.ptr = (uint8_t *)dTail.ptr + (size_t)mainM * dTail.strideBytes;
        dTail.y = tailM;
        sTail.ptr = (uint8_t *)sTail.ptr + (size_t)mainM * 4; // tile scales are [D / 128][vocabulary row]
        sTail.x = tailM;
        CK(ts2_pack_delta(&part.m, tailSplits, t.splitSlabBytes, tailM, D, VEC, nullptr, &dTail, &sTail, s));
    } else {
        CK(ts2_gemm_nt(&h, s));
    }
    return ts2_backprop_final_normalize(M->len, R, M->normState[depth].P(), M->mode, M->stateScale[depth].P(), M->dNormState.P(), M->stateGrad.P(),
        M->stateGradFast.P(), M->fastGradType, M->gradMaxNorm, s);
}

// CreateBackpropGraph, src/gpt/compute/gpu_transformer.cu:326-471 (one device, one micro batch)
int ModelBackprop(ts2_model *M, void *s)
{
    int D = M->cfg.dim, depth = (int)M->layers.size();
    CK(ModelForward(M, s));
    CK(Ts2ZeroRows(Flat(M->gradMaxNorm, 1, depth + 2, TS2_F32).P(), 1, (depth + 2) * 4, s));
    CK(Ts2FillFloats(M->gradMult, 1, 1.f, s)); // the multiplier the final normalisation applies to the fast gradient
    CK(FinalBackward(M, s));
    M->useKept = M->keep;
    struct TReset {
        ts2_model *M;
        ~TReset() { M->useKept = false; }
    } reset = {M};
    int stepId = 0;
    for (int d = depth - 1; d >= 0; --d, ++stepId) {
        float *prevMax = M->gradMaxNorm + stepId, *nextMax = M->gradMaxNorm + stepId + 1;
        float *gradScale = M->gradScale + stepId + 1, *gradMult = M->gradMult + stepId + 1;
        // the fast gradient is rewritten only when its power-of-two multiplier differs from the one its producer applied (the final
        // normalisation: 1, kept in gradMult[0]; a layer's normalisation backward: that layer's multiplier)
        CK(ts2_scale_grad(prevMax, M->gradMult + stepId, M->stateGrad.P(), M->stateGradFast.P(), M->fastGradType, M->len, gradScale, gradMult, s));
        CK(LayerBackward(M, d, gradScale, s));
        CK(ts2_backprop_layer_normalize(M->normState[d].P(), M->mode, M->stateScale[d].P(), M->dNormState.P(), nullptr, gradScale, gradMult,
            M->stateGrad.P(), M->stateGradFast.P(), M->fastGradType, nextMax, M->len, s));
    }
    return Ts2EmbedBackward(M->len, D, M->labelPtr, M->labels, M->stateGrad.P(), Flat(M->embed.delta.m.ptr, M->cfg.labelCount, D, TS2_F32).P(),
        M->cfg.labelCount, s);
}
} // namespace

extern "C" ts2_model *ts2_model_create(const ts2_model_config *cfg)
{
    if (!cfg || cfg->depth <= 0 || cfg->dim % 128 || cfg->vocab % 128 || cfg->maxLen <= 0 || (cfg->mode != TS2_I8 && cfg->mode != TS2_E4M3)) {
        return nullptr;
    }
    ts2_model *M = new ts2_model();
    M->cfg = *cfg;
    M->mode = cfg->mode;
    M->fastGradType = cfg->mode == TS2_I8 ? TS2_BF16 : TS2_E4M3;
    if (ts2_device_info(&M->cuCount, nullptr) != TS2_OK || M->cuCount <= 0) {
        delete M;
        return nullptr;
    }
    M->kTile = cfg->kTile > 0 ? cfg->kTile : 512;
    M->R = RoundUp(cfg->maxLen, M->kTile > 128 ? M->kTile : 128);
    int D = cfg->dim, H = cfg->headCount, F = cfg->ffnDim, X = cfg->expertDim, E = cfg->expertCount, V = cfg->vocab, R = M->R;
    int SelectDim = E > 0 ? RoundUp(E, 128) : 0;
    bool hasMoe = false;
    for (int d = 0; d < cfg->depth; ++d) {
        M->layerType.push_back(cfg->layerType[d]);
        M->layerAttId.push_back(cfg->layerAttId[d]);
        M->layerSlope.push_back(cfg->layerSlope[d]);
        hasMoe |= cfg->layerType[d] == LT_MOE;
    }
    if (hasMoe && (cfg->mode != TS2_E4M3 || E <= 0 || X % 128)) {
        delete M;
        return nullptr;
    }
    M->lenMoe = hasMoe ? RoundUp(R * cfg->moeSelected + 128 * E, 128) : 0;
    M->RP = R > M->lenMoe ? R : M->lenMoe;
    int maxW = D;
    maxW = F > maxW ? F : maxW;
    maxW = H * 128 > maxW ? H * 128 : maxW;
    if (hasMoe) {
        maxW = X > maxW ? X : maxW;
        maxW = SelectDim > maxW ? SelectDim : maxW;
    }
    M->maxW = maxW;
    bool ok = true;
    ok &= InitMatrix(M, &M->embed, D, cfg->labelCount, 1, false) == 0; // delta storage reused as fp32 [labelCount][D]: allocate separately below
    ok &= M->Alloc(&M->embed.delta, cfg->labelCount, D, TS2_F32);
    M->VP = (V >= 4096 && V % 256) ? RoundUp(V, 256) : V;
    const int VP = M->VP;
    ok &= InitMatrix(M, &M->finalW, D, VP, 1, false) == 0;
    M->bias = (float *)M->Dev((size_t)V * 4);
    M->layers.resize(cfg->depth);
    for (int d = 0; d < cfg->depth && ok; ++d) {
        TLayer &L = M->layers[d];
        L.type = cfg->layerType[d];
        L.slope = cfg->layerSlope[d];
        L.attId = cfg->layerAttId[d];
        if (L.type == LT_ATT) {
            for (int k = 0; k < 4; ++k) {
                ok &= InitMatrix(M, &L.w[k], D, H * 128, 1) == 0;
            }
            ok &= InitMatrix(M, &L.w[4], H * 128, D, 1) == 0;
            const int Q = H * 128;
            if (ok && M->mode == TS2_E4M3 && 4 * Q <= maxW && (Q % 256) == 0 && (D % 256) == 0) {
                L.qkvg.srcDim = D;
                L.qkvg.dstDim = 4 * Q;
                ok &= M->Alloc(&L.qkvg.delta, 4 * Q, D, TS2_I8) && M->Alloc(&L.qkvg.deltaTileScale, D / 128, 4 * Q, TS2_F32);
                for (int k = 0; k < 4 && ok; ++k) {
                    L.w[k].delta = L.qkvg.delta;
                    L.w[k].delta.m.ptr = (uint8_t *)L.qkvg.delta.m.ptr + (size_t)k * Q * L.qkvg.delta.m.strideBytes;
                    L.w[k].delta.m.y = Q;
                    L.w[k].deltaTileScale = L.qkvg.deltaTileScale;
                    L.w[k].deltaTileScale.m.ptr = (uint8_t *)L.qkvg.deltaTileScale.m.ptr + (size_t)k * Q * 4;
                    L.w[k].deltaTileScale.m.x = Q;
                }
                L.fusedDelta = ok;
            }
        } else if (L.type == LT_FFN) {
            ok &= InitMatrix(M, &L.w[0], D, F, 1) == 0;
            ok &= InitMatrix(M, &L.w[1], D, F, 1) == 0;
            ok &= InitMatrix(M, &L.w[2], F, D, 1) == 0;
        } else if (L.type == LT_MOE) {
            ok &= InitMatrix(M, &L.w[0], D, X, E) == 0;
            ok &= InitMatrix(M, &L.w[1], D, X, E) == 0;
            ok &= InitMatrix(M, &L.w[2], X, D, E) == 0;
            ok &= InitMatrix(M, &L.w[3], D, SelectDim, 1) == 0;
        } else {
            ok = false;
        }
    }
    // batch
    M->labelCap = R * 4;
    M->labelPtr = (int *)M->Dev((size_t)(R + 1) * 4);
    M->labels = (uint32_t *)M->Dev((size_t)M->labelCap * 4);
    M->target = (int *)M->Dev((size_t)R * 4);
    for (int a = 0; a < cfg->attTypeCount; ++a) {
        M->spanStart.push_back((int *)M->Dev((size_t)R * 4));
        M->spanFinish.push_back((int *)M->Dev((size_t)R * 4));
        M->revLo.push_back((int *)M->Dev((size_t)(R / 128) * 4));
        M->revHi.push_back((int *)M->Dev((size_t)(R / 128) * 4));
    }
    ok &= M->Alloc(&M->rope, R, 128, TS2_F32);
    // states
    ok &= M->Alloc(&M->state, R, D, TS2_F32) && M->Alloc(&M->stateGrad, R, D, TS2_F32) && M->Alloc(&M->stateGradFast, R, D, M->fastGradType) &&
          M->Alloc(&M->dNormState, R, D, TS2_F32);
    M->normState.resize(cfg->depth + 1);
    M->stateScale.resize(cfg->depth + 1);
    for (int d = 0; d <= cfg->depth; ++d) {
        ok &= M->Alloc(&M->normState[d], R, D, M->mode) && M->Alloc(&M->stateScale[d], D / 128, R, TS2_F32);
    }
    M->gradMaxNorm = (float *)M->Dev((size_t)(cfg->depth + 2) * 4);
    M->gradScale = (float *)M->Dev((size_t)(cfg->depth + 2) * 4);
    M->gradMult = (float *)M->Dev((size_t)(cfg->depth + 2) * 4);
    M->lossSum = (float *)M->Dev(4);
    // layer scratch
    int RP = M->RP;
    ok &= M->Alloc(&M->raw, RP, maxW, TS2_F32) && M->Alloc(&M->g32, RP, maxW, TS2_F32) && M->Alloc(&M->shared.rg8, RP, maxW, M->mode);
    for (int k = 0; k < 4; ++k) {
        ok &= M->Alloc(&M->shared.a16[k], RP, maxW, TS2_BF16) && M->Alloc(&M->g16[k], RP, maxW, TS2_BF16) &&
              M->Alloc(&M->gf[k], RP, maxW, M->fastGradType);
    }
    for (int k = 0; k < 2; ++k) {
        ok &= M->Alloc(&M->shared.tsc[k], maxW / 128, RP, TS2_F32);
    }
    ok &= M->Alloc(&M->shared.val16, RP, maxW, TS2_BF16);
    ok &= M->Alloc(&M->shared.swl, H > 0 ? H : 1, R, TS2_F32) && M->Alloc(&M->dScale, H > 0 ? H : 1, R, TS2_F32);
    // per-layer activation sets when they fit into half of the free device memory, else every layer shares one set and recomputes
    {
        size_t need = 0;
        for (int d = 0; d < cfg->depth; ++d) {
            int w = M->layers[d].type == LT_FFN ? F : H * 128;
            if (M->layers[d].type == LT_FFN) {
                need += (size_t)R * w * 5 + (size_t)R * (w / 128) * 4;
            } else if (M->layers[d].type == LT_ATT) {
                need += (size_t)R * w * 11 + (size_t)R * H * 12;
            }
        }
        size_t freeB = 0, totalB = 0;
        bool fits = hipMemGetInfo(&freeB, &totalB) == hipSuccess && need < freeB / 2;
        M->keep = ok && fits && cfg->recompute == 0;
        M->acts.resize(cfg->depth);
        for (int d = 0; d < cfg->depth && ok; ++d) {
            TLayer &L = M->layers[d];
            TActs &A = M->acts[d];
            L.acts = &M->shared;
            if (!M->keep || L.type == LT_MOE) {
                continue;
            }
            L.acts = &A;
            if (L.type == LT_FFN) {
                ok &= M->Alloc(&A.a16[0], R, F, TS2_BF16) && M->Alloc(&A.a16[1], R, F, TS2_BF16) && M->Alloc(&A.tsc[0], F / 128, R, TS2_F32) &&
                      M->Alloc(&A.rg8, R, F, M->mode);
            } else {
                int Q = H * 128;
                for (int k = 0; k < 4; ++k) {
                    ok &= M->Alloc(&A.a16[k], R, Q, TS2_BF16);
                }
                ok &= M->Alloc(&A.tsc[0], H, R, TS2_F32) && M->Alloc(&A.tsc[1], H, R, TS2_F32) && M->Alloc(&A.val16, R, Q, TS2_BF16) &&
                      M->Alloc(&A.rg8, R, Q, M->mode) && M->Alloc(&A.swl, H, R, TS2_F32);
            }
        }
    }
    // keep the two statistics arrays on one stride
    M->sGrad8 = (uint8_t *)M->Dev((size_t)RP * maxW);
    M->sGradT = (uint8_t *)M->Dev((size_t)RP * maxW);
    if (M->mode == TS2_E4M3) {
        M->sGradTa = (uint8_t *)M->Dev((size_t)RP * maxW);
        M->sGradTb = (uint8_t *)M->Dev((size_t)RP * maxW);
        ok &= M->sGradTa && M->sGradTb;
    }
    M->sSrcT = (uint8_t *)M->Dev((size_t)RP * maxW);
    M->sWT = (uint8_t *)M->Dev((size_t)4 * maxW * maxW); // up to four transposed weights side by side (BackpropDXGroup)
    M->sPartialFloats = (size_t)8 * 2048 * 2048; // eight slices of a 2048 x 2048 delta, four of a 4096 x 2048 one
    M->sPartial = (float *)M->Dev(M->sPartialFloats * 4);
    M->sRowScale = (float *)M->Dev((size_t)RP * 4);
    M->sTileMax = (float *)M->Dev((size_t)(RP / 128 + 1) * 4);
    M->sTileScale = (float *)M->Dev((size_t)(RP / 128 + 1) * 4);
    if (hasMoe) {
        int total = R * cfg->moeSelected;
        M->moe.sampleExpertIds = (int *)M->Dev((size_t)total * 4);
        M->moe.sampleExpertWeights = (float *)M->Dev((size_t)total * 4);
        M->moe.sampleExpertOffset = (int *)M->Dev((size_t)total * 4);
        M->moe.expertOffset = (int *)M->Dev((size_t)(E + 2) * 4);
        M->moe.xpTileExpertId = (int *)M->Dev((size_t)(M->lenMoe / 128) * 4);
        M->moe.xpSampleId = (int *)M->Dev((size_t)M->lenMoe * 4);
        M->moe.xpSampleWeight = (float *)M->Dev((size_t)M->lenMoe * 4);
        M->moe.blockCounts = (int *)M->Dev((size_t)((total + 255) / 256) * E * 4);
        M->dExpertWeight = (float *)M->Dev((size_t)M->lenMoe * 4);
        ok &= M->Alloc(&M->normMoe, M->lenMoe, D, M->mode) && M->Alloc(&M->sgMoe, M->lenMoe, D, M->fastGradType) &&
              M->Alloc(&M->moeSel, R, SelectDim, TS2_F32) && M->Alloc(&M->dMoeSel, R, SelectDim, M->fastGradType);
    }
    ok &= M->Alloc(&M->logits, R, VP, TS2_F32) && M->Alloc(&M->logits16, R, VP, TS2_F16) && M->Alloc(&M->gradV, R, VP, TS2_BF16) && M->Alloc(&M->gradVT, VP, R, TS2_BF16) &&
          M->Alloc(&M->fnT, D, R, TS2_BF16) && M->Alloc(&M->wfT, D, VP, TS2_BF16);
    if (!ok || !M->sGrad8 || !M->sGradT || !M->sSrcT || !M->sWT || !M->sPartial) {
        delete M;
        return nullptr;
    }
    return M;
}

extern "C" void ts2_model_destroy(ts2_model *M)
{
    delete M;
}

static int Ts2ValidateBatch(int len, int labelCap, int labelCount, int vocab, int attTypeCount, const int32_t *labelPtr, const uint32_t *labels,
    const int32_t *targetPerRow, const int32_t *const *spanStart, const int32_t *const *spanFinish)
{
    if (!labelPtr || !labels || !targetPerRow || (attTypeCount > 0 && (!spanStart || !spanFinish))) {
        return TS2_ERR_NULL;
    }
    if (len <= 0 || labelPtr[0] != 0) {
        return TS2_ERR_SHAPE;
    }
    for (int t = 0; t < len; ++t) {
        if (labelPtr[t + 1] < labelPtr[t] || labelPtr[t + 1] > labelCap) {
            return TS2_ERR_SHAPE;
        }
        if (targetPerRow[t] < -1 || targetPerRow[t] >= vocab) {
            return TS2_ERR_SHAPE;
        }
    }
    for (int i = 0, n = labelPtr[len]; i < n; ++i) {
        if ((labels[i] & 0x7fffffffu) >= (uint32_t)labelCount) {
            return TS2_ERR_SHAPE;
        }
    }
    for (int a = 0; a < attTypeCount; ++a) {
        if (!spanStart[a] || !spanFinish[a]) {
            return TS2_ERR_NULL;
        }
        for (int t = 0; t < len; ++t) {
            const int st = spanStart[a][t], fi = spanFinish[a][t];
            if (st < 0 || st > len || fi >= len || fi < -1) {
                return TS2_ERR_SHAPE;
            }
        }
    }
    return 0;
}

static TMatrix *FindMatrix(ts2_model *M, int layer, int matrixId)
{
    if (layer == TS2_LAYER_EMBED) {
        return &M->embed;
    }
    if (layer == TS2_LAYER_FINAL) {
        return &M->finalW;
    }
    if (layer < 0 || layer >= (int)M->layers.size() || matrixId < 0 || matrixId >= 5 || !M->layers[layer].w[matrixId].fast.m.ptr) {
        return nullptr;
    }
    return &M->layers[layer].w[matrixId];
}

extern "C" int ts2_model_set_matrix(ts2_model *M, int32_t layer, int32_t matrixId, const void *fastHost, int32_t rows, int32_t cols, float scale)
{
    TMatrix *W = M ? FindMatrix(M, layer, matrixId) : nullptr;
    if (!W || !fastHost) {
        return TS2_ERR_NULL;
    }
    if (cols != W->srcDim || rows > W->dstDim * W->slabs) {
        return TS2_ERR_SHAPE;
    }
    if (Copy2D(W->fast.m.ptr, W->fast.m.strideBytes, fastHost, cols, cols, rows, hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(W->scale, &scale, 4, hipMemcpyHostToDevice) != hipSuccess) {
        return TS2_ERR_LAUNCH;
    }
    W->fastTValid = false; // the kept transpose belongs to the old weights
    return 0;
}

// master weights of a matrix: allocates its optimiser state on first use, uploads the fp32 weights and derives the fast weights and the
// matrix scale from them on the device (TAgpuCudaModelMatrix::CopyToDevice, src/gpt/matrix/agpu_cuda.cuh:473-482)
extern "C" int ts2_model_set_master(ts2_model *M, int32_t layer, int32_t matrixId, const float *weightsHost, int32_t rows, int32_t cols,
    int32_t rowDispSize, float sparsity)
{
    TMatrix *W = M ? FindMatrix(M, layer, matrixId) : nullptr;
    if (!W || !weightsHost) {
        return TS2_ERR_NULL;
    }
    if (cols != W->srcDim || rows <= 0 || rows > W->dstDim * W->slabs || rowDispSize <= 0 || rows % rowDispSize) {
        return TS2_ERR_SHAPE;
    }
    if (W->hasOpt && W->optRows != rows) {
        return TS2_ERR_SHAPE;
    }
    if (!W->hasOpt) {
        ts2_opt_matrix &o = W->opt;
        bool ok = M->Alloc(&W->optWeights, rows, cols, TS2_F32) && M->Alloc(&W->optAvgGrad, rows, cols, TS2_F32);
        o.gradRowSum2 = (float *)M->Dev((size_t)rows * 4);
        o.weightsRowSum2 = (float *)M->Dev((size_t)rows * 4);
        o.rowScale = (float *)M->Dev((size_t)rows * 4);
        o.rowDisp = (float *)M->Dev((size_t)rows * 4); // room for any later rowDispSize
        o.sumWeight = (float *)M->Dev(4);
        o.sparsity = (float *)M->Dev(4);
        o.convertMult = (float *)M->Dev(4);
        if (!ok || !o.gradRowSum2 || !o.weightsRowSum2 || !o.rowScale || !o.rowDisp || !o.sumWeight || !o.sparsity || !o.convertMult) {
            return TS2_ERR_LAUNCH;
        }
        o.xSize = cols;
        o.ySize = rows;
        o.yBufSize = W->fast.m.y; // the conversion also clears the padding rows of the fast matrix
        o.weights = W->optWeights.m;
        o.avgGrad = W->optAvgGrad.m;
        o.fast = W->fast.m;
        o.fastType = M->mode;
        o.matrixScale = W->scale;
        W->optRows = rows;
        W->hasOpt = true;
    }
    W->opt.rowDispSize = rowDispSize;
    if (Copy2D(W->optWeights.m.ptr, W->optWeights.m.strideBytes, weightsHost, (size_t)cols * 4, (size_t)cols * 4, rows, hipMemcpyHostToDevice) !=
            hipSuccess ||
        hipMemcpy(W->opt.sparsity, &sparsity, 4, hipMemcpyHostToDevice) != hipSuccess ||
        hipMemset(W->optAvgGrad.m.ptr, 0, (size_t)W->optAvgGrad.m.strideBytes * rows) != hipSuccess ||
        hipMemset(W->opt.rowDisp, 0, (size_t)rows * 4) != hipSuccess || hipMemset(W->opt.sumWeight, 0, 4) != hipSuccess) {
        return TS2_ERR_LAUNCH;
    }
    W->fastTValid = false;
    return ts2_opt_convert(&W->opt, nullptr);
}

// one optimiser step over every matrix that has master weights: the packed delta of the last ts2_model_backprop is applied
// (TAgpuCudaModelMatrix::AddDelta with BM_GRAD_APPLY, agpu_cuda.cuh:564-590; the embedding's delta is fp32 and goes through the
// unpacked sequence, :536-562), new fast weights and scales replace the old ones and the kept transposes are dropped
extern "C" int ts2_model_apply_deltas(ts2_model *M, const ts2_add_gradient_params *paramsHost, void *stream)
{
    if (!M || !paramsHost) {
        return TS2_ERR_NULL;
    }
    if (!M->optParams) {
        M->optParams = (ts2_add_gradient_params *)M->Dev(sizeof(ts2_add_gradient_params));
        if (!M->optParams) {
            return TS2_ERR_LAUNCH;
        }
    }
    if (hipMemcpyAsync(M->optParams, paramsHost, sizeof(ts2_add_gradient_params), hipMemcpyHostToDevice, (hipStream_t)stream) != hipSuccess) {
        return TS2_ERR_LAUNCH;
    }
    auto apply = [&](TMatrix &W, bool packed) -> int {
        if (!W.hasOpt) {
            return 0;
        }
        W.fastTValid = false;
        const ts2_opt_matrix &o = W.opt;
        if (packed) {
            return ts2_opt_add_delta(&o, W.delta.P(), W.deltaTileScale.P(), TS2_BM_GRAD_APPLY, M->optParams, stream);
        }
        CK(ts2_matrix_row_sum2(o.xSize, o.ySize, W.delta.P(), o.gradRowSum2, stream));
        CK(ts2_update_global_row_disp(o.xSize, o.ySize, o.rowDispSize, o.gradRowSum2, M->optParams, o.sumWeight, o.rowDisp, o.rowScale, stream));
        CK(ts2_add_gradient(o.xSize, o.ySize, W.delta.P(), M->optParams, o.rowScale, o.sparsity, &o.avgGrad, &o.weights, o.weightsRowSum2, stream));
        return ts2_convert_matrix(o.xSize, o.ySize, o.yBufSize, o.xSize, o.ySize, &o.weights, o.weightsRowSum2, &o.fast, o.fastType, o.matrixScale,
            o.convertMult, stream);
    };
    CK(apply(M->embed, false));
    CK(apply(M->finalW, true));
    for (TLayer &L : M->layers) {
        for (int k = 0; k < 5; ++k) {
            if (L.w[k].fast.m.ptr) {
                CK(apply(L.w[k], true));
            }
        }
    }
    return 0;
}

// host copy of a matrix's master weights [rows][cols] (synchronises the device)
extern "C" int ts2_model_get_master(ts2_model *M, int32_t layer, int32_t matrixId, float *hostOut, int32_t rows, int32_t cols)
{
    TMatrix *W = M ? FindMatrix(M, layer, matrixId) : nullptr;
    if (!W || !hostOut) {
        return TS2_ERR_NULL;
    }
    if (!W->hasOpt || rows != W->optRows || cols != W->srcDim) {
        return TS2_ERR_SHAPE;
    }
    if (hipDeviceSynchronize() != hipSuccess ||
        Copy2D(hostOut, (size_t)cols * 4, W->optWeights.m.ptr, W->optWeights.m.strideBytes, (size_t)cols * 4, rows, hipMemcpyDeviceToHost) != hipSuccess) {
        return TS2_ERR_LAUNCH;
    }
    return 0;
}

// host copy of a matrix's fast weights [rows][cols] bytes and its scale (synchronises the device)
extern "C" int ts2_model_get_matrix(ts2_model *M, int32_t layer, int32_t matrixId, void *fastHostOut, int32_t rows, int32_t cols, float *scaleOut)
{
    TMatrix *W = M ? FindMatrix(M, layer, matrixId) : nullptr;
    if (!W || !fastHostOut || !scaleOut) {
        return TS2_ERR_NULL;
    }
    if (cols != W->srcDim || rows > W->dstDim * W->slabs) {
        return TS2_ERR_SHAPE;
    }
    if (hipDeviceSynchronize() != hipSuccess ||
        Copy2D(fastHostOut, cols, W->fast.m.ptr, W->fast.m.strideBytes, cols, rows, hipMemcpyDeviceToHost) != hipSuccess ||
        hipMemcpy(scaleOut, W->scale, 4, hipMemcpyDeviceToHost) != hipSuccess) {
        return TS2_ERR_LAUNCH;
    }
    return 0;
}

extern "C" int ts2_model_set_bias(ts2_model *M, const float *biasHost)
{
    if (!M || !biasHost) {
        return TS2_ERR_NULL;
    }
    return hipMemcpy(M->bias, biasHost, (size_t)M->cfg.vocab * 4, hipMemcpyHostToDevice) == hipSuccess ? 0 : TS2_ERR_LAUNCH;
}

// Host-side check of a batch (no device access): label CSR monotone and within capacity, label ids (low 31 bits; the top bit is the
// sign of the embedding term) below labelCount, targets in [-1, vocab), every span with 0 <= start <= len and -1 <= finish < len (finish < start = empty).
extern "C" int ts2_validate_batch(int32_t len, int32_t labelCap, int32_t labelCount, int32_t vocab, int32_t attTypeCount, const int32_t *labelPtr,
    const uint32_t *labels, const int32_t *targetPerRow, const int32_t *const *spanStart, const int32_t *const *spanFinish)
{
    return Ts2ValidateBatch(len, labelCap, labelCount, vocab, attTypeCount, labelPtr, labels, targetPerRow, spanStart, spanFinish);
}

extern "C" int ts2_model_set_batch(ts2_model *M, int32_t len, const int32_t *labelPtr, const uint32_t *labels, const int32_t *targetPerRow,
    const int32_t *const *spanStart, const int32_t *const *spanFinish, const float *ropeBuf, void *stream)
{
    if (!M || !labelPtr || !labels || !targetPerRow || !ropeBuf) {
        return TS2_ERR_NULL;
    }
    if (len <= 0 || len > M->cfg.maxLen) {
        return TS2_ERR_SHAPE;
    }
    // every index the kernels follow is checked here, before anything is copied: a label, a target or a span outside its range would
    // be an out-of-bounds access on the device (embedding rows, logit columns, key rows of the attention)
    int rcBatch = Ts2ValidateBatch(len, M->labelCap, M->cfg.labelCount, M->cfg.vocab, M->cfg.attTypeCount, labelPtr, labels, targetPerRow,
        spanStart, spanFinish);
    if (rcBatch != 0) {
        return rcBatch;
    }
    // the uploads below are blocking copies on the null stream; the step they feed must not still be running on a non-blocking stream
    if (stream && hipStreamSynchronize((hipStream_t)stream) != hipSuccess) {
        return TS2_ERR_LAUNCH;
    }
    M->len = len;
    int R = M->R;
    std::vector<int> tg(R, -1), st(R, 0), fi(R, -1);
    memcpy(tg.data(), targetPerRow, (size_t)len * 4);
    bool ok = hipMemcpy(M->labelPtr, labelPtr, (size_t)(len + 1) * 4, hipMemcpyHostToDevice) == hipSuccess;
    ok &= hipMemcpy(M->labels, labels, (size_t)labelPtr[len] * 4, hipMemcpyHostToDevice) == hipSuccess;
    ok &= hipMemcpy(M->target, tg.data(), (size_t)R * 4, hipMemcpyHostToDevice) == hipSuccess;
    ok &= Copy2D(M->rope.m.ptr, M->rope.m.strideBytes, ropeBuf, 128 * 4, 128 * 4, len, hipMemcpyHostToDevice) == hipSuccess;
    for (int a = 0; a < M->cfg.attTypeCount && ok; ++a) {
        std::fill(st.begin(), st.end(), 0);
        std::fill(fi.begin(), fi.end(), -1);
        memcpy(st.data(), spanStart[a], (size_t)len * 4);
        memcpy(fi.data(), spanFinish[a], (size_t)len * 4);
        ok &= hipMemcpy(M->spanStart[a], st.data(), (size_t)R * 4, hipMemcpyHostToDevice) == hipSuccess;
        ok &= hipMemcpy(M->spanFinish[a], fi.data(), (size_t)R * 4, hipMemcpyHostToDevice) == hipSuccess;
        if (ok) {
            int rc = ts2_att_build_rev(len, R, M->spanStart[a], M->spanFinish[a], M->revLo[a], M->revHi[a], stream);
            if (rc) {
                return rc;
            }
        }
    }
    return ok ? 0 : TS2_ERR_LAUNCH;
}

extern "C" int ts2_model_forward(ts2_model *M, void *stream)
{
    if (!M || M->len <= 0) {
        return TS2_ERR_NULL;
    }
    CK(ModelForward(M, stream));
    CK(FinalLogits(M, M->logits, stream));
    // probabilities in place of the logits; the gradient buffer is scratch here
    return Ts2FinalSoftmaxGrad(M->R, M->cfg.vocab, M->logits.P(), M->bias, M->target, 1.f, M->gradV.P(), nullptr, 1, stream);
}

extern "C" int ts2_model_backprop(ts2_model *M, void *stream)
{
    if (!M || M->len <= 0) {
        return TS2_ERR_NULL;
    }
    return ModelBackprop(M, stream);
}

extern "C" int ts2_layer_backward(ts2_model *M, int32_t layer, void *stream)
{
    if (!M || M->len <= 0 || layer < 0 || layer >= (int)M->layers.size()) {
        return TS2_ERR_NULL;
    }
    // gradient scale bookkeeping of one step of the backward loop, fed from stateGrad as it stands
    CK(ts2_scale_grad(M->gradMaxNorm, nullptr, M->stateGrad.P(), M->stateGradFast.P(), M->fastGradType, M->len, M->gradScale, M->gradMult, stream));
    CK(LayerBackward(M, layer, M->gradScale, stream));
    return ts2_backprop_layer_normalize(M->normState[layer].P(), M->mode, M->stateScale[layer].P(), M->dNormState.P(), nullptr, M->gradScale,
        M->gradMult, M->stateGrad.P(), M->stateGradFast.P(), M->fastGradType, M->gradMaxNorm + 1, M->len, stream);
}

extern "C" int ts2_layer_forward(ts2_model *M, int32_t layer, void *stream)
{
    if (!M || M->len <= 0 || layer < 0 || layer >= (int)M->layers.size()) {
        return TS2_ERR_NULL;
    }
    CK(ts2_layer_normalize_state_vecs(M->state.P(), TS2_F32, M->len, M->R, VEC, M->normState[layer].P(), M->mode, M->stateScale[layer].P(), stream));
    return LayerForward(M, layer, stream);
}

extern "C" int ts2_model_get_delta(ts2_model *M, int32_t layer, int32_t matrixId, float *hostOut, int32_t rows, int32_t cols)
{
    TMatrix *W = M ? FindMatrix(M, layer, matrixId) : nullptr;
    if (!W || !hostOut) {
        return TS2_ERR_NULL;
    }
    if (cols != W->srcDim || rows > W->dstDim * W->slabs) {
        return TS2_ERR_SHAPE;
    }
    if (hipDeviceSynchronize() != hipSuccess) {
        return TS2_ERR_LAUNCH;
    }
    if (layer == TS2_LAYER_EMBED) {
        return Copy2D(hostOut, (size_t)cols * 4, W->delta.m.ptr, W->delta.m.strideBytes, (size_t)cols * 4, rows, hipMemcpyDeviceToHost) ==
                       hipSuccess
                   ? 0
                   : TS2_ERR_LAUNCH;
    }
    int allRows = W->dstDim * W->slabs;
    std::vector<int8_t> d((size_t)rows * cols);
    std::vector<float> ts((size_t)(cols / 128) * allRows);
    if (Copy2D(d.data(), cols, W->delta.m.ptr, W->delta.m.strideBytes, cols, rows, hipMemcpyDeviceToHost) != hipSuccess ||
        Copy2D(ts.data(), (size_t)allRows * 4, W->deltaTileScale.m.ptr, W->deltaTileScale.m.strideBytes, (size_t)allRows * 4, cols / 128,
            hipMemcpyDeviceToHost) != hipSuccess) {
        return TS2_ERR_LAUNCH;
    }
    for (int y = 0; y < rows; ++y) {
        for (int x = 0; x < cols; ++x) {
            hostOut[(size_t)y * cols + x] = d[(size_t)y * cols + x] * ts[(size_t)(x / 128) * allRows + y];
        }
    }
    return 0;
}

extern "C" int ts2_model_array(ts2_model *M, const char *name, int32_t index, ts2_mat *out, int32_t *type)
{
    if (!M || !name || !out) {
        return TS2_ERR_NULL;
    }
    const Arr *a = nullptr;
    Arr tmp;
    if (!strcmp(name, "expertOffset") && M->moe.expertOffset) {
        tmp = Flat(M->moe.expertOffset, 1, M->cfg.expertCount + 2, TS2_I32); // first grouped row of each expert, rows in use, capacity
        a = &tmp;
    } else if (!strncmp(name, "act.", 4) && index >= 0 && index < (int)M->layers.size() && M->layers[index].acts) {
        // what layer `index` keeps from its forward pass (in recompute mode and for MoE layers: the shared set, valid for the layer that
        // ran last).  FFN: wide, gate (bf16), wideScale, rg (8-bit); attention: q, gate, k, v (bf16), qScale, vScale, val (bf16; holds dQ
        // after the layer's backward), vlg (8-bit), sumWeightLog
        const TLayer &L = M->layers[index];
        const TActs &A = *L.acts;
        const int R = M->R, W = L.type == LT_FFN ? M->cfg.ffnDim : M->cfg.headCount * 128, T = W / 128;
        const char *f = name + 4;
        if (!strcmp(f, "a0") || !strcmp(f, "a1") || !strcmp(f, "a2") || !strcmp(f, "a3")) {
            tmp = View(A.a16[f[1] - '0'], R, W);
        } else if (!strcmp(f, "scale0") || !strcmp(f, "scale1")) {
            tmp = View(A.tsc[f[5] - '0'], T, R);
        } else if (!strcmp(f, "rg")) {
            tmp = View(A.rg8, R, W);
        } else if (!strcmp(f, "val")) {
            tmp = View(A.val16, R, W);
        } else if (!strcmp(f, "swl")) {
            tmp = A.swl;
        } else {
            return TS2_ERR_UNSUPPORTED;
        }
        if (!tmp.m.ptr) {
            return TS2_ERR_UNSUPPORTED;
        }
        a = &tmp;
    } else if (!strncmp(name, "scratch.", 8) && index > 0) {
        // gradient scratch of the layer backward that ran last, `index` columns wide: g0..g3 bf16 (drg / dvlg, dVal, dK, dV),
        // f0..f3 fast-gradient type (dwide / dq, dgate, dk, dv), dscale fp32 [heads][lenRound]
        const char *f = name + 8;
        if ((f[0] == 'g' || f[0] == 'f') && f[1] >= '0' && f[1] <= '3' && !f[2] && index <= M->maxW) {
            tmp = View(f[0] == 'g' ? M->g16[f[1] - '0'] : M->gf[f[1] - '0'], M->R, index);
        } else if (!strcmp(f, "dscale")) {
            tmp = M->dScale;
        } else {
            return TS2_ERR_UNSUPPORTED;
        }
        a = &tmp;
    } else if (!strcmp(name, "gradMaxNorm")) {
        tmp = Flat(M->gradMaxNorm, 1, (int)M->layers.size() + 2, TS2_F32); // running maxima of |stateGrad|: [0] feeds ts2_layer_backward
        a = &tmp;
    } else if (!strcmp(name, "finalGrad")) {
        a = &M->gradV; // bf16 [lenRound][vocab]: the soft-max gradient of the last ts2_model_backprop
    } else if (!strcmp(name, "state")) {
        a = &M->state;
    } else if (!strcmp(name, "stateGrad")) {
        a = &M->stateGrad;
    } else if (!strcmp(name, "stateGradFast")) {
        a = &M->stateGradFast;
    } else if (!strcmp(name, "dNormState")) {
        a = &M->dNormState;
    } else if (!strcmp(name, "prediction")) {
        a = &M->logits;
    } else if (!strcmp(name, "normState") && index >= 0 && index < (int)M->normState.size()) {
        a = &M->normState[index];
    } else if (!strcmp(name, "stateScale") && index >= 0 && index < (int)M->stateScale.size()) {
        a = &M->stateScale[index];
    } else {
        return TS2_ERR_UNSUPPORTED;
    }
    *out = a->m;
    if (type) {
        *type = a->type;
    }
    return 0;
}

extern "C" int ts2_model_read(ts2_model *M, const char *name, int32_t index, void *hostOut, int64_t hostBytes)
{
    ts2_mat m;
    int32_t type = 0;
    int rc = ts2_model_array(M, name, index, &m, &type);
    if (rc != 0) {
        return rc;
    }
    int64_t rowBytes = (int64_t)m.x * ElemSz(type);
    if (!hostOut || hostBytes < rowBytes * m.y) {
        return TS2_ERR_SHAPE;
    }
    if (hipDeviceSynchronize() != hipSuccess ||
        Copy2D(hostOut, rowBytes, m.ptr, m.strideBytes, rowBytes, m.y, hipMemcpyDeviceToHost) != hipSuccess) {
        return TS2_ERR_LAUNCH;
    }
    return 0;
}

extern "C" int ts2_model_scalars(ts2_model *M, float *lossSumHost, int32_t *lenRound, int32_t *lenMoe)
{
    if (!M) {
        return TS2_ERR_NULL;
    }
    if (lossSumHost) {
        if (hipDeviceSynchronize() != hipSuccess || hipMemcpy(lossSumHost, M->lossSum, 4, hipMemcpyDeviceToHost) != hipSuccess) {
            return TS2_ERR_LAUNCH;
        }
    }
    if (lenRound) {
        *lenRound = M->R;
    }
    if (lenMoe) {
        *lenMoe = M->lenMoe;
    }
    return 0;
}
