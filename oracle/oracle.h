/*
 * CPU oracle for the TScale2 backward path.  TEST INFRASTRUCTURE ONLY: nothing outside tests/, the smoke check and the
 * cpu_baseline leg of the benchmark may link or load this.  Every function restates, loop for loop, one function of the
 * reference's fp32 CPU path (file:line given at each definition).  All matrices are dense row-major float arrays
 * [rows][cols]; "len" is the number of token rows.
 *
 * Pinning status (what each function is checked against in tests/; "ref" = the reference's own sources compiled into
 * oracle/_ref/libts2ref.so and the committed vectors they produced, tests/golden/ref_golden.npz):
 *   mul_forward, mul_backward_accum, sum_rank_one, normalize_state(+backward), lolu, backprop_lolu, fill_rope_buf, apply_rope,
 *   attention_forward, compute_dscale, attention_grad_q, attention_grad_k, transpose_attention, convert_i8, convert_e4m3,
 *   e4m3_to_float, cvt_i8, cvt_e4m3, model_schedule, make_causal_spans (+ the harness's labels and targets)
 *       -> bit-exact against ref (tests/test_oracle_vs_reference.py over tests/golden_cases.py).
 *   hist_sort_stable -> the hash the reference's own sort test holds for its Mersenne-twister input (tests/test_oracle_own_contract.py).
 *   unpack_delta, apply_delta -> closed forms of the update rule (tests/test_oracle_optim.py): unpack o compress = id within half a step,
 *       unit step length per row, geometric moving average, weight decay, block dispersion = mean over the block's rows.
 *   cvt_e4m3_rne, compress_delta, quantize_matrix_i8/e4m3, grad_mult, cpu_moe, cpu_backprop_moe, scale_experts,
 *   backprop_scale_experts, fwd/bwd_contract_matrix, layer_forward, layer_backward, final_backward, model_step
 *       -> their reference sources need cuda_runtime.h and cannot be compiled here; pinned by brute force over the code table,
 *          invariants, bilinear / adjoint identities and fp64 finite differences (tests/test_oracle_closed_forms.py).
 *   quant_rowmax_i8(_noise), quant_ktile_i8(_noise), gemm_i8_nt, gemm_i8_nt_rowscale, gemm_i8_nt_ktile, gemm_f32_nt, dequant_i8/e4m3, bf16_round,
 *   softmax2, embedding_forward/backward, and the same-contract layer functions (orc_sc_*)
 *       -> this library's own contracts and helpers: closed forms against numpy round-half-even and int64 products, torch's bfloat16
 *          conversion, scipy's softmax, adjoint identities (tests/test_oracle_own_contract.py, tests/test_same_contract_cpu.py).
 */
#ifndef TS2_ORACLE_H
#define TS2_ORACLE_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- constants: src/gpt/model_params/model_dim.h:9-29 ---- */
#define ORC_MODEL_DISCR_SCALE (1.f / 32)
#define ORC_LOG2 0.693147f
#define ORC_ATT_DOTPRODUCT_SCALE 0.5f
#define ORC_MOE_SCALE 0.5f
#define ORC_STATE_NORM_TILE 128
#define ORC_LOLU_SCALE 2.f

/* ---- linalg.c ---- */
void orc_mul_forward(const float *vec, const float *kqv, float *res, int len, int dim, int rDim);
void orc_mul_backward_accum(float *vecGrad, const float *kqv, const float *resGrad, int len, int dim, int rDim);
void orc_sum_rank_one(const float *vec, float *delta, const float *resGrad, int len, int dim, int rDim);
void orc_gemm_i8_nt(const int8_t *a, const int8_t *b, int32_t *c, int m, int n, int k);
void orc_gemm_i8_nt_rowscale(const int8_t *a, const float *aRowScale, const int8_t *b, float alpha, float *c, int m, int n, int k, int add);
void orc_gemm_i8_nt_ktile(const int8_t *a, const int8_t *b, const float *kTileScale, int kTile, float alpha, float *c, int m, int n, int k);
void orc_gemm_f32_nt(const float *a, const float *b, float *c, int m, int n, int k, float alpha, int add);

/* ---- norm_lolu.c ---- */
void orc_normalize_state(const float *state, float *res, int len, int dim, int headCount);
void orc_normalize_state_backward(const float *state, const float *dNorm, float *grad, int len, int dim, int headCount);
void orc_lolu(const float *gate, const float *vals, float *res, int len, int dim);
void orc_backprop_lolu(const float *gate, const float *vals, const float *grad, float *gradGate, float *gradVals, int len, int dim);

/* ---- attention.c ---- */
void orc_fill_rope_buf(float *buf, int width, int ropeLen);
void orc_apply_rope(const float *ropeBuf, int width, float dir, float *p, int len, int dim);
int orc_transpose_attention(int len, const int *spanPtr, const int *spans, int *resPtr, int *resSpans, int maxSpans);
void orc_make_causal_spans(int fragCount, int fragLen, int window, int *spanPtr, int *spans, int *spanCount);
void orc_attention_forward(int len, int heads, int qDim, int ttDim, float alibiSlope, float attScaleMult, const int *spanPtr,
    const int *spans, const float *q, const float *k, const float *v, float *valLookup, float *sumWeight, float *maxDP);
void orc_compute_dscale(int len, int heads, int ttDim, const float *valLookup, const float *dValLookup, float *dScale);
void orc_attention_grad_q(int len, int heads, int qDim, int ttDim, float alibiSlope, float attScaleMult, const int *spanPtr,
    const int *spans, const float *q, const float *k, const float *v, const float *dVal, const float *dScale, const float *sumWeight,
    const float *maxDP, float *dq);
void orc_attention_grad_k(int len, int heads, int qDim, int ttDim, float alibiSlope, float attScaleMult, const int *revPtr,
    const int *revSpans, const float *q, const float *k, const float *v, const float *dVal, const float *dScale, const float *sumWeight,
    const float *maxDP, float *dk, float *dv);

/* ---- quant.c ---- */
int8_t orc_cvt_i8(float x);
void orc_convert_i8(int8_t *dst, const float *src, int n, float mult);
uint8_t orc_cvt_e4m3(float x);
uint8_t orc_cvt_e4m3_rne(float x);
void orc_round_e4m3_rne(float *dst, const float *src, long n);
void orc_convert_e4m3(uint8_t *dst, const float *src, int n, float mult);
float orc_e4m3_to_float(int code);
float orc_quantize_matrix_i8(const float *w, int8_t *fast, int ySize, int xSize);
float orc_quantize_matrix_e4m3(const float *w, uint8_t *fast, int ySize, int xSize);
void orc_dequant_i8(const int8_t *fast, float *w, int n, float scale);
void orc_dequant_e4m3(const uint8_t *fast, float *w, int n, float scale);
void orc_compress_delta(const float *data, int8_t *delta, float *tileScale, int ySize, int xSize);
void orc_quant_rowmax_i8(const float *src, int8_t *dst, float *rowScale, int len, int dim);
void orc_quant_ktile_i8(const float *src, int8_t *dst, float *tileScale, int len, int dim, int kTile);
void orc_quant_rowmax_i8_noise(const float *src, const float *noise, int8_t *dst, float *rowScale, int len, int dim);
void orc_quant_ktile_i8_noise(const float *src, const float *noise, int8_t *dst, float *tileScale, int len, int dim, int kTile);
float orc_grad_mult(float maxNorm);
float orc_bf16_round(float x);

/* ---- sort.c ---- */
void orc_hist_sort_stable(const float *val, int nodeCount, int *order, int forceHist);
uint32_t orc_sort_result_hash(const int *order, int n);

/* ---- optim.c ---- */
typedef struct {
    float rate, l2Reg, beta1, weight0, weight1, dispDecay; /* TTrainingStep, src/gpt/train_config/train_step.h:4-27 */
} orc_train_step;
void orc_unpack_delta(const int8_t *delta, const float *tileScale, float *dst, int ySize, int xSize, int add);
double orc_apply_delta(float *weights, float *avgGrad, const float *delta, int ySize, int xSize, int rowDispSize, float *rowDisp, float *sumWeight,
    float sparsity, const orc_train_step *st, float *rowScaleOut);

/* ---- moe.c ---- */
void orc_cpu_moe(int len, int expertCount, int selectedCount, const float *moeSrc, float *res);
void orc_cpu_backprop_moe(int len, int expertCount, const float *moe, float *dMoe);
void orc_scale_experts(int len, int expertCount, int width, const float *moe, float *rg);
void orc_backprop_scale_experts(int len, int expertCount, int width, const float *moe, const float *rgSrc, float *gradMoe, float *gradRg);
void orc_fwd_contract_matrix(const float *src, float *res, int xpCount, int eSize, int xSize);
void orc_bwd_contract_matrix(const float *src, float *res, int xpCount, int eSize, int xSize);

/* ---- model.c ---- */
enum { ORC_LT_ATT = 0, ORC_LT_ATT_3LIN = 1, ORC_LT_FFN = 2, ORC_LT_MOE = 3 };

typedef struct {
    int dim, qDim, ttDim, headCount, ffnDim, expertDim, expertCount, moeSelected;
} orc_dims;

/* one layer's dequantised matrices (already multiplied by 1/32 and, except gate/select, by the matrix scale) */
typedef struct {
    int type;          /* ORC_LT_* */
    float alibiSlope;
    int attTypeId;
    const float *w[5]; /* MP_ATT_{Q,K,V,GATE,COMBINER} / MP_FFN_{EXPAND,GATE,CONTRACT} / MP_MOE_{EXPAND,GATE,CONTRACT,SELECT} */
    float *delta[5];   /* out (may be NULL): fp32 delta, same [out][in] shape as w */
} orc_layer;

typedef struct {
    int attTypeCount;
    const int *spanPtr[4];
    const int *spans[4];
    const int *revPtr[4];
    const int *revSpans[4];
    const float *ropeBuf; /* [len][qDim] */
} orc_common;

void orc_layer_forward(const orc_dims *d, const orc_layer *l, const orc_common *c, int len, const float *prevState, float *state);
void orc_layer_backward(const orc_dims *d, const orc_layer *l, const orc_common *c, int len, const float *prevState, float *grad);
int orc_model_schedule(int depth, int moeExpertCount, int wideWindow, int *layerType, int *layerAttId, float *layerSlope, int maxLayers,
    int *attWidth, int *attTypeCount);
void orc_embedding_forward(int len, int dim, const int *labelPtr, const uint32_t *labels, const float *embed, float *state);
void orc_embedding_backward(int len, int dim, int labelCount, const int *labelPtr, const uint32_t *labels, const float *grad, float *deltaLabel);
void orc_softmax2(const float *logits, const float *bias, float *pred, int len, int dim);
void orc_final_backward(int len, int dim, int vocab, const float *lastState, const float *finalW, const float *bias, int targetCount,
    const int *targetPairs, float *pred, float *grad, float *deltaFinal);
double orc_model_step(const orc_dims *d, int depth, orc_layer *layers, const orc_common *c, int len, int labelCount, int vocab,
    const int *labelPtr, const uint32_t *labels, const float *embed, const float *finalW, const float *bias, int targetCount,
    const int *targetPairs, float *states, float *stateGrad0, float *deltaEmbed, float *deltaFinal);

#ifdef __cplusplus
}
#endif
#endif
