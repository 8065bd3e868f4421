// Library-internal entry points (not part of the C ABI): kernels used only by the model driver.
#pragma once
#include "../../include/ts2_abi.h"

int Ts2EmbedForward(int len, int lenRound, int dim, const int *labelPtr, const uint32_t *labels, const ts2_mat *embed, int embType, float mult,
    const float *scalePtr, const ts2_mat *state, void *stream);
int Ts2EmbedBackward(int len, int dim, const int *labelPtr, const uint32_t *labels, const ts2_mat *grad, const ts2_mat *delta, int labelCount,
    void *stream);
int Ts2FinalSoftmaxGrad(int rows, int vocab, const ts2_mat *logits, const float *bias, const int *target, float gradMult, const ts2_mat *grad,
    float *lossSum, int keepProb, void *stream);
int Ts2FinalSoftmaxGradHalf(int rows, int vocab, const ts2_mat *logits, const float *bias, const int *target, float gradMult, const ts2_mat *grad,
    float *lossSum, void *stream);
int Ts2TransposeToBf16(int rows, int rowsRound, int cols, const ts2_mat *src, int srcType, const ts2_mat *dst, void *stream);
int Ts2RowsToBf16(int rows, int rowsRound, int cols, const ts2_mat *src, int srcType, const ts2_mat *dst, void *stream);
int Ts2ZeroRows(const ts2_mat *m, int rows, int rowBytes, void *stream);
int Ts2FillFloats(float *p, int n, float v, void *stream);
// ts2_transpose_quant with the k-tile maxima formed in the kernel from row maxima (rowAbsMax) when tileMax is null
int Ts2TransposeQuantRows(int len, int lenRound, const ts2_mat *src, int srcType, const float *rowMult, const float *tileMax, const float *rowAbsMax,
    int kTile, const int *rowIndex, const ts2_mat *dstT, int dstType, float *tileScale, void *stream, uint32_t ditherSeed = 0);
// resolves, for the current device, what ts2_moe_route_static otherwise resolves on its first call there (no stream operation)
int Ts2MoeRouteSetup();
