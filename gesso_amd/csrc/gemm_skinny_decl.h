// Host-side glue between the entry points and the two translation units that instantiate the kernels.
#pragma once
#include <hip/hip_runtime.h>

void gs_skinny_run_plain(const void* X, int ldx, int x_tiled, const float* res, const float* ssq, int nb, const float* norm_w,
                         float eps, const void* W, const void* Wt, void* Y, int y_dtype, int ldy, int M, int N, int K,
                         int epilogue, int y_tiled, hipStream_t stream);
bool gs_skinny_halves(int N);
void gs_skinny_run_residual(const void* X, int ldx, int x_tiled, const void* W, const void* Wt, float* res, float* ssq_out,
                            const float* next_w, void* xs_out, int xs_tiled, int M, int N, int K, hipStream_t stream);
void gs_skinny_run_conv(const void* X, int ldx, int x_tiled, const float* res, const float* ssq, int nb, const float* norm_w, float eps, const void* W,
                        const void* Wt, const float* taps, const float* conv_bias, float* state, const int* slots,
                        int conv_w, void* Y, int y_tiled, int M, int H, int K, hipStream_t stream);
void gs_skinny_run_parts(const void* X, int ldx, int x_tiled, const void* W, const void* Wt, float* part, int parts, int M, int N,
                         int K, hipStream_t stream);
