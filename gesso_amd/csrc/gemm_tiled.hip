// Y (M, N) = X (M, K) . W (N, K)^T + bias: the plain tiled matrix product.
//
// Every size is taken (bounds are checked per element), every mix of float32 and bfloat16
// storage for X, W and Y.  Products and sums are float32 FMAs: with float32 storage this is the
// true 32-bit path (no matrix-core input rounding).  Each output element is summed in one fixed order,
// so its value does not depend on M or on which rows share the launch: k in chunks of 64, each chunk
// from zero in ascending k, the chunks' sums added in ascending order.  (The streaming kernel for few
// rows, gemv_f32.hip, adds in the same order; a chunk is what one of its lanes takes.)
//
// 64 x 64 tile per block of 256 threads, 4 x 4 outputs per thread, k in steps of 16 through LDS.
#include "common.h"

#define TM 64
#define TN 64
#define TK 16
static_assert(GS_SUM_CHUNK % TK == 0 && ((GS_SUM_CHUNK / TK) & (GS_SUM_CHUNK / TK - 1)) == 0, "chunks are whole k steps");

template <typename TX, typename TW, typename TY>
__global__ void gemm_tiled_kernel(const TX* __restrict__ X, int ldx, const TW* __restrict__ W,
                                  const float* __restrict__ bias, TY* __restrict__ Y, int ldy, int M, int N, int K) {
  __shared__ float xs[TK][TM + 4];
  __shared__ float ws[TK][TN + 4];
  int tid = threadIdx.x;
  int tx = tid & 15, ty = tid >> 4;  // tx: columns (n), ty: rows (m)
  int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  float acc[4][4], tot[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = tot[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += TK) {
    // 64 rows x 16 k = 1024 elements per operand, 4 per thread
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      int idx = tid + e * 256;
      int r = idx >> 4, kk = idx & 15;
      int m = m0 + r, n = n0 + r, k = k0 + kk;
      xs[kk][r] = (m < M && k < K) ? to_f32(X[(size_t)m * ldx + k]) : 0.f;
      ws[kk][r] = (n < N && k < K) ? to_f32(W[(size_t)n * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < TK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
    if (((k0 / TK) & (GS_SUM_CHUNK / TK - 1)) == GS_SUM_CHUNK / TK - 1 || k0 + TK >= K) {   // a chunk is complete
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          tot[i][j] += acc[i][j];
          acc[i][j] = 0.f;
        }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = tot[i][j];
      if (bias) v += bias[n];
      Y[(size_t)m * ldy + n] = from_f32<TY>(v);
    }
  }
}

template <typename TX, typename TW, typename TY>
static int launch(const void* X, int ldx, const void* W, const float* bias, void* Y, int ldy, int M, int N, int K,
                  hipStream_t stream) {
  dim3 grid(gs_ceil_div(N, TN), gs_ceil_div(M, TM));
  gemm_tiled_kernel<TX, TW, TY>
      <<<grid, 256, 0, stream>>>((const TX*)X, ldx, (const TW*)W, bias, (TY*)Y, ldy, M, N, K);
  return 0;
}

extern "C" int gs_gemm_tiled(const void* X, int x_dtype, int ldx, const void* W, int w_dtype, const float* bias,
                             void* Y, int y_dtype, int ldy, int M, int N, int K, hipStream_t stream) {
  GS_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
  GS_REQUIRE(ldx >= K && ldy >= N, "gemm: row strides %d, %d below K=%d, N=%d", ldx, ldy, K, N);
  GS_REQUIRE(gs_ceil_div(M, TM) <= 65535, "gemm: M=%d too large for one launch", M);
  GS_REQUIRE((x_dtype | 1) == 1 && (w_dtype | 1) == 1 && (y_dtype | 1) == 1, "gemm: unknown dtypes %d %d %d", x_dtype,
             w_dtype, y_dtype);
  if (M == 0) return 0;
  int key = x_dtype * 4 + w_dtype * 2 + y_dtype;
  switch (key) {
    case 0: launch<float, float, float>(X, ldx, W, bias, Y, ldy, M, N, K, stream); break;
    case 1: launch<float, float, bf16>(X, ldx, W, bias, Y, ldy, M, N, K, stream); break;
    case 2: launch<float, bf16, float>(X, ldx, W, bias, Y, ldy, M, N, K, stream); break;
    case 3: launch<float, bf16, bf16>(X, ldx, W, bias, Y, ldy, M, N, K, stream); break;
    case 4: launch<bf16, float, float>(X, ldx, W, bias, Y, ldy, M, N, K, stream); break;
    case 5: launch<bf16, float, bf16>(X, ldx, W, bias, Y, ldy, M, N, K, stream); break;
    case 6: launch<bf16, bf16, float>(X, ldx, W, bias, Y, ldy, M, N, K, stream); break;
    case 7: launch<bf16, bf16, bf16>(X, ldx, W, bias, Y, ldy, M, N, K, stream); break;
    default: GS_REQUIRE(false, "gemm: unknown dtypes %d %d %d", x_dtype, w_dtype, y_dtype);
  }
  GS_LAUNCH_CHECK("gemm_tiled");
  return 0;
}
