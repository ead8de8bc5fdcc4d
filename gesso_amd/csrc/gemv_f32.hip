// y = x W^T (+ bias) for a few rows of x, everything float32: the true 32-bit path's product for decode steps.
//
// The weights are streamed once.  A wavefront owns pairs of rows of W (two outputs per row of x and pair): as many
// pairs as there are lanes to spare beyond the number of chunks.  The lanes of a pair take
// chunks of GS_SUM_CHUNK = 64 consecutive k each (lane l chunks l, l + span, ...), sum a chunk from zero in
// ascending k with FMAs, and leave the chunk's sum in LDS; then one lane per output adds that output's chunk
// sums in ascending order.  That is the order of the tiled kernel (gemm_tiled.hip), so an output's value does
// not depend on which of the two kernels computed it, on the number of rows or on what else is in the batch.
// No matrix cores, no reduced precision.
#include "common.h"

#define GV_WAVES 2
#define GV_MAXCHUNKS 128   // K up to 8192

template <int MB, typename TO>
__global__ __launch_bounds__(GV_WAVES * 64) void gemv_f32_kernel(const float* __restrict__ X, int ldx,
                                                                 const float* __restrict__ W,
                                                                 const float* __restrict__ bias, TO* __restrict__ Y,
                                                                 int ldy, int M, int N, int K, int span) {
  // span = lanes that share a pair of rows of W: the power of two at or above the number of chunks, at most 64.
  // A wavefront owns 64 / span pairs (for K = 2048, 32 chunks: two pairs, so that no lane idles).
  __shared__ float cs[GV_WAVES][2 * MB][GV_MAXCHUNKS + 1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int pairs = 64 / span;               // pairs of rows per wavefront
  const int grp = lane / span, sub = lane - grp * span;
  const int nw = (blockIdx.x * GV_WAVES + wave) * 2 * pairs;   // first row of W of this wavefront
  if (nw >= N) return;                       // whole wavefronts leave; no block-wide barrier follows
  const int n0 = nw + 2 * grp;
  const bool live = n0 < N, two = n0 + 1 < N;
  const float* w0 = W + (size_t)(live ? n0 : N - 1) * K;
  const float* w1 = W + (size_t)(two ? n0 + 1 : (live ? n0 : N - 1)) * K;
  const float* xr[MB];
#pragma unroll
  for (int m = 0; m < MB; ++m) xr[m] = X + (size_t)(m < M ? m : M - 1) * ldx;
  const int chunks = (K + GS_SUM_CHUNK - 1) / GS_SUM_CHUNK;
  for (int c = sub; c < chunks; c += span) {
    const int k0 = c * GS_SUM_CHUNK;
    const int len4 = ((K - k0 < GS_SUM_CHUNK ? K - k0 : GS_SUM_CHUNK) + 3) >> 2;   // K is a multiple of 4
    float a0[MB], a1[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) a0[m] = a1[m] = 0.f;
#pragma unroll 4
    for (int j = 0; j < len4; ++j) {
      const float4 u = *reinterpret_cast<const float4*>(w0 + k0 + 4 * j);
      const float4 v = *reinterpret_cast<const float4*>(w1 + k0 + 4 * j);
#pragma unroll
      for (int m = 0; m < MB; ++m) {
        const float4 x = *reinterpret_cast<const float4*>(xr[m] + k0 + 4 * j);
        a0[m] = fmaf(x.x, u.x, a0[m]); a0[m] = fmaf(x.y, u.y, a0[m]); a0[m] = fmaf(x.z, u.z, a0[m]); a0[m] = fmaf(x.w, u.w, a0[m]);
        a1[m] = fmaf(x.x, v.x, a1[m]); a1[m] = fmaf(x.y, v.y, a1[m]); a1[m] = fmaf(x.z, v.z, a1[m]); a1[m] = fmaf(x.w, v.w, a1[m]);
      }
    }
    // pair grp keeps its chunk sums at columns [grp * span, grp * span + chunks) when span < 64 (then chunks <= span)
    const int col = pairs > 1 ? grp * span + c : c;
#pragma unroll
    for (int m = 0; m < MB; ++m) {
      cs[wave][2 * m][col] = a0[m];
      cs[wave][2 * m + 1][col] = a1[m];
    }
  }
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_s_waitcnt(0xc07f);        // this wavefront's LDS writes are visible to its own lanes
  // one lane per output (pair g, row m of x, row r of the pair) adds that output's chunk sums in ascending order
  for (int o = lane; o < pairs * 2 * MB; o += 64) {
    const int g = o / (2 * MB), q = o - g * 2 * MB, m = q >> 1, r = q & 1;
    const int n = nw + 2 * g + r;
    float t = 0.f;
    for (int c = 0; c < chunks; ++c) t += cs[wave][q][pairs > 1 ? g * span + c : c];
    if (m < M && n < N) {
      if (bias) t += bias[n];
      Y[(size_t)m * ldy + n] = from_f32<TO>(t);
    }
  }
}

// Whether the streaming kernel takes the operands: up to 16 rows, K a multiple of 4 up to 8192, aligned rows.
extern "C" int gs_gemv_f32_supports(int M, int K, int ldx, const void* X, const void* W) {
  return M >= 1 && M <= 16 && K % 4 == 0 && K <= GV_MAXCHUNKS * GS_SUM_CHUNK && ldx % 4 == 0 &&
         ((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0;
}

extern "C" int gs_gemv_f32(const float* X, int ldx, const float* W, const float* bias, void* Y, int y_dtype, int ldy,
                           int M, int N, int K, hipStream_t stream) {
  GS_REQUIRE(N > 0 && K > 0 && ldx >= K && ldy >= N, "gemv_f32: bad sizes N=%d K=%d ldx=%d ldy=%d", N, K, ldx, ldy);
  GS_REQUIRE(gs_gemv_f32_supports(M, K, ldx, X, W), "gemv_f32: needs 1 to 16 rows, K a multiple of 4 up to 8192 and aligned rows (M=%d K=%d)", M, K);
  GS_REQUIRE(y_dtype == GS_F32 || y_dtype == GS_BF16, "gemv_f32: unknown output dtype %d", y_dtype);
  const int chunks = gs_ceil_div(K, GS_SUM_CHUNK);
  int span = 1;
  while (span < chunks && span < 64) span <<= 1;
  const int blocks = gs_ceil_div(N, 2 * (64 / span) * GV_WAVES);
#define GS_RUN(MB)                                                                                                  \
  if (y_dtype == GS_F32)                                                                                            \
    gemv_f32_kernel<MB, float><<<blocks, GV_WAVES * 64, 0, stream>>>(X, ldx, W, bias, (float*)Y, ldy, M, N, K, span);     \
  else                                                                                                              \
    gemv_f32_kernel<MB, bf16><<<blocks, GV_WAVES * 64, 0, stream>>>(X, ldx, W, bias, (bf16*)Y, ldy, M, N, K, span)
  if (M <= 1) { GS_RUN(1); } else if (M <= 2) { GS_RUN(2); } else if (M <= 4) { GS_RUN(4); } else if (M <= 8) { GS_RUN(8); } else { GS_RUN(16); }
#undef GS_RUN
  GS_LAUNCH_CHECK("gemv_f32");
  return 0;
}
