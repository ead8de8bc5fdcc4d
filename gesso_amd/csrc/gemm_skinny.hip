// Entry points of the weight-streaming products (see gemm_skinny_impl.h for the kernel).
//
// Each takes the weight as stored, W (N, K), and optionally its tile-major copy Wt; with Wt the
// kernels read that copy.  A tile-major copy exists only for K a multiple of 32 and row tiles that
// do not straddle a boundary of the epilogue (N, N/2 or N/3 a multiple of 16).
#include "common.h"

struct SkinnyExtra;
struct SkinnyCall;
#include "gemm_skinny_decl.h"

static int check_common(const void* W, int M, int N, int K) {
  GS_REQUIRE(M >= 0 && M <= 64, "gemm_skinny: %d rows; this kernel takes at most 64", M);
  GS_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "gemm_skinny: K=%d must be a positive multiple of 8 (N=%d)", K, N);
  GS_REQUIRE(((uintptr_t)W & 15) == 0, "gemm_skinny: the weight must be 16-byte aligned");
  return 0;
}

static int check_tiles(const void* Wt, int N, int K, int unit) {
  if (!Wt) return 0;
  GS_REQUIRE(K % 32 == 0 && unit % 16 == 0 && N % unit == 0 && ((uintptr_t)Wt & 15) == 0,
             "gemm_skinny: no tile-major copy exists for N=%d K=%d (row unit %d)", N, K, unit);
  return 0;
}

static int check_lazy(const float* res, const float* ssq, int nb, const float* norm_w, float eps) {
  GS_REQUIRE(res && ssq && norm_w && nb > 0 && eps > 0.f, "gemm_skinny: the norm prologue needs the stream, partial sums, a weight and eps");
  GS_REQUIRE(((uintptr_t)res & 15) == 0 && ((uintptr_t)norm_w & 15) == 0, "gemm_skinny: res and norm weight must be 16-byte aligned");
  return 0;
}

// X as rows (16-byte aligned, a row stride that is a multiple of 8) or as tiled rows (K a multiple of 32).
static int check_rows(const void* X, int ldx, int x_tiled, int K) {
  GS_REQUIRE(X && ((uintptr_t)X & 15) == 0, "gemm_skinny: X must be 16-byte aligned");
  if (x_tiled) {
    GS_REQUIRE(K % 32 == 0, "gemm_skinny: tiled rows need K=%d to be a multiple of 32", K);
  } else {
    GS_REQUIRE(ldx >= K && ldx % 8 == 0, "gemm_skinny: the row stride %d of X must be a multiple of 8 and at least K", ldx);
  }
  return 0;
}

// Rows that an epilogue writes for a following product, as tiled rows: their width is that product's K.
static int check_tiled_out(int tiled, int dtype, int width) {
  GS_REQUIRE(!tiled || (dtype == GS_BF16 && width % 32 == 0), "gemm_skinny: tiled rows are bfloat16 and a multiple of 32 wide, not %d", width);
  return 0;
}

// X is either given (bfloat16, aligned) or the normed residual stream (res != null).
static int check_x(const void* X, int ldx, int x_tiled, const float* res, const float* ssq, int nb, const float* norm_w, float eps,
                   int K) {
  if (res) {
    GS_REQUIRE(!x_tiled, "gemm_skinny: the norm prologue reads the stream, not tiled rows");
    return check_lazy(res, ssq, nb, norm_w, eps);
  }
  GS_REQUIRE(!ssq || (nb > 0 && eps > 0.f), "gemm_skinny: pre-weighted rows need their partial sums and eps");
  return check_rows(X, ldx, x_tiled, K);
}

// Plain and SwiGLU products of a given bfloat16 X, or of the normed residual stream (res != null).
extern "C" int gs_gemm_skinny(const void* X, int ldx, int x_tiled, const float* res, const float* ssq, int nb, const float* norm_w,
                              float eps, const void* W, const void* Wt, void* Y, int y_dtype, int ldy, int M, int N,
                              int K, int epilogue, int y_tiled, hipStream_t stream) {
  if (check_common(W, M, N, K)) return -1;
  GS_REQUIRE(!y_tiled || epilogue == 1, "gemm_skinny: only the SwiGLU epilogue writes tiled rows");
  if (check_tiled_out(y_tiled, y_dtype, N / 2)) return -1;
  GS_REQUIRE(epilogue == 0 || (epilogue == 1 && N % 2 == 0), "gemm_skinny: unknown epilogue %d (or odd N)", epilogue);
  GS_REQUIRE(ldy >= (epilogue == 1 ? N / 2 : N), "gemm_skinny: row stride %d of Y too small", ldy);
  GS_REQUIRE(y_dtype == GS_BF16 || y_dtype == GS_F32, "gemm_skinny: unknown output dtype %d", y_dtype);
  if (check_tiles(Wt, N, K, epilogue == 1 ? N / 2 : 16)) return -1;
  if (check_x(X, ldx, x_tiled, res, ssq, nb, norm_w, eps, K)) return -1;
  if (M == 0) return 0;
  gs_skinny_run_plain(X, ldx, x_tiled, res, ssq, nb, norm_w, eps, W, Wt, Y, y_dtype, ldy, M, N, K, epilogue, y_tiled, stream);
  GS_LAUNCH_CHECK("gemm_skinny");
  return 0;
}

// Partial sums per row that gs_gemm_skinny_residual writes for N columns.
extern "C" int gs_gemm_skinny_residual_blocks(int N, int tile_major) {
  return gs_ceil_div(N, tile_major && gs_skinny_halves(N) ? 8 : 16);
}

// res (M, N) += X W^T, and ssq_out (M, blocks) = partial sums of squares of the new rows.
extern "C" int gs_gemm_skinny_residual(const void* X, int ldx, int x_tiled, const void* W, const void* Wt, float* res,
                                       float* ssq_out, const float* next_w, void* xs_out, int xs_tiled, int M, int N,
                                       int K, hipStream_t stream) {
  if (check_common(W, M, N, K) || check_tiles(Wt, N, K, 16) || check_rows(X, ldx, x_tiled, K) ||
      check_tiled_out(xs_tiled, GS_BF16, N)) return -1;
  GS_REQUIRE(res && ssq_out, "gemm_skinny_residual: needs the stream and room for the partial sums");
  GS_REQUIRE(((uintptr_t)res & 15) == 0 && ((uintptr_t)next_w & 15) == 0, "gemm_skinny_residual: the stream and the norm weight must be 16-byte aligned");
  if (M == 0) return 0;
  GS_REQUIRE((next_w == nullptr) == (xs_out == nullptr), "gemm_skinny_residual: the next norm's weight and the room for the weighted rows come together");
  gs_skinny_run_residual(X, ldx, x_tiled, W, Wt, res, ssq_out, next_w, xs_out, xs_tiled, M, N, K, stream);
  GS_LAUNCH_CHECK("gemm_skinny_residual");
  return 0;
}

// part (parts, M, N) float32 = partial sums of X W^T over `parts` parts of K; gs_residual_from_parts adds them up.
extern "C" int gs_gemm_skinny_parts(const void* X, int ldx, int x_tiled, const void* W, const void* Wt, float* part, int parts,
                                    int M, int N, int K, hipStream_t stream) {
  if (check_common(W, M, N, K) || check_tiles(Wt, N, K, 16) || check_rows(X, ldx, x_tiled, K)) return -1;
  GS_REQUIRE(part && parts >= 1 && parts <= 64 && ((uintptr_t)part & 15) == 0, "gemm_skinny_parts: 1 to 64 parts and an aligned buffer");
  GS_REQUIRE(N <= 65535 * 32, "gemm_skinny_parts: %d weight rows are more than a launch takes", N);
  if (M == 0) return 0;
  gs_skinny_run_parts(X, ldx, x_tiled, W, Wt, part, parts, M, N, K, stream);
  GS_LAUNCH_CHECK("gemm_skinny_parts");
  return 0;
}

// mixed (M, H) = gated short convolution of (normed res) W_in^T for a decode step; W_in (3H, K).
extern "C" int gs_gemm_skinny_conv(const void* X, int ldx, int x_tiled, const float* res, const float* ssq, int nb, const float* norm_w, float eps,
                                   const void* W, const void* Wt, const float* taps, const float* conv_bias,
                                   float* state, const int* slots, int conv_w, void* Y, int y_tiled, int M, int H,
                                   int K, hipStream_t stream) {
  const int N = 3 * H;
  if (check_tiled_out(y_tiled, GS_BF16, H)) return -1;
  if (check_common(W, M, N, K) || check_tiles(Wt, N, K, H) || check_x(X, ldx, x_tiled, res, ssq, nb, norm_w, eps, K)) return -1;
  GS_REQUIRE(conv_w >= 2 && conv_w <= 16 && taps && state && slots, "gemm_skinny_conv: bad convolution operands (width %d)", conv_w);
  if (M == 0) return 0;
  gs_skinny_run_conv(X, ldx, x_tiled, res, ssq, nb, norm_w, eps, W, Wt, taps, conv_bias, state, slots, conv_w, Y, y_tiled, M, H, K, stream);
  GS_LAUNCH_CHECK("gemm_skinny_conv");
  return 0;
}

// Tile-major copy: out[(t * ksteps + s) * 512 + lane * 8 + j] = W[16 t + lane % 16][32 s + 8 (lane / 16) + j].
__global__ void tile_major_kernel(const bf16* __restrict__ W, bf16* __restrict__ out, int N, int K) {
  const int ksteps = K >> 5;
  const long unit = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);  // (row tile, k step)
  const int lane = threadIdx.x & 63;
  if (unit >= (long)(N >> 4) * ksteps) return;
  const int t = (int)(unit / ksteps), s = (int)(unit - (long)t * ksteps);
  const uint4 v = *reinterpret_cast<const uint4*>(W + (size_t)(16 * t + (lane & 15)) * K + 32 * s + 8 * (lane >> 4));
  *reinterpret_cast<uint4*>(out + (size_t)unit * 512 + lane * 8) = v;
}

extern "C" int gs_tile_major(const void* W, void* out, int N, int K, hipStream_t stream) {
  GS_REQUIRE(N > 0 && K > 0 && N % 16 == 0 && K % 32 == 0, "tile_major: N=%d must be a multiple of 16 and K=%d of 32", N, K);
  GS_REQUIRE(((uintptr_t)W & 15) == 0 && ((uintptr_t)out & 15) == 0, "tile_major: operands must be 16-byte aligned");
  const long units = (long)(N / 16) * (K / 32);
  tile_major_kernel<<<gs_ceil_div(units, 4), 256, 0, stream>>>((const bf16*)W, (bf16*)out, N, K);
  GS_LAUNCH_CHECK("tile_major");
  return 0;
}
