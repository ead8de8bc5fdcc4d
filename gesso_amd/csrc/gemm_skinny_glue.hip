// Fills the call record and hands it to the kernels that read rows or tiles.
#include "gemm_skinny_decl.h"
#include "gemm_skinny_impl.h"

void gs_skinny_plain_rows(const SkinnyCall& c);
void gs_skinny_residual_rows(const SkinnyCall& c);
void gs_skinny_conv_rows(const SkinnyCall& c);
void gs_skinny_plain_tiles(const SkinnyCall& c);
void gs_skinny_residual_tiles(const SkinnyCall& c);
void gs_skinny_residual_half_tiles(const SkinnyCall& c);
void gs_skinny_conv_tiles(const SkinnyCall& c);
void gs_skinny_parts_rows(const SkinnyCall& c, int parts);
void gs_skinny_parts_tiles(const SkinnyCall& c, int parts);
void gs_skinny_conv_half_tiles(const SkinnyCall& c);

static SkinnyCall base(const void* X, int ldx, int x_tiled, const void* W, const void* Wt, void* Y, int y_dtype, int ldy, int M,
                       int N, int K, int epilogue, hipStream_t stream) {
  SkinnyCall c = {};
  c.ex.x_tiled = x_tiled;
  c.x = (const bf16*)X; c.ldx = ldx; c.w = (const bf16*)(Wt ? Wt : W); c.Y = Y; c.y_dtype = y_dtype; c.ldy = ldy;
  c.M = M; c.N = N; c.K = K; c.epilogue = epilogue; c.stream = stream;
  return c;
}

static void lazy(SkinnyCall& c, const float* res, const float* ssq, int nb, const float* norm_w, float eps) {
  c.ex.res = res; c.ex.ssq = ssq; c.ex.nb = nb; c.ex.norm_w = norm_w; c.ex.eps = eps;
}

void gs_skinny_run_plain(const void* X, int ldx, int x_tiled, const float* res, const float* ssq, int nb, const float* norm_w,
                         float eps, const void* W, const void* Wt, void* Y, int y_dtype, int ldy, int M, int N, int K,
                         int epilogue, int y_tiled, hipStream_t stream) {
  SkinnyCall c = base(X, ldx, x_tiled, W, Wt, Y, y_dtype, ldy, M, N, K, epilogue, stream);
  c.ex.y_tiled = y_tiled;
  if (res || ssq) lazy(c, res, ssq, nb, norm_w, eps);
  Wt ? gs_skinny_plain_tiles(c) : gs_skinny_plain_rows(c);
}

// A weight of few rows is shared out in half tiles, so that twice as many blocks stream it.
bool gs_skinny_halves(int N) { return N % 16 == 0 && N / 16 <= 160; }

void gs_skinny_run_residual(const void* X, int ldx, int x_tiled, const void* W, const void* Wt, float* res, float* ssq_out,
                            const float* next_w, void* xs_out, int xs_tiled, int M, int N, int K, hipStream_t stream) {
  SkinnyCall c = base(X, ldx, x_tiled, W, Wt, nullptr, GS_F32, N, M, N, K, 2, stream);
  c.ex.y_tiled = xs_tiled;
  c.ex.res_out = res; c.ex.ssq_out = ssq_out; c.ex.next_w = next_w; c.ex.xs_out = (bf16*)xs_out;
  if (Wt && gs_skinny_halves(N)) gs_skinny_residual_half_tiles(c);
  else Wt ? gs_skinny_residual_tiles(c) : gs_skinny_residual_rows(c);
}

void gs_skinny_run_conv(const void* X, int ldx, int x_tiled, const float* res, const float* ssq, int nb, const float* norm_w, float eps, const void* W,
                        const void* Wt, const float* taps, const float* conv_bias, float* state, const int* slots,
                        int conv_w, void* Y, int y_tiled, int M, int H, int K, hipStream_t stream) {
  SkinnyCall c = base(X, ldx, x_tiled, W, Wt, Y, GS_BF16, H, M, 3 * H, K, 3, stream);
  c.ex.y_tiled = y_tiled;
  if (res || ssq) lazy(c, res, ssq, nb, norm_w, eps);
  c.ex.taps = taps; c.ex.conv_bias = conv_bias; c.ex.state = state; c.ex.slots = slots; c.ex.conv_w = conv_w;
  c.ex.conv_vec = conv_w >= 2 && conv_w <= 4 && H % 4 == 0 && H >= 4 &&
                  (((uintptr_t)taps | (uintptr_t)conv_bias | (uintptr_t)state) & 15) == 0;
  // c.N / 3 channels, as few as a narrow weight's rows; with many rows of X the blocks' reading of X outweighs that
  if (Wt && gs_skinny_halves(c.N / 3) && M <= 32) gs_skinny_conv_half_tiles(c);
  else Wt ? gs_skinny_conv_tiles(c) : gs_skinny_conv_rows(c);
}

void gs_skinny_run_parts(const void* X, int ldx, int x_tiled, const void* W, const void* Wt, float* part, int parts, int M, int N,
                         int K, hipStream_t stream) {
  SkinnyCall c = base(X, ldx, x_tiled, W, Wt, part, GS_F32, N, M, N, K, 5, stream);
  Wt ? gs_skinny_parts_tiles(c, parts) : gs_skinny_parts_rows(c, parts);
}
