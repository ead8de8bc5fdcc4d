// Gated short convolution over a batch of sequence segments, with per-request history.
//
// bcx (T, 3H) holds B, C, X side by side.  Per channel c and token t of a segment:
//   u[t]  = B[t,c] * X[t,c]
//   y[t]  = sum_{p=0}^{W-1} taps[c,p] * u[t-(W-1)+p]      (taps oldest to newest, current input last)
//   out   = C[t,c] * (y[t] + bias[c])
// where u before the segment's first token comes from the request's history
// state[slot, c, 0..W-2] (oldest to newest).  After the segment the history holds the last
// W-1 values of u (older history shifts out).  Products and sums are float32; the history is
// float32 in both precisions.
//
// Two kernels: outputs (one thread per token and channel, all reading the old history), then
// the history update (one thread per sequence and channel).  When every segment is a single
// token the first kernel also updates the history, since no other thread reads it.
#include "common.h"

#define GS_CONV_MAX_W 16

template <typename T>
__global__ void short_conv_kernel(const T* __restrict__ bcx, const float* __restrict__ taps,
                                  const float* __restrict__ bias, float* __restrict__ state,
                                  const int* __restrict__ seq_of_token, const int* __restrict__ q_start,
                                  const int* __restrict__ slots, T* __restrict__ out, int ntok, int H, int W,
                                  int update_state) {
  int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= H) return;
  const float* wt = taps + (size_t)c * W;
  for (int t = blockIdx.y; t < ntok; t += gridDim.y) {
    int s = seq_of_token[t];
    int t0 = q_start[s];
    float* hist = state + ((size_t)slots[s] * H + c) * (W - 1);
    float y = 0.f;
    float u_now = 0.f;
    for (int p = 0; p < W; ++p) {
      int j = t - (W - 1) + p;  // token index of this tap
      float u;
      if (j >= t0) {
        const T* row = bcx + (size_t)j * 3 * H;
        u = to_f32(row[c]) * to_f32(row[2 * H + c]);
      } else {
        // k = t0 - j tokens before the segment: history entry W-1-k
        u = hist[(W - 1) - (t0 - j)];
      }
      y += wt[p] * u;
      u_now = u;
    }
    if (bias) y += bias[c];
    out[(size_t)t * H + c] = from_f32<T>(to_f32(bcx[(size_t)t * 3 * H + H + c]) * y);
    if (update_state) {
      // single-token segment: shift by one, newest last
      for (int p = 0; p < W - 2; ++p) hist[p] = hist[p + 1];
      hist[W - 2] = u_now;
    }
  }
}

// Eight channels per thread: 16-byte loads of B, C and X rows.  H a multiple of 8, rows 16-byte aligned.
template <typename T>
__global__ void short_conv8_kernel(const T* __restrict__ bcx, const float* __restrict__ taps,
                                   const float* __restrict__ bias, float* __restrict__ state,
                                   const int* __restrict__ seq_of_token, const int* __restrict__ q_start,
                                   const int* __restrict__ slots, T* __restrict__ out, int ntok, int H, int W,
                                   int update_state) {
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (c >= H) return;
  for (int t = blockIdx.y; t < ntok; t += gridDim.y) {
    const int s = seq_of_token[t];
    const int t0 = q_start[s];
    float* hist = state + ((size_t)slots[s] * H + c) * (W - 1);   // channel c + i at hist + i (W - 1)
    float y[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, u[8];
    for (int p = 0; p < W; ++p) {
      const int j = t - (W - 1) + p;
      if (j >= t0) {
        float b8[8], x8[8];
        load8f(bcx + (size_t)j * 3 * H + c, b8);
        load8f(bcx + (size_t)j * 3 * H + 2 * H + c, x8);
#pragma unroll
        for (int i = 0; i < 8; ++i) u[i] = b8[i] * x8[i];
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) u[i] = hist[i * (W - 1) + (W - 1) - (t0 - j)];
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) y[i] += taps[(size_t)(c + i) * W + p] * u[i];
    }
    float c8[8];
    load8f(bcx + (size_t)t * 3 * H + H + c, c8);
#pragma unroll
    for (int i = 0; i < 8; ++i) y[i] = c8[i] * (bias ? y[i] + bias[c + i] : y[i]);
    store8f(out + (size_t)t * H + c, y);
    if (update_state) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float* h = hist + i * (W - 1);
        for (int p = 0; p < W - 2; ++p) h[p] = h[p + 1];
        h[W - 2] = u[i];
      }
    }
  }
}

// Every segment a single token, widths up to 4: a thread takes eight channels of one token; its history, its taps and
// its B, C and X values are asked for together (the history and the taps of eight channels lie side by side), where the
// kernel above walks them value by value behind one another.  Sums in the same order as there.
template <typename T, int W>
__global__ __launch_bounds__(64) void short_conv_single_kernel(const T* __restrict__ bcx, const float* __restrict__ taps,
                                                               const float* __restrict__ bias,
                                                               float* __restrict__ state,
                                                               const int* __restrict__ seq_of_token,
                                                               const int* __restrict__ slots, T* __restrict__ out,
                                                               int ntok, int H) {
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (c >= H) return;
  float tp[8 * W], bs[8];
#pragma unroll
  for (int q = 0; q < 2 * W; ++q)
    *reinterpret_cast<float4*>(tp + 4 * q) = *reinterpret_cast<const float4*>(taps + (size_t)c * W + 4 * q);
#pragma unroll
  for (int i = 0; i < 8; ++i) bs[i] = bias ? bias[c + i] : 0.f;
  for (int t = blockIdx.y; t < ntok; t += gridDim.y) {
    float* hist = state + ((size_t)slots[seq_of_token[t]] * H + c) * (W - 1);   // channel c + i at hist + i (W - 1)
    float h[8 * (W - 1)], b8[8], x8[8], c8[8], y[8];
#pragma unroll
    for (int q = 0; q < 2 * (W - 1); ++q)
      *reinterpret_cast<float4*>(h + 4 * q) = *reinterpret_cast<const float4*>(hist + 4 * q);
    const T* row = bcx + (size_t)t * 3 * H + c;
    load8f(row, b8);
    load8f(row + 2 * H, x8);
    load8f(row + H, c8);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float u = b8[i] * x8[i];
      float acc = 0.f;
#pragma unroll
      for (int p = 0; p < W - 1; ++p) acc += tp[i * W + p] * h[i * (W - 1) + p];
      acc += tp[i * W + W - 1] * u;
      y[i] = c8[i] * (bias ? acc + bs[i] : acc);
#pragma unroll
      for (int p = 0; p < W - 2; ++p) h[i * (W - 1) + p] = h[i * (W - 1) + p + 1];
      h[i * (W - 1) + W - 2] = u;
    }
    store8f(out + (size_t)t * H + c, y);
#pragma unroll
    for (int q = 0; q < 2 * (W - 1); ++q)
      *reinterpret_cast<float4*>(hist + 4 * q) = *reinterpret_cast<const float4*>(h + 4 * q);
  }
}

// Prompt portions: a thread takes eight channels and a run of TT consecutive tokens (4 or 2, see the launch), so every B and X row is read
// once (plus W - 1 rows of run-in), all loads of the run are issued before anything is computed, and the products
// u = B x stay in registers for the W tokens that use them.  Sums run over the taps in the same order as in the
// kernels above.  The first W - 1 tokens of a sequence take what they miss from the history, read where needed.
template <typename T, int W, int TT>
__global__ __launch_bounds__(64) void short_conv_run_kernel(const T* __restrict__ bcx, const float* __restrict__ taps,
                                                            const float* __restrict__ bias,
                                                            const float* __restrict__ state,
                                                            const int* __restrict__ seq_of_token,
                                                            const int* __restrict__ q_start,
                                                            const int* __restrict__ slots, T* __restrict__ out,
                                                            int ntok, int H) {
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (c >= H) return;
  const int ta = blockIdx.y * TT;
  float u[TT + W - 1][8], cc[TT][8];
#pragma unroll
  for (int r = 0; r < TT + W - 1; ++r) {
    const int j = ta - (W - 1) + r;
    if (j >= 0 && j < ntok) {
      float b8[8], x8[8];
      load8f(bcx + (size_t)j * 3 * H + c, b8);
      load8f(bcx + (size_t)j * 3 * H + 2 * H + c, x8);
#pragma unroll
      for (int k = 0; k < 8; ++k) u[r][k] = b8[k] * x8[k];
    } else {
#pragma unroll
      for (int k = 0; k < 8; ++k) u[r][k] = 0.f;
    }
  }
#pragma unroll
  for (int i = 0; i < TT; ++i) {
    if (ta + i < ntok) load8f(bcx + (size_t)(ta + i) * 3 * H + H + c, cc[i]);
  }
  float tp[8][W], bs[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    bs[k] = bias ? bias[c + k] : 0.f;
#pragma unroll
    for (int p = 0; p < W; ++p) tp[k][p] = taps[(size_t)(c + k) * W + p];
  }
#pragma unroll
  for (int i = 0; i < TT; ++i) {
    const int t = ta + i;
    if (t >= ntok) break;
    const int s = seq_of_token[t];
    const int t0 = q_start[s];
    float y[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int p = 0; p < W; ++p) {
      const int j = t - (W - 1) + p;
      if (j >= t0) {
#pragma unroll
        for (int k = 0; k < 8; ++k) y[k] += tp[k][p] * u[i + p][k];
      } else {
        const float* hist = state + ((size_t)slots[s] * H + c) * (W - 1);
#pragma unroll
        for (int k = 0; k < 8; ++k) y[k] += tp[k][p] * hist[k * (W - 1) + (W - 1) - (t0 - j)];
      }
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) y[k] = cc[i][k] * (bias ? y[k] + bs[k] : y[k]);
    store8f(out + (size_t)t * H + c, y);
  }
}

template <typename T>
__global__ void short_conv_state_kernel(const T* __restrict__ bcx, float* __restrict__ state,
                                        const int* __restrict__ q_start, const int* __restrict__ slots, int H,
                                        int W) {
  int c = blockIdx.x * blockDim.x + threadIdx.x;
  int s = blockIdx.y;
  if (c >= H) return;
  int t0 = q_start[s], t1 = q_start[s + 1];
  int n = t1 - t0;
  if (n <= 0) return;
  float* hist = state + ((size_t)slots[s] * H + c) * (W - 1);
  float nh[GS_CONV_MAX_W];
  for (int p = 0; p < W - 1; ++p) {
    int j = t1 - (W - 1) + p;  // token whose u lands in entry p
    if (j >= t0) {
      const T* row = bcx + (size_t)j * 3 * H;
      nh[p] = to_f32(row[c]) * to_f32(row[2 * H + c]);
    } else {
      nh[p] = hist[p + n];  // old entries move n places towards "older"
    }
  }
  for (int p = 0; p < W - 1; ++p) hist[p] = nh[p];
}

extern "C" int gs_short_conv(const void* bcx, int dtype, const float* taps, const float* bias, float* state,
                             const int* seq_of_token, const int* q_start, const int* slots, void* out, int ntok,
                             int nseq, int H, int W, int all_single, hipStream_t stream) {
  GS_REQUIRE(ntok >= 0 && nseq >= 0 && H > 0, "short_conv: bad sizes T=%d nseq=%d H=%d", ntok, nseq, H);
  GS_REQUIRE(W >= 2 && W <= GS_CONV_MAX_W, "short_conv: width %d outside [2, %d]", W, GS_CONV_MAX_W);
  if (ntok == 0) return 0;
  int threads = H >= 256 ? 256 : 64;
  int cx = gs_ceil_div(H, threads);
  dim3 grid(cx, ntok < 65535 ? ntok : 65535);  // the kernel strides over tokens beyond gridDim.y
  const bool vec = H % 8 == 0 && ((uintptr_t)bcx & 15) == 0 && ((uintptr_t)out & 15) == 0 &&
                   (dtype == GS_F32 || dtype == GS_BF16);
  if (vec && !all_single && W <= 4) {
    // runs of 4 tokens a thread, of 2 where runs of 4 would leave the chip short of wavefronts (narrow models, short
    // portions).  Measured, bfloat16, W = 3: 2,048 tokens of 2,048 channels 10.7 us with runs of 4, 11.1 with 2, 13.6
    // with 8; some 900 tokens of 1,024 channels 7.7 us with runs of 2, 11.5 with 4, 18.0 with 8
    const int cols = gs_ceil_div(H / 8, 64);
    const int tt = (long)cols * gs_ceil_div(ntok, 4) >= 2048 ? 4 : 2;
    dim3 gr(cols, gs_ceil_div(ntok, tt));
    GS_REQUIRE(gr.y <= 65535, "short_conv: %d tokens in one call; at most %d", ntok, 65535 * tt);
#define GS_RUN_CONV_T(TY, WW, TT)                                                                                    \
  short_conv_run_kernel<TY, WW, TT><<<gr, 64, 0, stream>>>((const TY*)bcx, taps, bias, state, seq_of_token, q_start, \
                                                           slots, (TY*)out, ntok, H)
#define GS_RUN_CONV(TY, WW)                                                                                          \
  do {                                                                                                               \
    if (tt == 4) GS_RUN_CONV_T(TY, WW, 4); else GS_RUN_CONV_T(TY, WW, 2);                                           \
  } while (0)
    if (dtype == GS_F32) {
      if (W == 2) GS_RUN_CONV(float, 2); else if (W == 3) GS_RUN_CONV(float, 3); else GS_RUN_CONV(float, 4);
    } else {
      if (W == 2) GS_RUN_CONV(bf16, 2); else if (W == 3) GS_RUN_CONV(bf16, 3); else GS_RUN_CONV(bf16, 4);
    }
#undef GS_RUN_CONV
#undef GS_RUN_CONV_T
  } else if (vec && all_single && W <= 4 && (((uintptr_t)taps | (uintptr_t)state) & 15) == 0) {
    dim3 gs(gs_ceil_div(H / 8, 64), grid.y);
#define GS_RUN_SINGLE(TY, WW)                                                                                          \
  short_conv_single_kernel<TY, WW><<<gs, 64, 0, stream>>>((const TY*)bcx, taps, bias, state, seq_of_token, slots,      \
                                                          (TY*)out, ntok, H)
    if (dtype == GS_F32) {
      if (W == 2) GS_RUN_SINGLE(float, 2); else if (W == 3) GS_RUN_SINGLE(float, 3); else GS_RUN_SINGLE(float, 4);
    } else {
      if (W == 2) GS_RUN_SINGLE(bf16, 2); else if (W == 3) GS_RUN_SINGLE(bf16, 3); else GS_RUN_SINGLE(bf16, 4);
    }
#undef GS_RUN_SINGLE
  } else if (vec) {
    int th = H / 8 >= 256 ? 256 : 64;
    dim3 g8(gs_ceil_div(H / 8, th), grid.y);
    if (dtype == GS_F32)
      short_conv8_kernel<float><<<g8, th, 0, stream>>>((const float*)bcx, taps, bias, state, seq_of_token, q_start,
                                                       slots, (float*)out, ntok, H, W, all_single);
    else
      short_conv8_kernel<bf16><<<g8, th, 0, stream>>>((const bf16*)bcx, taps, bias, state, seq_of_token, q_start,
                                                      slots, (bf16*)out, ntok, H, W, all_single);
  } else if (dtype == GS_F32)
    short_conv_kernel<float><<<grid, threads, 0, stream>>>((const float*)bcx, taps, bias, state, seq_of_token,
                                                            q_start, slots, (float*)out, ntok, H, W, all_single);
  else if (dtype == GS_BF16)
    short_conv_kernel<bf16><<<grid, threads, 0, stream>>>((const bf16*)bcx, taps, bias, state, seq_of_token,
                                                           q_start, slots, (bf16*)out, ntok, H, W, all_single);
  else
    GS_REQUIRE(false, "short_conv: unknown dtype %d", dtype);
  GS_LAUNCH_CHECK("short_conv");
  if (!all_single) {
    GS_REQUIRE(nseq <= 65535, "short_conv: more than 65535 sequences in one call");
    dim3 grid(cx, nseq);
    if (dtype == GS_F32)
      short_conv_state_kernel<float><<<grid, threads, 0, stream>>>((const float*)bcx, state, q_start, slots, H, W);
    else
      short_conv_state_kernel<bf16><<<grid, threads, 0, stream>>>((const bf16*)bcx, state, q_start, slots, H, W);
    GS_LAUNCH_CHECK("short_conv_state");
  }
  return 0;
}
