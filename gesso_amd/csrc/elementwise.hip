// Embedding gather, residual add + RMSNorm, SwiGLU activation, small fills.
//
// The residual stream is float32 in both precisions; the rows that feed matrix products
// are written in the activation type.  Sums of squares are float32 in a fixed order per row,
// so a row's result does not depend on which other rows share the launch.
#include <stdarg.h>
#include <string.h>

#include "common.h"

static thread_local char g_err[512] = "";

void gs_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

extern "C" const char* gs_last_error() { return g_err; }

extern "C" int gs_abi_version() { return 9; }

// ------------------------------------------------------------------ embedding

// out[t, :] = table[ids[t], :] * scale as float32 (scale 1 for most models; some multiply the embedding by a
// constant); an id outside the table gives a NaN row.
// With ssq: ssq[t] = sum of squares of the row (one partial sum per row, for a norm that follows).
// With next_w and xs: xs[t, :] = bfloat16(row * next_w), the rows pre-weighted for the first norm's consumer,
// as rows of H or, with xs_tiles = ceil(T / 16) > 0, as tiled rows.
template <typename T>
__global__ void embed_kernel(const int* __restrict__ ids, const T* __restrict__ table, float* __restrict__ out,
                             float* __restrict__ ssq, const float* __restrict__ next_w, bf16* __restrict__ xs,
                             int xs_tiles, int H, int V, float scale) {
  __shared__ float red[17];
  int t = blockIdx.x;
  int id = ids[t];
  float* o = out + (size_t)t * H;
  float ss = 0.f;
  if (id < 0 || id >= V) {
    for (int j = threadIdx.x; j < H; j += blockDim.x) o[j] = __uint_as_float(0x7fc00000u);
    ss = __uint_as_float(0x7fc00000u);
  } else {
    const T* row = table + (size_t)id * H;
    if ((H & 7) == 0 && aligned16(row) && aligned16(o) && (!xs || (aligned16(next_w) && aligned16(xs)))) {
      // eight values per thread and turn, 16-byte loads and stores
      for (int j = threadIdx.x * 8; j < H; j += blockDim.x * 8) {
        float v[8];
        load8f(row + j, v);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] *= scale;
        store8f(o + j, v);
#pragma unroll
        for (int i = 0; i < 8; ++i) ss += v[i] * v[i];
        if (xs) {
          float w[8];
          load8f(next_w + j, w);
#pragma unroll
          for (int i = 0; i < 8; ++i) w[i] *= v[i];
          store8f(xs + (xs_tiles ? tiled_index(t, j, xs_tiles) : (size_t)t * H + j), w);
        }
      }
    } else {
      for (int j = threadIdx.x; j < H; j += blockDim.x) {
        float v = to_f32(row[j]) * scale;
        o[j] = v;
        ss += v * v;
        if (xs) xs[xs_tiles ? tiled_index(t, j, xs_tiles) : (size_t)t * H + j] = f32_to_bf16(v * next_w[j]);
      }
    }
  }
  if (ssq) {
    ss = block_sum(ss, red);
    if (threadIdx.x == 0) ssq[t] = ss;
  }
}

extern "C" int gs_embed(const int* ids, const void* table, int table_dtype, float* out, float* ssq,
                        const float* next_w, void* xs, int xs_tiled, int T, int H, int V, float scale,
                        hipStream_t stream) {
  GS_REQUIRE(T >= 0 && H > 0 && V > 0, "embed: bad sizes T=%d H=%d V=%d", T, H, V);
  GS_REQUIRE(!xs_tiled || (xs && H % 32 == 0), "embed: tiled rows need a width that is a multiple of 32, not %d", H);
  const int xs_tiles = xs_tiled ? gs_ceil_div(T, 16) : 0;
  if (T == 0) return 0;
  if (table_dtype == GS_F32)
    embed_kernel<float><<<T, 256, 0, stream>>>(ids, (const float*)table, out, ssq, next_w, (bf16*)xs, xs_tiles, H, V, scale);
  else if (table_dtype == GS_BF16)
    embed_kernel<bf16><<<T, 256, 0, stream>>>(ids, (const bf16*)table, out, ssq, next_w, (bf16*)xs, xs_tiles, H, V, scale);
  else
    GS_REQUIRE(false, "embed: unknown dtype %d", table_dtype);
  GS_LAUNCH_CHECK("embed");
  return 0;
}

// ------------------------------------------------------------------ residual add from partial sums (+ RMSNorm)

// One block per row: delta = sum over the parts of K (in order), rounded to bfloat16 as a product's result is
// before the add; res += delta; ssq[row] = sum of squares of the new row; and, with next_w, the row normed for
// the norm that reads the stream next: normed = res / sqrt(mean(res^2) + eps) * next_w (as rows of N or, with
// tiles = ceil(M / 16) > 0, as tiled rows).
template <typename TO>
__global__ void residual_from_parts_kernel(const float* __restrict__ part, int parts, float* __restrict__ res,
                                           float* __restrict__ ssq, const float* __restrict__ next_w, float eps,
                                           TO* __restrict__ normed, int tiles, int M, int N) {
  __shared__ float red[17];
  const int m = blockIdx.x;
  float* x = res + (size_t)m * N;
  constexpr int MAXV = 4;                         // values kept in registers between the passes: rows up to 4096
  float keep[MAXV][4];
  float ss = 0.f;
  const bool vec = (N & 3) == 0;
  const int turns = (N + 4 * blockDim.x - 1) / (4 * blockDim.x);
  for (int u = 0; u < turns; ++u) {
    const int j = (u * blockDim.x + threadIdx.x) * 4;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    if (j < N) {
      float d[4] = {0.f, 0.f, 0.f, 0.f};
      if (vec) {
        // eight parts' loads are issued together, then added in the order of the parts
        for (int p0 = 0; p0 < parts; p0 += 8) {
          float4 a[8];
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            const int p = p0 + q < parts ? p0 + q : parts - 1;
            a[q] = *reinterpret_cast<const float4*>(part + ((size_t)p * M + m) * N + j);
          }
#pragma unroll
          for (int q = 0; q < 8; ++q)
            if (p0 + q < parts) {
              d[0] += a[q].x; d[1] += a[q].y; d[2] += a[q].z; d[3] += a[q].w;
            }
        }
      } else {
        for (int p = 0; p < parts; ++p) {
          const float* src = part + ((size_t)p * M + m) * N + j;
          for (int i = 0; i < 4; ++i)
            if (j + i < N) d[i] += src[i];
        }
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (j + i < N) {
          v[i] = x[j + i] + to_f32(f32_to_bf16(d[i]));
          x[j + i] = v[i];
          ss += v[i] * v[i];
        }
    }
    if (u < MAXV) {
#pragma unroll
      for (int i = 0; i < 4; ++i) keep[u][i] = v[i];
    }
  }
  ss = block_sum(ss, red);
  if (threadIdx.x == 0) ssq[m] = ss;
  if (!normed) return;
  const float inv = norm_inverse(ss, (float)N, eps);
  for (int u = 0; u < turns; ++u) {
    const int j = (u * blockDim.x + threadIdx.x) * 4;
    if (j >= N) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (j + i < N) {
        const float v = u < MAXV ? keep[u][i] : x[j + i];
        normed[tiles ? tiled_index(m, j + i, tiles) : (size_t)m * N + j + i] = from_f32<TO>(v * inv * next_w[j + i]);
      }
  }
}

extern "C" int gs_residual_from_parts(const float* part, int parts, float* res, float* ssq, const float* next_w,
                                      float eps, void* normed, int normed_dtype, int normed_tiled, int M, int N,
                                      hipStream_t stream) {
  GS_REQUIRE(!normed_tiled || (normed && normed_dtype == GS_BF16 && N % 32 == 0),
             "residual_from_parts: tiled rows are bfloat16 and a multiple of 32 wide, not %d", N);
  const int tiles = normed_tiled ? gs_ceil_div(M, 16) : 0;
  GS_REQUIRE(M >= 0 && N > 0 && parts >= 1, "residual_from_parts: bad sizes M=%d N=%d parts=%d", M, N, parts);
  GS_REQUIRE(part && res && ssq, "residual_from_parts: needs the partial sums, the stream and room for the sums of squares");
  GS_REQUIRE((next_w == nullptr) == (normed == nullptr), "residual_from_parts: the next norm's weight and the room for the normed rows come together");
  GS_REQUIRE(((uintptr_t)part & 15) == 0, "residual_from_parts: the partial sums must be 16-byte aligned");
  if (M == 0) return 0;
  const int threads = N >= 4096 ? 1024 : (N >= 2048 ? 512 : 256);   // four values a thread and turn
  if (!normed || normed_dtype == GS_BF16)
    residual_from_parts_kernel<bf16><<<M, threads, 0, stream>>>(part, parts, res, ssq, next_w, eps, (bf16*)normed, tiles, M, N);
  else if (normed_dtype == GS_F32)
    residual_from_parts_kernel<float><<<M, threads, 0, stream>>>(part, parts, res, ssq, next_w, eps, (float*)normed, tiles, M, N);
  else
    GS_REQUIRE(false, "residual_from_parts: unknown dtype %d", normed_dtype);
  GS_LAUNCH_CHECK("residual_from_parts");
  return 0;
}

// ------------------------------------------------------------------ rows <-> tiled rows

// One thread per eight consecutive columns of a row: out = the same values in the other order.
__global__ void retile_rows_kernel(const bf16* __restrict__ in, bf16* __restrict__ out, int M, int K, int ld,
                                   int tiles, int to_tiled) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const int k8 = K >> 3;
  if (i >= (long)M * k8) return;
  const int m = (int)(i / k8), k = (int)(i - (long)m * k8) * 8;
  const size_t rowwise = (size_t)m * ld + k, tiled = tiled_index(m, k, tiles);
  *reinterpret_cast<uint4*>(out + (to_tiled ? tiled : rowwise)) =
      *reinterpret_cast<const uint4*>(in + (to_tiled ? rowwise : tiled));
}

// rows (M, K) with row stride ld <-> tiled rows of (K / 32) * ceil(M / 16) * 512 elements; bfloat16.
// Rows beyond M inside the last row tile are left as they are.
extern "C" int gs_retile_rows(const void* in, void* out, int M, int K, int ld, int to_tiled, hipStream_t stream) {
  GS_REQUIRE(M >= 0 && K > 0 && K % 32 == 0 && ld >= K && ld % 8 == 0, "retile_rows: K=%d must be a multiple of 32, the row stride %d one of 8", K, ld);
  GS_REQUIRE(((uintptr_t)in & 15) == 0 && ((uintptr_t)out & 15) == 0, "retile_rows: operands must be 16-byte aligned");
  if (M == 0) return 0;
  const long n = (long)M * (K / 8);
  retile_rows_kernel<<<gs_ceil_div(n, 256), 256, 0, stream>>>((const bf16*)in, (bf16*)out, M, K, ld, gs_ceil_div(M, 16), to_tiled);
  GS_LAUNCH_CHECK("retile_rows");
  return 0;
}

// ------------------------------------------------------------------ add + RMSNorm

// One block per output row r.  Source row s = rows ? rows[r] : r.
//   x = res[s] (+ delta[s]);  out[r] = x / sqrt(mean(x^2) + eps) * w
// Without `rows` the sum is written back to res (the stream moves on); with `rows` (a gather
// at the model's end) res is left as it is, so a row may be asked for twice.
template <typename TD, typename TO>
__global__ void add_rmsnorm_kernel(float* __restrict__ res, const TD* __restrict__ delta, const float* __restrict__ w,
                                   float eps, TO* __restrict__ out, const int* __restrict__ rows, int H) {
  __shared__ float red[17];
  int r = blockIdx.x;
  int s = rows ? rows[r] : r;
  float* x = res + (size_t)s * H;
  const TD* dl = delta ? delta + (size_t)s * H : nullptr;
  float ss = 0.f;
  TO* o = out + (size_t)r * H;
  if ((H & 7) == 0 && aligned16(x) && aligned16(o) && aligned16(w) && (!dl || aligned16(dl))) {
    // eight values per thread and turn, 16-byte loads and stores; the row stays in registers between the passes
    constexpr int MAXV = 4;                       // turns kept in registers: rows up to 8 * 256 * 4 values
    float keep[MAXV][8];
    const int turns = (H / 8 + blockDim.x - 1) / blockDim.x;
    for (int u = 0; u < turns; ++u) {
      const int j = (u * blockDim.x + threadIdx.x) * 8;
      float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (j < H) {
        load8f(x + j, v);
        if (dl) {
          float d8[8];
          load8f(dl + j, d8);
#pragma unroll
          for (int i = 0; i < 8; ++i) v[i] += d8[i];
          if (!rows) store8f(x + j, v);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) ss += v[i] * v[i];
      }
      if (u < MAXV) {
#pragma unroll
        for (int i = 0; i < 8; ++i) keep[u][i] = v[i];
      }
    }
    ss = block_sum(ss, red);
    const float inv = norm_inverse(ss, (float)H, eps);
    for (int u = 0; u < turns; ++u) {
      const int j = (u * blockDim.x + threadIdx.x) * 8;
      if (j >= H) break;
      float v[8], w8[8];
      if (u < MAXV) {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = keep[u][i];
      } else {
        load8f(x + j, v);
        if (dl && rows) {
          float d8[8];
          load8f(dl + j, d8);
#pragma unroll
          for (int i = 0; i < 8; ++i) v[i] += d8[i];
        }
      }
      load8f(w + j, w8);
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = v[i] * inv * w8[i];
      store8f(o + j, v);
    }
    return;
  }
  for (int j = threadIdx.x; j < H; j += blockDim.x) {
    float v = x[j];
    if (dl) {
      v += to_f32(dl[j]);
      if (!rows) x[j] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, red);
  float inv = norm_inverse(ss, (float)H, eps);
  for (int j = threadIdx.x; j < H; j += blockDim.x) {
    float v = x[j];
    if (dl && rows) v += to_f32(dl[j]);
    o[j] = from_f32<TO>(v * inv * w[j]);
  }
}

extern "C" int gs_add_rmsnorm(float* res, const void* delta, int delta_dtype, const float* w, float eps, void* out,
                              int out_dtype, const int* rows, int n_out, int H, hipStream_t stream) {
  GS_REQUIRE(n_out >= 0 && H > 0, "add_rmsnorm: bad sizes rows=%d H=%d", n_out, H);
  GS_REQUIRE(eps > 0.f, "add_rmsnorm: eps must be positive");
  if (n_out == 0) return 0;
  int threads = H >= 1024 ? 256 : (H >= 256 ? 128 : 64);
#define GS_RUN(TD, TO)                                                                                          \
  add_rmsnorm_kernel<TD, TO><<<n_out, threads, 0, stream>>>(res, (const TD*)delta, w, eps, (TO*)out, rows, H)
  if (delta_dtype == GS_F32 && out_dtype == GS_F32)
    GS_RUN(float, float);
  else if (delta_dtype == GS_BF16 && out_dtype == GS_BF16)
    GS_RUN(bf16, bf16);
  else if (delta_dtype == GS_F32 && out_dtype == GS_BF16)
    GS_RUN(float, bf16);
  else if (delta_dtype == GS_BF16 && out_dtype == GS_F32)
    GS_RUN(bf16, float);
  else
    GS_REQUIRE(false, "add_rmsnorm: unknown dtypes %d %d", delta_dtype, out_dtype);
#undef GS_RUN
  GS_LAUNCH_CHECK("add_rmsnorm");
  return 0;
}

// out[t, :] = res[t, :] * inv_rms(t) * w, the row's sum of squares given as nb partial sums (added in a
// fixed order).  The norm of a stream whose sums a product's epilogue has already taken: no pass over
// the row is needed to find them.
// One wavefront per (row, chunk of 512 columns): every wavefront adds the row's partial sums itself
// (a few loads and shuffles), so there is no block-wide barrier and the loads of the row's values
// are under way while the sums are added.
template <typename TO>
__global__ void norm_from_ssq_kernel(const float* __restrict__ res, const float* __restrict__ ssq, int nb,
                                     const float* __restrict__ w, float eps, TO* __restrict__ out, int H) {
  const int t = blockIdx.y, lane = threadIdx.x;
  const int j0 = blockIdx.x * 512 + lane * 8;
  float x[8], wv[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    x[i] = (j0 + i < H) ? res[(size_t)t * H + j0 + i] : 0.f;
    wv[i] = (j0 + i < H) ? w[j0 + i] : 0.f;
  }
  float s = 0.f;
  for (int b = lane; b < nb; b += 64) s += ssq[(size_t)t * nb + b];
  s = wave_sum(s);
  const float inv = norm_inverse(s, (float)H, eps);
#pragma unroll
  for (int i = 0; i < 8; ++i)
    if (j0 + i < H) out[(size_t)t * H + j0 + i] = from_f32<TO>(x[i] * inv * wv[i]);
}

extern "C" int gs_norm_from_ssq(const float* res, const float* ssq, int nb, const float* w, float eps, void* out,
                                int out_dtype, int T, int H, hipStream_t stream) {
  GS_REQUIRE(T >= 0 && H > 0 && nb > 0 && eps > 0.f, "norm_from_ssq: bad sizes T=%d H=%d nb=%d", T, H, nb);
  GS_REQUIRE(T <= 65535, "norm_from_ssq: more than 65535 rows");
  if (T == 0) return 0;
  dim3 grid(gs_ceil_div(H, 512), T);
  if (out_dtype == GS_BF16)
    norm_from_ssq_kernel<bf16><<<grid, 64, 0, stream>>>(res, ssq, nb, w, eps, (bf16*)out, H);
  else if (out_dtype == GS_F32)
    norm_from_ssq_kernel<float><<<grid, 64, 0, stream>>>(res, ssq, nb, w, eps, (float*)out, H);
  else
    GS_REQUIRE(false, "norm_from_ssq: unknown dtype %d", out_dtype);
  GS_LAUNCH_CHECK("norm_from_ssq");
  return 0;
}

// res[t, :] += delta[t, :]   (the last sub-layer's output, when no norm follows it)
template <typename TD>
__global__ void add_kernel(float* __restrict__ res, const TD* __restrict__ delta, long n) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) res[i] += to_f32(delta[i]);
}

extern "C" int gs_residual_add(float* res, const void* delta, int delta_dtype, long n, hipStream_t stream) {
  GS_REQUIRE(n >= 0, "residual_add: bad size");
  if (n == 0) return 0;
  int blocks = gs_ceil_div(n, 256);
  if (delta_dtype == GS_F32)
    add_kernel<float><<<blocks, 256, 0, stream>>>(res, (const float*)delta, n);
  else if (delta_dtype == GS_BF16)
    add_kernel<bf16><<<blocks, 256, 0, stream>>>(res, (const bf16*)delta, n);
  else
    GS_REQUIRE(false, "residual_add: unknown dtype %d", delta_dtype);
  GS_LAUNCH_CHECK("residual_add");
  return 0;
}

// out[t, j] = y[t, j] + bias[j]: the bias of a product whose float32 sums a matrix-core kernel made; one rounding,
// after the bias.  Four columns per thread when N is a multiple of 4 and the rows are 16-byte aligned.
template <typename TOut, int V>
__global__ void add_bias_kernel(const float* __restrict__ y, const float* __restrict__ bias, TOut* __restrict__ out,
                                int N, long ldo, long n) {
  long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * V;
  if (i >= n) return;
  long t = i / N;
  int j = (int)(i - t * N);
#pragma unroll
  for (int k = 0; k < V; ++k) out[t * ldo + j + k] = from_f32<TOut>(y[i + k] + bias[j + k]);
}

extern "C" int gs_add_bias(const float* y, const float* bias, void* out, int out_dtype, int M, int N, long ldo,
                           hipStream_t stream) {
  GS_REQUIRE(M >= 0 && N > 0 && ldo >= N, "add_bias: bad sizes M=%d N=%d ldo=%ld", M, N, ldo);
  long n = (long)M * N;
  if (n == 0) return 0;
  const bool v4 = N % 4 == 0 && ldo % 4 == 0;
  long threads = v4 ? n / 4 : n;
  int blocks = (int)gs_ceil_div(threads, 256);
  if (out_dtype == GS_F32) {
    if (v4) add_bias_kernel<float, 4><<<blocks, 256, 0, stream>>>(y, bias, (float*)out, N, ldo, n);
    else add_bias_kernel<float, 1><<<blocks, 256, 0, stream>>>(y, bias, (float*)out, N, ldo, n);
  } else if (out_dtype == GS_BF16) {
    if (v4) add_bias_kernel<bf16, 4><<<blocks, 256, 0, stream>>>(y, bias, (bf16*)out, N, ldo, n);
    else add_bias_kernel<bf16, 1><<<blocks, 256, 0, stream>>>(y, bias, (bf16*)out, N, ldo, n);
  } else
    GS_REQUIRE(false, "add_bias: unknown dtype %d", out_dtype);
  GS_LAUNCH_CHECK("add_bias");
  return 0;
}

// ------------------------------------------------------------------ SwiGLU

// in (T, 2F): gate in columns [0, F), up in [F, 2F).  out[t, j] = silu(gate) * up, silu(g) = g / (1 + exp(-g)).
// Eight outputs per thread with 16-byte loads and stores; F a multiple of 8, rows 16-byte aligned.
template <typename T>
__global__ void swiglu8_kernel(const T* __restrict__ in, T* __restrict__ out, int F, long n8) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n8) return;
  const int f8 = F / 8;
  long t = i / f8;
  int j = (int)(i - t * f8) * 8;
  float g[8], u[8];
  load8f(in + t * 2 * F + j, g);
  load8f(in + t * 2 * F + F + j, u);
#pragma unroll
  for (int k = 0; k < 8; ++k) g[k] = g[k] / (1.0f + expf(-g[k])) * u[k];
  store8f(out + t * F + j, g);
}

template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ in, T* __restrict__ out, int F, long n) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  long t = i / F;
  int j = (int)(i - t * F);
  float g = to_f32(in[t * 2 * F + j]);
  float u = to_f32(in[t * 2 * F + F + j]);
  out[i] = from_f32<T>(g / (1.0f + expf(-g)) * u);
}

extern "C" int gs_swiglu(const void* in, void* out, int dtype, int T, int F, hipStream_t stream) {
  GS_REQUIRE(T >= 0 && F > 0, "swiglu: bad sizes T=%d F=%d", T, F);
  long n = (long)T * F;
  if (n == 0) return 0;
  if (F % 8 == 0 && ((uintptr_t)in & 15) == 0 && ((uintptr_t)out & 15) == 0 && (dtype == GS_F32 || dtype == GS_BF16)) {
    long n8 = n / 8;
    if (dtype == GS_F32)
      swiglu8_kernel<float><<<gs_ceil_div(n8, 256), 256, 0, stream>>>((const float*)in, (float*)out, F, n8);
    else
      swiglu8_kernel<bf16><<<gs_ceil_div(n8, 256), 256, 0, stream>>>((const bf16*)in, (bf16*)out, F, n8);
    GS_LAUNCH_CHECK("swiglu");
    return 0;
  }
  int blocks = gs_ceil_div(n, 256);
  if (dtype == GS_F32)
    swiglu_kernel<float><<<blocks, 256, 0, stream>>>((const float*)in, (float*)out, F, n);
  else if (dtype == GS_BF16)
    swiglu_kernel<bf16><<<blocks, 256, 0, stream>>>((const bf16*)in, (bf16*)out, F, n);
  else
    GS_REQUIRE(false, "swiglu: unknown dtype %d", dtype);
  GS_LAUNCH_CHECK("swiglu");
  return 0;
}

// ------------------------------------------------------------------ fills

// Soft cap of logits in place: x = cap * tanh(x / cap) (the reference's final_logit_softcap of the families that
// have one, src/Inference/architecture_spec.jl:248; not an LFM2 feature).
__global__ void softcap_kernel(float* p, float cap, long n) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = cap * tanhf(p[i] / cap);
}

extern "C" int gs_softcap(float* p, float cap, long n, hipStream_t stream) {
  GS_REQUIRE(n >= 0 && cap > 0.f, "softcap: the cap must be positive");
  if (n == 0) return 0;
  softcap_kernel<<<gs_ceil_div(n, 256), 256, 0, stream>>>(p, cap, n);
  GS_LAUNCH_CHECK("softcap");
  return 0;
}

// Reads a buffer once with 16-byte loads, eight in flight per lane, and folds what it read into one word per block:
// a measurement of what the memory system delivers to kernels of this library's kind (the ceiling that the decode
// step's weight streams are held against), nothing the model uses.  A block walks a contiguous share of the buffer,
// 32 KB a turn, as a weight-streaming product walks its rows (contiguous = 1), or the whole grid sweeps the buffer
// together, neighbours in the grid reading neighbours in memory (contiguous = 0).
__global__ __launch_bounds__(256) void stream_read_kernel(const uint4* __restrict__ p, long n16, int contiguous,
                                                          unsigned* __restrict__ sink) {
  unsigned acc = 0;
  long i, end, step, lane_step;
  if (contiguous) {
    const long per = ((n16 + gridDim.x - 1) / gridDim.x + 2047) / 2048 * 2048;   // whole turns of 8 x 256 words
    i = (long)blockIdx.x * per + threadIdx.x;
    end = (long)(blockIdx.x + 1) * per < n16 ? (long)(blockIdx.x + 1) * per : n16;
    lane_step = blockDim.x;
    step = 8 * lane_step;
  } else {
    lane_step = (long)gridDim.x * blockDim.x;
    i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    end = n16;
    step = 8 * lane_step;
  }
  for (; i + 7 * lane_step < end; i += step) {
    uint4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = p[i + u * lane_step];
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; i < end; i += lane_step) {
    const uint4 v = p[i];
    acc ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  if (acc == 0x9e3779b9u) sink[blockIdx.x] = acc;     // practically never: the store only keeps the loads alive
}

extern "C" int gs_stream_read(const void* p, long bytes, unsigned* sink, int blocks, int contiguous, hipStream_t stream) {
  GS_REQUIRE(bytes >= 0 && bytes % 16 == 0 && ((uintptr_t)p & 15) == 0, "stream_read: a 16-byte aligned buffer of whole 16-byte words");
  GS_REQUIRE(blocks > 0 && blocks <= 65535 && sink, "stream_read: 1 to 65535 blocks and a word per block to write to");
  if (bytes == 0) return 0;
  stream_read_kernel<<<blocks, 256, 0, stream>>>((const uint4*)p, bytes / 16, contiguous, sink);
  GS_LAUNCH_CHECK("stream_read");
  return 0;
}

// Fill chosen rows of a pool with one value: pool (outer, num_rows, row) of float32 or bfloat16, ids (n) rows to
// fill in every one of the `outer` planes (a negative id is skipped).  A request's state slots are rows of a pool
// with one plane, a cache page is a row in each layer's K and V plane.  Used to give a fresh slot its initial
// value and to poison what a request gave back.
template <typename T>
__global__ void fill_rows_kernel(T* pool, const int* ids, long row, long plane, T value) {
  const int id = ids[blockIdx.y];
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= 0 && i < row) pool[(size_t)blockIdx.z * plane + (size_t)id * row + i] = value;
}

extern "C" int gs_fill_rows(void* pool, int dtype, const int* ids, int n, long row, int outer, long num_rows, float value,
                            hipStream_t stream) {
  GS_REQUIRE(n >= 0 && row >= 0 && outer >= 0 && num_rows >= 0, "fill_rows: bad sizes");
  GS_REQUIRE(n <= 65535 && outer <= 65535, "fill_rows: %d rows in %d planes are more than one launch takes", n, outer);
  if (n == 0 || row == 0 || outer == 0) return 0;
  dim3 grid(gs_ceil_div(row, 256), n, outer);
  if (dtype == GS_F32)
    fill_rows_kernel<float><<<grid, 256, 0, stream>>>((float*)pool, ids, row, num_rows * row, value);
  else if (dtype == GS_BF16)
    fill_rows_kernel<bf16><<<grid, 256, 0, stream>>>((bf16*)pool, ids, row, num_rows * row, host_bf16(value));
  else
    GS_REQUIRE(false, "fill_rows: unknown dtype %d", dtype);
  GS_LAUNCH_CHECK("fill_rows");
  return 0;
}
