// Per-head RMSNorm of q and k, rotary position encoding, and the write of K and V into the cache pages.
//
// qkv (T, (nh + 2 nkv) d): q heads, then k heads, then v heads, each head d wide.
//   q, k: x = x / sqrt(mean(x^2) + eps) * w  over the head (when a weight is given), then for the
//         first rotary_dim features, pairs (a, b) = (i, i + rotary_dim/2) ("half-split") or, with `interleaved`,
//         (2i, 2i + 1) (reference src/Operators/cpu.jl:357-371):
//           x_a' = x_a cos - x_b sin,  x_b' = x_a sin + x_b cos,  angle = pos * theta^(-2i/rotary_dim)
//         with cos/sin row i from a table (max_position, rotary_dim/2) made on the host in float64.
//   q is written back in place; k (after norm and rotation) and v (as it is) go to the cache:
//   page = block_table[seq, pos / page_size], row = pos % page_size,
//   cache (num_pages, nkv, page_size, d).
// One wave per (token, head).  All arithmetic float32.
#include "common.h"

template <typename T>
__global__ void qknorm_rope_kv_kernel(T* __restrict__ qkv, const float* __restrict__ qw, const float* __restrict__ kw,
                                      float eps, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                      int rotary_dim, int interleaved, const int* __restrict__ positions,
                                      const int* __restrict__ seq_of_token, const int* __restrict__ block_table,
                                      int max_blocks, int page_size, T* __restrict__ kcache, T* __restrict__ vcache,
                                      int ntok, int nh, int nkv, int d, int write_kv) {
  int lane = threadIdx.x & 63;
  int heads = nh + 2 * nkv;
  long unit = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (unit >= (long)ntok * heads) return;
  int t = (int)(unit / heads);
  int hh = (int)(unit - (long)t * heads);
  T* x = qkv + ((size_t)t * heads + hh) * d;
  int pos = positions[t];

  T* dst = nullptr;  // cache row for k and v heads
  if (hh >= nh) {
    if (!write_kv) return;
    int kvh = hh < nh + nkv ? hh - nh : hh - nh - nkv;
    int page = block_table[(size_t)seq_of_token[t] * max_blocks + pos / page_size];
    T* base = hh < nh + nkv ? kcache : vcache;
    dst = base + (((size_t)page * nkv + kvh) * page_size + pos % page_size) * d;
  }
  if (hh >= nh + nkv) {  // v: copy
    for (int j = lane; j < d; j += 64) dst[j] = x[j];
    return;
  }

  const float* w = hh < nh ? qw : kw;
  float inv = 1.f;
  if (w) {
    float ss = 0.f;
    for (int j = lane; j < d; j += 64) {
      float v = to_f32(x[j]);
      ss += v * v;
    }
    ss = wave_sum(ss);
    inv = norm_inverse(ss, (float)d, eps);
  }
  T* o = hh < nh ? x : dst;
  int half = rotary_dim >> 1;
  const float* cr = cos_t ? cos_t + (size_t)pos * half : nullptr;
  const float* sr = sin_t ? sin_t + (size_t)pos * half : nullptr;
  for (int i = lane; i < half; i += 64) {
    const int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + half;
    float a = to_f32(x[ia]) * inv, b = to_f32(x[ib]) * inv;
    if (w) {
      a *= w[ia];
      b *= w[ib];
    }
    float c = cr[i], s = sr[i];
    o[ia] = from_f32<T>(a * c - b * s);
    o[ib] = from_f32<T>(a * s + b * c);
  }
  for (int j = rotary_dim + lane; j < d; j += 64) {  // features beyond the rotary part
    float a = to_f32(x[j]) * inv;
    if (w) a *= w[j];
    o[j] = from_f32<T>(a);
  }
}

// The same for head widths of 16, 32, 64 and 128 that are rotated whole (rotary_dim == d): L = d / 8 lanes per
// (token, head), eight features a lane, 16-byte loads and stores; the halves of a rotation pair sit L/2 lanes apart.
template <typename T, int L>
__global__ void qknorm_rope_kv_vec_kernel(T* __restrict__ qkv, const float* __restrict__ qw,
                                          const float* __restrict__ kw, float eps, const float* __restrict__ cos_t,
                                          const float* __restrict__ sin_t, const int* __restrict__ positions,
                                          const int* __restrict__ seq_of_token, const int* __restrict__ block_table,
                                          int max_blocks, int page_size, T* __restrict__ kcache,
                                          T* __restrict__ vcache, int ntok, int nh, int nkv, int write_kv) {
  constexpr int d = 8 * L, half = d / 2;
  const int heads = nh + 2 * nkv;
  const long unit = ((long)blockIdx.x * blockDim.x + threadIdx.x) / L;
  const int sub = threadIdx.x % L;
  const bool live = unit < (long)ntok * heads;   // lanes past the end run along for the shuffles, on unit 0
  const long un = live ? unit : 0;
  const int t = (int)(un / heads);
  const int hh = (int)(un - (long)t * heads);
  T* x = qkv + ((size_t)t * heads + hh) * d + sub * 8;
  const int pos = positions[t];
  const bool is_q = hh < nh, is_k = !is_q && hh < nh + nkv;
  T* o = x;
  if (!is_q) {
    const int kvh = is_k ? hh - nh : hh - nh - nkv;
    const int page = block_table[(size_t)seq_of_token[t] * max_blocks + pos / page_size];
    o = (is_k ? kcache : vcache) + (((size_t)page * nkv + kvh) * page_size + pos % page_size) * d + sub * 8;
  }
  float v[8];
  load8f(x, v);
  if (is_q || is_k) {
    const float* w = is_q ? qw : kw;
    if (w) {
      float ss = 0.f;
#pragma unroll
      for (int k = 0; k < 8; ++k) ss += v[k] * v[k];
#pragma unroll
      for (int m = 1; m < L; m <<= 1) ss += __shfl_xor(ss, m, 64);
      const float inv = norm_inverse(ss, (float)d, eps);
      float w8[8];
      load8f(w + sub * 8, w8);
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = v[k] * inv * w8[k];
    }
    const bool low = sub < L / 2;                 // holds the first halves (i) of its pairs, else the second (j)
    const int i0 = (low ? sub : sub - L / 2) * 8;
    float c8[8], s8[8];
    load8f(cos_t + (size_t)pos * half + i0, c8);
    load8f(sin_t + (size_t)pos * half + i0, s8);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float other = __shfl_xor(v[k], L / 2, 64);
      // x_i' = x_i cos - x_j sin,  x_j' = x_i sin + x_j cos
      v[k] = low ? v[k] * c8[k] - other * s8[k] : other * s8[k] + v[k] * c8[k];
    }
  }
  if (live && (is_q || write_kv)) store8f(o, v);
}

extern "C" int gs_qknorm_rope_kv(void* qkv, int dtype, const float* qw, const float* kw, float eps,
                                 const float* cos_t, const float* sin_t, int rotary_dim, int interleaved,
                                 int max_position, const int* positions, const int* seq_of_token, const int* block_table,
                                 int max_blocks, int page_size, void* kcache, void* vcache, int ntok, int nh, int nkv,
                                 int d, int write_kv, hipStream_t stream) {
  GS_REQUIRE(ntok >= 0 && nh > 0 && nkv > 0 && d > 0, "qknorm_rope_kv: bad sizes T=%d nh=%d nkv=%d d=%d", ntok, nh,
             nkv, d);
  GS_REQUIRE(rotary_dim >= 0 && rotary_dim <= d && rotary_dim % 2 == 0,
             "qknorm_rope_kv: rotary_dim %d must be even and at most the head width %d", rotary_dim, d);
  GS_REQUIRE(rotary_dim == 0 || (cos_t && sin_t && max_position > 0), "qknorm_rope_kv: rotation without a table");
  GS_REQUIRE(page_size > 0 && max_blocks > 0, "qknorm_rope_kv: bad page_size %d or max_blocks %d", page_size,
             max_blocks);
  GS_REQUIRE((qw == nullptr) == (kw == nullptr), "qknorm_rope_kv: q and k norm weights come together");
  if (ntok == 0) return 0;
  long units = (long)ntok * (nh + 2 * nkv);
  const bool vec = !interleaved && rotary_dim == d && (d == 16 || d == 32 || d == 64 || d == 128) && (dtype == GS_F32 || dtype == GS_BF16) &&
                   ((uintptr_t)qkv & 15) == 0 && ((uintptr_t)kcache & 15) == 0 && ((uintptr_t)vcache & 15) == 0 &&
                   ((uintptr_t)cos_t & 15) == 0 && ((uintptr_t)sin_t & 15) == 0 && ((uintptr_t)qw & 15) == 0 &&
                   ((uintptr_t)kw & 15) == 0;
  if (vec) {
    const int L = d / 8;
    const int vblocks = gs_ceil_div(units * L, 256);
#define GS_VEC(T, LL)                                                                                              \
  qknorm_rope_kv_vec_kernel<T, LL><<<vblocks, 256, 0, stream>>>((T*)qkv, qw, kw, eps, cos_t, sin_t, positions,     \
                                                                seq_of_token, block_table, max_blocks, page_size, \
                                                                (T*)kcache, (T*)vcache, ntok, nh, nkv, write_kv)
#define GS_VEC_T(T)                                                                     \
  switch (L) {                                                                          \
    case 2: GS_VEC(T, 2); break;                                                        \
    case 4: GS_VEC(T, 4); break;                                                        \
    case 8: GS_VEC(T, 8); break;                                                        \
    default: GS_VEC(T, 16); break;                                                      \
  }
    if (dtype == GS_F32) { GS_VEC_T(float) } else { GS_VEC_T(bf16) }
#undef GS_VEC_T
#undef GS_VEC
    GS_LAUNCH_CHECK("qknorm_rope_kv");
    return 0;
  }
  int blocks = gs_ceil_div(units, 4);
#define GS_RUN(T)                                                                                               \
  qknorm_rope_kv_kernel<T><<<blocks, 256, 0, stream>>>((T*)qkv, qw, kw, eps, cos_t, sin_t, rotary_dim, interleaved, positions, \
                                                       seq_of_token, block_table, max_blocks, page_size,        \
                                                       (T*)kcache, (T*)vcache, ntok, nh, nkv, d, write_kv)
  if (dtype == GS_F32)
    GS_RUN(float);
  else if (dtype == GS_BF16)
    GS_RUN(bf16);
  else
    GS_REQUIRE(false, "qknorm_rope_kv: unknown dtype %d", dtype);
#undef GS_RUN
  GS_LAUNCH_CHECK("qknorm_rope_kv");
  return 0;
}
