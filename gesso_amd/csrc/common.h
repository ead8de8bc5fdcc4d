// Shared helpers of the gfx950 kernels: storage types, conversions, reductions, error reporting.
//
// Every entry point is extern "C", takes raw device pointers, sizes and a stream, checks
// what it assumes about sizes on the host, and returns 0 or a negative code after recording
// a message that gs_last_error() returns.  dtype codes: 0 = float32, 1 = bfloat16.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#define GS_F32 0
#define GS_BF16 1

#define GS_WAVE 64

// The float32 products add k in chunks of this many, and then the chunks' sums, both in ascending order.
#define GS_SUM_CHUNK 64

extern "C" const char* gs_last_error();
void gs_set_error(const char* fmt, ...);

#define GS_REQUIRE(cond, ...)            \
  do {                                   \
    if (!(cond)) {                       \
      gs_set_error(__VA_ARGS__);         \
      return -1;                         \
    }                                    \
  } while (0)

#define GS_LAUNCH_CHECK(name)                                                 \
  do {                                                                        \
    hipError_t e_ = hipGetLastError();                                        \
    if (e_ != hipSuccess) {                                                   \
      gs_set_error("%s: launch failed: %s", name, hipGetErrorString(e_));     \
      return -2;                                                              \
    }                                                                         \
  } while (0)

// bfloat16 as bits; conversions are explicit so that every rounding is visible in the code.
struct bf16 {
  uint16_t x;
};

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16 v) { return __uint_as_float(((uint32_t)v.x) << 16); }

// round to nearest, ties to even; NaN stays NaN (gfx950 converts in hardware: v_cvt_pk_bf16_f32)
__device__ __forceinline__ bf16 f32_to_bf16(float f) {
  bf16 r;
  r.x = __builtin_bit_cast(uint16_t, (__bf16)f);
  return r;
}

template <typename T>
__device__ __forceinline__ T from_f32(float v);
template <>
__device__ __forceinline__ float from_f32<float>(float v) {
  return v;
}
template <>
__device__ __forceinline__ bf16 from_f32<bf16>(float v) {
  return f32_to_bf16(v);
}

// 1 / sqrt(mean + eps) of a norm, from the sum of squares ss over n values.  A denominator that is not finite or not
// positive (the reference raises a numerical-instability error there, src/Operators/cpu.jl:260-266) gives NaN: it
// poisons the row, so that the choice of the next token fails for this request alone, also where the row's values are
// finite and only their sum of squares has overflowed (1 / inf would quietly give a row of zeros).
__device__ __forceinline__ float norm_inverse(float ss, float n, float eps) {
  const float r = sqrtf(ss / n + eps);
  return (r > 0.f && r < INFINITY) ? 1.0f / r : __builtin_nanf("");
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, GS_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, GS_WAVE));
  return v;
}
__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, GS_WAVE);
  return v;
}

// Maximum and sum over the four lanes l, l ^ 16, l ^ 32, l ^ 48 (the lane groups that share a column of an
// MFMA result), by gfx950's row swaps: VALU moves, no trip through the LDS crossbar.
__device__ __forceinline__ float group4_max(float x) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float group4_sum(float x) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Maximum and sum over the wavefront without the LDS crossbar: data-parallel moves within rows of 16 lanes
// (quad swaps, then mirrors of 8 and of 16 lanes), then the row swaps.  The order of the additions is fixed.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float x) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float wave_max_dpp(float x) {
  x = fmaxf(x, dpp_move<0xB1>(x));   // quad_perm [1,0,3,2]
  x = fmaxf(x, dpp_move<0x4E>(x));   // quad_perm [2,3,0,1]
  x = fmaxf(x, dpp_move<0x141>(x));  // row_half_mirror
  x = fmaxf(x, dpp_move<0x140>(x));  // row_mirror
  return group4_max(x);
}
__device__ __forceinline__ float wave_sum_dpp(float x) {
  x += dpp_move<0xB1>(x);
  x += dpp_move<0x4E>(x);
  x += dpp_move<0x141>(x);
  x += dpp_move<0x140>(x);
  return group4_sum(x);
}

// Sum over a block of up to 1024 threads; every thread gets the result.  `red` holds 17 floats.
__device__ __forceinline__ float block_sum(float v, float* red) {
  int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = 0.f;
    for (int i = 0; i < nw; ++i) s += red[i];
    red[16] = s;
  }
  __syncthreads();
  return red[16];
}

// Eight consecutive values as float, from float32 or bfloat16 storage (16-byte aligned), and back.
__device__ __forceinline__ void load8f(const float* p, float* v) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load8f(const bf16* p, float* v) {
  const uint4 w = *reinterpret_cast<const uint4*>(p);
  const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    v[2 * e] = __uint_as_float(ww[e] << 16);
    v[2 * e + 1] = __uint_as_float(ww[e] & 0xffff0000u);
  }
}
__device__ __forceinline__ void store8f(float* p, const float* v) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ void store8f(bf16* p, const float* v) {
  uint4 w;
  w.x = (uint32_t)f32_to_bf16(v[0]).x | ((uint32_t)f32_to_bf16(v[1]).x << 16);
  w.y = (uint32_t)f32_to_bf16(v[2]).x | ((uint32_t)f32_to_bf16(v[3]).x << 16);
  w.z = (uint32_t)f32_to_bf16(v[4]).x | ((uint32_t)f32_to_bf16(v[5]).x << 16);
  w.w = (uint32_t)f32_to_bf16(v[6]).x | ((uint32_t)f32_to_bf16(v[7]).x << 16);
  *reinterpret_cast<uint4*>(p) = w;
}
template <typename T>
__device__ __forceinline__ bool aligned16(const T* p) {
  return (reinterpret_cast<uintptr_t>(p) & 15) == 0;
}

// "Tiled rows": M rows of K columns (K a multiple of 32) in the order a matrix-core product takes them as its
// second operand: the 16 rows x 32 columns tile of (k step, row tile) lies as 64 lanes x 16 bytes, lane l holding
// row l % 16, columns 8 (l / 16) .. + 7; the row tiles of a k step follow each other, then the next k step.
// `tiles` = ceil(M / 16); the buffer holds (K / 32) * tiles * 512 elements.
__host__ __device__ __forceinline__ size_t tiled_index(int m, int k, int tiles) {
  return ((((size_t)(k >> 5) * tiles + (m >> 4)) * 64) + ((k & 31) >> 3) * 16 + (m & 15)) * 8 + (k & 7);
}

static inline int gs_ceil_div(long a, long b) { return (int)((a + b - 1) / b); }

// A float as bfloat16 on the host: round to nearest, ties to even; NaN stays NaN.
static inline bf16 host_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  bf16 r;
  if ((u & 0x7fffffffu) > 0x7f800000u) {
    r.x = (uint16_t)((u >> 16) | 0x40);
  } else {
    r.x = (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
  }
  return r;
}
