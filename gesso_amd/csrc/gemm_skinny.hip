// Y (M, N) = X (M, K) . W (N, K)^T for few rows (M <= 64): the weight-streaming product of decoding.
//
// Every weight is read once from HBM; the time of this kernel is the time of that stream.  bfloat16
// inputs, float32 accumulation on the matrix cores (v_mfma_f32_16x16x32_bf16), bfloat16 or float32
// output.  One MFMA takes a 16 x 32 tile of W as its A operand, straight from global memory in the
// operand's own layout (lane l: row l % 16, eight consecutive k at 8 * (l / 16): one 16-byte load), and
// a 32 x 16 tile of X^T as its B operand (lane l: token l % 16, the same eight k).  The result tile
// holds, per lane, four consecutive output columns n for one token.
//
// A block of WAVES wavefronts owns 16 * R rows of W; its wavefronts split K among themselves and add
// their partial tiles through LDS.  R row tiles share each X fragment.  Rows beyond N, tokens beyond M
// and k beyond K are masked (K must be a multiple of 8 so that every 16-byte load is aligned).
//
// Epilogues: plain store; or SwiGLU, where W holds gate rows [0, N/2) and up rows [N/2, N) and the
// block computes both for the same columns and stores silu(gate) * up, N/2 wide.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

__device__ __forceinline__ bf16x8_t load8(const bf16* p) { return *reinterpret_cast<const bf16x8_t*>(p); }

__device__ __forceinline__ bf16x8_t zero8() {
  bf16x8_t z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
  return z;
}

template <typename T>
__device__ __forceinline__ void store4(T* p, f32x4_t v, int valid);
template <>
__device__ __forceinline__ void store4<float>(float* p, f32x4_t v, int valid) {
  if (valid >= 4 && ((uintptr_t)p & 15) == 0) {
    *reinterpret_cast<f32x4_t*>(p) = v;
  } else {
    for (int i = 0; i < valid && i < 4; ++i) p[i] = v[i];
  }
}
template <>
__device__ __forceinline__ void store4<bf16>(bf16* p, f32x4_t v, int valid) {
  if (valid >= 4 && ((uintptr_t)p & 7) == 0) {
    uint2 o;
    o.x = (uint32_t)f32_to_bf16(v[0]).x | ((uint32_t)f32_to_bf16(v[1]).x << 16);
    o.y = (uint32_t)f32_to_bf16(v[2]).x | ((uint32_t)f32_to_bf16(v[3]).x << 16);
    *reinterpret_cast<uint2*>(p) = o;
  } else {
    for (int i = 0; i < valid && i < 4; ++i) p[i] = f32_to_bf16(v[i]);
  }
}

// EPI: 0 plain, 1 SwiGLU (row tile r even: gate rows, odd: the matching up rows; R must be even)
template <int R, int MT, int WAVES, int EPI, typename TOut>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const bf16* __restrict__ X, int ldx,
                                                                  const bf16* __restrict__ W,
                                                                  TOut* __restrict__ Y, int ldy, int M, int N,
                                                                  int K) {
  extern __shared__ float red[];  // (WAVES - 1) x R x MT x 64 x 4 floats
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r16 = lane & 15, kg = lane >> 4;
  const int half = N >> 1;
  // rows of W this block owns
  int rowbase[R];
  if (EPI == 1) {
    const int n0 = blockIdx.x * 16 * (R / 2);
#pragma unroll
    for (int r = 0; r < R; ++r) rowbase[r] = n0 + (r >> 1) * 16 + ((r & 1) ? half : 0);
  } else {
    const int n0 = blockIdx.x * 16 * R;
#pragma unroll
    for (int r = 0; r < R; ++r) rowbase[r] = n0 + r * 16;
  }
  const int rowlimit = N;
  const bf16* wrow[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    int n = rowbase[r] + r16;
    if (EPI == 1 && !(r & 1) && n >= half) n = half - 1;  // gate rows end at N/2
    if (n >= rowlimit) n = rowlimit - 1;                  // clamped: loaded, never stored
    wrow[r] = W + (size_t)n * K;
  }
  const bf16* xrow[MT];
  bool xok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int m = mt * 16 + r16;
    xok[mt] = m < M;
    xrow[mt] = X + (size_t)(xok[mt] ? m : 0) * ldx;
  }

  f32x4_t acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[r][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // this wavefront's share of K, in steps of 32
  const int ksteps = (K + 31) >> 5;
  const int per = (ksteps + WAVES - 1) / WAVES;
  const int s0 = wave * per, s1 = (s0 + per < ksteps) ? s0 + per : ksteps;
  int s = s0;
  // four steps at a time, all their loads issued before the first product, so that many loads are in flight
  if ((K & 31) == 0) {
    for (; s + 4 <= s1; s += 4) {
      bf16x8_t a[4][R], b[4][MT];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int k = ((s + u) << 5) + kg * 8;
#pragma unroll
        for (int r = 0; r < R; ++r) a[u][r] = load8(wrow[r] + k);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) b[u][mt] = xok[mt] ? load8(xrow[mt] + k) : zero8();
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[r][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][r], b[u][mt], acc[r][mt], 0, 0, 0);
    }
  }
  for (; s < s1; ++s) {
    const int k = (s << 5) + kg * 8;
    const bool kin = k < K;
    bf16x8_t b[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) b[mt] = (kin && xok[mt]) ? load8(xrow[mt] + k) : zero8();
#pragma unroll
    for (int r = 0; r < R; ++r) {
      bf16x8_t a = kin ? load8(wrow[r] + k) : zero8();
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[r][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[mt], acc[r][mt], 0, 0, 0);
    }
  }

  // add the wavefronts' partial tiles: wave 0 keeps its own, the others pass theirs through LDS
  if (WAVES > 1) {
    if (wave > 0) {
      float* dst = red + ((size_t)(wave - 1) * R * MT) * 256;
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          *reinterpret_cast<f32x4_t*>(dst + ((r * MT + mt) * 64 + lane) * 4) = acc[r][mt];
    }
    __syncthreads();
    if (wave > 0) return;
    for (int w = 0; w < WAVES - 1; ++w) {
      const float* src = red + ((size_t)w * R * MT) * 256;
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          f32x4_t v = *reinterpret_cast<const f32x4_t*>(src + ((r * MT + mt) * 64 + lane) * 4);
          acc[r][mt] += v;
        }
    }
  }

  // lane l holds, for token mt*16 + l%16, columns rowbase + 4*(l/16) + 0..3
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + r16;
    if (m >= M) continue;
    if (EPI == 1) {
#pragma unroll
      for (int r = 0; r < R; r += 2) {
        const int n = rowbase[r] + kg * 4;  // output column in [0, N/2)
        f32x4_t g = acc[r][mt], u = acc[r + 1][mt], o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = g[i] / (1.0f + expf(-g[i])) * u[i];
        int valid = half - n;
        if (valid > 0) store4<TOut>(Y + (size_t)m * ldy + n, o, valid);
      }
    } else {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int n = rowbase[r] + kg * 4;
        int valid = N - n;
        if (valid > 0) store4<TOut>(Y + (size_t)m * ldy + n, acc[r][mt], valid);
      }
    }
  }
}

template <int R, int MT, int WAVES, int EPI, typename TOut>
static void launch_skinny(const bf16* X, int ldx, const bf16* W, TOut* Y, int ldy, int M, int N, int K,
                          hipStream_t stream) {
  const int rows_per_block = EPI == 1 ? 16 * (R / 2) : 16 * R;
  const int out_cols = EPI == 1 ? N / 2 : N;
  const int blocks = gs_ceil_div(out_cols, rows_per_block);
  const size_t lds = (size_t)(WAVES - 1) * R * MT * 256 * sizeof(float);
  gemm_skinny_kernel<R, MT, WAVES, EPI, TOut><<<blocks, WAVES * 64, lds, stream>>>(X, ldx, W, Y, ldy, M, N, K);
}

template <int EPI, typename TOut>
static int dispatch_skinny(const bf16* X, int ldx, const bf16* W, TOut* Y, int ldy, int M, int N, int K,
                           hipStream_t stream) {
  const int mt = (M + 15) / 16;
  const int out_cols = EPI == 1 ? N / 2 : N;
  // few output columns: more wavefronts per block split K further, so that the whole chip streams
  const bool narrow = out_cols <= 4096;
#define GS_GO(R, MT, WAVES) launch_skinny<R, MT, WAVES, EPI, TOut>(X, ldx, W, Y, ldy, M, N, K, stream)
  if (EPI == 1) {
    switch (mt) {
      case 1: narrow ? GS_GO(2, 1, 8) : GS_GO(2, 1, 4); break;
      case 2: narrow ? GS_GO(2, 2, 8) : GS_GO(2, 2, 4); break;
      case 3: narrow ? GS_GO(2, 3, 8) : GS_GO(2, 3, 4); break;
      default: narrow ? GS_GO(2, 4, 8) : GS_GO(2, 4, 4); break;
    }
  } else {
    switch (mt) {
      case 1: narrow ? GS_GO(1, 1, 16) : GS_GO(2, 1, 4); break;
      case 2: narrow ? GS_GO(1, 2, 16) : GS_GO(2, 2, 4); break;
      case 3: narrow ? GS_GO(1, 3, 8) : GS_GO(2, 3, 4); break;
      default: narrow ? GS_GO(1, 4, 8) : GS_GO(2, 4, 4); break;
    }
  }
#undef GS_GO
  return 0;
}

extern "C" int gs_gemm_skinny(const void* X, int ldx, const void* W, void* Y, int y_dtype, int ldy, int M, int N,
                              int K, int epilogue, hipStream_t stream) {
  GS_REQUIRE(M >= 0 && M <= 64, "gemm_skinny: %d rows; this kernel takes at most 64", M);
  GS_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "gemm_skinny: K=%d must be a positive multiple of 8 (N=%d)", K, N);
  GS_REQUIRE(ldx >= K && ldx % 8 == 0, "gemm_skinny: row stride %d of X must be a multiple of 8 and at least K", ldx);
  GS_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0, "gemm_skinny: operands must be 16-byte aligned");
  GS_REQUIRE(epilogue == 0 || (epilogue == 1 && N % 2 == 0), "gemm_skinny: unknown epilogue %d (or odd N)", epilogue);
  GS_REQUIRE(ldy >= (epilogue == 1 ? N / 2 : N), "gemm_skinny: row stride %d of Y too small", ldy);
  if (M == 0) return 0;
  const bf16* x = (const bf16*)X;
  const bf16* w = (const bf16*)W;
  if (y_dtype == GS_BF16) {
    if (epilogue == 1)
      dispatch_skinny<1, bf16>(x, ldx, w, (bf16*)Y, ldy, M, N, K, stream);
    else
      dispatch_skinny<0, bf16>(x, ldx, w, (bf16*)Y, ldy, M, N, K, stream);
  } else if (y_dtype == GS_F32) {
    if (epilogue == 1)
      dispatch_skinny<1, float>(x, ldx, w, (float*)Y, ldy, M, N, K, stream);
    else
      dispatch_skinny<0, float>(x, ldx, w, (float*)Y, ldy, M, N, K, stream);
  } else {
    GS_REQUIRE(false, "gemm_skinny: unknown output dtype %d", y_dtype);
  }
  GS_LAUNCH_CHECK("gemm_skinny");
  return 0;
}
