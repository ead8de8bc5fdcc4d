// Y (M, N) = X (M, K) . W (N, K)^T for many rows (prompts), on the matrix cores, with an optional SwiGLU epilogue.
//
// bfloat16 inputs, float32 accumulation (v_mfma_f32_32x32x16_bf16), bfloat16 or float32 output.  X and W both have K
// as their fast axis, which is the order the MFMA wants its operands in: lane l of a wavefront gives row l % 32,
// eight consecutive k at 8 (l / 32).  A block of WM x WN wavefronts computes a BM x BN tile of Y; per step of 64 in
// K it brings the BM rows of X and the BN rows of W into LDS (16-byte loads into registers, issued before the
// products of the tile at hand, written to the other of two LDS buffers after them), and every wavefront reads its
// (BM / WM) + (BN / WN) rows from there.  LDS rows are 64 + 8 elements long: the 144-byte stride sends the sixteen
// rows that a 16-byte read touches at a time to different banks.
//
// The result tile of one MFMA holds, per lane, one column n = l % 32 and sixteen rows m = 8 (e / 4) + 4 (l / 32) + e % 4.
//
// Tails: rows beyond M and N are loaded from the last valid row and never stored; K need only be a multiple of 8,
// the chunks of a last step beyond K are zero.
//
// EPI 1 (SwiGLU): W holds gate rows [0, N/2) then up rows; a block owns BN / 2 output columns and loads their gate and
// up rows, laid out in LDS so that every wavefront finds its columns' gate tiles in the first half of its rows and
// their up tiles in the second; it stores silu(gate) * up, N / 2 wide.  The gate | up product never goes to memory.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 gm_bf16x8_t;
typedef __attribute__((ext_vector_type(16))) float gm_f32x16_t;

constexpr int GM_BK = 64;            // k per step
constexpr int GM_LDR = GM_BK + 8;    // elements per LDS row

template <int BM, int BN, int WM, int WN, int EPI, typename TOut>
__global__ __launch_bounds__(WM * WN * 64) void gemm_mfma_kernel(const bf16* __restrict__ X, int ldx,
                                                                const bf16* __restrict__ W, TOut* __restrict__ Y,
                                                                int ldy, int M, int N, int K) {
  constexpr int NT = WM * WN * 64;
  constexpr int RM = BM / WM, RN = BN / WN;                // rows of X and of W per wavefront
  constexpr int TM = RM / 32, TN = RN / 32;                // 32 x 32 tiles per wavefront
  constexpr int LA = BM * 8 / NT, LB = BN * 8 / NT;        // 16-byte loads per thread and step
  constexpr int STAGE = (BM + BN) * GM_LDR;                // elements per LDS buffer: X rows, then W rows
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0 && (BM * 8) % NT == 0 && (BN * 8) % NT == 0, "tile shape");
  static_assert(EPI == 0 || TN % 2 == 0, "SwiGLU pairs a wavefront's gate tiles with its up tiles");
  extern __shared__ __align__(16) uint16_t gm_lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int l32 = lane & 31, kh = lane >> 5;
  const int F = N >> 1;                                    // EPI 1: output width
  // Blocks are handed to the eight XCDs in turn (block b runs on XCD b % 8), each with an L2 of its own.  A run of
  // consecutive tile numbers goes to one XCD, and tile numbers walk the output in bands of four row tiles, column by
  // column: the tiles in an XCD's L2 at one time then share few rows of X and few rows of W.
  const int tiles_m = (M + BM - 1) / BM;
  int bm, bn;
  {
    const int nb = (int)gridDim.x, per = nb / 8, rem = nb % 8;
    const int xcd = (int)blockIdx.x % 8, turn = (int)blockIdx.x / 8;
    const int t = xcd * per + (xcd < rem ? xcd : rem) + turn;        // XCD x owns per (+ 1) consecutive numbers
    const int tiles_n = nb / tiles_m;
    constexpr int BAND = 4;
    const int band = t / (BAND * tiles_n), in_band = t - band * BAND * tiles_n;
    const int rows = tiles_m - band * BAND < BAND ? tiles_m - band * BAND : BAND;   // the last band may be narrower
    bm = band * BAND + in_band % rows;
    bn = in_band / rows;
  }
  const int m0 = bm * BM;
  const int n0 = EPI == 1 ? bn * (BN / 2) : bn * BN;       // first output column of the block

  // this thread's loads: LDS row r0 + i * (NT / 8), chunk c of eight k
  const int r0 = tid >> 3, c = tid & 7;
  const bf16* ap[LA];
  const bf16* bp[LB];
#pragma unroll
  for (int i = 0; i < LA; ++i) {
    int m = m0 + r0 + i * (NT / 8);
    if (m >= M) m = M - 1;
    ap[i] = X + (size_t)m * ldx + c * 8;
  }
#pragma unroll
  for (int i = 0; i < LB; ++i) {
    const int rr = r0 + i * (NT / 8);
    int n;
    if (EPI == 1) {
      // LDS row rr belongs to wavefront column rr / RN; the first half of its rows are gate rows, the second up rows
      const int within = rr % RN, col = (rr / RN) * (RN / 2) + within % (RN / 2);
      int o = n0 + col;
      if (o >= F) o = F - 1;
      n = within < RN / 2 ? o : F + o;
    } else {
      n = n0 + rr;
      if (n >= N) n = N - 1;
    }
    bp[i] = W + (size_t)n * K + c * 8;
  }
  uint4 sa[LA], sb[LB];
#define GM_GLOAD(k0)                                                                                         \
  {                                                                                                          \
    _Pragma("unroll") for (int i = 0; i < LA; ++i) sa[i] = *reinterpret_cast<const uint4*>(ap[i] + (k0));      \
    _Pragma("unroll") for (int i = 0; i < LB; ++i) sb[i] = *reinterpret_cast<const uint4*>(bp[i] + (k0));      \
  }
#define GM_GLOAD_MASKED(k0)                                                                                  \
  {                                                                                                          \
    const bool in = (k0) + c * 8 < K;                      /* chunks beyond K: loaded from the row's start, zeroed */ \
    const int kk = in ? (k0) : -c * 8;                                                                       \
    _Pragma("unroll") for (int i = 0; i < LA; ++i) {                                                         \
      sa[i] = *reinterpret_cast<const uint4*>(ap[i] + kk);                                                   \
      sa[i] = in ? sa[i] : make_uint4(0, 0, 0, 0);                                                           \
    }                                                                                                        \
    _Pragma("unroll") for (int i = 0; i < LB; ++i) {                                                         \
      sb[i] = *reinterpret_cast<const uint4*>(bp[i] + kk);                                                   \
      sb[i] = in ? sb[i] : make_uint4(0, 0, 0, 0);                                                           \
    }                                                                                                        \
  }
#define GM_LSTORE(buf)                                                                                       \
  {                                                                                                          \
    _Pragma("unroll") for (int i = 0; i < LA; ++i)                                                           \
        *reinterpret_cast<uint4*>(gm_lds + (buf) * STAGE + (r0 + i * (NT / 8)) * GM_LDR + c * 8) = sa[i];      \
    _Pragma("unroll") for (int i = 0; i < LB; ++i)                                                           \
        *reinterpret_cast<uint4*>(gm_lds + (buf) * STAGE + (BM + r0 + i * (NT / 8)) * GM_LDR + c * 8) = sb[i]; \
  }
#define GM_COMPUTE(buf)                                                                                      \
  {                                                                                                          \
    const uint16_t* a_base = gm_lds + (buf) * STAGE + (wm * RM + l32) * GM_LDR + kh * 8;                     \
    const uint16_t* b_base = gm_lds + (buf) * STAGE + (BM + wn * RN + l32) * GM_LDR + kh * 8;                \
    _Pragma("unroll") for (int ks = 0; ks < GM_BK / 16; ++ks) {                                              \
      gm_bf16x8_t af[TM], bf[TN];                                                                            \
      _Pragma("unroll") for (int i = 0; i < TM; ++i)                                                         \
          af[i] = *reinterpret_cast<const gm_bf16x8_t*>(a_base + i * 32 * GM_LDR + ks * 16);                 \
      _Pragma("unroll") for (int j = 0; j < TN; ++j)                                                         \
          bf[j] = *reinterpret_cast<const gm_bf16x8_t*>(b_base + j * 32 * GM_LDR + ks * 16);                 \
      _Pragma("unroll") for (int i = 0; i < TM; ++i)                                                         \
        _Pragma("unroll") for (int j = 0; j < TN; ++j)                                                       \
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);             \
    }                                                                                                        \
  }

  gm_f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int nfull = K / GM_BK;                 // whole steps
  const bool tail = (K % GM_BK) != 0;          // and one more whose last chunks are zero
  const int nk = nfull + (tail ? 1 : 0);
  // the first step (masked: K may be below 64)
  GM_GLOAD_MASKED(0);
  GM_LSTORE(0);
  __syncthreads();
  int it = 0;
  for (; it + 1 < nfull; ++it) {
    const int buf = it & 1;
    GM_GLOAD((it + 1) * GM_BK);
    GM_COMPUTE(buf);
    GM_LSTORE(buf ^ 1);
    __syncthreads();
  }
  if (tail && nfull > 0) {
    // step nfull - 1 is in LDS; the last, partial step is loaded with its chunks beyond K zeroed
    const int buf = it & 1;
    GM_GLOAD_MASKED(nfull * GM_BK);
    GM_COMPUTE(buf);
    GM_LSTORE(buf ^ 1);
    __syncthreads();
  }
  GM_COMPUTE((nk - 1) & 1);
#undef GM_GLOAD
#undef GM_GLOAD_MASKED
#undef GM_LSTORE
#undef GM_COMPUTE

#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < (EPI == 1 ? TN / 2 : TN); ++j) {
      const int n = EPI == 1 ? n0 + wn * (RN / 2) + j * 32 + l32 : n0 + wn * RN + j * 32 + l32;
      if (n >= (EPI == 1 ? F : N)) continue;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int m = m0 + wm * RM + i * 32 + 8 * (e >> 2) + 4 * kh + (e & 3);
        if (m >= M) continue;
        float v = acc[i][j][e];
        if (EPI == 1) {
          // on the values as the unfused path stores them: rounded to bfloat16
          const float g = to_f32(f32_to_bf16(v)), u = to_f32(f32_to_bf16(acc[i][j + (EPI == 1 ? TN / 2 : 0)][e]));
          // (the hardware's exponential and reciprocal: a block has 32,768 of these to do, and the library's expf and
          // a float division, some eighty instructions an element, took a fifth of the kernel's time)
          v = g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g)) * u;
        }
        Y[(size_t)m * ldy + n] = from_f32<TOut>(v);
      }
    }
}

template <int BM, int BN, int WM, int WN, int EPI, typename TOut>
static void launch_mfma(const bf16* X, int ldx, const bf16* W, TOut* Y, int ldy, int M, int N, int K,
                        hipStream_t stream) {
  const int cols = EPI == 1 ? BN / 2 : BN;
  const int width = EPI == 1 ? N / 2 : N;
  const long tiles = (long)gs_ceil_div(M, BM) * gs_ceil_div(width, cols);
  const size_t lds = (size_t)2 * (BM + BN) * GM_LDR * sizeof(uint16_t);
  // more than the default limit of dynamic LDS: asked for once per kernel
  static const hipError_t asked = hipFuncSetAttribute(
      reinterpret_cast<const void*>(&gemm_mfma_kernel<BM, BN, WM, WN, EPI, TOut>),
      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  (void)asked;
  gemm_mfma_kernel<BM, BN, WM, WN, EPI, TOut><<<(unsigned)tiles, WM * WN * 64, lds, stream>>>(X, ldx, W, Y, ldy, M, N, K);
}

// epilogue 0: Y (M, N) = X W^T, bfloat16 or float32.  epilogue 1: Y (M, N / 2) = silu(X Wg^T) * (X Wu^T), bfloat16.
extern "C" int gs_gemm_mfma(const void* X, int ldx, const void* W, void* Y, int y_dtype, int ldy, int M, int N, int K,
                            int epilogue, hipStream_t stream) {
  GS_REQUIRE(M >= 0 && N > 0 && K > 0 && K % 8 == 0, "gemm_mfma: bad sizes M=%d N=%d K=%d (K must be a multiple of 8)", M, N, K);
  GS_REQUIRE(epilogue == 0 || (epilogue == 1 && N % 2 == 0 && y_dtype == GS_BF16), "gemm_mfma: unknown epilogue %d (SwiGLU needs an even N and a bfloat16 output)", epilogue);
  GS_REQUIRE(y_dtype == GS_BF16 || y_dtype == GS_F32, "gemm_mfma: unknown output dtype %d", y_dtype);
  GS_REQUIRE(ldx >= K && ldx % 8 == 0 && ((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0,
             "gemm_mfma: X and W must be 16-byte aligned, the row stride of X a multiple of 8");
  GS_REQUIRE(ldy >= (epilogue == 1 ? N / 2 : N), "gemm_mfma: row stride %d of Y too small", ldy);
  GS_REQUIRE((long)gs_ceil_div(M, 128) * gs_ceil_div(N, 64) < (1L << 31), "gemm_mfma: too many tiles");
  if (M == 0) return 0;
  const bf16 *x = (const bf16*)X, *w = (const bf16*)W;
  // tiles of 256 x 256 where they fill the chip (fewer bytes through LDS per product), else 128 x 128
  const int width = epilogue == 1 ? N / 2 : N;
  const long big = (long)gs_ceil_div(M, 256) * gs_ceil_div(width, epilogue == 1 ? 128 : 256);
  const bool use_big = M > 128 && big >= 150;
  if (epilogue == 1) {
    if (use_big) launch_mfma<256, 256, 4, 2, 1, bf16>(x, ldx, w, (bf16*)Y, ldy, M, N, K, stream);
    else launch_mfma<128, 256, 2, 2, 1, bf16>(x, ldx, w, (bf16*)Y, ldy, M, N, K, stream);
  } else if (y_dtype == GS_BF16) {
    if (use_big) launch_mfma<256, 256, 2, 4, 0, bf16>(x, ldx, w, (bf16*)Y, ldy, M, N, K, stream);
    else launch_mfma<128, 128, 2, 2, 0, bf16>(x, ldx, w, (bf16*)Y, ldy, M, N, K, stream);
  } else {
    if (use_big) launch_mfma<256, 256, 2, 4, 0, float>(x, ldx, w, (float*)Y, ldy, M, N, K, stream);
    else launch_mfma<128, 128, 2, 2, 0, float>(x, ldx, w, (float*)Y, ldy, M, N, K, stream);
  }
  GS_LAUNCH_CHECK("gemm_mfma");
  return 0;
}
