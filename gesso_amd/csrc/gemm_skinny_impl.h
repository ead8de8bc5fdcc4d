// Y (M, N) = X (M, K) . W (N, K)^T for few rows (M <= 64): the weight-streaming product of decoding,
// with what stands before and after it in a block folded in.
//
// Every weight is read once from HBM; the time of this kernel is the time of that stream.  bfloat16
// inputs, float32 accumulation on the matrix cores (v_mfma_f32_16x16x32_bf16).  One MFMA takes a 16 x 32
// tile of W as its A operand, straight from global memory in the operand's own layout (lane l: row
// l % 16, eight consecutive k at 8 * (l / 16): one 16-byte load), and a 32 x 16 tile of X^T as its B
// operand (lane l: token l % 16, the same eight k).  The result tile holds, per lane, four consecutive
// output columns n for one token.
//
// A block of WAVES wavefronts owns R tiles of 16 rows of W; its wavefronts split K among themselves and
// add their partial tiles through LDS in wavefront order.  Rows beyond N, tokens beyond M and k beyond K
// are masked (K must be a multiple of 8 so that every 16-byte load is aligned).
//
// The weight is read either as it is stored, rows of K (SHUF = 0), or from a tile-major copy
// (SHUF = 1) in which the 16 x 32 tile of (row tile, k step) lies as 64 lanes x 16 bytes in the
// operand's own order, tiles of a row tile one after the other: then every load of a wavefront is one
// contiguous kilobyte and a wavefront streams a contiguous range, which HBM serves faster than
// sixteen rows 2 K bytes apart.
//
// X is read either as rows of ldx elements or, with x_tiled, in the order the MFMA takes it ("tiled rows",
// tiled_index in common.h: the 16 x 32 tile of (k step, row tile) as 64 lanes x 16 bytes): then every load of X is one
// contiguous kilobyte instead of sixteen pieces of rows, which is what the products of many rows are bound by.  With
// y_tiled the epilogues that write rows for a following product (SwiGLU, convolution, pre-weighted rows) write them
// in that order.
//
// What feeds X (PRO):
//   0  X is given, bfloat16.
//   1  X is the RMSNorm of the float32 residual stream: x = res * inv_rms(row) * norm_weight, rounded to
//      bfloat16 as the norm kernel would store it; the row's sum of squares comes as partial sums
//      (row, nb), added in a fixed order.
//   0 with partial sums given: X holds rows already multiplied by the norm's weight (res * norm_weight,
//      written by the product that last added to the stream, EPI 2); the row's inverse root mean square,
//      which no single block of that product knew, multiplies this product's result instead:
//      (x inv) W^T = inv (x W^T).  The norm costs no kernel and no pass of its own.
// What is done with Y (EPI):
//   0  stored (bfloat16 or float32).
//   1  SwiGLU: W holds gate rows [0, N/2) then up rows; stores silu(gate) * up, N/2 wide.
//   5  partial sums: K is shared out over gridDim.x blocks as well (the weight tiles over gridDim.y), each writes its float32 (M, N) sheet; a second
//      kernel adds the sheets.  For many rows: every block reads all rows of X for its part of K, so the fewer
//      weight rows and the more of K a block takes, the more X traffic; sharing K over blocks caps it.
//   2  added to the residual stream in place (float32), and the sums of squares of the new rows over this
//      block's columns stored as partial sums for the next norm.
//   3  gated short convolution of a decode step: tiles are the B, C, X rows of 16 channels; u = B X,
//      y = taps . (history, u) + bias, out = C y, history shifted; one token per sequence.
#pragma once
#include "common.h"
#include <type_traits>

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

// Everything the prologues and epilogues need beside X, W, Y; unused fields stay null.
struct SkinnyExtra {
  // PRO 1
  const float* res;      // (M, K) float32 residual stream
  const float* ssq;      // (M, nb) partial sums of squares of res rows
  int nb;
  const float* norm_w;   // (K)
  float eps;
  // EPI 2
  float* res_out;        // (M, N) float32, updated in place
  float* ssq_out;        // (M, gridDim.x)
  const float* next_w;   // (N) weight of the norm that reads the stream next, or null
  bf16* xs_out;          // (M, N) res * next_w, for that norm's consumer
  // EPI 3
  const float* taps;     // (H, W)
  const float* conv_bias;
  float* state;          // (slots, H, W - 1)
  const int* slots;      // (M)
  int conv_w;
  int conv_vec;          // widths 2..4, H a multiple of 4, taps, bias and state 16-byte aligned: the epilogue keeps taps
                         // and history in registers and moves them sixteen bytes at a time
  // layouts
  int x_tiled;           // X comes as tiled rows (PRO 0 only; K a multiple of 32)
  int y_tiled;           // EPI 1, 3: Y, EPI 2: xs_out are written as tiled rows (their width a multiple of 32)
};

template <int R, int MT, int WAVES, int PRO, int EPI, int SHUF, typename TOut>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const bf16* __restrict__ X, int ldx,
                                                                  const bf16* __restrict__ W,
                                                                  TOut* __restrict__ Y, int ldy, int M, int N,
                                                                  int K, SkinnyExtra ex) {
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
  } else if (EPI == 3) {
    const int H = N / 3;
#pragma unroll
    for (int r = 0; r < R; ++r) rowbase[r] = blockIdx.x * (SHUF == 2 ? 8 : 16) + r * H;  // B, C, X rows of the same channels
  } else if (SHUF == 2) {
    rowbase[0] = blockIdx.x * 8;  // half a tile: twice the blocks for a weight of few rows
  } else {
    // (EPI 5: the grid is (parts of K, weight tiles), see below)
    const int n0 = (EPI == 5 ? blockIdx.y : blockIdx.x) * 16 * R;
#pragma unroll
    for (int r = 0; r < R; ++r) rowbase[r] = n0 + r * 16;
  }
  static_assert(SHUF != 2 || (R == 1 && EPI == 2) || EPI == 3, "half tiles are written for the residual and the convolution epilogues");
  const bool wact = SHUF != 2 || r16 < 8;  // half tiles: the lanes of the other eight rows load nothing
  const bf16* wrow[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    int n = rowbase[r] + r16;
    if (EPI == 1 && !(r & 1) && n >= half) n = half - 1;  // gate rows end at N/2
    if (EPI == 3 && n >= (r + 1) * (N / 3)) n = (r + 1) * (N / 3) - 1;
    if (n >= N) n = N - 1;                                // clamped: loaded, never stored
    if (SHUF == 2)
      wrow[r] = W + ((size_t)(rowbase[r] >> 4) * ((K + 31) >> 5)) * 512 + (kg * 16 + (rowbase[r] & 8) + (r16 & 7)) * 8;
    else if (SHUF) {
      // tile-major: the 16 x 32 tile of (row tile, k step) is 64 lanes x 16 bytes in the operand's own order
      // (a tile past the weight's last, where a block's tiles outnumber what is left, reads the last: loaded, never stored)
      const int tile = (rowbase[r] >> 4) < ((N + 15) >> 4) ? (rowbase[r] >> 4) : ((N + 15) >> 4) - 1;
      wrow[r] = W + ((size_t)tile * ((K + 31) >> 5)) * 512 + lane * 8;
    }
    else
      wrow[r] = W + (size_t)n * K + kg * 8;
  }
  bool xok[MT];
  const bf16* xrow[MT];
  const float* rrow[MT];
  float inv[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int m = mt * 16 + r16;
    xok[mt] = m < M;
    xrow[mt] = nullptr;
    rrow[mt] = nullptr;
    inv[mt] = 0.f;
    if (PRO == 0) {
      xrow[mt] = ex.x_tiled ? X + (size_t)(mt * 64 + lane) * 8 : X + (size_t)(xok[mt] ? m : 0) * ldx + kg * 8;
    } else {
      rrow[mt] = ex.res + (size_t)(xok[mt] ? m : 0) * K;
    }
    if (PRO == 1) {
      // the row's sum of squares: this lane group adds every fourth partial, then the four groups are added
      float s = 0.f;
      if (xok[mt])
        for (int b = kg; b < ex.nb; b += 4) s += ex.ssq[(size_t)m * ex.nb + b];
      s += __shfl_xor(s, 16, 64);
      s += __shfl_xor(s, 32, 64);
      inv[mt] = norm_inverse(s, (float)K, ex.eps);
    }
  }

  // Pre-weighted rows: the rows' inverse root mean squares are needed only at the end.  The wavefronts share
  // the rows; a lane adds every 64th partial sum and the wavefront adds its lanes (an order that depends on
  // nothing but the number of partials).  The first row's loads start here, under the product's own.
  __shared__ float inv_s[64];
  const bool scaled = PRO == 0 && ex.ssq != nullptr;
  float pre[4] = {0.f, 0.f, 0.f, 0.f};
  if (scaled && wave < M) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (lane + 64 * j < ex.nb) pre[j] = ex.ssq[(size_t)wave * ex.nb + lane + 64 * j];
  }

  // The convolution's slots, by scalar loads (the row number is the same for every lane), each lane then picking its
  // row's: the history's addresses wait for them, and scalar loads return on a counter of their own.
  int cslot[EPI == 3 ? MT : 1];
  if (EPI == 3) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      int mine = 0;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int row = mt * 16 + i;
        const int sv = ex.slots[row < M ? row : 0];
        mine = r16 == i ? sv : mine;
      }
      cslot[mt] = mine;
    }
  }

  // What the epilogue reads besides the product (the stream's old rows, the convolution's history and taps) is
  // loaded early, by the wavefront that runs the epilogue, so that these round trips pass under the product's own
  // instead of after it.  The stream's old rows are asked for here, before the weights.  The convolution's operands
  // are asked for right after the first weight loads (few row tiles), by loads that sit behind no branch and whose
  // values nothing touches before the epilogue: wherever a branch hides how many loads are in flight the compiler
  // waits for all of them, and with a test on each tap and each history value that was a round trip apiece before
  // the first weight was asked for (measured on cold weights of 6144 x 2048, 8 rows: 10.6 against 9.6 us a kernel).
  constexpr int PRE_TAPS = 4;                       // convolutions of up to this width are held in registers
  const bool half_ok = SHUF != 2 || kg < 2;
  f32x4_t rold[EPI == 2 ? R : 1][EPI == 2 ? MT : 1], nextw[EPI == 2 ? R : 1];
  float chist[EPI == 3 ? MT : 1][4][PRE_TAPS - 1], ctap[4][PRE_TAPS], cbias[4];
  const bool vec4 = (N & 3) == 0;
  if (EPI == 2 && wave == 0) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = rowbase[r] + kg * 4;
      const bool ok = n < N && half_ok;
      nextw[r] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      if (ok && ex.next_w) {
        if (vec4) nextw[r] = *reinterpret_cast<const f32x4_t*>(ex.next_w + n);
        else
          for (int i = 0; i < 4; ++i)
            if (n + i < N) nextw[r][i] = ex.next_w[n + i];
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        rold[r][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        if (ok && xok[mt]) {
          const float* p = ex.res_out + (size_t)(mt * 16 + r16) * N + n;
          if (vec4) rold[r][mt] = *reinterpret_cast<const f32x4_t*>(p);
          else
            for (int i = 0; i < 4; ++i)
              if (n + i < N) rold[r][mt][i] = p[i];
        }
      }
    }
  }
  const bool pre_conv = EPI == 3 && ex.conv_vec != 0;
  // A lane's four channels are neighbours, so their taps (4 x width floats), their bias and, per row, their history
  // (4 x (width - 1) floats) are each one run of memory: moved sixteen bytes at a time, the width a compile-time
  // number in each of the three forms.  A block's channels past H read the last four (loaded, never used), a row
  // past M its row 0's slot.
  // (macros, not closures: arrays that a closure takes by reference are not always kept in registers, and these
  // were not: taps and history went through scratch memory, a store after each load's arrival and a load before use)
#define GS_CONV_WIDTH(BODY)                                                                                            \
  switch (ex.conv_w) {                                                                                                  \
    case 2: { constexpr int WD = 2; BODY } break;                                                                       \
    case 3: { constexpr int WD = 3; BODY } break;                                                                       \
    default: { constexpr int WD = 4; BODY } break;                                                                      \
  }
#define GS_PRELOAD_CONV_BODY                                                                                           \
  {                                                                                                                     \
    f32x4_t tq[WD];                                                                                                     \
    _Pragma("unroll") for (int q = 0; q < WD; ++q) tq[q] = *reinterpret_cast<const f32x4_t*>(ex.taps + (size_t)cc0_ * WD + 4 * q); \
    _Pragma("unroll") for (int i = 0; i < 4; ++i)                                                                       \
      _Pragma("unroll") for (int p = 0; p < WD; ++p) ctap[i][p] = tq[(i * WD + p) / 4][(i * WD + p) % 4];               \
    _Pragma("unroll") for (int mt = 0; mt < MT; ++mt) {                                                                 \
      f32x4_t hq[WD - 1];                                                                                               \
      const float* hp = ex.state + ((size_t)cslot[mt] * H_ + cc0_) * (WD - 1);                                          \
      _Pragma("unroll") for (int q = 0; q < WD - 1; ++q) hq[q] = *reinterpret_cast<const f32x4_t*>(hp + 4 * q);         \
      _Pragma("unroll") for (int i = 0; i < 4; ++i)                                                                     \
        _Pragma("unroll") for (int p = 0; p < WD - 1; ++p)                                                              \
          chist[mt][i][p] = hq[(i * (WD - 1) + p) / 4][(i * (WD - 1) + p) % 4];                                         \
    }                                                                                                                   \
  }
#define GS_PRELOAD_CONV()                                                                                              \
  if (EPI == 3 && wave == 0 && pre_conv) {                                                                              \
    const int H_ = N / 3;                                                                                               \
    const int c0_ = blockIdx.x * (SHUF == 2 ? 8 : 16) + kg * 4;                                                         \
    const int cc0_ = c0_ + 3 < H_ ? c0_ : H_ - 4;                                                                       \
    const f32x4_t bv_ = *reinterpret_cast<const f32x4_t*>((ex.conv_bias ? ex.conv_bias : ex.taps) + cc0_);              \
    _Pragma("unroll") for (int i = 0; i < 4; ++i) cbias[i] = bv_[i];                                                    \
    GS_CONV_WIDTH(GS_PRELOAD_CONV_BODY)                                                                                 \
  }
#define GS_CONV_EPI_BODY                                                                                                \
        {                                                                                                              \
          f32x4_t out, nh[WD - 1];                                                                                     \
_Pragma("unroll")                                                                                                      \
          for (int i = 0; i < 4; ++i) {                                                                                \
            const float Bv = to_f32(f32_to_bf16(acc[0][mt][i])), Cv = to_f32(f32_to_bf16(acc[R > 1 ? 1 : 0][mt][i])),  \
                        Xv = to_f32(f32_to_bf16(acc[R > 2 ? 2 : 0][mt][i]));                                           \
            const float u = Bv * Xv;                                                                                   \
            float y = 0.f;                                                                                             \
_Pragma("unroll")                                                                                                      \
            for (int p = 0; p < WD - 1; ++p) y += ctap[i][p] * chist[mt][i][p];                                        \
            y += ctap[i][WD - 1] * u;                                                                                  \
            if (ex.conv_bias) y += cbias[i];                                                                           \
            out[i] = Cv * y;                                                                                           \
_Pragma("unroll")                                                                                                      \
            for (int p = 0; p < WD - 1; ++p)                                                                           \
              nh[(i * (WD - 1) + p) / 4][(i * (WD - 1) + p) % 4] = p < WD - 2 ? chist[mt][i][p + 1] : u;               \
          }                                                                                                            \
          store4<TOut>(Y + (ex.y_tiled ? tiled_index(m, c0, MT) : (size_t)m * ldy + c0), out, 4);                      \
          float* hp = ex.state + ((size_t)slot * H + c0) * (WD - 1);                                                   \
_Pragma("unroll")                                                                                                      \
          for (int q = 0; q < WD - 1; ++q) *reinterpret_cast<f32x4_t*>(hp + 4 * q) = nh[q];                            \
        }
  if (EPI == 3 && MT >= 3) GS_PRELOAD_CONV()   // the loop of many row tiles keeps its order
  f32x4_t acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[r][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  const int xstep = ex.x_tiled ? MT * 512 : 32;   // elements between a row tile's consecutive k steps
  auto load_x = [&](int mt, int s) -> bf16x8_t {
    if (PRO == 0) {
      return load8(xrow[mt] + (size_t)s * xstep);
    } else {
      const int k = (s << 5) + kg * 8;
      const f32x4_t a0 = *reinterpret_cast<const f32x4_t*>(rrow[mt] + k);
      const f32x4_t a1 = *reinterpret_cast<const f32x4_t*>(rrow[mt] + k + 4);
      const f32x4_t w0 = *reinterpret_cast<const f32x4_t*>(ex.norm_w + k);
      const f32x4_t w1 = *reinterpret_cast<const f32x4_t*>(ex.norm_w + k + 4);
      union {
        bf16x8_t v;
        uint16_t u[8];
      } o;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        o.u[i] = f32_to_bf16(a0[i] * inv[mt] * w0[i]).x;
        o.u[4 + i] = f32_to_bf16(a1[i] * inv[mt] * w1[i]).x;
      }
      return o.v;
    }
  };

  // this wavefront's share of K, in steps of 32
  // (EPI 5: the blocks that own the same weight rows share K among themselves first, blockIdx.x taking its part.  The part
  // runs fastest in launch order and blocks go to the eight XCDs in turn, so with eight parts every XCD works on one
  // part of K and holds that part of X alone in its L2; with four, two XCDs a part.)
  const int ksteps_all = (K + 31) >> 5;
  int kbeg = 0, kend = ksteps_all;
  if (EPI == 5) {
    const int part = (ksteps_all + (int)gridDim.x - 1) / (int)gridDim.x;
    kbeg = blockIdx.x * part;
    kend = kbeg + part < ksteps_all ? kbeg + part : ksteps_all;
    if (kend < kbeg) kend = kbeg;
  }
  const int per = (kend - kbeg + WAVES - 1) / WAVES;
  const int s0 = kbeg + wave * per, s1 = (s0 + per < kend) ? s0 + per : kend;
  int s = s0;
  // steps whose loads are issued together: as many as about a hundred registers hold (16 bytes a lane per tile)
  constexpr int UQ = (WAVES >= 16 ? 12 : 24) / (R + MT);   // sixteen wavefronts leave a lane 128 registers
  constexpr int U = UQ >= 8 ? 8 : (UQ >= 4 ? 4 : (UQ >= 2 ? 2 : 1));
  constexpr int WSTEP = SHUF ? 512 : 32;  // elements between a row tile's consecutive k steps
  if (MT < 3) {
    // few rows: the steps' loads are issued U at a time, then multiplied (the ring below costs registers, and with
    // them a resident wavefront per SIMD, which these shapes need more)
    if ((K & 31) == 0 || SHUF) {
      if (EPI == 3 && s + U <= s1) {
        bf16x8_t a[U][R], b[U][MT];
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
          for (int r = 0; r < R; ++r) a[u][r] = wact ? load8(wrow[r] + (size_t)(s + u) * WSTEP) : zero8();
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) b[u][mt] = xok[mt] ? load_x(mt, s + u) : zero8();
        }
        GS_PRELOAD_CONV()
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int r = 0; r < R; ++r)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
              acc[r][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][r], b[u][mt], acc[r][mt], 0, 0, 0);
        s += U;
      } else if (EPI == 3) {
        GS_PRELOAD_CONV()
      }
      for (; s + U <= s1; s += U) {
        bf16x8_t a[U][R], b[U][MT];
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
          for (int r = 0; r < R; ++r) a[u][r] = wact ? load8(wrow[r] + (size_t)(s + u) * WSTEP) : zero8();
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) b[u][mt] = xok[mt] ? load_x(mt, s + u) : zero8();
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int r = 0; r < R; ++r)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
              acc[r][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][r], b[u][mt], acc[r][mt], 0, 0, 0);
      }
    } else if (EPI == 3) {
      GS_PRELOAD_CONV()
    }
  } else if (((K & 31) == 0 || SHUF) && s1 - s0 >= U) {
    // many rows: a ring of U steps in registers: a step is multiplied as soon as it has arrived and its place is
    // asked for again at once, U steps ahead, so that loads are in flight the whole time (loads return in order).
    // Measured against issuing U steps at a time, both builds run in turn on one GPU, six repeats each, gate|up of
    // 16384 x 2048: 18.6-18.7 against 19.3-19.4 us at 64 rows, 16.8-16.9 against 17.2-17.3 us at 48 rows.
    bf16x8_t a[U][R], b[U][MT];
    auto fetch = [&](int u, int step) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        // every lane loads (its address is a valid one): a load under a lane mask would hide from the
        // compiler how many loads are in flight, and it would wait for all of them
        const bf16x8_t v = load8(wrow[r] + (size_t)step * WSTEP);
        a[u][r] = (SHUF != 2 || wact) ? v : zero8();
      }
      // rows past M read row 0 or the padding of the last tile; their columns of the result are never stored
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b[u][mt] = load_x(mt, step);
    };
    auto multiply = [&](int u) {
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[r][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][r], b[u][mt], acc[r][mt], 0, 0, 0);
    };
#pragma unroll
    for (int u = 0; u < U; ++u) fetch(u, s0 + u);
    const int groups = (s1 - s0) / U;
    for (int g = 1; g < groups; ++g) {
      const int base = s0 + g * U;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        multiply(u);
        fetch(u, base + u);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) multiply(u);
    s = s0 + groups * U;
  }
  for (; s < s1; ++s) {
    const int k = (s << 5) + kg * 8;
    const bool kin = k < K;
    bf16x8_t b[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) b[mt] = (kin && xok[mt]) ? load_x(mt, s) : zero8();
#pragma unroll
    for (int r = 0; r < R; ++r) {
      bf16x8_t a = ((kin || SHUF) && wact) ? load8(wrow[r] + (size_t)s * WSTEP) : zero8();
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[r][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[mt], acc[r][mt], 0, 0, 0);
    }
  }

  if (scaled) {
    // a wavefront's first row was asked for at the start; its further rows (row wave + WAVES, ...) are asked for here
    // in batches, every load of a batch in flight before the first is added, at addresses that always exist (a row
    // or a partial sum that does not is read from the first and counted as zero): no load sits behind a branch
    constexpr int RPW = (MT * 16 + WAVES - 1) / WAVES;
    constexpr int BATCH = RPW - 1 < 8 ? (RPW > 1 ? RPW - 1 : 1) : 8;
    if (wave < M) {
      float ssum = (pre[0] + pre[1]) + (pre[2] + pre[3]);
      for (int b = 256 + lane; b < ex.nb; b += 64) ssum += ex.ssq[(size_t)wave * ex.nb + b];
      ssum = wave_sum_dpp(ssum);
      if (lane == 0) inv_s[wave] = norm_inverse(ssum, (float)K, ex.eps);
    }
    if (MT == 1) {   // at most one further row: the plain loop is the smallest code, and the step of few rows feels it
      for (int m = wave + WAVES; m < M; m += WAVES) {
        float ssum = 0.f;
        for (int b = lane; b < ex.nb; b += 64) ssum += ex.ssq[(size_t)m * ex.nb + b];
        ssum = wave_sum_dpp(ssum);
        if (lane == 0) inv_s[m] = norm_inverse(ssum, (float)K, ex.eps);
      }
    }
#pragma unroll
    for (int i0 = 1; MT > 1 && i0 < RPW; i0 += BATCH) {
      if (wave + i0 * WAVES < M) {
        float q[BATCH][4];
#pragma unroll
        for (int i = 0; i < BATCH; ++i) {
          const int m = wave + (i0 + i) * WAVES;
          const float* row = ex.ssq + (size_t)(m < M ? m : wave) * ex.nb;
#pragma unroll
          for (int j = 0; j < 4; ++j) q[i][j] = row[lane + 64 * j < ex.nb ? lane + 64 * j : 0];
        }
#pragma unroll
        for (int i = 0; i < BATCH; ++i) {
          const int m = wave + (i0 + i) * WAVES;
#pragma unroll
          for (int j = 0; j < 4; ++j) q[i][j] = lane + 64 * j < ex.nb ? q[i][j] : 0.f;
          float ssum = (q[i][0] + q[i][1]) + (q[i][2] + q[i][3]);
          if (ex.nb > 256 && m < M)
            for (int b = 256 + lane; b < ex.nb; b += 64) ssum += ex.ssq[(size_t)m * ex.nb + b];
          ssum = wave_sum_dpp(ssum);
          if (lane == 0 && i0 + i < RPW && m < M) inv_s[m] = norm_inverse(ssum, (float)K, ex.eps);
        }
      }
    }
    if (WAVES == 1) __syncthreads();
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

  // rows that came pre-weighted get their inverse root mean square now
  if (scaled) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const float iv = inv_s[(mt * 16 + r16 < M) ? mt * 16 + r16 : 0];
#pragma unroll
      for (int r = 0; r < R; ++r) acc[r][mt] *= iv;
    }
  }

  // lane l holds, for token mt*16 + l%16, columns rowbase + 4*(l/16) + 0..3 of every tile
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + r16;
    const bool live = m < M;
    if (EPI == 0 || EPI == 5) {
      if (!live) continue;
      TOut* Yp = EPI == 5 ? Y + (size_t)blockIdx.x * M * ldy : Y;   // partial sums: one (M, N) sheet per part of K
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int n = rowbase[r] + kg * 4;
        if (N - n > 0) store4<TOut>(Yp + (size_t)m * ldy + n, acc[r][mt], N - n);
      }
    } else if (EPI == 1) {
      if (!live) continue;
#pragma unroll
      for (int r = 0; r < R; r += 2) {
        const int n = rowbase[r] + kg * 4;  // output column in [0, N/2)
        f32x4_t g = acc[r][mt], u = acc[r + 1][mt], o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = g[i] / (1.0f + expf(-g[i])) * u[i];
        if (half - n > 0) store4<TOut>(Y + (ex.y_tiled ? tiled_index(m, n, MT) : (size_t)m * ldy + n), o, half - n);
      }
    } else if (EPI == 2) {
      // every lane takes part in the shuffles, live or not
      float ss = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int n = rowbase[r] + kg * 4;
        if (live && n < N && half_ok) {
          float* p = ex.res_out + (size_t)m * N + n;
          f32x4_t nv, xv;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            // the product is rounded to bfloat16 first, as the unfused path stores it before the add
            nv[i] = rold[r][mt][i] + to_f32(f32_to_bf16(acc[r][mt][i]));
            if (n + i < N) ss += nv[i] * nv[i];
            xv[i] = nv[i] * nextw[r][i];
          }
          if (vec4) *reinterpret_cast<f32x4_t*>(p) = nv;
          else
            for (int i = 0; i < 4; ++i)
              if (n + i < N) p[i] = nv[i];
          if (ex.xs_out) store4<bf16>(ex.xs_out + (ex.y_tiled ? tiled_index(m, n, MT) : (size_t)m * N + n), xv, N - n);
        }
      }
      ss += __shfl_xor(ss, 16, 64);
      ss += __shfl_xor(ss, 32, 64);
      if (live && kg == 0) ex.ssq_out[(size_t)m * gridDim.x + blockIdx.x] = ss;
    } else if (EPI == 3) {
      if (!live) continue;
      const int H = N / 3, Wd = ex.conv_w;
      const int slot = cslot[mt];
      const int c0 = blockIdx.x * (SHUF == 2 ? 8 : 16) + kg * 4;
      if (pre_conv) {
        if (c0 >= H || !half_ok) continue;
        GS_CONV_WIDTH(GS_CONV_EPI_BODY)
        continue;
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = c0 + i;
        if (c >= H || !half_ok) break;
        const float Bv = to_f32(f32_to_bf16(acc[0][mt][i])), Cv = to_f32(f32_to_bf16(acc[R > 1 ? 1 : 0][mt][i])),
                    Xv = to_f32(f32_to_bf16(acc[R > 2 ? 2 : 0][mt][i]));
        const float u = Bv * Xv;
        float* hist = ex.state + ((size_t)slot * H + c) * (Wd - 1);
        const float* wt = ex.taps + (size_t)c * Wd;
        float y = 0.f;
        for (int p = 0; p < Wd - 1; ++p) y += wt[p] * hist[p];
        y += wt[Wd - 1] * u;
        if (ex.conv_bias) y += ex.conv_bias[c];
        Y[ex.y_tiled ? tiled_index(m, c, MT) : (size_t)m * ldy + c] = from_f32<TOut>(Cv * y);
        for (int p = 0; p < Wd - 2; ++p) hist[p] = hist[p + 1];
        hist[Wd - 2] = u;
      }
    }
  }
}

template <int R, int MT, int WAVES, int PRO, int EPI, int SHUF, typename TOut>
static void launch_skinny(int blocks, const bf16* X, int ldx, const bf16* W, TOut* Y, int ldy, int M, int N, int K,
                          const SkinnyExtra& ex, hipStream_t stream) {
  const size_t lds = (size_t)(WAVES - 1) * R * MT * 256 * sizeof(float);
  if (lds > 64 * 1024) {
    // more than the default limit of dynamic LDS: asked for once per kernel
    static const hipError_t asked = hipFuncSetAttribute(
        reinterpret_cast<const void*>(&gemm_skinny_kernel<R, MT, WAVES, PRO, EPI, SHUF, TOut>),
        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    (void)asked;
  }
  gemm_skinny_kernel<R, MT, WAVES, PRO, EPI, SHUF, TOut>
      <<<blocks, WAVES * 64, lds, stream>>>(X, ldx, W, Y, ldy, M, N, K, ex);
}

template <int R, int MT, int WAVES, int SHUF>
static void launch_skinny_parts(int blocks, int parts, const bf16* X, int ldx, const bf16* W, float* Y, int M, int N,
                                int K, const SkinnyExtra& ex, hipStream_t stream) {
  const size_t lds = (size_t)(WAVES - 1) * R * MT * 256 * sizeof(float);
  gemm_skinny_kernel<R, MT, WAVES, 0, 5, SHUF, float>
      <<<dim3(parts, blocks), WAVES * 64, lds, stream>>>(X, ldx, W, Y, N, M, N, K, ex);
}

// MT from M; the wavefronts per block are given per MT so that the LDS for the partial tiles,
// (WAVES - 1) * R * MT KB, stays within 64 KB
#define GS_BY_MT4(R, W1, W2, W3, W4, PRO, EPI, TOut, blocks)                                                            \
  switch ((M + 15) / 16) {                                                                                              \
    case 1: launch_skinny<R, 1, W1, PRO, EPI, SHUF, TOut>(blocks, x, ldx, w, (TOut*)Y, ldy, M, N, K, ex, stream); break;  \
    case 2: launch_skinny<R, 2, W2, PRO, EPI, SHUF, TOut>(blocks, x, ldx, w, (TOut*)Y, ldy, M, N, K, ex, stream); break;  \
    case 3: launch_skinny<R, 3, W3, PRO, EPI, SHUF, TOut>(blocks, x, ldx, w, (TOut*)Y, ldy, M, N, K, ex, stream); break;  \
    default: launch_skinny<R, 4, W4, PRO, EPI, SHUF, TOut>(blocks, x, ldx, w, (TOut*)Y, ldy, M, N, K, ex, stream); break; \
  }
#define GS_BY_MT(R, WAVES, PRO, EPI, TOut, blocks) GS_BY_MT4(R, WAVES, WAVES, WAVES, WAVES, PRO, EPI, TOut, blocks)

// What the entry points pass on after their checks.
struct SkinnyCall {
  const bf16* x;
  int ldx;
  const bf16* w;   // row-major (SHUF = 0) or tile-major (SHUF = 1)
  void* Y;
  int y_dtype, ldy, M, N, K, epilogue;
  SkinnyExtra ex;
  hipStream_t stream;
};

template <int SHUF>
static void skinny_plain(const SkinnyCall& c) {
  const bf16 *x = c.x, *w = c.w;
  void* Y = c.Y;
  const int ldx = c.ldx, ldy = c.ldy, M = c.M, N = c.N, K = c.K;
  const SkinnyExtra& ex = c.ex;
  hipStream_t stream = c.stream;
  const bool pro = ex.res != nullptr, f32 = c.y_dtype == GS_F32;
  const int cols = c.epilogue == 1 ? N / 2 : N;
  const bool narrow = cols <= 8192;
  // few output columns: more wavefronts per block split K further, so that the whole chip streams
  if (c.epilogue == 1) {
    const int blocks = gs_ceil_div(cols, 16);
    if (pro) { if (f32) { GS_BY_MT4(2, 8, 8, 4, 4, 1, 1, float, blocks) } else { GS_BY_MT4(2, 8, 8, 4, 4, 1, 1, bf16, blocks) } }
    else     { if (f32) { GS_BY_MT4(2, 8, 8, 4, 4, 0, 1, float, blocks) } else { GS_BY_MT4(2, 8, 8, 4, 4, 0, 1, bf16, blocks) } }
  } else if (narrow) {
    const int blocks = gs_ceil_div(cols, 16);
    if (pro) { if (f32) { GS_BY_MT(1, 8, 1, 0, float, blocks) } else { GS_BY_MT(1, 8, 1, 0, bf16, blocks) } }
    else     { if (f32) { GS_BY_MT(1, 8, 0, 0, float, blocks) } else { GS_BY_MT(1, 8, 0, 0, bf16, blocks) } }
  } else {
    const int blocks = gs_ceil_div(cols, 32);
    if (pro) { if (f32) { GS_BY_MT4(2, 8, 8, 4, 4, 1, 0, float, blocks) } else { GS_BY_MT4(2, 8, 8, 4, 4, 1, 0, bf16, blocks) } }
    else     { if (f32) { GS_BY_MT4(2, 8, 8, 4, 4, 0, 0, float, blocks) } else { GS_BY_MT4(2, 8, 8, 4, 4, 0, 0, bf16, blocks) } }
  }
}

template <int SHUF>
static void skinny_residual(const SkinnyCall& c) {
  const bf16 *x = c.x, *w = c.w;
  float* Y = nullptr;
  const int ldx = c.ldx, ldy = c.N, M = c.M, N = c.N, K = c.K;
  const SkinnyExtra& ex = c.ex;
  hipStream_t stream = c.stream;
  const int blocks = gs_ceil_div(N, SHUF == 2 ? 8 : 16);
  if (SHUF == 2) { GS_BY_MT(1, 8, 0, 2, float, blocks) }
  else if (K >= 4096) { GS_BY_MT(1, 16, 0, 2, float, blocks) } else { GS_BY_MT(1, 8, 0, 2, float, blocks) }
}

// Partial sums over `parts` parts of K into Y (parts, M, N) float32: two weight tiles a block, four wavefronts.
template <int SHUF>
static void skinny_parts(const SkinnyCall& c, int parts) {
  const int blocks = gs_ceil_div(c.N, 32);
  switch ((c.M + 15) / 16) {
    case 1: launch_skinny_parts<2, 1, 4, SHUF>(blocks, parts, c.x, c.ldx, c.w, (float*)c.Y, c.M, c.N, c.K, c.ex, c.stream); break;
    case 2: launch_skinny_parts<2, 2, 4, SHUF>(blocks, parts, c.x, c.ldx, c.w, (float*)c.Y, c.M, c.N, c.K, c.ex, c.stream); break;
    case 3: launch_skinny_parts<2, 3, 4, SHUF>(blocks, parts, c.x, c.ldx, c.w, (float*)c.Y, c.M, c.N, c.K, c.ex, c.stream); break;
    default: launch_skinny_parts<2, 4, 4, SHUF>(blocks, parts, c.x, c.ldx, c.w, (float*)c.Y, c.M, c.N, c.K, c.ex, c.stream); break;
  }
}

template <int SHUF>
static void skinny_conv(const SkinnyCall& c) {
  const bf16 *x = c.x, *w = c.w;
  void* Y = c.Y;
  const int ldx = c.ldx, ldy = c.ldy, M = c.M, N = c.N, K = c.K;
  const SkinnyExtra& ex = c.ex;
  hipStream_t stream = c.stream;
  const int blocks = gs_ceil_div(N / 3, SHUF == 2 ? 8 : 16);
  if (ex.res) { GS_BY_MT4(3, 8, 8, 4, 4, 1, 3, bf16, blocks) } else { GS_BY_MT4(3, 8, 8, 8, 8, 0, 3, bf16, blocks) }
}
