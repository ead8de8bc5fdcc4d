// Decode attention: one query token per sequence over its paged keys and values, bfloat16 cache.
//
// The step reads every cached key and value of the live sequences once; that stream is all the
// work there is.  A block owns (split, key head, sequence): a contiguous share of the sequence's
// keys, for all G query heads that share the key head, so keys and values are read once per group.
//
// Inside a block each wavefront takes tiles of 64 keys.  Scores: lane = key; the lane reads its key row
// (D bfloat16, 16-byte loads) and dots it with the G queries held in LDS as float32.  Softmax
// runs online per head across the wavefront (running maximum and sum).  Values: lane = (key
// group of 8, chunk of 8 features); 16-byte loads of V rows, probabilities broadcast from LDS.
// Wavefronts, then splits, are merged by the usual (max, sum, accumulator) rule in a fixed order.
// With one split the block writes the output itself; with more, each block writes its partial
// (accumulator, max, sum) and a second small kernel merges them in split order.  (Merging in the
// last block to arrive would save that launch, but the device-wide fence it needs writes back and
// invalidates the L2 in every block, which costs far more than the launch.)  Scores, maxima, sums
// and accumulators are float32.
//
// Everything that changes between steps (positions, block table) is read from device memory, so the
// launch can be recorded into a graph.  q (T, q_stride), head h at [h D, (h+1) D); caches
// (pages, nkv, page_size, D); out (T, nh D).  Window: keys lo..pos with lo = pos - window + 1.
#include "common.h"

#define DEC_WAVES 4
#define DEC_MAXG 8

template <int D, int G>
__global__ __launch_bounds__(DEC_WAVES * 64) void attention_decode_kernel(
    const bf16* __restrict__ q, int q_stride, const bf16* __restrict__ kcache, const bf16* __restrict__ vcache,
    const int* __restrict__ positions, const int* __restrict__ block_table, int max_blocks, int page_size, int window,
    float scale, bf16* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml, int nh, int nkv) {
  constexpr int DC = D / 8;        // 16-byte chunks per row
  constexpr int KG = 64 / DC;      // key groups per wavefront in the value phase
  static_assert(D % 8 == 0 && 64 % DC == 0, "head width must be 8, 16, 32, 64, 128, 256 or 512");
  __shared__ float qs[G][D];
  __shared__ float ps[DEC_WAVES][64][G];
  __shared__ long vrow[DEC_WAVES][64];
  __shared__ float wm[DEC_WAVES][G], wl[DEC_WAVES][G];
  __shared__ float wacc[DEC_WAVES][G][D];

  const int split = blockIdx.x, nsplit = gridDim.x, kvh = blockIdx.y, seq = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int pos = positions[seq];
  const int lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;
  const int nkeys = pos - lo + 1;
  // this block's share of the keys, in whole tiles of 64
  const int tiles = (nkeys + 63) >> 6;
  const int tper = (tiles + nsplit - 1) / nsplit;
  const int t0 = split * tper, t1 = (t0 + tper < tiles) ? t0 + tper : tiles;
  const int* bt = block_table + (size_t)seq * max_blocks;

  for (int i = tid; i < G * D; i += blockDim.x) {
    int g = i / D, j = i - g * D;
    qs[g][j] = to_f32(q[(size_t)seq * q_stride + (size_t)(kvh * G + g) * D + j]) * scale;
  }
  __syncthreads();

  float m[G], l[G], acc[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[g][j] = 0.f;
  }
  const int dc = lane % DC, kq = lane / DC;

  for (int t = t0 + wave; t < t1; t += DEC_WAVES) {
    const int u = lo + (t << 6) + lane;  // this lane's key
    float s[G];
    long off = 0;
    if (u <= pos) {
      const int page = bt[u / page_size];
      off = (((long)page * nkv + kvh) * page_size + u % page_size) * D;
      const uint4* kr = reinterpret_cast<const uint4*>(kcache + off);
#pragma unroll
      for (int g = 0; g < G; ++g) s[g] = 0.f;
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        uint4 w = kr[c];
        const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float k0 = __uint_as_float(ww[e] << 16), k1 = __uint_as_float(ww[e] & 0xffff0000u);
#pragma unroll
          for (int g = 0; g < G; ++g) s[g] += qs[g][c * 8 + 2 * e] * k0 + qs[g][c * 8 + 2 * e + 1] * k1;
        }
      }
    } else {
#pragma unroll
      for (int g = 0; g < G; ++g) s[g] = -INFINITY;
    }
    float alpha[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float mn = fmaxf(m[g], wave_max(s[g]));
      float p = u <= pos ? expf(s[g] - mn) : 0.f;
      alpha[g] = expf(m[g] - mn);
      l[g] = l[g] * alpha[g] + wave_sum(p);
      m[g] = mn;
      ps[wave][lane][g] = p;
    }
    vrow[wave][lane] = off;
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f);  // LDS writes of this wavefront are visible to its own lanes
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[g][j] *= alpha[g];
    const int nk = pos - (lo + (t << 6)) + 1 < 64 ? pos - (lo + (t << 6)) + 1 : 64;
    for (int kk = kq; kk < nk; kk += KG) {
      uint4 w = *reinterpret_cast<const uint4*>(vcache + vrow[wave][kk] + dc * 8);
      const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
      float v[8];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[2 * e] = __uint_as_float(ww[e] << 16);
        v[2 * e + 1] = __uint_as_float(ww[e] & 0xffff0000u);
      }
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float p = ps[wave][kk][g];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[g][j] += p * v[j];
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  // key groups of a wavefront hold partial sums over different keys for the same features: add them
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float v = acc[g][j];
      for (int o = DC; o < 64; o <<= 1) v += __shfl_xor(v, o, 64);
      acc[g][j] = v;
    }
  if (kq == 0) {
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int j = 0; j < 8; ++j) wacc[wave][g][dc * 8 + j] = acc[g][j];
  }
  if (lane == 0) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      wm[wave][g] = m[g];
      wl[wave][g] = l[g];
    }
  }
  __syncthreads();

  // merge the wavefronts, in wavefront order
  const size_t unit = ((size_t)seq * nkv + kvh) * nsplit + split;  // this block's partial
  for (int i = tid; i < G * D; i += blockDim.x) {
    int g = i / D, j = i - g * D;
    float M = -INFINITY;
    for (int w = 0; w < DEC_WAVES; ++w) M = fmaxf(M, wm[w][g]);
    float o = 0.f, L = 0.f;
    if (M > -INFINITY)
      for (int w = 0; w < DEC_WAVES; ++w)
        if (wm[w][g] > -INFINITY) {
          float f = expf(wm[w][g] - M);
          o += wacc[w][g][j] * f;
          L += wl[w][g] * f;
        }
    if (nsplit == 1) {
      out[((size_t)seq * nh + kvh * G + g) * D + j] = f32_to_bf16(o / L);
    } else {
      part_o[(unit * G + g) * D + j] = o;
      if (j == 0) {
        part_ml[(unit * G + g) * 2] = M;
        part_ml[(unit * G + g) * 2 + 1] = L;
      }
    }
  }
}

// Merge the splits of each (sequence, head), in split order.  One block per (sequence, key head).
__global__ void attention_decode_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                              bf16* __restrict__ out, int nsplit, int nh, int nkv, int G, int D) {
  const int kvh = blockIdx.x, seq = blockIdx.y;
  const size_t base = ((size_t)seq * nkv + kvh) * nsplit;
  for (int i = threadIdx.x; i < G * D; i += blockDim.x) {
    int g = i / D, j = i - g * D;
    float M = -INFINITY;
    for (int sp = 0; sp < nsplit; ++sp) M = fmaxf(M, part_ml[((base + sp) * G + g) * 2]);
    float o = 0.f, L = 0.f;
    for (int sp = 0; sp < nsplit; ++sp) {
      float ms = part_ml[((base + sp) * G + g) * 2];
      if (ms > -INFINITY) {
        float f = expf(ms - M);
        o += part_o[((base + sp) * G + g) * D + j] * f;
        L += part_ml[((base + sp) * G + g) * 2 + 1] * f;
      }
    }
    out[((size_t)seq * nh + kvh * G + g) * D + j] = f32_to_bf16(o / L);
  }
}

template <int D>
static int launch_decode(int G, dim3 grid, hipStream_t stream, const bf16* q, int q_stride, const bf16* kc,
                         const bf16* vc, const int* positions, const int* bt, int max_blocks, int page_size,
                         int window, float scale, bf16* out, float* part_o, float* part_ml, int nh, int nkv) {
#define GS_RUN(GG)                                                                                                  \
  attention_decode_kernel<D, GG><<<grid, DEC_WAVES * 64, 0, stream>>>(q, q_stride, kc, vc, positions, bt, max_blocks, \
                                                                      page_size, window, scale, out, part_o,       \
                                                                      part_ml, nh, nkv)
  switch (G) {
    case 1: GS_RUN(1); break;
    case 2: GS_RUN(2); break;
    case 3: GS_RUN(3); break;
    case 4: GS_RUN(4); break;
    case 5: GS_RUN(5); break;
    case 6: GS_RUN(6); break;
    case 7: GS_RUN(7); break;
    case 8: GS_RUN(8); break;
    default: return -1;
  }
#undef GS_RUN
  return 0;
}

// Whether this kernel takes the sizes: head widths 16, 32, 64, 128 and groups of up to 8 heads.
extern "C" int gs_attention_decode_supports(int nh, int nkv, int d) {
  if (nkv <= 0 || nh % nkv) return 0;
  int g = nh / nkv;
  return (d == 16 || d == 32 || d == 64 || d == 128) && g >= 1 && g <= DEC_MAXG;
}

// Floats of workspace for nseq sequences: partial outputs, then (max, sum) pairs.
extern "C" long gs_attention_decode_workspace(int nseq, int nh, int nkv, int d, int nsplit) {
  return (long)nseq * nh * nsplit * (d + 2);
}

extern "C" int gs_attention_decode(const void* q, int q_stride, const void* kcache, const void* vcache,
                                   const int* positions, const int* block_table, int max_blocks, int page_size,
                                   int window, float scale, void* out, float* workspace, int nseq, int nh, int nkv,
                                   int d, int nsplit, hipStream_t stream) {
  GS_REQUIRE(gs_attention_decode_supports(nh, nkv, d), "attention_decode: sizes nh=%d nkv=%d d=%d are not taken", nh, nkv, d);
  GS_REQUIRE(nseq >= 0 && nseq <= 65535 && nkv <= 65535, "attention_decode: bad batch %d", nseq);
  GS_REQUIRE(nsplit >= 1 && nsplit <= 64, "attention_decode: %d splits outside [1, 64]", nsplit);
  GS_REQUIRE(page_size > 0 && max_blocks > 0 && window >= 0, "attention_decode: bad page_size/max_blocks/window");
  GS_REQUIRE(q_stride >= nh * d && q_stride % 1 == 0, "attention_decode: q_stride %d below nh*d", q_stride);
  GS_REQUIRE((d * (int)sizeof(bf16)) % 16 == 0 && ((uintptr_t)kcache & 15) == 0 && ((uintptr_t)vcache & 15) == 0,
             "attention_decode: cache rows must be 16-byte aligned");
  if (nseq == 0) return 0;
  int G = nh / nkv;
  dim3 grid(nsplit, nkv, nseq);
  float* part_o = workspace;
  float* part_ml = workspace + (size_t)nseq * nh * nsplit * d;
  int rc = -1;
#define GS_ARGS                                                                                                   \
  G, grid, stream, (const bf16*)q, q_stride, (const bf16*)kcache, (const bf16*)vcache, positions, block_table,    \
      max_blocks, page_size, window, scale, (bf16*)out, part_o, part_ml, nh, nkv
  switch (d) {
    case 16: rc = launch_decode<16>(GS_ARGS); break;
    case 32: rc = launch_decode<32>(GS_ARGS); break;
    case 64: rc = launch_decode<64>(GS_ARGS); break;
    case 128: rc = launch_decode<128>(GS_ARGS); break;
  }
#undef GS_ARGS
  GS_REQUIRE(rc == 0, "attention_decode: no kernel for group %d", G);
  GS_LAUNCH_CHECK("attention_decode");
  if (nsplit > 1) {
    dim3 mgrid(nkv, nseq);
    attention_decode_merge_kernel<<<mgrid, 256, 0, stream>>>(part_o, part_ml, (bf16*)out, nsplit, nh, nkv, G, d);
    GS_LAUNCH_CHECK("attention_decode_merge");
  }
  return 0;
}
