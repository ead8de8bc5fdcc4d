// Decode attention: one query token per sequence over its paged keys and values, bfloat16 cache.
//
// The step reads every cached key and value of the live sequences once; that stream is all the
// work there is, and for a few hundred keys the kernel's time is a chain of memory round trips
// (position, page number, rows), so the chain is kept short: a wavefront issues all the loads of a
// tile of 64 keys, keys and values, before it computes anything, and (where registers allow) the next
// tile's loads before it computes the current one.
//
// A block owns (split, key head, sequence): a contiguous share of the sequence's keys, for all G
// query heads that share the key head, so keys and values are read once per group.  Inside a block
// each wavefront takes tiles of 64 keys.  Scores run on the matrix cores (v_mfma_f32_16x16x32_bf16:
// 16 keys x 16 head columns, of which G are used, per instruction), with the key rows loaded straight
// in operand order and the queries held in registers.  Softmax runs online per head (running maximum
// and sum, base-2 exponentials of scores scaled by log2 e).  Values: lane = (key group, chunk of 8
// features); 16-byte loads of V rows, probabilities broadcast from LDS.  Wavefronts, then splits, are merged by the usual (max, sum, accumulator) rule
// in a fixed order.  With one split the block writes the output itself; with more, each block writes
// its partial (accumulator, max, sum) and a second small kernel merges them in split order.  (Merging
// in the last block to arrive would save that launch, but the device-wide fence it needs writes back
// and invalidates the L2 in every block, which costs far more than the launch.)  A block has eight
// wavefronts, so that for contexts of up to about a thousand keys one block per (sequence, key head)
// covers them in a pass or two and no merge kernel is needed.  Scores, maxima, sums and accumulators
// are float32.
//
// Everything that changes between steps (positions, block table) is read from device memory, so the
// launch can be recorded into a graph.  q (T, q_stride), head h at [h D, (h+1) D); caches
// (pages, nkv, page_size, D); out (T, nh D).  Window: keys lo..pos with lo = pos - window + 1.
#include "common.h"
#include "no_alloc.h"
#include <mutex>

#define DEC_MAXG 8
#define DEC_LOG2E 1.4426950408889634f

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

// With RAW, q points at rows of q|k|v as their product left them (q heads, then k heads, then v heads), and the
// kernel does what comes between that product and attention itself: the head norms of q and k, the rotation, and
// the write of the new key and value into their page.  Every block norms and rotates its own queries; the block
// whose keys end with the new one norms and rotates it, keeps it and the value in LDS for its scores, and writes
// both to the cache for the steps to come.  Heads of 64 or 128, rotated whole.
// Where column c of sequence seq's output goes: a row of `width`, or tiled rows (out_tiles = ceil(nseq / 16) > 0),
// the order in which the product that follows takes them.
__device__ __forceinline__ size_t out_index(int seq, int c, int width, int out_tiles) {
  return out_tiles ? tiled_index(seq, c, out_tiles) : (size_t)seq * width + c;
}

struct DecodeRaw {
  const float* qw;       // (D) head norm weights, or null for no norm
  const float* kw;
  float eps;
  const float* cos_t;    // (positions, D / 2)
  const float* sin_t;
  int write_kv;          // 0: another layer owns the cache; the new key is already in it
};

template <int D, int G, int W, int RAW>
__global__ __launch_bounds__(W * 64) void attention_decode_kernel(
    const bf16* __restrict__ q, int q_stride, bf16* kcache, bf16* vcache,
    const int* __restrict__ positions, const int* __restrict__ block_table, int max_blocks, int page_size,
    unsigned page_magic, int window, float scale, bf16* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml, int nh, int nkv, int out_tiles, DecodeRaw raw) {
  static_assert(!RAW || D == 64 || D == 128, "the fused head norm and rotation are written for heads of 64 and 128");
  constexpr int DC = D / 8;               // 16-byte chunks per row
  constexpr int KG = 64 / DC;             // key groups per wavefront in the value phase
  constexpr int NI = 64 / KG;             // keys per lane in the value phase
  constexpr int KS = (D + 31) / 32;       // steps of 32 features in the score products
  static_assert(D % 8 == 0 && 64 % DC == 0 && G <= 16, "head width must be 8, 16, 32, 64, 128, 256 or 512");
  // What the registers allow (256 a lane at eight wavefronts a block): the next tile's rows in flight while
  // this one is computed, for rows of up to 64.
  constexpr bool PIPE = D <= 64;
  __shared__ float ps[W][G][64];          // a tile's probabilities, then read per key in the value phase
  __shared__ float al[W][G];              // by how much a tile shrinks what was accumulated before it
  __shared__ float wm[W][G], wl[W][G];
  __shared__ float wacc[W][G][D];

  const int split = blockIdx.x, nsplit = gridDim.x, kvh = blockIdx.y, seq = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, kg = lane >> 4;
  const int pos = positions[seq];
  const int lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;
  const int nkeys = pos - lo + 1;
  // this block's share of the keys, in whole tiles of 64
  const int tiles = (nkeys + 63) >> 6;
  const int tper = (tiles + nsplit - 1) / nsplit;
  const int t0 = split * tper, t1 = (t0 + tper < tiles) ? t0 + tper : tiles;
  const int* bt = block_table + (size_t)seq * max_blocks;
  const int dc = lane % DC, kq = lane / DC;

  // where key u's row starts in the caches (u <= pos)
  // (u / page_size as one multiplication, page_magic = floor(2^32 / page_size) + 1, exact while u page_size < 2^32:
  // no branch near the loads, which would make the compiler wait for every load in flight)
  auto row_off = [&](int u) -> long {
    const int pg = (int)__umulhi((unsigned)u, page_magic);
    const int r = u - pg * page_size;
    return (((long)bt[pg] * nkv + kvh) * page_size + r) * D;
  };
  // The loads of tile t.  Keys, as the first operand of the score products: lane (r16, kg) holds, of the four
  // keys 4 r16 + kt, features 32 s + 8 kg .. + 8.  Values: the lane's chunk of eight features of the value rows
  // of its NI keys.  Keys beyond pos are read from key pos (they are masked, their probabilities are zero).
  auto issue = [&](int t, bf16x8_t (*kreg)[KS], uint4* vreg) {
    const int base = lo + (t << 6);
    long ko[4], vo[NI];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      const int u = base + 4 * r16 + kt;
      ko[kt] = row_off(u <= pos ? u : pos) + kg * 8;
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int uu = base + kq + i * KG;
      vo[i] = row_off(uu <= pos ? uu : pos) + dc * 8;
    }
#pragma unroll
    for (int kt = 0; kt < 4; ++kt)
#pragma unroll
      for (int st = 0; st < KS; ++st) {
        if (32 * st + 8 * kg < D)
          kreg[kt][st] = *reinterpret_cast<const bf16x8_t*>(kcache + ko[kt] + 32 * st);
        else
          kreg[kt][st] = bf16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
      }
#pragma unroll
    for (int i = 0; i < NI; ++i) vreg[i] = *reinterpret_cast<const uint4*>(vcache + vo[i]);
  };

  // Loads in the order of what they wait for: the queries, the norm weights and the step's own key and value
  // (they wait for nothing), the rotation factors and the page numbers (for the position), the key and value rows
  // (for the page numbers).  Loads return in order, so the queries are normed and rotated while the rows are on
  // their way.
  // the queries as the second operand: lane (r16, kg) holds head r16's features 32 s + 8 kg .. + 8
  // (lanes past the group load head 0's: every lane loads, no branch hides a load from the compiler's count)
  bf16x8_t qreg[KS];
#pragma unroll
  for (int st = 0; st < KS; ++st) {
    if (32 * st + 8 * kg < D)
      qreg[st] = *reinterpret_cast<const bf16x8_t*>(q + (size_t)seq * q_stride + (size_t)(kvh * G + (r16 < G ? r16 : 0)) * D + 32 * st + 8 * kg);
    else
      qreg[st] = bf16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
    if (!RAW && r16 >= G) qreg[st] = bf16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
  }
  // Every wavefront keeps a copy of its own of the step's key and value in LDS (the wavefront whose tile holds the
  // new key reads them there: the cache's rows were loaded before they were written), so no wavefront waits for
  // another; wavefront 0 of the block whose keys end with the new one also writes them to the cache.
  __shared__ __align__(16) uint16_t knew[RAW ? W : 1][RAW ? D : 8], vnew[RAW ? W : 1][RAW ? D : 8];
  const bool has_new = RAW && raw.write_kv && t0 < t1 && t1 == tiles;   // this block's keys end with the new one
  constexpr int E = D >= 64 ? D / 64 : 1;
  float qw8[RAW ? KS : 1][8], c8[RAW ? KS / 2 : 1][8], s8[RAW ? KS / 2 : 1][8];
  float kraw_f[E], kw_f[E], kc_f = 1.f, ks_f = 0.f;
  bf16 vraw_b[E];
  if constexpr (RAW != 0) {
    if (raw.qw) {
#pragma unroll
      for (int st = 0; st < KS; ++st) load8f(raw.qw + 32 * st + 8 * kg, qw8[st]);
    }
    const bf16* kraw = q + (size_t)seq * q_stride + (size_t)(nh + kvh) * D;
    const bf16* vraw = q + (size_t)seq * q_stride + (size_t)(nh + nkv + kvh) * D;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      kraw_f[e] = to_f32(kraw[lane + 64 * e]);
      vraw_b[e] = vraw[lane + 64 * e];
      kw_f[e] = raw.kw ? raw.kw[lane + 64 * e] : 1.f;
    }
    // (weights and rotation factors in 16-byte loads: the tables' rows and this lane's offsets are multiples of 8)
#pragma unroll
    for (int st = 0; st < KS / 2; ++st) {
      load8f(raw.cos_t + (size_t)pos * (D / 2) + 32 * st + 8 * kg, c8[st]);
      load8f(raw.sin_t + (size_t)pos * (D / 2) + 32 * st + 8 * kg, s8[st]);
    }
    const int pi = E == 2 ? lane : (lane & 31);          // index of this lane's pair of the key
    kc_f = raw.cos_t[(size_t)pos * (D / 2) + pi];
    ks_f = raw.sin_t[(size_t)pos * (D / 2) + pi];
  }
  bf16x8_t kn[4][KS];
  uint4 vn[NI];
  int t = t0 + wave;
  // (a wavefront without a tile asks for the block's first one: its address is a valid one, and a load behind a
  // branch would make the compiler wait for every load in flight where it needs the queries)
  issue(t < t1 ? t : (t0 < tiles ? t0 : 0), kn, vn);

  if constexpr (RAW != 0) {
    // head norm and rotation of this lane's part of its query: float32 arithmetic on the product's bfloat16
    // values, rounded to bfloat16 again, as the separate kernel does.  The halves of a rotation pair (i, i + D/2)
    // are steps KS/2 apart in the same lane.
    float qf[KS][8];
    float ss = 0.f;
#pragma unroll
    for (int st = 0; st < KS; ++st)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        qf[st][j] = (float)qreg[st][j];
        ss += qf[st][j] * qf[st][j];
      }
    if (raw.qw) {
      const float inv = norm_inverse(group4_sum(ss), (float)D, raw.eps);
#pragma unroll
      for (int st = 0; st < KS; ++st)
#pragma unroll
        for (int j = 0; j < 8; ++j) qf[st][j] = qf[st][j] * inv * qw8[st][j];
    }
#pragma unroll
    for (int st = 0; st < KS / 2; ++st)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float a = qf[st][j], b = qf[st + KS / 2][j];
        qf[st][j] = a * c8[st][j] - b * s8[st][j];
        qf[st + KS / 2][j] = a * s8[st][j] + b * c8[st][j];
      }
#pragma unroll
    for (int st = 0; st < KS; ++st)
#pragma unroll
      for (int j = 0; j < 8; ++j) qreg[st][j] = (r16 < G) ? (__bf16)qf[st][j] : (__bf16)0.f;
    // the new key and value: lane = feature (and feature + 64 for heads of 128)
    if (raw.write_kv) {
      float kf[E];
      float ks = 0.f;
#pragma unroll
      for (int e = 0; e < E; ++e) {
        kf[e] = kraw_f[e];
        ks += kf[e] * kf[e];
      }
      if (raw.kw) {
        const float inv = norm_inverse(wave_sum_dpp(ks), (float)D, raw.eps);
#pragma unroll
        for (int e = 0; e < E; ++e) kf[e] = kf[e] * inv * kw_f[e];
      }
      if (E == 2) {
        const float a = kf[0], b = kf[E - 1];
        kf[0] = a * kc_f - b * ks_f;
        kf[E - 1] = a * ks_f + b * kc_f;
      } else {
        const float other = __shfl_xor(kf[0], 32, 64);
        kf[0] = lane < 32 ? kf[0] * kc_f - other * ks_f : other * ks_f + kf[0] * kc_f;
      }
      const long row = row_off(pos);
#pragma unroll
      for (int e = 0; e < E; ++e) {
        const bf16 kb = f32_to_bf16(kf[e]);
        knew[wave][lane + 64 * e] = kb.x;
        vnew[wave][lane + 64 * e] = vraw_b[e].x;
        if (has_new && wave == 0) {
          kcache[row + lane + 64 * e] = kb;
          vcache[row + lane + 64 * e] = vraw_b[e];
        }
      }
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_s_waitcnt(0xc07f);  // LDS writes of this wavefront are visible to its own lanes
    }
  }
  const float qscale = scale * DEC_LOG2E;   // scores are scaled after the product, in float32

  // lanes r16 < G keep the running maximum and sum of head r16; every lane keeps its share of all heads' sums
  float m = -INFINITY, l = 0.f;
  float acc[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[g][j] = 0.f;

  // one tile: scores, online softmax, values
  auto compute = [&](int t, bf16x8_t (*kc)[KS], uint4* vc) {
    const int base = lo + (t << 6);
    if (RAW && has_new && t == tiles - 1) {
      // the new key's row and the new value's row come from LDS: the cache's rows were loaded before they were written.
      // So do the places past it, which were loaded from the same row of the cache: their probabilities are zero, but
      // what that row held before this step (anything: the page may have been another request's) must not meet them
      const int rel = pos - base;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
        if (4 * r16 + kt >= rel) {
#pragma unroll
          for (int st = 0; st < KS; ++st) kc[kt][st] = *reinterpret_cast<const bf16x8_t*>(&knew[wave][32 * st + 8 * kg]);
        }
#pragma unroll
      for (int i = 0; i < NI; ++i)
        if (kq + i * KG >= rel) vc[i] = *reinterpret_cast<const uint4*>(&vnew[wave][dc * 8]);
    }
    // sc[kt][i]: head r16, key base + 4 (4 kg + i) + kt
    f32x4_t sc[4];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      sc[kt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int st = 0; st < KS; ++st) sc[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kc[kt][st], qreg[st], sc[kt], 0, 0, 0);
    }
    float mx = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 4; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool valid = base + 4 * (4 * kg + i) + kt <= pos;
        sc[kt][i] = valid ? sc[kt][i] * qscale : -INFINITY;
        mx = fmaxf(mx, sc[kt][i]);
      }
    const float mn = fmaxf(m, group4_max(mx));   // finite: a tile holds at least one key
    float sum = 0.f;
#pragma unroll
    for (int kt = 0; kt < 4; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        sc[kt][i] = __builtin_amdgcn_exp2f(sc[kt][i] - mn);   // 0 for masked keys
        sum += sc[kt][i];
      }
    const float alpha = __builtin_amdgcn_exp2f(m - mn);
    l = l * alpha + group4_sum(sum);
    m = mn;
    if (r16 < G) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        *reinterpret_cast<f32x4_t*>(&ps[wave][r16][4 * (4 * kg + i)]) = f32x4_t{sc[0][i], sc[1][i], sc[2][i], sc[3][i]};
      if (kg == 0) al[wave][r16] = alpha;
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f);  // LDS writes of this wavefront are visible to its own lanes
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const float a = al[wave][g];
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[g][j] *= a;
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const uint32_t ww[4] = {vc[i].x, vc[i].y, vc[i].z, vc[i].w};
      float v[8];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[2 * e] = __uint_as_float(ww[e] << 16);
        v[2 * e + 1] = __uint_as_float(ww[e] & 0xffff0000u);
      }
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const float p = ps[wave][g][kq + i * KG];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[g][j] += p * v[j];
      }
    }
    __builtin_amdgcn_wave_barrier();
  };

  if (PIPE) {
    // the next tile's loads are in flight while this one is computed: two sets of row registers
    for (; t < t1; t += W) {
      bf16x8_t kc[4][KS];
      uint4 vc[NI];
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int st = 0; st < KS; ++st) kc[kt][st] = kn[kt][st];
#pragma unroll
      for (int i = 0; i < NI; ++i) vc[i] = vn[i];
      if (t + W < t1) issue(t + W, kn, vn);
      compute(t, kc, vc);
    }
  } else {
    // one set of row registers: the first tile's loads were issued above
    if (t < t1) {
      compute(t, kn, vn);
      t += W;
    }
    for (; t < t1; t += W) {
      issue(t, kn, vn);
      compute(t, kn, vn);
    }
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
  if (lane < G) {
    wm[wave][lane] = m;
    wl[wave][lane] = l;
  }
  __syncthreads();

  // merge the wavefronts, in wavefront order
  const size_t unit = ((size_t)seq * nkv + kvh) * nsplit + split;  // this block's partial
  for (int i = tid; i < G * D; i += blockDim.x) {
    int g = i / D, j = i - g * D;
    float M = -INFINITY;
    for (int w = 0; w < W; ++w) M = fmaxf(M, wm[w][g]);
    float o = 0.f, L = 0.f;
    if (M > -INFINITY)
      for (int w = 0; w < W; ++w)
        if (wm[w][g] > -INFINITY) {
          float f = __builtin_amdgcn_exp2f(wm[w][g] - M);
          o += wacc[w][g][j] * f;
          L += wl[w][g] * f;
        }
    if (nsplit == 1) {
      out[out_index(seq, (kvh * G + g) * D + j, nh * D, out_tiles)] = f32_to_bf16(o / L);
    } else {
      part_o[(unit * G + g) * D + j] = o;
      if (j == 0) {
        part_ml[(unit * G + g) * 2] = M;
        part_ml[(unit * G + g) * 2 + 1] = L;
      }
    }
  }
}

// Merge the splits of each (sequence, head), in split order.  One block per (sequence, key head).  The splits'
// maxima and sums go through LDS, so that each head's weights are computed once and the loads of the partial
// outputs are independent of one another.
#define DEC_MAXSPLIT 64
__global__ void attention_decode_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                              bf16* __restrict__ out, int nsplit, int nh, int nkv, int G, int D,
                                              int out_tiles) {
  __shared__ float sm[DEC_MAXSPLIT][DEC_MAXG], sl[DEC_MAXSPLIT][DEC_MAXG], sf[DEC_MAXSPLIT][DEC_MAXG];
  __shared__ float sinv[DEC_MAXG];
  const int kvh = blockIdx.x, seq = blockIdx.y;
  const size_t base = ((size_t)seq * nkv + kvh) * nsplit;
  for (int i = threadIdx.x; i < nsplit * G; i += blockDim.x) {
    const int sp = i / G, g = i - sp * G;
    sm[sp][g] = part_ml[((base + sp) * G + g) * 2];
    sl[sp][g] = part_ml[((base + sp) * G + g) * 2 + 1];
  }
  __syncthreads();
  if (threadIdx.x < G) {
    const int g = threadIdx.x;
    float M = -INFINITY;
    for (int sp = 0; sp < nsplit; ++sp) M = fmaxf(M, sm[sp][g]);
    float L = 0.f;
    for (int sp = 0; sp < nsplit; ++sp) {
      const float f = sm[sp][g] > -INFINITY ? __builtin_amdgcn_exp2f(sm[sp][g] - M) : 0.f;   // maxima are in base-2 units
      sf[sp][g] = f;
      L += sl[sp][g] * f;
    }
    sinv[g] = 1.0f / L;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < G * D; i += blockDim.x) {
    const int g = i / D, j = i - g * D;
    float o = 0.f;
    int sp = 0;
    for (; sp + 8 <= nsplit; sp += 8) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = part_o[((base + sp + u) * G + g) * D + j];
#pragma unroll
      for (int u = 0; u < 8; ++u) o += v[u] * sf[sp + u][g];
    }
    for (; sp < nsplit; ++sp) o += part_o[((base + sp) * G + g) * D + j] * sf[sp][g];
    out[out_index(seq, (kvh * G + g) * D + j, nh * D, out_tiles)] = f32_to_bf16(o * sinv[g]);
  }
}

#define DEC_WAVES 8

// Wavefronts a block: eight, so that one block covers about a thousand keys in a pass or two; four where the grid
// holds more blocks than the chip has compute units (many sequences): blocks of four leave a lane's registers
// to two blocks a compute unit, whose chains of round trips then overlap (measured at 48 and at 64 sequences of
// 8 key heads: 18.5 against 23.8 us, 21 against 27).
template <int D, int RAW, int WV>
static int launch_decode_w(int G, dim3 grid, hipStream_t stream, const bf16* q, int q_stride, bf16* kc, bf16* vc,
                         const int* positions, const int* bt, int max_blocks, int page_size, unsigned page_magic,
                         int window, float scale, bf16* out, float* part_o, float* part_ml, int nh, int nkv,
                         int out_tiles, DecodeRaw raw) {
#define GS_RUN(GG)                                                                                                     \
  attention_decode_kernel<D, GG, WV, RAW><<<grid, WV * 64, 0, stream>>>(                                 \
      q, q_stride, kc, vc, positions, bt, max_blocks, page_size, page_magic, window, scale, out, part_o, part_ml, nh, \
      nkv, out_tiles, raw)
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

static int g_decode_cus = 0;   // compute units of the device, asked for once

template <int D, int RAW>
static int launch_decode(int G, dim3 grid, hipStream_t stream, const bf16* q, int q_stride, bf16* kc, bf16* vc,
                         const int* positions, const int* bt, int max_blocks, int page_size, unsigned page_magic,
                         int window, float scale, bf16* out, float* part_o, float* part_ml, int nh, int nkv,
                         int out_tiles, DecodeRaw raw) {
  if (g_decode_cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    g_decode_cus = n;
  }
  const long blocks = (long)grid.x * grid.y * grid.z;
  if (D <= 64 && blocks > 1L * g_decode_cus)
    return launch_decode_w<D, RAW, 4>(G, grid, stream, q, q_stride, kc, vc, positions, bt, max_blocks, page_size, page_magic,
                                      window, scale, out, part_o, part_ml, nh, nkv, out_tiles, raw);
  return launch_decode_w<D, RAW, DEC_WAVES>(G, grid, stream, q, q_stride, kc, vc, positions, bt, max_blocks, page_size,
                                            page_magic, window, scale, out, part_o, part_ml, nh, nkv, out_tiles, raw);
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

static int decode_entry(const void* q, int q_stride, void* kcache, void* vcache, const int* positions,
                        const int* block_table, int max_blocks, int page_size, int window, float scale, void* out,
                        int out_tiled, float* workspace, int nseq, int nh, int nkv, int d, int nsplit,
                        const DecodeRaw* raw, hipStream_t stream) {
  GS_REQUIRE(!out_tiled || (nh * d) % 32 == 0, "attention_decode: tiled rows need a width that is a multiple of 32, not %d", nh * d);
  const int out_tiles = out_tiled ? gs_ceil_div(nseq, 16) : 0;
  GS_REQUIRE(gs_attention_decode_supports(nh, nkv, d), "attention_decode: sizes nh=%d nkv=%d d=%d are not taken", nh, nkv, d);
  GS_REQUIRE(nseq >= 0 && nseq <= 65535 && nkv <= 65535, "attention_decode: bad batch %d", nseq);
  GS_REQUIRE(nsplit >= 1 && nsplit <= 64, "attention_decode: %d splits outside [1, 64]", nsplit);
  GS_REQUIRE(page_size > 0 && max_blocks > 0 && window >= 0, "attention_decode: bad page_size/max_blocks/window");
  GS_REQUIRE(q_stride >= (raw ? nh + 2 * nkv : nh) * d, "attention_decode: q_stride %d below the row's width", q_stride);
  GS_REQUIRE(q_stride % 8 == 0 && ((uintptr_t)q & 15) == 0, "attention_decode: query rows must be 16-byte aligned");
  GS_REQUIRE((d * (int)sizeof(bf16)) % 16 == 0 && ((uintptr_t)kcache & 15) == 0 && ((uintptr_t)vcache & 15) == 0,
             "attention_decode: cache rows must be 16-byte aligned");
  if (nseq == 0) return 0;
  int G = nh / nkv;
  dim3 grid(nsplit, nkv, nseq);
  GS_REQUIRE(page_size >= 2 && (long)max_blocks * page_size * page_size < (1L << 32),
             "attention_decode: page_size %d with %d blocks a sequence is outside what the kernel's division takes", page_size, max_blocks);
  const unsigned page_magic = (unsigned)((1ull << 32) / (unsigned)page_size + 1);
  float* part_o = workspace;
  float* part_ml = workspace + (size_t)nseq * nh * nsplit * d;
  int rc = -1;
  const DecodeRaw none = {};
#define GS_ARGS                                                                                             \
  G, grid, stream, (const bf16*)q, q_stride, (bf16*)kcache, (bf16*)vcache, positions, block_table, max_blocks, \
      page_size, page_magic, window, scale, (bf16*)out, part_o, part_ml, nh, nkv, out_tiles
  if (raw) {
    switch (d) {
      case 64: rc = launch_decode<64, 1>(GS_ARGS, *raw); break;
      case 128: rc = launch_decode<128, 1>(GS_ARGS, *raw); break;
    }
  } else {
    switch (d) {
      case 16: rc = launch_decode<16, 0>(GS_ARGS, none); break;
      case 32: rc = launch_decode<32, 0>(GS_ARGS, none); break;
      case 64: rc = launch_decode<64, 0>(GS_ARGS, none); break;
      case 128: rc = launch_decode<128, 0>(GS_ARGS, none); break;
    }
  }
#undef GS_ARGS
  GS_REQUIRE(rc == 0, "attention_decode: no kernel for group %d and head width %d", G, d);
  GS_LAUNCH_CHECK("attention_decode");
  if (nsplit > 1) {
    dim3 mgrid(nkv, nseq);
    attention_decode_merge_kernel<<<mgrid, 256, 0, stream>>>(part_o, part_ml, (bf16*)out, nsplit, nh, nkv, G, d, out_tiles);
    GS_LAUNCH_CHECK("attention_decode_merge");
  }
  return 0;
}

extern "C" int gs_attention_decode(const void* q, int q_stride, const void* kcache, const void* vcache,
                                   const int* positions, const int* block_table, int max_blocks, int page_size,
                                   int window, float scale, void* out, int out_tiled, float* workspace, int nseq, int nh,
                                   int nkv, int d, int nsplit, hipStream_t stream) {
  return decode_entry(q, q_stride, (void*)kcache, (void*)vcache, positions, block_table, max_blocks, page_size, window,
                      scale, out, out_tiled, workspace, nseq, nh, nkv, d, nsplit, nullptr, stream);
}

// ---- the entry point that allocates nothing (declared and described in no_alloc.h)
//
// `scratch` is the name of the device array as host code sees it: a stand-in, not a device address.  Its address on
// the current GPU comes from hipGetSymbolAddress, once per device with that device current (each GPU holds its own
// copy at its own address), and only that pointer goes to kernels.
static __device__ __align__(256) float scratch[GS_DECODE_STATIC_FLOATS];

#define GS_MAX_DEVICES 64
static float* g_scratch_ptr[GS_MAX_DEVICES];
static std::mutex g_scratch_mutex;

static int static_workspace(float** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  GS_REQUIRE(e == hipSuccess, "attention_decode_static: no current device: %s", hipGetErrorString(e));
  GS_REQUIRE(dev >= 0 && dev < GS_MAX_DEVICES, "attention_decode_static: device %d outside [0, %d)", dev, GS_MAX_DEVICES);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    float* p = nullptr;
    e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
    GS_REQUIRE(e == hipSuccess && p != nullptr, "attention_decode_static: the static workspace has no address on device %d: %s",
               dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return 0;
}

extern "C" int gs_attention_decode_static(const void* q, int q_stride, const void* kcache, const void* vcache,
                                          const int* positions, const int* block_table, int max_blocks, int page_size,
                                          int window, float scale, void* out, int out_tiled, int nseq, int nh, int nkv,
                                          int d, int nsplit, hipStream_t stream) {
  GS_REQUIRE(nseq >= 0 && nh > 0 && nkv > 0 && d > 0 && nsplit >= 1 && nsplit <= 64,
             "attention_decode_static: bad sizes nseq=%d nh=%d nkv=%d d=%d nsplit=%d", nseq, nh, nkv, d, nsplit);
  const long need = gs_attention_decode_workspace(nseq, nh, nkv, d, nsplit);
  GS_REQUIRE(need <= (long)GS_DECODE_STATIC_FLOATS,
             "attention_decode_static: %ld floats of workspace needed (nseq=%d nh=%d d=%d nsplit=%d), the static one holds %ld",
             need, nseq, nh, d, nsplit, (long)GS_DECODE_STATIC_FLOATS);
  float* ws = nullptr;
  if (static_workspace(&ws) != 0) return -1;
  return decode_entry(q, q_stride, (void*)kcache, (void*)vcache, positions, block_table, max_blocks, page_size, window,
                      scale, out, out_tiled, ws, nseq, nh, nkv, d, nsplit, nullptr, stream);
}

// Whether the kernel also takes the head norms, the rotation and the cache write: heads of 64 or 128 rotated whole.
extern "C" int gs_attention_decode_raw_supports(int nh, int nkv, int d, int rotary_dim) {
  return gs_attention_decode_supports(nh, nkv, d) && (d == 64 || d == 128) && rotary_dim == d;
}

// qkv (nseq, q_stride): the rows of q|k|v as their product left them.  The kernel norms and rotates q and the new
// key, writes the new key and value into their pages (unless write_kv is 0), and attends.
extern "C" int gs_attention_decode_raw(const void* qkv, int q_stride, void* kcache, void* vcache, const int* positions,
                                       const int* block_table, int max_blocks, int page_size, int window, float scale,
                                       const float* qw, const float* kw, float eps, const float* cos_t,
                                       const float* sin_t, int rotary_dim, int write_kv, void* out, int out_tiled,
                                       float* workspace, int nseq, int nh, int nkv, int d, int nsplit,
                                       hipStream_t stream) {
  GS_REQUIRE(gs_attention_decode_raw_supports(nh, nkv, d, rotary_dim), "attention_decode_raw: sizes nh=%d nkv=%d d=%d rotary=%d are not taken", nh, nkv, d, rotary_dim);
  GS_REQUIRE((qw == nullptr) == (kw == nullptr) && cos_t && sin_t, "attention_decode_raw: q and k norm weights come together; the rotation needs its tables");
  GS_REQUIRE((((uintptr_t)qw | (uintptr_t)kw | (uintptr_t)cos_t | (uintptr_t)sin_t) & 15) == 0, "attention_decode_raw: weights and tables must be 16-byte aligned");
  DecodeRaw raw = {qw, kw, eps, cos_t, sin_t, write_kv};
  return decode_entry(qkv, q_stride, kcache, vcache, positions, block_table, max_blocks, page_size, window, scale, out,
                      out_tiled, workspace, nseq, nh, nkv, d, nsplit, &raw, stream);
}
