// Prompt attention on the matrix cores: many queries per sequence over the paged cache, bfloat16.
//
// A block owns 16 consecutive queries of one sequence and one key head; its G wavefronts are the G query
// heads that share the key head, so keys and values are fetched once per group.  Keys are walked in steps
// of 32 with a running maximum and sum per query (online softmax, float32).
//
// Both products are computed transposed, so that everything a lane holds concerns one query (lane % 16):
//   S^T = K Q^T   A = K tile (16 keys x 32 features, 16-byte loads straight from the page, lane l: key
//                 l % 16, features 8 (l / 16) ..), B = Q^T (the wavefront's query fragment, kept in
//                 registers), result: lane l holds keys 4 (l / 16) + 0..3 for query l % 16.
//   O^T = V^T P^T B = P^T is exactly the lane's own eight probabilities of a step (two key blocks of
//                 four), A = V^T read from LDS, where the step's 32 value rows are staged transposed once
//                 per block.  Result: lane l holds features 4 (l / 16) + 0..3 (per tile of 16) of query l % 16.
// No probability ever crosses lanes; the only cross-lane traffic is the maximum and the sum over the four
// lane groups.  v_mfma_f32_16x16x32_bf16 throughout.
//
// Causal rule: the query at position p sees keys lo..p, lo = 0 or p - window + 1.  Tiles of queries come
// from the host: tile i covers rows tile_row[i] .. + tile_n[i] (at most 16 QT) of the flattened tokens, of
// sequence tile_seq[i].  Exponentials are base 2 on scores scaled by log2(e): one v_exp_f32 each.  q (T, q_stride), head h at [h D, (h+1) D); caches (pages, nkv, page_size, D); out (T, nh D).
#include <type_traits>

#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

#define PF_KSTEP 32
#define PF_PAD 4
#define PF_MAXPAGES 2048
#define PF_SLACK 6.0f
#define PF_LOG2E 1.4426950408889634f

// QT: tiles of 16 queries per wavefront; a key fragment and a value fragment feed QT products each.
template <int D, int G, int QT>
__global__ __launch_bounds__(G * 64) void attention_prefill_kernel(
    const bf16* __restrict__ q, int q_stride, const bf16* __restrict__ kcache, const bf16* __restrict__ vcache,
    const int* __restrict__ positions, const int* __restrict__ tile_seq, const int* __restrict__ tile_row,
    const int* __restrict__ tile_n, const int* __restrict__ block_table, int max_blocks, int page_size, int window,
    float scale, bf16* __restrict__ out, int nh, int nkv) {
  constexpr int KK = D / 32;   // feature steps of the score product
  constexpr int DT = D / 16;   // feature tiles of the output
  __shared__ uint16_t vt[D][PF_KSTEP + PF_PAD];
  __shared__ int pages[PF_MAXPAGES];
  const int tile = gridDim.x - 1 - blockIdx.x, kvh = blockIdx.y;   // late tiles walk the most keys: they start first
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, kg = lane >> 4;
  const int h = kvh * G + wave;
  const int seq = tile_seq[tile], row0 = tile_row[tile], nq = tile_n[tile];
  const int* bt = block_table + (size_t)seq * max_blocks;
  const int pos0 = positions[row0];                  // positions of a tile are consecutive
  const int last_key = pos0 + nq - 1;
  const int first_key = window > 0 ? (pos0 - window + 1 > 0 ? pos0 - window + 1 : 0) : 0;
  // scores are kept in units of log2(e), so that the exponentials are single v_exp_f32
  const float sc = scale * PF_LOG2E;
  const int ps_shift = (page_size & (page_size - 1)) == 0 ? __ffs(page_size) - 1 : -1;

  bool live[QT];
  int my_pos[QT], my_lo[QT];
  bf16x8_t qf[QT][KK];   // the queries as the B operand: lane (query r16, features 8 kg ..)
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    const int r = t * 16 + r16;
    live[t] = r < nq;
    my_pos[t] = pos0 + (live[t] ? r : nq - 1);
    my_lo[t] = window > 0 ? (my_pos[t] - window + 1 > 0 ? my_pos[t] - window + 1 : 0) : 0;
    const bf16* qrow = q + (size_t)(row0 + (live[t] ? r : 0)) * q_stride + (size_t)h * D + kg * 8;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) qf[t][kk] = *reinterpret_cast<const bf16x8_t*>(qrow + kk * 32);
  }
  float m[QT], l[QT];
  f32x4_t acc[QT][DT];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    m[t] = -INFINITY;
    l[t] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[t][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  // The tile's part of the block table goes to LDS first: a key's row is then one global load away, not
  // two dependent ones (page number, then row).  Longer ranges than the LDS copy holds look pages up in memory.
  const int blk0 = ps_shift >= 0 ? (first_key >> ps_shift) : first_key / page_size;
  const int blk1 = ps_shift >= 0 ? (last_key >> ps_shift) : last_key / page_size;
  const bool in_lds = blk1 - blk0 < PF_MAXPAGES;
  if (in_lds)
    for (int i = tid; i <= blk1 - blk0; i += G * 64) pages[i] = bt[blk0 + i];
  __syncthreads();
  // Rows outside first_key..last_key are never seen (their scores are masked): their addresses are clamped
  // into the range, so that every load is of a row the sequence holds and no load needs a branch.
  auto row_of = [&](int u) -> size_t {
    u = u < first_key ? first_key : (u > last_key ? last_key : u);
    int blk, offs;
    if (ps_shift >= 0) {
      blk = u >> ps_shift;
      offs = u & ((1 << ps_shift) - 1);
    } else {
      blk = u / page_size;
      offs = u % page_size;
    }
    const int page = in_lds ? pages[blk - blk0] : bt[blk];
    return (((size_t)page * nkv + kvh) * page_size + offs) * D;
  };
  // The loads of a step are issued one step ahead and land in registers while the step before is computed.
  constexpr int VPT = (PF_KSTEP * (D / 8) + G * 64 - 1) / (G * 64);   // value chunks per thread and step
  bf16x8_t kn[2][KK];
  uint4 vn[VPT];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const bf16* krow = kcache + row_of(k0 + b * 16 + r16) + kg * 8;   // the key whose row this lane loads
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) kn[b][kk] = *reinterpret_cast<const bf16x8_t*>(krow + kk * 32);
    }
#pragma unroll
    for (int x = 0; x < VPT; ++x) {
      const int i = (tid + x * G * 64) % (PF_KSTEP * (D / 8));
      const int key = i / (D / 8), c = i % (D / 8);
      vn[x] = *reinterpret_cast<const uint4*>(vcache + row_of(k0 + key) + c * 8);
    }
  };
  // per query: the last key it sees and the first, relative to this lane's rows of a score tile (4 kg + i)
  int hi[QT], lo[QT];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    hi[t] = live[t] ? my_pos[t] - kg * 4 : -(1 << 30);
    lo[t] = my_lo[t] - kg * 4;
  }
  const int kstart = (first_key / PF_KSTEP) * PF_KSTEP;
  fetch(kstart);
  for (int k0 = kstart; k0 <= last_key; k0 += PF_KSTEP) {
    bf16x8_t kc[2][KK];
    uint4 vc[VPT];
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) kc[b][kk] = kn[b][kk];
#pragma unroll
    for (int x = 0; x < VPT; ++x) vc[x] = vn[x];
    fetch(k0 + PF_KSTEP);          // beyond the last step the addresses are clamped and the loads are spare
    // stage the step's value rows transposed: thread (key, chunk of 8 features)
    __syncthreads();
#pragma unroll
    for (int x = 0; x < VPT; ++x) {
      const int i = tid + x * G * 64;
      if (i < PF_KSTEP * (D / 8)) {
        const int key = i / (D / 8), c = i % (D / 8);
        const uint32_t ww[4] = {vc[x].x, vc[x].y, vc[x].z, vc[x].w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          vt[c * 8 + 2 * e][key] = (uint16_t)(ww[e] & 0xffffu);
          vt[c * 8 + 2 * e + 1][key] = (uint16_t)(ww[e] >> 16);
        }
      }
    }
    // scores of two blocks of 16 keys: S^T = K Q^T; lane holds keys k0 + 16 b + 4 kg + i for its query
    float s[QT][8];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      f32x4_t st[QT];
#pragma unroll
      for (int t = 0; t < QT; ++t) st[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < KK; ++kk)
#pragma unroll
        for (int t = 0; t < QT; ++t) st[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kc[b][kk], qf[t][kk], st[t], 0, 0, 0);
#pragma unroll
      for (int t = 0; t < QT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = k0 + b * 16 + i;           // + 4 kg, which hi and lo already hold
          s[t][b * 4 + i] = (key <= hi[t] && key >= lo[t]) ? st[t][i] * sc : -INFINITY;
        }
    }
    bf16x8_t pf[QT];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      float mloc = s[t][0];
#pragma unroll
      for (int j = 1; j < 8; ++j) mloc = fmaxf(mloc, s[t][j]);
      mloc = group4_max(mloc);
      // The reference point of the exponentials moves only when the maximum has grown by more than 2^PF_SLACK
      // (or at the first keys): probabilities then stay below 2^PF_SLACK, well inside float32 and bfloat16,
      // and the accumulators are rescaled on few steps instead of on every one.
      if (mloc > m[t] + PF_SLACK || m[t] == -INFINITY) {
        if (mloc > -INFINITY) {
          const float a = m[t] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m[t] - mloc);
          l[t] *= a;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) acc[t][dt] *= a;
          m[t] = mloc;
        }
      }
      float p[8], lsum = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        p[j] = m[t] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(s[t][j] - m[t]);
        lsum += p[j];
      }
      l[t] += group4_sum(lsum);
#pragma unroll
      for (int j = 0; j < 8; ++j) pf[t][j] = (__bf16)p[j];
    }
    __syncthreads();   // the staged values are in place
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      // A = V^T tile: lane (feature 16 dt + r16, key slots 8 kg + j <-> block j / 4, key 4 kg + j % 4)
      union {
        bf16x8_t v;
        uint2 u2[2];
      } a;
      a.u2[0] = *reinterpret_cast<const uint2*>(&vt[dt * 16 + r16][kg * 4]);
      a.u2[1] = *reinterpret_cast<const uint2*>(&vt[dt * 16 + r16][16 + kg * 4]);
#pragma unroll
      for (int t = 0; t < QT; ++t) acc[t][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, pf[t], acc[t][dt], 0, 0, 0);
    }
  }
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    if (!live[t]) continue;
    const float inv = 1.0f / l[t];
    bf16* orow = out + (size_t)(row0 + t * 16 + r16) * nh * D + (size_t)h * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      uint2 o;
      o.x = (uint32_t)f32_to_bf16(acc[t][dt][0] * inv).x | ((uint32_t)f32_to_bf16(acc[t][dt][1] * inv).x << 16);
      o.y = (uint32_t)f32_to_bf16(acc[t][dt][2] * inv).x | ((uint32_t)f32_to_bf16(acc[t][dt][3] * inv).x << 16);
      *reinterpret_cast<uint2*>(orow + dt * 16 + kg * 4) = o;
    }
  }
}

// Head widths 32, 64, 128; groups of 1 to 8 heads (the block has one wavefront per head of the group).
extern "C" int gs_attention_prefill_supports(int nh, int nkv, int d) {
  if (nkv <= 0 || nh % nkv) return 0;
  int g = nh / nkv;
  return (d == 32 || d == 64 || d == 128) && g >= 1 && g <= 8;
}

template <int D, int QT>
static int launch_prefill(int G, dim3 grid, hipStream_t stream, const bf16* q, int q_stride, const bf16* kc,
                          const bf16* vc, const int* positions, const int* tile_seq, const int* tile_row,
                          const int* tile_n, const int* bt, int max_blocks, int page_size, int window, float scale,
                          bf16* out, int nh, int nkv) {
#define GS_RUN(GG)                                                                                                   \
  attention_prefill_kernel<D, GG, QT><<<grid, GG * 64, 0, stream>>>(q, q_stride, kc, vc, positions, tile_seq, tile_row, \
                                                                tile_n, bt, max_blocks, page_size, window, scale,   \
                                                                out, nh, nkv)
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

extern "C" int gs_attention_prefill(const void* q, int q_stride, const void* kcache, const void* vcache,
                                    const int* positions, const int* tile_seq, const int* tile_row,
                                    const int* tile_n, int ntiles, const int* block_table, int max_blocks,
                                    int page_size, int window, float scale, void* out, int nh, int nkv, int d,
                                    int tile_rows, hipStream_t stream) {
  GS_REQUIRE(gs_attention_prefill_supports(nh, nkv, d), "attention_prefill: sizes nh=%d nkv=%d d=%d are not taken", nh, nkv, d);
  GS_REQUIRE(ntiles >= 0 && nkv <= 65535, "attention_prefill: bad grid");
  GS_REQUIRE(tile_rows == 16 || tile_rows == 32, "attention_prefill: tiles hold 16 or 32 queries, not %d", tile_rows);
  GS_REQUIRE(page_size > 0 && max_blocks > 0 && window >= 0, "attention_prefill: bad page_size/max_blocks/window");
  GS_REQUIRE(q_stride >= nh * d && q_stride % 8 == 0 && ((uintptr_t)q & 15) == 0, "attention_prefill: q rows must be 16-byte aligned");
  GS_REQUIRE(((uintptr_t)kcache & 15) == 0 && ((uintptr_t)vcache & 15) == 0 && ((uintptr_t)out & 7) == 0,
             "attention_prefill: cache and output must be aligned");
  if (ntiles == 0) return 0;
  dim3 grid(ntiles, nkv);
  int rc = -1;
#define GS_ARGS                                                                                                      \
  nh / nkv, grid, stream, (const bf16*)q, q_stride, (const bf16*)kcache, (const bf16*)vcache, positions, tile_seq,  \
      tile_row, tile_n, block_table, max_blocks, page_size, window, scale, (bf16*)out, nh, nkv
  if (tile_rows == 16) {
    switch (d) {
      case 32: rc = launch_prefill<32, 1>(GS_ARGS); break;
      case 64: rc = launch_prefill<64, 1>(GS_ARGS); break;
      case 128: rc = launch_prefill<128, 1>(GS_ARGS); break;
    }
  } else {
    switch (d) {
      case 32: rc = launch_prefill<32, 2>(GS_ARGS); break;
      case 64: rc = launch_prefill<64, 2>(GS_ARGS); break;
      case 128: rc = launch_prefill<128, 2>(GS_ARGS); break;
    }
  }
#undef GS_ARGS
  GS_REQUIRE(rc == 0, "attention_prefill: no kernel for this group size");
  GS_LAUNCH_CHECK("attention_prefill");
  return 0;
}
