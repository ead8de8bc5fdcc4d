// Prompt attention on the matrix cores: many queries per sequence over the paged cache, bfloat16.
//
// A block owns 16 consecutive queries of one sequence and one key head; its G wavefronts are the G query
// heads that share the key head, so keys and values are fetched once per group.  Keys are walked in steps
// of 64 (32 for wide heads) with a running maximum and sum per query (online softmax, float32).
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
#pragma once
#include <type_traits>

#include "attention_prefill_decl.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

#define PF_PAD 4
#define PF_MAXPAGES 2048
#define PF_SLACK 6.0f
#define PF_LOG2E 1.4426950408889634f

// QT: tiles of 16 queries per wavefront; a key fragment and a value fragment feed QT products each.
// KSPLIT: sets of G wavefronts that share a tile's keys between them, step by step in turn, and add up their
// (maximum, sum, accumulator) at the end.  A step is a long chain of dependent instructions for one wavefront;
// the last tiles of a long prompt walk the most keys and set the kernel's time, so their walk is shared out.
template <int D, int G, int QT, int KSPLIT>
__global__ __launch_bounds__(G * KSPLIT * 64) void attention_prefill_kernel(
    const bf16* __restrict__ q, int q_stride, const bf16* __restrict__ kcache, const bf16* __restrict__ vcache,
    const int* __restrict__ positions, const int* __restrict__ tile_seq, const int* __restrict__ tile_row,
    const int* __restrict__ tile_n, const int* __restrict__ block_table, int max_blocks, int page_size,
    unsigned page_magic, int window, float scale, bf16* __restrict__ out, int nh, int nkv) {
  constexpr int PF_KSTEP = D <= 64 ? 64 : 32;   // keys per step: what three sets of row registers allow
  constexpr int KK = D / 32;   // feature steps of the score product
  constexpr int DT = D / 16;   // feature tiles of the output
  constexpr int NB = PF_KSTEP / 16;   // blocks of 16 keys per step
  constexpr int GT = G * 64;       // threads of a set of wavefronts
  __shared__ uint16_t vt[KSPLIT][D][PF_KSTEP + PF_PAD];
  __shared__ int pages[PF_MAXPAGES];
  // Blocks in launch order: key head fastest, tiles from the last one back.  Late tiles walk the most keys, so the
  // longest walks all start first whatever their head; and consecutive blocks go to consecutive dies, so a die sees
  // few key heads and their pages stay in its L2.
  const int kvh = blockIdx.x % nkv, tile = (int)(gridDim.x / nkv) - 1 - (int)(blockIdx.x / nkv);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, kg = lane >> 4;
  const int grp = wave / G, gtid = tid - grp * GT;                 // the set, and the thread within it
  const int h = kvh * G + wave % G;
  const int seq = tile_seq[tile], row0 = tile_row[tile], nq = tile_n[tile];
  const int* bt = block_table + (size_t)seq * max_blocks;
  const int pos0 = positions[row0];                  // positions of a tile are consecutive
  const int last_key = pos0 + nq - 1;
  const int first_key = window > 0 ? (pos0 - window + 1 > 0 ? pos0 - window + 1 : 0) : 0;
  // scores are kept in units of log2(e), so that the exponentials are single v_exp_f32
  const float sc = scale * PF_LOG2E;

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
  // two dependent ones (page number, then row), and the address arithmetic has no branch in it (a branch
  // around a load makes the compiler wait for every load in flight).  The LDS copy holds PF_MAXPAGES pages; a
  // longer key range is walked window by window.  u / page_size is a multiplication: page_magic =
  // floor(2^32 / page_size) + 1 is exact for u page_size < 2^32.
  const int blk0 = (int)__umulhi((unsigned)first_key, page_magic);
  const int blk1 = (int)__umulhi((unsigned)last_key, page_magic);
  int win_blk = blk0, win_first = first_key, win_last = last_key;   // the window's pages and keys
  // Rows outside the window's keys are never seen (their scores are masked): their addresses are clamped
  // into the range, so that every load is of a row the sequence holds and no load needs a branch.
  auto row_of = [&](int u, bool clamp) -> size_t {
    if (clamp) u = u < win_first ? win_first : (u > win_last ? win_last : u);
    const int blk = (int)__umulhi((unsigned)u, page_magic);
    const int offs = u - blk * page_size;
    return (((size_t)pages[blk - win_blk] * nkv + kvh) * page_size + offs) * D;
  };
  // The loads of a step are issued two steps ahead and land in registers while the steps before are computed:
  // three sets of row registers, used in turn (the step loop is unrolled by three, so the turns are static).
  constexpr int VPT = (PF_KSTEP * (D / 8) + GT - 1) / GT;   // value chunks per thread and step
  bf16x8_t kb[3][NB][KK];
  uint4 vb[3][VPT];
  // (steps that lie wholly inside the window's keys need no clamping: `inner`, a compile-time flag)
  auto fetch_as = [&](auto stage, auto inner, int k0) {
    constexpr int S = decltype(stage)::value;
    constexpr bool CLAMP = !decltype(inner)::value;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const bf16* krow = kcache + row_of(k0 + b * 16 + r16, CLAMP) + kg * 8;   // the key whose row this lane loads
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) kb[S][b][kk] = *reinterpret_cast<const bf16x8_t*>(krow + kk * 32);
    }
#pragma unroll
    for (int x = 0; x < VPT; ++x) {
      const int i = (gtid + x * GT) % (PF_KSTEP * (D / 8));
      const int key = i / (D / 8), c = i % (D / 8);
      vb[S][x] = *reinterpret_cast<const uint4*>(vcache + row_of(k0 + key, CLAMP) + c * 8);
    }
  };
  auto fetch = [&](auto stage, int k0) {
    if (k0 >= win_first && k0 + PF_KSTEP - 1 <= win_last) fetch_as(stage, std::true_type{}, k0);
    else fetch_as(stage, std::false_type{}, k0);
  };
  // per query: the last key it sees and the first, relative to this lane's rows of a score tile (4 kg + i)
  int hi[QT], lo[QT];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    hi[t] = live[t] ? my_pos[t] - kg * 4 : -(1 << 30);
    lo[t] = my_lo[t] - kg * 4;
  }

  // A step whose keys every query of the tile sees (`inner`: below the diagonal, inside the windows) needs no
  // masks; most steps are such, and the masks are a third of a step's instructions.
  auto step_as = [&](auto stage, auto inner, int k0) {
    constexpr int S = decltype(stage)::value;
    constexpr bool MASK = !decltype(inner)::value;
    fetch(std::integral_constant<int, (S + 2) % 3>{}, k0 + 2 * KSPLIT * PF_KSTEP);   // beyond the last step the addresses are clamped and the loads are spare
    // stage the step's value rows transposed: thread (key, chunk of 8 features)
    __syncthreads();
#pragma unroll
    for (int x = 0; x < VPT; ++x) {
      const int i = gtid + x * GT;
      if (i < PF_KSTEP * (D / 8)) {
        const int key = i / (D / 8), c = i % (D / 8);
        const uint32_t ww[4] = {vb[S][x].x, vb[S][x].y, vb[S][x].z, vb[S][x].w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          vt[grp][c * 8 + 2 * e][key] = (uint16_t)(ww[e] & 0xffffu);
          vt[grp][c * 8 + 2 * e + 1][key] = (uint16_t)(ww[e] >> 16);
        }
      }
    }
    // scores of NB blocks of 16 keys: S^T = K Q^T; lane holds keys k0 + 16 b + 4 kg + i for its query
    const int whi = win_last - kg * 4, wlo = win_first - kg * 4;   // keys of other windows are theirs to count
    float s[QT][NB * 4];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      f32x4_t st[QT];
#pragma unroll
      for (int t = 0; t < QT; ++t) st[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < KK; ++kk)
#pragma unroll
        for (int t = 0; t < QT; ++t) st[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb[S][b][kk], qf[t][kk], st[t], 0, 0, 0);
#pragma unroll
      for (int t = 0; t < QT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = k0 + b * 16 + i;           // + 4 kg, which hi and lo already hold
          if (MASK) s[t][b * 4 + i] = (key <= hi[t] && key >= lo[t] && key <= whi && key >= wlo) ? st[t][i] : -INFINITY;
          else s[t][b * 4 + i] = st[t][i];
        }
    }
    bf16x8_t pf[QT][NB / 2];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      float mloc = s[t][0];
#pragma unroll
      for (int j = 1; j < NB * 4; ++j) mloc = fmaxf(mloc, s[t][j]);
      mloc = group4_max(mloc) * sc;        // sc > 0: the scaled maximum is the maximum of the scaled scores
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
      const bool none = MASK && m[t] == -INFINITY;    // nothing seen yet: every key so far was masked
      const float nm = none ? 0.f : -m[t];
      float lsum = 0.f;
#pragma unroll
      for (int j = 0; j < NB * 4; ++j) {
        const float pj = none ? 0.f : __builtin_amdgcn_exp2f(fmaf(s[t][j], sc, nm));
        lsum += pj;
        pf[t][j / 8][j % 8] = (__bf16)pj;
      }
      l[t] += group4_sum(lsum);
    }
    __syncthreads();   // the staged values are in place
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int ns = 0; ns < NB / 2; ++ns) {
        // A = V^T tile: lane (feature 16 dt + r16, key slots 8 kg + j <-> block 2 ns + j / 4, key 4 kg + j % 4)
        union {
          bf16x8_t v;
          uint2 u2[2];
        } a;
        a.u2[0] = *reinterpret_cast<const uint2*>(&vt[grp][dt * 16 + r16][ns * 32 + kg * 4]);
        a.u2[1] = *reinterpret_cast<const uint2*>(&vt[grp][dt * 16 + r16][ns * 32 + 16 + kg * 4]);
#pragma unroll
        for (int t = 0; t < QT; ++t) acc[t][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, pf[t][ns], acc[t][dt], 0, 0, 0);
      }
  };
  const int last_lo = window > 0 ? (last_key - window + 1 > 0 ? last_key - window + 1 : 0) : 0;
  auto step = [&](auto stage, int k0) {
    const bool inner = k0 + PF_KSTEP - 1 <= pos0 && k0 >= last_lo && k0 >= win_first && k0 + PF_KSTEP - 1 <= win_last &&
                       nq == 16 * QT;
    if (inner) step_as(stage, std::true_type{}, k0);
    else step_as(stage, std::false_type{}, k0);
  };

  for (win_blk = blk0; win_blk <= blk1; win_blk += PF_MAXPAGES) {
    const int wend = win_blk + PF_MAXPAGES - 1 < blk1 ? win_blk + PF_MAXPAGES - 1 : blk1;
    __syncthreads();                 // nobody reads the previous window any more
    for (int i = tid; i <= wend - win_blk; i += GT * KSPLIT) pages[i] = bt[win_blk + i];
    __syncthreads();
    win_first = win_blk * page_size > first_key ? win_blk * page_size : first_key;
    win_last = (wend + 1) * page_size - 1 < last_key ? (wend + 1) * page_size - 1 : last_key;
    // the sets take the steps in turn; all make the same number of steps (the barriers are the block's), a set
    // whose step lies beyond the keys computes on masked scores
    const int kstart = (win_first / PF_KSTEP) * PF_KSTEP + grp * PF_KSTEP;
    constexpr int STRIDE = KSPLIT * PF_KSTEP;
    fetch(std::integral_constant<int, 0>{}, kstart);
    fetch(std::integral_constant<int, 1>{}, kstart + STRIDE);
    for (int k0 = kstart; k0 - grp * PF_KSTEP <= win_last; k0 += 3 * STRIDE) {
      step(std::integral_constant<int, 0>{}, k0);
      if (k0 - grp * PF_KSTEP + STRIDE > win_last) break;
      step(std::integral_constant<int, 1>{}, k0 + STRIDE);
      if (k0 - grp * PF_KSTEP + 2 * STRIDE > win_last) break;
      step(std::integral_constant<int, 2>{}, k0 + 2 * STRIDE);
    }
  }
  if (KSPLIT > 1) {
    // add up the sets, in set order: set 0 takes the others' (reference point, sum, accumulator) through LDS,
    // one tile of queries at a time
    __shared__ float mrg[KSPLIT > 1 ? KSPLIT - 1 : 1][KSPLIT > 1 ? GT : 1][DT * 4 + 2];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      __syncthreads();
      if (grp > 0) {
        float* dst = mrg[grp - 1][gtid];
        dst[0] = m[t];
        dst[1] = l[t];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int i = 0; i < 4; ++i) dst[2 + dt * 4 + i] = acc[t][dt][i];
      }
      __syncthreads();
      if (grp == 0) {
#pragma unroll
        for (int g2 = 0; g2 < KSPLIT - 1; ++g2) {
          const float* src = mrg[g2][gtid];
          const float m2 = src[0];
          if (m2 > -INFINITY) {
            const float mm = fmaxf(m[t], m2);
            const float a1 = m[t] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m[t] - mm);
            const float a2 = __builtin_amdgcn_exp2f(m2 - mm);
            l[t] = l[t] * a1 + src[1] * a2;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
              for (int i = 0; i < 4; ++i) acc[t][dt][i] = acc[t][dt][i] * a1 + src[2 + dt * 4 + i] * a2;
            m[t] = mm;
          }
        }
      }
    }
    if (grp > 0) return;
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

template <int D, int QT, int KSPLIT>
static int launch_prefill(int G, dim3 grid, hipStream_t stream, const bf16* q, int q_stride, const bf16* kc,
                          const bf16* vc, const int* positions, const int* tile_seq, const int* tile_row,
                          const int* tile_n, const int* bt, int max_blocks, int page_size, unsigned page_magic,
                          int window, float scale, bf16* out, int nh, int nkv) {
#define GS_RUN(GG)                                                                                                   \
  if constexpr (KSPLIT > 1 && GG > 4) return -1;                                                                        \
  else attention_prefill_kernel<D, GG, QT, KSPLIT><<<grid, GG * KSPLIT * 64, 0, stream>>>(q, q_stride, kc, vc, positions, tile_seq, tile_row, \
                                                                tile_n, bt, max_blocks, page_size, page_magic, window, \
                                                                scale, out, nh, nkv)
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



// All the kernels of one head width (a translation unit each, so that they compile side by side).
template <int D>
static int prefill_for_width(const PrefillCall& c) {
  dim3 grid((unsigned)c.ntiles * (unsigned)c.nkv);
  const int G = c.nh / c.nkv;
  // groups of up to four heads share a tile's keys between two sets of wavefronts
  const bool split = G <= 4;
#define GS_ARGS                                                                                                    \
  G, grid, c.stream, c.q, c.q_stride, c.kc, c.vc, c.positions, c.tile_seq, c.tile_row, c.tile_n, c.bt, c.max_blocks, \
      c.page_size, c.page_magic, c.window, c.scale, c.out, c.nh, c.nkv
  if (c.tile_rows == 16) return split ? launch_prefill<D, 1, 2>(GS_ARGS) : launch_prefill<D, 1, 1>(GS_ARGS);
  return split ? launch_prefill<D, 2, 2>(GS_ARGS) : launch_prefill<D, 2, 1>(GS_ARGS);
#undef GS_ARGS
}
