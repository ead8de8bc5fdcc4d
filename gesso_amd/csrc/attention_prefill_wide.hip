// Prompt attention for long portions: 32 queries a wavefront, keys and values shared by a block through LDS.
//
// The kernel of attention_prefill_impl.h gives a wavefront 16 or 32 queries, loads keys straight into registers
// and meets at two barriers per 64 keys; its wavefronts move in step, so the matrix cores wait while the softmax's
// arithmetic runs and the other way round.  Here a block's wavefronts meet once per 64 keys, keys and values are
// staged once for all of them, and their rows are asked for two steps before they are used:
//
//   * A block owns one key head and WQ sub-tiles of up to 32 consecutive queries of one sequence; wavefront w takes
//     query head w % G of the group and sub-tile w / G.  (WQ = 8, 4, 2, 2, 1 for groups of 1, 2, 3, 4 and more
//     heads: up to eight wavefronts share what is staged.)  The sub-tiles of a block need not be neighbours: for a
//     causal prompt the host gives a block late sub-tiles together with early ones (the first half of its entries
//     the late ones, the second half their partners, so that the two wavefronts that share a SIMD are one of each),
//     and every block then walks about as many steps, its wavefronts taken together; with consecutive sub-tiles the
//     blocks of a prompt of 2,048 tokens walk 1 to 32 steps and the launch takes as long as the longest.
//   * Keys are walked in steps of 64.  A step's key rows (as they lie in the pages) and value rows (transposed:
//     features x keys) are staged in LDS, two buffers: the loads of step s + 1 are issued before step s is
//     computed and written to the other buffer after it; one barrier a step.  Where each key's row starts in the
//     caches (a division by the page size, a look into the block table, a product) is worked out once per key and
//     block, by one wavefront, three steps ahead, and lies in LDS: a thread that loads a row reads one word.
//   * v_mfma_f32_32x32x16_bf16, both products transposed so that everything a lane holds concerns one query
//     (lane % 32):  S^T = K Q^T  (A: 32 keys x 16 features from LDS, B: the query fragment, in registers; the
//     lane gets keys 8 (i / 4) + 4 (lane / 32) + i % 4, i = 0 .. 15, of each 32-key half),  O^T = V^T P^T  (A: 32
//     features x 16 keys from the transposed values in LDS, B: the lane's own probabilities as they are).  No
//     probability crosses lanes; the maximum and the sum of a row are exchanged between lanes l and l ^ 32.
//   * Online softmax in float32, base-2 exponentials of scores scaled by log2 e; the reference point moves only
//     when the maximum has grown by more than 2^6 (see attention_prefill_impl.h).  Steps that every query of the
//     wavefront sees whole carry no masks.
//
//   * Short prompts (fewer blocks than compute units): KS = 2 halves the longest walk.  The block's sub-tiles are
//     then WQ / 2, each held by two wavefronts per head; the first walks the first half of the block's steps, the
//     second the second half, both halves' keys and values staged side by side, and at the end the second hands its
//     maximum, sum and accumulator to the first through LDS (the usual merge of two softmax parts).
//
// Bank conflicts: key rows are 16 bytes longer than the head; the transposed values put key k of feature f at
// column k ^ 8 ((f / 8) % 8), which spreads the sixteen-byte chunks that one wavefront writes (eight features of two
// keys a lane) over all banks and keeps every group of four keys that a product reads in one piece.
//
// Causal rule, window, tiles, q, caches and out as in attention_prefill_impl.h.  Heads 64 wide.
#include <type_traits>

#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 pw_bf16x8_t;
typedef __attribute__((ext_vector_type(16))) float pw_f32x16_t;
typedef __attribute__((ext_vector_type(4))) uint32_t pw_u32x4_t;   // (a plain vector type: arrays of it stay in registers)

#define PW_KS 64
#define PW_SLACK 6.0f
#define PW_LOG2E 1.4426950408889634f

// maximum and sum over the lanes l and l ^ 32, by a row swap (a VALU move, no trip through LDS)
__device__ __forceinline__ float pair_max(float x) {
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float pair_sum(float x) {
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

template <int D, int G, int WQ, int KS>
__global__ __launch_bounds__(G * WQ * 64) void attention_prefill_wide_kernel(
    const bf16* __restrict__ q, int q_stride, const bf16* __restrict__ kcache, const bf16* __restrict__ vcache,
    const int* __restrict__ positions, const int* __restrict__ tile_seq, const int* __restrict__ tile_row,
    const int* __restrict__ tile_n, const int* __restrict__ block_table, int max_blocks, int page_size,
    unsigned page_magic, int window, float scale, bf16* __restrict__ out, int nh, int nkv) {
  constexpr int NT = G * WQ * 64;
  constexpr int KK = D / 16;                  // feature steps of a score product
  constexpr int FT = D / 32;                  // feature tiles of the output
  constexpr int DC = D / 8;                   // 16-byte chunks of a row
  constexpr int KROW = D + 8, VROW = PW_KS + 4;
  constexpr int SUBS = WQ / KS;               // sub-tiles of queries a block
  constexpr int NKC1 = PW_KS * DC, NKC = KS * NKC1;             // key chunks of a step (of one half, of all)
  constexpr int NVU1 = (PW_KS / 2) * DC, NVU = KS * NVU1;       // value units of a step: two keys x one chunk
  constexpr int CK = (NKC + NT - 1) / NT, CV = (NVU + NT - 1) / NT;
  static_assert(D == 64, "the swizzle of the transposed values is written for heads of 64");
  static_assert((KS == 1 || KS == 2) && WQ % KS == 0, "the keys of a block are walked whole or in two halves");
  __shared__ __align__(16) uint16_t ks[KS][2][PW_KS][KROW];
  __shared__ __align__(16) uint16_t vt[KS][2][D][VROW];
  __shared__ __align__(8) uint32_t rowoff[KS][3][PW_KS];   // (read two at a time) where a step's key rows start in the caches, in units of 16 bytes

  // blocks in launch order: key head fastest, tiles from the last one back (late tiles walk the most keys).  Blocks go to
  // the eight XCDs in turn, so with 1, 2, 4 or 8 key heads all blocks of one key head run on the same XCDs and meet their
  // keys and values in those XCDs' L2 (block b: key head b % nkv, XCD b % 8)
  const int kvh = blockIdx.x % nkv, tile = (int)(gridDim.x / nkv) - 1 - (int)(blockIdx.x / nkv);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hf = lane >> 5;
  const int h = kvh * G + wave % G, qsub = (wave / G) / KS, kh = (wave / G) % KS;
  // A block's SUBS sub-tiles of up to 32 queries each are entries tile * SUBS .. + SUBS - 1 of the three lists (sequence,
  // first row, count; a count of 0: no such sub-tile).  They belong to one sequence and need not be neighbours: the
  // host pairs a late sub-tile, which sees many keys, with an early one, which sees few, so that every block of a
  // causal prompt walks about as many steps for its wavefronts taken together (a wavefront sits out the steps its
  // queries see nothing of).  The block walks from the first key any of them sees to the last.
  const int seq = tile_seq[tile * SUBS];
  const int* bt = block_table + (size_t)seq * max_blocks;
  int last_key = 0, first_key = 0x7fffffff;
#pragma unroll
  for (int j = 0; j < SUBS; ++j) {
    const int n = tile_n[tile * SUBS + j];
    const int p0 = positions[tile_row[tile * SUBS + j]];          // (an absent sub-tile names a valid row)
    const int lo = window > 0 ? (p0 - window + 1 > 0 ? p0 - window + 1 : 0) : 0;
    if (n > 0) {
      last_key = p0 + n - 1 > last_key ? p0 + n - 1 : last_key;
      first_key = lo < first_key ? lo : first_key;
    }
  }
  if (first_key > last_key) return;                               // a block without queries (the same for all its threads)
  const int kbeg = (first_key / PW_KS) * PW_KS;
  const int nsteps_all = (last_key - kbeg) / PW_KS + 1;
  const int nsteps = (nsteps_all + KS - 1) / KS;                  // steps of the walk: half h takes steps h nsteps .. of the keys
  const float sc = scale * PW_LOG2E;

  // this wavefront's queries
  const int nqs = tile_n[tile * SUBS + qsub];
  const bool has_rows = nqs > 0;
  const int r0 = tile_row[tile * SUBS + qsub];
  const int pfirst = positions[r0], plast = pfirst + (has_rows ? nqs : 1) - 1;   // positions of a sub-tile are consecutive
  const bool live = l32 < nqs;
  const int my_pos = pfirst + (live ? l32 : (has_rows ? nqs - 1 : 0));
  const int my_lo = window > 0 ? (my_pos - window + 1 > 0 ? my_pos - window + 1 : 0) : 0;
  pw_bf16x8_t qf[KK];
  {
    const bf16* qrow = q + (size_t)(has_rows ? r0 + (live ? l32 : nqs - 1) : r0) * q_stride + (size_t)h * D + hf * 8;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) qf[kk] = *reinterpret_cast<const pw_bf16x8_t*>(qrow + kk * 16);
  }
  float m = -INFINITY, l = 0.f;
  pw_f32x16_t acc[FT];
#pragma unroll
  for (int ft = 0; ft < FT; ++ft)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[ft][e] = 0.f;

  // ---- staging: row starts of a step into rowoff, rows of a step into registers, registers into LDS
  // Key u of step s is looked up by thread u - (first key of the step) of the first wavefront: its page is loaded
  // early (page_of), its row start put into LDS late (put_rows).  u is clamped to the keys of this tile: rows
  // beyond are masked, and every load is of a row the sequence holds.
  // (thread t < 64 KS looks up key t % 64 of half t / 64)
  auto key_of = [&](int s) -> int {
    const int u = kbeg + ((tid / PW_KS) * nsteps + s) * PW_KS + tid % PW_KS;
    return u < first_key ? first_key : (u > last_key ? last_key : u);
  };
  auto page_of = [&](int s) -> int {
    if (tid >= KS * PW_KS) return 0;
    return bt[(int)__umulhi((unsigned)key_of(s), page_magic)];
  };
  auto put_rows = [&](int s, int page) {
    if (tid < KS * PW_KS) {
      const int u = key_of(s);
      const int offs = u - (int)__umulhi((unsigned)u, page_magic) * page_size;
      rowoff[tid / PW_KS][s % 3][tid % PW_KS] =
          (((uint32_t)page * (uint32_t)nkv + (uint32_t)kvh) * (uint32_t)page_size + (uint32_t)offs) * DC;
    }
  };
  const pw_u32x4_t* k16 = reinterpret_cast<const pw_u32x4_t*>(kcache);
  const pw_u32x4_t* v16 = reinterpret_cast<const pw_u32x4_t*>(vcache);
  // two sets of row registers: the rows of step s + 2 are asked for while step s is computed, so that a block
  // alone on its compute unit (a prompt of a few thousand tokens: one block a unit, or two) does not wait a memory
  // round trip in every step
  pw_u32x4_t kreg[2][CK], vreg[2][CV][2];
  // (as macros: arrays that closures take by reference are not always kept in registers)
#define PW_ISSUE(s, S)                                                                                                  \
  {                                                                                                                     \
    _Pragma("unroll") for (int x = 0; x < CK; ++x) {                                                                    \
      /* a thread past the step's last chunk loads the last one again: every register is written, none is stored */     \
      const int i = (NKC % NT == 0 || tid + x * NT < NKC) ? tid + x * NT : NKC - 1;                                     \
      kreg[S][x] = k16[(size_t)rowoff[i / NKC1][(s) % 3][(i % NKC1) / DC] + (i % DC)];                                  \
    }                                                                                                                   \
    _Pragma("unroll") for (int x = 0; x < CV; ++x) {                                                                    \
      const int i = (NVU % NT == 0 || tid + x * NT < NVU) ? tid + x * NT : NVU - 1;                                     \
      const int kp = (i % NVU1) / DC, c = i % DC;                                                                       \
      const uint2 two = *reinterpret_cast<const uint2*>(&rowoff[i / NVU1][(s) % 3][2 * kp]);                            \
      vreg[S][x][0] = v16[(size_t)two.x + c];                                                                           \
      vreg[S][x][1] = v16[(size_t)two.y + c];                                                                           \
    }                                                                                                                   \
  }
#define PW_STASH(buf, S)                                                                                                \
  {                                                                                                                     \
    _Pragma("unroll") for (int x = 0; x < CK; ++x) {                                                                    \
      const int i = tid + x * NT;                                                                                       \
      if (NKC % NT == 0 || i < NKC)                                                                                     \
        *reinterpret_cast<pw_u32x4_t*>(&ks[i / NKC1][buf][(i % NKC1) / DC][(i % DC) * 8]) = kreg[S][x];                 \
    }                                                                                                                   \
    _Pragma("unroll") for (int x = 0; x < CV; ++x) {                                                                    \
      const int i = tid + x * NT;                                                                                       \
      if (NVU % NT == 0 || i < NVU) {                                                                                   \
        const int kp = (i % NVU1) / DC, c = i % DC, hv = i / NVU1;                                                      \
        const int col = (2 * kp) ^ (8 * (c & 7));         /* features 8 c .. 8 c + 7 share the swizzle */               \
        const pw_u32x4_t a = vreg[S][x][0], b = vreg[S][x][1];                                                          \
        _Pragma("unroll") for (int e = 0; e < 4; ++e) {                                                                 \
          *reinterpret_cast<uint32_t*>(&vt[hv][buf][c * 8 + 2 * e][col]) = (a[e] & 0xffffu) | (b[e] << 16);             \
          *reinterpret_cast<uint32_t*>(&vt[hv][buf][c * 8 + 2 * e + 1][col]) = (a[e] >> 16) | (b[e] & 0xffff0000u);     \
        }                                                                                                               \
      }                                                                                                                 \
    }                                                                                                                   \
  }

  // ---- one step of this wavefront's queries over the 64 keys of its half in buffer `buf`
  auto compute = [&](int buf, int k0, auto masked) {
    constexpr bool MASK = decltype(masked)::value;
    pw_f32x16_t st[2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
      for (int e = 0; e < 16; ++e) st[kt][e] = 0.f;
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        const pw_bf16x8_t a = *reinterpret_cast<const pw_bf16x8_t*>(&ks[kh][buf][kt * 32 + l32][kk * 16 + hf * 8]);
        st[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[kk], st[kt], 0, 0, 0);
      }
    }
    if (MASK) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int key = k0 + kt * 32 + 8 * (e >> 2) + 4 * hf + (e & 3);
          if (key > my_pos || key < my_lo) st[kt][e] = -INFINITY;
        }
    }
    float mloc = st[0][0];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int e = 0; e < 16; ++e) mloc = fmaxf(mloc, st[kt][e]);
    mloc = pair_max(mloc) * sc;                 // sc > 0: the scaled maximum is the maximum of the scaled scores
    if (mloc > m + PW_SLACK || m == -INFINITY) {
      if (mloc > -INFINITY) {
        const float a = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - mloc);
        l *= a;
#pragma unroll
        for (int ft = 0; ft < FT; ++ft)
#pragma unroll
          for (int e = 0; e < 16; ++e) acc[ft][e] *= a;
        m = mloc;
      }
    }
    const bool none = MASK && m == -INFINITY;   // nothing seen yet: every key so far was masked
    const float nm = none ? 0.f : -m;
    float lsum = 0.f;
    pw_bf16x8_t pf[4];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float pj = none ? 0.f : __builtin_amdgcn_exp2f(fmaf(st[kt][e], sc, nm));
        lsum += pj;
        pf[kt * 2 + (e >> 3)][e & 7] = (__bf16)pj;
      }
    l += pair_sum(lsum);
    // O^T += V^T P^T: chunk c holds, for the lanes of half hf, the keys kb .. kb + 3 and kb + 8 .. kb + 11
#pragma unroll
    for (int ft = 0; ft < FT; ++ft) {
      const int f = ft * 32 + l32;
      const int swz = 8 * ((f >> 3) & 7);
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int kb = (c >> 1) * 32 + (c & 1) * 16 + hf * 4;
        union {
          pw_bf16x8_t v;
          uint2 u2[2];
        } a;
        a.u2[0] = *reinterpret_cast<const uint2*>(&vt[kh][buf][f][kb ^ swz]);
        a.u2[1] = *reinterpret_cast<const uint2*>(&vt[kh][buf][f][(kb + 8) ^ swz]);
        acc[ft] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, pf[c], acc[ft], 0, 0, 0);
      }
    }
  };

  put_rows(0, page_of(0));
  if (nsteps > 1) put_rows(1, page_of(1));
  if (nsteps > 2) put_rows(2, page_of(2));
  __syncthreads();
  PW_ISSUE(0, 0);
  PW_STASH(0, 0);
  if (nsteps > 1) PW_ISSUE(1, 1);
  __syncthreads();
  // step s: the rows of step s + 2 are asked for into the set that step s's rows have left, step s is computed, the
  // rows of step s + 1 (asked for a step ago) go into the other buffer
#define PW_STEP(s, MINE, NEXT)                                                                                        \
  {                                                                                                                     \
    const int k0 = kbeg + (kh * nsteps + (s)) * PW_KS;                                                                  \
    const int page_ahead = (s) + 3 < nsteps ? page_of((s) + 3) : 0;                                                     \
    if ((s) + 2 < nsteps) PW_ISSUE((s) + 2, MINE);                                                                     \
    /* the wavefront computes where its queries see any of the step's keys */                                           \
    if (has_rows && k0 <= plast && (window == 0 || k0 + PW_KS - 1 >= pfirst - window + 1)) {                            \
      const bool inner = k0 + PW_KS - 1 <= pfirst && (window == 0 || k0 >= plast - window + 1);                         \
      if (inner) compute((s) & 1, k0, std::false_type{});                                                               \
      else compute((s) & 1, k0, std::true_type{});                                                                      \
    }                                                                                                                   \
    if ((s) + 1 < nsteps) PW_STASH(((s) + 1) & 1, NEXT);                                                                 \
    if ((s) + 3 < nsteps) put_rows((s) + 3, page_ahead);   /* rowoff[s % 3] was last read when step s was issued */     \
    __syncthreads();                                                                                                    \
  }
  for (int s = 0; s < nsteps; s += 2) {
    PW_STEP(s, 0, 1);
    if (s + 1 < nsteps) PW_STEP(s + 1, 1, 0);
  }
#undef PW_STEP
#undef PW_ISSUE
#undef PW_STASH

  if (KS > 1) {
    // the second half's wavefront hands over what it has; the first merges: both parts' weights are relative to a
    // reference of their own, the common one is the larger
    float* hand = reinterpret_cast<float*>(&ks[0][0][0][0]) + (size_t)(qsub * G + wave % G) * (FT * 16 + 2) * 64 + lane;
    static_assert(KS == 1 || (size_t)G * SUBS * (FT * 16 + 2) * 64 * sizeof(float) <= sizeof(ks), "the hand-over fits where the keys were staged");
    if (kh == 1) {
#pragma unroll
      for (int ft = 0; ft < FT; ++ft)
#pragma unroll
        for (int e = 0; e < 16; ++e) hand[(ft * 16 + e) * 64] = acc[ft][e];
      hand[FT * 16 * 64] = m;
      hand[(FT * 16 + 1) * 64] = l;
    }
    __syncthreads();
    if (kh == 1) return;
    const float m1 = hand[FT * 16 * 64], l1 = hand[(FT * 16 + 1) * 64];
    const float mm = fmaxf(m, m1);
    const float a0 = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - mm);
    const float a1 = m1 == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m1 - mm);
    l = l * a0 + l1 * a1;
#pragma unroll
    for (int ft = 0; ft < FT; ++ft)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[ft][e] = acc[ft][e] * a0 + hand[(ft * 16 + e) * 64] * a1;
  }
  if (!live) return;
  const float inv = 1.0f / l;
  bf16* orow = out + (size_t)(r0 + l32) * nh * D + (size_t)h * D;
#pragma unroll
  for (int ft = 0; ft < FT; ++ft)
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      uint2 o;
      o.x = (uint32_t)f32_to_bf16(acc[ft][g4 * 4 + 0] * inv).x | ((uint32_t)f32_to_bf16(acc[ft][g4 * 4 + 1] * inv).x << 16);
      o.y = (uint32_t)f32_to_bf16(acc[ft][g4 * 4 + 2] * inv).x | ((uint32_t)f32_to_bf16(acc[ft][g4 * 4 + 3] * inv).x << 16);
      *reinterpret_cast<uint2*>(orow + ft * 32 + g4 * 8 + hf * 4) = o;
    }
}

// Queries a block of this kernel holds for a group of g query heads to a key head when it walks the keys whole: 32 per
// wavefront, and as many wavefronts per head as make eight to a block.  (Blocks of four wavefronts, twice as many, were
// measured too: 61.5 against 58.0 us at 2,048 tokens, 970 against 776 us over a prefix of 30,720.)
static int wide_rows(int g) {
  const int wq = g == 1 ? 8 : (g == 2 ? 4 : (g <= 4 ? 2 : 1));
  return 32 * wq;
}

extern "C" int gs_attention_prefill_wide_supports(int nh, int nkv, int d) {
  if (nkv <= 0 || nh % nkv) return 0;
  const int g = nh / nkv;
  return d == 64 && g >= 1 && g <= 8;
}

// The most queries a block may hold: 32 for each of its sub-tiles.
extern "C" int gs_attention_prefill_wide_rows(int nh, int nkv) { return nkv > 0 ? wide_rows(nh / nkv) : 0; }

extern "C" int gs_attention_prefill_wide(const void* q, int q_stride, const void* kcache, const void* vcache,
                                         const int* positions, const int* tile_seq, const int* tile_row,
                                         const int* tile_n, int ntiles /* blocks: tile_rows / 32 entries of the three lists each */,
                                         const int* block_table, int max_blocks,
                                         int page_size, long cache_pages, int window, float scale, void* out, int nh,
                                         int nkv, int d, int tile_rows, int key_splits, hipStream_t stream) {
  GS_REQUIRE(gs_attention_prefill_wide_supports(nh, nkv, d), "attention_prefill_wide: sizes nh=%d nkv=%d d=%d are not taken", nh, nkv, d);
  const int G = nh / nkv;
  GS_REQUIRE(key_splits == 1 || (key_splits == 2 && wide_rows(G) >= 64),
             "attention_prefill_wide: the keys are walked whole or, for groups of up to 4 heads, in two halves, not in %d parts", key_splits);
  GS_REQUIRE(tile_rows * key_splits == wide_rows(G),
             "attention_prefill_wide: blocks of a group of %d heads hold up to %d queries (%d with the keys in two halves), not %d",
             G, wide_rows(G), wide_rows(G) / 2, tile_rows);
  GS_REQUIRE(ntiles >= 0 && (long)ntiles * nkv < (1L << 31), "attention_prefill_wide: %d tiles x %d key heads are too many blocks", ntiles, nkv);
  GS_REQUIRE(page_size > 0 && max_blocks > 0 && window >= 0, "attention_prefill_wide: bad page_size/max_blocks/window");
  GS_REQUIRE(q_stride >= nh * d && q_stride % 8 == 0 && ((uintptr_t)q & 15) == 0, "attention_prefill_wide: q rows must be 16-byte aligned");
  GS_REQUIRE(((uintptr_t)kcache & 15) == 0 && ((uintptr_t)vcache & 15) == 0 && ((uintptr_t)out & 7) == 0,
             "attention_prefill_wide: cache and output must be aligned");
  GS_REQUIRE(page_size >= 2 && (long)max_blocks * page_size * page_size < (1L << 32),
             "attention_prefill_wide: page_size %d with %d blocks a sequence is outside what the kernel's division takes", page_size, max_blocks);
  // row starts are kept as 32-bit counts of 16 bytes
  GS_REQUIRE(cache_pages > 0 && (double)cache_pages * nkv * page_size * (d / 8) < 4294967296.0,
             "attention_prefill_wide: a cache of %ld pages is beyond the 64 GB a layer that the kernel's row index takes", cache_pages);
  if (ntiles == 0) return 0;
  const unsigned page_magic = (unsigned)((1ull << 32) / (unsigned)page_size + 1);
  dim3 grid((unsigned)ntiles * (unsigned)nkv);
#define GS_RUN2(GG, WQ, KS)                                                                                           \
  attention_prefill_wide_kernel<64, GG, WQ, KS><<<grid, GG * WQ * 64, 0, stream>>>(                                   \
      (const bf16*)q, q_stride, (const bf16*)kcache, (const bf16*)vcache, positions, tile_seq, tile_row, tile_n,       \
      block_table, max_blocks, page_size, page_magic, window, scale, (bf16*)out, nh, nkv)
#define GS_RUN(GG, WQ) { if (key_splits == 2) GS_RUN2(GG, WQ, 2); else GS_RUN2(GG, WQ, 1); }
  switch (G) {
    case 1: GS_RUN(1, 8) break;
    case 2: GS_RUN(2, 4) break;
    case 3: GS_RUN(3, 2) break;
    case 4: GS_RUN(4, 2) break;
    case 5: GS_RUN2(5, 1, 1); break;
    case 6: GS_RUN2(6, 1, 1); break;
    case 7: GS_RUN2(7, 1, 1); break;
    default: GS_RUN2(8, 1, 1); break;
  }
#undef GS_RUN
#undef GS_RUN2
  GS_LAUNCH_CHECK("attention_prefill_wide");
  return 0;
}
