// Choosing a token from a row of float32 logits: argmax, temperature sampling by inverse CDF, nucleus sampling.
//
// argmax: ties go to the lowest id; a NaN or infinity anywhere in the row sets the row's flag
// (no token may be emitted from such a row).
// temperature: weights exp((x - max) / T) and their total in float64; the uniform number u in
// [0, 1) comes from the caller (one draw per token); the id returned is the first, in id order,
// whose running sum exceeds u * total.  The weights are made by many blocks a row, each thread the sum of four
// consecutive ids; one block a row then finds where the running sum of those sums crosses the target.
#include "common.h"

#define SAMP_THREADS 1024

// First maximum of one row by the whole block; thread 0 returns (id, bad) through the pointers.
__device__ void row_argmax(const float* __restrict__ x, int V, int* id_out, int* bad_out) {
  __shared__ float bv[SAMP_THREADS / 64];
  __shared__ int bi[SAMP_THREADS / 64];
  __shared__ int bbad;
  if (threadIdx.x == 0) bbad = 0;
  __syncthreads();
  float best = -INFINITY;
  int idx = 0x7fffffff;
  int notfinite = 0;
  // 16-byte loads, eight of them under way at a time (a row of 65,536 logits is then two round trips for the block's
  // 1,024 threads; sixteen need more registers than 1,024 threads leave a lane); ids are visited in ascending order per
  // thread, and a later equal value never replaces an earlier one
  constexpr int AHEAD = 8;
  const int V4 = ((reinterpret_cast<uintptr_t>(x) & 15) == 0) ? (V >> 2) : 0;
  typedef float __attribute__((ext_vector_type(4))) row4_t;   // (a plain vector type: an array of it stays in registers)
  const row4_t* x4 = reinterpret_cast<const row4_t*>(x);
  for (int q0 = threadIdx.x; q0 < V4; q0 += AHEAD * blockDim.x) {
    row4_t v[AHEAD];
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
      int q = q0 + u * blockDim.x;
      v[u] = q < V4 ? x4[q] : row4_t{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
    }
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
      int q = q0 + u * blockDim.x;
      if (q < V4) {            // (no break: the loop must unroll whole, or the loads' array is indexed at run time)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float e = v[u][i];
          if (!(fabsf(e) <= 3.402823466e38f)) notfinite = 1;
          if (e > best) {
            best = e;
            idx = 4 * q + i;
          }
        }
      }
    }
  }
  for (int j = 4 * V4 + threadIdx.x; j < V; j += blockDim.x) {
    float v = x[j];
    if (!(fabsf(v) <= 3.402823466e38f)) notfinite = 1;
    if (v > best || (v == best && j < idx)) {
      best = v;
      idx = j;
    }
  }
  for (int o = 32; o > 0; o >>= 1) {
    float ov = __shfl_xor(best, o, 64);
    int oi = __shfl_xor(idx, o, 64);
    if (ov > best || (ov == best && oi < idx)) {
      best = ov;
      idx = oi;
    }
  }
  if (notfinite) atomicOr(&bbad, 1);
  int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    bv[wave] = best;
    bi[wave] = idx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w)
      if (bv[w] > best || (bv[w] == best && bi[w] < idx)) {
        best = bv[w];
        idx = bi[w];
      }
    *id_out = idx == 0x7fffffff ? 0 : idx;
    *bad_out = bbad;
  }
}

__global__ void argmax_rows_kernel(const float* __restrict__ logits, int V, int* __restrict__ ids,
                                   int* __restrict__ bad) {
  int row = blockIdx.x;
  row_argmax(logits + (size_t)row * V, V, ids + row, bad + row);
}

extern "C" int gs_argmax_rows(const float* logits, int rows, int V, int* ids, int* bad, hipStream_t stream) {
  GS_REQUIRE(rows >= 0 && V > 0, "argmax: bad sizes rows=%d V=%d", rows, V);
  if (rows == 0) return 0;
  argmax_rows_kernel<<<rows, SAMP_THREADS, 0, stream>>>(logits, V, ids, bad);
  GS_LAUNCH_CHECK("argmax_rows");
  return 0;
}

// ------------------------------------------------------------------ nucleus (top-p) sampling
//
// The reference orders ids by weight, descending and stable (ties keep id order), keeps the
// shortest prefix whose mass reaches top_p * total, draws r = u * (mass kept) and returns the
// first id of that order whose running sum exceeds r (src/Inference/sampling.jl:62-73).  No sort
// is needed for that: positive float64 bit patterns order like their values, so a radix descent
// over the pattern (eight passes of one byte, each a histogram of masses) finds the weight at
// which a running sum in that order crosses a target, and the mass above it; ties at that weight
// are then counted off in id order.  Done twice: for the nucleus' edge, and for the draw.
// Sums run in another order than a sequential walk, so results differ from it by rounding only.
//
// The same row, temperature, top_p and draw give the same id in every run: the histogram's masses are summed as
// 64-bit integers (each weight scaled so that the largest weight a pass can meet, times V, still fits), and integer
// addition does not care in which order the threads' atomic adds arrive.  A weight more than about 2^-45 below the
// largest of its pass counts as zero mass there; it keeps its count, and the pass that narrows down to it scales anew.
//
// wbuf (rows, V) float64 is scratch for the weights.

struct Crossing {
  unsigned long long bits;  // pattern of the weight at which the running sum crosses the target
  double above;             // mass of all weights greater than it
  int nlist;                // ids gathered into the caller's list (all whose weight shares the pattern are among them), or -1
};

// strict = 0: first running sum >= target; strict = 1: first running sum > target.
//
// The first passes read the whole row.  Once a pass has narrowed the candidates down to NUC_LIST or fewer (after its
// second byte the weights left lie within a few percent of each other, a handful in a peaked row), their ids and
// their weights' patterns are gathered into lists in LDS (a wavefront takes its places in the lists with one atomic
// add, a lane its place among the wavefront's by counting the lanes before it) and the later passes read only those,
// from LDS; as soon as a pass leaves NUC_DIRECT candidates or fewer under its prefix they are settled at once, a
// candidate to a thread.
#define NUC_LIST 8192
#define NUC_DIRECT 256
//
// ghist, when given: the histograms of the first two bytes, made ahead by many blocks (choose_weights_kernel) with the
// scales that passes 0 and 1 use here: NUC_G0 sums for the first byte (0x3B, standing for everything below 2^-63, to
// 0x3F: a weight is at most 1), then 256 for the second byte under each first byte from 0x3C on; after these
// NUC_GHIST sums the counts, in the same order.  Where the first byte's crossing falls below 2^-63 the passes start
// again and read the row themselves.
#define NUC_G0 8
#define NUC_GHIST (NUC_G0 + 4 * 256)
__device__ Crossing radix_descend(const double* __restrict__ w, int V, double target, int strict,
                                  unsigned long long* hmass, int* hcount, Crossing* shared_out, int* clist,
                                  unsigned long long* lbits, const unsigned long long* __restrict__ ghist = nullptr) {
  __shared__ int cn, picked;
  __shared__ unsigned long long cbits[NUC_DIRECT], cmass[NUC_DIRECT];
  unsigned long long prefix = 0;
  double above = 0.0;
  int lv = 1;                                   // V <= 2^lv
  while ((1 << lv) < V && lv < 30) ++lv;
  int nlist = -1;                               // ids in the list, or -1: no list yet
  for (int pass = 0; pass < 8; ++pass) {
    int shift = 56 - 8 * pass;
    for (int b = threadIdx.x; b < 256; b += blockDim.x) {
      hmass[b] = 0ull;
      hcount[b] = 0;
    }
    __syncthreads();
    unsigned long long himask = pass == 0 ? 0ull : (~0ull) << (shift + 8);
    // the largest weight this pass can meet: 1 (the row's maximum has weight exp(0)) or the largest pattern under the prefix
    const double wmax = pass == 0 ? 1.0 : __longlong_as_double((long long)(prefix | ((1ull << (shift + 8)) - 1ull)));
    const double scale = exp2((double)(62 - lv)) / wmax, unscale = 1.0 / scale;
    // a thread adds up what falls into one bucket in a row before it goes to the histogram: in the first passes (sign,
    // exponent) nearly every weight of the row shares a bucket, and one atomic add per weight on one address would
    // queue up; the sums are integers, so neither this nor the order of the adds changes them
    int run_b = -1, run_n = 0;
    unsigned long long run_m = 0ull;
    const bool ready = ghist != nullptr && pass < 2;
    if (ready && pass == 0) {
      for (int b = threadIdx.x; b < 5; b += blockDim.x) {
        hmass[0x3B + b] = ghist[b];
        hcount[0x3B + b] = (int)ghist[NUC_GHIST + b];
      }
    } else if (ready) {
      const int under = (int)(prefix >> 56) - 0x3C;
      for (int b = threadIdx.x; b < 256; b += blockDim.x) {
        hmass[b] = ghist[NUC_G0 + under * 256 + b];
        hcount[b] = (int)ghist[NUC_GHIST + NUC_G0 + under * 256 + b];
      }
    }
    const int n = ready ? 0 : (nlist >= 0 ? nlist : V);
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
      const unsigned long long bits = nlist >= 0 ? lbits[i] : (unsigned long long)__double_as_longlong(w[i]);
      if ((bits & himask) == prefix) {
        int b = (int)((bits >> shift) & 0xff);
        if (b != run_b) {
          if (run_n) {
            atomicAdd(&hmass[run_b], run_m);
            atomicAdd(&hcount[run_b], run_n);
          }
          run_b = b;
          run_m = 0ull;
          run_n = 0;
        }
        run_m += (unsigned long long)__double2ll_rn(__longlong_as_double((long long)bits) * scale);
        run_n += 1;
      }
    }
    if (run_n) {
      atomicAdd(&hmass[run_b], run_m);
      atomicAdd(&hcount[run_b], run_n);
    }
    __syncthreads();
    // the walk over the buckets, heaviest first, by one wavefront, four buckets a lane: running sums of the masses
    // (integers, exact), each turned into a float64 once; the first bucket whose running sum crosses the target, or
    // the last one that holds anything where rounding left the target just above the whole mass
    if (threadIdx.x < 64) {
      const int lane = threadIdx.x;
      unsigned long long m[4], run[4];
      int c[4];
      unsigned long long mine = 0ull;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int b = 255 - (4 * lane + i);
        m[i] = hmass[b];
        c[i] = hcount[b];
        mine += m[i];
        run[i] = mine;
      }
      unsigned long long incl = mine;                      // running sum over the lanes, this lane included
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const unsigned long long v = __shfl_up(incl, off, 64);
        if (lane >= off) incl += v;
      }
      const unsigned long long before = incl - mine;
      int hit = -1, full = -1;
#pragma unroll
      for (int i = 3; i >= 0; --i) {
        if (c[i] > 0) {
          const double next = above + (double)(before + run[i]) * unscale;
          if (strict ? (target < next) : (next >= target)) hit = i;
          if (full < 0) full = i;
        }
      }
      const unsigned long long hits = __ballot(hit >= 0), fulls = __ballot(full >= 0);
      const int hl = hits ? __ffsll((long long)hits) - 1 : -1;
      const int fl = fulls ? 63 - __clzll((long long)fulls) : -1;
      const int owner = hl >= 0 ? hl : (fl >= 0 ? fl : 63);
      if (lane == owner) {
        const int i = hl >= 0 ? hit : (full >= 0 ? full : 3);
        const int pick = 255 - (4 * lane + i);
        shared_out->bits = prefix | ((unsigned long long)pick << shift);
        shared_out->above = above + (double)(before + run[i] - m[i]) * unscale;
        picked = c[i];
        cn = 0;
      }
    }
    __syncthreads();
    prefix = shared_out->bits;
    above = shared_out->above;
    const int left = picked;
    __syncthreads();
    if (ghist != nullptr && pass == 0 && (prefix >> 56) < 0x3C) {   // below what the ready-made histograms resolve
      ghist = nullptr;
      prefix = 0;
      above = 0.0;
      pass = -1;
      continue;
    }
    if (nlist < 0 && pass >= 1 && pass <= 5 && left <= NUC_LIST) {
      const unsigned long long sofar = (~0ull) << shift;
      const int lane = threadIdx.x & 63;
      // One compute unit pulls a row of 65,536 weights (512 KB) no faster than its loads in flight allow: eight loads
      // a thread are asked for before the first is looked at (a turn of the loop is otherwise a round trip to memory,
      // 64 of them a row; loads of two weights, and sixteen in flight, need more registers than 1,024 threads leave
      // a lane and came out slower: 72 to 80 us against 64 for the step's three kernels on peaked rows).
      constexpr int GATHER = 8;
      for (int j0 = 0; j0 < V; j0 += GATHER * blockDim.x) {   // every thread makes every turn: the wavefront votes
        unsigned long long got[GATHER];
#pragma unroll
        for (int g = 0; g < GATHER; ++g) {
          const int j = j0 + g * blockDim.x + threadIdx.x;
          got[g] = j < V ? (unsigned long long)__double_as_longlong(w[j]) : 0ull;
        }
#pragma unroll
        for (int g = 0; g < GATHER; ++g) {
          const int j = j0 + g * blockDim.x + threadIdx.x;
          const bool take = j < V && (got[g] & sofar) == prefix;
          const unsigned long long votes = __ballot(take);
          if (votes) {
            const int first = __ffsll((long long)votes) - 1;
            int base = 0;
            if (lane == first) base = atomicAdd(&cn, __popcll(votes));
            base = __shfl(base, first, 64);
            if (take) {
              const int at = base + __popcll(votes & ((1ull << lane) - 1ull));
              clist[at] = j;
              lbits[at] = got[g];
            }
          }
        }
      }
      __syncthreads();
      nlist = cn;
      __syncthreads();
    }
    if (nlist >= 0 && left <= NUC_DIRECT && pass < 7) {
      // Few candidates are left under the prefix: no more passes.  They are picked out of the list, a thread to each;
      // each adds up the masses of the candidates heavier than its own and of those as heavy (integers, scaled to the
      // largest weight under the prefix); the pattern at which the running sum crosses the target is the one whose
      // candidates see the target between these two sums.
      const int t = threadIdx.x;
      const unsigned long long sofar = (~0ull) << shift;
      if (t == 0) cn = 0;
      __syncthreads();
      for (int i = t; i < nlist; i += blockDim.x) {
        const unsigned long long bits = lbits[i];
        if ((bits & sofar) == prefix) cbits[atomicAdd(&cn, 1)] = bits;       // as many as the pass counted: `left`
      }
      __syncthreads();
      const int m_ = cn;
      __syncthreads();
      const double top = __longlong_as_double((long long)(prefix | ((1ull << shift) - 1ull)));
      const double sc = exp2((double)(62 - lv)) / top, unsc = 1.0 / sc;
      unsigned long long mybits = 0ull;
      if (t < m_) {
        mybits = cbits[t];
        cmass[t] = (unsigned long long)__double2ll_rn(__longlong_as_double((long long)mybits) * sc);
      }
      if (t == 0) {
        cn = 0x7fffffff;      // the lowest thread at the crossing
        picked = 0x7fffffff;  // the lowest thread with the lightest pattern, should nothing cross
      }
      __syncthreads();
      unsigned long long heavier = 0ull, same = 0ull, lightest = ~0ull;
      for (int j = 0; t < m_ && j < m_; ++j) {
        const unsigned long long b = cbits[j], m = cmass[j];
        heavier += b > mybits ? m : 0ull;
        same += b == mybits ? m : 0ull;
        lightest = b < lightest ? b : lightest;
      }
      if (t < m_) {
        const double lo = above + (double)heavier * unsc, hi = above + (double)(heavier + same) * unsc;
        const bool crossed = strict ? (target < hi && !(target < lo)) : (hi >= target && !(lo >= target));
        if (crossed) atomicMin(&cn, t);
        if (mybits == lightest) atomicMin(&picked, t);
      }
      __syncthreads();
      const int owner = cn != 0x7fffffff ? cn : picked;
      if (t == owner) {
        shared_out->bits = mybits;
        shared_out->above = above + (double)heavier * unsc;
      }
      __syncthreads();
      Crossing c;
      c.bits = shared_out->bits;
      c.above = shared_out->above;
      c.nlist = nlist;
      __syncthreads();
      return c;
    }
  }
  Crossing c;
  c.bits = prefix;
  c.above = above;
  c.nlist = nlist;
  return c;
}

// The draw from the nucleus of a row whose weights w (V float64) and their total are at hand, by the whole block:
// P in (0, 1), u in [0, 1); ghist as in radix_descend.  One thread returns (id, bad) through the pointers (a barrier
// before another thread reads them).
__device__ void row_nucleus_pick(const double* __restrict__ w, int V, double P, double uu, double total,
                                 const unsigned long long* __restrict__ ghist, int* id_out, int* bad_out) {
  __shared__ unsigned long long hmass[256];
  __shared__ int hcount[256];
  __shared__ Crossing cross;
  __shared__ int tie_before[SAMP_THREADS];
  __shared__ int clist[NUC_LIST];
  __shared__ unsigned long long lbits[NUC_LIST];
  __shared__ int ntie;
  const int tid = threadIdx.x;
  // the nucleus' edge: weight tau at which the sorted running sum reaches top_p * total
  double target = P * total;
  Crossing edge = radix_descend(w, V, target, 0, hmass, hcount, &cross, clist, lbits, ghist);
  double tau = __longlong_as_double((long long)edge.bits);
  // ties at tau that belong to the nucleus: added one by one until the sum reaches the target
  double need = target - edge.above;
  long long ties_kept = tau > 0.0 ? (long long)ceil(need / tau) : 1;
  if (ties_kept < 1) ties_kept = 1;
  double cut = edge.above + (double)ties_kept * tau;

  // the draw: first running sum above r = u * cut, in the same order
  double r = uu * cut;
  Crossing hit = radix_descend(w, V, r, 1, hmass, hcount, &cross, clist, lbits, ghist);
  double wv = __longlong_as_double((long long)hit.bits);
  long long k = wv > 0.0 ? (long long)floor((r - hit.above) / wv) : 0;  // 0-based tie in id order
  if (k < 0) k = 0;
  // the k-th id, in id order, whose weight has exactly this pattern (the last such, if k overshoots)
  if (hit.nlist >= 0) {
    // they are all in the list: their ids are picked out of it (as many as there are threads; more than that, a row of
    // a thousand equal weights at the draw, goes the long way below), then a thread to each: its place among them is
    // the number of those with a lower id
    if (tid == 0) ntie = 0;
    __syncthreads();
    for (int i = tid; i < hit.nlist; i += blockDim.x)
      if (lbits[i] == hit.bits) {
        const int at = atomicAdd(&ntie, 1);
        if (at < (int)blockDim.x) tie_before[at] = clist[i];
      }
    __syncthreads();
    const int ties = ntie;
    if (ties == 0) {
      if (tid == 0) {
        *id_out = 0;
        *bad_out = 0;
      }
      return;
    }
    if (ties <= (int)blockDim.x) {
      const long long kk = k < ties ? k : ties - 1;
      if (tid < ties) {
        const int id = tie_before[tid];
        long long lower = 0;
        for (int i = 0; i < ties; ++i) lower += tie_before[i] < id ? 1 : 0;
        if (lower == kk) {
          *id_out = id;
          *bad_out = 0;
        }
      }
      return;
    }
    __syncthreads();
  }
  int per = (V + blockDim.x - 1) / blockDim.x;
  int j0 = tid * per, j1 = j0 + per < V ? j0 + per : V;
  int cnt = 0;
  for (int j = j0; j < j1; ++j) cnt += ((unsigned long long)__double_as_longlong(w[j]) == hit.bits);
  tie_before[tid] = cnt;
  __syncthreads();
  for (int off = 1; off < (int)blockDim.x; off <<= 1) {    // running counts over the threads' ranges, in id order
    const int v = tid >= off ? tie_before[tid - off] : 0;
    __syncthreads();
    tie_before[tid] += v;
    __syncthreads();
  }
  const long long ties = tie_before[blockDim.x - 1];
  if (ties == 0) {
    if (tid == 0) {
      *id_out = 0;
      *bad_out = 0;
    }
    return;
  }
  const long long kk = k < ties ? k : ties - 1;
  const long long before = tie_before[tid] - cnt;
  if (cnt > 0 && before <= kk && kk < before + cnt) {      // the thread whose range holds it walks there
    long long seen = before;
    for (int j = j0; j < j1; ++j)
      if ((unsigned long long)__double_as_longlong(w[j]) == hit.bits) {
        if (seen == kk) {
          *id_out = j;
          *bad_out = 0;
          break;
        }
        ++seen;
      }
  }
}

// The decode loop's choice, made to be recorded into a HIP graph: everything that changes from step to
// step is read from device memory.  This is the form for steps in which every row is greedy, one kernel; rows that
// draw take the three kernels below.  Row r's step is counter[r] (each row counts its own steps, so no block waits for
// another).  The chosen id goes to next_ids[r] (the token fed back) and, with the row's flag, to
// ring[step * rows + r] and bad_ring[...], which the host reads once per run.  Then the row moves on:
// its counter counts up and, if the row is live, so do its position and its number of keys.
__global__ void decode_choose_kernel(const float* __restrict__ logits, int V, int* __restrict__ counter,
                                     int* __restrict__ next_ids, int* __restrict__ ring, int* __restrict__ bad_ring,
                                     int* __restrict__ positions, int* __restrict__ kv_len,
                                     const int* __restrict__ live, int max_steps) {
  __shared__ int sid, sbad;
  int row = blockIdx.x, rows = gridDim.x;
  int step = counter[row];
  // a counter that the host forgot to reset must not write past the rings: such a step goes to the last ring row
  // and marks itself bad, so the run fails loudly instead of overwriting a neighbour
  bool over = step < 0 || step >= max_steps;
  if (over) step = max_steps - 1;
  row_argmax(logits + (size_t)row * V, V, &sid, &sbad);
  if (threadIdx.x == 0) {
    next_ids[row] = sid;
    ring[(size_t)step * rows + row] = sid;
    bad_ring[(size_t)step * rows + row] = over ? 1 : sbad;
    counter[row] = over ? max_steps : step + 1;
    if (live[row]) {
      positions[row] += 1;
      kv_len[row] += 1;
    }
  }
}

extern "C" int gs_decode_choose(const float* logits, int rows, int V, int* counter, int* next_ids, int* ring, int* bad_ring,
                                int* positions, int* kv_len, const int* live, int max_steps, hipStream_t stream) {
  GS_REQUIRE(rows > 0 && V > 0, "decode_choose: bad sizes rows=%d V=%d", rows, V);
  GS_REQUIRE(max_steps > 0, "decode_choose: the rings hold %d steps", max_steps);
  GS_REQUIRE(counter && positions && kv_len && live, "decode_choose: needs the rows' counters, positions, key counts and live flags");
  decode_choose_kernel<<<rows, SAMP_THREADS, 0, stream>>>(logits, V, counter, next_ids, ring, bad_ring, positions, kv_len, live,
                                                          max_steps);
  GS_LAUNCH_CHECK("decode_choose");
  return 0;
}

// ------------------------------------------------------------------ the decode loop's choice when rows draw
//
// One block a row weighs 65,536 logits in float64 in some 40 us (a compute unit's float64 rate), and a step of a few
// rows leaves the rest of the chip idle meanwhile.  So when rows draw, the choice is three kernels: the rows' first
// maxima (and whether they are finite); the weights exp((x - max) / T) by many blocks a row, each thread the sum of
// four consecutive ids; then one block a row that finds where the running sum of those sums, in id order, crosses
// u * total, and walks the four ids there.  Greedy rows take their maximum's id; rows that draw from a nucleus go on
// from the same weights.  part: rows x nparts float64, nparts = gs_choice_parts(V).
#define WIDE_CH 4
#define WIDE_SPAN (SAMP_THREADS * WIDE_CH)

extern "C" int gs_choice_parts(int V) { return ((V + WIDE_SPAN - 1) / WIDE_SPAN) * SAMP_THREADS; }

__global__ void choose_max_kernel(const float* __restrict__ logits, int V, int* __restrict__ ids, int* __restrict__ bad,
                                  unsigned long long* __restrict__ ghist) {
  const int row = blockIdx.x;
  if (ghist)   // sums that the next kernel's blocks add to: they start at zero in every step (a fill by a kernel)
    for (int i = threadIdx.x; i < 2 * NUC_GHIST; i += blockDim.x) ghist[(size_t)row * 2 * NUC_GHIST + i] = 0ull;
  row_argmax(logits + (size_t)row * V, V, ids + row, bad + row);
}

__global__ __launch_bounds__(SAMP_THREADS) void choose_weights_kernel(
    const float* __restrict__ logits, int V, const double* __restrict__ temperature, const double* __restrict__ top_p,
    const int* __restrict__ amax, const int* __restrict__ bad0, double* __restrict__ wbuf, double* __restrict__ part,
    int nparts, unsigned long long* __restrict__ ghist) {
  __shared__ unsigned long long lm[NUC_GHIST];
  __shared__ int lc[NUC_GHIST];
  const int row = blockIdx.y;
  const double T = temperature[row];
  if (!(T > 0.0) || bad0[row]) return;
  const float* x = logits + (size_t)row * V;
  const double hi = (double)x[amax[row]];
  const int j0 = blockIdx.x * WIDE_SPAN + threadIdx.x * WIDE_CH;
  float xv[WIDE_CH];
  if (j0 + WIDE_CH <= V && ((reinterpret_cast<uintptr_t>(x + j0) & 15) == 0)) {
    const float4 v = *reinterpret_cast<const float4*>(x + j0);
    xv[0] = v.x; xv[1] = v.y; xv[2] = v.z; xv[3] = v.w;
  } else {
#pragma unroll
    for (int k = 0; k < WIDE_CH; ++k) xv[k] = j0 + k < V ? x[j0 + k] : -INFINITY;
  }
  double w[WIDE_CH], p = 0.0;
#pragma unroll
  for (int k = 0; k < WIDE_CH; ++k) {
    w[k] = j0 + k < V ? exp(((double)xv[k] - hi) / T) : 0.0;
    p += w[k];
  }
  part[(size_t)row * nparts + blockIdx.x * SAMP_THREADS + threadIdx.x] = p;
  if (wbuf && top_p && top_p[row] < 1.0) {
#pragma unroll
    for (int k = 0; k < WIDE_CH; ++k)
      if (j0 + k < V) wbuf[(size_t)row * V + j0 + k] = w[k];
    if (ghist) {
      // the histograms of the weights' first two bytes, as passes 0 and 1 of radix_descend make them (same scales,
      // integer sums): in LDS for this block's ids, then added to the row's
      for (int i = threadIdx.x; i < NUC_GHIST; i += blockDim.x) {
        lm[i] = 0ull;
        lc[i] = 0;
      }
      __syncthreads();
      int lv = 1;
      while ((1 << lv) < V && lv < 30) ++lv;
      const double scale0 = exp2((double)(62 - lv));
#pragma unroll
      for (int k = 0; k < WIDE_CH; ++k) {
        if (j0 + k >= V) continue;
        const unsigned long long bits = (unsigned long long)__double_as_longlong(w[k]);
        const int b0 = (int)(bits >> 56);
        const int i0 = b0 < 0x3C ? 0 : b0 - 0x3B;
        atomicAdd(&lm[i0], (unsigned long long)__double2ll_rn(w[k] * scale0));
        atomicAdd(&lc[i0], 1);
        if (b0 >= 0x3C) {
          const double wmax = __longlong_as_double((long long)(((unsigned long long)b0 << 56) | ((1ull << 56) - 1ull)));
          const int i1 = NUC_G0 + (b0 - 0x3C) * 256 + (int)((bits >> 48) & 0xff);
          atomicAdd(&lm[i1], (unsigned long long)__double2ll_rn(w[k] * (scale0 / wmax)));
          atomicAdd(&lc[i1], 1);
        }
      }
      __syncthreads();
      unsigned long long* g = ghist + (size_t)row * 2 * NUC_GHIST;
      for (int i = threadIdx.x; i < NUC_GHIST; i += blockDim.x)
        if (lc[i]) {
          atomicAdd(&g[i], lm[i]);
          atomicAdd(&g[NUC_GHIST + i], (unsigned long long)lc[i]);
        }
    }
  }
}

__global__ __launch_bounds__(SAMP_THREADS) void choose_pick_kernel(
    const float* __restrict__ logits, int V, const double* __restrict__ temperature, const double* __restrict__ top_p,
    double* __restrict__ wbuf, const double* __restrict__ part, int nparts, const int* __restrict__ amax,
    const int* __restrict__ bad0, const double* __restrict__ u, int* __restrict__ counter, int* __restrict__ next_ids,
    int* __restrict__ ring, int* __restrict__ bad_ring, int* __restrict__ positions, int* __restrict__ kv_len,
    const int* __restrict__ live, int max_steps, const unsigned long long* __restrict__ ghist) {
  __shared__ int sid, sbad, first_t;
  __shared__ double scan[SAMP_THREADS];
  const int row = blockIdx.x, rows = gridDim.x, tid = threadIdx.x;
  int step = counter[row];
  const bool over = step < 0 || step >= max_steps;
  if (over) step = max_steps - 1;
  const double T = temperature[row];
  const float* x = logits + (size_t)row * V;
  const double P = top_p ? top_p[row] : 1.0;
  const double uu = u[(size_t)step * rows + row];
  if (bad0[row] || !(T > 0.0)) {
    if (tid == 0) {
      sid = bad0[row] ? 0 : amax[row];
      sbad = bad0[row];
    }
  } else {
    const double* pr = part + (size_t)row * nparts;
    const int per = nparts / SAMP_THREADS;
    double ls = 0.0;
    for (int i = 0; i < per; ++i) ls += pr[tid * per + i];
    scan[tid] = ls;
    if (tid == 0) first_t = SAMP_THREADS;
    __syncthreads();
    for (int off = 1; off < SAMP_THREADS; off <<= 1) {     // running sums over the threads, in id order
      const double v = tid >= off ? scan[tid - off] : 0.0;
      __syncthreads();
      scan[tid] += v;
      __syncthreads();
    }
    if (P < 1.0) {
      const double total = scan[SAMP_THREADS - 1];
      __syncthreads();
      row_nucleus_pick(wbuf + (size_t)row * V, V, P, uu, total,
                       ghist ? ghist + (size_t)row * 2 * NUC_GHIST : nullptr, &sid, &sbad);
      goto chosen;
    }
    const double r = uu * scan[SAMP_THREADS - 1];
    if (r < scan[tid]) atomicMin(&first_t, tid);
    __syncthreads();
    const int ft = first_t;
    if (ft == SAMP_THREADS) {
      if (tid == 0) {
        sid = V - 1;
        sbad = 0;
      }
    } else if (tid == ft) {
      const double hi = (double)x[amax[row]];
      double acc = tid ? scan[tid - 1] : 0.0;
      int pick = -1, last = V - 1;
      for (int i = 0; i < per && pick < 0; ++i) {
        const int q = tid * per + i;
        const double pq = pr[q];
        const int j0 = (q / SAMP_THREADS) * WIDE_SPAN + (q % SAMP_THREADS) * WIDE_CH;
        if (j0 >= V) break;
        if (r < acc + pq) {
          double a2 = acc;
          for (int k = 0; k < WIDE_CH && j0 + k < V; ++k) {
            a2 += exp(((double)x[j0 + k] - hi) / T);
            last = j0 + k;
            if (r < a2) {
              pick = j0 + k;
              break;
            }
          }
          if (pick < 0) pick = last;      // the sum of the four, added on its own, lay a rounding above their running sum
        }
        acc += pq;
      }
      sid = pick >= 0 ? pick : V - 1;
      sbad = 0;
    }
  }
chosen:
  __syncthreads();
  if (tid == 0) {
    next_ids[row] = sid;
    ring[(size_t)step * rows + row] = sid;
    bad_ring[(size_t)step * rows + row] = over ? 1 : sbad;
    counter[row] = over ? max_steps : step + 1;
    if (live[row]) {
      positions[row] += 1;
      kv_len[row] += 1;
    }
  }
}

// The decode loop's choice in three kernels, for steps in which rows draw.  Row r: temperature[r] <= 0 greedy, else a
// draw with u[step * rows + r] from the whole row or, with top_p[r] < 1, from its nucleus.  top_p (rows), wbuf
// (rows x V float64, the weights) and hist (rows x gs_choice_hist() 64-bit integers, cleared here in every call) come
// together or not at all (then every draw is from the whole row).  amax, bad0: rows int32 each; part: rows x
// gs_choice_parts(V) float64.
extern "C" int gs_choice_hist() { return 2 * NUC_GHIST; }

extern "C" int gs_decode_choose_wide(const float* logits, int rows, int V, const double* temperature, const double* top_p,
                                     double* wbuf, double* part, int* amax, int* bad0, unsigned long long* hist,
                                     const double* u, int* counter,
                                     int* next_ids, int* ring, int* bad_ring, int* positions, int* kv_len, const int* live,
                                     int max_steps, hipStream_t stream) {
  GS_REQUIRE(rows > 0 && V > 0, "decode_choose: bad sizes rows=%d V=%d", rows, V);
  GS_REQUIRE(max_steps > 0, "decode_choose: the rings hold %d steps", max_steps);
  GS_REQUIRE(counter && positions && kv_len && live && part && amax && bad0,
             "decode_choose: needs the rows' counters, positions, key counts, live flags and scratch");
  GS_REQUIRE((top_p == nullptr) == (wbuf == nullptr), "decode_choose: top_p and its scratch come together");
  GS_REQUIRE(rows <= 65535, "decode_choose: %d rows in one call", rows);
  const int nparts = gs_choice_parts(V);
  GS_REQUIRE(hist != nullptr || top_p == nullptr, "decode_choose: draws from a nucleus need the histograms' room");
  choose_max_kernel<<<rows, SAMP_THREADS, 0, stream>>>(logits, V, amax, bad0, top_p ? hist : nullptr);
  GS_LAUNCH_CHECK("decode_choose (maxima)");
  choose_weights_kernel<<<dim3(nparts / SAMP_THREADS, rows), SAMP_THREADS, 0, stream>>>(
      logits, V, temperature, top_p, amax, bad0, wbuf, part, nparts, top_p ? hist : nullptr);
  GS_LAUNCH_CHECK("decode_choose (weights)");
  choose_pick_kernel<<<rows, SAMP_THREADS, 0, stream>>>(logits, V, temperature, top_p, wbuf, part, nparts, amax, bad0, u,
                                                        counter, next_ids, ring, bad_ring, positions, kv_len, live, max_steps,
                                                        top_p ? hist : nullptr);
  GS_LAUNCH_CHECK("decode_choose (pick)");
  return 0;
}
