// Choosing a token from a row of float32 logits: argmax, and temperature sampling by inverse CDF.
//
// argmax: ties go to the lowest id; a NaN or infinity anywhere in the row sets the row's flag
// (no token may be emitted from such a row).
// temperature: weights exp((x - max) / T) and their total in float64; the uniform number u in
// [0, 1) comes from the caller (one draw per token); the id returned is the first, in id order,
// whose running sum exceeds u * total.  Each thread owns a contiguous range of ids, so the walk
// is in id order: ranges are summed, scanned, and the range that holds the target is walked.
#include "common.h"

#define SAMP_THREADS 1024

__global__ void argmax_rows_kernel(const float* __restrict__ logits, int V, int* __restrict__ ids,
                                   int* __restrict__ bad) {
  __shared__ float bv[SAMP_THREADS / 64];
  __shared__ int bi[SAMP_THREADS / 64];
  __shared__ int bbad;
  int row = blockIdx.x;
  const float* x = logits + (size_t)row * V;
  if (threadIdx.x == 0) bbad = 0;
  __syncthreads();
  float best = -INFINITY;
  int idx = 0x7fffffff;
  int notfinite = 0;
  for (int j = threadIdx.x; j < V; j += blockDim.x) {
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
    ids[row] = idx == 0x7fffffff ? 0 : idx;
    bad[row] = bbad;
  }
}

extern "C" int gs_argmax_rows(const float* logits, int rows, int V, int* ids, int* bad, hipStream_t stream) {
  GS_REQUIRE(rows >= 0 && V > 0, "argmax: bad sizes rows=%d V=%d", rows, V);
  if (rows == 0) return 0;
  argmax_rows_kernel<<<rows, SAMP_THREADS, 0, stream>>>(logits, V, ids, bad);
  GS_LAUNCH_CHECK("argmax_rows");
  return 0;
}

// One block per row.  temperature[row] > 0, u[row] in [0, 1).
__global__ void sample_temperature_kernel(const float* __restrict__ logits, int V,
                                          const double* __restrict__ temperature, const double* __restrict__ u,
                                          int* __restrict__ ids, int* __restrict__ bad) {
  __shared__ double part[SAMP_THREADS];
  __shared__ float redf[SAMP_THREADS / 64];
  __shared__ int bbad;
  int row = blockIdx.x;
  const float* x = logits + (size_t)row * V;
  int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nw = blockDim.x >> 6;
  if (tid == 0) bbad = 0;
  __syncthreads();
  // contiguous range of this thread
  int per = (V + blockDim.x - 1) / blockDim.x;
  int j0 = tid * per, j1 = j0 + per < V ? j0 + per : V;

  float mx = -INFINITY;
  int notfinite = 0;
  for (int j = j0; j < j1; ++j) {
    float v = x[j];
    if (!(fabsf(v) <= 3.402823466e38f)) notfinite = 1;
    mx = fmaxf(mx, v);
  }
  if (notfinite) atomicOr(&bbad, 1);
  mx = wave_max(mx);
  if (lane == 0) redf[wave] = mx;
  __syncthreads();
  mx = redf[0];
  for (int w = 1; w < nw; ++w) mx = fmaxf(mx, redf[w]);
  if (bbad) {
    if (tid == 0) {
      ids[row] = 0;
      bad[row] = 1;
    }
    return;
  }
  double hi = (double)mx, T = temperature[row];
  double s = 0.0;
  for (int j = j0; j < j1; ++j) s += exp(((double)x[j] - hi) / T);
  part[tid] = s;
  __syncthreads();
  // total, then the walk in id order, by one thread: whole ranges are skipped by their sums and
  // only the range that holds the target is walked id by id
  if (tid == 0) {
    double total = 0.0;
    for (int i = 0; i < (int)blockDim.x; ++i) total += part[i];
    double r = u[row] * total;
    double acc = 0.0;
    int pick = V - 1;
    bool found = false;
    for (int i = 0; i < (int)blockDim.x && !found; ++i) {
      if (r < acc + part[i]) {
        int a = i * per, b = a + per < V ? a + per : V;
        for (int j = a; j < b; ++j) {
          acc += exp(((double)x[j] - hi) / T);
          if (r < acc) {
            pick = j;
            found = true;
            break;
          }
        }
      } else {
        acc += part[i];
      }
    }
    ids[row] = pick;
    bad[row] = 0;
  }
}

extern "C" int gs_sample_temperature(const float* logits, int rows, int V, const double* temperature,
                                     const double* u, int* ids, int* bad, hipStream_t stream) {
  GS_REQUIRE(rows >= 0 && V > 0, "sample: bad sizes rows=%d V=%d", rows, V);
  if (rows == 0) return 0;
  sample_temperature_kernel<<<rows, SAMP_THREADS, 0, stream>>>(logits, V, temperature, u, ids, bad);
  GS_LAUNCH_CHECK("sample_temperature");
  return 0;
}
