// Causal grouped-query attention over the paged cache: the generic kernel.
//
// Takes every head width up to 256, any number of heads and groups, any page size, an optional
// window, float32 or bfloat16 storage; all arithmetic is float32.  One wave per (query token,
// query head).  The query at position p of sequence s sees keys lo..p of that sequence, lo = 0
// or p - window + 1; keys are read from the cache through the block table (this step's own
// keys were written there before).  Keys are walked in tiles of 64 starting at lo, with a running
// maximum and sum (online softmax), so the result for a position is the same however the
// sequence was cut into steps.
//
//   s_u = (q . k_u) * scale;  p_u = exp(s_u - max);  o = sum_u p_u v_u / sum_u p_u
//
// q (T, q_stride) with head h at columns [h d, (h+1) d); out (T, nh d); caches
// (num_pages, nkv, page_size, d).
#include "common.h"

#define GS_ATTN_MAX_D 256

template <typename T>
__global__ void attention_generic_kernel(const T* __restrict__ q, int q_stride, const T* __restrict__ kcache,
                                         const T* __restrict__ vcache, const int* __restrict__ positions,
                                         const int* __restrict__ seq_of_token, const int* __restrict__ block_table,
                                         int max_blocks, int page_size, int window, float scale, T* __restrict__ out,
                                         int nh, int nkv, int d) {
  __shared__ float qs[GS_ATTN_MAX_D];
  __shared__ float ps[64];
  __shared__ long rowoff[64];
  int lane = threadIdx.x;
  int t = blockIdx.x, h = blockIdx.y;
  int kvh = h / (nh / nkv);
  int pos = positions[t];
  int seq = seq_of_token[t];
  const int* bt = block_table + (size_t)seq * max_blocks;
  for (int j = lane; j < d; j += 64) qs[j] = to_f32(q[(size_t)t * q_stride + (size_t)h * d + j]);
  __syncthreads();

  int lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;
  float m = -INFINITY, l = 0.f;
  float acc[GS_ATTN_MAX_D / 64];
#pragma unroll
  for (int i = 0; i < GS_ATTN_MAX_D / 64; ++i) acc[i] = 0.f;

  for (int base = lo; base <= pos; base += 64) {
    int u = base + lane;
    float s = -INFINITY;
    long off = 0;
    if (u <= pos) {
      int page = bt[u / page_size];
      off = (((long)page * nkv + kvh) * page_size + u % page_size) * d;
      const T* kr = kcache + off;
      float dot = 0.f;
      for (int j = 0; j < d; ++j) dot += qs[j] * to_f32(kr[j]);
      s = dot * scale;
    }
    float m_new = fmaxf(m, wave_max(s));
    float p = u <= pos ? expf(s - m_new) : 0.f;
    float alpha = expf(m - m_new);  // 0 on the first tile (m = -inf), since m_new is finite there
    l = l * alpha + wave_sum(p);
    m = m_new;
    __syncthreads();
    ps[lane] = p;
    rowoff[lane] = off;
    __syncthreads();
    int nk = pos - base + 1 < 64 ? pos - base + 1 : 64;
#pragma unroll
    for (int i = 0; i < GS_ATTN_MAX_D / 64; ++i) {
      int j = lane + 64 * i;
      if (j < d) {
        float a = acc[i] * alpha;
        for (int k = 0; k < nk; ++k) a += ps[k] * to_f32(vcache[rowoff[k] + j]);
        acc[i] = a;
      }
    }
  }
  float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < GS_ATTN_MAX_D / 64; ++i) {
    int j = lane + 64 * i;
    if (j < d) out[((size_t)t * nh + h) * d + j] = from_f32<T>(acc[i] * inv);
  }
}

extern "C" int gs_attention_generic(const void* q, int q_stride, const void* kcache, const void* vcache, int dtype,
                                    const int* positions, const int* seq_of_token, const int* block_table,
                                    int max_blocks, int page_size, int window, float scale, void* out, int ntok,
                                    int nh, int nkv, int d, hipStream_t stream) {
  GS_REQUIRE(ntok >= 0 && nh > 0 && nkv > 0 && d > 0, "attention: bad sizes T=%d nh=%d nkv=%d d=%d", ntok, nh, nkv, d);
  GS_REQUIRE(nh % nkv == 0, "attention: %d query heads are no multiple of %d key heads", nh, nkv);
  GS_REQUIRE(d <= GS_ATTN_MAX_D, "attention: head width %d above the kernel's limit %d", d, GS_ATTN_MAX_D);
  GS_REQUIRE(nh <= 65535, "attention: more than 65535 heads");
  GS_REQUIRE(page_size > 0 && max_blocks > 0 && window >= 0, "attention: bad page_size/max_blocks/window");
  GS_REQUIRE(q_stride >= nh * d, "attention: q_stride %d below nh*d %d", q_stride, nh * d);
  if (ntok == 0) return 0;
  dim3 grid(ntok, nh);
  if (dtype == GS_F32)
    attention_generic_kernel<float><<<grid, 64, 0, stream>>>((const float*)q, q_stride, (const float*)kcache,
                                                              (const float*)vcache, positions, seq_of_token,
                                                              block_table, max_blocks, page_size, window, scale,
                                                              (float*)out, nh, nkv, d);
  else if (dtype == GS_BF16)
    attention_generic_kernel<bf16><<<grid, 64, 0, stream>>>((const bf16*)q, q_stride, (const bf16*)kcache,
                                                             (const bf16*)vcache, positions, seq_of_token,
                                                             block_table, max_blocks, page_size, window, scale,
                                                             (bf16*)out, nh, nkv, d);
  else
    GS_REQUIRE(false, "attention: unknown dtype %d", dtype);
  GS_LAUNCH_CHECK("attention_generic");
  return 0;
}
