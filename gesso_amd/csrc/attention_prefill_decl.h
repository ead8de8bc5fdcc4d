// What the entry point of the prompt attention hands to the kernels of one head width.
#pragma once
#include "common.h"

struct PrefillCall {
  const bf16 *q, *kc, *vc;
  const int *positions, *tile_seq, *tile_row, *tile_n, *bt;
  int q_stride, max_blocks, page_size, window, nh, nkv, tile_rows, ntiles;
  unsigned page_magic;
  float scale;
  bf16* out;
  hipStream_t stream;
};
int gs_attention_prefill_d32(const PrefillCall& c);
int gs_attention_prefill_d64(const PrefillCall& c);
int gs_attention_prefill_d128(const PrefillCall& c);
