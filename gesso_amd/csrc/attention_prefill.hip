// Prompt attention on the matrix cores: the entry point; the kernels are in attention_prefill_impl.h, compiled
// per head width in attention_prefill_d*.hip.
#include "attention_prefill_decl.h"


// Head widths 32, 64, 128; groups of 1 to 8 heads (the block has one wavefront per head of the group).
extern "C" int gs_attention_prefill_supports(int nh, int nkv, int d) {
  if (nkv <= 0 || nh % nkv) return 0;
  int g = nh / nkv;
  return (d == 32 || d == 64 || d == 128) && g >= 1 && g <= 8;
}

extern "C" int gs_attention_prefill(const void* q, int q_stride, const void* kcache, const void* vcache,
                                    const int* positions, const int* tile_seq, const int* tile_row,
                                    const int* tile_n, int ntiles, const int* block_table, int max_blocks,
                                    int page_size, int window, float scale, void* out, int nh, int nkv, int d,
                                    int tile_rows, hipStream_t stream) {
  GS_REQUIRE(gs_attention_prefill_supports(nh, nkv, d), "attention_prefill: sizes nh=%d nkv=%d d=%d are not taken", nh, nkv, d);
  GS_REQUIRE(ntiles >= 0 && nkv > 0 && (long)ntiles * nkv < (1L << 31), "attention_prefill: %d tiles x %d key heads are too many blocks", ntiles, nkv);
  GS_REQUIRE(tile_rows == 16 || tile_rows == 32, "attention_prefill: tiles hold 16 or 32 queries, not %d", tile_rows);
  GS_REQUIRE(page_size > 0 && max_blocks > 0 && window >= 0, "attention_prefill: bad page_size/max_blocks/window");
  GS_REQUIRE(q_stride >= nh * d && q_stride % 8 == 0 && ((uintptr_t)q & 15) == 0, "attention_prefill: q rows must be 16-byte aligned");
  GS_REQUIRE(((uintptr_t)kcache & 15) == 0 && ((uintptr_t)vcache & 15) == 0 && ((uintptr_t)out & 7) == 0,
             "attention_prefill: cache and output must be aligned");
  // the kernel divides by page_size with one multiplication, exact while key index x page_size < 2^32
  GS_REQUIRE(page_size >= 2 && (long)max_blocks * page_size * page_size < (1L << 32),
             "attention_prefill: page_size %d with %d blocks a sequence is outside what the kernel's division takes", page_size, max_blocks);
  if (ntiles == 0) return 0;
  const unsigned page_magic = (unsigned)((1ull << 32) / (unsigned)page_size + 1);
  PrefillCall c = {(const bf16*)q, (const bf16*)kcache, (const bf16*)vcache, positions, tile_seq, tile_row, tile_n,
                   block_table, q_stride, max_blocks, page_size, window, nh, nkv, tile_rows, ntiles, page_magic, scale,
                   (bf16*)out, stream};
  int rc = -1;
  switch (d) {
    case 32: rc = gs_attention_prefill_d32(c); break;
    case 64: rc = gs_attention_prefill_d64(c); break;
    case 128: rc = gs_attention_prefill_d128(c); break;
  }
  GS_REQUIRE(rc == 0, "attention_prefill: no kernel for this group size");
  GS_LAUNCH_CHECK("attention_prefill");
  return 0;
}
