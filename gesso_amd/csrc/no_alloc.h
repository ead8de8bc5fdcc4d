// The one entry point of this library that touches no allocator.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device memory: code under
// HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Every other entry point takes its
// workspace from the caller (who allocates it); this one keeps it in a file-scope device array.
#pragma once
#include <hip/hip_runtime.h>

// Floats the static workspace holds: 4 MiB on each GPU the library runs on, until the process ends.
#define GS_DECODE_STATIC_FLOATS (1 << 20)

extern "C" {

// Floats of workspace a call needs: nseq * nh * nsplit * (d + 2).
long gs_attention_decode_workspace(int nseq, int nh, int nkv, int d, int nsplit);

// gs_attention_decode without the workspace argument: split-key decode attention whose partial results (one
// accumulator, maximum and sum per sequence, head and split) lie in a static device array of
// GS_DECODE_STATIC_FLOATS floats.  A call that needs more is refused with an error (gs_last_error says how many);
// nothing is launched then.  No hipMalloc, hipFree or other allocating call is made, on any path.
//
// All calls on one GPU share that GPU's array: calls that may overlap there (two streams, two threads) race and
// must be ordered by the caller.  The array keeps the last call's contents; nothing in it has to start at zero,
// because every partial result that the merge reads is written by the same call first.
int gs_attention_decode_static(const void* q, int q_stride, const void* kcache, const void* vcache,
                               const int* positions, const int* block_table, int max_blocks, int page_size,
                               int window, float scale, void* out, int out_tiled, int nseq, int nh, int nkv, int d,
                               int nsplit, hipStream_t stream);
}
