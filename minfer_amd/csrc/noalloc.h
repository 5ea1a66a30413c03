// An entry point that allocates nothing.
//
// It has no counterpart in yusiwen/minfer.  It is for callers that cannot allocate device memory
// around a call: code under HIP graph capture, tight serving loops, harnesses that forbid
// hipMalloc.  `mf_attn_decode_bf16_noalloc` is `mf_attn_decode_bf16` (attention of single query
// tokens over the paged bfloat16 cache, keys split over blocks) with the partial results of the
// key splits kept in a fixed array of the library instead of a workspace that the caller brings:
// the caller passes inputs and outputs only.
//
// * The array holds MF_NOALLOC_SCRATCH_FLOATS floats (4 MiB), on every GPU the library runs on,
//   until the process ends.  A call needs n_tok * n_heads * n_splits * (head_dim + 2) of them when
//   n_splits > 1 and none otherwise; a call that needs more is refused with
//   MF_NOALLOC_TOO_LARGE and launches nothing.
// * Nothing in the array has to start at zero: every split of every (token, head) writes its whole
//   partial before the merge reads it, so what an earlier call left behind is never read.
// * All calls on one GPU share that GPU's array.  Calls that overlap there (on different
//   streams) race; calls on one stream, or ordered by events, do not.
// * No hipMalloc, hipFree or other allocating call is made; the first call on a device asks the
//   runtime for the array's address on that device (hipGetSymbolAddress) and keeps it.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

#define MF_NOALLOC_SCRATCH_FLOATS ((size_t)1 << 20)
#define MF_NOALLOC_TOO_LARGE (-3)

extern "C" {

// Arguments as mf_attn_decode_bf16 without `part` and `base_splits` (every token's keys go over
// all n_splits splits): q, out [n_tok][nh][hd] bfloat16; kc
// [pages][nk][64][hd]; vt [pages][nk][2][hd][32]; page_table [sequences][pt_stride] int32;
// positions, seq_of_tok [n_tok] int32; 1 <= n_splits <= 64.  Returns 0, a hipError_t, or
// MF_NOALLOC_TOO_LARGE.
int mf_attn_decode_bf16_noalloc(const void* q, const void* kc, const void* vt, const int* page_table,
                                int pt_stride, const int* positions, const int* seq_of_tok, void* out, int n_tok,
                                int nh, int nk, int hd, float scale, int window, int n_splits, hipStream_t stream);

// floats of the array (MF_NOALLOC_SCRATCH_FLOATS), for callers that plan their split counts
size_t mf_attn_decode_bf16_noalloc_capacity(void);

}
