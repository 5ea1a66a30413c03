// bfloat16 instantiation of the per-token cache attention (bfloat16 q, cache and output;
// scores, softmax and accumulation in 32-bit).
#include "attn_tokens_impl.h"

MF_API int mf_attn_tokens_bf16(const void* q, const void* kc, const void* vc, const int* page_table,
                               int pt_stride, const int* positions, const int* seq_of_tok, void* out,
                               float* part, int n_tok, int nh, int nk, int hd, float scale, int window,
                               int n_splits, int split_len, hipStream_t stream) {
  return attn_tokens::launch<bf16>(q, kc, vc, page_table, pt_stride, positions, seq_of_tok, out, part,
                                   n_tok, nh, nk, hd, scale, window, n_splits, split_len, stream);
}
