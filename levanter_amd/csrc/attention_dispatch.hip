// Entry point of the matrix-core attention of ONE head size (LEV_HD, one library per head size): checks the
// sizes and calls the kernels.
#include "common.h"
#include "attention_config.h"

#ifndef LEV_HD
#error "compile with -DLEV_HD=<head size>"
#endif
#define LEV_CAT2(a, b) a##b
#define LEV_CAT(a, b) LEV_CAT2(a, b)
#define LEV_HD_ENTRY LEV_CAT(lev_attention_mfma_hd, LEV_HD)

extern "C" int LEV_HD_ENTRY(const void*, long, void*, long, void*, void*, const int*, const int*, const int*, int, const int*, int,
                            const int*, int, const void*, const void*, long, const int*, void*, int, int, int, int, float, int,
                            float, const float*, int, hipStream_t);

extern "C" int lev_attention_mfma_head_dim() { return LEV_HD; }

extern "C" int lev_attention_mfma(const void* q, long q_stride, void* out, long o_stride, void* k_pages, void* v_pages,
                                  const int* positions, const int* token_seq, const int* block_tables, int bt_stride,
                                  const int* prefill_tiles, int n_prefill_tiles, const int* decode_tokens, int n_decode,
                                  const void* k_new, const void* v_new, long kv_stride, const int* dest, void* workspace, int H,
                                  int KVH, int HD, int PS, int splits, float scale, int window, float softcap,
                                  const float* score_bias, int bias_len, hipStream_t stream) {
  LEV_REQUIRE(H > 0 && KVH > 0 && H % KVH == 0, "attention: bad head counts heads=%d kv_heads=%d", H, KVH);
  LEV_REQUIRE(H / KVH <= 16, "attention (matrix cores): at most 16 query heads per kv head, got %d", H / KVH);
  LEV_REQUIRE(HD == LEV_HD, "attention (matrix cores): this library is built for head_dim=%d, not %d", LEV_HD, HD);
  LEV_REQUIRE(PS > 0 && PS % 16 == 0, "attention: page_size=%d must be a multiple of 16", PS);
  LEV_REQUIRE(H <= 65535 && KVH <= 65535 && splits >= 1 && splits <= 64, "attention: grid too large (heads=%d) or more than 64 splits (%d)", H, splits);
  LEV_REQUIRE(window >= 0, "attention: window=%d must not be negative", window);
  LEV_REQUIRE(softcap >= 0.f && (!score_bias || bias_len >= 1), "attention: soft cap %g must not be negative and a bias table needs entries (%d)",
              (double)softcap, bias_len);
  LEV_REQUIRE(q_stride % 8 == 0 && o_stride % 4 == 0 && ((uintptr_t)q & 15) == 0 && ((uintptr_t)out & 7) == 0,
              "attention (matrix cores): q rows must be 16-byte aligned and out rows 8-byte aligned");
  LEV_REQUIRE(n_prefill_tiles == 0 || prefill_tiles, "attention: prefill tiles are missing");
  LEV_REQUIRE(n_decode == 0 || decode_tokens, "attention: decode tokens are missing");
  LEV_REQUIRE(n_decode == 0 || splits == 1 || workspace, "attention: split decoding needs a workspace");
  LEV_REQUIRE((k_new == nullptr) == (v_new == nullptr), "attention: new keys and values come together");
  LEV_REQUIRE(!k_new || (n_prefill_tiles == 0 && dest && kv_stride % 8 == 0 && ((uintptr_t)k_new & 15) == 0),
              "attention: new keys and values in the same launch need a step of single tokens, destinations and 16-byte aligned rows");
  return LEV_HD_ENTRY(q, q_stride, out, o_stride, k_pages, v_pages, positions, token_seq, block_tables, bt_stride, prefill_tiles,
                      n_prefill_tiles, decode_tokens, n_decode, k_new, v_new, kv_stride, dest, workspace, H, KVH, PS, splits, scale,
                      window, softcap, score_bias, bias_len, stream);
}
