// Facts about the matrix-core attention that the host needs before (and without) loading a kernel of a head size.
#include "common.h"
#include "attention_config.h"

// bytes of workspace for the partial results of n_decode single-token queries in `splits` splits
extern "C" long lev_attention_mfma_workspace(int n_decode, int splits, int H, int KVH, int HD) {
  (void)KVH;
  return (long)n_decode * splits * H * (HD + 2) * (long)sizeof(float);
}

// query rows of one prefill tile: the host cuts runs longer than one token into tiles of at most this many rows
extern "C" int lev_attention_prefill_tile_rows() { return PF_ROWS; }
