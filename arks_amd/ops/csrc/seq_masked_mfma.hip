// placeholder until the kernels below are written
#include "seq_common.h"
extern "C" int arks_seq_attn_masked_mfma(
    void* out, int64_t ldo, const void* q, const void* k_cache, int64_t ldk,
    const void* v_cache, int64_t ldv, const void* block_tables,
    const void* seq_lens, const void* cu, const void* token_seq, float scale,
    const void* sink_w, float softcap, int window, int keep_first,
    float out_scale, int T, int H, int G, int D, int V, int bs, int max_blocks,
    int num_seqs, int single_rows, hipStream_t stream) {
  return 1;
}
