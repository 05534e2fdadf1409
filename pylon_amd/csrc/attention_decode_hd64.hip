// The decode attention kernels of head size 64 (attention_decode.h).
#include "attention_decode.h"

int pylon_decode_run_64(AD_RUN_ARGS) {
  return decode_run<1>(mode, out, q, k_cache, v_cache, block_table, table_width, tok_row, positions, tokens, n_heads,
                       n_kv_heads, page_size, window, scale, n_waves, prep, n_cuts, partial, stream);
}
