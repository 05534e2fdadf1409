// The entry points of the decode attention kernels (attention_decode.h; one translation unit
// per head size holds the kernels).
#include "attention_decode.h"

static int decode_run_by_head_dim(int head_dim, AD_RUN_ARGS) {
  switch (head_dim / 64) {
    case 1:
      return pylon_decode_run_64(mode, out, q, k_cache, v_cache, block_table, table_width, tok_row, positions, tokens,
                                 n_heads, n_kv_heads, page_size, window, scale, n_waves, prep, n_cuts, partial, stream);
    case 2:
      return pylon_decode_run_128(mode, out, q, k_cache, v_cache, block_table, table_width, tok_row, positions, tokens,
                                  n_heads, n_kv_heads, page_size, window, scale, n_waves, prep, n_cuts, partial, stream);
    default:
      return pylon_decode_run_256(mode, out, q, k_cache, v_cache, block_table, table_width, tok_row, positions, tokens,
                                  n_heads, n_kv_heads, page_size, window, scale, n_waves, prep, n_cuts, partial, stream);
  }
}

// Floats of scratch that n_cuts > 1 needs.
extern "C" long long pylon_attention_decode_scratch_floats(int tokens, int n_heads, int head_dim, int n_cuts) {
  if (n_cuts <= 1) return 0;
  return static_cast<long long>(tokens) * n_heads * n_cuts * (head_dim + 2);
}

static int check_decode_cuts(const char* name, int tokens, int n_heads, int head_dim, int n_cuts,
                             const float* partial, long long partial_floats) {
  PYLON_REQUIRE(n_cuts >= 1 && n_cuts <= 64, "%s: the keys can be cut over 1..64 workgroups, got %d", name, n_cuts);
  PYLON_REQUIRE(n_cuts == 1 || (partial != nullptr && partial_floats >= pylon_attention_decode_scratch_floats(
                                                                            tokens, n_heads, head_dim, n_cuts)),
                "%s: %d cuts need a scratch buffer of %lld floats", name, n_cuts,
                pylon_attention_decode_scratch_floats(tokens, n_heads, head_dim, n_cuts));
  return 0;
}

static int check_decode_geometry(const char* name, int tokens, int n_heads, int n_kv_heads, int head_dim,
                                 int page_size, int table_width, int window, int n_waves) {
  PYLON_REQUIRE(tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
                "%s: %d query heads cannot be grouped over %d key/value heads", name, n_heads, n_kv_heads);
  PYLON_REQUIRE(n_heads / n_kv_heads <= AD_MAX_GROUP, "%s: at most %d query heads per key/value head", name,
                AD_MAX_GROUP);
  PYLON_REQUIRE(head_dim == 64 || head_dim == 128 || head_dim == 256, "%s: head_dim %d is not 64, 128 or 256",
                name, head_dim);
  PYLON_REQUIRE(page_size > 0 && table_width > 0 && window >= 0, "%s: bad page size, width or window", name);
  PYLON_REQUIRE(n_waves == 1 || n_waves == 2 || n_waves == 4 || n_waves == 8,
                "%s: 1, 2, 4 or 8 waves per (token, head), got %d", name, n_waves);
  PYLON_REQUIRE(tokens <= 65535 && n_kv_heads <= 65535, "%s: too many tokens or heads for one launch", name);
  return 0;
}

// q, out: [tokens, n_heads, head_dim] bf16; n_waves (1, 2, 4 or 8) wavefronts share
// the keys of one (token, key/value head), after n_cuts workgroups have shared them first
// (n_cuts > 1 needs `partial`, scratch of pylon_attention_decode_scratch_floats floats).
extern "C" int pylon_attention_decode(void* out, const void* q, const void* k_cache, const void* v_cache,
                                      const int* block_table, int table_width, const int* tok_row,
                                      const int* positions, int tokens, int n_heads, int n_kv_heads,
                                      int head_dim, int page_size, int window, float scale, int n_waves,
                                      int n_cuts, float* partial, long long partial_floats,
                                      hipStream_t stream) {
  if (check_decode_geometry("attention_decode", tokens, n_heads, n_kv_heads, head_dim, page_size, table_width,
                            window, n_waves) ||
      check_decode_cuts("attention_decode", tokens, n_heads, head_dim, n_cuts, partial, partial_floats))
    return 1;
  if (tokens == 0) return 0;
  const DecodePrep none = {};
  decode_run_by_head_dim(head_dim, AD_MODE_QUERIES, out, q, const_cast<void*>(k_cache), const_cast<void*>(v_cache),
                         block_table, table_width, tok_row, positions, tokens, n_heads, n_kv_heads, page_size, window,
                         scale, n_waves, none, n_cuts, partial, stream);
  PYLON_LAUNCHED("attention_decode");
}

// The same from the raw projection qkv: [tokens, row_stride] bf16 with q heads first, then
// (if slot_map is given) k heads, then v heads; or, with qkv_parts > 0, that many float
// partial sums of it, part_stride elements apart, which the kernel adds and rounds to bf16.  Each token's key and value are normed,
// rotated (inv_freq: head_dim/2 frequencies for a rotation of the whole head, or null) and
// stored at slot_map[t] before the cache is read; a negative slot stores nothing.  With
// slot_map null only the queries are prepared (a layer that reads another layer's cache).
extern "C" int pylon_attention_decode_fused(void* out, const void* qkv, long long row_stride, int qkv_parts,
                                            long long part_stride, const float* q_weight, const float* k_weight, float eps,
                                            const float* inv_freq, void* k_cache, void* v_cache,
                                            const int* slot_map, const int* block_table, int table_width,
                                            const int* tok_row, const int* positions, int tokens,
                                            int n_heads, int n_kv_heads, int head_dim, int page_size,
                                            int window, float scale, int n_waves, int n_cuts,
                                            float* partial, long long partial_floats, hipStream_t stream) {
  if (check_decode_geometry("attention_decode_fused", tokens, n_heads, n_kv_heads, head_dim, page_size,
                            table_width, window, n_waves) ||
      check_decode_cuts("attention_decode_fused", tokens, n_heads, head_dim, n_cuts, partial, partial_floats))
    return 1;
  const long long heads = n_heads + (slot_map != nullptr ? 2ll * n_kv_heads : 0);
  PYLON_REQUIRE(row_stride >= heads * head_dim, "attention_decode_fused: row stride %lld is shorter than %lld heads of %d",
                row_stride, heads, head_dim);
  PYLON_REQUIRE(row_stride % 8 == 0 && (reinterpret_cast<uintptr_t>(qkv) & 15) == 0,
                "attention_decode_fused: the projection's rows must be 16-byte aligned");
  PYLON_REQUIRE(qkv_parts >= 0 && qkv_parts <= 64, "attention_decode_fused: 0 to 64 partial sums, got %d", qkv_parts);
  PYLON_REQUIRE(qkv_parts == 0 || (part_stride % 4 == 0 && part_stride >= static_cast<long long>(tokens - 1) * row_stride + heads * head_dim),
                "attention_decode_fused: the partial sums overlap or are not 16-byte aligned");
  if (tokens == 0) return 0;
  const DecodePrep prep = {qkv, row_stride, qkv_parts, part_stride, q_weight, k_weight, eps, inv_freq, slot_map};
  decode_run_by_head_dim(head_dim, qkv_parts > 0 ? AD_MODE_PARTIAL_SUMS : AD_MODE_PROJECTION, out, nullptr, k_cache,
                         v_cache, block_table, table_width, tok_row, positions, tokens, n_heads, n_kv_heads, page_size,
                         window, scale, n_waves, prep, n_cuts, partial, stream);
  PYLON_LAUNCHED("attention_decode_fused");
}
