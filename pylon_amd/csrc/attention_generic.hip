// Paged causal grouped-query attention, the exact and general form: any element type,
// any head size that is a multiple of 16 (up to 512), any number of heads and groups,
// any page size, optional sliding window.  One wavefront owns one (token, query head):
// it walks that token's visible keys 64 at a time (one key per lane), keeps a running
// maximum and sum in float, and accumulates the weighted values with one lane per
// output element.  The walk starts at the first visible key of the token, so the order
// of every sum depends only on the token's position and never on how the batch was cut.
#include "common.h"

#define ATT_WAVES 4

template <typename T>
struct Vec8;  // eight consecutive elements, loaded as wide as the type allows

template <>
struct Vec8<float> {
  static __device__ __forceinline__ float dot(const float* __restrict__ q, const float* __restrict__ k, float acc) {
    const float4 a = *reinterpret_cast<const float4*>(k);
    const float4 b = *reinterpret_cast<const float4*>(k + 4);
    acc = fmaf(q[0], a.x, acc);
    acc = fmaf(q[1], a.y, acc);
    acc = fmaf(q[2], a.z, acc);
    acc = fmaf(q[3], a.w, acc);
    acc = fmaf(q[4], b.x, acc);
    acc = fmaf(q[5], b.y, acc);
    acc = fmaf(q[6], b.z, acc);
    acc = fmaf(q[7], b.w, acc);
    return acc;
  }
};

template <>
struct Vec8<bf16_t> {
  static __device__ __forceinline__ float dot(const float* __restrict__ q, const bf16_t* __restrict__ k, float acc) {
    const uint4 raw = *reinterpret_cast<const uint4*>(k);
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      acc = fmaf(q[2 * i], __uint_as_float(w[i] << 16), acc);
      acc = fmaf(q[2 * i + 1], __uint_as_float(w[i] & 0xffff0000u), acc);
    }
    return acc;
  }
};

template <typename T, int DIMS_PER_LANE>
__global__ void paged_attention_kernel(T* __restrict__ out, const T* __restrict__ q,
                                       const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                                       const int* __restrict__ block_table, int table_width,
                                       const int* __restrict__ tok_row, const int* __restrict__ positions,
                                       long long items, int n_heads, int n_kv_heads, int head_dim,
                                       int page_size, int window, float scale) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x & (PYLON_WAVE - 1);
  const int wave = threadIdx.x / PYLON_WAVE;
  float* qbuf = lds + wave * head_dim;
  const long long item = static_cast<long long>(blockIdx.x) * ATT_WAVES + wave;
  const bool active = item < items;
  int t = 0, h = 0;
  if (active) {
    t = static_cast<int>(item / n_heads);
    h = static_cast<int>(item - static_cast<long long>(t) * n_heads);
    const T* qr = q + (static_cast<size_t>(t) * n_heads + h) * head_dim;
    for (int i = lane; i < head_dim; i += PYLON_WAVE) qbuf[i] = to_float(qr[i]);
  }
  __syncthreads();
  if (!active) return;

  const int kvh = h / (n_heads / n_kv_heads);
  const int pos = positions[t];
  const int* table = block_table + static_cast<size_t>(tok_row[t]) * table_width;
  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;

  float m = -INFINITY, l = 0.f;
  float acc[DIMS_PER_LANE];
#pragma unroll
  for (int i = 0; i < DIMS_PER_LANE; ++i) acc[i] = 0.f;

  for (int base = first; base <= pos; base += PYLON_WAVE) {
    const int j = base + lane;
    const bool valid = j <= pos;
    int phys = 0;
    float s = -INFINITY;
    if (valid) {
      phys = table[j / page_size] * page_size + (j % page_size);
      const T* kr = k_cache + (static_cast<size_t>(phys) * n_kv_heads + kvh) * head_dim;
      float dot = 0.f;
      for (int d = 0; d < head_dim; d += 8) dot = Vec8<T>::dot(qbuf + d, kr + d, dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);
    l = l * corr + wave_sum(p);
#pragma unroll
    for (int i = 0; i < DIMS_PER_LANE; ++i) acc[i] *= corr;
    const int count = (pos - base + 1 < PYLON_WAVE) ? pos - base + 1 : PYLON_WAVE;
    for (int kk = 0; kk < count; ++kk) {
      const float pk = __shfl(p, kk, PYLON_WAVE);
      const int physk = __shfl(phys, kk, PYLON_WAVE);
      const T* vr = v_cache + (static_cast<size_t>(physk) * n_kv_heads + kvh) * head_dim;
#pragma unroll
      for (int i = 0; i < DIMS_PER_LANE; ++i) {
        const int d = lane + PYLON_WAVE * i;
        if (d < head_dim) acc[i] = fmaf(pk, to_float(vr[d]), acc[i]);
      }
    }
    m = m_new;
  }
  T* orow = out + (static_cast<size_t>(t) * n_heads + h) * head_dim;
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < DIMS_PER_LANE; ++i) {
    const int d = lane + PYLON_WAVE * i;
    if (d < head_dim) orow[d] = from_float<T>(acc[i] * inv);
  }
}

template <typename T>
static int launch_paged_attention(T* out, const T* q, const T* k_cache, const T* v_cache,
                                  const int* block_table, int table_width, const int* tok_row,
                                  const int* positions, int tokens, int n_heads, int n_kv_heads,
                                  int head_dim, int page_size, int window, float scale,
                                  hipStream_t stream) {
  const long long items = static_cast<long long>(tokens) * n_heads;
  const long long blocks = (items + ATT_WAVES - 1) / ATT_WAVES;
  dim3 grid((unsigned)blocks), block(ATT_WAVES * PYLON_WAVE);
  const size_t lds = sizeof(float) * ATT_WAVES * head_dim;
#define LAUNCH(DPL)                                                                                  \
  hipLaunchKernelGGL((paged_attention_kernel<T, DPL>), grid, block, lds, stream, out, q, k_cache,    \
                     v_cache, block_table, table_width, tok_row, positions, items, n_heads,          \
                     n_kv_heads, head_dim, page_size, window, scale)
  if (head_dim <= 64)
    LAUNCH(1);
  else if (head_dim <= 128)
    LAUNCH(2);
  else if (head_dim <= 256)
    LAUNCH(4);
  else
    LAUNCH(8);
#undef LAUNCH
  return 0;
}

// q, out: [tokens, n_heads, head_dim]. Caches: [pages*page_size, n_kv_heads, head_dim].
// block_table: [rows, table_width] page ids; tok_row[t] names the table row of token t;
// positions[t] is the token's index in its request; keys first(t)..positions[t] are read,
// first(t) = max(0, positions[t] - window + 1) when window > 0, else 0.
extern "C" int pylon_paged_attention(void* out, const void* q, const void* k_cache, const void* v_cache,
                                     int dtype, const int* block_table, int table_width,
                                     const int* tok_row, const int* positions, int tokens, int n_heads,
                                     int n_kv_heads, int head_dim, int page_size, int window,
                                     float scale, hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(dtype), "paged_attention: unknown dtype");
  PYLON_REQUIRE(tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
                "paged_attention: %d query heads cannot be grouped over %d key/value heads", n_heads,
                n_kv_heads);
  PYLON_REQUIRE(head_dim >= 16 && head_dim % 16 == 0 && head_dim <= 512,
                "paged_attention: head_dim %d must be a multiple of 16 between 16 and 512", head_dim);
  PYLON_REQUIRE(page_size > 0 && table_width > 0, "paged_attention: bad page size or table width");
  PYLON_REQUIRE(window >= 0, "paged_attention: window must be 0 (none) or positive");
  if (tokens == 0) return 0;
  PYLON_REQUIRE(static_cast<long long>(tokens) * n_heads / ATT_WAVES < (1ll << 31),
                "paged_attention: too many (token, head) pairs for one launch");
  if (dtype == PYLON_F32)
    launch_paged_attention<float>((float*)out, (const float*)q, (const float*)k_cache,
                                  (const float*)v_cache, block_table, table_width, tok_row, positions,
                                  tokens, n_heads, n_kv_heads, head_dim, page_size, window, scale, stream);
  else
    launch_paged_attention<bf16_t>((bf16_t*)out, (const bf16_t*)q, (const bf16_t*)k_cache,
                                   (const bf16_t*)v_cache, block_table, table_width, tok_row, positions,
                                   tokens, n_heads, n_kv_heads, head_dim, page_size, window, scale,
                                   stream);
  PYLON_LAUNCHED("paged_attention");
}
