// Paged attention for steps with few query tokens (decode): bfloat16, head sizes 64, 128
// and 256, any grouping of up to 16 query heads per key/value head.
// It is bound by reading each request's keys and values once, so the work is cut along
// the keys: one wavefront takes one (token, key/value head, range of keys), handles all
// query heads of the group together, and leaves a partial result (running maximum, sum
// and weighted values in float); a second kernel merges the ranges of a token's head.
//
// Scores come from the 16x16x32 bf16 matrix instruction with 16 keys as rows and the
// group's query heads as columns (unused columns are zero).  The weighted sum of values
// runs on the vector units with one lane per pair of output elements, so values are read
// as whole contiguous rows.  Softmax statistics are float throughout.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

#define AD_MAX_GROUP 16
#define AD_TILE 16  // keys per score tile

// A lane owns EPL consecutive elements of a head (EPL = head_dim / 64).
template <int EPL>
__device__ __forceinline__ void load_bf16_elems(const uint16_t* p, float* v);
template <>
__device__ __forceinline__ void load_bf16_elems<1>(const uint16_t* p, float* v) {
  v[0] = bf16_bits_to_float(*p);
}
template <>
__device__ __forceinline__ void load_bf16_elems<2>(const uint16_t* p, float* v) {
  const uint32_t two = *reinterpret_cast<const uint32_t*>(p);
  v[0] = __uint_as_float(two << 16);
  v[1] = __uint_as_float(two & 0xffff0000u);
}
template <>
__device__ __forceinline__ void load_bf16_elems<4>(const uint16_t* p, float* v) {
  const uint2 four = *reinterpret_cast<const uint2*>(p);
  v[0] = __uint_as_float(four.x << 16);
  v[1] = __uint_as_float(four.x & 0xffff0000u);
  v[2] = __uint_as_float(four.y << 16);
  v[3] = __uint_as_float(four.y & 0xffff0000u);
}
template <int EPL>
__device__ __forceinline__ void store_bf16_elems(uint16_t* p, const float* v) {
#pragma unroll
  for (int i = 0; i < EPL; ++i) p[i] = float_to_bf16_bits(v[i]);
}

template <int EPL, int KSTEPS>  // EPL = head_dim / 64, KSTEPS = head_dim / 32
__global__ __launch_bounds__(PYLON_WAVE) void attention_decode_kernel(
    uint16_t* __restrict__ out, float* __restrict__ part_acc, float* __restrict__ part_ml,
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k_cache,
    const uint16_t* __restrict__ v_cache, const int* __restrict__ block_table, int table_width,
    const int* __restrict__ tok_row, const int* __restrict__ positions, int n_heads, int n_kv_heads,
    int page_size, int window, float scale, int n_splits) {
  constexpr int HD = EPL * 64;
  __shared__ float p_tile[AD_TILE][AD_MAX_GROUP];
  const int lane = threadIdx.x;
  const int col = lane & 15, grp = lane >> 4;
  const int split = blockIdx.x, kvh = blockIdx.y, t = blockIdx.z;
  const int group = n_heads / n_kv_heads;
  const int pos = positions[t];
  const int* table = block_table + static_cast<size_t>(tok_row[t]) * table_width;

  // the keys of this split
  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int n_keys = pos + 1 - first;
  int per_split = (n_keys + n_splits - 1) / n_splits;
  per_split = (per_split + AD_TILE - 1) / AD_TILE * AD_TILE;
  const int k_begin = first + split * per_split;
  int k_end = k_begin + per_split;
  if (k_end > pos + 1) k_end = pos + 1;

  // query fragments: column `col` is head kvh*group + col of the token
  bf16x8 qf[KSTEPS];
  {
    const bool valid = col < group;
    const uint16_t* qrow = q + (static_cast<size_t>(t) * n_heads + kvh * group + (valid ? col : 0)) * HD;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      if (valid) {
        qf[ks] = *reinterpret_cast<const bf16x8*>(qrow + ks * 32 + grp * 8);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) qf[ks][i] = (__bf16)0.0f;
      }
    }
  }

  float m_run = -INFINITY, l_run = 0.f;  // for head `col` (same in the 4 lanes that share it)
  float acc[AD_MAX_GROUP][EPL];  // only the first `group` rows are used
#pragma unroll
  for (int h = 0; h < AD_MAX_GROUP; ++h)
#pragma unroll
    for (int i = 0; i < EPL; ++i) acc[h][i] = 0.f;

  for (int base = k_begin; base < k_end; base += AD_TILE) {
    // row `col` of the tile is key base + col; rows past the end repeat the last key
    const int key = (base + col < k_end) ? base + col : k_end - 1;
    const int phys = table[key / page_size] * page_size + key % page_size;
    const uint16_t* krow = k_cache + (static_cast<size_t>(phys) * n_kv_heads + kvh) * HD;
    floatx4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const bf16x8 kf = *reinterpret_cast<const bf16x8*>(krow + ks * 32 + grp * 8);
      s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[ks], s, 0, 0, 0);
    }
    // lane holds, for head `col`, the scores of keys base + 4*grp + r
    float sv[4];
    float tile_max = -INFINITY;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const bool live = base + 4 * grp + r < k_end;
      sv[r] = live ? s[r] * scale : -INFINITY;
      tile_max = fmaxf(tile_max, sv[r]);
    }
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, PYLON_WAVE));
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, PYLON_WAVE));
    const float m_new = fmaxf(m_run, tile_max);  // finite: key `base` is always live
    const float corr = expf(m_run - m_new);
    float tile_sum = 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float p = expf(sv[r] - m_new);  // exp(-inf) = 0 for keys past the end
      tile_sum += p;
      if (col < AD_MAX_GROUP) p_tile[4 * grp + r][col] = p;
    }
    tile_sum += __shfl_xor(tile_sum, 16, PYLON_WAVE);
    tile_sum += __shfl_xor(tile_sum, 32, PYLON_WAVE);
    l_run = l_run * corr + tile_sum;
    m_run = m_new;
    __syncthreads();
    // rescale what has been accumulated: the factor of head h sits in lane h
#pragma unroll
    for (int h = 0; h < AD_MAX_GROUP; ++h) {
      if (h < group) {
        const float c = __shfl(corr, h, PYLON_WAVE);
#pragma unroll
        for (int i = 0; i < EPL; ++i) acc[h][i] *= c;
      }
    }
    const int live_keys = (k_end - base < AD_TILE) ? k_end - base : AD_TILE;
    for (int kk = 0; kk < live_keys; ++kk) {
      const int pk = __shfl(phys, kk, PYLON_WAVE);
      const uint16_t* vrow = v_cache + (static_cast<size_t>(pk) * n_kv_heads + kvh) * HD;
      float vv[EPL];
      load_bf16_elems<EPL>(vrow + lane * EPL, vv);
#pragma unroll
      for (int h = 0; h < AD_MAX_GROUP; ++h) {
        if (h < group) {
          const float p = p_tile[kk][h];
#pragma unroll
          for (int i = 0; i < EPL; ++i) acc[h][i] = fmaf(p, vv[i], acc[h][i]);
        }
      }
    }
    __syncthreads();
  }

  // results: acc[h][i] is element lane*EPL + i of head h
  if (n_splits == 1) {
#pragma unroll
    for (int h = 0; h < AD_MAX_GROUP; ++h) {
      if (h < group) {
        const float inv = 1.0f / __shfl(l_run, h, PYLON_WAVE);
        uint16_t* orow = out + (static_cast<size_t>(t) * n_heads + kvh * group + h) * HD;
        float o[EPL];
#pragma unroll
        for (int i = 0; i < EPL; ++i) o[i] = acc[h][i] * inv;
        store_bf16_elems<EPL>(orow + lane * EPL, o);
      }
    }
  } else {
#pragma unroll
    for (int h = 0; h < AD_MAX_GROUP; ++h) {
      if (h < group) {
        const size_t item = (static_cast<size_t>(t) * n_heads + kvh * group + h) * n_splits + split;
        float* arow = part_acc + item * HD;
#pragma unroll
        for (int i = 0; i < EPL; ++i) arow[lane * EPL + i] = acc[h][i];
        const float mh = __shfl(m_run, h, PYLON_WAVE), lh = __shfl(l_run, h, PYLON_WAVE);
        if (lane == 0) {
          part_ml[item * 2] = mh;
          part_ml[item * 2 + 1] = lh;
        }
      }
    }
  }
}

// One wavefront per (token, head): combine the key ranges' partial results.
template <int EPL>
__global__ __launch_bounds__(PYLON_WAVE) void attention_merge_kernel(uint16_t* __restrict__ out,
                                                                     const float* __restrict__ part_acc,
                                                                     const float* __restrict__ part_ml,
                                                                     int n_splits) {
  constexpr int HD = EPL * 64;
  const int lane = threadIdx.x;
  const size_t item = blockIdx.x;
  const float* ml = part_ml + item * n_splits * 2;
  float m = -INFINITY;
  for (int s = 0; s < n_splits; ++s) m = fmaxf(m, ml[2 * s]);
  float l = 0.f;
  float acc[EPL];
#pragma unroll
  for (int i = 0; i < EPL; ++i) acc[i] = 0.f;
  for (int s = 0; s < n_splits; ++s) {
    const float ls = ml[2 * s + 1];
    if (ls == 0.f) continue;  // an empty range
    const float f = expf(ml[2 * s] - m);
    l += ls * f;
    const float* arow = part_acc + (item * n_splits + s) * HD;
#pragma unroll
    for (int i = 0; i < EPL; ++i) acc[i] = fmaf(arow[lane * EPL + i], f, acc[i]);
  }
  const float inv = 1.0f / l;
  uint16_t* orow = out + item * HD;
  float o[EPL];
#pragma unroll
  for (int i = 0; i < EPL; ++i) o[i] = acc[i] * inv;
  store_bf16_elems<EPL>(orow + lane * EPL, o);
}

template <int EPL>
static void launch_decode(void* out, float* part_acc, float* part_ml, const void* q, const void* k_cache,
                          const void* v_cache, const int* block_table, int table_width,
                          const int* tok_row, const int* positions, int tokens, int n_heads,
                          int n_kv_heads, int page_size, int window, float scale, int n_splits,
                          hipStream_t stream) {
  dim3 grid(n_splits, n_kv_heads, tokens), block(PYLON_WAVE);
  hipLaunchKernelGGL((attention_decode_kernel<EPL, EPL * 2>), grid, block, 0, stream, (uint16_t*)out,
                     part_acc, part_ml, (const uint16_t*)q, (const uint16_t*)k_cache,
                     (const uint16_t*)v_cache, block_table, table_width, tok_row, positions, n_heads,
                     n_kv_heads, page_size, window, scale, n_splits);
  if (n_splits > 1)
    hipLaunchKernelGGL((attention_merge_kernel<EPL>), dim3(tokens * n_heads), block, 0, stream,
                       (uint16_t*)out, part_acc, part_ml, n_splits);
}

// q, out: [tokens, n_heads, head_dim] bf16. part_acc: float [tokens*n_heads*n_splits*head_dim],
// part_ml: float [tokens*n_heads*n_splits*2] (both unused when n_splits == 1).
extern "C" int pylon_attention_decode(void* out, float* part_acc, float* part_ml, const void* q,
                                      const void* k_cache, const void* v_cache, const int* block_table,
                                      int table_width, const int* tok_row, const int* positions,
                                      int tokens, int n_heads, int n_kv_heads, int head_dim,
                                      int page_size, int window, float scale, int n_splits,
                                      hipStream_t stream) {
  PYLON_REQUIRE(tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
                "attention_decode: %d query heads cannot be grouped over %d key/value heads", n_heads,
                n_kv_heads);
  PYLON_REQUIRE(n_heads / n_kv_heads <= AD_MAX_GROUP,
                "attention_decode: at most %d query heads per key/value head", AD_MAX_GROUP);
  PYLON_REQUIRE(head_dim == 64 || head_dim == 128 || head_dim == 256,
                "attention_decode: head_dim %d is not 64, 128 or 256", head_dim);
  PYLON_REQUIRE(page_size > 0 && table_width > 0 && window >= 0, "attention_decode: bad page size, width or window");
  PYLON_REQUIRE(n_splits >= 1 && n_splits <= 64, "attention_decode: 1..64 key ranges");
  PYLON_REQUIRE(n_splits == 1 || (part_acc && part_ml), "attention_decode: key ranges need partial buffers");
  PYLON_REQUIRE(tokens <= 65535 && n_kv_heads <= 65535, "attention_decode: too many tokens or heads for one launch");
  if (tokens == 0) return 0;
#define GO(D)                                                                                           \
  launch_decode<D>(out, part_acc, part_ml, q, k_cache, v_cache, block_table, table_width, tok_row,     \
                   positions, tokens, n_heads, n_kv_heads, page_size, window, scale, n_splits, stream)
  switch (head_dim / 64) {
    case 1: GO(1); break;
    case 2: GO(2); break;
    default: GO(4); break;
  }
#undef GO
  PYLON_LAUNCHED("attention_decode");
}
