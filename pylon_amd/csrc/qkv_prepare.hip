// What happens between the fused q/k/v projection and attention, in one pass over the
// projection's output: per-head RMSNorm of q and k (optional), rotary position encoding
// of q and k (optional), q written out head-major, k and v scattered into their cache
// pages.  One wavefront handles one head of one token.  Norm, angles and rotation are
// computed in float and rounded once on the store.
#include "common.h"
#include "head_prepare.h"

#define QKV_WAVES 4

template <typename T>
__global__ void qkv_prepare_kernel(T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                   const T* __restrict__ qkv, long long row_stride,
                                   const float* __restrict__ q_weight, const float* __restrict__ k_weight,
                                   float eps, const float* __restrict__ inv_freq, int rot_dim,
                                   const int* __restrict__ positions, const int* __restrict__ slot_map,
                                   long long items, int n_heads, int n_kv_heads, int head_dim,
                                   int heads_per_token) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x & (PYLON_WAVE - 1);
  const int wave = threadIdx.x / PYLON_WAVE;
  float* buf = lds + wave * head_dim;
  const long long item = static_cast<long long>(blockIdx.x) * QKV_WAVES + wave;
  const bool active = item < items;

  int t = 0, s = 0;
  const T* src = nullptr;
  T* dst = nullptr;
  const float* weight = nullptr;
  bool rotate = false;
  if (active) {
    t = static_cast<int>(item / heads_per_token);
    s = static_cast<int>(item - static_cast<long long>(t) * heads_per_token);
    const T* row = qkv + static_cast<size_t>(t) * row_stride;
    if (s < n_heads) {
      src = row + static_cast<size_t>(s) * head_dim;
      dst = q_out + (static_cast<size_t>(t) * n_heads + s) * head_dim;
      weight = q_weight;
      rotate = inv_freq != nullptr;
    } else {
      const int slot = slot_map[t];
      const int j = (s - n_heads) % n_kv_heads;
      const bool is_key = (s - n_heads) < n_kv_heads;
      src = row + (static_cast<size_t>(n_heads) + (is_key ? 0 : n_kv_heads) + j) * head_dim;
      if (slot >= 0) {
        T* base = is_key ? k_cache : v_cache;
        dst = base + (static_cast<size_t>(slot) * n_kv_heads + j) * head_dim;
      }
      weight = is_key ? k_weight : nullptr;
      rotate = is_key && inv_freq != nullptr;
    }
  }

  float ss = 0.f;
  if (active) {
    for (int i = lane; i < head_dim; i += PYLON_WAVE) {
      const float v = to_float(src[i]);
      buf[i] = v;
      ss += v * v;
    }
  }
  ss = wave_sum(ss);
  __syncthreads();
  if (active && weight != nullptr) {
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(head_dim) + eps);
    for (int i = lane; i < head_dim; i += PYLON_WAVE) buf[i] = (buf[i] * inv) * weight[i];
  }
  __syncthreads();
  if (active && rotate) {
    const int half = rot_dim / 2;
    const float pos = static_cast<float>(positions[t]);
    for (int i = lane; i < half; i += PYLON_WAVE) {
      const float angle = pos * inv_freq[i];
      const float c = cosf(angle);
      const float sn = sinf(angle);
      const float a = buf[i];
      const float b = buf[i + half];
      buf[i] = a * c - b * sn;
      buf[i + half] = b * c + a * sn;
    }
  }
  __syncthreads();
  if (active && dst != nullptr) {
    for (int i = lane; i < head_dim; i += PYLON_WAVE) dst[i] = from_float<T>(buf[i]);
  }
}

// The same for head sizes that are multiples of 64 with the whole head rotated (or none of
// it): a lane owns head_dim/64 consecutive elements, loads and stores them as one vector,
// and finds its rotation partner (element i + head_dim/2) in lane + 32.  No LDS.
template <typename T, int EPL>
__global__ void qkv_prepare_wide_kernel(T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                        const T* __restrict__ qkv, long long row_stride,
                                        const float* __restrict__ q_weight, const float* __restrict__ k_weight,
                                        float eps, const float* __restrict__ inv_freq,
                                        const int* __restrict__ positions, const int* __restrict__ slot_map,
                                        long long items, int n_heads, int n_kv_heads, int heads_per_token) {
  constexpr int HD = EPL * 64;
  const int lane = threadIdx.x & (PYLON_WAVE - 1);
  const int wave = threadIdx.x / PYLON_WAVE;
  const long long item = static_cast<long long>(blockIdx.x) * QKV_WAVES + wave;
  if (item >= items) return;
  const int t = static_cast<int>(item / heads_per_token);
  const int s = static_cast<int>(item - static_cast<long long>(t) * heads_per_token);
  const T* row = qkv + static_cast<size_t>(t) * row_stride;
  const T* src;
  T* dst = nullptr;
  const float* weight = nullptr;
  bool rotate = false;
  if (s < n_heads) {
    src = row + static_cast<size_t>(s) * HD;
    dst = q_out + (static_cast<size_t>(t) * n_heads + s) * HD;
    weight = q_weight;
    rotate = inv_freq != nullptr;
  } else {
    const int slot = slot_map[t];
    const int j = (s - n_heads) % n_kv_heads;
    const bool is_key = (s - n_heads) < n_kv_heads;
    src = row + (static_cast<size_t>(n_heads) + (is_key ? 0 : n_kv_heads) + j) * HD;
    if (slot >= 0) dst = (is_key ? k_cache : v_cache) + (static_cast<size_t>(slot) * n_kv_heads + j) * HD;
    weight = is_key ? k_weight : nullptr;
    rotate = is_key && inv_freq != nullptr;
  }
  float v[EPL];
  if (sizeof(T) == 2) {
    if (EPL == 1) {
      v[0] = to_float(src[lane]);
    } else if (EPL == 2) {
      const uint32_t two = *reinterpret_cast<const uint32_t*>(src + lane * 2);
      v[0] = __uint_as_float(two << 16);
      v[EPL - 1] = __uint_as_float(two & 0xffff0000u);
    } else {
#pragma unroll
      for (int e = 0; e < EPL; e += 2) {
        const uint32_t two = *reinterpret_cast<const uint32_t*>(src + lane * EPL + e);
        v[e] = __uint_as_float(two << 16);
        v[e + 1 < EPL ? e + 1 : e] = __uint_as_float(two & 0xffff0000u);
      }
    }
  } else {
#pragma unroll
    for (int e = 0; e < EPL; ++e) v[e] = to_float(src[lane * EPL + e]);
  }
  norm_rotate_head<EPL>(v, lane, weight, eps, rotate ? inv_freq : nullptr,
                        rotate ? static_cast<float>(positions[t]) : 0.f);
  if (dst != nullptr) {
#pragma unroll
    for (int e = 0; e < EPL; ++e) dst[lane * EPL + e] = from_float<T>(v[e]);
  }
}

// bfloat16 at head sizes 64/128/256 with the whole head rotated (or none of it): a
// workgroup takes a share of one token's heads.  The token's rotation table is computed once
// into LDS; then each wave prepares 512/head_dim heads at a time with 16-byte accesses.
template <int HD>
__global__ __launch_bounds__(QKV_WAVES* PYLON_WAVE) void qkv_prepare_rows_kernel(
    uint16_t* __restrict__ q_out, uint16_t* __restrict__ k_cache, uint16_t* __restrict__ v_cache,
    const uint16_t* __restrict__ qkv, long long row_stride, const float* __restrict__ q_weight,
    const float* __restrict__ k_weight, float eps, const float* __restrict__ inv_freq,
    const int* __restrict__ positions, const int* __restrict__ slot_map, int n_heads, int n_kv_heads,
    int heads_per_token, int heads_per_block) {
  constexpr int LPH = HD / 8, HPW = PYLON_WAVE / LPH;
  __shared__ float cs[HD];
  const int lane = threadIdx.x & (PYLON_WAVE - 1);
  const int wave = threadIdx.x / PYLON_WAVE;
  const int t = blockIdx.x;
  if (inv_freq != nullptr) {
    rotation_table<HD>(cs, inv_freq, static_cast<float>(positions[t]));
    __syncthreads();
  }
  const int h_begin = blockIdx.y * heads_per_block;
  const int h_end = h_begin + heads_per_block < heads_per_token ? h_begin + heads_per_block : heads_per_token;
  const int slot = heads_per_token > n_heads ? slot_map[t] : -1;
  const uint16_t* row = qkv + static_cast<size_t>(t) * row_stride;
  const int j = lane % LPH;
  for (int h0 = h_begin + wave * HPW; h0 < h_end; h0 += QKV_WAVES * HPW) {
    const int mine = h0 + lane / LPH;
    const bool valid = mine < h_end;
    const int s = valid ? mine : h_end - 1;
    const uint16_t* src = row + static_cast<size_t>(s) * HD + 8 * j;  // heads lie in the order q, k, v
    uint16_t* dst = nullptr;
    const float* weight = nullptr;
    bool rotate = false;
    if (s < n_heads) {
      dst = q_out + (static_cast<size_t>(t) * n_heads + s) * HD + 8 * j;
      weight = q_weight;
      rotate = true;
    } else {
      const bool is_key = s - n_heads < n_kv_heads;
      const int kvh = is_key ? s - n_heads : s - n_heads - n_kv_heads;
      if (slot >= 0) dst = (is_key ? k_cache : v_cache) + (static_cast<size_t>(slot) * n_kv_heads + kvh) * HD + 8 * j;
      weight = is_key ? k_weight : nullptr;
      rotate = is_key;
    }
    float v[8];
    load8_bf16(src, v);
    norm_rotate8<HD>(v, j, weight, eps, (rotate && inv_freq != nullptr) ? cs : nullptr);
    if (valid && dst != nullptr) store8_bf16(dst, v);
  }
}

static bool launch_rows(uint16_t* q_out, uint16_t* k_cache, uint16_t* v_cache, const uint16_t* qkv,
                        long long row_stride, const float* q_weight, const float* k_weight, float eps,
                        const float* inv_freq, const int* positions, const int* slot_map, int tokens,
                        int n_heads, int n_kv_heads, int head_dim, int heads_per_token, hipStream_t stream) {
  // enough workgroups to fill the chip when there are few tokens
  const int per_round = QKV_WAVES * (512 / head_dim);  // heads a workgroup prepares at a time
  int shares = 1;
  while (tokens * shares < 1024 && shares * per_round < heads_per_token) shares *= 2;
  int heads_per_block = (heads_per_token + shares - 1) / shares;
  heads_per_block = (heads_per_block + per_round - 1) / per_round * per_round;
  shares = (heads_per_token + heads_per_block - 1) / heads_per_block;
  dim3 grid(tokens, shares), block(QKV_WAVES * PYLON_WAVE);
#define GO(HD)                                                                                          \
  hipLaunchKernelGGL((qkv_prepare_rows_kernel<HD>), grid, block, 0, stream, q_out, k_cache, v_cache, qkv, \
                     row_stride, q_weight, k_weight, eps, inv_freq, positions, slot_map, n_heads,       \
                     n_kv_heads, heads_per_token, heads_per_block)
  switch (head_dim) {
    case 64: GO(64); return true;
    case 128: GO(128); return true;
    case 256: GO(256); return true;
    default: return false;
  }
#undef GO
}

template <typename T>
static bool launch_wide(T* q_out, T* k_cache, T* v_cache, const T* qkv, long long row_stride,
                        const float* q_weight, const float* k_weight, float eps, const float* inv_freq,
                        const int* positions, const int* slot_map, long long items, int n_heads,
                        int n_kv_heads, int head_dim, int heads_per_token, dim3 grid, dim3 block,
                        hipStream_t stream) {
#define GO(EPL)                                                                                       \
  hipLaunchKernelGGL((qkv_prepare_wide_kernel<T, EPL>), grid, block, 0, stream, q_out, k_cache,       \
                     v_cache, qkv, row_stride, q_weight, k_weight, eps, inv_freq, positions, slot_map, \
                     items, n_heads, n_kv_heads, heads_per_token)
  switch (head_dim) {
    case 64: GO(1); return true;
    case 128: GO(2); return true;
    case 256: GO(4); return true;
    default: return false;
  }
#undef GO
}

// qkv: [tokens, row_stride] with q heads first, then (if store_kv) k heads, then v heads.
// q_out: [tokens, n_heads, head_dim]. k_cache/v_cache: [slots, n_kv_heads, head_dim] where a
// slot is page*page_size + offset; slot_map[t] < 0 stores nothing for token t.
extern "C" int pylon_qkv_prepare(void* q_out, void* k_cache, void* v_cache, const void* qkv, int dtype,
                                 long long row_stride, const float* q_weight, const float* k_weight,
                                 float eps, const float* inv_freq, int rot_dim, const int* positions,
                                 const int* slot_map, int tokens, int n_heads, int n_kv_heads,
                                 int head_dim, int store_kv, hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(dtype), "qkv_prepare: unknown dtype");
  PYLON_REQUIRE(tokens >= 0 && n_heads > 0 && n_kv_heads > 0, "qkv_prepare: bad head counts");
  PYLON_REQUIRE(head_dim > 0 && head_dim <= 1024, "qkv_prepare: head_dim %d is outside 1..1024", head_dim);
  const int heads_per_token = n_heads + (store_kv ? 2 * n_kv_heads : 0);
  PYLON_REQUIRE(row_stride >= static_cast<long long>(heads_per_token) * head_dim,
                "qkv_prepare: row stride %lld is shorter than %d heads of %d", row_stride,
                heads_per_token, head_dim);
  if (inv_freq != nullptr) {
    PYLON_REQUIRE(rot_dim > 0 && rot_dim % 2 == 0 && rot_dim <= head_dim,
                  "qkv_prepare: rotary dim %d must be even and at most head_dim %d", rot_dim, head_dim);
    PYLON_REQUIRE(positions != nullptr, "qkv_prepare: rotary encoding needs positions");
  }
  if (store_kv) PYLON_REQUIRE(k_cache && v_cache && slot_map, "qkv_prepare: storing k/v needs the cache and a slot map");
  if (tokens == 0) return 0;
  const long long items = static_cast<long long>(tokens) * heads_per_token;
  const long long blocks = (items + QKV_WAVES - 1) / QKV_WAVES;
  PYLON_REQUIRE(blocks < (1ll << 31), "qkv_prepare: too many heads to process in one launch");
  dim3 grid((unsigned)blocks), block(QKV_WAVES * PYLON_WAVE);
  const size_t lds = sizeof(float) * QKV_WAVES * head_dim;
  // whole-head rotation (or none) at head sizes 64/128/256 takes the vector form
  if ((inv_freq == nullptr || rot_dim == head_dim) && row_stride % 2 == 0) {
    bool done;
    const bool vectors = dtype == PYLON_BF16 && row_stride % 8 == 0 &&
                         (reinterpret_cast<uintptr_t>(qkv) & 15) == 0 &&
                         (reinterpret_cast<uintptr_t>(q_out) & 15) == 0;
    if (vectors)
      done = launch_rows((uint16_t*)q_out, (uint16_t*)k_cache, (uint16_t*)v_cache, (const uint16_t*)qkv,
                         row_stride, q_weight, k_weight, eps, inv_freq, positions, slot_map, tokens, n_heads,
                         n_kv_heads, head_dim, heads_per_token, stream);
    else if (dtype == PYLON_F32)
      done = launch_wide<float>((float*)q_out, (float*)k_cache, (float*)v_cache, (const float*)qkv, row_stride,
                                q_weight, k_weight, eps, inv_freq, positions, slot_map, items, n_heads,
                                n_kv_heads, head_dim, heads_per_token, grid, block, stream);
    else
      done = launch_wide<bf16_t>((bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, (const bf16_t*)qkv,
                                 row_stride, q_weight, k_weight, eps, inv_freq, positions, slot_map, items,
                                 n_heads, n_kv_heads, head_dim, heads_per_token, grid, block, stream);
    if (done) PYLON_LAUNCHED("qkv_prepare");
  }
  if (dtype == PYLON_F32)
    hipLaunchKernelGGL(qkv_prepare_kernel<float>, grid, block, lds, stream, (float*)q_out, (float*)k_cache,
                       (float*)v_cache, (const float*)qkv, row_stride, q_weight, k_weight, eps, inv_freq,
                       rot_dim, positions, slot_map, items, n_heads, n_kv_heads, head_dim, heads_per_token);
  else
    hipLaunchKernelGGL(qkv_prepare_kernel<bf16_t>, grid, block, lds, stream, (bf16_t*)q_out,
                       (bf16_t*)k_cache, (bf16_t*)v_cache, (const bf16_t*)qkv, row_stride, q_weight,
                       k_weight, eps, inv_freq, rot_dim, positions, slot_map, items, n_heads, n_kv_heads,
                       head_dim, heads_per_token);
  PYLON_LAUNCHED("qkv_prepare");
}
