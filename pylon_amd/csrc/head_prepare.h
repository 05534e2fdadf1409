// One wavefront prepares one head of a token's q/k/v projection: per-head RMSNorm (if a
// weight is given) and the rotation of element i with element i + head_dim/2 (if
// frequencies are given), in float.  Head sizes are multiples of 64; a lane owns
// head_dim/64 consecutive elements and finds its rotation partner in lane + 32.
#pragma once
#include "common.h"

// src: head_dim bf16 values (4-byte aligned for EPL >= 2).  On return v[e] is element
// lane*EPL + e.
template <int EPL>
__device__ __forceinline__ void load_head_bf16(const uint16_t* __restrict__ src, int lane, float v[EPL]) {
  if (EPL == 1) {
    v[0] = __uint_as_float(static_cast<uint32_t>(src[lane]) << 16);
  } else {
#pragma unroll
    for (int e = 0; e < EPL; e += 2) {
      const uint32_t two = *reinterpret_cast<const uint32_t*>(src + lane * EPL + e);
      v[e] = __uint_as_float(two << 16);
      v[e + 1 < EPL ? e + 1 : e] = __uint_as_float(two & 0xffff0000u);
    }
  }
}

template <int EPL>
__device__ __forceinline__ void norm_rotate_head(float v[EPL], int lane, const float* __restrict__ weight,
                                                 float eps, const float* __restrict__ inv_freq, float pos) {
  constexpr int HD = EPL * 64;
  if (weight != nullptr) {
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < EPL; ++e) ss += v[e] * v[e];
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(HD) + eps);
#pragma unroll
    for (int e = 0; e < EPL; ++e) v[e] = (v[e] * inv) * weight[lane * EPL + e];
  }
  if (inv_freq != nullptr) {
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      const float other = __shfl_xor(v[e], 32, PYLON_WAVE);
      const int pair = (lane & 31) * EPL + e;  // index of the (i, i + HD/2) pair
      const float angle = pos * inv_freq[pair];
      const float c = cosf(angle), sn = sinf(angle);
      v[e] = (lane < 32) ? v[e] * c - other * sn : v[e] * c + other * sn;
    }
  }
}

// dst: head_dim bf16 values (4-byte aligned for EPL >= 2).
template <int EPL>
__device__ __forceinline__ void store_head_bf16(uint16_t* __restrict__ dst, int lane, const float v[EPL]) {
  if (EPL == 1) {
    dst[lane] = float_to_bf16_bits(v[0]);
  } else {
#pragma unroll
    for (int e = 0; e < EPL; e += 2) {
      const uint32_t lo = float_to_bf16_bits(v[e]), hi = float_to_bf16_bits(v[e + 1 < EPL ? e + 1 : e]);
      *reinterpret_cast<uint32_t*>(dst + lane * EPL + e) = lo | (hi << 16);
    }
  }
}

// ---- the same for bfloat16 with 16-byte accesses -----------------------------------------
// head_dim/8 lanes share a head, 8 consecutive elements each, so a wavefront prepares
// 512/head_dim heads at once.  j is the lane's index within its head (lane % (HD/8)).
// Every lane of the wave must call these together (they exchange values inside a head).

// cos(pos * f_i) and sin(pos * f_i) for the HD/2 rotation pairs of one token, by the whole
// workgroup: cs[i] and cs[HD/2 + i].  A barrier must follow before cs is read.
template <int HD>
__device__ __forceinline__ void rotation_table(float* __restrict__ cs, const float* __restrict__ inv_freq, float pos) {
  for (int i = threadIdx.x; i < HD / 2; i += blockDim.x) {
    const float angle = pos * inv_freq[i];
    cs[i] = cosf(angle);
    cs[HD / 2 + i] = sinf(angle);
  }
}

__device__ __forceinline__ void load8_bf16(const uint16_t* __restrict__ src, float v[8]) {
  const uint4 raw = *reinterpret_cast<const uint4*>(src);
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(w[i] << 16);
    v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}

// v = the sum of n_parts float vectors of 8 (32-byte aligned), stride elements apart, added in
// order and rounded to bfloat16 once.  For the usual counts every load is issued before the
// first addition.
__device__ __forceinline__ void sum8_parts(const float* __restrict__ src, int n_parts, long long stride, float v[8]) {
  auto take = [&](int p, float4& a, float4& b) {
    const float4* at = reinterpret_cast<const float4*>(src + p * stride);
    a = at[0], b = at[1];
  };
  float4 lo, hi;
  if (n_parts == 2 || n_parts == 4) {
    float4 a[4], b[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) take(p < n_parts ? p : 0, a[p], b[p]);
    lo = a[0], hi = b[0];
#pragma unroll
    for (int p = 1; p < 4; ++p) {
      if (p < n_parts) {
        lo.x += a[p].x, lo.y += a[p].y, lo.z += a[p].z, lo.w += a[p].w;
        hi.x += b[p].x, hi.y += b[p].y, hi.z += b[p].z, hi.w += b[p].w;
      }
    }
  } else {
    take(0, lo, hi);
    for (int p = 1; p < n_parts; ++p) {
      float4 a, b;
      take(p, a, b);
      lo.x += a.x, lo.y += a.y, lo.z += a.z, lo.w += a.w;
      hi.x += b.x, hi.y += b.y, hi.z += b.z, hi.w += b.w;
    }
  }
  const float sums[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = __uint_as_float(static_cast<uint32_t>(float_to_bf16_bits(sums[e])) << 16);
}

__device__ __forceinline__ void store8_bf16(uint16_t* __restrict__ dst, const float v[8]) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    w[i] = static_cast<uint32_t>(float_to_bf16_bits(v[2 * i])) |
           (static_cast<uint32_t>(float_to_bf16_bits(v[2 * i + 1])) << 16);
  *reinterpret_cast<uint4*>(dst) = uint4{w[0], w[1], w[2], w[3]};
}

// v: elements 8j .. 8j+7 of a head.  weight: the head's RMSNorm weight or null (per lane:
// heads in one wave may differ).  cs: the token's rotation table or null.
template <int HD>
__device__ __forceinline__ void norm_rotate8(float v[8], int j, const float* __restrict__ weight, float eps,
                                             const float* __restrict__ cs) {
  constexpr int LPH = HD / 8;
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) ss += v[e] * v[e];
#pragma unroll
  for (int off = 1; off < LPH; off <<= 1) ss += __shfl_xor(ss, off, PYLON_WAVE);
  if (weight != nullptr) {
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(HD) + eps);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (v[e] * inv) * weight[8 * j + e];
  }
  const bool rotate = cs != nullptr;
  const bool low = j < LPH / 2;
  const int pair0 = 8 * (j & (LPH / 2 - 1));
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float other = __shfl_xor(v[e], LPH / 2, PYLON_WAVE);
    if (rotate) {
      const float c = cs[pair0 + e], sn = cs[HD / 2 + pair0 + e];
      v[e] = low ? v[e] * c - other * sn : v[e] * c + other * sn;
    }
  }
}
