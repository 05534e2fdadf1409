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
