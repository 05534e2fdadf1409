// Shared helpers of the gfx950 kernels: element types, wave-level reductions, and the
// error convention of the C entry points (0 = launched, non-zero = refused, with the
// reason in pylon_last_error()).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define PYLON_WAVE 64

// Element type codes shared with the Python side.
enum PylonDtype { PYLON_F32 = 0, PYLON_BF16 = 1 };

// bfloat16 is carried as its raw 16 bits; all arithmetic is done in float.
struct bf16_t {
  uint16_t bits;
};

__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) {
  return __uint_as_float(static_cast<uint32_t>(b) << 16);
}

// Round to nearest, ties to even; NaN stays NaN.
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) { return bf16_bits_to_float(v.bits); }

template <typename T>
__device__ __forceinline__ T from_float(float v);
template <>
__device__ __forceinline__ float from_float<float>(float v) {
  return v;
}
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float v) {
  bf16_t r;
  r.bits = float_to_bf16_bits(v);
  return r;
}

// Sum / max over the 64 lanes of a wavefront; every lane gets the result.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = PYLON_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, PYLON_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = PYLON_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, PYLON_WAVE));
  return v;
}

// Sum over a workgroup of up to 1024 threads. `scratch` holds >= 16 floats of LDS.
// Every thread gets the result; the order of additions depends only on blockDim.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (PYLON_WAVE - 1);
  const int wave = threadIdx.x / PYLON_WAVE;
  const int nwaves = (blockDim.x + PYLON_WAVE - 1) / PYLON_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int i = 0; i < nwaves; ++i) total += scratch[i];
  return total;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x & (PYLON_WAVE - 1);
  const int wave = threadIdx.x / PYLON_WAVE;
  const int nwaves = (blockDim.x + PYLON_WAVE - 1) / PYLON_WAVE;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = scratch[0];
  for (int i = 1; i < nwaves; ++i) total = fmaxf(total, scratch[i]);
  return total;
}

// ---- host side -------------------------------------------------------------------

extern thread_local char pylon_error_text[512];

#define PYLON_REFUSE(...)                                              \
  do {                                                                 \
    snprintf(pylon_error_text, sizeof(pylon_error_text), __VA_ARGS__); \
    return 1;                                                          \
  } while (0)

#define PYLON_REQUIRE(cond, ...)       \
  do {                                 \
    if (!(cond)) PYLON_REFUSE(__VA_ARGS__); \
  } while (0)

// After a launch: report a launch error (bad configuration and the like) as a refusal.
#define PYLON_LAUNCHED(name)                                                          \
  do {                                                                                \
    hipError_t e_ = hipGetLastError();                                                \
    if (e_ != hipSuccess) {                                                           \
      snprintf(pylon_error_text, sizeof(pylon_error_text), "%s: launch failed: %s",   \
               name, hipGetErrorString(e_));                                          \
      return 2;                                                                       \
    }                                                                                 \
    return 0;                                                                         \
  } while (0)

// Compute units of the current device (0 if there is none); asked of the runtime once per device.
extern "C" int pylon_compute_units();

static inline bool pylon_valid_dtype(int d) { return d == PYLON_F32 || d == PYLON_BF16; }
static inline size_t pylon_dtype_size(int d) { return d == PYLON_F32 ? 4 : 2; }
