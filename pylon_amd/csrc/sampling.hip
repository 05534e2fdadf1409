// Choosing the next token from float logits, one workgroup per row:
//   temperature 0  -> the index of the largest logit (the lowest index among equals);
//   temperature T  -> p = softmax(logits / T); with top_p < 1 only tokens whose
//                     strictly-more-likely mass is at most top_p are kept; the token is
//                     read off the cumulative distribution (in index order) at u in [0,1).
// The uniform number u comes from the host, one per row, so that a request's random
// stream does not depend on what else is in the batch.
#include "common.h"

#define SAMPLE_THREADS 1024

// Order-preserving map from float to unsigned: a < b  <=>  key(a) < key(b).
__device__ __forceinline__ uint32_t float_key(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct ArgBest {
  float value;
  int index;
};

__device__ __forceinline__ ArgBest better(ArgBest a, ArgBest b) {
  if (b.value > a.value || (b.value == a.value && b.index < a.index)) return b;
  return a;
}

__device__ int block_argmax(const float* __restrict__ row, int vocab, ArgBest* scratch) {
  ArgBest best = {-INFINITY, 0x7fffffff};
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
    const float v = row[i];
    if (v > best.value || best.index == 0x7fffffff) best = {v, i};
  }
  for (int off = PYLON_WAVE / 2; off > 0; off >>= 1) {
    ArgBest other;
    other.value = __shfl_xor(best.value, off, PYLON_WAVE);
    other.index = __shfl_xor(best.index, off, PYLON_WAVE);
    best = better(best, other);
  }
  const int lane = threadIdx.x & (PYLON_WAVE - 1), wave = threadIdx.x / PYLON_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = best;
  __syncthreads();
  ArgBest total = scratch[0];
  const int nwaves = (blockDim.x + PYLON_WAVE - 1) / PYLON_WAVE;
  for (int i = 1; i < nwaves; ++i) total = better(total, scratch[i]);
  return total.index;
}

// The chosen id goes to out[row] and, if asked for, also to chosen[place[row]]: a table
// with one entry per request from which the next step's embedding can take its token.
__device__ __forceinline__ void emit(int* __restrict__ out, int* __restrict__ chosen,
                                     const int* __restrict__ place, int row, int id) {
  out[row] = id;
  if (chosen != nullptr) chosen[place[row]] = id;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void argmax_kernel(int* __restrict__ out,
                                                                const float* __restrict__ logits,
                                                                int vocab, long long row_stride,
                                                                int* __restrict__ chosen,
                                                                const int* __restrict__ place) {
  __shared__ ArgBest scratch[16];
  const float* row = logits + static_cast<size_t>(blockIdx.x) * row_stride;
  const int idx = block_argmax(row, vocab, scratch);
  if (threadIdx.x == 0) emit(out, chosen, place, blockIdx.x, idx);
}

// chosen and place are both null or both given (place: one index into chosen per row).
extern "C" int pylon_argmax(int* out, const float* logits, int rows, int vocab, long long row_stride,
                            int* chosen, const int* place, hipStream_t stream) {
  PYLON_REQUIRE((chosen == nullptr) == (place == nullptr), "argmax: chosen and place go together");
  PYLON_REQUIRE(rows >= 0 && vocab > 0 && row_stride >= vocab, "argmax: bad sizes rows=%d vocab=%d", rows, vocab);
  if (rows == 0) return 0;
  hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, out, logits, vocab,
                     row_stride, chosen, place);
  PYLON_LAUNCHED("argmax");
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    int* __restrict__ out, const float* __restrict__ logits, int vocab, long long row_stride,
    const float* __restrict__ temperature, const float* __restrict__ top_p,
    const float* __restrict__ uniform, int* __restrict__ chosen, const int* __restrict__ place) {
  __shared__ ArgBest best_scratch[16];
  __shared__ float scratch[16];
  __shared__ float wave_totals[16];
  __shared__ int found;
  const int r = blockIdx.x;
  const float* row = logits + static_cast<size_t>(r) * row_stride;
  const float temp = temperature[r];
  if (temp <= 0.f) {
    const int idx = block_argmax(row, vocab, best_scratch);
    if (threadIdx.x == 0) emit(out, chosen, place, r, idx);
    return;
  }
  const float inv_temp = 1.0f / temp;
  float mx = -INFINITY;
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) mx = fmaxf(mx, row[i]);
  mx = block_max(mx, scratch);
  float z = 0.f;
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) z += expf((row[i] - mx) * inv_temp);
  z = block_sum(z, scratch);

  uint32_t threshold = 0;  // tokens with key >= threshold are kept
  float kept_mass = z;
  const float p = top_p[r];
  if (p < 1.0f) {
    const float target = p * z;
    uint32_t lo = 0, hi = float_key(mx);
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo) / 2;
      float above = 0.f;
      for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
        const float v = row[i];
        if (float_key(v) > mid) above += expf((v - mx) * inv_temp);
      }
      above = block_sum(above, scratch);
      if (above <= target)
        hi = mid;
      else
        lo = mid + 1;
    }
    threshold = lo;
    float kept = 0.f;
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
      const float v = row[i];
      if (float_key(v) >= threshold) kept += expf((v - mx) * inv_temp);
    }
    kept_mass = block_sum(kept, scratch);
  }

  const float target = uniform[r] * kept_mass;
  if (threadIdx.x == 0) found = 0x7fffffff;
  __syncthreads();
  const int lane = threadIdx.x & (PYLON_WAVE - 1), wave = threadIdx.x / PYLON_WAVE;
  const int nwaves = blockDim.x / PYLON_WAVE;
  float running = 0.f;
  int last_kept = -1;
  for (int base = 0; base < vocab; base += blockDim.x) {
    const int i = base + threadIdx.x;
    float e = 0.f;
    if (i < vocab) {
      const float v = row[i];
      if (float_key(v) >= threshold) {
        e = expf((v - mx) * inv_temp);
        last_kept = i;
      }
    }
    // inclusive scan over the workgroup
    float scan = e;
    for (int off = 1; off < PYLON_WAVE; off <<= 1) {
      const float up = __shfl_up(scan, off, PYLON_WAVE);
      if (lane >= off) scan += up;
    }
    if (lane == PYLON_WAVE - 1) wave_totals[wave] = scan;
    __syncthreads();
    float before = running;
    for (int wv = 0; wv < wave; ++wv) before += wave_totals[wv];
    float tile_total = 0.f;
    for (int wv = 0; wv < nwaves; ++wv) tile_total += wave_totals[wv];
    const float cum = before + scan;
    if (e > 0.f && cum > target) atomicMin(&found, i);
    __syncthreads();
    if (found != 0x7fffffff) break;
    running += tile_total;
  }
  if (found == 0x7fffffff) {
    // Rounding left the cumulative sum just below the target: take the last kept token.
    int lk = last_kept;
    for (int off = PYLON_WAVE / 2; off > 0; off >>= 1) lk = max(lk, __shfl_xor(lk, off, PYLON_WAVE));
    __shared__ int last_scratch[16];
    if (lane == 0) last_scratch[wave] = lk;
    __syncthreads();
    if (threadIdx.x == 0) {
      int v = -1;
      for (int wv = 0; wv < nwaves; ++wv) v = max(v, last_scratch[wv]);
      emit(out, chosen, place, r, v < 0 ? 0 : v);
    }
  } else if (threadIdx.x == 0) {
    emit(out, chosen, place, r, found);
  }
}

extern "C" int pylon_sample(int* out, const float* logits, int rows, int vocab, long long row_stride,
                            const float* temperature, const float* top_p, const float* uniform,
                            int* chosen, const int* place, hipStream_t stream) {
  PYLON_REQUIRE((chosen == nullptr) == (place == nullptr), "sample: chosen and place go together");
  PYLON_REQUIRE(rows >= 0 && vocab > 0 && row_stride >= vocab, "sample: bad sizes rows=%d vocab=%d", rows, vocab);
  PYLON_REQUIRE(temperature && top_p && uniform, "sample: temperature, top_p and uniform are required");
  if (rows == 0) return 0;
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, out, logits, vocab,
                     row_stride, temperature, top_p, uniform, chosen, place);
  PYLON_LAUNCHED("sample");
}
