// Choosing the next token from float logits:
//   temperature 0  -> the index of the largest logit (the lowest index among equals);
//   temperature T  -> p = softmax(logits / T); with top_p < 1 only tokens whose
//                     strictly-more-likely mass is at most top_p are kept; the token is
//                     read off the cumulative distribution (in index order) at u in [0,1).
// The uniform number u comes from the host, one per row, so that a request's random
// stream does not depend on what else is in the batch.
//
// Probability masses are summed as 64-bit fixed-point integers (exp(.) * 2^40): integer
// sums do not depend on the order of addition, so the kept set and the chosen token are
// the same on every run, however the work is spread over threads, and no rounding can
// leave the cumulative sum short of its target.
//
// argmax alone runs in two launches, many workgroups per row and then a merge.  sample
// runs one workgroup per row; its sixteen waves each walk one stretch of the row, and what
// bounds a pass is the arithmetic per element, not the reading:
//   1. the maximum;
//   2. the mass of every stretch and, for top_p < 1, a histogram of mass over 2048 bins that
//      are monotone in the logit, which names the one bin the top-p boundary falls into;
//   3. the tokens of that bin are gathered in LDS (beside them, per stretch, the mass of the
//      bins before) and the exact boundary key is found there by bisection (if they do not
//      fit, by bisection with passes over the row);
//   4. the cumulative mass of kept tokens in index order: the stretch by the totals that the
//      earlier passes left, then a sixteenth of it, then a scan.
#include "common.h"
#include "no_alloc.h"

#include <mutex>

typedef unsigned long long u64;

#define SAMPLE_THREADS 1024
#define SAMPLE_WAVES (SAMPLE_THREADS / PYLON_WAVE)
#define ARGMAX_THREADS 256
#define ARGMAX_MAX_CHUNKS 64
#define ARGMAX_MIN_CHUNK 1024
#define BINS 2048
#define CANDIDATES 4096
#define FIXED_ONE 1099511627776.0f  // 2^40
// exp(-28) * 2^40 < 1: a token that far below the maximum has no mass in fixed point.
#define BIN_RANGE 28.0f

// Order-preserving map from float to unsigned: a < b  <=>  key(a) < key(b).
__device__ __forceinline__ uint32_t float_key(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ float clean(float x) { return x != x ? -INFINITY : x; }

struct ArgBest {
  float value;
  int index;
};

__device__ __forceinline__ ArgBest better(ArgBest a, ArgBest b) {
  if (b.value > a.value || (b.value == a.value && b.index < a.index)) return b;
  return a;
}

// f(value, index) for every element of row[begin, end), spread over the workgroup's
// threads in no particular order, with 16-byte loads where the address allows.
template <typename F>
__device__ __forceinline__ void for_each(const float* __restrict__ row, int begin, int end, F f) {
  const float* p = row + begin;
  const int n = end - begin;
  int head = static_cast<int>((4 - ((reinterpret_cast<uintptr_t>(p) >> 2) & 3)) & 3);
  if (head > n) head = n;
  if (static_cast<int>(threadIdx.x) < head) f(p[threadIdx.x], begin + static_cast<int>(threadIdx.x));
  const float4* v = reinterpret_cast<const float4*>(p + head);
  const int nv = (n - head) >> 2;
  // Eight loads of a thread are issued before the first of them is used: a workgroup alone on
  // its compute unit is bound by what it has in flight.
  constexpr int DEPTH = 8;
  for (int i0 = threadIdx.x; i0 < nv; i0 += DEPTH * blockDim.x) {
    float4 q[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int i = i0 + d * blockDim.x;
      q[d] = v[i < nv ? i : i0];
    }
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int i = i0 + d * blockDim.x;
      if (i < nv) {
        const int base = begin + head + 4 * i;
        f(q[d].x, base);
        f(q[d].y, base + 1);
        f(q[d].z, base + 2);
        f(q[d].w, base + 3);
      }
    }
  }
  const int tail = head + 4 * nv;
  if (static_cast<int>(threadIdx.x) < n - tail)
    f(p[tail + threadIdx.x], begin + tail + static_cast<int>(threadIdx.x));
}

// The largest element of row[begin, end) and its lowest index, for every thread.
// NaN counts as -inf; an empty or all -inf range gives index 0x7fffffff or its first index.
__device__ ArgBest block_argbest(const float* __restrict__ row, int begin, int end, ArgBest* scratch) {
  ArgBest best = {-INFINITY, 0x7fffffff};
  for_each(row, begin, end, [&](float v, int i) {
    v = clean(v);
    if (v > best.value || (v == best.value && i < best.index)) best = {v, i};
  });
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
  return total;
}

// The chosen id goes to out[row] and, if asked for, also to chosen[place[row]]: a table
// with one entry per request from which the next step's embedding can take its token.
__device__ __forceinline__ void emit(int* __restrict__ out, int* __restrict__ chosen,
                                     const int* __restrict__ place, int row, int id) {
  out[row] = id;
  if (chosen != nullptr) chosen[place[row]] = id;
}

// ---- argmax: many workgroups per row, then a merge -------------------------------------
__global__ __launch_bounds__(ARGMAX_THREADS) void argmax_partial_kernel(
    ArgBest* __restrict__ partial, const float* __restrict__ logits, int vocab, long long row_stride,
    int chunk_len) {
  __shared__ ArgBest scratch[ARGMAX_THREADS / PYLON_WAVE];
  const int r = blockIdx.y, c = blockIdx.x;
  const float* row = logits + static_cast<size_t>(r) * row_stride;
  const int begin = c * chunk_len;
  const int end = begin + chunk_len < vocab ? begin + chunk_len : vocab;
  const ArgBest best = block_argbest(row, begin, end, scratch);
  if (threadIdx.x == 0) partial[static_cast<size_t>(r) * gridDim.x + c] = best;
}

__global__ __launch_bounds__(PYLON_WAVE) void argmax_merge_kernel(
    int* __restrict__ out, const ArgBest* __restrict__ partial, int chunks, int* __restrict__ chosen,
    const int* __restrict__ place) {
  const int r = blockIdx.x;
  ArgBest best = {-INFINITY, 0x7fffffff};
  for (int c = threadIdx.x; c < chunks; c += PYLON_WAVE)
    best = better(best, partial[static_cast<size_t>(r) * chunks + c]);
  for (int off = PYLON_WAVE / 2; off > 0; off >>= 1) {
    ArgBest other;
    other.value = __shfl_xor(best.value, off, PYLON_WAVE);
    other.index = __shfl_xor(best.index, off, PYLON_WAVE);
    best = better(best, other);
  }
  if (threadIdx.x == 0) emit(out, chosen, place, r, best.index == 0x7fffffff ? 0 : best.index);
}

extern "C" long long pylon_argmax_scratch_bytes(int rows) {
  return static_cast<long long>(rows > 0 ? rows : 0) * ARGMAX_MAX_CHUNKS * sizeof(ArgBest);
}

// chosen and place are both null or both given (place: one index into chosen per row).
// scratch: device memory of at least pylon_argmax_scratch_bytes(rows) bytes.
extern "C" int pylon_argmax(int* out, const float* logits, int rows, int vocab, long long row_stride,
                            int* chosen, const int* place, void* scratch, long long scratch_bytes,
                            hipStream_t stream) {
  PYLON_REQUIRE((chosen == nullptr) == (place == nullptr), "argmax: chosen and place go together");
  PYLON_REQUIRE(rows >= 0 && vocab > 0 && row_stride >= vocab, "argmax: bad sizes rows=%d vocab=%d", rows, vocab);
  if (rows == 0) return 0;
  PYLON_REQUIRE(rows <= 65535, "argmax: at most 65535 rows, got %d", rows);
  PYLON_REQUIRE(scratch != nullptr && scratch_bytes >= pylon_argmax_scratch_bytes(rows),
                "argmax: scratch must hold %lld bytes", pylon_argmax_scratch_bytes(rows));
  int chunks = vocab / ARGMAX_MIN_CHUNK;
  chunks = chunks < 1 ? 1 : (chunks > ARGMAX_MAX_CHUNKS ? ARGMAX_MAX_CHUNKS : chunks);
  const int chunk_len = (((vocab + chunks - 1) / chunks) + 3) & ~3;
  chunks = (vocab + chunk_len - 1) / chunk_len;
  hipLaunchKernelGGL(argmax_partial_kernel, dim3(chunks, rows), dim3(ARGMAX_THREADS), 0, stream,
                     static_cast<ArgBest*>(scratch), logits, vocab, row_stride, chunk_len);
  hipLaunchKernelGGL(argmax_merge_kernel, dim3(rows), dim3(PYLON_WAVE), 0, stream, out,
                     static_cast<const ArgBest*>(scratch), chunks, chosen, place);
  PYLON_LAUNCHED("argmax");
}

// ---- argmax without a scratch argument -----------------------------------------------------
// The first launch's partial results in an array of the library's own.  In host code the
// array's name is only a stand-in for the symbol; the address on a device comes from
// hipGetSymbolAddress, once per device, and only that address is handed to kernels.
static __device__ __align__(256) unsigned char scratch[PYLON_ARGMAX_STATIC_MAX_ROWS * ARGMAX_MAX_CHUNKS *
                                                        sizeof(ArgBest)];
#define STATIC_MAX_DEVICES 64
static void* static_scratch_ptr[STATIC_MAX_DEVICES];  // by device ordinal; null: not resolved yet
static std::mutex static_scratch_lock;

static int static_scratch(void** ptr) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) PYLON_REFUSE("argmax_static: no current device: %s", hipGetErrorString(e));
  PYLON_REQUIRE(dev >= 0 && dev < STATIC_MAX_DEVICES, "argmax_static: device ordinal %d is beyond %d", dev,
                STATIC_MAX_DEVICES);
  std::lock_guard<std::mutex> guard(static_scratch_lock);
  if (static_scratch_ptr[dev] == nullptr) {
    void* found = nullptr;
    e = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
    if (e != hipSuccess || found == nullptr)
      PYLON_REFUSE("argmax_static: the scratch array has no address on device %d: %s", dev, hipGetErrorString(e));
    static_scratch_ptr[dev] = found;
  }
  *ptr = static_scratch_ptr[dev];
  return 0;
}

extern "C" int pylon_argmax_static_init(void) {
  void* ptr = nullptr;
  return static_scratch(&ptr);
}

extern "C" int pylon_argmax_static(int* out, const float* logits, int rows, int vocab, long long row_stride,
                                   int* chosen, const int* place, hipStream_t stream) {
  PYLON_REQUIRE(rows <= PYLON_ARGMAX_STATIC_MAX_ROWS,
                "argmax_static: takes at most %d rows (the size of its fixed scratch array), got %d",
                PYLON_ARGMAX_STATIC_MAX_ROWS, rows);
  void* ptr = nullptr;
  if (static_scratch(&ptr)) return 1;
  return pylon_argmax(out, logits, rows, vocab, row_stride, chosen, place, ptr,
                      static_cast<long long>(sizeof(scratch)), stream);
}

// ---- sample ------------------------------------------------------------------------------
__device__ __forceinline__ u64 wave_sum_u64(u64 v) {
#pragma unroll
  for (int off = PYLON_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, PYLON_WAVE);
  return v;
}

// Sum over the workgroup, for every thread.  `scratch` holds SAMPLE_WAVES values.
__device__ __forceinline__ u64 block_sum_u64(u64 v, u64* scratch) {
  const int lane = threadIdx.x & (PYLON_WAVE - 1), wave = threadIdx.x / PYLON_WAVE;
  v = wave_sum_u64(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  u64 total = 0;
  for (int i = 0; i < SAMPLE_WAVES; ++i) total += scratch[i];
  return total;
}

// floor(f) for 0 <= f <= 2^40, in five instructions: the upper word by a truncating conversion,
// the rest exactly (f has 24 significant bits), truncated again.
__device__ __forceinline__ u64 floor_u64(float f) {
  const uint32_t hi = static_cast<uint32_t>(f * 0x1p-32f);
  const float rest = fmaf(-static_cast<float>(hi), 0x1p32f, f);
  return (static_cast<u64>(hi) << 32) | static_cast<uint32_t>(rest);
}

// A token's probability mass relative to the most likely one, in units of 2^-40.
// `rate` is log2(e) / temperature.
__device__ __forceinline__ u64 mass_of(float x, float mx, float rate) {
  return floor_u64(__builtin_amdgcn_exp2f((x - mx) * rate) * FIXED_ONE);
}

// Bin 0 holds the most likely tokens; a larger logit never lands in a later bin.
__device__ __forceinline__ int bin_of(float x, float mx, float inv_temp) {
  const float t = (mx - x) * inv_temp * (BINS / BIN_RANGE);
  return t >= static_cast<float>(BINS - 1) ? BINS - 1 : static_cast<int>(t);
}

// Four consecutive logits from index i (a multiple of 4 past an aligned row), -inf past `end`.
__device__ __forceinline__ float4 load_four(const float* __restrict__ row, int i, int end, bool aligned) {
  if (aligned && i + 3 < end) return *reinterpret_cast<const float4*>(row + i);
  float4 v;
  v.x = i < end ? row[i] : -INFINITY;
  v.y = i + 1 < end ? row[i + 1] : -INFINITY;
  v.z = i + 2 < end ? row[i + 2] : -INFINITY;
  v.w = i + 3 < end ? row[i + 3] : -INFINITY;
  return v;
}

// f(value, index) for the elements of row[s0, s1) over the lanes of one wave (s0 a multiple of
// 4), four loads of a lane issued before the first is used.  The last group of four may reach
// past s1: f then sees -inf at an index >= s1.  A wave's 256 consecutive elements are passed
// over where none of them exceeds `above` (NaN does not): the logits of a trained model lie
// mostly far below the largest, where a pass has nothing to do.
template <bool SKIP, typename F>
__device__ __forceinline__ void wave_each(const float* __restrict__ row, int s0, int s1, bool aligned, float above,
                                          F f) {
  const int lane = threadIdx.x & (PYLON_WAVE - 1);
  constexpr int DEPTH = 4, STEP = 4 * PYLON_WAVE;
  for (int i0 = s0 + 4 * lane; i0 < s1; i0 += DEPTH * STEP) {
    float4 q[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) q[d] = load_four(row, i0 + d * STEP, s1, aligned);
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int i = i0 + d * STEP;
      if (SKIP && __ballot(fmaxf(fmaxf(q[d].x, q[d].y), fmaxf(q[d].z, q[d].w)) > above) == 0) continue;
      f(q[d].x, i);
      f(q[d].y, i + 1);
      f(q[d].z, i + 2);
      f(q[d].w, i + 3);
    }
  }
}

// The row is walked in sixteen consecutive stretches, one per wave, the same stretches by which
// pass 4 narrows first: what a wave sums over its stretch in an earlier pass is that level's total.
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    int* __restrict__ out, const float* __restrict__ logits, int vocab, long long row_stride,
    const float* __restrict__ temperature, const float* __restrict__ top_p,
    const float* __restrict__ uniform, int* __restrict__ chosen, const int* __restrict__ place) {
  // The histogram first; once the boundary bin is known, that bin's tokens (key, index, mass).
  __shared__ __align__(16) unsigned char pool[CANDIDATES * (2 * sizeof(uint32_t) + sizeof(u64))];
  __shared__ float max_scratch[SAMPLE_WAVES];
  __shared__ int index_scratch[SAMPLE_WAVES];
  __shared__ u64 sum_scratch[SAMPLE_WAVES];
  __shared__ u64 seg_total[SAMPLE_WAVES];
  __shared__ u64 shared_mass[2];  // [0]: mass in the bins before the boundary bin; [1]: kept mass
  __shared__ int shared_bin;
  __shared__ int cand_count;
  __shared__ uint32_t key_range[2];
  __shared__ uint32_t shared_threshold;

  const int r = blockIdx.x;
  const float* row = logits + static_cast<size_t>(r) * row_stride;
  const int lane = threadIdx.x & (PYLON_WAVE - 1), wave = threadIdx.x / PYLON_WAVE;
  const bool aligned = (reinterpret_cast<uintptr_t>(row) & 15) == 0;
  const float temp = temperature[r];
  int first_seg = (vocab + SAMPLE_WAVES - 1) / SAMPLE_WAVES;
  first_seg = (first_seg + 4 * PYLON_WAVE - 1) / (4 * PYLON_WAVE) * (4 * PYLON_WAVE);
  const int w0 = wave * first_seg < vocab ? wave * first_seg : vocab;  // this wave's stretch
  const int w1 = w0 + first_seg < vocab ? w0 + first_seg : vocab;

  // pass 1: the maximum (NaN counts as -inf: the hardware's maximum passes the other operand)
  float mx = -INFINITY;
  wave_each<false>(row, w0, w1, aligned, 0.f, [&](float x, int) { mx = fmaxf(mx, x); });
  for (int off = PYLON_WAVE / 2; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, PYLON_WAVE));
  if (lane == 0) max_scratch[wave] = mx;
  __syncthreads();
  for (int i = 0; i < SAMPLE_WAVES; ++i) mx = fmaxf(mx, max_scratch[i]);
  // The lowest index that holds the maximum (0 for an empty row): what a row without a
  // temperature takes, and what never leaves out[] unset.
  auto top_index = [&]() -> int {
    int best = 0x7fffffff;
    wave_each<false>(row, w0, w1, aligned, 0.f, [&](float x, int i) {
      if (clean(x) == mx && i < w1 && i < best) best = i;
    });
    for (int off = PYLON_WAVE / 2; off > 0; off >>= 1) {
      const int other = __shfl_xor(best, off, PYLON_WAVE);
      best = other < best ? other : best;
    }
    __syncthreads();
    if (lane == 0) index_scratch[wave] = best;
    __syncthreads();
    for (int i = 0; i < SAMPLE_WAVES; ++i) best = index_scratch[i] < best ? index_scratch[i] : best;
    return best == 0x7fffffff ? 0 : best;
  };
  if (temp <= 0.f || !(mx > -INFINITY) || !(mx < INFINITY)) {
    const int index = top_index();
    if (threadIdx.x == 0) emit(out, chosen, place, r, index);
    return;
  }
  const float inv_temp = 1.0f / temp;
  const float rate = inv_temp * 1.44269504088896340736f;
  const float p = top_p[r];
  const bool restricted = p < 1.0f;

  // pass 2: the mass of every stretch and, for top_p < 1, the histogram
  u64* hist = reinterpret_cast<u64*>(pool);
  if (restricted) {
    for (int b = threadIdx.x; b < BINS; b += SAMPLE_THREADS) hist[b] = 0;
    if (threadIdx.x == 0) {
      cand_count = 0;
      key_range[0] = 0xffffffffu;
      key_range[1] = 0;
    }
    __syncthreads();
  }
  // 2^-41.1 of the largest mass is less than one unit: nothing at or below this logit has mass
  const float massless = mx - 28.5f * temp;
  u64 zq = 0;
  wave_each<true>(row, w0, w1, aligned, massless, [&](float x, int) {
    x = clean(x);
    const u64 q = mass_of(x, mx, rate);
    zq += q;
    if (restricted && q != 0) atomicAdd(&hist[bin_of(x, mx, inv_temp)], q);
  });
  zq = wave_sum_u64(zq);
  __syncthreads();
  if (lane == 0) seg_total[wave] = zq;
  __syncthreads();
  zq = 0;
  for (int i = 0; i < SAMPLE_WAVES; ++i) zq += seg_total[i];  // >= 2^40: the maximum itself

  uint32_t threshold = 0;  // tokens with key >= threshold are kept
  u64 kept_mass = zq;
  auto kept_mass_of = [&](float x) -> u64 {
    x = clean(x);
    return float_key(x) >= threshold ? mass_of(x, mx, rate) : 0;
  };
  if (restricted) {
    u64 target = static_cast<u64>(static_cast<double>(p) * static_cast<double>(zq));
    if (target >= zq) target = zq - 1;
    // The boundary bin: mass before it <= target < mass before it + its own mass.  Every
    // thread takes two neighbouring bins; the waves' sums meet in LDS.
    {
      static_assert(BINS == 2 * SAMPLE_THREADS, "two bins a thread");
      const u64 h0 = hist[2 * threadIdx.x], h1 = hist[2 * threadIdx.x + 1];
      u64 scan = h0 + h1;
      for (int off = 1; off < PYLON_WAVE; off <<= 1) {
        const u64 up = __shfl_up(scan, off, PYLON_WAVE);
        if (lane >= off) scan += up;
      }
      if (lane == PYLON_WAVE - 1) sum_scratch[wave] = scan;
      __syncthreads();
      u64 before = scan - (h0 + h1);
      for (int i = 0; i < wave; ++i) before += sum_scratch[i];
      if (before <= target && target < before + h0) {
        shared_bin = 2 * threadIdx.x;
        shared_mass[0] = before;
      } else if (before + h0 <= target && target < before + h0 + h1) {
        shared_bin = 2 * threadIdx.x + 1;
        shared_mass[0] = before + h0;
      }
    }
    __syncthreads();
    const int boundary = shared_bin;
    const u64 before_bin = shared_mass[0];
    __syncthreads();  // the histogram is read; its memory now takes the bin's tokens

    // pass 3: the boundary bin's tokens into LDS; beside them what this wave's stretch holds in
    // the bins before, which is kept whatever the threshold turns out to be
    uint32_t* cand_key = reinterpret_cast<uint32_t*>(pool);
    uint32_t* cand_index = reinterpret_cast<uint32_t*>(pool + CANDIDATES * sizeof(uint32_t));
    u64* cand_mass = reinterpret_cast<u64*>(pool + 2 * CANDIDATES * sizeof(uint32_t));
    // logits this far below the largest lie behind the boundary bin, whatever bin_of rounds to
    const float behind = mx - (static_cast<float>(boundary) + 1.5f) * (BIN_RANGE / BINS) * temp;
    u64 above = 0;
    wave_each<true>(row, w0, w1, aligned, behind, [&](float x, int i) {
      x = clean(x);
      const int bin = bin_of(x, mx, inv_temp);
      if (bin > boundary) return;
      const u64 q = mass_of(x, mx, rate);
      if (bin < boundary) {
        above += q;
        return;
      }
      if (q == 0) return;
      const uint32_t key = float_key(x);
      atomicMin(&key_range[0], key);
      atomicMax(&key_range[1], key);
      const int at = atomicAdd(&cand_count, 1);
      if (at < CANDIDATES) {
        cand_key[at] = key;
        cand_index[at] = static_cast<uint32_t>(i);
        cand_mass[at] = q;
      }
    });
    above = wave_sum_u64(above);
    __syncthreads();
    const int count = cand_count;
    // The smallest key k with (mass of keys > k) <= target lies in [lo, hi]: at hi only the
    // earlier bins are above, at lo - 1 the whole boundary bin would be as well.
    uint32_t lo = key_range[0], hi = key_range[1];
    if (count <= CANDIDATES) {
      // Sixteen probes a round, one per wave, spread evenly over [lo, hi): the mass above a
      // probe falls as the probe rises, so the answer lies between the last probe that has
      // too much above it and the first that has not.
      while (lo < hi) {
        const uint32_t mid =
            lo + static_cast<uint32_t>(static_cast<u64>(hi - lo) * (wave + 1) / (SAMPLE_WAVES + 1));
        u64 over = 0;
        for (int j = lane; j < count; j += PYLON_WAVE)
          if (cand_key[j] > mid) over += cand_mass[j];
        over = before_bin + wave_sum_u64(over);
        __syncthreads();
        if (lane == 0) index_scratch[wave] = over <= target ? 1 : 0;
        __syncthreads();
        int first = 0;
        while (first < SAMPLE_WAVES && index_scratch[first] == 0) ++first;
        const uint32_t span = hi - lo;
        if (first < SAMPLE_WAVES)
          hi = lo + static_cast<uint32_t>(static_cast<u64>(span) * (first + 1) / (SAMPLE_WAVES + 1));
        if (first > 0) lo = lo + static_cast<uint32_t>(static_cast<u64>(span) * first / (SAMPLE_WAVES + 1)) + 1;
      }
      if (wave == 0) {
        u64 kept = 0;
        for (int j = lane; j < count; j += PYLON_WAVE)
          if (cand_key[j] >= lo) kept += cand_mass[j];
        kept = before_bin + wave_sum_u64(kept);
        if (lane == 0) {
          shared_threshold = lo;
          shared_mass[1] = kept;
        }
      }
      __syncthreads();
      threshold = shared_threshold;
      kept_mass = shared_mass[1];
      // this stretch's kept mass: the bins before, and the bin's tokens from the threshold up
      u64 mine = 0;
      for (int j = lane; j < count; j += PYLON_WAVE) {
        const int at = static_cast<int>(cand_index[j]);
        if (cand_key[j] >= threshold && at >= w0 && at < w1) mine += cand_mass[j];
      }
      mine = above + wave_sum_u64(mine);
      if (lane == 0) seg_total[wave] = mine;
    } else {
      // More tokens in one bin than LDS holds (thousands of near-equal logits): bisect
      // with a pass over the row for each probe.
      while (lo < hi) {
        const uint32_t mid = lo + (hi - lo) / 2;
        u64 over = 0;
        wave_each<true>(row, w0, w1, aligned, massless, [&](float x, int) {
          x = clean(x);
          if (float_key(x) > mid) over += mass_of(x, mx, rate);
        });
        over = block_sum_u64(over, sum_scratch);
        if (over <= target)
          hi = mid;
        else
          lo = mid + 1;
      }
      threshold = lo;
      u64 kept = 0;
      wave_each<true>(row, w0, w1, aligned, massless, [&](float x, int) { kept += kept_mass_of(x); });
      kept = wave_sum_u64(kept);
      __syncthreads();
      if (lane == 0) seg_total[wave] = kept;
      __syncthreads();
      kept_mass = 0;
      for (int i = 0; i < SAMPLE_WAVES; ++i) kept_mass += seg_total[i];
    }
    __syncthreads();
  }

  // pass 4: the first index, in index order, at which the cumulative kept mass exceeds
  // u * (kept mass): narrowed to one of sixteen stretches (the first time by the totals the
  // passes above left), then to a sixteenth of that, then scanned.
  float u = uniform[r];
  u = u < 0.f ? 0.f : u;
  u64 target = static_cast<u64>(static_cast<double>(u) * static_cast<double>(kept_mass));
  if (target >= kept_mass) target = kept_mass - 1;
  int begin = 0, end = vocab;
  u64 before = 0;
  bool lost = false, have_totals = true;
  while (end - begin > 4 * PYLON_WAVE * 4) {
    int seg = (end - begin + SAMPLE_WAVES - 1) / SAMPLE_WAVES;
    seg = (seg + 4 * PYLON_WAVE - 1) / (4 * PYLON_WAVE) * (4 * PYLON_WAVE);
    if (!have_totals) {
      const int s0 = begin + wave * seg < end ? begin + wave * seg : end;
      const int s1 = s0 + seg < end ? s0 + seg : end;
      u64 mine = 0;
      wave_each<true>(row, s0, s1, aligned, massless, [&](float x, int) { mine += kept_mass_of(x); });
      mine = wave_sum_u64(mine);
      __syncthreads();
      if (lane == 0) seg_total[wave] = mine;
      __syncthreads();
    }
    have_totals = false;
    int pick = -1;
    for (int w = 0; w < SAMPLE_WAVES; ++w) {
      const u64 t = seg_total[w];
      if (before + t > target) {
        pick = w;
        break;
      }
      before += t;
    }
    if (pick < 0) {
      lost = true;
      break;
    }
    begin += pick * seg;
    end = begin + seg < end ? begin + seg : end;
  }
  if (lost) {  // cannot happen while the masses are summed as integers; never leave out[] unset
    const int index = top_index();
    if (threadIdx.x == 0) emit(out, chosen, place, r, index);
    return;
  }
  if (wave == 0) {
    int found = -1;
    for (int sub = begin; sub < end && found < 0; sub += 4 * PYLON_WAVE) {
      const int i = sub + 4 * lane;
      const float4 v = load_four(row, i, end, aligned);
      const u64 q0 = kept_mass_of(v.x), q1 = kept_mass_of(v.y), q2 = kept_mass_of(v.z), q3 = kept_mass_of(v.w);
      const u64 mine = q0 + q1 + q2 + q3;
      u64 scan = mine;
      for (int off = 1; off < PYLON_WAVE; off <<= 1) {
        const u64 up = __shfl_up(scan, off, PYLON_WAVE);
        if (lane >= off) scan += up;
      }
      const u64 crossing = __ballot(before + scan > target);
      if (crossing != 0) {
        const int first = __ffsll(static_cast<long long>(crossing)) - 1;
        int index = -1;
        if (lane == first) {
          u64 cum = before + scan - mine;
          if (cum + q0 > target) index = i;
          else if (cum + q0 + q1 > target) index = i + 1;
          else if (cum + q0 + q1 + q2 > target) index = i + 2;
          else index = i + 3;
        }
        found = __shfl(index, first, PYLON_WAVE);
      } else {
        before += __shfl(scan, PYLON_WAVE - 1, PYLON_WAVE);
      }
    }
    if (lane == 0) {
      shared_bin = found;
      if (found >= 0) emit(out, chosen, place, r, found);
    }
  }
  __syncthreads();
  if (shared_bin < 0) {  // cannot happen either; never leave out[] unset
    const int index = top_index();
    if (threadIdx.x == 0) emit(out, chosen, place, r, index);
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
