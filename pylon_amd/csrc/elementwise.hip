// Row-wise kernels of the decoder: embedding gather, RMSNorm (alone, or fused with the
// residual sum that precedes it), and the gated activation of the feed-forward.
// All reductions and all arithmetic are in float; only loads and stores see bf16.
#include "common.h"

// ---- embedding ------------------------------------------------------------------
// out[t, :] = table[ids[t], :] * scale, written as float (the residual stream).
// A negative id -(1 + s) stands for "the token that the sampler left in chosen[s]": a
// request's last sampled token can be fed back without a trip through the host.
template <typename T>
__global__ void embed_kernel(float* __restrict__ out, const T* __restrict__ table,
                             const int* __restrict__ ids, const int* __restrict__ chosen, int hidden,
                             int vocab, float scale) {
  const int t = blockIdx.x;
  int id = ids[t];
  if (id < 0 && chosen != nullptr) id = chosen[-1 - id];
  // The host checks ids; the clamp only keeps a bad id from reading outside the table.
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* row = table + static_cast<size_t>(id) * hidden;
  float* dst = out + static_cast<size_t>(t) * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_float(row[i]) * scale;
}

// chosen may be null; then every id must be a table row.  The host guarantees that a
// negative id -(1 + s) names an entry s inside chosen.
extern "C" int pylon_embed(float* out, const void* table, int table_dtype, const int* ids,
                           const int* chosen, int tokens, int hidden, int vocab, float scale,
                           hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(table_dtype), "embed: unknown table dtype %d", table_dtype);
  PYLON_REQUIRE(tokens >= 0 && hidden > 0 && vocab > 0, "embed: bad sizes tokens=%d hidden=%d vocab=%d",
                tokens, hidden, vocab);
  if (tokens == 0) return 0;
  dim3 grid(tokens), block(256);
  if (table_dtype == PYLON_F32)
    hipLaunchKernelGGL(embed_kernel<float>, grid, block, 0, stream, out, (const float*)table, ids,
                       chosen, hidden, vocab, scale);
  else
    hipLaunchKernelGGL(embed_kernel<bf16_t>, grid, block, 0, stream, out, (const bf16_t*)table, ids,
                       chosen, hidden, vocab, scale);
  PYLON_LAUNCHED("embed");
}

// Four consecutive elements number 4c .. 4c+3 of a row, as floats.
__device__ __forceinline__ float4 load4(const float* p, long long c) {
  return reinterpret_cast<const float4*>(p)[c];
}
__device__ __forceinline__ float4 load4(const bf16_t* p, long long c) {
  const uint2 raw = reinterpret_cast<const uint2*>(p)[c];
  return float4{__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u),
                __uint_as_float(raw.y << 16), __uint_as_float(raw.y & 0xffff0000u)};
}
__device__ __forceinline__ void store4(float* p, long long c, float a, float b, float d, float e) {
  reinterpret_cast<float4*>(p)[c] = float4{a, b, d, e};
}
__device__ __forceinline__ void store4(bf16_t* p, long long c, float a, float b, float d, float e) {
  uint2 raw;
  raw.x = static_cast<uint32_t>(float_to_bf16_bits(a)) | (static_cast<uint32_t>(float_to_bf16_bits(b)) << 16);
  raw.y = static_cast<uint32_t>(float_to_bf16_bits(d)) | (static_cast<uint32_t>(float_to_bf16_bits(e)) << 16);
  reinterpret_cast<uint2*>(p)[c] = raw;
}

// ---- RMSNorm ----------------------------------------------------------------------
// y = (x * 1/sqrt(mean(x^2) + eps)) * w, in float, rounded once on the store.
// One workgroup per output row. `row_idx` (optional) picks the input row of each
// output row. With `delta`, the input is resid + delta (float sum); `write_resid`
// stores that sum back into resid (only meaningful without row_idx).
// At most 512 threads per workgroup, so that a thread may hold the eight partial sums of its
// sixteen elements in registers (a kernel that may be launched with 1,024 threads gets 128).
template <typename TX, typename TD, typename TO>
__global__ __launch_bounds__(512) void rmsnorm_kernel(TO* __restrict__ out, TX* x, const TD* __restrict__ delta,
                               int n_delta, long long delta_stride,
                               const float* __restrict__ w, const int* __restrict__ row_idx,
                               int dim, float eps, int write_resid) {
  __shared__ float scratch[16];
  const int r_out = blockIdx.x;
  const int r_in = row_idx ? row_idx[r_out] : r_out;
  TX* xr = x + static_cast<size_t>(r_in) * dim;
  const TD* dr = delta ? delta + static_cast<size_t>(r_in) * dim : nullptr;
  TO* yr = out + static_cast<size_t>(r_out) * dim;

  // Fast path (float rows whose length is a multiple of 4 and fits the registers): every
  // load of the row is a 16-byte load issued before anything is stored, so the row costs
  // one trip to memory.
  constexpr int VEC = 4;  // float4 chunks per thread
  if (sizeof(TX) == 4 && (dim & 3) == 0 && dim <= 4 * VEC * static_cast<int>(blockDim.x) &&
      (delta_stride & 3) == 0) {
    const int chunks = dim >> 2;
    const float4* x4 = reinterpret_cast<const float4*>(xr);
    const float4* w4 = reinterpret_cast<const float4*>(w);
    float4 held[VEC], wt[VEC];
#pragma unroll
    for (int n = 0; n < VEC; ++n) {
      const int c = threadIdx.x + n * blockDim.x;
      held[n] = (c < chunks) ? x4[c] : float4{0.f, 0.f, 0.f, 0.f};
      wt[n] = (c < chunks) ? w4[c] : float4{0.f, 0.f, 0.f, 0.f};
    }
    if (dr) {
      // Partial sums of the previous matrix product are added in a fixed order.  For the
      // usual counts every load is issued before the first addition: a loop over a count
      // only known at run time would wait for memory once per partial sum.
      const long long stride4 = delta_stride >> 2;
      float4 d[VEC];
#define PYLON_SUM_PARTS(ND)                                                                   \
  do {                                                                                        \
    float4 e[ND][VEC];                                                                        \
    _Pragma("unroll") for (int p = 0; p < ND; ++p) _Pragma("unroll") for (int n = 0; n < VEC; ++n) { \
      const int c = threadIdx.x + n * blockDim.x;                                             \
      e[p][n] = (c < chunks) ? load4(dr, c + p * stride4) : float4{0.f, 0.f, 0.f, 0.f};       \
    }                                                                                         \
    _Pragma("unroll") for (int n = 0; n < VEC; ++n) {                                         \
      d[n] = e[0][n];                                                                         \
      _Pragma("unroll") for (int p = 1; p < ND; ++p) {                                        \
        d[n].x += e[p][n].x; d[n].y += e[p][n].y; d[n].z += e[p][n].z; d[n].w += e[p][n].w;   \
      }                                                                                       \
    }                                                                                         \
  } while (0)
      if (n_delta == 1) {
        PYLON_SUM_PARTS(1);
      } else if (n_delta == 2) {
        PYLON_SUM_PARTS(2);
      } else if (n_delta == 4) {
        PYLON_SUM_PARTS(4);
      } else if (n_delta == 8) {
        PYLON_SUM_PARTS(8);
      } else {
        PYLON_SUM_PARTS(1);
        for (int p = 1; p < n_delta; ++p) {
#pragma unroll
          for (int n = 0; n < VEC; ++n) {
            const int c = threadIdx.x + n * blockDim.x;
            if (c < chunks) {
              const float4 e = load4(dr, c + p * stride4);
              d[n].x += e.x; d[n].y += e.y; d[n].z += e.z; d[n].w += e.w;
            }
          }
        }
      }
#undef PYLON_SUM_PARTS
#pragma unroll
      for (int n = 0; n < VEC; ++n) {
        held[n].x += d[n].x; held[n].y += d[n].y; held[n].z += d[n].z; held[n].w += d[n].w;
      }
    }
    float ss = 0.f;
#pragma unroll
    for (int n = 0; n < VEC; ++n)
      ss += held[n].x * held[n].x + held[n].y * held[n].y + held[n].z * held[n].z + held[n].w * held[n].w;
    const float total = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(total / static_cast<float>(dim) + eps);
#pragma unroll
    for (int n = 0; n < VEC; ++n) {
      const int c = threadIdx.x + n * blockDim.x;
      if (c < chunks) {
        if (dr && write_resid) reinterpret_cast<float4*>(xr)[c] = held[n];
        const float y0 = (held[n].x * inv) * wt[n].x, y1 = (held[n].y * inv) * wt[n].y;
        const float y2 = (held[n].z * inv) * wt[n].z, y3 = (held[n].w * inv) * wt[n].w;
        store4(yr, c, y0, y1, y2, y3);
      }
    }
    return;
  }

  float ss = 0.f;
  for (int i = threadIdx.x; i < dim; i += blockDim.x) {
    float v = to_float(xr[i]);
    if (dr) {
      float d = to_float(dr[i]);
      for (int p = 1; p < n_delta; ++p) d += to_float(dr[i + p * delta_stride]);
      v += d;
      if (write_resid) xr[i] = from_float<TX>(v);
    }
    ss += v * v;
  }
  const float total = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(total / static_cast<float>(dim) + eps);
  for (int i = threadIdx.x; i < dim; i += blockDim.x) {
    float v = to_float(xr[i]);
    if (dr && !write_resid) {
      float d = to_float(dr[i]);
      for (int p = 1; p < n_delta; ++p) d += to_float(dr[i + p * delta_stride]);
      v += d;
    }
    yr[i] = from_float<TO>((v * inv) * w[i]);
  }
}

// The same arithmetic, in the same order, for steps of many rows (prompt portions): a
// workgroup takes R rows and issues the loads of all of them before the first sum, so that one
// row's stores travel beside the next row's loads instead of every workgroup of the launch
// reading at one time and writing at another (2,048 rows of 2,560: 19.5 -> 15.8 us on data
// that no cache holds; four rows per workgroup lose again, 19.2 us).  Float residual, one
// delta, rows of a multiple of 4 elements that fit 16 per thread; as many threads as the
// kernel for few rows has at this width, so that a row's sum is formed in the same order.
template <typename TD, typename TO, int R, int THREADS>
__global__ __launch_bounds__(THREADS) void add_rmsnorm_many_kernel(TO* __restrict__ out, float* resid,
                                                               const TD* __restrict__ delta,
                                                               const float* __restrict__ w, int rows, int dim,
                                                               float eps) {
  __shared__ float scratch[16];
  constexpr int VEC = 4;
  const int chunks = dim >> 2;
  const float4* w4 = reinterpret_cast<const float4*>(w);
  float4 held[R][VEC], wt[VEC];
  const int r0 = blockIdx.x * R;
#pragma unroll
  for (int n = 0; n < VEC; ++n) {
    const int c = threadIdx.x + n * THREADS;
    wt[n] = (c < chunks) ? w4[c] : float4{0.f, 0.f, 0.f, 0.f};
  }
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const bool live = r0 + i < rows;
    const float* xr = resid + static_cast<size_t>(live ? r0 + i : r0) * dim;
    const TD* dr = delta + static_cast<size_t>(live ? r0 + i : r0) * dim;
#pragma unroll
    for (int n = 0; n < VEC; ++n) {
      const int c = threadIdx.x + n * THREADS;
      if (c < chunks) {
        const float4 x = reinterpret_cast<const float4*>(xr)[c];
        const float4 d = load4(dr, c);
        held[i][n] = float4{x.x + d.x, x.y + d.y, x.z + d.z, x.w + d.w};
      } else {
        held[i][n] = float4{0.f, 0.f, 0.f, 0.f};
      }
    }
  }
#pragma unroll
  for (int i = 0; i < R; ++i) {
    if (r0 + i >= rows) break;  // the same for the whole workgroup
    float ss = 0.f;
#pragma unroll
    for (int n = 0; n < VEC; ++n)
      ss += held[i][n].x * held[i][n].x + held[i][n].y * held[i][n].y + held[i][n].z * held[i][n].z +
            held[i][n].w * held[i][n].w;
    const float total = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(total / static_cast<float>(dim) + eps);
    float* xr = resid + static_cast<size_t>(r0 + i) * dim;
    TO* yr = out + static_cast<size_t>(r0 + i) * dim;
#pragma unroll
    for (int n = 0; n < VEC; ++n) {
      const int c = threadIdx.x + n * THREADS;
      if (c < chunks) {
        reinterpret_cast<float4*>(xr)[c] = held[i][n];
        store4(yr, c, (held[i][n].x * inv) * wt[n].x, (held[i][n].y * inv) * wt[n].y,
               (held[i][n].z * inv) * wt[n].z, (held[i][n].w * inv) * wt[n].w);
      }
    }
  }
}

#define PYLON_NORM_MANY_ROWS 512  // from this many rows on, a workgroup takes two

template <typename TX, typename TD>
static void launch_rmsnorm_out(void* out, int out_dtype, TX* x, const TD* delta, int n_delta,
                               long long delta_stride, const float* w, const int* row_idx, int rows,
                               int dim, float eps, int write_resid, hipStream_t stream) {
  if constexpr (sizeof(TX) == 4) {
    if (rows >= PYLON_NORM_MANY_ROWS && delta != nullptr && n_delta == 1 && row_idx == nullptr && write_resid &&
        (dim & 3) == 0 && dim <= 8192) {
      constexpr int R = 2;
      dim3 grid((rows + R - 1) / R);
#define GO(TO, THREADS)                                                                                    \
  hipLaunchKernelGGL((add_rmsnorm_many_kernel<TD, TO, R, THREADS>), grid, dim3(THREADS), 0, stream, (TO*)out, x, \
                     delta, w, rows, dim, eps)
      if (dim > 4096) {
        if (out_dtype == PYLON_F32) GO(float, 512); else GO(bf16_t, 512);
      } else {
        if (out_dtype == PYLON_F32) GO(float, 256); else GO(bf16_t, 256);
      }
#undef GO
      return;
    }
  }
  dim3 grid(rows), block(dim > 4096 ? 512 : 256);
  if (out_dtype == PYLON_F32)
    hipLaunchKernelGGL((rmsnorm_kernel<TX, TD, float>), grid, block, 0, stream, (float*)out, x, delta,
                       n_delta, delta_stride, w, row_idx, dim, eps, write_resid);
  else
    hipLaunchKernelGGL((rmsnorm_kernel<TX, TD, bf16_t>), grid, block, 0, stream, (bf16_t*)out, x,
                       delta, n_delta, delta_stride, w, row_idx, dim, eps, write_resid);
}

// out[r] = rmsnorm(x[idx(r)]) for any input dtype.
extern "C" int pylon_rmsnorm(void* out, int out_dtype, const void* x, int x_dtype, const float* w,
                             const int* row_idx, int rows, int dim, float eps, hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(out_dtype) && pylon_valid_dtype(x_dtype), "rmsnorm: unknown dtype");
  PYLON_REQUIRE(rows >= 0 && dim > 0, "rmsnorm: bad sizes rows=%d dim=%d", rows, dim);
  PYLON_REQUIRE(eps >= 0.f, "rmsnorm: eps must not be negative");
  if (rows == 0) return 0;
  if (x_dtype == PYLON_F32)
    launch_rmsnorm_out<float, float>(out, out_dtype, (float*)x, nullptr, 0, 0, w, row_idx, rows, dim,
                                     eps, 0, stream);
  else
    launch_rmsnorm_out<bf16_t, bf16_t>(out, out_dtype, (bf16_t*)x, nullptr, 0, 0, w, row_idx, rows, dim,
                                       eps, 0, stream);
  PYLON_LAUNCHED("rmsnorm");
}

// resid (float) += delta, then out = rmsnorm(resid). With row_idx the sum is formed only
// for the picked rows and resid is left untouched. delta may come as n_delta partial sums,
// delta_stride elements apart, which are added up first.
extern "C" int pylon_add_rmsnorm(void* out, int out_dtype, float* resid, const void* delta,
                                 int delta_dtype, int n_delta, long long delta_stride, const float* w,
                                 const int* row_idx, int rows, int dim, float eps, hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(out_dtype), "add_rmsnorm: unknown out dtype");
  PYLON_REQUIRE(delta == nullptr || pylon_valid_dtype(delta_dtype), "add_rmsnorm: unknown delta dtype");
  PYLON_REQUIRE(rows >= 0 && dim > 0, "add_rmsnorm: bad sizes rows=%d dim=%d", rows, dim);
  PYLON_REQUIRE(delta == nullptr || (n_delta >= 1 && n_delta <= 64), "add_rmsnorm: 1..64 partial sums");
  if (rows == 0) return 0;
  const int write_resid = (delta != nullptr && row_idx == nullptr) ? 1 : 0;
  if (delta == nullptr || delta_dtype == PYLON_F32)
    launch_rmsnorm_out<float, float>(out, out_dtype, resid, (const float*)delta, n_delta, delta_stride,
                                     w, row_idx, rows, dim, eps, write_resid, stream);
  else
    launch_rmsnorm_out<float, bf16_t>(out, out_dtype, resid, (const bf16_t*)delta, n_delta,
                                      delta_stride, w, row_idx, rows, dim, eps, write_resid, stream);
  PYLON_LAUNCHED("add_rmsnorm");
}

// resid (float) += delta, nothing else (the last residual sum when no norm follows).
template <typename TD>
__global__ void add_kernel(float* __restrict__ resid, const TD* __restrict__ delta, size_t n) {
  size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (; i < n; i += step) resid[i] += to_float(delta[i]);
}

extern "C" int pylon_residual_add(float* resid, const void* delta, int delta_dtype, long long count,
                                  hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(delta_dtype), "residual_add: unknown dtype");
  PYLON_REQUIRE(count >= 0, "residual_add: negative count");
  if (count == 0) return 0;
  long long blocks = (count + 255) / 256;
  if (blocks > 65535 * 16) blocks = 65535 * 16;
  dim3 grid((unsigned)blocks), block(256);
  if (delta_dtype == PYLON_F32)
    hipLaunchKernelGGL(add_kernel<float>, grid, block, 0, stream, resid, (const float*)delta, (size_t)count);
  else
    hipLaunchKernelGGL(add_kernel<bf16_t>, grid, block, 0, stream, resid, (const bf16_t*)delta,
                       (size_t)count);
  PYLON_LAUNCHED("residual_add");
}

// ---- gated activation -----------------------------------------------------------------
// out[t, i] = silu(gu[t, i]) * gu[t, inter + i]; silu(z) = z / (1 + exp(-z)).
template <typename TI, typename TO>
__global__ void silu_gate_kernel(TO* __restrict__ out, const TI* __restrict__ gu, int inter, size_t total) {
  size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (; i < total; i += step) {
    const size_t t = i / inter;
    const size_t c = i - t * inter;
    const float g = to_float(gu[t * 2 * inter + c]);
    const float u = to_float(gu[t * 2 * inter + inter + c]);
    const float s = g / (1.0f + expf(-g));
    out[i] = from_float<TO>(s * u);
  }
}

// bfloat16 rows whose length is a multiple of 8: eight elements (16 bytes) per thread.
__global__ void silu_gate_bf16x8_kernel(uint4* __restrict__ out, const uint4* __restrict__ gu, int chunks,
                                        size_t total) {
  size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (; i < total; i += step) {
    const size_t t = i / chunks;
    const size_t c = i - t * chunks;
    const uint4 g = gu[t * 2 * chunks + c];
    const uint4 u = gu[t * 2 * chunks + chunks + c];
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
    uint32_t r[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float g0 = __uint_as_float(gw[j] << 16), g1 = __uint_as_float(gw[j] & 0xffff0000u);
      const float u0 = __uint_as_float(uw[j] << 16), u1 = __uint_as_float(uw[j] & 0xffff0000u);
      const float a0 = (g0 / (1.0f + expf(-g0))) * u0;
      const float a1 = (g1 / (1.0f + expf(-g1))) * u1;
      r[j] = static_cast<uint32_t>(float_to_bf16_bits(a0)) | (static_cast<uint32_t>(float_to_bf16_bits(a1)) << 16);
    }
    out[i] = uint4{r[0], r[1], r[2], r[3]};
  }
}

// gate_up: [tokens, 2 * inter] of in_dtype; out: [tokens, inter] of out_dtype (float sums of a
// product may come in as float and leave as bfloat16: one rounding, after the activation).
extern "C" int pylon_silu_gate(void* out, int out_dtype, const void* gate_up, int in_dtype, int tokens, int inter,
                               hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(in_dtype) && pylon_valid_dtype(out_dtype), "silu_gate: unknown dtype");
  PYLON_REQUIRE(tokens >= 0 && inter > 0, "silu_gate: bad sizes tokens=%d inter=%d", tokens, inter);
  const size_t total = static_cast<size_t>(tokens) * inter;
  if (total == 0) return 0;
  if (in_dtype == PYLON_BF16 && out_dtype == PYLON_BF16 && inter % 8 == 0 &&
      (reinterpret_cast<uintptr_t>(out) & 15) == 0 && (reinterpret_cast<uintptr_t>(gate_up) & 15) == 0) {
    const size_t chunks_total = total / 8;
    size_t nblocks = (chunks_total + 255) / 256;
    if (nblocks > 65535u * 16u) nblocks = 65535u * 16u;
    hipLaunchKernelGGL(silu_gate_bf16x8_kernel, dim3((unsigned)nblocks), dim3(256), 0, stream, (uint4*)out,
                       (const uint4*)gate_up, inter / 8, chunks_total);
    PYLON_LAUNCHED("silu_gate");
  }
  size_t blocks = (total + 255) / 256;
  if (blocks > 65535u * 16u) blocks = 65535u * 16u;
  dim3 grid((unsigned)blocks), block(256);
#define GO(TI, TO) \
  hipLaunchKernelGGL((silu_gate_kernel<TI, TO>), grid, block, 0, stream, (TO*)out, (const TI*)gate_up, inter, total)
  if (in_dtype == PYLON_F32 && out_dtype == PYLON_F32) GO(float, float);
  else if (in_dtype == PYLON_F32) GO(float, bf16_t);
  else if (out_dtype == PYLON_F32) GO(bf16_t, float);
  else GO(bf16_t, bf16_t);
#undef GO
  PYLON_LAUNCHED("silu_gate");
}
