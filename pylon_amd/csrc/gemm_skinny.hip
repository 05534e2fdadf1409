// out[M, N] = x[M, K] * w[N, K]^T for a few rows of x (M <= 64) in bfloat16: the matrix
// products of a decode step, which are bound by reading w from memory exactly once.
//
// A workgroup of four wavefronts owns 16 rows of w (16 output columns).  The waves take
// turns along K in steps of 64: in a step a lane reads 32 contiguous bytes of one w row,
// so a wave reads one full 128-byte line of each of its 16 rows.  Products go through
// the 16x16x32 bf16 matrix instruction with w as the row operand and x as the column
// operand (x is padded to tiles of 16 rows by re-reading its last row; those columns are
// never stored).  The four waves' partial sums are added in a fixed order through LDS.
// For matrices with few rows, K can further be cut over blockIdx.y; each cut writes its
// own float partial result, which the consumer adds (the fused residual norm does).
//
// With GATED the x operand is formed on the fly as silu(g) * u from a [M, 2K] input
// (g = columns 0..K-1, u = columns K..2K-1), rounded to bfloat16 as the separate
// activation kernel rounds it.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

#define SK_WAVES 4
#define SK_STEP 64

__device__ __forceinline__ bf16x8 load8(const uint16_t* p) {
  return *reinterpret_cast<const bf16x8*>(p);
}
__device__ __forceinline__ bf16x8 load8_stream(const uint16_t* p) {
  // weights are read once: do not keep them in the caches
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return *reinterpret_cast<bf16x8*>(&v);
}
__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
  return z;
}

__device__ __forceinline__ bf16x8 gated8(const uint16_t* g, const uint16_t* u) {
  const uint4 gr = *reinterpret_cast<const uint4*>(g);
  const uint4 ur = *reinterpret_cast<const uint4*>(u);
  const uint32_t gw[4] = {gr.x, gr.y, gr.z, gr.w};
  const uint32_t uw[4] = {ur.x, ur.y, ur.z, ur.w};
  uint32_t packed[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float g0 = __uint_as_float(gw[i] << 16), g1 = __uint_as_float(gw[i] & 0xffff0000u);
    const float u0 = __uint_as_float(uw[i] << 16), u1 = __uint_as_float(uw[i] & 0xffff0000u);
    const float a0 = (g0 / (1.0f + expf(-g0))) * u0;
    const float a1 = (g1 / (1.0f + expf(-g1))) * u1;
    packed[i] = static_cast<uint32_t>(float_to_bf16_bits(a0)) |
                (static_cast<uint32_t>(float_to_bf16_bits(a1)) << 16);
  }
  uint4 out = {packed[0], packed[1], packed[2], packed[3]};
  return *reinterpret_cast<bf16x8*>(&out);
}

template <int MT, bool GATED, typename TO>
__global__ __launch_bounds__(SK_WAVES* PYLON_WAVE) void gemm_skinny_kernel(
    TO* __restrict__ out, const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, int M, int N,
    int K, long long ldx, long long ldw, long long ldo, long long part_stride) {
  __shared__ floatx4 red[SK_WAVES][MT][PYLON_WAVE];
  const int lane = threadIdx.x & (PYLON_WAVE - 1);
  const int wave = threadIdx.x / PYLON_WAVE;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int parts = gridDim.y, part = blockIdx.y;

  const int steps = (K + SK_STEP - 1) / SK_STEP;
  const int per_part = (steps + parts - 1) / parts;
  const int s_begin = part * per_part;
  const int s_end = (s_begin + per_part < steps) ? s_begin + per_part : steps;

  const int wrow = (n0 + r < N) ? n0 + r : N - 1;
  const uint16_t* wp = w + static_cast<size_t>(wrow) * ldw;
  const uint16_t* xp[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = (t * 16 + r < M) ? t * 16 + r : M - 1;
    xp[t] = x + static_cast<size_t>(m) * ldx;
  }

  floatx4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};

#pragma unroll 2
  for (int s = s_begin + wave; s < s_end; s += SK_WAVES) {
    const int k = s * SK_STEP + g * 16;
    const bool in0 = k < K, in1 = k + 8 < K;
    const bf16x8 a0 = in0 ? load8_stream(wp + k) : zero8();
    const bf16x8 a1 = in1 ? load8_stream(wp + k + 8) : zero8();
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      bf16x8 b0, b1;
      if (GATED) {
        b0 = in0 ? gated8(xp[t] + k, xp[t] + K + k) : zero8();
        b1 = in1 ? gated8(xp[t] + k + 8, xp[t] + K + k + 8) : zero8();
      } else {
        b0 = in0 ? load8(xp[t] + k) : zero8();
        b1 = in1 ? load8(xp[t] + k + 8) : zero8();
      }
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, b0, acc[t], 0, 0, 0);
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, b1, acc[t], 0, 0, 0);
    }
  }
#pragma unroll
  for (int t = 0; t < MT; ++t) red[wave][t][lane] = acc[t];
  __syncthreads();
  for (int t = wave; t < MT; t += SK_WAVES) {
    floatx4 sum = red[0][t][lane];
#pragma unroll
    for (int wv = 1; wv < SK_WAVES; ++wv) {
      const floatx4 other = red[wv][t][lane];
      sum += other;
    }
    const int m = t * 16 + r;
    if (m < M) {
      TO* dst = out + static_cast<size_t>(part) * part_stride + static_cast<size_t>(m) * ldo;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + 4 * g + i;
        if (n < N) dst[n] = from_float<TO>(sum[i]);
      }
    }
  }
}

template <int MT, bool GATED>
static void launch_skinny(void* out, int out_dtype, const void* x, const void* w, int M, int N, int K,
                          long long ldx, long long ldw, long long ldo, int parts, long long part_stride,
                          hipStream_t stream) {
  dim3 grid((N + 15) / 16, parts), block(SK_WAVES * PYLON_WAVE);
  if (out_dtype == PYLON_F32)
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, GATED, float>), grid, block, 0, stream, (float*)out,
                       (const uint16_t*)x, (const uint16_t*)w, M, N, K, ldx, ldw, ldo, part_stride);
  else
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, GATED, bf16_t>), grid, block, 0, stream, (bf16_t*)out,
                       (const uint16_t*)x, (const uint16_t*)w, M, N, K, ldx, ldw, ldo, part_stride);
}

// x: [M, ldx] bf16 (for gated: g in columns 0..K-1, u in K..2K-1); w: [N, ldw] bf16;
// out: `parts` results [M, ldo] spaced part_stride elements apart (parts > 1 needs float out).
extern "C" int pylon_gemm_skinny(void* out, int out_dtype, const void* x, const void* w, int M, int N,
                                 int K, long long ldx, long long ldw, long long ldo, int parts,
                                 long long part_stride, int gated, hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(out_dtype), "gemm_skinny: unknown output dtype");
  PYLON_REQUIRE(M >= 0 && M <= 64, "gemm_skinny: takes at most 64 rows, got %d", M);
  PYLON_REQUIRE(N > 0 && K > 0, "gemm_skinny: bad sizes N=%d K=%d", N, K);
  PYLON_REQUIRE(K % 8 == 0, "gemm_skinny: K=%d must be a multiple of 8", K);
  PYLON_REQUIRE(ldx % 8 == 0 && ldw % 8 == 0, "gemm_skinny: row strides must be multiples of 8 elements");
  PYLON_REQUIRE(ldw >= K && ldx >= (gated ? 2 * K : K) && ldo >= N, "gemm_skinny: a row stride is too short");
  PYLON_REQUIRE((reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0,
                "gemm_skinny: operands must be 16-byte aligned");
  PYLON_REQUIRE(parts >= 1 && parts <= 64, "gemm_skinny: parts must be 1..64");
  PYLON_REQUIRE(parts == 1 || out_dtype == PYLON_F32, "gemm_skinny: partial results must be float");
  PYLON_REQUIRE(parts == 1 || part_stride >= static_cast<long long>(M) * ldo,
                "gemm_skinny: partial results overlap");
  if (M == 0) return 0;
  const int mt = (M + 15) / 16;
#define GO(MT)                                                                                          \
  if (gated)                                                                                            \
    launch_skinny<MT, true>(out, out_dtype, x, w, M, N, K, ldx, ldw, ldo, parts, part_stride, stream);  \
  else                                                                                                  \
    launch_skinny<MT, false>(out, out_dtype, x, w, M, N, K, ldx, ldw, ldo, parts, part_stride, stream)
  switch (mt) {
    case 1: GO(1); break;
    case 2: GO(2); break;
    case 3: GO(3); break;
    default: GO(4); break;
  }
#undef GO
  PYLON_LAUNCHED("gemm_skinny");
}
