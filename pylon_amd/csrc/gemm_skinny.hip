// out[M, N] = x[M, K] * w[N, K]^T for a few rows of x (M <= 64) in bfloat16: the matrix
// products of a decode step, which are bound by reading w from memory exactly once.
//
// A workgroup of 4 or 8 wavefronts owns 16 rows of w (16 output columns), or 32 rows as two
// tiles for matrices with many rows (the rows of x it loads then serve both; measured
// 151 us against 165 us for a 151936 x 2560 matrix).  The waves take
// turns along K in steps of 64: in a step a wave reads one full 128-byte line of each of
// its 16 rows, as two loads that each cover a contiguous 64-byte half of every line.
// All loads of a batch of steps are issued before the first product, so a wave with few
// steps pays the memory latency once.  Products go through the 16x16x32 bf16 matrix
// instruction with w as the row operand and x as the column operand (x is padded to tiles
// of 16 rows by re-reading its last row; those columns are never stored).  The waves'
// partial sums are added in a fixed order through LDS.  For matrices with few rows, K can
// further be cut over blockIdx.y; each cut writes its own float partial result, which the
// consumer adds (the fused residual norm does).
//
// With GLU the workgroup also owns the 16 rows of w that lie N rows further down (the "up"
// half of a fused gate/up matrix) and writes silu(gate) * up, rounded once.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

#define SK_WAVES 4
#define SK_STEP 64

__device__ __forceinline__ bf16x8 load8(const uint16_t* p) {
  return *reinterpret_cast<const bf16x8*>(p);
}
__device__ __forceinline__ bf16x8 load8_stream(const uint16_t* p) {
  // Plain loads: non-temporal loads measured about 20 % slower for this access pattern.
  return *reinterpret_cast<const bf16x8*>(p);
}
__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
  return z;
}

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }

// RT: 16-row tiles of w per workgroup (with GLU: RT tiles of gate rows and RT of up rows).
// A wave multiplies every tile of w with every tile of x, so RT tiles of w pay for the rows of
// x once: with many rows of x, x (read from the cache) would else be most of the traffic.
template <int MT, int WAVES, bool GLU, int RT, typename TO>
__global__ __launch_bounds__(WAVES* PYLON_WAVE) void gemm_skinny_kernel(
    TO* __restrict__ out, const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, int M, int N,
    int K, long long ldx, long long ldw, long long ldo, long long part_stride) {
  constexpr int TILES = GLU ? 2 * RT : RT;  // row tiles of w per workgroup
  __shared__ floatx4 red[WAVES][TILES][MT][PYLON_WAVE];
  const int lane = threadIdx.x & (PYLON_WAVE - 1);
  const int wave = threadIdx.x / PYLON_WAVE;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 16 * RT;
  const int parts = gridDim.y, part = blockIdx.y;

  const int steps = (K + SK_STEP - 1) / SK_STEP;
  const int per_part = (steps + parts - 1) / parts;
  const int s_begin = part * per_part;
  const int s_end = (s_begin + per_part < steps) ? s_begin + per_part : steps;

  const uint16_t* wp[TILES];
#pragma unroll
  for (int j = 0; j < TILES; ++j) {
    const int row = n0 + 16 * (j % RT) + r;
    const int wrow = (row < N) ? row : N - 1;
    wp[j] = w + static_cast<size_t>((GLU && j >= RT) ? N + wrow : wrow) * ldw;
  }
  const uint16_t* xp[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = (t * 16 + r < M) ? t * 16 + r : M - 1;
    xp[t] = x + static_cast<size_t>(m) * ldx;
  }

  floatx4 acc[TILES][MT];
#pragma unroll
  for (int j = 0; j < TILES; ++j)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[j][t] = floatx4{0.f, 0.f, 0.f, 0.f};

  // steps whose loads are issued together: about 16 loads of 16 bytes per lane and half step
  constexpr int BATCH = (MT == 1) ? (TILES == 2 ? 5 : 10) : (16 / (TILES + MT) > 0 ? 16 / (TILES + MT) : 1);
  for (int s0 = s_begin + wave; s0 < s_end; s0 += WAVES * BATCH) {
    bf16x8 a[BATCH][TILES][2], b[BATCH][MT][2];
#pragma unroll
    for (int u = 0; u < BATCH; ++u) {
      const int s = s0 + u * WAVES;
      const int k = s * SK_STEP + g * 8;
      const bool in0 = s < s_end && k < K, in1 = s < s_end && k + 32 < K;
#pragma unroll
      for (int j = 0; j < TILES; ++j) {
        a[u][j][0] = in0 ? load8(wp[j] + k) : zero8();
        a[u][j][1] = in1 ? load8(wp[j] + k + 32) : zero8();
      }
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        b[u][t][0] = in0 ? load8(xp[t] + k) : zero8();
        b[u][t][1] = in1 ? load8(xp[t] + k + 32) : zero8();
      }
    }
#pragma unroll
    for (int u = 0; u < BATCH; ++u)
#pragma unroll
      for (int j = 0; j < TILES; ++j)
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][j][0], b[u][t][0], acc[j][t], 0, 0, 0);
          acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][j][1], b[u][t][1], acc[j][t], 0, 0, 0);
        }
  }
#pragma unroll
  for (int j = 0; j < TILES; ++j)
#pragma unroll
    for (int t = 0; t < MT; ++t) red[wave][j][t][lane] = acc[j][t];
  __syncthreads();
  for (int t = wave; t < MT; t += WAVES) {
    floatx4 sum[TILES];
#pragma unroll
    for (int j = 0; j < TILES; ++j) {
      sum[j] = red[0][j][t][lane];
#pragma unroll
      for (int wv = 1; wv < WAVES; ++wv) {
        const floatx4 other = red[wv][j][t][lane];
        sum[j] += other;
      }
    }
    const int m = t * 16 + r;
    if (m < M) {
      TO* dst = out + static_cast<size_t>(part) * part_stride + static_cast<size_t>(m) * ldo;
      if (GLU) {
#pragma unroll
        for (int j = 0; j < RT; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int n = n0 + 16 * j + 4 * g + i;
            if (n < N) dst[n] = from_float<TO>(silu_f(sum[j][i]) * sum[RT + j][i]);
          }
      } else {
#pragma unroll
        for (int j = 0; j < TILES; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int n = n0 + 16 * j + 4 * g + i;
            if (n < N) dst[n] = from_float<TO>(sum[j][i]);
          }
      }
    }
  }
}

template <int MT, int WAVES, bool GLU, int RT>
static void launch_skinny(void* out, int out_dtype, const void* x, const void* w, int M, int N, int K,
                          long long ldx, long long ldw, long long ldo, int parts, long long part_stride,
                          hipStream_t stream) {
  constexpr int ROWS = 16 * RT;
  dim3 grid((N + ROWS - 1) / ROWS, parts), block(WAVES * PYLON_WAVE);
  if (out_dtype == PYLON_F32)
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, WAVES, GLU, RT, float>), grid, block, 0, stream, (float*)out,
                       (const uint16_t*)x, (const uint16_t*)w, M, N, K, ldx, ldw, ldo, part_stride);
  else
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, WAVES, GLU, RT, bf16_t>), grid, block, 0, stream, (bf16_t*)out,
                       (const uint16_t*)x, (const uint16_t*)w, M, N, K, ldx, ldw, ldo, part_stride);
}

template <int MT>
static void launch_skinny_mt(void* out, int out_dtype, const void* x, const void* w, int M, int N, int K,
                             long long ldx, long long ldw, long long ldo, int parts,
                             long long part_stride, int glu, hipStream_t stream) {
  // Four waves measured faster than eight at every shape of a 4B-class decoder; the
  // eight-wave form is kept for very long K only.
  const int steps = (K + SK_STEP - 1) / SK_STEP / parts;
  const bool wide = steps >= 512;
#define GO(W, G, R) launch_skinny<MT, W, G, R>(out, out_dtype, x, w, M, N, K, ldx, ldw, ldo, parts, part_stride, stream)
  if (glu) {
    if (wide) GO(8, true, 1); else GO(4, true, 1);
  } else if (MT == 1 && parts == 1 && N >= 4096) {
    // Two tiles of w per workgroup pay for one tile of x rows.  Matrices with few rows
    // (which also cut K) keep one tile: they need the workgroups more than the saving.
    if (wide) GO(8, false, 2); else GO(4, false, 2);
  } else {
    if (wide) GO(8, false, 1); else GO(4, false, 1);
  }
#undef GO
}

// x: [M, ldx] bf16; w: [N, ldw] bf16 (with glu: [2N, ldw], gate rows first, then up rows);
// out: `parts` results [M, ldo] spaced part_stride elements apart (parts > 1 needs float out
// and no glu).
extern "C" int pylon_gemm_skinny(void* out, int out_dtype, const void* x, const void* w, int M, int N,
                                 int K, long long ldx, long long ldw, long long ldo, int parts,
                                 long long part_stride, int glu, hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(out_dtype), "gemm_skinny: unknown output dtype");
  PYLON_REQUIRE(M >= 0 && M <= 64, "gemm_skinny: takes at most 64 rows, got %d", M);
  PYLON_REQUIRE(N > 0 && K > 0, "gemm_skinny: bad sizes N=%d K=%d", N, K);
  PYLON_REQUIRE(K % 8 == 0, "gemm_skinny: K=%d must be a multiple of 8", K);
  PYLON_REQUIRE(ldx % 8 == 0 && ldw % 8 == 0, "gemm_skinny: row strides must be multiples of 8 elements");
  PYLON_REQUIRE(ldw >= K && ldx >= K && ldo >= N, "gemm_skinny: a row stride is too short");
  PYLON_REQUIRE((reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0,
                "gemm_skinny: operands must be 16-byte aligned");
  PYLON_REQUIRE(parts >= 1 && parts <= 64, "gemm_skinny: parts must be 1..64");
  PYLON_REQUIRE(parts == 1 || out_dtype == PYLON_F32, "gemm_skinny: partial results must be float");
  PYLON_REQUIRE(parts == 1 || !glu, "gemm_skinny: the gated epilogue needs the whole of K");
  PYLON_REQUIRE(parts == 1 || part_stride >= static_cast<long long>(M) * ldo,
                "gemm_skinny: partial results overlap");
  if (M == 0) return 0;
  switch ((M + 15) / 16) {
    case 1: launch_skinny_mt<1>(out, out_dtype, x, w, M, N, K, ldx, ldw, ldo, parts, part_stride, glu, stream); break;
    case 2: launch_skinny_mt<2>(out, out_dtype, x, w, M, N, K, ldx, ldw, ldo, parts, part_stride, glu, stream); break;
    case 3: launch_skinny_mt<3>(out, out_dtype, x, w, M, N, K, ldx, ldw, ldo, parts, part_stride, glu, stream); break;
    default: launch_skinny_mt<4>(out, out_dtype, x, w, M, N, K, ldx, ldw, ldo, parts, part_stride, glu, stream); break;
  }
  PYLON_LAUNCHED("gemm_skinny");
}
