// out[M, N] = x[M, K] * w[N, K]^T in bfloat16 for 17 to 64 rows of x: the matrix products of
// a decode step with many requests, still bound by reading w once, but with x no longer
// small beside a workgroup's share of w.
//
// A workgroup of four wavefronts owns 64 or 128 columns of the output (each wave one or two
// tiles of 16 rows of w) over a range of K; K is cut over blockIdx.y and every cut writes
// its own float partial result, which the consumer adds (the fused residual norm does), or,
// with one cut, the result itself.  The workgroup walks its range in chunks of 128 elements.
// The rows of x of a chunk go from memory straight into LDS (buffer_load_dwordx4 ... lds: a wave
// fills 1 KB of consecutive LDS from 64 places of its choice, here the 16 rows x 4 pieces of
// 16 bytes that are one column operand of the 16x16x32 matrix instruction, in lane order, so
// that reading an operand back is one conflict-free 16-byte read per lane) and are shared by
// the four waves; each wave loads its own tiles of w into registers in the layout of the
// row operand.  Three chunks are in flight: while chunk c is multiplied, c + 1 and c + 2
// travel.  There is one barrier per chunk, preceded by a counted wait for this wave's loads of
// chunk c only, so the later loads stay in flight across it.  No sums cross waves: a wave owns its columns.
//
// All loads go through buffer descriptors (of the workgroup's rows of w; of x): rows beyond N
// and elements beyond K are read as zeros without a memory access and without a branch, so
// every wave issues the same number of loads per chunk and the counted waits below are exact.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef int intx4 __attribute__((ext_vector_type(4)));

#define GR_CHUNK 128
#define GR_STAGES 3
#define GR_WAVES 4
#define GR_GLOBAL(T) __attribute__((address_space(1))) T
#define GR_LDS(T) __attribute__((address_space(3))) T
#define GR_OOB 0x80000000u


// A bare barrier: the waits that must precede it are counted by hand below.  (A release
// fence on LDS would wait for every outstanding load, because the loads that write LDS are
// among them, and the chunks in flight would drain at every barrier.)
__device__ __forceinline__ void gr_barrier() { asm volatile("s_barrier" ::: "memory"); }

// vmcnt <= N (N < 16); the other counters are left alone.
template <int N>
__device__ __forceinline__ void gr_wait_loads() {
  static_assert(N >= 0 && N < 16, "vmcnt beyond the low field");
  __builtin_amdgcn_s_waitcnt(0x0f70 | N);
}

// MT: tiles of 16 rows of x (2..4); CT: tiles of 16 rows of w per wave (1 or 2).
// (The body is a device function: the host pass does not know the descriptor type and would
// drop a kernel that names it, launch stub and all.)
template <int MT, int CT, typename TO>
__device__ __forceinline__ void gemm_rows_body(
    TO* __restrict__ out, const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, int M, int N,
    int K, long long ldx, long long ldw, long long ldo, long long part_stride, int chunks_per_part) {
  constexpr int FRAGS = MT * 4;             // operands of x per chunk: tile t, step s -> 4 t + s
  constexpr int XL = FRAGS / GR_WAVES;      // of which a wave fetches this many
  constexpr int LOADS = XL + 4 * CT;        // loads a wave issues per chunk
  static_assert(FRAGS % GR_WAVES == 0, "the waves share the operands of x evenly");
  __shared__ __attribute__((aligned(1024))) unsigned char xs[GR_STAGES][FRAGS][1024];

  const int lane = threadIdx.x & (PYLON_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / PYLON_WAVE);
  const int r = lane & 15, g = lane >> 4;
  const int wg_row0 = blockIdx.x * (GR_WAVES * CT * 16);  // first row of w of this workgroup
  const int n0 = wg_row0 + wave * CT * 16;                // and of this wave
  const int part = blockIdx.y;
  const int chunks = (K + GR_CHUNK - 1) / GR_CHUNK;
  const int c_begin = part * chunks_per_part;
  const int c_end = (c_begin + chunks_per_part < chunks) ? c_begin + chunks_per_part : chunks;

  // w: a descriptor over this workgroup's rows, so that offsets fit 31 bits whatever N is.
  const int wg_rows = (N - wg_row0 < GR_WAVES * CT * 16) ? N - wg_row0 : GR_WAVES * CT * 16;
  const __amdgpu_buffer_rsrc_t wres = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(w + static_cast<size_t>(wg_row0) * ldw), 0,
      static_cast<int>((static_cast<long long>(wg_rows - 1) * ldw + K) * 2), 0x00020000);
  unsigned w_row[CT];  // byte offset of this lane's row in each tile, or out of range
#pragma unroll
  for (int j = 0; j < CT; ++j) {
    const int row = wave * CT * 16 + 16 * j + r;
    w_row[j] = (wg_row0 + row < N) ? static_cast<unsigned>(row) * static_cast<unsigned>(ldw) * 2u : GR_OOB;
  }
  // x: operand f = wave + 4 i of a chunk is fetched by this wave; its row and step.  Rows
  // beyond M repeat the last one (their columns of the result are never stored).
  const __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(x), 0, static_cast<int>((static_cast<long long>(M - 1) * ldx + K) * 2), 0x00020000);
  unsigned x_row[XL];
  int x_step[XL];
#pragma unroll
  for (int i = 0; i < XL; ++i) {
    const int f = wave + GR_WAVES * i, t = f >> 2;
    const int m = (t * 16 + r < M) ? t * 16 + r : M - 1;
    x_row[i] = static_cast<unsigned>(m) * static_cast<unsigned>(ldx) * 2u;
    x_step[i] = (f & 3) * 32 + g * 8;
  }

  intx4 wreg[GR_STAGES][CT][4];
  floatx4 acc[CT][MT];
#pragma unroll
  for (int j = 0; j < CT; ++j)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[j][t] = floatx4{0.f, 0.f, 0.f, 0.f};

  // The loads of chunk C into stage S.  A chunk beyond the range issues the same loads with
  // every offset out of range: nothing is fetched, and the count of loads per turn stays fixed.
#define GR_ISSUE(C, S)                                                                               \
  do {                                                                                               \
    const int k0 = (C) * GR_CHUNK;                                                                   \
    const bool live = (C) < c_end;                                                                   \
    _Pragma("unroll") for (int i = 0; i < XL; ++i) {                                                 \
      const int k = k0 + x_step[i];                                                                  \
      __builtin_amdgcn_raw_ptr_buffer_load_lds(xres, (GR_LDS(void)*)(&xs[S][wave + GR_WAVES * i][0]),    \
                                           16, (live && k < K) ? x_row[i] + 2u * k : GR_OOB, 0, 0, 0); \
    }                                                                                                \
    _Pragma("unroll") for (int j = 0; j < CT; ++j) _Pragma("unroll") for (int s = 0; s < 4; ++s) {   \
      const int k = k0 + s * 32 + g * 8;                                                             \
      const unsigned at = (live && k < K && w_row[j] != GR_OOB) ? w_row[j] + 2u * k : GR_OOB;        \
      wreg[S][j][s] = __builtin_amdgcn_raw_buffer_load_b128(wres, at, 0, 0);                                \
    }                                                                                                \
  } while (0)

#define GR_COMPUTE(S)                                                                                \
  do {                                                                                               \
    _Pragma("unroll") for (int s = 0; s < 4; ++s) {                                                  \
      bf16x8 xf[MT];                                                                                 \
      _Pragma("unroll") for (int t = 0; t < MT; ++t)                                                 \
        xf[t] = *reinterpret_cast<const GR_LDS(bf16x8)*>(                                            \
            (const GR_LDS(unsigned char)*)(&xs[S][4 * t + s][0]) + lane * 16);                       \
      _Pragma("unroll") for (int j = 0; j < CT; ++j) _Pragma("unroll") for (int t = 0; t < MT; ++t)  \
        acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(                                         \
            __builtin_bit_cast(bf16x8, wreg[S][j][s]), xf[t], acc[j][t], 0, 0, 0);                   \
    }                                                                                                \
  } while (0)

  // Chunk c lives in stage c % 3.  On entry the loads of chunks c and c + 1 are outstanding;
  // chunk c has landed once at most those of c + 1 are.  After the barrier every wave is past
  // the products of chunk c - 1, whose stage chunk c + 2 takes.
#define GR_TURN(S)                                                                                   \
  do {                                                                                               \
    __builtin_amdgcn_sched_barrier(0); /* the counted wait relies on the order of issue */          \
    gr_wait_loads<LOADS>();                                                                          \
    gr_barrier();                                                                                    \
    __builtin_amdgcn_sched_barrier(0);                                                               \
    GR_ISSUE(c + 2, ((S) + 2) % GR_STAGES);                                                          \
    __builtin_amdgcn_sched_barrier(0);                                                               \
    GR_COMPUTE(S);                                                                                   \
    ++c;                                                                                             \
  } while (0)

  // Turns come in threes without a way out in between: a branch after a turn would let the
  // compiler sink that turn's loads of w behind it, next to their first use.  Up to two turns
  // past the range multiply zeros.
  int c = c_begin;
  GR_ISSUE(c, 0);
  __builtin_amdgcn_sched_barrier(0);
  GR_ISSUE(c + 1, 1);
  for (int rounds = (c_end - c_begin + GR_STAGES - 1) / GR_STAGES; rounds > 0; --rounds) {
    GR_TURN(0);
    GR_TURN(1);
    GR_TURN(2);
  }
#undef GR_TURN
#undef GR_COMPUTE
#undef GR_ISSUE

  // acc[j][t][i] is out[16 t + r][n0 + 16 j + 4 g + i]
  TO* dst = out + static_cast<size_t>(part) * part_stride;
  // four sums of a lane go out as one 16-byte store where every row of every part is aligned
  const bool wide = sizeof(TO) == 4 && (ldo & 3) == 0 && (part_stride & 3) == 0 &&
                    (reinterpret_cast<uintptr_t>(out) & 15) == 0;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = t * 16 + r;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < CT; ++j) {
      const int n = n0 + 16 * j + 4 * g;
      TO* p = dst + static_cast<size_t>(m) * ldo + n;
      if constexpr (sizeof(TO) == 4) {
        if (wide && n + 3 < N) {
          *reinterpret_cast<floatx4*>(p) = acc[j][t];
          continue;
        }
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n + i < N) p[i] = from_float<TO>(acc[j][t][i]);
    }
  }
}

template <int MT, int CT, typename TO>
__global__ __launch_bounds__(GR_WAVES* PYLON_WAVE) void gemm_rows_kernel(
    TO* __restrict__ out, const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, int M, int N,
    int K, long long ldx, long long ldw, long long ldo, long long part_stride, int chunks_per_part) {
  gemm_rows_body<MT, CT, TO>(out, x, w, M, N, K, ldx, ldw, ldo, part_stride, chunks_per_part);
}

template <int MT, int CT>
static void launch_rows(void* out, int out_dtype, const void* x, const void* w, int M, int N, int K,
                        long long ldx, long long ldw, long long ldo, int parts, long long part_stride,
                        hipStream_t stream) {
  const int chunks = (K + GR_CHUNK - 1) / GR_CHUNK;
  const int per_part = (chunks + parts - 1) / parts;
  dim3 grid((N + GR_WAVES * CT * 16 - 1) / (GR_WAVES * CT * 16), parts), block(GR_WAVES * PYLON_WAVE);
  if (out_dtype == PYLON_F32)
    hipLaunchKernelGGL((gemm_rows_kernel<MT, CT, float>), grid, block, 0, stream, (float*)out,
                       (const uint16_t*)x, (const uint16_t*)w, M, N, K, ldx, ldw, ldo, part_stride, per_part);
  else
    hipLaunchKernelGGL((gemm_rows_kernel<MT, CT, bf16_t>), grid, block, 0, stream, (bf16_t*)out,
                       (const uint16_t*)x, (const uint16_t*)w, M, N, K, ldx, ldw, ldo, part_stride, per_part);
}

// x: [M, ldx] bf16, 1 <= M <= 64; w: [N, ldw] bf16; out: `parts` results [M, ldo] spaced
// part_stride elements apart (parts > 1 needs float out).  col_tiles: tiles of 16 columns per
// wave, 1 or 2 (a workgroup then covers 64 or 128 columns).
extern "C" int pylon_gemm_rows(void* out, int out_dtype, const void* x, const void* w, int M, int N, int K,
                               long long ldx, long long ldw, long long ldo, int parts, long long part_stride,
                               int col_tiles, hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(out_dtype), "gemm_rows: unknown output dtype");
  PYLON_REQUIRE(M >= 0 && M <= 64, "gemm_rows: takes at most 64 rows, got %d", M);
  PYLON_REQUIRE(N > 0 && K > 0, "gemm_rows: bad sizes N=%d K=%d", N, K);
  PYLON_REQUIRE(K % 8 == 0, "gemm_rows: K=%d must be a multiple of 8", K);
  PYLON_REQUIRE(ldx % 8 == 0 && ldw % 8 == 0, "gemm_rows: row strides must be multiples of 8 elements");
  PYLON_REQUIRE(ldw >= K && ldx >= K && ldo >= N, "gemm_rows: a row stride is too short");
  PYLON_REQUIRE(ldw <= (1ll << 22), "gemm_rows: rows of w longer than 4M elements are not supported");
  PYLON_REQUIRE((reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0,
                "gemm_rows: operands must be 16-byte aligned");
  PYLON_REQUIRE(col_tiles == 1 || col_tiles == 2, "gemm_rows: col_tiles is 1 or 2, got %d", col_tiles);
  PYLON_REQUIRE(parts >= 1 && parts <= 64, "gemm_rows: parts must be 1..64");
  PYLON_REQUIRE(parts == 1 || out_dtype == PYLON_F32, "gemm_rows: partial results must be float");
  PYLON_REQUIRE(parts == 1 || part_stride >= static_cast<long long>(M) * ldo,
                "gemm_rows: partial results overlap");
  if (M == 0) return 0;
#define GO(MT)                                                                                              \
  do {                                                                                                      \
    if (col_tiles == 2) launch_rows<MT, 2>(out, out_dtype, x, w, M, N, K, ldx, ldw, ldo, parts, part_stride, stream); \
    else launch_rows<MT, 1>(out, out_dtype, x, w, M, N, K, ldx, ldw, ldo, parts, part_stride, stream);      \
  } while (0)
  switch ((M + 15) / 16) {
    case 1: GO(1); break;
    case 2: GO(2); break;
    case 3: GO(3); break;
    default: GO(4); break;
  }
#undef GO
  PYLON_LAUNCHED("gemm_rows");
}
