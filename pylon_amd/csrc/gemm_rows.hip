// out[M, N] = x[M, K] * w[N, K]^T in bfloat16 for up to 64 rows of x a workgroup (up to 128 a
// launch, as two halves with workgroups of their own): the matrix products of a decode step,
// bound by reading w once, with x from 17 rows on no longer small beside a workgroup's share
// of w.
//
// A workgroup of four wavefronts owns 64 or 128 columns of the output (each wave one or two
// tiles of 16 rows of w) over a range of K; K is cut over blockIdx.y and every cut writes
// its own float partial result, which the consumer adds (the fused residual norm does), or,
// with one cut, the result itself.  The workgroup walks its range in chunks of 128 elements.
//
// Both operands travel from memory straight into LDS (buffer_load_dwordx4 ... lds: a wave
// fills 1 KB of consecutive LDS from 64 places of its choice) in whole row segments: one
// load takes the 256 contiguous bytes that a chunk is of each of four rows.  (A load that
// takes 64 bytes of each of 16 rows, the shape of a matrix-instruction operand, moves less
// than half as much per compute unit: measured 21 us against 8 us for the rows of x of a
// 19456 x 2560 product.)  The rows of x of a chunk are shared by the four waves; each wave
// brings its own tiles of w.  In LDS a tile is 16 rows of 256 bytes, and the 16-byte piece q
// of row R lies at position q ^ R of that row, so that the operand reads (lane r takes piece
// 4 s + g of row r) of 16 lanes fall into 16 different groups of banks.  Several chunks are in
// flight: while chunk c is multiplied, the next two or three travel.  There is one barrier
// per chunk, preceded by a counted wait for this wave's loads of chunk c only, so the later
// loads stay in flight across it.  No sums cross waves: a wave owns its columns.
//
// A workgroup takes `wg_cols` columns, at most what its waves' tiles hold and not necessarily
// that many: the host gives every workgroup of a launch the same share of the columns, chosen
// so that the workgroups are a whole number of rounds over the compute units.  Its waves take
// full tiles in turn; the rows of a tile beyond the workgroup's columns are out of range and
// fetch nothing, and a wave left without columns only helps to bring the rows of x.  (The
// gate/up product of 2 x 9728 columns: 38 per workgroup, one workgroup per unit, 20.0 us
// against 21.0 for 64 or 48 columns per workgroup where some units stream half as much again
// as others.)
//
// All loads go through buffer descriptors (of the workgroup's rows of w; of x): rows beyond
// N or M and elements beyond K are read as zeros without a memory access and without a
// branch, so every wave issues the same number of loads per chunk and the counted waits
// are exact.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

#define GR_CHUNK 128
#define GR_TILE_BYTES 4096  // 16 rows of one chunk
#define GR_LDS(T) __attribute__((address_space(3))) T
#define GR_OOB 0x80000000u

// A barrier behind a wait for this wave's reads of LDS only.  The invariant it keeps: when a
// wave passes it, every wave's operand reads of the chunk before have returned, so the loads
// issued next may overwrite that chunk's stage.  The loads from memory that must have landed
// are counted by hand below and are not waited for here.  (A release fence on LDS would wait
// for every outstanding load, because the loads that write LDS are among them, and the
// chunks in flight would drain at every barrier.)
__device__ __forceinline__ void gr_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

__device__ __forceinline__ float gr_silu(float z) { return z / (1.0f + expf(-z)); }

// vmcnt <= N (N < 64); the other counters are left alone.
template <int N>
__device__ __forceinline__ void gr_wait_loads() {
  static_assert(N >= 0 && N < 64, "vmcnt has six bits");
  __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}

// Stages of LDS for MT tiles of x and WAVES * CT tiles of w per chunk.
template <int MT, int CT, int WAVES>
struct GrShape {
  static constexpr int TILES = MT + WAVES * CT;
  static constexpr int STAGE_BYTES = TILES * GR_TILE_BYTES;
  // Four stages where they fit and a wave brings one tile of w per chunk; with two tiles a wave
  // (36 KB a stage and more) three do better by 1 to 2 % (gate/up 2 x 9728 x 2560 at 8 rows:
  // 19.6 against 20.0 us; the head 139.1 against 140.2), and with one tile a wave three lose
  // 4 to 7 %; six stages are slower everywhere.
  static constexpr int STAGES = (4 * STAGE_BYTES <= 144 * 1024 && CT == 1) ? 4 : 3;
};

// MT: tiles of 16 rows of x (1..4); CT: tiles of 16 rows of w per wave (1 or 2).
// GLU (CT = 2): w is a fused gate/up matrix of 2 N rows; a wave's first tile is 16 gate rows,
// its second the 16 up rows that lie N rows further down, and it writes silu(gate) * up.
// (The body is a device function: the host pass does not know the descriptor type and would
// drop a kernel that names it, launch stub and all.)
template <int MT, int CT, bool GLU, int WAVES, typename TO>
__device__ __forceinline__ void gemm_rows_body(
    TO* __restrict__ out, const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, int M, int N,
    int K, long long ldx, long long ldw, long long ldo, long long part_stride, int chunks_per_part,
    int wg_cols, int group) {
  typedef GrShape<MT, CT, WAVES> Shape;
  constexpr int QW = 4 / WAVES;  // quarters of every tile of x that a wave fills
  constexpr int STAGES = Shape::STAGES;
  constexpr int LOADS = QW * MT + 4 * CT;  // loads a wave issues per chunk
  __shared__ __attribute__((aligned(1024))) unsigned char lds[STAGES * Shape::STAGE_BYTES];

  const int lane = threadIdx.x & (PYLON_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / PYLON_WAVE);
  const int r = lane & 15, g = lane >> 4;
  constexpr int WAVE_COLS = (GLU ? 1 : CT) * 16;  // columns of the output per wave
  const int wg_row0 = group * wg_cols;  // first row of w the descriptor covers
  const int wg_end = (N - wg_row0 < wg_cols) ? N : wg_row0 + wg_cols;
  const int n0 = wg_row0 + wave * WAVE_COLS;
  const int n_end = (wg_end - n0 < WAVE_COLS) ? wg_end : n0 + WAVE_COLS;  // <= n0: a wave without columns
  const int part = blockIdx.y;
  const int chunks = (K + GR_CHUNK - 1) / GR_CHUNK;
  const int c_begin = part * chunks_per_part;
  const int c_end = (c_begin + chunks_per_part < chunks) ? c_begin + chunks_per_part : chunks;

  // The descriptor of w starts at the workgroup's first row (with GLU it reaches N rows
  // further, to its up rows).
  const int wg_rows = wg_end - wg_row0;
  const __amdgpu_buffer_rsrc_t wres = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(w + static_cast<size_t>(wg_row0) * ldw), 0,
      static_cast<int>((static_cast<long long>((GLU ? N : 0) + wg_rows - 1) * ldw + K) * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(x), 0, static_cast<int>((static_cast<long long>(M - 1) * ldx + K) * 2), 0x00020000);

  // A load fills rows 4 q .. 4 q + 3 of a tile (q: the quarter): lane l brings, for row
  // R = 4 q + l / 16, the piece (l % 16) ^ R.
  // x: this wave fills quarters QW * wave .. of every tile of x.
  const int lrow = lane >> 4, lpos = lane & 15;
  unsigned x_at[QW][MT];  // byte offset of this lane's piece in chunk 0, or out of range
  int x_k[QW];            // its first element within a chunk
#pragma unroll
  for (int u = 0; u < QW; ++u) {
    const int R = 4 * (QW * wave + u) + lrow;
    x_k[u] = (lpos ^ R) * 8;
#pragma unroll
    for (int t = 0; t < MT; ++t)
      x_at[u][t] = (16 * t + R < M)
                       ? static_cast<unsigned>(16 * t + R) * static_cast<unsigned>(ldx) * 2u + 2u * x_k[u]
                       : GR_OOB;
  }
  // w: this wave fills all four quarters of its own CT tiles.
  unsigned w_at[CT][4];
  int w_k[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int R = 4 * q + lrow;
    w_k[q] = (lpos ^ R) * 8;
#pragma unroll
    for (int j = 0; j < CT; ++j) {
      // the row within the workgroup's columns, and where it lies from the descriptor's base
      const int col = n0 - wg_row0 + (GLU ? R : 16 * j + R);
      const unsigned row = static_cast<unsigned>(col) + ((GLU && j == 1) ? static_cast<unsigned>(N) : 0u);
      w_at[j][q] = (wg_row0 + col < n_end) ? row * static_cast<unsigned>(ldw) * 2u + 2u * w_k[q] : GR_OOB;
    }
  }
  // Operand reads: lane (r, g) takes piece 4 s + g of row r of a tile.
  unsigned piece_at[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) piece_at[s] = (r >> 2) * 1024 + (r & 3) * 256 + (((4 * s + g) ^ r) * 16);

  floatx4 acc[CT][MT];
#pragma unroll
  for (int j = 0; j < CT; ++j)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[j][t] = floatx4{0.f, 0.f, 0.f, 0.f};

  // The loads of chunk c into a stage.  A chunk beyond the range issues the same loads with
  // every offset out of range: nothing is fetched, and the count of loads per turn stays fixed.
  auto issue = [&](int c, int stage) {
    const bool live = c < c_end;
    const unsigned k0 = static_cast<unsigned>(c) * GR_CHUNK;
    unsigned char* base = lds + stage * Shape::STAGE_BYTES;
#pragma unroll
    for (int u = 0; u < QW; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const bool ok = live && x_at[u][t] != GR_OOB && static_cast<int>(k0) + x_k[u] < K;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            xres, (GR_LDS(void)*)(base + t * GR_TILE_BYTES + (QW * wave + u) * 1024), 16,
            ok ? x_at[u][t] + 2u * k0 : GR_OOB, 0, 0, 0);
      }
#pragma unroll
    for (int j = 0; j < CT; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const bool ok = live && w_at[j][q] != GR_OOB && static_cast<int>(k0) + w_k[q] < K;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            wres, (GR_LDS(void)*)(base + (MT + wave * CT + j) * GR_TILE_BYTES + q * 1024), 16,
            ok ? w_at[j][q] + 2u * k0 : GR_OOB, 0, 0, 0);
      }
  };
  auto compute = [&](int stage) {
    const GR_LDS(unsigned char)* base = (const GR_LDS(unsigned char)*)(lds + stage * Shape::STAGE_BYTES);
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      bf16x8 xf[MT], wf[CT];
#pragma unroll
      for (int t = 0; t < MT; ++t)
        xf[t] = *reinterpret_cast<const GR_LDS(bf16x8)*>(base + t * GR_TILE_BYTES + piece_at[s]);
#pragma unroll
      for (int j = 0; j < CT; ++j)
        wf[j] = *reinterpret_cast<const GR_LDS(bf16x8)*>(base + (MT + wave * CT + j) * GR_TILE_BYTES + piece_at[s]);
#pragma unroll
      for (int j = 0; j < CT; ++j)
#pragma unroll
        for (int t = 0; t < MT; ++t)
          acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[j], xf[t], acc[j][t], 0, 0, 0);
    }
  };

  // Chunk c lives in stage (c - c_begin) % STAGES.  At the top of turn c the loads of chunks
  // c .. c + STAGES - 2 are outstanding; chunk c has landed once at most those of the later
  // ones are.  After the barrier every wave is past the products of chunk c - 1, whose stage
  // chunk c + STAGES - 1 takes.
#pragma unroll
  for (int i = 0; i < STAGES - 1; ++i) issue(c_begin + i, i);
  int stage = 0;
  for (int c = c_begin; c < c_end; ++c) {
    gr_wait_loads<LOADS*(STAGES - 2)>();
    gr_barrier();
    issue(c + STAGES - 1, stage == 0 ? STAGES - 1 : stage - 1);
    if (n0 < n_end) compute(stage);
    stage = (stage + 1 == STAGES) ? 0 : stage + 1;
  }
  // The loads still outstanding are those past the range: they fetch nothing but do write
  // (zeros) into LDS when they complete, so the wave sees them through before it leaves.
  gr_wait_loads<0>();

  // acc[j][t][i] is out[16 t + r][n0 + 16 j + 4 g + i] (with GLU: gate and up of column
  // n0 + 4 g + i).  Four values of a lane go out as one store where every row of every part
  // is aligned for it.
  TO* dst = out + static_cast<size_t>(part) * part_stride;
  const bool wide = (ldo & 3) == 0 && (part_stride & 3) == 0 &&
                    (reinterpret_cast<uintptr_t>(out) & (4 * sizeof(TO) - 1)) == 0;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = t * 16 + r;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < (GLU ? 1 : CT); ++j) {
      const int n = n0 + 16 * j + 4 * g;
      floatx4 v = acc[j][t];
      if constexpr (GLU) {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = gr_silu(acc[0][t][i]) * acc[1][t][i];
      }
      TO* p = dst + static_cast<size_t>(m) * ldo + n;
      if (wide && n + 3 < n_end && (n & 3) == 0) {
        if constexpr (sizeof(TO) == 4) {
          *reinterpret_cast<floatx4*>(p) = v;
        } else {
          uint2 packed;
          packed.x = float_to_bf16_bits(v[0]) | (static_cast<uint32_t>(float_to_bf16_bits(v[1])) << 16);
          packed.y = float_to_bf16_bits(v[2]) | (static_cast<uint32_t>(float_to_bf16_bits(v[3])) << 16);
          *reinterpret_cast<uint2*>(p) = packed;
        }
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < n_end) p[i] = from_float<TO>(v[i]);
      }
    }
  }
}

template <int MT, int CT, bool GLU, int WAVES, typename TO>
__global__ __launch_bounds__(WAVES* PYLON_WAVE) void gemm_rows_kernel(
    TO* __restrict__ out, const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, int M, int N,
    int K, long long ldx, long long ldw, long long ldo, long long part_stride, int chunks_per_part,
    int wg_cols, int groups, int row_split) {
  // More than 64 rows of x go as two halves of `row_split` rows, each to workgroups of its
  // own that take the same columns: blockIdx.x counts eight groups of columns for the first
  // half, the same eight for the second, then the next eight, so that the two workgroups that
  // stream the same rows of w start together and on the same die (a die takes every eighth
  // workgroup), where the second finds in the cache what the first brought.
  int group = blockIdx.x;
  if (row_split > 0) {
    const int half = (blockIdx.x >> 3) & 1;
    group = ((blockIdx.x >> 4) << 3) | (blockIdx.x & 7);
    if (group >= groups) return;  // the grid is padded to whole sixteens
    x += static_cast<size_t>(half) * row_split * ldx;
    out += static_cast<size_t>(half) * row_split * ldo;
    M = (M - half * row_split < row_split) ? M - half * row_split : row_split;
  }
  gemm_rows_body<MT, CT, GLU, WAVES, TO>(out, x, w, M, N, K, ldx, ldw, ldo, part_stride, chunks_per_part, wg_cols,
                                         group);
}

// How a product is laid over the chip: wavefronts per workgroup, workgroups along the columns,
// and the columns each of them takes.
struct GrLaunch {
  int waves, groups, wg_cols;
};

// units: compute units of the device.  waves: 4, 2, or 0 for two where four would give fewer
// workgroups than half the units.  cols: columns per workgroup, or 0 for the rule: an equal
// share for every workgroup of as many whole rounds over the units as workgroups of full
// width would need (at least 16 columns), unless that makes the workgroups re-read more rows
// of x than they stream rows of w; then, and beyond 16 rows of x in launches of several rounds
// whose last is not mostly empty, the full width.  Measured at 2560 x 9728, K cut in eight, 32 rows: 13.2 us with 80 columns
// (256 workgroups) against 14.9 with 128 (160); 2560 x 4096 cut in four, 48 rows: 9.15 with
// 40 columns against 9.08 with 64; the head of 151936 rows at 8 rows of x: 136.5 with 119
// columns against 141; at 64 rows of x (4.6 rounds): 181 against 170.5; a gate/up matrix of
// 2 x 17408 rows at 17 rows of x (1.06 rounds of 64 columns): 34 columns in 512 workgroups.
static GrLaunch gr_launch_shape(int M, int N, int parts, int col_tiles, int glu, int waves, int units, int cols) {
  const int wave_cols = (glu ? 1 : col_tiles) * 16;
  if (waves == 0)
    waves = (static_cast<long long>((N + 4 * wave_cols - 1) / (4 * wave_cols)) * parts < units / 2) ? 2 : 4;
  const int full = waves * wave_cols;
  if (cols <= 0) {
    const long long least = static_cast<long long>((N + full - 1) / full) * parts;  // workgroups of full width
    const long long rounds = (least + units - 1) / units;
    const long long groups = rounds * units / parts;
    int even = groups > 0 ? static_cast<int>((N + groups - 1) / groups) : full;
    even = even < 16 ? 16 : (even > full ? full : even);
    // several rounds of full width are left alone unless the last is mostly empty
    const bool uneven = rounds == 1 || least * 100 < rounds * units * 85;
    const bool pays = M <= 16 || (uneven && even * (glu ? 2 : 1) >= M);
    cols = pays ? even : full;
  }
  return GrLaunch{waves, (N + cols - 1) / cols, cols};
}

template <int MT, int CT, bool GLU, int WAVES>
static void launch_rows_waves(void* out, int out_dtype, const void* x, const void* w, int M, int N, int K,
                              long long ldx, long long ldw, long long ldo, int parts, long long part_stride,
                              const GrLaunch& shape, int row_split, hipStream_t stream) {
  const int chunks = (K + GR_CHUNK - 1) / GR_CHUNK;
  const int per_part = (chunks + parts - 1) / parts;
  dim3 grid(row_split > 0 ? 2 * ((shape.groups + 7) / 8 * 8) : shape.groups, parts), block(WAVES * PYLON_WAVE);
  if (out_dtype == PYLON_F32)
    hipLaunchKernelGGL((gemm_rows_kernel<MT, CT, GLU, WAVES, float>), grid, block, 0, stream, (float*)out,
                       (const uint16_t*)x, (const uint16_t*)w, M, N, K, ldx, ldw, ldo, part_stride, per_part,
                       shape.wg_cols, shape.groups, row_split);
  else
    hipLaunchKernelGGL((gemm_rows_kernel<MT, CT, GLU, WAVES, bf16_t>), grid, block, 0, stream, (bf16_t*)out,
                       (const uint16_t*)x, (const uint16_t*)w, M, N, K, ldx, ldw, ldo, part_stride, per_part,
                       shape.wg_cols, shape.groups, row_split);
}

// Workgroups of four waves, or of two where four would leave compute units without one.
template <int MT, int CT, bool GLU>
static void launch_rows(void* out, int out_dtype, const void* x, const void* w, int M, int N, int K,
                        long long ldx, long long ldw, long long ldo, int parts, long long part_stride,
                        const GrLaunch& shape, int row_split, hipStream_t stream) {
  if (shape.waves == 2)
    launch_rows_waves<MT, CT, GLU, 2>(out, out_dtype, x, w, M, N, K, ldx, ldw, ldo, parts, part_stride, shape,
                                      row_split, stream);
  else
    launch_rows_waves<MT, CT, GLU, 4>(out, out_dtype, x, w, M, N, K, ldx, ldw, ldo, parts, part_stride, shape,
                                      row_split, stream);
}

// What pylon_gemm_rows would launch for these arguments on a device of `units` compute units
// (0: the current device's): shape[0] wavefronts per workgroup, shape[1] workgroups along
// the columns (times `parts` along K), shape[2] the columns each of them takes.
// Touches no device memory; with units given it runs without a GPU.
extern "C" int pylon_gemm_rows_shape(int M, int N, int parts, int col_tiles, int glu, int waves, int units,
                                     int cols, int* shape) {
  PYLON_REQUIRE(shape != nullptr && M >= 1 && N > 0 && parts >= 1 && cols >= 0, "gemm_rows_shape: bad arguments");
  PYLON_REQUIRE(col_tiles == 1 || col_tiles == 2, "gemm_rows_shape: col_tiles is 1 or 2");
  PYLON_REQUIRE(waves == 0 || waves == 2 || waves == 4, "gemm_rows_shape: waves is 0, 2 or 4");
  if (units <= 0) units = pylon_compute_units();
  PYLON_REQUIRE(units > 0, "gemm_rows_shape: no device to take the number of compute units from");
  // beyond 64 rows each half of the rows has workgroups of its own: shape[1] of them per half
  const GrLaunch l = gr_launch_shape(M > 64 ? (M + 1) / 2 : M, N, parts, col_tiles, glu, waves, units, cols);
  shape[0] = l.waves, shape[1] = l.groups, shape[2] = l.wg_cols;
  return 0;
}

// x: [M, ldx] bf16, 1 <= M <= 128 (beyond 64 rows two halves of (M + 1) / 2 and the rest, each to
// workgroups of its own); w: [N, ldw] bf16 (with glu: [2N, ldw], gate rows first, then
// up rows); out: `parts` results [M, ldo] spaced part_stride elements apart (parts > 1 needs
// float out and no glu).  col_tiles: tiles of 16 columns per wave, 1 or 2; with glu a wave
// takes 16 gate rows and their 16 up rows.  waves: wavefronts per workgroup, 4 or 2 (0: two if
// four would give fewer workgroups than half the device's compute units).  cols: columns per
// workgroup, at most what its waves' tiles hold (0: the rule of gr_launch_shape); the sums do
// not depend on it.
extern "C" int pylon_gemm_rows(void* out, int out_dtype, const void* x, const void* w, int M, int N, int K,
                               long long ldx, long long ldw, long long ldo, int parts, long long part_stride,
                               int col_tiles, int glu, int waves, int cols, hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(out_dtype), "gemm_rows: unknown output dtype");
  PYLON_REQUIRE(M >= 0 && M <= 128, "gemm_rows: takes at most 128 rows, got %d", M);
  PYLON_REQUIRE(N > 0 && K > 0, "gemm_rows: bad sizes N=%d K=%d", N, K);
  PYLON_REQUIRE(K % 8 == 0, "gemm_rows: K=%d must be a multiple of 8", K);
  PYLON_REQUIRE(ldx % 8 == 0 && ldw % 8 == 0, "gemm_rows: row strides must be multiples of 8 elements");
  PYLON_REQUIRE(ldw >= K && ldx >= K && ldo >= N, "gemm_rows: a row stride is too short");
  PYLON_REQUIRE(ldw <= (1ll << 22) && ldx <= (1ll << 22),
                "gemm_rows: row strides beyond 4M elements are not supported");
  PYLON_REQUIRE((reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0,
                "gemm_rows: operands must be 16-byte aligned");
  PYLON_REQUIRE(col_tiles == 1 || col_tiles == 2, "gemm_rows: col_tiles is 1 or 2, got %d", col_tiles);
  PYLON_REQUIRE(parts >= 1 && parts <= 64, "gemm_rows: parts must be 1..64");
  PYLON_REQUIRE(parts == 1 || out_dtype == PYLON_F32, "gemm_rows: partial results must be float");
  PYLON_REQUIRE(parts == 1 || !glu, "gemm_rows: the gated epilogue needs the whole of K");
  PYLON_REQUIRE(parts == 1 || part_stride >= static_cast<long long>(M) * ldo,
                "gemm_rows: partial results overlap");
  PYLON_REQUIRE(!glu || (static_cast<long long>(N) + 64) * ldw * 2 < (1ll << 31),
                "gemm_rows: a fused gate/up matrix of %d rows of %lld elements is beyond the 2 GB a "
                "workgroup's view of it may span", 2 * N, ldw);
  PYLON_REQUIRE(waves == 0 || waves == 2 || waves == 4, "gemm_rows: waves is 0, 2 or 4, got %d", waves);
  if (M == 0) return 0;
  const int units = pylon_compute_units();
  PYLON_REQUIRE(units > 0, "gemm_rows: the device's number of compute units is unknown");
  // beyond 64 rows: two halves, each to workgroups of its own
  const int row_split = M > 64 ? (M + 1) / 2 : 0;
  const int rows_each = row_split > 0 ? row_split : M;
  const GrLaunch shape = gr_launch_shape(rows_each, N, parts, col_tiles, glu, waves, units, cols);
  PYLON_REQUIRE(cols >= 0 && cols <= shape.waves * (glu ? 1 : col_tiles) * 16,
                "gemm_rows: %d columns per workgroup are more than the tiles of its %d waves hold", cols, shape.waves);
#define GO(MT)                                                                                              \
  do {                                                                                                      \
    if (glu) launch_rows<MT, 2, true>(out, out_dtype, x, w, M, N, K, ldx, ldw, ldo, parts, part_stride, shape, row_split, stream); \
    else if (col_tiles == 2) launch_rows<MT, 2, false>(out, out_dtype, x, w, M, N, K, ldx, ldw, ldo, parts, part_stride, shape, row_split, stream); \
    else launch_rows<MT, 1, false>(out, out_dtype, x, w, M, N, K, ldx, ldw, ldo, parts, part_stride, shape, row_split, stream); \
  } while (0)
  switch ((rows_each + 15) / 16) {
    case 1: GO(1); break;
    case 2: GO(2); break;
    case 3: GO(3); break;
    default: GO(4); break;
  }
#undef GO
  PYLON_LAUNCHED("gemm_rows");
}
