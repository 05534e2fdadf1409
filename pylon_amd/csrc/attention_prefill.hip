// Paged causal attention for prompt portions: bfloat16, head sizes 64, 128 and 256, any
// grouping of query heads.  Flash-attention on the 16x16x32 bf16 matrix instruction.
//
// A workgroup of four wavefronts takes one tile of consecutive tokens of one request and
// one key/value head, together with all query heads of that head's group: a (token, head)
// pair is one of up to 64 or 128 query rows, 16 or 32 per wave.  Keys and values are walked
// 64 at a time.  Scores are computed transposed (keys as rows, queries as columns): the
// result registers of a score tile then already have the layout the row operand of the
// value product needs, and the running maximum of a query lives in the lanes of its
// column.  Scores, softmax and the output accumulators are float; exponentials are exp2
// with scale*log2(e) folded into one multiply-add; the sums of the probabilities come out
// of the matrix cores (a product with a tile of ones).
//
// Two kernels share this arithmetic and differ in how a block of keys and values reaches
// the matrix cores.  The general one (attention_prefill_kernel) fetches the next block into
// registers while the current one is used and writes it to LDS at the top of an iteration:
// the 64 keys row-major, the 64 values transposed (a thread holds eight elements of four
// consecutive keys and writes, per element, the four keys as one 8-byte word), so that a
// lane reads the column operand of the value product as two 8-byte words.  The one for head
// size 128 and block-aligned pages (attention_prefill_direct_kernel, further down) lets the
// memory system write LDS itself and transposes on the way out of LDS.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

#define AP_BK 64       // keys per iteration
#define AP_VSTRIDE 68  // keys per row of the transposed value tile (136 bytes: 8-byte aligned rows)
#define AP_SLACK 8.0f  // how far (as a power of two) a score may exceed the maximum in use
#define AP_TABLE 4096  // most pages a request may hold: its block-table row is kept in LDS

// Two floats to two bfloat16 (round to nearest even) in one word: the hardware conversion.
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{lo, hi}, bf16x2));
}

// The queries of a wave: column `col` of query tile qt is (token, head) pair
// wave*16*QT + qt*16 + col of the workgroup's tile; its position (or -1 if the tile has no
// such pair) and its elements as column operands of the score product.
template <int HD, int QT>
__device__ __forceinline__ void load_queries(int (&qpos)[QT], bf16x8 (&qf)[QT][HD / 32], const uint16_t* __restrict__ q,
                                             int wave, int col, int grp, int group, int tok0, int ntok, int pos0,
                                             int n_heads, int head0) {
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int rr = wave * (16 * QT) + qt * 16 + col;
    const int ti = rr / group, hh = rr - ti * group;
    const bool valid = ti < ntok;
    qpos[qt] = valid ? pos0 + ti : -1;
    const uint16_t* qrow = q + (static_cast<size_t>(tok0 + (valid ? ti : 0)) * n_heads + head0 + hh) * HD;
#pragma unroll
    for (int ks = 0; ks < HD / 32; ++ks) {
      if (valid) {
        qf[qt][ks] = *reinterpret_cast<const bf16x8*>(qrow + ks * 32 + grp * 8);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) qf[qt][ks][i] = (__bf16)0.0f;
      }
    }
  }
}

// One block of 64 keys for one query tile of a wave, first half: s holds the transposed
// scores (lane (col, grp) has keys kb + 16*kt + 4*grp + r of query column col).  Masks,
// keeps the running maximum and rescales the NT accumulator tiles when the maximum moves.
// Returns what to add to scale_log2 * score before the exponential.
template <int NT>
__device__ __forceinline__ float softmax_prepare(floatx4 (&s)[AP_BK / 16], float& m_run, floatx4 (&o)[NT], int qp,
                                                 int kb, bool masked, int window, int grp, float scale_log2,
                                                 float slack) {
  if (masked) {
    // key kb + 16*kt + 4*grp + r is seen if it is at most qp and inside the window: compared
    // as 16*kt + r (a constant) against two numbers of this lane
    const int last_seen = qp - kb - 4 * grp;
    const int first_seen = (window > 0) ? last_seen - window + 1 : -(1 << 30);
#pragma unroll
    for (int kt = 0; kt < AP_BK / 16; ++kt)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (!(kt * 16 + r <= last_seen && kt * 16 + r >= first_seen)) s[kt][r] = -INFINITY;
  } else if (qp < 0) {  // a column that holds no query
#pragma unroll
    for (int kt = 0; kt < AP_BK / 16; ++kt) s[kt] = floatx4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
  }
  // The maximum that the exponentials are taken against is raised only when a score
  // exceeds it by more than AP_SLACK (in units of exp2's argument): until then
  // probabilities may reach 2^AP_SLACK instead of 1, which float sums and bfloat16
  // operands hold just as well, and neither the cross-lane maximum nor the rescaling
  // of the accumulators is needed.  The result is the same up to rounding.
  float tile_max = -INFINITY;
#pragma unroll
  for (int kt = 0; kt < AP_BK / 16; ++kt)
#pragma unroll
    for (int r = 0; r < 4; ++r) tile_max = fmaxf(tile_max, s[kt][r]);
  if (__ballot(tile_max > m_run + slack) != 0) {  // the same for the whole wave
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, PYLON_WAVE));
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, PYLON_WAVE));
    const float m_new = fmaxf(m_run, tile_max);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;  // a row that has seen no key yet
    const float corr = __builtin_amdgcn_exp2f((m_run - m_use) * scale_log2);
    m_run = m_new;
    // the accumulators of this lane belong to query rows 4*grp + r: fetch their factors
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float c = __shfl(corr, 4 * grp + r, PYLON_WAVE);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) o[nt][r] *= c;
    }
  }
  return (m_run == -INFINITY) ? 0.f : -m_run * scale_log2;
}

// Second half: the probabilities of keys 32*kg .. 32*kg + 31 as a row operand of the value
// product.  Operand slot j of a lane is key 32*kg + 4*grp + j (j < 4) or
// 32*kg + 16 + 4*grp + (j - 4).  The row sums are not kept here: the caller multiplies the
// probabilities by a tile of ones as well, so that the last accumulator tile holds, in
// every column, the sum of exactly the rounded probabilities that weigh the values.
__device__ __forceinline__ bf16x8 probabilities(const floatx4 (&s)[AP_BK / 16], int kg, float scale_log2,
                                                float shift) {
  float p[2][4];
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int r = 0; r < 4; ++r) p[h][r] = __builtin_amdgcn_exp2f(fmaf(s[2 * kg + h][r], scale_log2, shift));
  const u32x4 packed = {pack_bf16(p[0][0], p[0][1]), pack_bf16(p[0][2], p[0][3]), pack_bf16(p[1][0], p[1][1]),
                        pack_bf16(p[1][2], p[1][3])};
  return __builtin_bit_cast(bf16x8, packed);
}

// out = acc / sum for a wave's query tiles; a lane holds rows 4*grp + r, element dt*16 + col,
// and the rows' sums in the tile after the last.
template <int HD, int QT>
__device__ __forceinline__ void store_tile(uint16_t* __restrict__ out, const floatx4 (&o)[QT][HD / 16 + 1], int wave,
                                           int col, int grp, int group, int tok0, int ntok, int n_heads,
                                           int head0) {
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float l = o[qt][HD / 16][r];
      const int rr = wave * (16 * QT) + qt * 16 + 4 * grp + r;
      const int ti = rr / group, hh = rr - ti * group;
      if (ti < ntok) {
        const float inv = 1.0f / l;
        uint16_t* orow = out + (static_cast<size_t>(tok0 + ti) * n_heads + head0 + hh) * HD;
#pragma unroll
        for (int dt = 0; dt < HD / 16; ++dt) orow[dt * 16 + col] = float_to_bf16_bits(o[qt][dt][r] * inv);
      }
    }
  }
}

// QT: 16-row query tiles per wave (1: 64 rows per workgroup, 2: 128).  PAGING says how a
// key's place in the cache is found: 0 by a division by the page size (some twenty
// instructions, eight times per thread and block), 1 by a shift and a mask (the page size is
// a power of two), 2 once per block of 64 keys, which then lies inside one page (a power of
// two of at least 64).
template <int HD, int QT, int PAGING>
__global__ __launch_bounds__(256, 2) void attention_prefill_kernel(
    uint16_t* __restrict__ out, const uint16_t* __restrict__ q, const uint16_t* __restrict__ k_cache,
    const uint16_t* __restrict__ v_cache, const int* __restrict__ block_table, int table_width,
    const int* __restrict__ tiles, int n_heads, int n_kv_heads, int group,
    int page_size, int window, float scale) {
  constexpr int KS = HD / 32;        // 32-wide steps along the head for a score tile
  constexpr int DT = HD / 16;        // 16-wide output tiles along the head
  constexpr int KSTR = HD + 8;       // row stride of the key tile (elements)
  constexpr int CHUNKS = HD / 8;     // 16-byte chunks per key or value row
  constexpr int KP = AP_BK * CHUNKS / 256;          // 16-byte pieces of keys per thread and block
  constexpr int VC = (CHUNKS * 16 + 255) / 256;     // (chunk, four keys) items of values per thread
  __shared__ __attribute__((aligned(16))) uint16_t k_lds[AP_BK * KSTR];
  __shared__ __attribute__((aligned(16))) uint16_t v_lds[HD * AP_VSTRIDE];
  __shared__ int table_lds[AP_TABLE];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, grp = lane >> 4;
  // Workgroups start in the order of blockIdx.x and go round the chip's eight dies, each with
  // a cache of its own: neighbours take the same tile for different key/value heads, so the
  // heaviest tiles of all heads start first and a die meets few heads.
  const int kvh = blockIdx.x % n_kv_heads, tile = blockIdx.x / n_kv_heads;
  const int* td = tiles + tile * 4;
  const int tok0 = td[0], ntok = td[1], trow = td[2], pos0 = td[3];
  const int* table = block_table + static_cast<size_t>(trow) * table_width;
  const int kv_last = pos0 + ntok - 1;
  const int k_lo = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
  const int kb_first = (k_lo / AP_BK) * AP_BK;
  // The request's page ids go to LDS once, so that finding a key's page costs no trip to
  // memory inside the loop (the host refuses requests with more pages than fit).
  const int pages_used = kv_last / page_size + 1;
  for (int i = tid; i < pages_used; i += 256) table_lds[i] = table[i];
  __syncthreads();

  // The block of keys and values on its way from the cache.  Keys: piece i of a thread is
  // 8 elements of key (i*256 + tid) / CHUNKS.  Values: item i is chunk (i*256 + tid) / 16
  // of keys 4*((i*256 + tid) % 16) .. +3.  Keys past the end repeat the last key.
  u32x4 kreg[KP], vreg[VC][4];
  const int page_shift = __ffs(page_size) - 1, page_mask = page_size - 1;
  const size_t row_elems = static_cast<size_t>(n_kv_heads) * HD;
  const unsigned row_elems32 = n_kv_heads * HD;  // a block of 64 rows spans far less than 4 GiB
  const uint16_t* k_head = k_cache + static_cast<size_t>(kvh) * HD;
  const uint16_t* v_head = v_cache + static_cast<size_t>(kvh) * HD;
#define AP_SLOT(J, PHYS)                                                                               \
  do {                                                                                                 \
    const int pg = PAGING ? (J) >> page_shift : (J) / page_size;                                       \
    const int off = PAGING ? (J) & page_mask : (J) - pg * page_size;                                   \
    PHYS = table_lds[pg] * page_size + off;                                                            \
  } while (0)
#define AP_FETCH(KB)                                                                                   \
  do {                                                                                                 \
    if constexpr (PAGING == 2) {                                                                       \
      const int page_row = table_lds[(KB) >> page_shift] * page_size + ((KB) & page_mask);             \
      const uint16_t* k_block = k_head + static_cast<size_t>(page_row) * row_elems;                    \
      const uint16_t* v_block = v_head + static_cast<size_t>(page_row) * row_elems;                    \
      const unsigned last = kv_last - (KB);                                                            \
      _Pragma("unroll") for (int i = 0; i < KP; ++i) {                                                 \
        const unsigned idx = i * 256 + tid;                                                            \
        const unsigned key = idx / CHUNKS, chunk = idx - key * CHUNKS;                                 \
        const unsigned j = key < last ? key : last;                                                    \
        kreg[i] = *reinterpret_cast<const u32x4*>(k_block + (j * row_elems32 + chunk * 8));            \
      }                                                                                                \
      _Pragma("unroll") for (int i = 0; i < VC; ++i) {                                                 \
        const unsigned idx = i * 256 + tid;                                                            \
        const unsigned chunk = idx >> 4, quad = idx & 15;                                              \
        if (chunk < CHUNKS) {                                                                          \
          _Pragma("unroll") for (int p = 0; p < 4; ++p) {                                              \
            const unsigned j = 4 * quad + p < last ? 4 * quad + p : last;                              \
            vreg[i][p] = *reinterpret_cast<const u32x4*>(v_block + (j * row_elems32 + chunk * 8));     \
          }                                                                                            \
        }                                                                                              \
      }                                                                                                \
    } else {                                                                                           \
      _Pragma("unroll") for (int i = 0; i < KP; ++i) {                                                 \
        const int idx = i * 256 + tid;                                                                 \
        const int key = idx / CHUNKS, chunk = idx - key * CHUNKS;                                      \
        const int j = ((KB) + key < kv_last) ? (KB) + key : kv_last;                                   \
        int phys;                                                                                      \
        AP_SLOT(j, phys);                                                                              \
        kreg[i] = *reinterpret_cast<const u32x4*>(k_head + static_cast<size_t>(phys) * row_elems + chunk * 8); \
      }                                                                                                \
      _Pragma("unroll") for (int i = 0; i < VC; ++i) {                                                 \
        const int idx = i * 256 + tid;                                                                 \
        const int chunk = idx >> 4, quad = idx & 15;                                                   \
        if (chunk < CHUNKS) {                                                                          \
          _Pragma("unroll") for (int p = 0; p < 4; ++p) {                                              \
            const int j = ((KB) + 4 * quad + p < kv_last) ? (KB) + 4 * quad + p : kv_last;             \
            int phys;                                                                                  \
            AP_SLOT(j, phys);                                                                          \
            vreg[i][p] = *reinterpret_cast<const u32x4*>(v_head + static_cast<size_t>(phys) * row_elems + chunk * 8); \
          }                                                                                            \
        }                                                                                              \
      }                                                                                                \
    }                                                                                                  \
  } while (0)

  AP_FETCH(kb_first);

  int qpos[QT];
  bf16x8 qf[QT][KS];
  load_queries<HD, QT>(qpos, qf, q, wave, col, grp, group, tok0, ntok, pos0, n_heads, kvh * group);

  float m_run[QT];          // the running maximum, in units of raw scores
  floatx4 o[QT][DT + 1];    // the output tiles and, last, the rows' sums
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    m_run[qt] = -INFINITY;
#pragma unroll
    for (int dt = 0; dt <= DT; ++dt) o[qt][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  }
  const bf16x8 ones = __builtin_bit_cast(bf16x8, u32x4{0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u});

  const float scale_log2 = scale * 1.44269504088896340736f;
  const float slack = AP_SLACK / scale_log2;  // in units of raw scores
  for (int kb = kb_first; kb <= kv_last; kb += AP_BK) {
    __syncthreads();  // the last block's readers are done
    // registers -> LDS: keys row-major, values transposed
#pragma unroll
    for (int i = 0; i < KP; ++i) {
      const int idx = i * 256 + tid;
      const int key = idx / CHUNKS, chunk = idx - key * CHUNKS;
      *reinterpret_cast<u32x4*>(&k_lds[key * KSTR + chunk * 8]) = kreg[i];
    }
#pragma unroll
    for (int i = 0; i < VC; ++i) {
      const int idx = i * 256 + tid;
      const int chunk = idx >> 4, quad = idx & 15;
      if (chunk < CHUNKS) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {  // elements chunk*8 + 2e and + 2e + 1 of the four keys
          const uint32_t w0 = vreg[i][0][e], w1 = vreg[i][1][e], w2 = vreg[i][2][e], w3 = vreg[i][3][e];
          // byte selects: the low halves of two words side by side, and the high halves
          const u32x2 even = {__builtin_amdgcn_perm(w1, w0, 0x05040100u), __builtin_amdgcn_perm(w3, w2, 0x05040100u)};
          const u32x2 odd = {__builtin_amdgcn_perm(w1, w0, 0x07060302u), __builtin_amdgcn_perm(w3, w2, 0x07060302u)};
          *reinterpret_cast<u32x2*>(&v_lds[(chunk * 8 + 2 * e) * AP_VSTRIDE + 4 * quad]) = even;
          *reinterpret_cast<u32x2*>(&v_lds[(chunk * 8 + 2 * e + 1) * AP_VSTRIDE + 4 * quad]) = odd;
        }
      }
    }
    if (kb + AP_BK <= kv_last) AP_FETCH(kb + AP_BK);  // the next block travels during this one's math
    __syncthreads();

    // transposed scores: rows = keys of a 16-key tile, columns = the query tile's rows
    floatx4 s[QT][AP_BK / 16];
#pragma unroll
    for (int kt = 0; kt < AP_BK / 16; ++kt) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const bf16x8 kf = *reinterpret_cast<const bf16x8*>(&k_lds[(kt * 16 + col) * KSTR + ks * 32 + grp * 8]);
#pragma unroll
        for (int qt = 0; qt < QT; ++qt)
          s[qt][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              kf, qf[qt][ks], ks == 0 ? floatx4{0.f, 0.f, 0.f, 0.f} : s[qt][kt], 0, 0, 0);
      }
    }

    // mask (only blocks that reach past the tile's first query, or a window's edge, need
    // it), running softmax, and the probabilities as row operands of the value product
    const bool masked = kb + AP_BK - 1 > pos0 || window > 0;
    bf16x8 pa[QT][AP_BK / 32];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
      const float shift = softmax_prepare<DT + 1>(s[qt], m_run[qt], o[qt], qpos[qt], kb, masked, window, grp,
                                                  scale_log2, slack);
#pragma unroll
      for (int kg = 0; kg < AP_BK / 32; ++kg) pa[qt][kg] = probabilities(s[qt], kg, scale_log2, shift);
    }

    // out += P * V, the values in the same order of keys as the probabilities
#pragma unroll
    for (int kg = 0; kg < AP_BK / 32; ++kg) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const uint16_t* vrow = &v_lds[(dt * 16 + col) * AP_VSTRIDE + kg * 32 + 4 * grp];
        const u32x2 first = *reinterpret_cast<const u32x2*>(vrow);
        const u32x2 second = *reinterpret_cast<const u32x2*>(vrow + 16);
        const u32x4 vv = {first[0], first[1], second[0], second[1]};
        const bf16x8 vf = __builtin_bit_cast(bf16x8, vv);
#pragma unroll
        for (int qt = 0; qt < QT; ++qt)
          o[qt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa[qt][kg], vf, o[qt][dt], 0, 0, 0);
      }
#pragma unroll
      for (int qt = 0; qt < QT; ++qt)
        o[qt][DT] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa[qt][kg], ones, o[qt][DT], 0, 0, 0);
    }
  }
#undef AP_FETCH
#undef AP_SLOT

  store_tile<HD, QT>(out, o, wave, col, grp, group, tok0, ntok, n_heads, kvh * group);
}

// The same for head size 128 and pages that are powers of two of at least 64, with two
// instructions of gfx950 that take the copying out of the loop (global_load_lds_dwordx4 and
// ds_read_b64_tr_b16):
//
//  * Keys and values go from the cache straight into LDS (16 bytes per lane, a wave fills
//    1 KB of consecutive LDS from 64 places of its choice), two buffers each, so that the
//    next block travels while this one is used, with one barrier per block and no staging
//    registers.  A row of a tile is 256 bytes without padding; bank conflicts are avoided
//    by a swizzle on the way in: the 16-byte piece c of key row r lies at piece c ^ (r % 16)
//    (keys) or c ^ (2 * (r % 8)) (values).
//  * The values stay row-major: the transposing LDS read hands a lane, for its column of
//    the output tile, the elements of four consecutive keys, which is the column operand of
//    the value product (lane p of a group of 16 names row p / 4, elements 4 * (p % 4) .. + 3;
//    lane i receives element i % 4 of lanes i / 4, i / 4 + 4, i / 4 + 8, i / 4 + 12).
typedef short s16x4 __attribute__((ext_vector_type(4)));
#define AP_VAHEAD 4  // value operands (16-element output tiles) read ahead of their products
#define AP_LDS(T) __attribute__((address_space(3))) T
#define AP_GLOBAL(T) __attribute__((address_space(1))) T

template <int QT>
__global__ __launch_bounds__(256, 2) void attention_prefill_direct_kernel(
    uint16_t* __restrict__ out, const uint16_t* __restrict__ q, const uint16_t* __restrict__ k_cache,
    const uint16_t* __restrict__ v_cache, const int* __restrict__ block_table, int table_width,
    const int* __restrict__ tiles, int n_heads, int n_kv_heads, int group,
    int page_size, int window, float scale) {
  constexpr int HD = 128, KS = HD / 32, DT = HD / 16;
  constexpr int ROW = HD * 2;  // bytes of a key or value row in LDS
  __shared__ __attribute__((aligned(16))) uint16_t k_a[AP_BK * HD];
  __shared__ __attribute__((aligned(16))) uint16_t k_b[AP_BK * HD];
  __shared__ __attribute__((aligned(16))) uint16_t v_a[AP_BK * HD];
  __shared__ __attribute__((aligned(16))) uint16_t v_b[AP_BK * HD];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 15, grp = lane >> 4;
  // Workgroups start in the order of blockIdx.x and go round the chip's eight dies, each with
  // a cache of its own: neighbours take the same tile for different key/value heads, so the
  // heaviest tiles of all heads start first and a die meets few heads.
  const int kvh = blockIdx.x % n_kv_heads, tile = blockIdx.x / n_kv_heads;
  const int page_shift = __ffs(page_size) - 1, page_mask = page_size - 1;
  const size_t row_elems = static_cast<size_t>(n_kv_heads) * HD;
  const unsigned row_elems32 = n_kv_heads * HD;
  const uint16_t* k_head = k_cache + static_cast<size_t>(kvh) * HD;
  const uint16_t* v_head = v_cache + static_cast<size_t>(kvh) * HD;

  // Where this lane reads its operands (bytes from a tile's start).  Keys: row col of a
  // 16-key tile, piece ks*4 + grp.  Values: row 4*grp + col/4 of a 32-key group, the 8 bytes
  // at element dt*16 + 4*(col%4).
  unsigned k_at[KS], v_at[DT];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) k_at[ks] = col * ROW + (((ks * 4 + grp) ^ col) * 16);
  {
    const unsigned vrow = 4 * grp + (col >> 2), swizzle = 2 * (vrow & 7);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
      v_at[dt] = vrow * ROW + (((2 * dt + ((col & 3) >> 1)) ^ swizzle) * 16) + (col & 1) * 8;
  }
  // What this lane brings in: load i of its wave fills rows 16*wave + 4*i + grp, piece col.
  unsigned k_piece[4], v_piece[4];  // element offsets inside the cache row, swizzle applied
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const unsigned r = 4 * i + grp;
    k_piece[i] = (col ^ r) * 8;
    v_piece[i] = (col ^ (2 * (r & 7))) * 8;
  }

  const int* td = tiles + tile * 4;
  const int tok0 = td[0], ntok = td[1], trow = td[2], pos0 = td[3];
  const int* table = block_table + static_cast<size_t>(trow) * table_width;
  const int kv_last = pos0 + ntok - 1;
  const int k_lo = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
  const int kb_first = (k_lo / AP_BK) * AP_BK;

  // A block of 64 keys lies inside one page.  Rows past the last key repeat it.
#define APD_FETCH(KB, KBUF, VBUF)                                                                      \
  do {                                                                                                 \
    const int page_row = table[(KB) >> page_shift] * page_size + ((KB) & page_mask);                   \
    const uint16_t* k_block = k_head + static_cast<size_t>(page_row) * row_elems;                      \
    const uint16_t* v_block = v_head + static_cast<size_t>(page_row) * row_elems;                      \
    const unsigned last = kv_last - (KB);                                                              \
    _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                                    \
      const unsigned r = 16 * wave + 4 * i + grp;                                                      \
      const unsigned row = (r < last ? r : last) * row_elems32;                                        \
      __builtin_amdgcn_global_load_lds((const AP_GLOBAL(void)*)(k_block + (row + k_piece[i])),         \
                                       (AP_LDS(void)*)((KBUF) + (16 * wave + 4 * i) * HD), 16, 0, 0);  \
      __builtin_amdgcn_global_load_lds((const AP_GLOBAL(void)*)(v_block + (row + v_piece[i])),         \
                                       (AP_LDS(void)*)((VBUF) + (16 * wave + 4 * i) * HD), 16, 0, 0);  \
    }                                                                                                  \
  } while (0)

  APD_FETCH(kb_first, k_a, v_a);

  int qpos[QT];
  bf16x8 qf[QT][KS];
  load_queries<HD, QT>(qpos, qf, q, wave, col, grp, group, tok0, ntok, pos0, n_heads, kvh * group);

  float m_run[QT];          // the running maximum, in units of raw scores
  floatx4 o[QT][DT + 1];    // the output tiles and, last, the rows' sums
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    m_run[qt] = -INFINITY;
#pragma unroll
    for (int dt = 0; dt <= DT; ++dt) o[qt][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  }
  const bf16x8 ones = __builtin_bit_cast(bf16x8, u32x4{0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u});
  const float scale_log2 = scale * 1.44269504088896340736f;
  const float slack = AP_SLACK / scale_log2;  // in units of raw scores

  // One block: wait for its keys and values (this wave's loads, then everyone's), send for
  // the next block into the other buffers (their last readers are past the barrier), and
  // do the math from LDS.
#define APD_BLOCK(KB, KCUR, VCUR, KNEXT, VNEXT)                                                        \
  do {                                                                                                 \
    __builtin_amdgcn_s_waitcnt(0);                                                                     \
    __syncthreads();                                                                                   \
    if ((KB) + AP_BK <= kv_last) APD_FETCH((KB) + AP_BK, KNEXT, VNEXT);                                \
    const AP_LDS(char)* k_tile = (const AP_LDS(char)*)(KCUR);                                          \
    const AP_LDS(char)* v_tile = (const AP_LDS(char)*)(VCUR);                                          \
    /* scores: the operands of the next 16 keys are read while this tile's products run */             \
    floatx4 s[QT][AP_BK / 16];                                                                         \
    bf16x8 kf[2][KS];                                                                                  \
    _Pragma("unroll") for (int ks = 0; ks < KS; ++ks)                                                  \
      kf[0][ks] = *reinterpret_cast<const AP_LDS(bf16x8)*>(k_tile + k_at[ks]);                         \
    _Pragma("unroll") for (int kt = 0; kt < AP_BK / 16; ++kt) {                                        \
      if (kt + 1 < AP_BK / 16) {                                                                       \
        _Pragma("unroll") for (int ks = 0; ks < KS; ++ks)                                              \
          kf[(kt + 1) & 1][ks] =                                                                       \
              *reinterpret_cast<const AP_LDS(bf16x8)*>(k_tile + k_at[ks] + (kt + 1) * 16 * ROW);       \
      }                                                                                                \
      __builtin_amdgcn_sched_barrier(0);                                                               \
      _Pragma("unroll") for (int ks = 0; ks < KS; ++ks)                                                \
        _Pragma("unroll") for (int qt = 0; qt < QT; ++qt)                                              \
          s[qt][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(                                         \
              kf[kt & 1][ks], qf[qt][ks], ks == 0 ? floatx4{0.f, 0.f, 0.f, 0.f} : s[qt][kt], 0, 0, 0); \
      __builtin_amdgcn_sched_barrier(0);                                                               \
    }                                                                                                  \
    /* the first values are on their way from LDS during the softmax */                                \
    s16x4 vf[AP_VAHEAD][2];                                                                            \
    _Pragma("unroll") for (int a = 0; a < AP_VAHEAD; ++a) {                                            \
      vf[a][0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((AP_LDS(s16x4)*)(v_tile + v_at[a]));          \
      vf[a][1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((AP_LDS(s16x4)*)(v_tile + v_at[a] + 16 * ROW)); \
    }                                                                                                  \
    __builtin_amdgcn_sched_barrier(0);                                                                 \
    const bool masked = (KB) + AP_BK - 1 > pos0 || window > 0;                                         \
    bf16x8 pa[QT][AP_BK / 32];                                                                         \
    float shift[QT];                                                                                   \
    _Pragma("unroll") for (int qt = 0; qt < QT; ++qt) {                                                \
      shift[qt] = softmax_prepare<DT + 1>(s[qt], m_run[qt], o[qt], qpos[qt], (KB), masked, window,     \
                                          grp, scale_log2, slack);                                     \
      pa[qt][0] = probabilities(s[qt], 0, scale_log2, shift[qt]);                                      \
    }                                                                                                  \
    __builtin_amdgcn_sched_barrier(0);                                                                 \
    /* the products of the first 32 keys run while the vector unit takes the exponentials of the */    \
    /* other 32: per output tile two value reads, QT products, and a share of that arithmetic */       \
    _Pragma("unroll") for (int qt = 0; qt < QT; ++qt)                                                  \
      pa[qt][1] = probabilities(s[qt], 1, scale_log2, shift[qt]);                                      \
    _Pragma("unroll") for (int it = 0; it < DT; ++it) {                                                \
      const bf16x8 vnow = __builtin_bit_cast(                                                          \
          bf16x8, __builtin_shufflevector(vf[it % AP_VAHEAD][0], vf[it % AP_VAHEAD][1], 0, 1, 2, 3, 4, 5, 6, 7)); \
      vf[it % AP_VAHEAD][0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(                                 \
          (AP_LDS(s16x4)*)(v_tile + v_at[(it + AP_VAHEAD) % DT] + ((it + AP_VAHEAD) / DT) * 32 * ROW)); \
      vf[it % AP_VAHEAD][1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(                                 \
          (AP_LDS(s16x4)*)(v_tile + v_at[(it + AP_VAHEAD) % DT] + ((it + AP_VAHEAD) / DT) * 32 * ROW + 16 * ROW)); \
      _Pragma("unroll") for (int qt = 0; qt < QT; ++qt)                                                \
        o[qt][it] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa[qt][0], vnow, o[qt][it], 0, 0, 0);      \
    }                                                                                                  \
    _Pragma("unroll") for (int it = 0; it < DT; ++it) {                                                \
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  /* LDS reads */                              \
      __builtin_amdgcn_sched_group_barrier(0x008, QT, 0); /* matrix products */                        \
      __builtin_amdgcn_sched_group_barrier(0x402, (20 * QT + DT - 1) / DT, 0); /* vector arithmetic */ \
    }                                                                                                  \
    __builtin_amdgcn_sched_barrier(0);                                                                 \
    _Pragma("unroll") for (int it = DT; it < 2 * DT; ++it) {                                           \
      const bf16x8 vnow = __builtin_bit_cast(                                                          \
          bf16x8, __builtin_shufflevector(vf[it % AP_VAHEAD][0], vf[it % AP_VAHEAD][1], 0, 1, 2, 3, 4, 5, 6, 7)); \
      if (it + AP_VAHEAD < 2 * DT) {                                                                   \
        vf[it % AP_VAHEAD][0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(                               \
            (AP_LDS(s16x4)*)(v_tile + v_at[(it + AP_VAHEAD) % DT] + 32 * ROW));                        \
        vf[it % AP_VAHEAD][1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(                               \
            (AP_LDS(s16x4)*)(v_tile + v_at[(it + AP_VAHEAD) % DT] + 32 * ROW + 16 * ROW));             \
      }                                                                                                \
      __builtin_amdgcn_sched_barrier(0);                                                               \
      _Pragma("unroll") for (int qt = 0; qt < QT; ++qt)                                                \
        o[qt][it % DT] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa[qt][1], vnow, o[qt][it % DT], 0, 0, 0); \
      __builtin_amdgcn_sched_barrier(0);                                                               \
    }                                                                                                  \
    _Pragma("unroll") for (int kg = 0; kg < AP_BK / 32; ++kg)                                          \
      _Pragma("unroll") for (int qt = 0; qt < QT; ++qt)                                                \
        o[qt][DT] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa[qt][kg], ones, o[qt][DT], 0, 0, 0);     \
  } while (0)

  for (int kb = kb_first;; kb += 2 * AP_BK) {
    APD_BLOCK(kb, k_a, v_a, k_b, v_b);
    if (kb + AP_BK > kv_last) break;
    APD_BLOCK(kb + AP_BK, k_b, v_b, k_a, v_a);
    if (kb + 2 * AP_BK > kv_last) break;
  }
#undef APD_BLOCK
#undef APD_FETCH

  store_tile<HD, QT>(out, o, wave, col, grp, group, tok0, ntok, n_heads, kvh * group);
}

// tiles: [n_tiles, 4] = (index of the tile's first token in q/out, its token count, its row of
// the block table, the position of its first token).  A tile holds consecutive tokens of one
// request, at most floor(rows / group) of them; rows (64 or 128) is the number of (token,
// head) query rows a workgroup takes.
extern "C" int pylon_attention_prefill(void* out, const void* q, const void* k_cache, const void* v_cache,
                                       const int* block_table, int table_width, const int* tiles,
                                       int n_tiles, int n_heads, int n_kv_heads, int head_dim,
                                       int page_size, int window, float scale, int rows, hipStream_t stream) {
  PYLON_REQUIRE(rows == 64 || rows == 128, "attention_prefill: 64 or 128 query rows per workgroup, got %d", rows);
  PYLON_REQUIRE(n_tiles >= 0 && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
                "attention_prefill: %d query heads cannot be grouped over %d key/value heads", n_heads,
                n_kv_heads);
  PYLON_REQUIRE(n_heads / n_kv_heads <= rows, "attention_prefill: at most %d query heads per key/value head",
                rows);
  PYLON_REQUIRE(head_dim == 64 || head_dim == 128 || head_dim == 256,
                "attention_prefill: head_dim %d is not 64, 128 or 256", head_dim);
  PYLON_REQUIRE(page_size > 0 && table_width > 0 && window >= 0, "attention_prefill: bad page size, width or window");
  PYLON_REQUIRE(table_width <= AP_TABLE, "attention_prefill: a request may hold at most %d pages, the table has %d columns",
                AP_TABLE, table_width);
  PYLON_REQUIRE(static_cast<long long>(n_tiles) * n_kv_heads < (1LL << 31), "attention_prefill: too many tiles for one launch");
  if (n_tiles == 0) return 0;
  const int group = n_heads / n_kv_heads;
  dim3 grid(n_tiles * n_kv_heads), block(256);
  const bool pow2 = (page_size & (page_size - 1)) == 0;
  const int paging = !pow2 ? 0 : (page_size >= AP_BK ? 2 : 1);
  PYLON_REQUIRE(static_cast<long long>(n_kv_heads) * head_dim * AP_BK < (1LL << 31),
                "attention_prefill: %d key/value heads of %d elements are too wide", n_kv_heads, head_dim);
#define GO_PAGING(HD, QT, PG)                                                                            \
  hipLaunchKernelGGL((attention_prefill_kernel<HD, QT, PG>), grid, block, 0, stream, (uint16_t*)out,     \
                     (const uint16_t*)q, (const uint16_t*)k_cache, (const uint16_t*)v_cache, block_table, \
                     table_width, tiles, n_heads, n_kv_heads, group, page_size, window, scale)
#define GO(HD, QT)                                                                                       \
  do {                                                                                                   \
    if (paging == 2) GO_PAGING(HD, QT, 2);                                                               \
    else if (paging == 1) GO_PAGING(HD, QT, 1);                                                          \
    else GO_PAGING(HD, QT, 0);                                                                           \
  } while (0)
  if (head_dim == 128 && paging == 2) {
#define GO_DIRECT(QT)                                                                                    \
  hipLaunchKernelGGL((attention_prefill_direct_kernel<QT>), grid, block, 0, stream, (uint16_t*)out,      \
                     (const uint16_t*)q, (const uint16_t*)k_cache, (const uint16_t*)v_cache, block_table, \
                     table_width, tiles, n_heads, n_kv_heads, group, page_size, window, scale)
    if (rows == 64) GO_DIRECT(1); else GO_DIRECT(2);
#undef GO_DIRECT
  } else if (rows == 64) {
    if (head_dim == 64) GO(64, 1);
    else if (head_dim == 128) GO(128, 1);
    else GO(256, 1);
  } else {
    if (head_dim == 64) GO(64, 2);
    else if (head_dim == 128) GO(128, 2);
    else GO(256, 2);
  }
#undef GO
#undef GO_PAGING
  PYLON_LAUNCHED("attention_prefill");
}
