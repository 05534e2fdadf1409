// Paged attention for steps with few query tokens (decode): bfloat16, head sizes 64, 128
// and 256, any grouping of up to 16 query heads per key/value head.
//
// A decode step waits on memory latency more than on bandwidth, so the kernel is built to
// make few trips to memory.  One workgroup takes one (token, key/value head) and handles
// all query heads of the group together.  Its wavefronts cut the token's keys into equal
// ranges; a wave issues the loads of up to 64 keys and of their values all at once, then
// computes.  The waves' partial results (running maximum, sum, weighted values, in float)
// meet in LDS and are merged in the order of the ranges, so no partial result ever goes
// through global memory and there is no second kernel.
//
// Few tokens with long contexts would leave most of the chip idle that way.  Then the keys
// of a (token, head) are first cut over several workgroups (gridDim.z); each leaves its
// merged partial result (maximum, sum, unnormalised values, float) in a scratch buffer,
// and a second small kernel merges those in the order of the cuts.
//
// Scores come from the 16x16x32 bf16 matrix instruction with 16 keys as rows and the
// group's query heads as columns (unused columns are zero).  The weighted sum of values
// runs on the vector units: a value row is read by head_dim/8 lanes, 16 bytes each, so one
// load instruction fetches the rows of several keys; every lane accumulates its eight
// elements over its keys and the lane groups are summed at the end.  Softmax statistics are float throughout.
//
// The kernel can also take over the step that precedes attention: given the raw q/k/v
// projection instead of prepared queries, each workgroup first norms and rotates its
// group's query heads (kept in LDS) and its key head, and stores that key and its value
// head at the token's cache slot.  The loads of older keys do not wait for that: the new
// row is taken from LDS.  One launch and one pass over the projection less per layer.
#pragma once
#include "common.h"
#include "head_prepare.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

#define AD_MAX_GROUP 16
#define AD_TILE 16   // keys per score tile
#define AD_SUPER 64  // most keys whose loads are in flight together (four score tiles)
#define AD_MAX_WAVES 8

// What the kernel needs to prepare q, k and v itself (PREP): the raw projection
// [tokens, row_stride] with q heads first, then k heads, then v heads.
// With n_parts > 0 the projection comes as that many float partial sums (a product whose K
// was cut over workgroups), part_stride elements apart; the kernel adds them in order and
// rounds the sum to bfloat16 once, which is what a projection stored as bfloat16 holds.
struct DecodePrep {
  const void* qkv;
  long long row_stride;
  int n_parts;
  long long part_stride;
  const float* q_weight;  // per-head RMSNorm weights, or null
  const float* k_weight;
  float eps;
  const float* inv_freq;  // head_dim/2 rotation frequencies, or null
  const int* slot_map;    // cache slot of each token's key and value; null: store nothing
};

// With PREP the kernel writes the caches before it reads them, so they are neither const
// nor restrict there.
template <bool PREP>
struct DecodeCache {
  typedef const uint16_t* __restrict__ ptr;
};
template <>
struct DecodeCache<true> {
  typedef uint16_t* ptr;
};

static __host__ __device__ size_t decode_lds_floats(int n_waves, int gp, int head_dim) {
  const size_t n = static_cast<size_t>(n_waves) * AD_SUPER * gp + static_cast<size_t>(n_waves) * gp * head_dim +
                   static_cast<size_t>(n_waves) * gp * 2;
  return (n + 3) & ~static_cast<size_t>(3);  // what follows stays 16-byte aligned
}

// EPL = head_dim / 64, KSTEPS = head_dim / 32, GP = heads per group rounded up to 1, 2, 4, 8, 16
// PARTS (with PREP): the projection comes as float partial sums (an instance of its own, so
// that the others keep their registers).
template <int EPL, int KSTEPS, int GP, bool PREP, bool PARTS = false>
__global__ __launch_bounds__(AD_MAX_WAVES* PYLON_WAVE) void attention_decode_kernel(
    uint16_t* __restrict__ out, const uint16_t* __restrict__ q, typename DecodeCache<PREP>::ptr k_cache,
    typename DecodeCache<PREP>::ptr v_cache, const int* __restrict__ block_table, int table_width,
    const int* __restrict__ tok_row, const int* __restrict__ positions, int n_heads, int n_kv_heads,
    int page_size, int window, float scale, DecodePrep prep, float* __restrict__ partial) {
  constexpr int HD = EPL * 64;
  // keys whose loads are in flight together: 64 (four score tiles), or 32 where the
  // fragments of 64 keys and the accumulators would not fit the registers
  constexpr int SUPER = (EPL == 4 || GP >= 8) ? AD_SUPER / 2 : AD_SUPER;
  constexpr int TILES = SUPER / AD_TILE;
  // per wave: probabilities of the keys in flight; then the waves' partial results
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int n_waves = blockDim.x / PYLON_WAVE;
  const int lane = threadIdx.x & (PYLON_WAVE - 1);
  const int wave = threadIdx.x / PYLON_WAVE;
  float(*p_tile)[GP] = reinterpret_cast<float(*)[GP]>(lds + wave * AD_SUPER * GP);
  float* part_acc = lds + n_waves * AD_SUPER * GP;  // [wave][GP][HD]
  float* part_ml = part_acc + n_waves * GP * HD;    // [wave][GP][2]
  uint16_t* q_lds = reinterpret_cast<uint16_t*>(lds + decode_lds_floats(n_waves, GP, HD));  // [GP][HD], PREP only
  const int col = lane & 15, grp = lane >> 4;
  const int kvh = blockIdx.x, t = blockIdx.y;
  const int group = n_heads / n_kv_heads;
  // When tok_row is null, token t uses row t of the block table.  Its first 64 entries are
  // then fetched together with the position (one trip to memory instead of two); lane i
  // keeps entry i.
  const int* table = block_table + static_cast<size_t>(tok_row ? tok_row[t] : t) * table_width;
  const int table_entry = (lane < table_width) ? table[lane] : 0;
  const int pos = positions[t];

  // the keys of this workgroup (all of them unless gridDim.z cuts them), then of this wave
  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int n_cuts = gridDim.z, cut = blockIdx.z;
  int per_cut = (pos + 1 - first + n_cuts - 1) / n_cuts;
  per_cut = (per_cut + AD_TILE - 1) / AD_TILE * AD_TILE;
  const int c_begin = first + cut * per_cut;
  const int c_end = c_begin + per_cut < pos + 1 ? c_begin + per_cut : pos + 1;
  const bool holds_last = pos >= c_begin && pos < c_begin + per_cut;  // true for exactly one cut
  const int n_keys = c_end > c_begin ? c_end - c_begin : 0;
  // A wave's range is a whole number of the batches it loads at once: with few keys, fewer
  // waves take part, rather than all of them loading a mostly empty batch each.
  int per_wave = (n_keys + n_waves - 1) / n_waves;
  per_wave = (per_wave + SUPER - 1) / SUPER * SUPER;
  const int k_begin = c_begin + wave * per_wave;
  int k_end = k_begin + per_wave;
  if (k_end > c_end) k_end = c_end;

  // PREP: the token's own key and value, as they go into the cache, also stay in LDS: the
  // loads of old keys need not wait for those stores, and the new row is taken from here.
  uint16_t* kv_new = reinterpret_cast<uint16_t*>(reinterpret_cast<float*>(q_lds + GP * HD) + n_waves * HD);
  bool stored_new = false;
  if constexpr (PREP) {
    // 512/head_dim heads per wave at a time: the group's query heads into LDS, then this
    // key head and this value head into the token's cache slot.
    constexpr int LPH = HD / 8, HPW = PYLON_WAVE / LPH;
    // the token's rotation table, one private copy per wave: no workgroup barrier before use
    float* cs = reinterpret_cast<float*>(q_lds + GP * HD) + wave * HD;
    const size_t row_at = static_cast<size_t>(t) * prep.row_stride;
    // the new key and value are stored by the one workgroup whose keys include them
    const int slot = (prep.slot_map != nullptr && holds_last) ? prep.slot_map[t] : -1;
    const int jobs = group + (slot >= 0 ? 2 : 0);
    stored_new = slot >= 0;
    const int j = lane % LPH;
    // job -> where its head lies in the projection's row
    auto load = [&](int job, float v[8]) {
      const int head = job < group ? kvh * group + job : n_heads + (job == group ? 0 : n_kv_heads) + kvh;
      const size_t at = row_at + static_cast<size_t>(head) * HD + 8 * j;
      if constexpr (PARTS) {
        sum8_parts(static_cast<const float*>(prep.qkv) + at, prep.n_parts, prep.part_stride, v);
      } else {
        load8_bf16(static_cast<const uint16_t*>(prep.qkv) + at, v);
      }
    };
    // The first round's loads do not wait for the position.
    int job = wave * HPW + lane / LPH;
    float v[8];
    load(job < jobs ? job : jobs - 1, v);
    if (prep.inv_freq != nullptr && wave * HPW < jobs) {
      const float fpos = static_cast<float>(pos);
      for (int i = lane; i < HD / 2; i += PYLON_WAVE) {
        const float angle = fpos * prep.inv_freq[i];
        cs[i] = cosf(angle);
        cs[HD / 2 + i] = sinf(angle);
      }
      __builtin_amdgcn_wave_barrier();  // private to the wave: program order suffices
    }
    for (int h0 = wave * HPW; h0 < jobs; h0 += n_waves * HPW) {
      job = h0 + lane / LPH;
      const bool valid = job < jobs;
      if (!valid) job = jobs - 1;
      if (h0 != wave * HPW) load(job, v);
      const bool is_q = job < group, is_key = job == group;
      const float* weight = is_q ? prep.q_weight : (is_key ? prep.k_weight : nullptr);
      norm_rotate8<HD>(v, j, weight, prep.eps, (prep.inv_freq != nullptr && (is_q || is_key)) ? cs : nullptr);
      if (valid && is_q) {
        store8_bf16(q_lds + job * HD + 8 * j, v);
      } else if (valid) {
        uint16_t* dst = (is_key ? k_cache : v_cache) + (static_cast<size_t>(slot) * n_kv_heads + kvh) * HD + 8 * j;
        store8_bf16(dst, v);
        store8_bf16(kv_new + (is_key ? 0 : HD) + 8 * j, v);
      }
    }
  }

  // Every load of 64 keys and values is issued before the first is used.  Lane `lane`
  // owns key BASE + lane for the value rows; for the score tiles, row `col` of tile `kt`
  // is key BASE + 16*kt + col.  Keys past the end repeat the last key.  Values: LPK lanes
  // read one key's row, 8 elements each; KPI keys per load instruction.
  constexpr int LPK = HD / 8;             // lanes that share one key's value row
  constexpr int KPI = PYLON_WAVE / LPK;   // keys per value load instruction
  const int vkey = lane / LPK, vchunk = lane % LPK;
  bf16x8 kf[TILES][KSTEPS];
  uint4 vv[SUPER / KPI];
#define AD_LOAD(BASE)                                                                                  \
  do {                                                                                                 \
    const int my_key = ((BASE) + lane < k_end) ? (BASE) + lane : k_end - 1;                            \
    const int my_page = my_key / page_size;                                                            \
    int page_id = __shfl(table_entry, my_page & (PYLON_WAVE - 1), PYLON_WAVE);                         \
    if (my_page >= PYLON_WAVE) page_id = table[my_page];                                               \
    const int my_phys = page_id * page_size + my_key % page_size;                                      \
    _Pragma("unroll") for (int kt = 0; kt < TILES; ++kt) {                                             \
      const int phys = __shfl(my_phys, kt * 16 + col, PYLON_WAVE);                                     \
      const uint16_t* krow = k_cache + (static_cast<size_t>(phys) * n_kv_heads + kvh) * HD;            \
      _Pragma("unroll") for (int ks = 0; ks < KSTEPS; ++ks)                                            \
          kf[kt][ks] = *reinterpret_cast<const bf16x8*>(krow + ks * 32 + grp * 8);                     \
    }                                                                                                  \
    _Pragma("unroll") for (int i = 0; i < SUPER / KPI; ++i) {                                       \
      const int pk = __shfl(my_phys, i * KPI + vkey, PYLON_WAVE);                                      \
      const uint16_t* vrow = v_cache + (static_cast<size_t>(pk) * n_kv_heads + kvh) * HD;              \
      vv[i] = *reinterpret_cast<const uint4*>(vrow + vchunk * 8);                                      \
    }                                                                                                  \
  } while (0)

  if (k_begin < k_end) AD_LOAD(k_begin);  // on their way while the queries settle in LDS
  if constexpr (PREP) {
    // Only LDS has to be in order across this barrier (the queries, the new key and value):
    // the loads above and the stores into the cache stay in flight.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
  }
  // query fragments: column `col` is head kvh*group + col of the token
  bf16x8 qf[KSTEPS];
  {
    const bool valid = col < group;
    const uint16_t* qrow = PREP ? q_lds + (valid ? col : 0) * HD
                                : q + (static_cast<size_t>(t) * n_heads + kvh * group + (valid ? col : 0)) * HD;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      if (valid) {
        qf[ks] = *reinterpret_cast<const bf16x8*>(qrow + ks * 32 + grp * 8);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) qf[ks][i] = (__bf16)0.0f;
      }
    }
  }

  float m_run = -INFINITY, l_run = 0.f;  // for head `col` (same in the 4 lanes that share it)
  float acc[GP][8];  // elements vchunk*8 .. +7 over this lane's keys; rows past `group` unused
#pragma unroll
  for (int h = 0; h < GP; ++h)
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[h][i] = 0.f;

  // this wave's keys end with the token's own, which the cache may not hold yet
  const bool patch = PREP && stored_new && k_end == pos + 1;
  for (int base = k_begin; base < k_end; base += SUPER) {
    if (base != k_begin) AD_LOAD(base);
    if (patch && base + SUPER >= k_end) {
      // rows of the new key (and of the lanes past the end, which repeat it) come from LDS
#pragma unroll
      for (int kt = 0; kt < TILES; ++kt) {
        if (base + kt * 16 + col >= pos) {
#pragma unroll
          for (int ks = 0; ks < KSTEPS; ++ks)
            kf[kt][ks] = *reinterpret_cast<const bf16x8*>(kv_new + ks * 32 + grp * 8);
        }
      }
#pragma unroll
      for (int i = 0; i < SUPER / KPI; ++i) {
        if (base + i * KPI + vkey >= pos) vv[i] = *reinterpret_cast<const uint4*>(kv_new + HD + vchunk * 8);
      }
    }

    floatx4 s[TILES];
#pragma unroll
    for (int kt = 0; kt < TILES; ++kt) {
      s[kt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks)
        s[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[kt][ks], qf[ks], s[kt], 0, 0, 0);
    }
    // lane holds, for head `col`, the scores of keys base + 16*kt + 4*grp + r
    float tile_max = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < TILES; ++kt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const bool live = base + 16 * kt + 4 * grp + r < k_end;
        s[kt][r] = live ? s[kt][r] * scale : -INFINITY;
        tile_max = fmaxf(tile_max, s[kt][r]);
      }
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, PYLON_WAVE));
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, PYLON_WAVE));
    const float m_new = fmaxf(m_run, tile_max);  // finite: key `base` is always live
    const float corr = expf(m_run - m_new);
    float tile_sum = 0.f;
    __builtin_amdgcn_wave_barrier();  // the previous round's reads of p_tile come first
#pragma unroll
    for (int kt = 0; kt < TILES; ++kt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float p = expf(s[kt][r] - m_new);  // exp(-inf) = 0 for keys past the end
        tile_sum += p;
        if (col < GP) p_tile[16 * kt + 4 * grp + r][col] = p;
      }
    tile_sum += __shfl_xor(tile_sum, 16, PYLON_WAVE);
    tile_sum += __shfl_xor(tile_sum, 32, PYLON_WAVE);
    l_run = l_run * corr + tile_sum;
    m_run = m_new;
    __builtin_amdgcn_wave_barrier();  // p_tile is private to the wave: program order suffices
    // rescale what has been accumulated: the factor of head h sits in lane h
#pragma unroll
    for (int h = 0; h < GP; ++h) {
      const float c = __shfl(corr, h, PYLON_WAVE);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[h][i] *= c;
    }
    // keys past the end weigh 0 and their value row is the (finite) last key's
#pragma unroll
    for (int i = 0; i < SUPER / KPI; ++i) {
      const uint32_t w[4] = {vv[i].x, vv[i].y, vv[i].z, vv[i].w};
      float v[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[2 * j] = __uint_as_float(w[j] << 16);
        v[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
      }
#pragma unroll
      for (int h = 0; h < GP; ++h) {
        const float p = p_tile[i * KPI + vkey][h];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[h][j] = fmaf(p, v[j], acc[h][j]);
      }
    }
  }
  // sum over the lane groups that took different keys (a fixed tree of additions)
#pragma unroll
  for (int h = 0; h < GP; ++h)
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int off = LPK; off < PYLON_WAVE; off <<= 1) acc[h][j] += __shfl_xor(acc[h][j], off, PYLON_WAVE);

  // leave this wave's partial result in LDS: acc[h][j] is element vchunk*8 + j of head h
#pragma unroll
  for (int h = 0; h < GP; ++h) {
    float* arow = part_acc + (static_cast<size_t>(wave) * GP + h) * HD;
    if (vkey == 0) {
#pragma unroll
      for (int j = 0; j < 8; ++j) arow[vchunk * 8 + j] = acc[h][j];
    }
    const float mh = __shfl(m_run, h, PYLON_WAVE), lh = __shfl(l_run, h, PYLON_WAVE);
    if (lane == 0) {
      part_ml[(wave * GP + h) * 2] = mh;
      part_ml[(wave * GP + h) * 2 + 1] = lh;
    }
  }
  __syncthreads();
  // wave h merges head h over all ranges, in the order of the ranges
  for (int h = wave; h < group; h += n_waves) {
    float m = -INFINITY;
    for (int w = 0; w < n_waves; ++w) m = fmaxf(m, part_ml[(w * GP + h) * 2]);
    float l = 0.f;
    float o[EPL];
#pragma unroll
    for (int i = 0; i < EPL; ++i) o[i] = 0.f;
    for (int w = 0; w < n_waves; ++w) {
      const float lw = part_ml[(w * GP + h) * 2 + 1];
      const float f = (lw == 0.f) ? 0.f : expf(part_ml[(w * GP + h) * 2] - m);  // an empty range
      l += lw * f;
      const float* arow = part_acc + (static_cast<size_t>(w) * GP + h) * HD;
#pragma unroll
      for (int i = 0; i < EPL; ++i) o[i] = fmaf(arow[lane * EPL + i], f, o[i]);
    }
    if (n_cuts > 1) {
      // [token][head][cut][HD values, maximum, sum]
      float* prow = partial + ((static_cast<size_t>(t) * n_heads + kvh * group + h) * n_cuts + cut) * (HD + 2);
#pragma unroll
      for (int i = 0; i < EPL; ++i) prow[lane * EPL + i] = o[i];
      if (lane == 0) {
        prow[HD] = m;
        prow[HD + 1] = l;
      }
    } else {
      const float inv = 1.0f / l;
      uint16_t* orow = out + (static_cast<size_t>(t) * n_heads + kvh * group + h) * HD + lane * EPL;
#pragma unroll
      for (int i = 0; i < EPL; ++i) orow[i] = float_to_bf16_bits(o[i] * inv);
    }
  }
}

#undef AD_LOAD

// One wave per (token, query head) merges the partial results of the cuts (at most 64), in
// their order.  Lane c takes the maximum and the sum of cut c, so that all of them come in one
// trip to memory, and the weighted values come eight cuts a batch, every load of a batch issued
// before its first addition: the time no longer grows by a trip to memory per cut (32 cuts:
// 19 us before).
template <int EPL>
__global__ __launch_bounds__(PYLON_WAVE) void attention_decode_merge_kernel(
    uint16_t* __restrict__ out, const float* __restrict__ partial, int n_heads, int n_cuts) {
  constexpr int HD = EPL * 64;
  constexpr int BATCH = 8;
  const int lane = threadIdx.x;
  const size_t row = static_cast<size_t>(blockIdx.y) * n_heads + blockIdx.x;
  const float* prow = partial + row * n_cuts * (HD + 2);
  float mc = -INFINITY, lc = 0.f;
  if (lane < n_cuts) {
    mc = prow[lane * (HD + 2) + HD];
    lc = prow[lane * (HD + 2) + HD + 1];
  }
  float m = mc;
#pragma unroll
  for (int off = PYLON_WAVE / 2; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, PYLON_WAVE));
  const float fc = (lc == 0.f) ? 0.f : expf(mc - m);  // a cut without keys
  const float wc = lc * fc;
  float l = 0.f, o[EPL];
#pragma unroll
  for (int i = 0; i < EPL; ++i) o[i] = 0.f;
  for (int c0 = 0; c0 < n_cuts; c0 += BATCH) {
    float v[BATCH][EPL];
#pragma unroll
    for (int u = 0; u < BATCH; ++u) {
      const int c = (c0 + u < n_cuts) ? c0 + u : n_cuts - 1;  // past the end: a cut again, unused
#pragma unroll
      for (int i = 0; i < EPL; ++i) v[u][i] = prow[c * (HD + 2) + lane * EPL + i];
    }
#pragma unroll
    for (int u = 0; u < BATCH; ++u) {
      const int c = c0 + u;
      const float f = __shfl(fc, c & (PYLON_WAVE - 1), PYLON_WAVE);
      const float w = __shfl(wc, c & (PYLON_WAVE - 1), PYLON_WAVE);
      if (c < n_cuts) {
        l += w;
#pragma unroll
        for (int i = 0; i < EPL; ++i) o[i] = fmaf(v[u][i], f, o[i]);
      }
    }
  }
  const float inv = 1.0f / l;
  uint16_t* orow = out + row * HD + lane * EPL;
#pragma unroll
  for (int i = 0; i < EPL; ++i) orow[i] = float_to_bf16_bits(o[i] * inv);
}

static inline size_t decode_lds_bytes(int n_waves, int gp, int head_dim, bool prep) {
  return sizeof(float) * decode_lds_floats(n_waves, gp, head_dim) +
         (prep ? sizeof(uint16_t) * static_cast<size_t>(gp) * head_dim + sizeof(float) * n_waves * head_dim +
                     sizeof(uint16_t) * 2 * head_dim
               : 0);
}

template <int EPL, bool PREP, bool PARTS = false>
static int launch_decode(void* out, const void* q, void* k_cache, void* v_cache,
                         const int* block_table, int table_width, const int* tok_row,
                         const int* positions, int tokens, int n_heads, int n_kv_heads, int page_size,
                         int window, float scale, int n_waves, DecodePrep prep, int n_cuts, float* partial,
                         hipStream_t stream) {
  const int group = n_heads / n_kv_heads;
  const int gp = group <= 1 ? 1 : group <= 2 ? 2 : group <= 4 ? 4 : group <= 8 ? 8 : 16;
  // the partial results of all waves have to fit into 64 KB of LDS
  while (n_waves > 1 && decode_lds_bytes(n_waves, gp, EPL * 64, PREP) > 65536) n_waves /= 2;
  const size_t lds = decode_lds_bytes(n_waves, gp, EPL * 64, PREP);
  dim3 grid(n_kv_heads, tokens, n_cuts), block(n_waves * PYLON_WAVE);
#define LAUNCH(GP)                                                                                         \
  hipLaunchKernelGGL((attention_decode_kernel<EPL, EPL * 2, GP, PREP, PARTS>), grid, block, lds, stream,   \
                     (uint16_t*)out, (const uint16_t*)q, (typename DecodeCache<PREP>::ptr)k_cache,         \
                     (typename DecodeCache<PREP>::ptr)v_cache, block_table, table_width, tok_row, positions, \
                     n_heads, n_kv_heads, page_size, window, scale, prep, partial)
  switch (gp) {
    case 1: LAUNCH(1); break;
    case 2: LAUNCH(2); break;
    case 4: LAUNCH(4); break;
    case 8: LAUNCH(8); break;
    default: LAUNCH(16); break;
  }
#undef LAUNCH
  if (n_cuts > 1)
    hipLaunchKernelGGL((attention_decode_merge_kernel<EPL>), dim3(n_heads, tokens), dim3(PYLON_WAVE), 0, stream,
                       (uint16_t*)out, partial, n_heads, n_cuts);
  return 0;
}

// The launches of one head size, by what the kernel starts from (mode 0: prepared queries; 1: the
// raw projection in bfloat16; 2: float partial sums of it).  Each head size is a translation unit
// of its own, so that the many instances compile side by side.
#define AD_MODE_QUERIES 0
#define AD_MODE_PROJECTION 1
#define AD_MODE_PARTIAL_SUMS 2
#define AD_RUN_ARGS                                                                                     \
  int mode, void *out, const void *q, void *k_cache, void *v_cache, const int *block_table, int table_width, \
      const int *tok_row, const int *positions, int tokens, int n_heads, int n_kv_heads, int page_size,    \
      int window, float scale, int n_waves, DecodePrep prep, int n_cuts, float *partial, hipStream_t stream
int pylon_decode_run_64(AD_RUN_ARGS);
int pylon_decode_run_128(AD_RUN_ARGS);
int pylon_decode_run_256(AD_RUN_ARGS);

template <int EPL>
static int decode_run(AD_RUN_ARGS) {
  if (mode == AD_MODE_QUERIES)
    return launch_decode<EPL, false>(out, q, k_cache, v_cache, block_table, table_width, tok_row, positions, tokens,
                                     n_heads, n_kv_heads, page_size, window, scale, n_waves, prep, n_cuts, partial,
                                     stream);
  if (mode == AD_MODE_PROJECTION)
    return launch_decode<EPL, true>(out, nullptr, k_cache, v_cache, block_table, table_width, tok_row, positions,
                                    tokens, n_heads, n_kv_heads, page_size, window, scale, n_waves, prep, n_cuts,
                                    partial, stream);
  return launch_decode<EPL, true, true>(out, nullptr, k_cache, v_cache, block_table, table_width, tok_row, positions,
                                        tokens, n_heads, n_kv_heads, page_size, window, scale, n_waves, prep, n_cuts,
                                        partial, stream);
}
