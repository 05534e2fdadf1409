// Paged causal attention for prompt portions: bfloat16, head sizes 64, 128 and 256, any
// grouping of query heads.  Flash-attention on the 16x16x32 bf16 matrix instruction.
//
// A workgroup of four wavefronts takes one tile of consecutive tokens of one request and
// one key/value head, together with all query heads of that head's group: a (token, head)
// pair is one of up to 64 query rows, 16 per wave.  Keys and values are walked 64 at a
// time.  The workgroup stages the 64 keys (row-major) and the 64 values (transposed, so
// that a lane can read four consecutive keys of one element) in LDS.  Scores are computed
// transposed (keys as rows, queries as columns): the result registers of a score tile then
// already have the layout the row operand of the value product needs, and the running
// maximum and sum of a query live in the lanes of its column.  Scores, softmax and the
// output accumulators are float.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

#define AP_BK 64       // keys per iteration
#define AP_ROWS 64     // query rows per workgroup
#define AP_QT 1        // 16-row query tiles per wave
#define AP_VSTRIDE 66  // keys per row of the transposed value tile (+2: spreads LDS banks)

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  return static_cast<uint32_t>(float_to_bf16_bits(lo)) | (static_cast<uint32_t>(float_to_bf16_bits(hi)) << 16);
}

template <int HD>
__global__ __launch_bounds__(256) void attention_prefill_kernel(
    uint16_t* __restrict__ out, const uint16_t* __restrict__ q, const uint16_t* __restrict__ k_cache,
    const uint16_t* __restrict__ v_cache, const int* __restrict__ block_table, int table_width,
    const int* __restrict__ tiles, int n_heads, int n_kv_heads, int group, int page_size, int window,
    float scale) {
  constexpr int KS = HD / 32;        // 32-wide steps along the head for a score tile
  constexpr int DT = HD / 16;        // 16-wide output tiles along the head
  constexpr int KSTR = HD + 8;       // row stride of the key tile (elements)
  constexpr int CHUNKS = HD / 8;     // 16-byte chunks per key row
  __shared__ __attribute__((aligned(16))) uint16_t k_lds[AP_BK * KSTR];
  __shared__ __attribute__((aligned(16))) uint16_t v_lds[HD * AP_VSTRIDE];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int kvh = blockIdx.y;
  const int* td = tiles + blockIdx.x * 4;
  const int tok0 = td[0], ntok = td[1], trow = td[2], pos0 = td[3];
  const int* table = block_table + static_cast<size_t>(trow) * table_width;

  // this lane's query column in each of the wave's query tiles
  int qpos[AP_QT];
  bf16x8 qf[AP_QT][KS];
#pragma unroll
  for (int qt = 0; qt < AP_QT; ++qt) {
    const int rr = wave * (16 * AP_QT) + qt * 16 + col;
    const int ti = rr / group, hh = rr - ti * group;
    const bool valid = ti < ntok;
    qpos[qt] = valid ? pos0 + ti : -1;
    const uint16_t* qrow = q + (static_cast<size_t>(tok0 + (valid ? ti : 0)) * n_heads + kvh * group + hh) * HD;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (valid) {
        qf[qt][ks] = *reinterpret_cast<const bf16x8*>(qrow + ks * 32 + grp * 8);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) qf[qt][ks][i] = (__bf16)0.0f;
      }
    }
  }

  float m_run[AP_QT], l_run[AP_QT];
  floatx4 o[AP_QT][DT];
#pragma unroll
  for (int qt = 0; qt < AP_QT; ++qt) {
    m_run[qt] = -INFINITY;
    l_run[qt] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[qt][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  const float scale_log2 = scale * 1.44269504088896340736f;
  const int kv_last = pos0 + ntok - 1;
  const int k_lo = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
  for (int kb = (k_lo / AP_BK) * AP_BK; kb <= kv_last; kb += AP_BK) {
    __syncthreads();
    // stage 64 keys row-major and 64 values transposed
#pragma unroll
    for (int pass = 0; pass < AP_BK * CHUNKS / 256; ++pass) {
      const int idx = pass * 256 + tid;
      const int key = idx / CHUNKS, chunk = idx - key * CHUNKS;
      const int j = (kb + key < kv_last) ? kb + key : kv_last;  // past the end: repeat the last key
      const int phys = table[j / page_size] * page_size + j % page_size;
      const size_t src = (static_cast<size_t>(phys) * n_kv_heads + kvh) * HD + chunk * 8;
      const uint4 kvec = *reinterpret_cast<const uint4*>(k_cache + src);
      const uint4 vvec = *reinterpret_cast<const uint4*>(v_cache + src);
      *reinterpret_cast<uint4*>(&k_lds[key * KSTR + chunk * 8]) = kvec;
      const uint32_t vw[4] = {vvec.x, vvec.y, vvec.z, vvec.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v_lds[(chunk * 8 + 2 * i) * AP_VSTRIDE + key] = static_cast<uint16_t>(vw[i] & 0xffffu);
        v_lds[(chunk * 8 + 2 * i + 1) * AP_VSTRIDE + key] = static_cast<uint16_t>(vw[i] >> 16);
      }
    }
    __syncthreads();

    // transposed scores: rows = keys of a 16-key tile, columns = the query tile's rows
    floatx4 s[AP_QT][AP_BK / 16];
#pragma unroll
    for (int qt = 0; qt < AP_QT; ++qt)
#pragma unroll
      for (int kt = 0; kt < AP_BK / 16; ++kt) s[qt][kt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kt = 0; kt < AP_BK / 16; ++kt) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const bf16x8 kf = *reinterpret_cast<const bf16x8*>(&k_lds[(kt * 16 + col) * KSTR + ks * 32 + grp * 8]);
#pragma unroll
        for (int qt = 0; qt < AP_QT; ++qt)
          s[qt][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[qt][ks], s[qt][kt], 0, 0, 0);
      }
    }

    // mask, running softmax, and the probabilities as row operands of the value product.
    // Scores are scaled by scale*log2(e) so that the exponentials are single exp2
    // instructions; the running maximum is kept in the same units.
    bf16x8 pa[AP_QT][AP_BK / 32];
#pragma unroll
    for (int qt = 0; qt < AP_QT; ++qt) {
      const int qp = qpos[qt];
      const int lo = (window > 0) ? qp - window + 1 : 0;
      float tile_max = -INFINITY;
#pragma unroll
      for (int kt = 0; kt < AP_BK / 16; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int key = kb + kt * 16 + 4 * grp + r;
          const float v = (key <= qp && key >= lo) ? s[qt][kt][r] * scale_log2 : -INFINITY;
          s[qt][kt][r] = v;
          tile_max = fmaxf(tile_max, v);
        }
      tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, PYLON_WAVE));
      tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, PYLON_WAVE));
      const float m_new = fmaxf(m_run[qt], tile_max);
      const float m_use = (m_new == -INFINITY) ? 0.f : m_new;  // a row that has seen no key yet
      const float corr = __builtin_amdgcn_exp2f(m_run[qt] - m_use);
      float tile_sum = 0.f;
      float p[AP_BK / 16][4];
#pragma unroll
      for (int kt = 0; kt < AP_BK / 16; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          p[kt][r] = __builtin_amdgcn_exp2f(s[qt][kt][r] - m_use);
          tile_sum += p[kt][r];
        }
      tile_sum += __shfl_xor(tile_sum, 16, PYLON_WAVE);
      tile_sum += __shfl_xor(tile_sum, 32, PYLON_WAVE);
      l_run[qt] = l_run[qt] * corr + tile_sum;
      m_run[qt] = m_new;
#pragma unroll
      for (int kg = 0; kg < AP_BK / 32; ++kg) {
        uint4 packed;
        packed.x = pack_bf16(p[2 * kg][0], p[2 * kg][1]);
        packed.y = pack_bf16(p[2 * kg][2], p[2 * kg][3]);
        packed.z = pack_bf16(p[2 * kg + 1][0], p[2 * kg + 1][1]);
        packed.w = pack_bf16(p[2 * kg + 1][2], p[2 * kg + 1][3]);
        pa[qt][kg] = *reinterpret_cast<bf16x8*>(&packed);
      }
      // the accumulators of this lane belong to query rows 4*grp + r: fetch their factors
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float c = __shfl(corr, 4 * grp + r, PYLON_WAVE);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[qt][dt][r] *= c;
      }
    }

    // out += P * V; operand slot j of a lane is key 32*kg + 4*grp + j (j < 4) or
    // 32*kg + 16 + 4*grp + (j - 4), for P and V alike
#pragma unroll
    for (int kg = 0; kg < AP_BK / 32; ++kg) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const uint16_t* vrow = &v_lds[(dt * 16 + col) * AP_VSTRIDE + kg * 32 + 4 * grp];
        uint4 vv;
        vv.x = *reinterpret_cast<const uint32_t*>(vrow);
        vv.y = *reinterpret_cast<const uint32_t*>(vrow + 2);
        vv.z = *reinterpret_cast<const uint32_t*>(vrow + 16);
        vv.w = *reinterpret_cast<const uint32_t*>(vrow + 18);
        const bf16x8 vf = *reinterpret_cast<bf16x8*>(&vv);
#pragma unroll
        for (int qt = 0; qt < AP_QT; ++qt)
          o[qt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa[qt][kg], vf, o[qt][dt], 0, 0, 0);
      }
    }
  }

  // out = acc / sum; this lane holds rows 4*grp + r, element dt*16 + col
#pragma unroll
  for (int qt = 0; qt < AP_QT; ++qt) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float l = __shfl(l_run[qt], 4 * grp + r, PYLON_WAVE);
      const int rr = wave * (16 * AP_QT) + qt * 16 + 4 * grp + r;
      const int ti = rr / group, hh = rr - ti * group;
      if (ti < ntok) {
        const float inv = 1.0f / l;
        uint16_t* orow = out + (static_cast<size_t>(tok0 + ti) * n_heads + kvh * group + hh) * HD;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) orow[dt * 16 + col] = float_to_bf16_bits(o[qt][dt][r] * inv);
      }
    }
  }
}

// tiles: [n_tiles, 4] = (index of the tile's first token in q/out, its token count, its row of
// the block table, the position of its first token).  A tile holds consecutive tokens of one
// request, at most floor(64 / group) of them.
extern "C" int pylon_attention_prefill(void* out, const void* q, const void* k_cache, const void* v_cache,
                                       const int* block_table, int table_width, const int* tiles,
                                       int n_tiles, int n_heads, int n_kv_heads, int head_dim,
                                       int page_size, int window, float scale, hipStream_t stream) {
  PYLON_REQUIRE(n_tiles >= 0 && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
                "attention_prefill: %d query heads cannot be grouped over %d key/value heads", n_heads,
                n_kv_heads);
  PYLON_REQUIRE(n_heads / n_kv_heads <= AP_ROWS, "attention_prefill: at most %d query heads per key/value head",
                AP_ROWS);
  PYLON_REQUIRE(head_dim == 64 || head_dim == 128 || head_dim == 256,
                "attention_prefill: head_dim %d is not 64, 128 or 256", head_dim);
  PYLON_REQUIRE(page_size > 0 && table_width > 0 && window >= 0, "attention_prefill: bad page size, width or window");
  PYLON_REQUIRE(n_kv_heads <= 65535, "attention_prefill: too many key/value heads for one launch");
  if (n_tiles == 0) return 0;
  const int group = n_heads / n_kv_heads;
  dim3 grid(n_tiles, n_kv_heads), block(256);
#define GO(HD)                                                                                         \
  hipLaunchKernelGGL((attention_prefill_kernel<HD>), grid, block, 0, stream, (uint16_t*)out,           \
                     (const uint16_t*)q, (const uint16_t*)k_cache, (const uint16_t*)v_cache,           \
                     block_table, table_width, tiles, n_heads, n_kv_heads, group, page_size, window, scale)
  if (head_dim == 64)
    GO(64);
  else if (head_dim == 128)
    GO(128);
  else
    GO(256);
#undef GO
  PYLON_LAUNCHED("attention_prefill");
}
