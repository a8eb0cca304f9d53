// Paged attention on the matrix cores for the score rules and cache shapes the head-size-specialised
// kernels do not take (bfloat16): keys and values of different widths, values that are the first
// elements of the key rows themselves (a layer that caches one vector per token), a bias on the
// scores that is linear in the distance or read from a table by the distance, chunks of positions, a
// window (behind which the first `keep` tokens of a request may stay visible, at their true positions),
// sinks in the softmax's denominator (of score 0, or of a score per head).  Same arithmetic as ts_paged_attention_generic: scores, bias, masks and softmax in
// 32-bit; products of bfloat16 operands accumulated in 32-bit.
//
// A workgroup of four wavefronts owns 64 query rows and walks the keys they may see in tiles of 64:
//   * prompt portions: the rows are 64 consecutive tokens of one request and one query head (the
//     tile list comes from the host);
//   * single tokens: the rows are the query heads of one KV head for one request's token; the keys
//     are shared out over `splits` workgroups whose unnormalised sums ts_attention_tiles_combine
//     puts together.
// A tile of keys goes global memory -> registers -> LDS ([key][Dk], and the values as [Dv][key]: from
// the transposed value pages as they are, or turned while being staged when they lie in the key
// rows); the next tile's loads are in flight while this one is computed.  Per wavefront: S (16 rows
// x 64 keys) = Q K^T by v_mfma_f32_16x16x32_bf16, online softmax in the accumulator layout, P
// through LDS into the operand layout, O += P V.
//
// Sizes: Dk (up to 384; 448 with the values inside the key rows) and Dv (up to 256; 384) multiples of 8; pages of 8 tokens or more (a multiple of 8).
#include "common.hpp"

typedef __bf16 fa_bf16x8 __attribute__((ext_vector_type(8)));
typedef float fa_f32x4 __attribute__((ext_vector_type(4)));

#define FA_ROWS 64
#define FA_KEYS 64
#define FA_THREADS 256
#define FA_PAD 8  // elements of padding behind an LDS row

struct FaRule {
  float scale;
  float softcap;
  float sinks;
  int window;
  int chunk;
  int keep;  // the keys 0 .. keep - 1 are seen also below the window's lower bound
};

// Sum and maximum over the 16 lanes that hold one row of an accumulator tile (a row of lanes for
// the data-parallel moves): every lane returns its row's result.
__device__ __forceinline__ float row16_sum(float v) {
  v += lanes_moved<0xB1, 0xF>(0.f, v);   // quad_perm [1,0,3,2]
  v += lanes_moved<0x4E, 0xF>(0.f, v);   // quad_perm [2,3,0,1]
  v += lanes_moved<0x141, 0xF>(0.f, v);  // row_half_mirror
  v += lanes_moved<0x140, 0xF>(0.f, v);  // row_mirror
  return v;
}

__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, lanes_moved<0xB1, 0xF>(v, v));
  v = fmaxf(v, lanes_moved<0x4E, 0xF>(v, v));
  v = fmaxf(v, lanes_moved<0x141, 0xF>(v, v));
  v = fmaxf(v, lanes_moved<0x140, 0xF>(v, v));
  return v;
}

__device__ __forceinline__ int fa_lowest(int p, int window, int chunk) {
  int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  if (chunk > 0) lo = max(lo, (p / chunk) * chunk);
  return lo;
}

// KD: 32-element pieces of a key row (Dk rounded up), VD: 16-element pieces of a value row.
// SINGLE: the single-token layout.  VALUES_IN_KEYS: no value pages.
template <int KD, int VD, bool SINGLE, bool VALUES_IN_KEYS>
__global__ void __launch_bounds__(FA_THREADS, (KD <= 4 ? 2 : 1))  // small tiles: two workgroups a compute unit
attention_tiles_kernel(uint16_t* __restrict__ out, float* __restrict__ partial_o, float* __restrict__ partial_ml,
                       const uint16_t* __restrict__ q, long q_stride, const uint16_t* __restrict__ k_pages,
                       const uint16_t* __restrict__ v_pages, const int* __restrict__ block_table, int table_width,
                       const int* __restrict__ query_start_loc, const int* __restrict__ context_lens,
                       const int* __restrict__ tiles, int first_seq, int heads, int kv_heads, int dk, int dv,
                       int block_size, const float* __restrict__ slopes, FaRule rule, int splits,
                       const float* __restrict__ sink_scores, const float* __restrict__ distance_bias, int bias_len) {
  extern __shared__ __attribute__((aligned(16))) uint16_t fa_lds[];
  constexpr int K_ROW = KD * 32 + FA_PAD;       // elements of a staged key row
  constexpr int V_ROW = FA_KEYS + FA_PAD;       // elements of a staged value column (64 keys)
  constexpr int P_ROW = FA_KEYS + FA_PAD;
  uint16_t* ks = fa_lds;                        // [FA_KEYS][K_ROW]
  uint16_t* vs = ks + FA_KEYS * K_ROW;          // [VD * 16][V_ROW]
  uint16_t* ps = vs + VD * 16 * V_ROW;          // [4 wavefronts][16][P_ROW]

  const int tid = threadIdx.x;
  const int wave = tid / TS_WAVE, lane = tid % TS_WAVE;
  const int r16 = lane % 16, group = lane / 16;
  const int group_heads = heads / kv_heads;

  // Which rows: (token row of the step, head, position) of row r; rows beyond the tile are idle.
  int seq, kvh, tile_first_row = 0, tile_rows, head_first = 0;
  if (SINGLE) {
    seq = first_seq + blockIdx.x;
    const int head_tiles = (group_heads + FA_ROWS - 1) / FA_ROWS;
    kvh = blockIdx.y / head_tiles;
    head_first = kvh * group_heads + (blockIdx.y % head_tiles) * FA_ROWS;
    tile_rows = min(FA_ROWS, kvh * group_heads + group_heads - head_first);
    tile_first_row = query_start_loc[seq];
  } else {
    // Heads are the fast index of the grid, so workgroups start in the order of the tile list: the
    // host puts the tiles with the most keys first.
    seq = tiles[2 * blockIdx.y];
    tile_first_row = tiles[2 * blockIdx.y + 1];
    tile_rows = min(FA_ROWS, query_start_loc[seq + 1] - tile_first_row);
    head_first = blockIdx.x;
    kvh = head_first / group_heads;
  }
  const int context = context_lens[seq];
  const int first_position = context - (query_start_loc[seq + 1] - query_start_loc[seq]);
  auto row_token = [&](int r) { return SINGLE ? tile_first_row : tile_first_row + r; };
  auto row_head = [&](int r) { return SINGLE ? head_first + r : head_first; };
  auto row_position = [&](int r) {
    return SINGLE ? first_position : first_position + (tile_first_row - query_start_loc[seq]) + r;
  };
  const int* table = block_table + (size_t)seq * table_width;

  // The keys this workgroup walks: from the lowest any row sees to the highest, in aligned tiles;
  // of a shared-out walk its share of the tiles.
  const int p_first = row_position(0), p_last = row_position(tile_rows - 1);
  const int key_lo = fa_lowest(p_first, rule.window, rule.chunk);
  // The walk: the tiles of the kept first keys that lie below the window's tiles, then the window's.
  // Walk index w is tile w below `kept_tiles`, and tile w + window_shift from there on.
  const int window_begin = key_lo / FA_KEYS;
  const int kept_tiles = min((rule.keep + FA_KEYS - 1) / FA_KEYS, window_begin);
  const int window_shift = window_begin - kept_tiles;
  int tile_begin = 0, tile_end = kept_tiles + p_last / FA_KEYS + 1 - window_begin;
  if (splits > 1) {
    const int per = (tile_end - tile_begin + splits - 1) / splits;
    tile_begin = tile_begin + (int)blockIdx.z * per;
    tile_end = min(tile_end, tile_begin + per);
  }
  auto tile_of = [&](int w) { return w < kept_tiles ? w : w + window_shift; };
  // Keys from this one on (rounded up to 8) up to key_lo may lie in pages that were given back.
  const int keep_end = (rule.keep + 7) & ~7;

  // The wavefront's queries as first operands: row wave * 16 + r16, elements 32 kd + 8 group ..
  ts_u32x4 qf[KD];
  {
    const int r = wave * 16 + r16;
    const bool live = r < tile_rows;
    const uint16_t* src = q + (size_t)row_token(live ? r : 0) * q_stride + (size_t)row_head(live ? r : 0) * dk;
#pragma unroll
    for (int kd = 0; kd < KD; ++kd) {
      const int at = 32 * kd + 8 * group;
      qf[kd] = (live && at < dk) ? *reinterpret_cast<const ts_u32x4*>(src + at) : ts_u32x4{0u, 0u, 0u, 0u};
    }
  }
  // Per accumulator row i of this lane (row wave * 16 + 4 group + i): position, lowest key, slope.
  int pos[4], low[4];
  float slope[4], sink_at[4];
  const float* bias_row[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = wave * 16 + 4 * group + i;
    const bool live = r < tile_rows;
    pos[i] = live ? row_position(r) : -1;  // an idle row sees nothing
    low[i] = live ? fa_lowest(pos[i], rule.window, rule.chunk) : 0;
    slope[i] = (slopes && live) ? slopes[row_head(r)] : 0.f;
    // The row's line of the bias table (read by distance); an idle row reads head 0's and is masked.
    bias_row[i] = distance_bias ? distance_bias + (size_t)(live ? row_head(r) : 0) * bias_len : nullptr;
    sink_at[i] = (sink_scores && live) ? sink_scores[row_head(r)] : 0.f;
  }
  // (Key rows that hold their values have no variant with a bias: the launch refuses it.)
  const bool biased = !VALUES_IN_KEYS && distance_bias != nullptr;
  fa_f32x4 o[VD];
#pragma unroll
  for (int vt = 0; vt < VD; ++vt) o[vt] = fa_f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run[4], l_run[4];
  // A sink is a key of score 0 that is always there; where the keys are shared out, the combining
  // kernel counts it, once.
  const bool own_sinks = rule.sinks > 0.f && splits == 1;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    m_run[i] = own_sinks ? sink_at[i] : -INFINITY;
    l_run[i] = own_sinks ? rule.sinks : 0.f;
  }

  // What this thread fetches of a tile: 16-byte pieces (key, 8 elements) of the keys, and of paged
  // values pieces (value element, 8 keys); which pieces is the same for every tile.  Key rows whose
  // first elements are also the values are turned into the value tile's columns while they are
  // staged, two bytes at a time: there a wavefront's lanes take the 64 keys of one 8-element piece,
  // so that its LDS writes fall into different banks; otherwise consecutive lanes take consecutive
  // pieces of a row (whole cache lines).
  const int k_pieces_row = dk / 8;
  const int k_pieces = FA_KEYS * k_pieces_row;
  constexpr int K_MINE = (FA_KEYS * KD * 4 + FA_THREADS - 1) / FA_THREADS;
  constexpr int V_MINE = (VD * 16 * (FA_KEYS / 8) + FA_THREADS - 1) / FA_THREADS;
  const int v_pieces = dv * (FA_KEYS / 8);
  const int block_mask = block_size - 1, block_shift = __builtin_ctz(block_size);  // pages hold a power of two
  int k_key[K_MINE], k_at[K_MINE];
#pragma unroll
  for (int j = 0; j < K_MINE; ++j) {
    const int piece = tid + j * FA_THREADS;
    k_key[j] = VALUES_IN_KEYS ? piece % FA_KEYS : piece / k_pieces_row;
    k_at[j] = 8 * (VALUES_IN_KEYS ? piece / FA_KEYS : piece % k_pieces_row);
    if (piece >= k_pieces) k_key[j] = -1;
  }
  ts_u32x4 k_reg[K_MINE];
  ts_u32x4 v_reg[VALUES_IN_KEYS ? 1 : V_MINE];
  const int last_key = context - 1;
  auto fetch = [&](int tile) __attribute__((always_inline)) {
    const int key0 = tile * FA_KEYS;
#pragma unroll
    for (int j = 0; j < K_MINE; ++j) {
      // Outside key_lo .. last: a live key again (its page may have been given back, or never taken); masked later.
      int key = min(key0 + max(k_key[j], 0), last_key);
      if (key >= keep_end) key = max(key, key_lo);
      const int page = table[key >> block_shift];
      const uint16_t* src = k_pages + ((((size_t)page * kv_heads + kvh) << block_shift) + (key & block_mask)) * dk + k_at[j];
      k_reg[j] = k_key[j] >= 0 ? *reinterpret_cast<const ts_u32x4*>(src) : ts_u32x4{0u, 0u, 0u, 0u};
    }
    if (!VALUES_IN_KEYS) {
#pragma unroll
      for (int j = 0; j < V_MINE; ++j) {
        const int piece = tid + j * FA_THREADS;
        const int d = piece / (FA_KEYS / 8);
        int key = min(key0 + 8 * (piece % (FA_KEYS / 8)), last_key & ~7);  // eight keys of one page
        if (key >= keep_end) key = max(key, key_lo & ~7);
        const int page = table[key >> block_shift];
        const uint16_t* src = v_pages + ((((size_t)page * kv_heads + kvh) * dv + d) << block_shift) + (key & block_mask);
        v_reg[j] = piece < v_pieces ? *reinterpret_cast<const ts_u32x4*>(src) : ts_u32x4{0u, 0u, 0u, 0u};
      }
    }
  };
  auto stage = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < K_MINE; ++j) {
      if (k_key[j] >= 0) {
        const int key = k_key[j], at = k_at[j];
        *reinterpret_cast<ts_u32x4*>(ks + key * K_ROW + at) = k_reg[j];
        if (VALUES_IN_KEYS && at < dv) {
          // The row's first Dv elements are the key's value: turned into the value tile's columns.
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            vs[(at + 2 * e) * V_ROW + key] = (uint16_t)(k_reg[j][e] & 0xffffu);
            vs[(at + 2 * e + 1) * V_ROW + key] = (uint16_t)(k_reg[j][e] >> 16);
          }
        }
      }
    }
    if (!VALUES_IN_KEYS) {
#pragma unroll
      for (int j = 0; j < V_MINE; ++j) {
        const int piece = tid + j * FA_THREADS;
        if (piece < v_pieces)
          *reinterpret_cast<ts_u32x4*>(vs + (piece / (FA_KEYS / 8)) * V_ROW + 8 * (piece % (FA_KEYS / 8))) = v_reg[j];
      }
    }
  };
  // What the sizes leave unused of the staged tiles is read as operands all the same: zero, once
  // (the key rows' elements from Dk on, the value rows from Dv on).
  for (int i = tid; i < FA_KEYS * (K_ROW - dk); i += FA_THREADS) ks[(i / (K_ROW - dk)) * K_ROW + dk + i % (K_ROW - dk)] = 0;
  for (int i = tid + dv * V_ROW; i < VD * 16 * V_ROW; i += FA_THREADS) vs[i] = 0;
  __syncthreads();

  uint16_t* my_p = ps + wave * 16 * P_ROW;
  if (tile_begin < tile_end) fetch(tile_of(tile_begin));
  for (int walk = tile_begin; walk < tile_end; ++walk) {
    __syncthreads();  // everyone has read the tile before
    stage();
    __syncthreads();
    if (walk + 1 < tile_end) fetch(tile_of(walk + 1));  // in flight while this tile is computed
    const int key0 = tile_of(walk) * FA_KEYS;
    // The biases of this lane's 16 scores, asked for in one stretch ahead of the first product, so
    // that they arrive while it runs (asked for where they are added, each is waited for on its own).
    float bias_of[4][4];
    if (biased) {
#pragma unroll
      for (int ct = 0; ct < 4; ++ct) {
        const int key = key0 + 16 * ct + r16;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const bool seen = (key >= low[i] || key < rule.keep) && key <= pos[i];
          bias_of[ct][i] = bias_row[i][seen ? min(pos[i] - key, bias_len - 1) : 0];
        }
      }
    }
    // S = Q K^T: four tiles of 16 keys.
    fa_f32x4 s[4];
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) s[ct] = fa_f32x4{0.f, 0.f, 0.f, 0.f};
    // (Every piece of the size class is multiplied, also those past Dk, which hold zeros: a test
    // per piece would cut this stretch into pieces that each wait for their own LDS reads.)
#pragma unroll
    for (int kd = 0; kd < KD; ++kd) {
#pragma unroll
      for (int ct = 0; ct < 4; ++ct) {
        const ts_u32x4 kf = *reinterpret_cast<const ts_u32x4*>(ks + (16 * ct + r16) * K_ROW + 32 * kd + 8 * group);
        s[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(fa_bf16x8, qf[kd]),
                                                        __builtin_bit_cast(fa_bf16x8, kf), s[ct], 0, 0, 0);
      }
    }
    if (rule.softcap > 0.f) {
#pragma unroll
      for (int ct = 0; ct < 4; ++ct)
#pragma unroll
        for (int i = 0; i < 4; ++i) s[ct][i] = rule.softcap / rule.scale * tanhf(s[ct][i] * rule.scale / rule.softcap);
    }
    // Scores of this lane: row 4 group + i, key key0 + 16 ct + r16.
    float tile_max[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) tile_max[i] = -INFINITY;
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) {
      const int key = key0 + 16 * ct + r16;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = fmaf(slope[i], (float)(key - pos[i]), s[ct][i] * rule.scale);
        const bool seen = (key >= low[i] || key < rule.keep) && key <= pos[i];
        if (biased) v += bias_of[ct][i];
        v = seen ? v : -INFINITY;
        s[ct][i] = v;
        tile_max[i] = fmaxf(tile_max[i], v);
      }
    }
    float alpha[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float v = row16_max(tile_max[i]);
      const float m_new = fmaxf(m_run[i], v);
      // A row that has seen nothing yet keeps a zero sum: exp(-inf - -inf) must not be formed.
      alpha[i] = m_new == -INFINITY ? 1.f : expf(m_run[i] - m_new);
      m_run[i] = m_new;
    }
    float sum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = s[ct][i] == -INFINITY ? 0.f : expf(s[ct][i] - m_run[i]);
        // The probability as the second product sees it: rounded; the denominator counts the same value.
        const bf16_t rounded = from_float<bf16_t>(p);
        sum[i] += to_float(rounded);
        my_p[(4 * group + i) * P_ROW + 16 * ct + r16] = rounded.bits;
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      l_run[i] = l_run[i] * alpha[i] + row16_sum(sum[i]);
    }
#pragma unroll
    for (int vt = 0; vt < VD; ++vt)
#pragma unroll
      for (int i = 0; i < 4; ++i) o[vt][i] *= alpha[i];
    __builtin_amdgcn_s_waitcnt(0xc07f);  // the wavefront's own LDS writes of P have landed (lgkmcnt 0)
    __builtin_amdgcn_wave_barrier();
    // O += P V over the tile's 64 keys.
#pragma unroll
    for (int kk = 0; kk < FA_KEYS / 32; ++kk) {
      const ts_u32x4 pf = *reinterpret_cast<const ts_u32x4*>(my_p + r16 * P_ROW + 32 * kk + 8 * group);
#pragma unroll
      for (int vt = 0; vt < VD; ++vt) {
        const ts_u32x4 vf = *reinterpret_cast<const ts_u32x4*>(vs + (16 * vt + r16) * V_ROW + 32 * kk + 8 * group);
        o[vt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(fa_bf16x8, pf),
                                                        __builtin_bit_cast(fa_bf16x8, vf), o[vt], 0, 0, 0);
      }
    }
  }

  // o[vt][i]: row 4 group + i, value element 16 vt + r16.
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = wave * 16 + 4 * group + i;
    if (r >= tile_rows) continue;
    if (splits == 1) {
      const float inv = l_run[i] > 0.f ? 1.f / l_run[i] : 0.f;
      uint16_t* dst = out + ((size_t)row_token(r) * heads + row_head(r)) * dv;
#pragma unroll
      for (int vt = 0; vt < VD; ++vt)
        if (16 * vt + r16 < dv) dst[16 * vt + r16] = from_float<bf16_t>(o[vt][i] * inv).bits;
    } else {
      // Unnormalised sums with the maximum they were taken against: [request, head, split].
      const size_t slot = ((size_t)blockIdx.x * heads + row_head(r)) * splits + blockIdx.z;
      float* dst = partial_o + slot * dv;
#pragma unroll
      for (int vt = 0; vt < VD; ++vt)
        if (16 * vt + r16 < dv) dst[16 * vt + r16] = o[vt][i];
      if (r16 == 0) {
        partial_ml[2 * slot] = m_run[i];
        partial_ml[2 * slot + 1] = l_run[i];
      }
    }
  }
}

// out[request's token, head, :] from the shares of its keys: one block per (request, head).  The
// shares' maxima and sums are fetched side by side (one thread each) and turned into weights in LDS.
#define FA_MAX_SPLITS 64
__global__ void __launch_bounds__(128)
attention_tiles_combine_kernel(uint16_t* __restrict__ out, const float* __restrict__ partial_o,
                               const float* __restrict__ partial_ml, const int* __restrict__ query_start_loc,
                               int first_seq, int heads, int dv, int splits, float sinks,
                               const float* __restrict__ sink_scores) {
  __shared__ float weight[FA_MAX_SPLITS];
  __shared__ float scratch[16];
  const int item = blockIdx.x, h = blockIdx.y;
  const size_t base = ((size_t)item * heads + h) * splits;
  const int sp = threadIdx.x;
  const float ms = sp < splits ? partial_ml[2 * (base + sp)] : -INFINITY;
  const float ls = sp < splits ? partial_ml[2 * (base + sp) + 1] : 0.f;
  const float sink_at = sink_scores ? sink_scores[h] : 0.f;
  const float m = fmaxf(block_max(ms, scratch), sinks > 0.f ? sink_at : -INFINITY);
  const float w = ms == -INFINITY ? 0.f : expf(ms - m);
  if (sp < splits) weight[sp] = w;
  const float l = block_sum(ls * w, scratch) + (sinks > 0.f ? sinks * expf(sink_at - m) : 0.f);  // (its barriers publish the weights)
  const float inv = l > 0.f ? 1.f / l : 0.f;
  const int row = query_start_loc[first_seq + item];
  for (int d = threadIdx.x; d < dv; d += blockDim.x) {
    float acc = 0.f;
    for (int first = 0; first < splits; first += 8) {  // eight loads in flight
      float v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = partial_o[(base + min(first + j, splits - 1)) * dv + d];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (first + j < splits) acc = fmaf(v[j], weight[first + j], acc);
    }
    out[((size_t)row * heads + h) * dv + d] = from_float<bf16_t>(acc * inv).bits;
  }
}

template <int KD, int VD>
static int tiles_launch(bool single, bool values_in_keys, dim3 grid, hipStream_t stream, uint16_t* out, float* partial_o,
                        float* partial_ml, const uint16_t* q, long q_stride, const uint16_t* k_pages,
                        const uint16_t* v_pages, const int* block_table, int table_width, const int* query_start_loc,
                        const int* context_lens, const int* tiles, int first_seq, int heads, int kv_heads, int dk, int dv,
                        int block_size, const float* slopes, FaRule rule, int splits, const float* sink_scores,
                        const float* distance_bias, int bias_len) {
  constexpr size_t lds = (size_t)(FA_KEYS * (KD * 32 + FA_PAD) + VD * 16 * (FA_KEYS + FA_PAD) + 4 * 16 * (FA_KEYS + FA_PAD)) * sizeof(uint16_t);
  static_assert(lds <= 160 * 1024, "the staged tiles must fit in LDS");
#define FA_GO(SINGLE, INKEYS)                                                                                          \
  do {                                                                                                                 \
    static bool raised = false;                                                                                        \
    if (!raised) {                                                                                                     \
      if (hipFuncSetAttribute((const void*)attention_tiles_kernel<KD, VD, SINGLE, INKEYS>,                             \
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)                     \
        return TS_ERR_LAUNCH;                                                                                          \
      raised = true;                                                                                                   \
    }                                                                                                                  \
    hipLaunchKernelGGL((attention_tiles_kernel<KD, VD, SINGLE, INKEYS>), grid, dim3(FA_THREADS), lds, stream, out,     \
                       partial_o, partial_ml, q, q_stride, k_pages, v_pages, block_table, table_width, query_start_loc, \
                       context_lens, tiles, first_seq, heads, kv_heads, dk, dv, block_size, slopes, rule, splits,      \
                       sink_scores, distance_bias, bias_len);                                                          \
  } while (0)
  if (single && values_in_keys) FA_GO(true, true);
  else if (single) FA_GO(true, false);
  else if (values_in_keys) FA_GO(false, true);
  else FA_GO(false, false);
#undef FA_GO
  return ts_launch_status();
}

// mode 0: prompt portions, `items` tiles (pairs: request, first row), each for every head;
// mode 1: `items` requests of one token each from `first_seq` on, their keys shared out over `splits`.
// out [T, heads, Dv] bfloat16.  v_pages null: the values are the keys' first Dv elements.
// sink_scores [heads] (32-bit) or null: the score of the sinks, 0 without; distance_bias [heads, bias_len]
// (32-bit) or null: the score of a key at distance n gets distance_bias[h][min(n, bias_len - 1)] added.
extern "C" int ts_attention_tiles(void* out, void* partial_o, void* partial_ml, const void* q, long q_stride,
                                  const void* k_pages, const void* v_pages, const int* block_table, int table_width,
                                  const int* query_start_loc, const int* context_lens, const int* tiles, int items,
                                  int first_seq, int heads, int kv_heads, int dk, int dv, int block_size, float scale,
                                  float softcap, int window, int chunk, float sinks, const float* slopes, int mode,
                                  int splits, const float* sink_scores, const float* distance_bias, int bias_len,
                                  int keep_first, hipStream_t stream) {
  if (items == 0) return TS_OK;
  if (keep_first < 0 || (keep_first > 0 && chunk > 0)) return TS_ERR_ARG;
  if (!out || !q || !k_pages || !block_table || !query_start_loc || !context_lens) return TS_ERR_ARG;
  if (mode == 0 && (!tiles || splits != 1)) return TS_ERR_ARG;
  if (mode == 1 && splits > 1 && (!partial_o || !partial_ml)) return TS_ERR_ARG;
  if (mode < 0 || mode > 1 || splits < 1 || splits > FA_MAX_SPLITS) return TS_ERR_ARG;
  if ((sink_scores && !(sinks > 0.f)) || (distance_bias && (bias_len < 1 || !v_pages))) return TS_ERR_ARG;
  if (heads < 1 || kv_heads < 1 || heads % kv_heads != 0 || heads > 65535) return TS_ERR_SHAPE;
  if (dk < 8 || dk > 448 || dk % 8 != 0 || dv < 8 || dv > 384 || dv % 8 != 0 || block_size < 8 || block_size % 8 != 0)
    return TS_ERR_SHAPE;
  if (!v_pages && dv > dk) return TS_ERR_SHAPE;
  if (block_size & (block_size - 1)) return TS_ERR_SHAPE;  // slots are taken apart by shift and mask
  if (v_pages && (dk > 384 || dv > 256)) return TS_ERR_SHAPE;  // the widest tiles are built for values inside the key rows
  if ((((uintptr_t)q | (uintptr_t)k_pages | (uintptr_t)v_pages) & 15) != 0 || (q_stride % 8) != 0) return TS_ERR_ARG;
  const FaRule rule = {scale, softcap, sinks, window, chunk, keep_first};
  const int group_heads = heads / kv_heads;
  if (mode == 0 && items > 65535) return TS_ERR_SHAPE;
  const dim3 grid = mode == 0 ? dim3(heads, items, 1) : dim3(items, kv_heads * ((group_heads + FA_ROWS - 1) / FA_ROWS), splits);
  const bool single = mode == 1, in_keys = v_pages == nullptr;
  const int kd = (dk + 31) / 32, vd = (dv + 15) / 16;
#define FA_SIZE(KD, VD)                                                                                                 \
  return tiles_launch<KD, VD>(single, in_keys, grid, stream, (uint16_t*)out, (float*)partial_o, (float*)partial_ml,     \
                              (const uint16_t*)q, q_stride, (const uint16_t*)k_pages, (const uint16_t*)v_pages,         \
                              block_table, table_width, query_start_loc, context_lens, tiles, first_seq, heads, kv_heads, \
                              dk, dv, block_size, slopes, rule, splits, sink_scores, distance_bias, bias_len)
  if (kd <= 2 && vd <= 4) FA_SIZE(2, 4);
  if (kd <= 4 && vd <= 8) FA_SIZE(4, 8);
  if (kd <= 4 && vd <= 16) FA_SIZE(4, 16);
  if (kd <= 8 && vd <= 8) FA_SIZE(8, 8);
  if (kd <= 8 && vd <= 16) FA_SIZE(8, 16);
  if (kd <= 10 && vd <= 16) FA_SIZE(10, 16);
  if (kd <= 12 && vd <= 16) FA_SIZE(12, 16);
  if (kd <= 14 && vd <= 24) FA_SIZE(14, 24);
#undef FA_SIZE
  return TS_ERR_SHAPE;
}

extern "C" int ts_attention_tiles_combine(void* out, const void* partial_o, const void* partial_ml,
                                          const int* query_start_loc, int items, int first_seq, int heads, int dv,
                                          int splits, float sinks, const float* sink_scores, hipStream_t stream) {
  if (items == 0) return TS_OK;
  if (!out || !partial_o || !partial_ml || !query_start_loc || splits < 1 || splits > FA_MAX_SPLITS || heads < 1 || heads > 65535 || dv < 1)
    return TS_ERR_ARG;
  hipLaunchKernelGGL(attention_tiles_combine_kernel, dim3(items, heads), dim3(128), 0, stream, (uint16_t*)out,
                     (const float*)partial_o, (const float*)partial_ml, query_start_loc, first_seq, heads, dv, splits, sinks, sink_scores);
  return ts_launch_status();
}
