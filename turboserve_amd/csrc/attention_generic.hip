// Paged attention for any mix of query lengths, in the storage type's own precision for loads
// and 32-bit everywhere else (scores, softmax state, accumulators).
//
// One wavefront per (token, query head).  The token at absolute position p of request s sees
// the keys lo..p of that request, lo = max(0, p - window + 1) for a windowed layer and 0
// otherwise (src/turboserve/engine/model/attention.py:139-148: keys <= ctx - q_len + j; the
// window bound is this engine's), and with keep_first > 0 also the keys 0 .. keep_first - 1 that lie
// below lo (the first tokens of a request stay visible behind a window, at their true positions); with chunk > 0 also lo >= (p / chunk) * chunk: a token sees its
// own chunk of positions only, chunks counted from position 0 of the request.  sinks > 0 adds that
// many keys of score 0 without a value to the softmax's denominator; with sink_scores [Hq] their score
// is the head's entry instead of 0 (it is not scaled and gets no bias).  distance_bias [Hq, L] (32-bit)
// adds distance_bias[h][min(p - key, L - 1)] to the score of a key, after scale and cap.  Without value pages the
// values are the first vdim elements of the keys themselves (a mixer that caches one vector per
// token).  Keys and values are read through the request's block table
// from key pages [NB, Hkv, BS, D] and transposed value pages [NB, Hkv, Dv, BS] (values may be wider
// or narrower than keys); with softcap c > 0 a scaled score s becomes c * tanh(s / c) before the
// bias and the softmax; KV head j serves
// query heads j*G .. j*G+G-1
// (attention.py:196-199).  Online softmax over tiles of 64 keys, as the reference's decode
// kernel does over blocks (src/turboserve/engine/model/triton_attention.py:127-166).
//
// This is the kernel of the true 32-bit path and the one every faster kernel is checked
// against: its result for a token is a function of (p, lo, the request's keys) only, so it is
// bitwise independent of how the request was cut into steps and of the batch around it.
#include "common.hpp"

#define ATTN_MAX_DIM 1024
#define ATTN_TILE 64

template <typename T>
__global__ void __launch_bounds__(64)
paged_attention_generic_kernel(T* __restrict__ out, const T* __restrict__ q, long q_stride,
                               const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                               const int* __restrict__ block_table, int table_width,
                               const int* __restrict__ token_seq, const int* __restrict__ positions,
                               int heads, int kv_heads, int dim, int vdim, int block_size, float scale,
                               float softcap, int window, const float* __restrict__ slopes, int chunk, float sinks,
                               const float* __restrict__ sink_scores, const float* __restrict__ distance_bias,
                               int bias_len, int keep_first) {
  __shared__ float qs[ATTN_MAX_DIM];
  __shared__ float ps[ATTN_TILE];
  __shared__ long long rows[ATTN_TILE];  // per key of the tile: offset of its value column

  const int t = blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x;
  const int kvh = h / (heads / kv_heads);
  const int seq = token_seq[t];
  const int p = positions[t];
  int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  if (chunk > 0 && (p / chunk) * chunk > lo) lo = (p / chunk) * chunk;
  // Values in pages of their own (transposed: a column per key) or inside the key rows.
  const T* __restrict__ v_src = v_pages ? v_pages : k_pages;
  const long long v_step = v_pages ? block_size : 1;
  const int* table = block_table + (size_t)seq * table_width;
  // A position encoding may bias the scores by the distance: + slope[h] * (key - p), in 32-bit.
  const float slope = slopes ? slopes[h] : 0.f;
  const float* bias_row = distance_bias ? distance_bias + (size_t)h * bias_len : nullptr;

  const T* qrow = q + (size_t)t * q_stride + (size_t)h * dim;
  for (int d = lane; d < dim; d += ATTN_TILE) qs[d] = to_float(qrow[d]) * scale;
  __syncthreads();

  constexpr int CHUNKS = ATTN_MAX_DIM / ATTN_TILE;
  float acc[CHUNKS];
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) acc[c] = 0.f;
  // A sink is a key of score 0 that is always there: the running maximum starts at its score.
  float m_run = sinks > 0.f ? (sink_scores ? sink_scores[h] : 0.f) : -INFINITY;
  float l_run = sinks > 0.f ? sinks : 0.f;

  // Two stretches of keys: the kept first ones below the window, then lo .. p.
  const int kept = min(keep_first, lo);
  for (int stretch = kept > 0 ? 0 : 1; stretch < 2; ++stretch) {
  const int first = stretch == 0 ? 0 : lo, last = stretch == 0 ? kept - 1 : p;
  for (int base = first; base <= last; base += ATTN_TILE) {
    const int key = base + lane;
    const bool valid = key <= last;
    float score = -INFINITY;
    long long row = 0;
    if (valid) {
      const int blk = table[key / block_size];
      const long long head_base = ((long long)blk * kv_heads + kvh) * block_size * dim;
      row = v_pages ? ((long long)blk * kv_heads + kvh) * block_size * vdim + (key % block_size)
                    : head_base + (long long)(key % block_size) * dim;
      const T* krow = k_pages + head_base + (long long)(key % block_size) * dim;
      float s = 0.f;
      for (int d = 0; d < dim; ++d) s = fmaf(qs[d], to_float(krow[d]), s);
      if (softcap > 0.f) s = softcap * tanhf(s / softcap);
      score = slopes ? fmaf(slope, (float)(key - p), s) : s;
      if (bias_row) score += bias_row[min(p - key, bias_len - 1)];
    }
    const float m_new = fmaxf(m_run, wave_max(score));
    const float alpha = expf(m_run - m_new);  // 0 on the first tile (m_run = -inf, m_new finite)
    const float prob = valid ? expf(score - m_new) : 0.f;
    l_run = l_run * alpha + wave_sum(prob);
    m_run = m_new;
    __syncthreads();  // the previous tile's readers are done with ps / rows
    ps[lane] = prob;
    rows[lane] = row;
    __syncthreads();
    const int count = (last - base + 1 < ATTN_TILE) ? last - base + 1 : ATTN_TILE;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      const int d = lane + c * ATTN_TILE;
      if (d < vdim) {
        float a = acc[c] * alpha;
        for (int j = 0; j < count; ++j)
          a = fmaf(ps[j], to_float(v_src[rows[j] + (long long)d * v_step]), a);
        acc[c] = a;
      }
    }
  }
  }

  T* orow = out + ((size_t)t * heads + h) * vdim;
  const float inv = 1.f / l_run;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int d = lane + c * ATTN_TILE;
    if (d < vdim) orow[d] = from_float<T>(acc[c] * inv);
  }
}

// out [T, Hq, Dv] contiguous; q rows are q_stride elements apart (the fused projection output).
// slopes [Hq] (32-bit) or null: the score of key j for the query at position p gets
// slopes[h] * (j - p) added.  v_pages null: the values are the keys' first vdim elements.
// sink_scores [Hq] (32-bit) or null; distance_bias [Hq, bias_len] (32-bit) or null.
extern "C" int ts_paged_attention_generic(void* out, const void* q, long q_stride,
                                          const void* k_pages, const void* v_pages,
                                          const int* block_table, int table_width,
                                          const int* token_seq, const int* positions, int tokens,
                                          int heads, int kv_heads, int dim, int vdim, int block_size,
                                          float scale, float softcap, int window, const float* slopes, int chunk,
                                          float sinks, const float* sink_scores, const float* distance_bias,
                                          int bias_len, int keep_first, int dtype, hipStream_t stream) {
  if (tokens == 0) return TS_OK;
  if (keep_first < 0 || (keep_first > 0 && chunk > 0)) return TS_ERR_ARG;
  if (!out || !q || !k_pages || !block_table || !token_seq || !positions) return TS_ERR_ARG;
  if (chunk < 0 || !(sinks >= 0.f) || (!v_pages && vdim > dim)) return TS_ERR_ARG;
  if ((sink_scores && !(sinks > 0.f)) || (distance_bias && bias_len < 1)) return TS_ERR_ARG;
  if (heads < 1 || kv_heads < 1 || heads % kv_heads != 0 || heads > 65535) return TS_ERR_SHAPE;
  if (dim < 1 || dim > ATTN_MAX_DIM || vdim < 1 || vdim > ATTN_MAX_DIM || block_size < 1 || table_width < 1)
    return TS_ERR_SHAPE;
  dim3 grid(tokens, heads), block(ATTN_TILE);
  if (dtype == TS_F32)
    hipLaunchKernelGGL(paged_attention_generic_kernel<float>, grid, block, 0, stream, (float*)out, (const float*)q, q_stride, (const float*)k_pages, (const float*)v_pages, block_table, table_width, token_seq, positions, heads, kv_heads, dim, vdim, block_size, scale, softcap, window, slopes, chunk, sinks, sink_scores, distance_bias, bias_len, keep_first);
  else if (dtype == TS_BF16)
    hipLaunchKernelGGL(paged_attention_generic_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)out, (const bf16_t*)q, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, block_table, table_width, token_seq, positions, heads, kv_heads, dim, vdim, block_size, scale, softcap, window, slopes, chunk, sinks, sink_scores, distance_bias, bias_len, keep_first);
  else
    return TS_ERR_DTYPE;
  return ts_launch_status();
}
