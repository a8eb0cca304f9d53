// Per-head normalisation of queries and keys, optional rotary encoding, and the scatter of keys
// and values into cache pages, for a projection output [T, Hq D + Hkv D + Hkv Dv] (q heads, k
// heads, v heads; values may have a width of their own).  The projection is of type T, or
// `splits` 32-bit partial sums that are added up here.
//
// A q or k head x of D elements becomes x * rsqrt(mean(x^2) + eps) * (gain_offset + gain[d]) in
// 32-bit (the gain vector is shared by the heads; a null gain skips the norm), is then rotated by
// the angles of the token's position where tables are given (pairs (i, i + D/2), as
// ts_rope_store), and is rounded once.  Queries go to q_out (rows q_stride apart; with a
// projection of type T this may be the projection itself), keys to key pages [NB, Hkv, BS, D] at
// slot = page * BS + offset, values to the transposed value pages [NB, Hkv, Dv, BS].  A negative
// slot or slots == nullptr: nothing is stored for that token.
//
// HeadShape holds what a mixer may ask beyond that: `normed` (divide by the root mean square also without a
// gain), `norm_after` (the norm follows the rotation instead of preceding it), `rot_dims` (only the first
// rot_dims elements of a head are turned, pairs (i, i + rot_dims/2), tables [capacity, rot_dims/2]; the
// rest pass), `values_are_keys` (there are no value columns: the values are the key heads as projected,
// before norm and rotation), `temp_coef`/`temp_every` (a query at position p is multiplied by 1 + temp_coef
// ln(floor((p + 1) / temp_every) + 1), last of all), `tail` (a row of the projection holds that many columns
// more behind the heads, which are left alone).
//
// Values may be blended with another layer's values of the same tokens before they are stored
// (ValueBlend): `keep` [T, Hkv Dv] 32-bit, if given, receives this layer's values as projected;
// `other` [T, Hkv Dv] 32-bit, if given, makes the stored value (1 - weight) v + weight other, in 32-bit.
#include <type_traits>

#include "common.hpp"

#define HNS_MAX_DIM 512
#define HNS_WAVES 4

struct HeadShape {
  int normed;
  int norm_after;
  int rot_dims;
  int values_are_keys;
  float temp_coef;
  int temp_every;
  int tail;  // columns of a projection's row behind the heads, read by others
};

struct ValueBlend {
  float* keep;
  const float* other;
  float weight;
};

__device__ __forceinline__ float blended(float v, size_t at, ValueBlend blend) {
  if (blend.keep) blend.keep[at] = v;
  return blend.other ? fmaf(blend.weight, blend.other[at], (1.f - blend.weight) * v) : v;
}

template <typename P>
__device__ __forceinline__ float sum_of_splits(const P* p, int splits, size_t stride) {
  if (splits == 1) return to_float(p[0]);
  float s = 0.f;
  for (int first = 0; first < splits; first += 8) {  // eight loads in flight, added in split order
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = to_float(p[(size_t)min(first + j, splits - 1) * stride]);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (first + j < splits) s += v[j];
  }
  return s;
}

// One wavefront per (token, q or k head) and, with `with_values`, per (token, v head) as well: a
// step of few tokens then stores its values in the same launch.
template <typename T, typename P>
__global__ void __launch_bounds__(64 * HNS_WAVES)
head_norm_store_kernel(T* q_out, long q_stride, const P* proj, int splits, size_t split_stride,
                       T* __restrict__ k_pages, T* __restrict__ v_pages, int with_values,
                       const T* __restrict__ q_gain, const T* __restrict__ k_gain,
                       float eps, float gain_offset, const float* __restrict__ cos_table,
                       const float* __restrict__ sin_table, const int* __restrict__ positions,
                       const int* __restrict__ slots, int tokens, int heads, int kv_heads, int dim, int vdim,
                       int block_size, ValueBlend blend, HeadShape shape) {
  __shared__ float held[HNS_WAVES][HNS_MAX_DIM];
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x % TS_WAVE;
  const int qk_heads = heads + kv_heads;
  const int all_heads = qk_heads + (with_values ? kv_heads : 0);
  const long item = (long)blockIdx.x * HNS_WAVES + wave;
  const size_t width = (size_t)qk_heads * dim + (shape.values_are_keys ? (size_t)0 : (size_t)kv_heads * vdim) + shape.tail;
  const size_t value_col0 = (size_t)(shape.values_are_keys ? heads : qk_heads) * dim;
  const int item_token = (int)(item / all_heads), item_head = (int)(item % all_heads);
  const bool is_value = item < (long)tokens * all_heads && item_head >= qk_heads;
  if (is_value) {
    // A value head: no norm, no rotation; element d of the token goes to row d of the transposed page.
    const int slot = slots ? slots[item_token] : -1;
    if (slot >= 0) {
      const int kvh = item_head - qk_heads;
      const P* values = proj + (size_t)item_token * width + value_col0 + (size_t)kvh * vdim;
      T* page = v_pages + ((size_t)(slot / block_size) * kv_heads + kvh) * vdim * block_size + slot % block_size;
      const size_t at = ((size_t)item_token * kv_heads + kvh) * vdim;
      for (int d = lane; d < vdim; d += TS_WAVE)
        page[(size_t)d * block_size] = from_float<T>(blended(sum_of_splits(values + d, splits, split_stride), at + d, blend));
    }
  }
  // (A value wavefront goes on as an idle one: the barrier below is the whole block's.)
  const bool active = item < (long)tokens * all_heads && !is_value;
  const int t = active ? item_token : 0;
  const int h = active ? item_head : 0;
  const P* row = proj + (size_t)t * width + (size_t)h * dim;
  const T* gain = h < heads ? q_gain : k_gain;
  constexpr int PER_LANE = HNS_MAX_DIM / TS_WAVE;
  float x[PER_LANE];
#pragma unroll
  for (int c = 0; c < PER_LANE; ++c) {
    const int d = lane + c * TS_WAVE;
    x[c] = (active && d < dim) ? sum_of_splits(row + d, splits, split_stride) : 0.f;
  }
  const bool normed = gain != nullptr || shape.normed;
  auto norm = [&]() __attribute__((always_inline)) {
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < PER_LANE; ++c) ss += x[c] * x[c];
    ss = wave_sum(ss);
    const float r = rsqrtf(ss / (float)dim + eps);
#pragma unroll
    for (int c = 0; c < PER_LANE; ++c) {
      const int d = lane + c * TS_WAVE;
      if (d < dim) x[c] = x[c] * r * (gain ? gain_offset + to_float(gain[d]) : 1.f);
    }
  };
  if (normed && !shape.norm_after) norm();
  if (cos_table) {
#pragma unroll
    for (int c = 0; c < PER_LANE; ++c) {
      const int d = lane + c * TS_WAVE;
      if (d < dim) held[wave][d] = x[c];
    }
    __syncthreads();
    const int turned = shape.rot_dims > 0 ? shape.rot_dims : dim;
    const int half = turned / 2;
    const size_t at = (size_t)positions[t] * half;
#pragma unroll
    for (int c = 0; c < PER_LANE; ++c) {
      const int d = lane + c * TS_WAVE;
      if (d < turned) {
        const int i = d < half ? d : d - half;
        const float x1 = held[wave][i], x2 = held[wave][i + half];
        const float cv = cos_table[at + i], sv = sin_table[at + i];
        x[c] = d < half ? __builtin_fmaf(x1, cv, -(x2 * sv)) : __builtin_fmaf(x2, cv, x1 * sv);
      }
    }
  }
  if (normed && shape.norm_after) norm();
  if (shape.temp_coef != 0.f && h < heads) {
    const float by = 1.f + shape.temp_coef * logf(floorf((float)(positions[t] + 1) / (float)shape.temp_every) + 1.f);
#pragma unroll
    for (int c = 0; c < PER_LANE; ++c) x[c] *= by;
  }
  if (!active) return;
  T* dst = nullptr;
  if (h < heads) {
    dst = q_out + (size_t)t * q_stride + (size_t)h * dim;
  } else {
    const int slot = slots ? slots[t] : -1;
    if (slot >= 0)
      dst = k_pages + (((size_t)(slot / block_size) * kv_heads + (h - heads)) * block_size + slot % block_size) * dim;
  }
  if (!dst) return;
#pragma unroll
  for (int c = 0; c < PER_LANE; ++c) {
    const int d = lane + c * TS_WAVE;
    if (d < dim) dst[d] = from_float<T>(x[c]);
  }
}

// The same for many tokens (prompt portions): bfloat16 in and out, no partial sums, no rotation,
// head size a multiple of 8 and at most 128.  Sixteen lanes per (token, q or k head), eight
// elements a lane with one 16-byte load and one 16-byte store; the sum of squares is formed over
// the sixteen lanes of a row by data-parallel moves.  Per element the arithmetic of the kernel
// above.
__global__ void __launch_bounds__(256)
head_norm_store_rows_kernel(bf16_t* q_out, long q_stride, const bf16_t* proj, bf16_t* __restrict__ k_pages,
                            const bf16_t* __restrict__ q_gain, const bf16_t* __restrict__ k_gain, float eps,
                            float gain_offset, const int* __restrict__ slots, int tokens, int heads, int kv_heads,
                            int dim, int vdim, int block_size) {
  const int qk_heads = heads + kv_heads;
  const long items = (long)tokens * qk_heads;
  const long asked = (long)blockIdx.x * 16 + threadIdx.x / 16;
  const bool valid = asked < items;  // rows beyond the last item read the last item and store nothing
  const long item = valid ? asked : items - 1;
  const int piece = threadIdx.x % 16;
  const int t = (int)(item / qk_heads), h = (int)(item % qk_heads);
  const bool holds = piece * 8 < dim;
  const size_t width = (size_t)qk_heads * dim + (size_t)kv_heads * vdim;
  const bf16_t* row = proj + (size_t)t * width + (size_t)h * dim;
  const bf16_t* gain = h < heads ? q_gain : k_gain;
  ts_u32x4 raw = {0u, 0u, 0u, 0u}, graw = {0u, 0u, 0u, 0u};
  if (holds) {
    raw = *reinterpret_cast<const ts_u32x4*>(row + piece * 8);
    if (gain) graw = *reinterpret_cast<const ts_u32x4*>(gain + piece * 8);
  }
  float x[8], g[8];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    x[2 * e] = __uint_as_float(raw[e] << 16);
    x[2 * e + 1] = __uint_as_float(raw[e] & 0xffff0000u);
    g[2 * e] = __uint_as_float(graw[e] << 16);
    g[2 * e + 1] = __uint_as_float(graw[e] & 0xffff0000u);
    ss += x[2 * e] * x[2 * e] + x[2 * e + 1] * x[2 * e + 1];
  }
  if (gain) {
    // Over the row of sixteen lanes (the first four steps of wave_sum).
    ss += lanes_moved<0xB1, 0xF>(0.f, ss);
    ss += lanes_moved<0x4E, 0xF>(0.f, ss);
    ss += lanes_moved<0x141, 0xF>(0.f, ss);
    ss += lanes_moved<0x140, 0xF>(0.f, ss);
    const float r = rsqrtf(ss / (float)dim + eps);
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = x[e] * r * (gain_offset + g[e]);
  }
  bf16_t* dst = nullptr;
  if (h < heads) {
    dst = q_out + (size_t)t * q_stride + (size_t)h * dim;
  } else {
    const int slot = slots ? slots[t] : -1;
    if (slot >= 0)
      dst = k_pages + (((size_t)(slot / block_size) * kv_heads + (h - heads)) * block_size + slot % block_size) * dim;
  }
  if (!dst || !holds || !valid) return;
  ts_u32x4 packed;
#pragma unroll
  for (int e = 0; e < 4; ++e)
    packed[e] = (uint32_t)from_float<bf16_t>(x[2 * e]).bits | ((uint32_t)from_float<bf16_t>(x[2 * e + 1]).bits << 16);
  *reinterpret_cast<ts_u32x4*>(dst + piece * 8) = packed;
}

// Values: one block per (group of 8 consecutive tokens, KV head); a thread collects one value
// dimension of the 8 tokens.  Where the group's slots are 8 consecutive ones that start at a
// multiple of 8 inside one page, a bfloat16 group leaves as one 16-byte store.
constexpr int HNS_GROUP = 8;

template <typename T, typename P>
__global__ void __launch_bounds__(64)
value_store_kernel(const P* proj, int splits, size_t split_stride, T* __restrict__ v_pages,
                   const int* __restrict__ slots, int tokens, int heads, int kv_heads, int dim, int vdim,
                   int block_size, ValueBlend blend, int values_are_keys, int tail) {
  const int t0 = blockIdx.x * HNS_GROUP;
  const int kvh = blockIdx.y;
  const int count = min(HNS_GROUP, tokens - t0);
  const size_t width = (size_t)(heads + kv_heads) * dim + (values_are_keys ? (size_t)0 : (size_t)kv_heads * vdim) + tail;
  int slot[HNS_GROUP];
#pragma unroll
  for (int j = 0; j < HNS_GROUP; ++j) slot[j] = j < count ? slots[t0 + j] : -1;
  bool run = sizeof(T) == 2 && count == HNS_GROUP && slot[0] >= 0 && (slot[0] & 7) == 0 && (block_size & 7) == 0;
#pragma unroll
  for (int j = 1; j < HNS_GROUP; ++j) run = run && slot[j] == slot[0] + j;
  const P* column = proj + (size_t)t0 * width + (size_t)(values_are_keys ? heads : heads + kv_heads) * dim + (size_t)kvh * vdim;
  for (int d = threadIdx.x; d < vdim; d += blockDim.x) {
    alignas(16) T v[HNS_GROUP];
#pragma unroll
    for (int j = 0; j < HNS_GROUP; ++j)
      v[j] = from_float<T>(j < count ? blended(sum_of_splits(column + (size_t)j * width + d, splits, split_stride),
                                               ((size_t)(t0 + j) * kv_heads + kvh) * vdim + d, blend)
                                     : 0.f);
    if (run) {
      T* dst = v_pages + (((size_t)(slot[0] / block_size) * kv_heads + kvh) * vdim + d) * block_size + slot[0] % block_size;
      *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(v);
    } else {
#pragma unroll
      for (int j = 0; j < HNS_GROUP; ++j) {
        if (slot[j] < 0) continue;
        v_pages[(((size_t)(slot[j] / block_size) * kv_heads + kvh) * vdim + d) * block_size + slot[j] % block_size] = v[j];
      }
    }
  }
}

template <typename T, typename P>
static void launch_head_norm_store(void* q_out, long q_stride, const void* proj, int splits, long split_stride,
                                   void* k_pages, void* v_pages, const void* q_gain, const void* k_gain, float eps,
                                   float gain_offset, const float* cos_table, const float* sin_table,
                                   const int* positions, const int* slots, int tokens, int heads, int kv_heads,
                                   int dim, int vdim, int block_size, ValueBlend blend, HeadShape shape, hipStream_t stream) {
  const bool few = tokens < 4 * HNS_GROUP || splits > 1;  // values in the same launch, a wavefront per value head
  const long items = (long)tokens * (heads + kv_heads + (few && slots ? kv_heads : 0));
  const bool aligned = ((uintptr_t)q_out | (uintptr_t)proj | (uintptr_t)k_pages | (uintptr_t)q_gain | (uintptr_t)k_gain) % 16 == 0 &&
                       q_stride % 8 == 0 && vdim % 8 == 0;
  const bool plain = (!shape.normed || q_gain) && !shape.norm_after && !shape.values_are_keys && shape.temp_coef == 0.f && shape.tail == 0;
  if (std::is_same<T, bf16_t>::value && std::is_same<P, bf16_t>::value && splits == 1 && !cos_table && dim % 8 == 0 &&
      dim <= 128 && !few && aligned && plain)
    hipLaunchKernelGGL(head_norm_store_rows_kernel, dim3((unsigned)((items + 15) / 16)), dim3(256), 0, stream, (bf16_t*)q_out,
                       q_stride, (const bf16_t*)proj, (bf16_t*)k_pages, (const bf16_t*)q_gain, (const bf16_t*)k_gain, eps,
                       gain_offset, slots, tokens, heads, kv_heads, dim, vdim, block_size);
  else
    hipLaunchKernelGGL((head_norm_store_kernel<T, P>), dim3((unsigned)((items + HNS_WAVES - 1) / HNS_WAVES)),
                       dim3(64 * HNS_WAVES), 0, stream, (T*)q_out, q_stride, (const P*)proj, splits, (size_t)split_stride,
                       (T*)k_pages, (T*)v_pages, few && slots ? 1 : 0, (const T*)q_gain, (const T*)k_gain, eps, gain_offset,
                       cos_table, sin_table, positions, slots, tokens, heads, kv_heads, dim, vdim, block_size, blend, shape);
  if (slots && !few)
    hipLaunchKernelGGL((value_store_kernel<T, P>), dim3((tokens + HNS_GROUP - 1) / HNS_GROUP, kv_heads), dim3(64), 0,
                       stream, (const P*)proj, splits, (size_t)split_stride, (T*)v_pages, slots, tokens, heads, kv_heads,
                       dim, vdim, block_size, blend, shape.values_are_keys, shape.tail);
}

extern "C" int ts_head_norm_store(void* q_out, long q_stride, const void* proj, int in_f32, int splits,
                                  long split_stride, void* k_pages, void* v_pages, const void* q_gain,
                                  const void* k_gain, float eps, float gain_offset, const float* cos_table,
                                  const float* sin_table, const int* positions, const int* slots, int tokens,
                                  int heads, int kv_heads, int dim, int vdim, int block_size, int dtype,
                                  float* v_keep, const float* v_other, float v_weight, int normed, int norm_after,
                                  int rot_dims, int values_are_keys, float temp_coef, int temp_every, int tail, hipStream_t stream) {
  if (tokens == 0) return TS_OK;
  const HeadShape shape = {normed, norm_after, rot_dims, values_are_keys, temp_coef, temp_every, tail};
  if (rot_dims < 0 || rot_dims > dim || (rot_dims & 1) || (values_are_keys && vdim != dim) || (temp_coef != 0.f && temp_every < 1) || tail < 0)
    return TS_ERR_ARG;
  if ((v_keep || v_other) && !slots) return TS_ERR_ARG;  // values are only walked where they are stored
  const ValueBlend blend = {v_keep, v_other, v_weight};
  if (!q_out || !proj || !positions || heads < 1 || kv_heads < 1 || dim < 1 || dim > HNS_MAX_DIM || vdim < 1 ||
      block_size < 1 || splits < 1 || kv_heads > 65535)
    return TS_ERR_ARG;
  if ((cos_table == nullptr) != (sin_table == nullptr) || (cos_table && rot_dims == 0 && (dim & 1))) return TS_ERR_ARG;
  if ((q_gain == nullptr) != (k_gain == nullptr)) return TS_ERR_ARG;
  if (slots && (!k_pages || !v_pages)) return TS_ERR_ARG;
  if (dtype == TS_F32)
    launch_head_norm_store<float, float>(q_out, q_stride, proj, splits, split_stride, k_pages, v_pages, q_gain, k_gain, eps, gain_offset, cos_table, sin_table, positions, slots, tokens, heads, kv_heads, dim, vdim, block_size, blend, shape, stream);
  else if (dtype == TS_BF16 && in_f32)
    launch_head_norm_store<bf16_t, float>(q_out, q_stride, proj, splits, split_stride, k_pages, v_pages, q_gain, k_gain, eps, gain_offset, cos_table, sin_table, positions, slots, tokens, heads, kv_heads, dim, vdim, block_size, blend, shape, stream);
  else if (dtype == TS_BF16)
    launch_head_norm_store<bf16_t, bf16_t>(q_out, q_stride, proj, splits, split_stride, k_pages, v_pages, q_gain, k_gain, eps, gain_offset, cos_table, sin_table, positions, slots, tokens, heads, kv_heads, dim, vdim, block_size, blend, shape, stream);
  else
    return TS_ERR_DTYPE;
  return ts_launch_status();
}
