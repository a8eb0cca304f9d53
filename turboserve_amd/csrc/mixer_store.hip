// Row-wise kernels around mixers that are not per-head rotary attention:
//
//   ts_span_norm_store   queries and keys normalised over their whole projection (all heads at once)
//                        and the scatter of keys and values into cache pages;
//   ts_latent_store      a latent-attention layer's pass over its projection: the compressed
//                        vector is normalised, the shared rotated key part and the queries' rotated
//                        parts are turned by the position's angles, latent and rotated key go into
//                        the key pages as one row, the queries are split for what follows;
//   ts_head_gate         every head's output times the sigmoid of a gate column of the projection;
//   ts_scaled_pair       a_scale * a + b_scale * b of two parts' outputs, 32-bit;
//   ts_stream_fold       residual (+)= a part's output (a tensor of the run type or 32-bit partial sums);
//   ts_stream_pair       [x | origin] of two 32-bit streams side by side, in the run type.
//
// A projection is of type T (the run's), or `splits` 32-bit partial sums that are added up here.
// Statistics, gains and rotations are 32-bit; a value is rounded once, where it is stored.
#include <type_traits>

#include "common.hpp"

// The sum of a projection's partial sums, added in split order, eight loads in flight at a time (a
// loop of load, wait, add would cost a trip to memory per split).
template <typename P>
__device__ __forceinline__ float folded(const P* p, int splits, size_t stride) {
  if (splits == 1) return to_float(p[0]);
  float s = 0.f;
  for (int first = 0; first < splits; first += 8) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = to_float(p[(size_t)min(first + j, splits - 1) * stride]);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (first + j < splits) s += v[j];
  }
  return s;
}

// ---------------------------------------------------------------------------------------------
// One block per token.  Row of the projection: [Hq D queries | Hkv D keys | Hkv Dv values].
// q <- q * rsqrt(mean_all(q^2) + eps) * (gain_offset + q_gain[i]), i over all Hq D elements; the keys
// likewise over their Hkv D.  Keys go to [NB, Hkv, BS, D], values to the transposed [NB, Hkv, Dv, BS].
// ---------------------------------------------------------------------------------------------
template <typename T, typename P>
__global__ void __launch_bounds__(1024)
span_norm_store_kernel(T* q_out, long q_stride, const P* proj, int splits, size_t split_stride,
                       T* __restrict__ k_pages, T* __restrict__ v_pages, const T* __restrict__ q_gain,
                       const T* __restrict__ k_gain, float eps, float gain_offset, const int* __restrict__ slots,
                       int heads, int kv_heads, int dim, int vdim, int block_size) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const int q_size = heads * dim, k_size = kv_heads * dim, v_size = kv_heads * vdim;
  const P* row = proj + (size_t)t * (q_size + k_size + v_size);
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < q_size; i += blockDim.x) {
    const float x = folded(row + i, splits, split_stride);
    sq = fmaf(x, x, sq);
  }
  for (int i = threadIdx.x; i < k_size; i += blockDim.x) {
    const float x = folded(row + q_size + i, splits, split_stride);
    sk = fmaf(x, x, sk);
  }
  sq = block_sum(sq, scratch);
  sk = block_sum(sk, scratch);
  const float rq = rsqrtf(sq / (float)q_size + eps);
  const float rk = rsqrtf(sk / (float)k_size + eps);
  T* q_row = q_out + (size_t)t * q_stride;
  for (int i = threadIdx.x; i < q_size; i += blockDim.x) {
    const float x = folded(row + i, splits, split_stride);
    q_row[i] = from_float<T>(x * rq * (gain_offset + to_float(q_gain[i])));
  }
  const int slot = slots ? slots[t] : -1;
  if (slot < 0) return;
  const size_t page = (size_t)(slot / block_size), offset = (size_t)(slot % block_size);
  for (int i = threadIdx.x; i < k_size; i += blockDim.x) {
    const float x = folded(row + q_size + i, splits, split_stride);
    const int kvh = i / dim, d = i % dim;
    k_pages[((page * kv_heads + kvh) * block_size + offset) * dim + d] =
        from_float<T>(x * rk * (gain_offset + to_float(k_gain[i])));
  }
  for (int i = threadIdx.x; i < v_size; i += blockDim.x) {
    const float x = folded(row + q_size + k_size + i, splits, split_stride);
    const int kvh = i / vdim, d = i % vdim;
    v_pages[((page * kv_heads + kvh) * vdim + d) * block_size + offset] = from_float<T>(x);
  }
}

template <typename T, typename P>
static int span_norm_store_launch(void* q_out, long q_stride, const void* proj, int splits, long split_stride,
                                  void* k_pages, void* v_pages, const void* q_gain, const void* k_gain, float eps,
                                  float gain_offset, const int* slots, int tokens, int heads, int kv_heads, int dim,
                                  int vdim, int block_size, hipStream_t stream) {
  // A step of few tokens has few blocks: each then takes a whole compute unit's threads.
  hipLaunchKernelGGL((span_norm_store_kernel<T, P>), dim3(tokens), dim3(tokens <= 64 ? 1024 : 256), 0, stream, (T*)q_out, q_stride,
                     (const P*)proj, splits, (size_t)split_stride, (T*)k_pages, (T*)v_pages, (const T*)q_gain,
                     (const T*)k_gain, eps, gain_offset, slots, heads, kv_heads, dim, vdim, block_size);
  return ts_launch_status();
}

extern "C" int ts_span_norm_store(void* q_out, long q_stride, const void* proj, int in_f32, int splits,
                                  long split_stride, void* k_pages, void* v_pages, const void* q_gain,
                                  const void* k_gain, float eps, float gain_offset, const int* slots, int tokens,
                                  int heads, int kv_heads, int dim, int vdim, int block_size, int dtype,
                                  hipStream_t stream) {
  if (tokens == 0) return TS_OK;
  if (!q_out || !proj || !q_gain || !k_gain || (slots && (!k_pages || !v_pages))) return TS_ERR_ARG;
  if (heads < 1 || kv_heads < 1 || dim < 1 || vdim < 1 || block_size < 1 || splits < 1) return TS_ERR_SHAPE;
  if (dtype == TS_F32)
    return span_norm_store_launch<float, float>(q_out, q_stride, proj, splits, split_stride, k_pages, v_pages, q_gain, k_gain, eps, gain_offset, slots, tokens, heads, kv_heads, dim, vdim, block_size, stream);
  if (dtype == TS_BF16 && in_f32)
    return span_norm_store_launch<bf16_t, float>(q_out, q_stride, proj, splits, split_stride, k_pages, v_pages, q_gain, k_gain, eps, gain_offset, slots, tokens, heads, kv_heads, dim, vdim, block_size, stream);
  if (dtype == TS_BF16)
    return span_norm_store_launch<bf16_t, bf16_t>(q_out, q_stride, proj, 1, 0, k_pages, v_pages, q_gain, k_gain, eps, gain_offset, slots, tokens, heads, kv_heads, dim, vdim, block_size, stream);
  return TS_ERR_DTYPE;
}

// ---------------------------------------------------------------------------------------------
// One block per token.  Row of the projection: [H (D plain | R rotated) queries | C latent | R
// rotated key | `tail` more columns that are not read here].  Of a rotated part the first `turned`
// elements are turned in pairs (i, i + turned / 2), or with `neighbours` in pairs (2 i, 2 i + 1), by
// the angles of the token's position (tables [capacity, turned / 2], 32-bit, which may carry a
// factor on both the cosine and the sine); the rest pass unchanged.
//   key page row [NB, 1, BS, C + R] at the token's slot  <- [latent * rsqrt(mean(latent^2) + eps) * gain | turned key]
//   q_plain [T H, D]                                     <- the queries' plain parts
//   q_wide  [T, H, C + R], elements C..C+R-1 only        <- the queries' turned parts
// (elements 0..C-1 of q_wide are the plain parts carried through the keys' up-projection, which a
// product writes afterwards).
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float turned_element(const float* part, int i, int turned, const float* cos_row,
                                                const float* sin_row, int neighbours) {
  const int half = turned / 2;
  if (i >= turned) return part[i];
  if (neighbours) {  // pairs (2 j, 2 j + 1), angle j
    const int j = i / 2;
    if ((i & 1) == 0) return __builtin_fmaf(part[i], cos_row[j], -(part[i + 1] * sin_row[j]));
    return __builtin_fmaf(part[i], cos_row[j], part[i - 1] * sin_row[j]);
  }
  if (i < half) return __builtin_fmaf(part[i], cos_row[i], -(part[i + half] * sin_row[i]));
  return __builtin_fmaf(part[i], cos_row[i - half], part[i - half] * sin_row[i - half]);
}

template <typename T, typename P>
__global__ void __launch_bounds__(1024)
latent_store_kernel(T* __restrict__ q_plain, T* __restrict__ q_wide, const P* proj, int splits, size_t split_stride,
                    T* __restrict__ k_pages, const T* __restrict__ gain, float eps,
                    const float* __restrict__ cos_table, const float* __restrict__ sin_table,
                    const int* __restrict__ positions, const int* __restrict__ slots, int heads, int dim,
                    int rot, int rank, int turned, int block_size, int neighbours, int tail) {
  extern __shared__ float held[];  // [heads * rot] the queries' rotated parts, [rot] the key's, then the latent
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const int per_head = dim + rot;
  const int q_size = heads * per_head;
  const P* row = proj + (size_t)t * (q_size + rank + rot + tail);
  float* q_rot = held;
  float* k_rot = held + heads * rot;
  float* latent = k_rot + rot;
  float ss = 0.f;
  for (int i = threadIdx.x; i < heads * rot; i += blockDim.x)
    q_rot[i] = folded(row + (size_t)(i / rot) * per_head + dim + i % rot, splits, split_stride);
  for (int i = threadIdx.x; i < rank; i += blockDim.x) {
    const float x = folded(row + q_size + i, splits, split_stride);
    latent[i] = x;
    ss = fmaf(x, x, ss);
  }
  for (int i = threadIdx.x; i < rot; i += blockDim.x) k_rot[i] = folded(row + q_size + rank + i, splits, split_stride);
  ss = block_sum(ss, scratch);  // (its barriers also publish what was just held)
  const float r = rsqrtf(ss / (float)rank + eps);
  const size_t at = (size_t)positions[t] * (turned / 2);
  const float* cos_row = cos_table + at;
  const float* sin_row = sin_table + at;
  const int wide = rank + rot;
  for (int i = threadIdx.x; i < heads * dim; i += blockDim.x) {
    const int h = i / dim, d = i % dim;
    q_plain[((size_t)t * heads + h) * dim + d] = from_float<T>(folded(row + (size_t)h * per_head + d, splits, split_stride));
  }
  for (int i = threadIdx.x; i < heads * rot; i += blockDim.x) {
    const int h = i / rot, d = i % rot;
    q_wide[((size_t)t * heads + h) * wide + rank + d] = from_float<T>(turned_element(q_rot + h * rot, d, turned, cos_row, sin_row, neighbours));
  }
  const int slot = slots ? slots[t] : -1;
  if (slot < 0) return;
  T* dst = k_pages + (size_t)slot * wide;  // one key head: row `slot` of [NB * BS, C + R]
  for (int i = threadIdx.x; i < rank; i += blockDim.x) dst[i] = from_float<T>(latent[i] * r * to_float(gain[i]));
  for (int i = threadIdx.x; i < rot; i += blockDim.x)
    dst[rank + i] = from_float<T>(turned_element(k_rot, i, turned, cos_row, sin_row, neighbours));
}

template <typename T, typename P>
static int latent_store_launch(void* q_plain, void* q_wide, const void* proj, int splits, long split_stride, void* k_pages,
                               const void* gain, float eps, const float* cos_table, const float* sin_table,
                               const int* positions, const int* slots, int tokens, int heads, int dim, int rot, int rank,
                               int turned, int block_size, int neighbours, int tail, hipStream_t stream) {
  const size_t lds = (size_t)(heads * rot + rot + rank) * sizeof(float);
  if (lds > 60 * 1024) return TS_ERR_SHAPE;
  hipLaunchKernelGGL((latent_store_kernel<T, P>), dim3(tokens), dim3(tokens <= 64 ? 1024 : 256), lds, stream, (T*)q_plain, (T*)q_wide,
                     (const P*)proj, splits, (size_t)split_stride, (T*)k_pages, (const T*)gain, eps, cos_table, sin_table,
                     positions, slots, heads, dim, rot, rank, turned, block_size, neighbours, tail);
  return ts_launch_status();
}

extern "C" int ts_latent_store(void* q_plain, void* q_wide, const void* proj, int in_f32, int splits, long split_stride,
                               void* k_pages, const void* gain, float eps, const float* cos_table,
                               const float* sin_table, const int* positions, const int* slots, int tokens, int heads,
                               int dim, int rot, int rank, int turned, int block_size, int neighbours, int tail, int dtype,
                               hipStream_t stream) {
  if (tokens == 0) return TS_OK;
  if (!q_plain || !q_wide || !proj || !gain || !cos_table || !sin_table || !positions || (slots && !k_pages))
    return TS_ERR_ARG;
  if (heads < 1 || dim < 1 || rot < 1 || rank < 1 || turned < 2 || turned > rot || (turned & 1) || block_size < 1 || splits < 1 || tail < 0)
    return TS_ERR_SHAPE;
  if (dtype == TS_F32)
    return latent_store_launch<float, float>(q_plain, q_wide, proj, splits, split_stride, k_pages, gain, eps, cos_table, sin_table, positions, slots, tokens, heads, dim, rot, rank, turned, block_size, neighbours, tail, stream);
  if (dtype == TS_BF16 && in_f32)
    return latent_store_launch<bf16_t, float>(q_plain, q_wide, proj, splits, split_stride, k_pages, gain, eps, cos_table, sin_table, positions, slots, tokens, heads, dim, rot, rank, turned, block_size, neighbours, tail, stream);
  if (dtype == TS_BF16)
    return latent_store_launch<bf16_t, bf16_t>(q_plain, q_wide, proj, 1, 0, k_pages, gain, eps, cos_table, sin_table, positions, slots, tokens, heads, dim, rot, rank, turned, block_size, neighbours, tail, stream);
  return TS_ERR_DTYPE;
}

// ---------------------------------------------------------------------------------------------
// out [T, H, Dv] of the run type: head h's row of the 32-bit `values` [T, H, Dv] times the sigmoid of
// the head's gate, which is column gate_at + h of the token's row of a projection (`width` columns; of
// type T, or `splits` 32-bit partial sums).  32-bit arithmetic, one rounding.
// ---------------------------------------------------------------------------------------------
template <typename V>
__device__ __forceinline__ float4 gate_values4(const V* at);
template <>
__device__ __forceinline__ float4 gate_values4<float>(const float* at) {
  return *reinterpret_cast<const float4*>(at);
}
template <>
__device__ __forceinline__ float4 gate_values4<bf16_t>(const bf16_t* at) {
  const uint2 raw = *reinterpret_cast<const uint2*>(at);
  return make_float4(__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u), __uint_as_float(raw.y << 16),
                     __uint_as_float(raw.y & 0xffff0000u));
}

// V: the type of the values, 32-bit or the run's.
template <typename T, typename P, typename V>
__global__ void __launch_bounds__(256)
head_gate_kernel(T* __restrict__ out, const V* __restrict__ values, const P* __restrict__ proj, int splits,
                 size_t split_stride, int width, int gate_at, int heads, int vdim, float scale, size_t out_stride) {
  const int t = blockIdx.x;
  const int per = heads * vdim;
  for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < per; i += gridDim.y * blockDim.x) {
    const float g = folded(proj + (size_t)t * width + gate_at + i / vdim, splits, split_stride);
    out[(size_t)t * out_stride + i] = from_float<T>(scale * to_float(values[(size_t)t * per + i]) / (1.f + expf(-g)));
  }
}

// The same, four elements of one head a thread (vdim a multiple of 4, 16-byte aligned rows).
template <typename T, typename P, typename V>
__global__ void __launch_bounds__(256)
head_gate_vec4_kernel(T* __restrict__ out, const V* __restrict__ values, const P* __restrict__ proj, int splits,
                      size_t split_stride, int width, int gate_at, int heads, int vdim, float scale, size_t out_stride) {
  const int t = blockIdx.x;
  const int per = heads * vdim;
  const int i = 4 * (blockIdx.y * blockDim.x + threadIdx.x);
  if (i >= per) return;
  const float4 v = gate_values4<V>(values + (size_t)t * per + i);
  const float g = folded(proj + (size_t)t * width + gate_at + i / vdim, splits, split_stride);
  const float d = (1.f + expf(-g)) / scale;
  T* to = out + (size_t)t * out_stride + i;
  if constexpr (std::is_same<T, float>::value) {
    *reinterpret_cast<float4*>(to) = make_float4(v.x / d, v.y / d, v.z / d, v.w / d);
  } else {
    uint2 packed;
    packed.x = (uint32_t)from_float<bf16_t>(v.x / d).bits | ((uint32_t)from_float<bf16_t>(v.y / d).bits << 16);
    packed.y = (uint32_t)from_float<bf16_t>(v.z / d).bits | ((uint32_t)from_float<bf16_t>(v.w / d).bits << 16);
    *reinterpret_cast<uint2*>(to) = packed;
  }
}

template <typename T, typename P, typename V>
static void launch_head_gate(void* out, const void* values, const void* proj, int splits, size_t split_stride, int tokens,
                             int width, int gate_at, int heads, int vdim, float scale, size_t out_stride, hipStream_t stream) {
  const int per = heads * vdim;
  if (vdim % 4 == 0 && ((uintptr_t)out | (uintptr_t)values) % 16 == 0 && out_stride % 4 == 0 && scale != 0.f) {
    const dim3 grid(tokens, (per / 4 + 255) / 256);
    hipLaunchKernelGGL((head_gate_vec4_kernel<T, P, V>), grid, dim3(256), 0, stream, (T*)out, (const V*)values, (const P*)proj,
                       splits, split_stride, width, gate_at, heads, vdim, scale, out_stride);
  } else {
    const dim3 grid(tokens, (per + 1023) / 1024);
    hipLaunchKernelGGL((head_gate_kernel<T, P, V>), grid, dim3(256), 0, stream, (T*)out, (const V*)values, (const P*)proj,
                       splits, split_stride, width, gate_at, heads, vdim, scale, out_stride);
  }
}

// values_f32: the values are 32-bit (else of the run's type, as the attention kernels leave them).  The result
// is multiplied by `scale` as well, and its rows lie `out_stride` elements apart (a part of a wider buffer).
extern "C" int ts_head_gate(void* out, const void* values, int values_f32, const void* proj, int in_f32, int splits,
                            long split_stride, int tokens, int width, int gate_at, int heads, int vdim, int dtype,
                            float scale, long out_stride, hipStream_t stream) {
  if (tokens == 0) return TS_OK;
  if (!out || !values || !proj || heads < 1 || vdim < 1 || splits < 1 || gate_at < 0 || gate_at + heads > width ||
      out_stride < (long)heads * vdim)
    return TS_ERR_ARG;
  if (dtype == TS_F32)
    launch_head_gate<float, float, float>(out, values, proj, splits, (size_t)split_stride, tokens, width, gate_at, heads, vdim, scale, (size_t)out_stride, stream);
  else if (dtype == TS_BF16 && in_f32 && values_f32)
    launch_head_gate<bf16_t, float, float>(out, values, proj, splits, (size_t)split_stride, tokens, width, gate_at, heads, vdim, scale, (size_t)out_stride, stream);
  else if (dtype == TS_BF16 && in_f32)
    launch_head_gate<bf16_t, float, bf16_t>(out, values, proj, splits, (size_t)split_stride, tokens, width, gate_at, heads, vdim, scale, (size_t)out_stride, stream);
  else if (dtype == TS_BF16 && values_f32)
    launch_head_gate<bf16_t, bf16_t, float>(out, values, proj, 1, (size_t)0, tokens, width, gate_at, heads, vdim, scale, (size_t)out_stride, stream);
  else if (dtype == TS_BF16)
    launch_head_gate<bf16_t, bf16_t, bf16_t>(out, values, proj, 1, (size_t)0, tokens, width, gate_at, heads, vdim, scale, (size_t)out_stride, stream);
  else
    return TS_ERR_DTYPE;
  return ts_launch_status();
}

// ---------------------------------------------------------------------------------------------
// out[i] = a_scale * a[i] + b_scale * b[i] in 32-bit: two parts' outputs (each a tensor of the run type or
// 32-bit partial sums) as one addend of the residual stream.
// ---------------------------------------------------------------------------------------------
template <typename A, typename B>
__global__ void scaled_pair_kernel(float* __restrict__ out, const A* __restrict__ a, int a_splits, size_t a_stride, float a_scale,
                                   const B* __restrict__ b, int b_splits, size_t b_stride, float b_scale, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  out[idx] = fmaf(a_scale, folded(a + idx, a_splits, a_stride), b_scale * folded(b + idx, b_splits, b_stride));
}

extern "C" int ts_scaled_pair(float* out, const void* a, int a_f32, int a_splits, long a_stride, float a_scale, const void* b,
                              int b_f32, int b_splits, long b_stride, float b_scale, long total, int dtype, hipStream_t stream) {
  if (total == 0) return TS_OK;
  if (!out || !a || !b || total < 0 || a_splits < 1 || b_splits < 1) return TS_ERR_ARG;
  if (dtype != TS_F32 && dtype != TS_BF16) return TS_ERR_DTYPE;
  const dim3 grid((unsigned)((total + 255) / 256)), block(256);
  const bool wide_a = a_f32 || dtype == TS_F32, wide_b = b_f32 || dtype == TS_F32;
#define SP_GO(A, B)                                                                                                  \
  hipLaunchKernelGGL((scaled_pair_kernel<A, B>), grid, block, 0, stream, out, (const A*)a, a_splits, (size_t)a_stride, \
                     a_scale, (const B*)b, b_splits, (size_t)b_stride, b_scale, (size_t)total)
  if (wide_a && wide_b) SP_GO(float, float);
  else if (wide_a) SP_GO(float, bf16_t);
  else if (wide_b) SP_GO(bf16_t, float);
  else SP_GO(bf16_t, bf16_t);
#undef SP_GO
  return ts_launch_status();
}

// ---------------------------------------------------------------------------------------------
// residual[i] = (assign ? 0 : residual[i]) + sum over splits of part[i], 32-bit.
// ---------------------------------------------------------------------------------------------
template <typename P>
__global__ void stream_fold_kernel(float* __restrict__ residual, const P* __restrict__ part, int splits,
                                   size_t split_stride, int assign, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const float s = folded(part + idx, splits, split_stride);
  residual[idx] = assign ? s : residual[idx] + s;
}

extern "C" int ts_stream_fold(float* residual, const void* part, int part_f32, int splits, long split_stride, long total,
                              int assign, int dtype, hipStream_t stream) {
  if (total == 0) return TS_OK;
  if (!residual || !part || total < 0 || splits < 1) return TS_ERR_ARG;
  const dim3 grid((unsigned)((total + 255) / 256)), block(256);
  if (part_f32 || dtype == TS_F32)
    hipLaunchKernelGGL(stream_fold_kernel<float>, grid, block, 0, stream, residual, (const float*)part, splits, (size_t)split_stride, assign, (size_t)total);
  else if (dtype == TS_BF16)
    hipLaunchKernelGGL(stream_fold_kernel<bf16_t>, grid, block, 0, stream, residual, (const bf16_t*)part, 1, (size_t)0, assign, (size_t)total);
  else
    return TS_ERR_DTYPE;
  return ts_launch_status();
}

// ---------------------------------------------------------------------------------------------
// out [T, 2 H] of the run type: row t is [x[t] | origin[t]], each rounded once.
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void stream_pair_kernel(T* __restrict__ out, const float* __restrict__ x, const float* __restrict__ origin,
                                   int hidden, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t t = idx / (2 * (size_t)hidden);
  const int i = (int)(idx % (2 * (size_t)hidden));
  out[idx] = from_float<T>(i < hidden ? x[t * hidden + i] : origin[t * hidden + i - hidden]);
}

extern "C" int ts_stream_pair(void* out, const float* x, const float* origin, int tokens, int hidden, int dtype,
                              hipStream_t stream) {
  if (tokens == 0) return TS_OK;
  if (!out || !x || !origin || hidden < 1) return TS_ERR_ARG;
  const size_t total = (size_t)tokens * 2 * hidden;
  const dim3 grid((unsigned)((total + 255) / 256)), block(256);
  if (dtype == TS_F32)
    hipLaunchKernelGGL(stream_pair_kernel<float>, grid, block, 0, stream, (float*)out, x, origin, hidden, total);
  else if (dtype == TS_BF16)
    hipLaunchKernelGGL(stream_pair_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)out, x, origin, hidden, total);
  else
    return TS_ERR_DTYPE;
  return ts_launch_status();
}
