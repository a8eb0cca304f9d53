// A norm without statistics, and a cap on the logits.
//
// ts_add_tanh_norm: s = residual + pending (+ also), in 32-bit; residual = s; y = round_T(tanh(alpha s) * w + b)
// with a scalar alpha and vectors w, b of the row's size.  With `rows` the kernel reads rows[i] and
// writes y[i] only (residual untouched): the final norm at the wanted positions.  `pending` is of type
// T, or `splits` 32-bit partial sums `split_stride` elements apart that are added up here; `also` is a
// second addend of 32-bit partial sums.  Nothing is reduced over a row, so a thread owns four
// neighbouring elements (or one, where the row's size is no multiple of four) and a row may be
// spread over several workgroups.
//
// ts_tanh_cap: x <- cap * tanh(x / cap) in place over 32-bit values.
#include "common.hpp"

template <typename P>
__device__ __forceinline__ float tn_add_splits(const P* p, int splits, size_t stride, float init) {
  float s = init;
  if (splits == 1) return s + to_float(p[0]);
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

template <typename T, typename P, int PER>
__global__ void __launch_bounds__(256)
add_tanh_norm_kernel(T* __restrict__ y, float* __restrict__ residual, const P* __restrict__ pending, int splits,
                     size_t split_stride, const T* __restrict__ w, const T* __restrict__ b, float alpha,
                     const int* __restrict__ rows, int hidden, const float* __restrict__ also, int also_splits,
                     size_t also_stride) {
  const int first = (blockIdx.y * blockDim.x + threadIdx.x) * PER;
  if (first >= hidden) return;
  const int src = rows ? rows[blockIdx.x] : blockIdx.x;
  const size_t in_base = (size_t)src * hidden + first;
  const size_t out_base = (size_t)blockIdx.x * hidden + first;
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    float s = residual[in_base + e];
    if (pending) s = tn_add_splits(pending + in_base + e, splits, split_stride, s);
    if (also) s = tn_add_splits(also + in_base + e, also_splits, also_stride, s);
    if ((pending || also) && !rows) residual[in_base + e] = s;
    y[out_base + e] = from_float<T>(fmaf(tanhf(alpha * s), to_float(w[first + e]), to_float(b[first + e])));
  }
}

template <typename T, typename P>
static void launch_add_tanh_norm(void* y, float* residual, const void* pending, int splits, long split_stride, const void* w,
                                 const void* b, float alpha, const int* rows, int out_rows, int hidden, const float* also,
                                 int also_splits, long also_stride, hipStream_t stream) {
  if (hidden % 4 == 0) {
    const dim3 grid(out_rows, (hidden / 4 + 255) / 256);
    hipLaunchKernelGGL((add_tanh_norm_kernel<T, P, 4>), grid, dim3(256), 0, stream, (T*)y, residual, (const P*)pending, splits,
                       (size_t)split_stride, (const T*)w, (const T*)b, alpha, rows, hidden, also, also_splits, (size_t)also_stride);
  } else {
    const dim3 grid(out_rows, (hidden + 255) / 256);
    hipLaunchKernelGGL((add_tanh_norm_kernel<T, P, 1>), grid, dim3(256), 0, stream, (T*)y, residual, (const P*)pending, splits,
                       (size_t)split_stride, (const T*)w, (const T*)b, alpha, rows, hidden, also, also_splits, (size_t)also_stride);
  }
}

extern "C" int ts_add_tanh_norm(void* y, float* residual, const void* pending, int pending_f32, int splits, long split_stride,
                                const void* w, const void* b, float alpha, const int* rows, int out_rows, int hidden,
                                int dtype, const float* also, int also_splits, long also_stride, hipStream_t stream) {
  if (out_rows == 0) return TS_OK;
  if (!y || !residual || !w || !b || hidden < 1 || splits < 1 || (also && also_splits < 1)) return TS_ERR_ARG;
  if (dtype == TS_F32)
    launch_add_tanh_norm<float, float>(y, residual, pending, splits, split_stride, w, b, alpha, rows, out_rows, hidden, also, also_splits, also_stride, stream);
  else if (dtype == TS_BF16 && pending_f32)
    launch_add_tanh_norm<bf16_t, float>(y, residual, pending, splits, split_stride, w, b, alpha, rows, out_rows, hidden, also, also_splits, also_stride, stream);
  else if (dtype == TS_BF16)
    launch_add_tanh_norm<bf16_t, bf16_t>(y, residual, pending, splits, split_stride, w, b, alpha, rows, out_rows, hidden, also, also_splits, also_stride, stream);
  else
    return TS_ERR_DTYPE;
  return ts_launch_status();
}

__global__ void __launch_bounds__(256) tanh_cap_kernel(float* __restrict__ x, size_t total, float cap) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < total) x[i] = cap * tanhf(x[i] / cap);
}

extern "C" int ts_tanh_cap(float* x, long total, float cap, hipStream_t stream) {
  if (total == 0) return TS_OK;
  if (!x || !(cap > 0.f)) return TS_ERR_ARG;
  hipLaunchKernelGGL(tanh_cap_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, x, (size_t)total, cap);
  return ts_launch_status();
}
