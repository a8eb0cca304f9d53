// A short causal convolution over time on each channel of a projection, with the last inputs of every
// request carried from step to step.
//
// `proj` is a projection output [T, width] of type T, or `splits` 32-bit partial sums `split_stride`
// elements apart that are added up here; the convolved channels are its columns first_col .. first_col +
// channels - 1.  y_t[c] = sum_j taps[c][j] * u_(t - K + 1 + j)[c], where u is the request's own sequence of
// inputs: those of this step's earlier rows, and before them the K - 1 inputs the request's state slot
// holds (state [slots, K - 1, channels] 32-bit, oldest first; zero for a request that starts).  With
// `activation` 1 the result goes through silu.  The result is [T, channels] of type T, or 32-bit.
//
// ts_short_conv computes every row of the step and leaves the state alone; ts_short_conv_carry, launched
// behind it, moves each request's last K - 1 inputs into its slot.  In a step whose requests all bring one
// token (`single`), the thread that computes a channel of a request also moves the channel's state on, and
// nothing is launched behind it.  Prompt portions in bfloat16 take four channels a thread with 8-byte
// accesses (short_conv_rows_kernel), the same arithmetic.
#include "common.hpp"

template <typename P>
__device__ __forceinline__ float sc_input(const P* p, int splits, size_t stride) {
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

#define SC_MAX_TAPS 8

template <typename T, typename P, typename O>
__global__ void __launch_bounds__(256)
short_conv_kernel(O* __restrict__ out, const P* __restrict__ proj, int splits, size_t split_stride, int width, int first_col,
                  int channels, const T* __restrict__ taps, int k,
                  float* state, const int* __restrict__ state_slots, const int* __restrict__ token_seq,
                  const int* __restrict__ query_start_loc, int activation, int single) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int t = blockIdx.x;
  const int seq = single ? t : token_seq[t];
  const int row0 = single ? t : query_start_loc[seq];
  const int index = t - row0;  // the token's place in its request's portion
  float* held = state + (size_t)state_slots[seq] * (k - 1) * channels + c;
  float y = 0.f;
  float mine = 0.f;  // the token's own input
#pragma unroll
  for (int j = 0; j < SC_MAX_TAPS; ++j) {
    if (j >= k) break;
    const int back = index - (k - 1) + j;
    const float u = back >= 0 ? sc_input(proj + (size_t)(row0 + back) * width + first_col + c, splits, split_stride)
                              : held[(size_t)(k - 1 + back) * channels];
    // In a step of single tokens the thread owns this channel of the request's state: every place takes
    // what the next one held, read just now.
    if (single && back < 0 && j > 0) held[(size_t)(j - 1) * channels] = u;
    if (j == k - 1) mine = u;
    y = fmaf(to_float(taps[(size_t)c * k + j]), u, y);
  }
  if (single && k > 1) held[(size_t)(k - 2) * channels] = mine;
  if (activation == 1) y = y / (1.f + expf(-y));
  out[(size_t)t * channels + c] = from_float<O>(y);
}

// Prompt portions: bfloat16 in, four neighbouring channels a thread, 8-byte loads of the inputs and of
// nothing else per tap (the taps of a thread's channels are read once).  Per element the arithmetic of the
// kernel above.
template <typename O, int K>
__global__ void __launch_bounds__(256)
short_conv_rows_kernel(O* __restrict__ out, const bf16_t* __restrict__ proj, int width, int first_col, int channels,
                       const bf16_t* __restrict__ taps, const float* __restrict__ state,
                       const int* __restrict__ state_slots, const int* __restrict__ token_seq,
                       const int* __restrict__ query_start_loc, int activation) {
  const int c = 4 * (blockIdx.y * blockDim.x + threadIdx.x);
  if (c >= channels) return;
  const int t = blockIdx.x;
  const int seq = token_seq[t];
  const int row0 = query_start_loc[seq];
  const int index = t - row0;
  constexpr int k = K;
  const float* held = state + (size_t)state_slots[seq] * (k - 1) * channels + c;
  float y[4] = {0.f, 0.f, 0.f, 0.f};
  // The 4 K taps of the thread's channels lie side by side: K loads of four.
  float w[4 * K];
#pragma unroll
  for (int f = 0; f < K; ++f) {
    const uint2 raw = *reinterpret_cast<const uint2*>(taps + (size_t)c * k + 4 * f);
    w[4 * f] = __uint_as_float(raw.x << 16);
    w[4 * f + 1] = __uint_as_float(raw.x & 0xffff0000u);
    w[4 * f + 2] = __uint_as_float(raw.y << 16);
    w[4 * f + 3] = __uint_as_float(raw.y & 0xffff0000u);
  }
#pragma unroll
  for (int j = 0; j < K; ++j) {
    const int back = index - (k - 1) + j;
    float u[4];
    if (back >= 0) {
      const uint2 raw = *reinterpret_cast<const uint2*>(proj + (size_t)(row0 + back) * width + first_col + c);
      u[0] = __uint_as_float(raw.x << 16);
      u[1] = __uint_as_float(raw.x & 0xffff0000u);
      u[2] = __uint_as_float(raw.y << 16);
      u[3] = __uint_as_float(raw.y & 0xffff0000u);
    } else {
      const float4 raw = *reinterpret_cast<const float4*>(held + (size_t)(k - 1 + back) * channels);
      u[0] = raw.x; u[1] = raw.y; u[2] = raw.z; u[3] = raw.w;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) y[e] = fmaf(w[e * K + j], u[e], y[e]);
  }
#pragma unroll
  for (int e = 0; e < 4; ++e)
    if (activation == 1) y[e] = y[e] / (1.f + expf(-y[e]));
  O* to = out + (size_t)t * channels + c;
  if constexpr (sizeof(O) == 4) {
    *reinterpret_cast<float4*>(to) = make_float4(y[0], y[1], y[2], y[3]);
  } else {
    uint2 packed;
    packed.x = (uint32_t)from_float<bf16_t>(y[0]).bits | ((uint32_t)from_float<bf16_t>(y[1]).bits << 16);
    packed.y = (uint32_t)from_float<bf16_t>(y[2]).bits | ((uint32_t)from_float<bf16_t>(y[3]).bits << 16);
    *reinterpret_cast<uint2*>(to) = packed;
  }
}

template <typename P>
__global__ void __launch_bounds__(256)
short_conv_carry_kernel(float* __restrict__ state, const P* __restrict__ proj, int splits, size_t split_stride, int width,
                        int first_col, int channels, int k, const int* __restrict__ state_slots,
                        const int* __restrict__ query_start_loc) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int seq = blockIdx.x;
  const int row0 = query_start_loc[seq];
  const int count = query_start_loc[seq + 1] - row0;
  float* held = state + (size_t)state_slots[seq] * (k - 1) * channels + c;
  // Place i takes the input count - (k - 1) + i of this step, or, where the step is shorter than the
  // state, the place i + count of what was held: a place further on, read before it is written.
  for (int i = 0; i < k - 1; ++i) {
    const int from = count - (k - 1) + i;
    held[(size_t)i * channels] = from >= 0 ? sc_input(proj + (size_t)(row0 + from) * width + first_col + c, splits, split_stride)
                                           : held[(size_t)(i + count) * channels];
  }
}

// dtype: the run's type (taps, and the projection unless it is partial sums); out_f32: a 32-bit result.
extern "C" int ts_short_conv(void* out, int out_f32, const void* proj, int in_f32, int splits, long split_stride, int width,
                             int first_col, int channels, const void* taps, int k, float* state,
                             const int* state_slots, const int* token_seq, const int* query_start_loc, int tokens,
                             int activation, int single, int dtype, hipStream_t stream) {
  if (tokens == 0) return TS_OK;
  if (!out || !proj || !taps || (!state && k > 1) || !state_slots || !token_seq || !query_start_loc) return TS_ERR_ARG;
  if (k < 1 || k > SC_MAX_TAPS || channels < 1 || first_col < 0 || first_col + channels > width || splits < 1) return TS_ERR_SHAPE;
  if (activation < 0 || activation > 1) return TS_ERR_ARG;
  const dim3 grid(tokens, (channels + 255) / 256), block(256);
  if (grid.y > 65535) return TS_ERR_SHAPE;
  if (dtype == TS_BF16 && !in_f32 && !single && tokens >= 32 && channels % 4 == 0 && width % 4 == 0 && first_col % 4 == 0 &&
      ((uintptr_t)proj | (uintptr_t)out | (uintptr_t)state | (uintptr_t)taps) % 16 == 0) {
    const dim3 wide(tokens, (channels / 4 + 255) / 256);
#define SC_ROWS(K)                                                                                                       \
  case K:                                                                                                                \
    if (out_f32)                                                                                                         \
      hipLaunchKernelGGL((short_conv_rows_kernel<float, K>), wide, block, 0, stream, (float*)out, (const bf16_t*)proj, width,       \
                         first_col, channels, (const bf16_t*)taps, state, state_slots, token_seq, query_start_loc, activation);  \
    else                                                                                                                 \
      hipLaunchKernelGGL((short_conv_rows_kernel<bf16_t, K>), wide, block, 0, stream, (bf16_t*)out, (const bf16_t*)proj, width,     \
                         first_col, channels, (const bf16_t*)taps, state, state_slots, token_seq, query_start_loc, activation);  \
    break;
    switch (k) {
      SC_ROWS(1) SC_ROWS(2) SC_ROWS(3) SC_ROWS(4) SC_ROWS(5) SC_ROWS(6) SC_ROWS(7) SC_ROWS(8)
    }
#undef SC_ROWS
    return ts_launch_status();
  }
#define SC_GO(T, P, O)                                                                                                   \
  hipLaunchKernelGGL((short_conv_kernel<T, P, O>), grid, block, 0, stream, (O*)out, (const P*)proj, splits, (size_t)split_stride, \
                     width, first_col, channels, (const T*)taps, k, state, state_slots, token_seq, query_start_loc, activation, single)
  if (dtype == TS_F32) SC_GO(float, float, float);
  else if (dtype == TS_BF16 && in_f32 && out_f32) SC_GO(bf16_t, float, float);
  else if (dtype == TS_BF16 && in_f32) SC_GO(bf16_t, float, bf16_t);
  else if (dtype == TS_BF16 && out_f32) SC_GO(bf16_t, bf16_t, float);
  else if (dtype == TS_BF16) SC_GO(bf16_t, bf16_t, bf16_t);
  else return TS_ERR_DTYPE;
#undef SC_GO
  return ts_launch_status();
}

extern "C" int ts_short_conv_carry(float* state, const void* proj, int in_f32, int splits, long split_stride, int width,
                                   int first_col, int channels, int k, const int* state_slots, const int* query_start_loc,
                                   int num_seqs, int dtype, hipStream_t stream) {
  if (num_seqs == 0 || k == 1) return TS_OK;  // one tap: nothing is carried
  if (!state || !proj || !state_slots || !query_start_loc) return TS_ERR_ARG;
  if (k < 1 || k > SC_MAX_TAPS || channels < 1 || first_col < 0 || first_col + channels > width || splits < 1) return TS_ERR_SHAPE;
  const dim3 grid(num_seqs, (channels + 255) / 256), block(256);
  if (grid.y > 65535) return TS_ERR_SHAPE;
  if (dtype == TS_F32 || in_f32)
    hipLaunchKernelGGL((short_conv_carry_kernel<float>), grid, block, 0, stream, state, (const float*)proj, splits,
                       (size_t)split_stride, width, first_col, channels, k, state_slots, query_start_loc);
  else if (dtype == TS_BF16)
    hipLaunchKernelGGL((short_conv_carry_kernel<bf16_t>), grid, block, 0, stream, state, (const bf16_t*)proj, splits,
                       (size_t)split_stride, width, first_col, channels, k, state_slots, query_start_loc);
  else
    return TS_ERR_DTYPE;
  return ts_launch_status();
}
