// The gated delta rule: per head and request a 32-bit state S [D, Dv] that every token decays, corrects
// and reads,
//     S <- diag(g) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q,
// with unit vectors k and q (q also times D^-1/2), a decay per key channel g = exp(-exp(A) softplus(a2 . low
// + dt)) and beta = sigmoid(.).  Everything here is 32-bit arithmetic.
//
// Three launches a step:
//   ts_delta_prepare  per token: q and k of every key head made unit vectors and their product k . q, the
//                     decays of every head from the low-rank input, beta;
//   ts_delta_scan     per (request, head, 32 value columns): the request's tokens in order, the state
//                     from and to the request's slot;
//   ts_delta_finish   per (token, head): o divided by its root mean square, times a gain [Dv] shared by
//                     the heads, times sigmoid(g2 . low'), rounded once to the run's type.
// `u` [T, 2 G D + H Dv] (32-bit) holds the convolved q | k | v; `proj` is the fused projection [T, width]
// of the run's type, or `splits` 32-bit partial sums, of which the columns named by *_at are read.
#include "common.hpp"

#define DS_MAX_LOW 128
#define DS_PARTS 8    // lanes that share a value column of the scan, each with a stretch of the state's rows
#define DS_COLS 32    // value columns of a workgroup of the scan
#define DS_BATCH 16   // tokens staged at a time

template <typename P>
__device__ __forceinline__ float ds_input(const P* p, int splits, size_t stride) {
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

// Block (t, item): item < G makes key head `item`'s unit q and k; item >= G the decays and beta of head
// item - G.
template <typename T, typename P>
__global__ void __launch_bounds__(64)
delta_prepare_kernel(float* __restrict__ qn, float* __restrict__ kn, float* __restrict__ kq, float* __restrict__ decay,
                     float* __restrict__ beta, const float* __restrict__ u, const P* __restrict__ proj, int splits, size_t split_stride, int width,
                     int beta_at, int low_at, int low, const T* __restrict__ a2, const T* __restrict__ dt_bias,
                     const float* __restrict__ a_log, int heads, int kv_heads, int dim, int vdim) {
  __shared__ float lows[DS_MAX_LOW];
  const int t = blockIdx.x, item = blockIdx.y, lane = threadIdx.x;
  const size_t u_width = (size_t)2 * kv_heads * dim + (size_t)heads * vdim;
  if (item < kv_heads) {
    const float* q = u + (size_t)t * u_width + (size_t)item * dim;
    const float* k = q + (size_t)kv_heads * dim;
    float qq = 0.f, kk = 0.f;
    for (int d = lane; d < dim; d += TS_WAVE) {
      qq = fmaf(q[d], q[d], qq);
      kk = fmaf(k[d], k[d], kk);
    }
    qq = wave_sum(qq);
    kk = wave_sum(kk);
    const float q_by = rsqrtf(qq + 1e-6f) * rsqrtf((float)dim), k_by = rsqrtf(kk + 1e-6f);
    const size_t at = ((size_t)t * kv_heads + item) * dim;
    float both = 0.f;
    for (int d = lane; d < dim; d += TS_WAVE) {
      const float qd = q[d] * q_by, kd = k[d] * k_by;
      qn[at + d] = qd;
      kn[at + d] = kd;
      both = fmaf(kd, qd, both);
    }
    both = wave_sum(both);
    if (lane == 0) kq[(size_t)t * kv_heads + item] = both;
    return;
  }
  const int h = item - kv_heads;
  const P* row = proj + (size_t)t * width;
  for (int r = lane; r < low; r += TS_WAVE) lows[r] = ds_input(row + low_at + r, splits, split_stride);
  __syncthreads();
  if (lane == 0) beta[(size_t)t * heads + h] = 1.f / (1.f + expf(-ds_input(row + beta_at + h, splits, split_stride)));
  const float rate = expf(a_log[h]);
  for (int d = lane; d < dim; d += TS_WAVE) {
    const size_t channel = (size_t)h * dim + d;
    const T* w = a2 + channel * low;
    float z = to_float(dt_bias[channel]);
    for (int r = 0; r < low; ++r) z = fmaf(to_float(w[r]), lows[r], z);
    const float step = z > 20.f ? z : log1pf(expf(z));
    decay[((size_t)t * heads + h) * dim + d] = expf(-rate * step);
  }
}

// NR: state rows a thread holds.  Eight neighbouring lanes share a value column; lane part p of them
// holds rows p NR .. p NR + NR - 1 (rows from `dim` on are padding and stay zero).
template <int NR>
__global__ void __launch_bounds__(DS_PARTS * DS_COLS)
delta_scan_kernel(float* __restrict__ o, float* __restrict__ state, const float* __restrict__ qn, const float* __restrict__ kn,
                  const float* __restrict__ kq, const float* __restrict__ decay, const float* __restrict__ beta,
                  const float* __restrict__ u, const int* __restrict__ state_slots, const int* __restrict__ query_start_loc,
                  int first_seq, int heads, int kv_heads, int dim, int vdim) {
  constexpr int ROWS = DS_PARTS * NR;
  __shared__ __attribute__((aligned(16))) float ks[DS_BATCH][ROWS];
  __shared__ __attribute__((aligned(16))) float qs[DS_BATCH][ROWS];
  __shared__ __attribute__((aligned(16))) float gs[DS_BATCH][ROWS];
  __shared__ float vs[DS_BATCH][DS_COLS];
  __shared__ float bs[DS_BATCH], kqs[DS_BATCH];
  const int seq = first_seq + blockIdx.x, h = blockIdx.y;
  const int g = h / (heads / kv_heads);
  const int tid = threadIdx.x;
  const int part = tid % DS_PARTS, col_in = tid / DS_PARTS;
  const int c = blockIdx.z * DS_COLS + col_in;
  const bool live = c < vdim;
  const int row0 = query_start_loc[seq], count = query_start_loc[seq + 1] - row0;
  const size_t u_width = (size_t)2 * kv_heads * dim + (size_t)heads * vdim;
  float* held = state + ((size_t)state_slots[seq] * heads + h) * dim * vdim;
  float s[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int d = part * NR + i;
    s[i] = (live && d < dim) ? held[(size_t)d * vdim + c] : 0.f;
  }
  for (int base = 0; base < count; base += DS_BATCH) {
    const int batch = min(DS_BATCH, count - base);
    __syncthreads();  // the batch before has been read
    for (int i = tid; i < batch * ROWS; i += blockDim.x) {
      const int j = i / ROWS, d = i % ROWS;
      const size_t t = (size_t)(row0 + base + j);
      const bool in = d < dim;
      ks[j][d] = in ? kn[(t * kv_heads + g) * dim + d] : 0.f;
      qs[j][d] = in ? qn[(t * kv_heads + g) * dim + d] : 0.f;
      gs[j][d] = in ? decay[(t * heads + h) * dim + d] : 0.f;
    }
    for (int i = tid; i < batch * DS_COLS; i += blockDim.x) {
      const int j = i / DS_COLS, cc = blockIdx.z * DS_COLS + i % DS_COLS;
      vs[j][i % DS_COLS] = cc < vdim ? u[(size_t)(row0 + base + j) * u_width + (size_t)2 * kv_heads * dim + (size_t)h * vdim + cc] : 0.f;
    }
    if (tid < batch) {
      bs[tid] = beta[(size_t)(row0 + base + tid) * heads + h];
      kqs[tid] = kq[(size_t)(row0 + base + tid) * kv_heads + g];
    }
    __syncthreads();
    for (int j = 0; j < batch; ++j) {
      // One pass decays the rows and forms what the key and the query read of the decayed state (four
      // running sums each, so that the additions do not wait for one another); the token's own write
      // reaches the read-out through k . q: o = (gS)^T q + w (k . q).
      float rk[4] = {0.f, 0.f, 0.f, 0.f}, rq[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < NR; i += 4) {
        const float4 kk = *reinterpret_cast<const float4*>(&ks[j][part * NR + i]);
        const float4 qq = *reinterpret_cast<const float4*>(&qs[j][part * NR + i]);
        const float4 gg = *reinterpret_cast<const float4*>(&gs[j][part * NR + i]);
        s[i] *= gg.x; s[i + 1] *= gg.y; s[i + 2] *= gg.z; s[i + 3] *= gg.w;
        rk[0] = fmaf(s[i], kk.x, rk[0]); rk[1] = fmaf(s[i + 1], kk.y, rk[1]);
        rk[2] = fmaf(s[i + 2], kk.z, rk[2]); rk[3] = fmaf(s[i + 3], kk.w, rk[3]);
        rq[0] = fmaf(s[i], qq.x, rq[0]); rq[1] = fmaf(s[i + 1], qq.y, rq[1]);
        rq[2] = fmaf(s[i + 2], qq.z, rq[2]); rq[3] = fmaf(s[i + 3], qq.w, rq[3]);
      }
      float read_k = (rk[0] + rk[1]) + (rk[2] + rk[3]), read_q = (rq[0] + rq[1]) + (rq[2] + rq[3]);
      // Over the eight lanes of the column.
      read_k += lanes_moved<0xB1, 0xF>(0.f, read_k);
      read_q += lanes_moved<0xB1, 0xF>(0.f, read_q);
      read_k += lanes_moved<0x4E, 0xF>(0.f, read_k);
      read_q += lanes_moved<0x4E, 0xF>(0.f, read_q);
      read_k += lanes_moved<0x141, 0xF>(0.f, read_k);
      read_q += lanes_moved<0x141, 0xF>(0.f, read_q);
      const float write = bs[j] * (vs[j][col_in] - read_k);
#pragma unroll
      for (int i = 0; i < NR; i += 4) {
        const float4 kk = *reinterpret_cast<const float4*>(&ks[j][part * NR + i]);
        s[i] = fmaf(kk.x, write, s[i]); s[i + 1] = fmaf(kk.y, write, s[i + 1]);
        s[i + 2] = fmaf(kk.z, write, s[i + 2]); s[i + 3] = fmaf(kk.w, write, s[i + 3]);
      }
      if (part == 0 && live) o[((size_t)(row0 + base + j) * heads + h) * vdim + c] = fmaf(write, kqs[j], read_q);
    }
  }
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int d = part * NR + i;
    if (live && d < dim) held[(size_t)d * vdim + c] = s[i];
  }
}

template <typename T, typename P>
__global__ void __launch_bounds__(64)
delta_finish_kernel(T* __restrict__ y, const float* __restrict__ o, const P* __restrict__ proj, int splits, size_t split_stride,
                    int width, int low_at, int low, const T* __restrict__ g2, const T* __restrict__ gain, float eps, int heads,
                    int vdim) {
  __shared__ float lows[DS_MAX_LOW];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const P* row = proj + (size_t)t * width;
  for (int r = lane; r < low; r += TS_WAVE) lows[r] = ds_input(row + low_at + r, splits, split_stride);
  __syncthreads();
  const float* mine = o + ((size_t)t * heads + h) * vdim;
  float ss = 0.f;
  for (int c = lane; c < vdim; c += TS_WAVE) ss = fmaf(mine[c], mine[c], ss);
  ss = wave_sum(ss);
  const float by = rsqrtf(ss / (float)vdim + eps);
  for (int c = lane; c < vdim; c += TS_WAVE) {
    const T* w = g2 + ((size_t)h * vdim + c) * low;
    float z = 0.f;
    for (int r = 0; r < low; ++r) z = fmaf(to_float(w[r]), lows[r], z);
    y[((size_t)t * heads + h) * vdim + c] = from_float<T>(mine[c] * by * to_float(gain[c]) / (1.f + expf(-z)));
  }
}

extern "C" int ts_delta_prepare(float* qn, float* kn, float* kq, float* decay, float* beta, const float* u, const void* proj, int in_f32,
                                int splits, long split_stride, int width, int beta_at, int low_at, int low, const void* a2,
                                const void* dt_bias, const float* a_log, int tokens, int heads, int kv_heads, int dim, int vdim,
                                int dtype, hipStream_t stream) {
  if (tokens == 0) return TS_OK;
  if (!qn || !kn || !kq || !decay || !beta || !u || !proj || !a2 || !dt_bias || !a_log) return TS_ERR_ARG;
  if (heads < 1 || kv_heads < 1 || heads % kv_heads != 0 || heads + kv_heads > 65535 || dim < 1 || vdim < 1 || low < 1 ||
      low > DS_MAX_LOW || splits < 1 || beta_at < 0 || beta_at + heads > width || low_at < 0 || low_at + low > width)
    return TS_ERR_SHAPE;
  const dim3 grid(tokens, kv_heads + heads), block(64);
#define DS_GO(T, P)                                                                                                      \
  hipLaunchKernelGGL((delta_prepare_kernel<T, P>), grid, block, 0, stream, qn, kn, kq, decay, beta, u, (const P*)proj, splits, \
                     (size_t)split_stride, width, beta_at, low_at, low, (const T*)a2, (const T*)dt_bias, a_log, heads,    \
                     kv_heads, dim, vdim)
  if (dtype == TS_F32) DS_GO(float, float);
  else if (dtype == TS_BF16 && in_f32) DS_GO(bf16_t, float);
  else if (dtype == TS_BF16) DS_GO(bf16_t, bf16_t);
  else return TS_ERR_DTYPE;
#undef DS_GO
  return ts_launch_status();
}

extern "C" int ts_delta_scan(float* o, float* state, const float* qn, const float* kn, const float* kq, const float* decay, const float* beta,
                             const float* u, const int* state_slots, const int* query_start_loc, int first_seq, int num_seqs,
                             int heads, int kv_heads, int dim, int vdim, hipStream_t stream) {
  if (num_seqs == 0) return TS_OK;
  if (!o || !state || !qn || !kn || !kq || !decay || !beta || !u || !state_slots || !query_start_loc) return TS_ERR_ARG;
  if (heads < 1 || kv_heads < 1 || heads % kv_heads != 0 || heads > 65535 || dim < 1 || dim > 256 || vdim < 1) return TS_ERR_SHAPE;
  const dim3 grid(num_seqs, heads, (vdim + DS_COLS - 1) / DS_COLS), block(DS_PARTS * DS_COLS);
  if (grid.z > 65535) return TS_ERR_SHAPE;
#define DS_GO(NR)                                                                                                     \
  hipLaunchKernelGGL((delta_scan_kernel<NR>), grid, block, 0, stream, o, state, qn, kn, kq, decay, beta, u, state_slots,  \
                     query_start_loc, first_seq, heads, kv_heads, dim, vdim)
  if (dim <= 32) DS_GO(4);
  else if (dim <= 64) DS_GO(8);
  else if (dim <= 128) DS_GO(16);
  else DS_GO(32);
#undef DS_GO
  return ts_launch_status();
}

extern "C" int ts_delta_finish(void* y, const float* o, const void* proj, int in_f32, int splits, long split_stride, int width,
                               int low_at, int low, const void* g2, const void* gain, float eps, int tokens, int heads, int vdim,
                               int dtype, hipStream_t stream) {
  if (tokens == 0) return TS_OK;
  if (!y || !o || !proj || !g2 || !gain) return TS_ERR_ARG;
  if (heads < 1 || heads > 65535 || vdim < 1 || low < 1 || low > DS_MAX_LOW || splits < 1 || low_at < 0 || low_at + low > width)
    return TS_ERR_SHAPE;
  const dim3 grid(tokens, heads), block(64);
#define DS_GO(T, P)                                                                                                   \
  hipLaunchKernelGGL((delta_finish_kernel<T, P>), grid, block, 0, stream, (T*)y, o, (const P*)proj, splits,            \
                     (size_t)split_stride, width, low_at, low, (const T*)g2, (const T*)gain, eps, heads, vdim)
  if (dtype == TS_F32) DS_GO(float, float);
  else if (dtype == TS_BF16 && in_f32) DS_GO(bf16_t, float);
  else if (dtype == TS_BF16) DS_GO(bf16_t, bf16_t);
  else return TS_ERR_DTYPE;
#undef DS_GO
  return ts_launch_status();
}
