// The gated delta rule: per head and request a 32-bit state S [D, Dv] that every token decays, corrects
// and reads,
//     S <- diag(g) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q,
// with unit vectors k and q (q also times D^-1/2), a decay per key channel g = exp(-exp(A) softplus(a2 . low
// + dt)) and beta = sigmoid(.).  Everything here is 32-bit arithmetic.
//
// Three launches a step:
//   ts_delta_prepare  per token: q and k of every key head made unit vectors and their product k . q, the
//                     decays of every head from the low-rank input, beta;
//   ts_delta_scan     per (request, head, 8 or 32 value columns): the request's tokens in order, the state
//                     from and to the request's slot;
//   ts_delta_finish   per (token, head): o divided by its root mean square, times a gain [Dv] shared by
//                     the heads, times sigmoid(g2 . low') (and a scale), rounded once to the run's type; its
//                     rows may be a part of a wider buffer's.
// Of the two low-rank matrices a2 [H D, R] and g2 [H Dv, R'] a lane walks its channel's row; over a prompt a
// wavefront of the launches around the walk takes eight tokens, so that it reads its rows once for all eight (in a
// step of few tokens: one token each).
// `u` [T, 2 G D + H Dv] (32-bit) holds the convolved q | k | v; `proj` is the fused projection [T, width]
// of the run's type, or `splits` 32-bit partial sums, of which the columns named by *_at are read.
#include "common.hpp"

#define DS_MAX_LOW 256

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

// A workgroup of four wavefronts, each with an item of its own.  The first `qk_blocks` workgroups make unit q
// and k: item = (token, key head).  The others make decays and beta: item = (tile of DS_TOKENS tokens, head).
// A lane walks its channel's row of the low-rank matrix once (neighbouring elements: wide loads) for all the
// tile's tokens, whose low-rank inputs lie side by side in the wavefront's own stretch of LDS.
#define DS_ITEMS 4
template <typename T, typename P, int DS_TOKENS>
__global__ void __launch_bounds__(64 * DS_ITEMS)
delta_prepare_kernel(float* __restrict__ qn, float* __restrict__ kn, float* __restrict__ kq, float* __restrict__ decay,
                     float* __restrict__ beta, const float* __restrict__ u, const P* __restrict__ proj, int splits, size_t split_stride, int width,
                     int beta_at, int low_at, int low, const T* __restrict__ a2, const T* __restrict__ dt_bias,
                     const float* __restrict__ a_log, int tokens, int heads, int kv_heads, int dim, int vdim, int qk_blocks) {
  __shared__ __attribute__((aligned(16))) float lows_of[DS_ITEMS][DS_MAX_LOW][DS_TOKENS];  // the tokens of a tile side by side
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x % TS_WAVE;
  const size_t u_width = (size_t)2 * kv_heads * dim + (size_t)heads * vdim;
  if ((int)blockIdx.x < qk_blocks) {
    const long item = (long)blockIdx.x * DS_ITEMS + wave;
    if (item >= (long)tokens * kv_heads) return;
    const int t = (int)(item / kv_heads), g = (int)(item % kv_heads);
    const float* q = u + (size_t)t * u_width + (size_t)g * dim;
    const float* k = q + (size_t)kv_heads * dim;
    float qq = 0.f, kk = 0.f;
    for (int d = lane; d < dim; d += TS_WAVE) {
      qq = fmaf(q[d], q[d], qq);
      kk = fmaf(k[d], k[d], kk);
    }
    qq = wave_sum(qq);
    kk = wave_sum(kk);
    const float q_by = rsqrtf(qq + 1e-6f) * rsqrtf((float)dim), k_by = rsqrtf(kk + 1e-6f);
    const size_t at = ((size_t)t * kv_heads + g) * dim;
    float both = 0.f;
    for (int d = lane; d < dim; d += TS_WAVE) {
      const float qd = q[d] * q_by, kd = k[d] * k_by;
      qn[at + d] = qd;
      kn[at + d] = kd;
      both = fmaf(kd, qd, both);
    }
    both = wave_sum(both);
    if (lane == 0) kq[(size_t)t * kv_heads + g] = both;
    return;
  }
  // (Every wavefront of such a workgroup reaches the barrier; one without an item does nothing around it.)
  const int tiles = (tokens + DS_TOKENS - 1) / DS_TOKENS;
  const long item = (long)((int)blockIdx.x - qk_blocks) * DS_ITEMS + wave;
  const bool mine = item < (long)tiles * heads;
  const int h = mine ? (int)(item % heads) : 0;
  const int t0 = mine ? (int)(item / heads) * DS_TOKENS : 0;
  const int count = mine ? min(DS_TOKENS, tokens - t0) : 0;
  float (*lows)[DS_TOKENS] = lows_of[wave];
  for (int i = lane; i < DS_TOKENS * low; i += TS_WAVE) {
    const int tt = i / low, r = i % low;
    lows[r][tt] = tt < count ? ds_input(proj + (size_t)(t0 + tt) * width + low_at + r, splits, split_stride) : 0.f;
  }
  __syncthreads();
  if (!mine) return;
  if (lane < count)
    beta[(size_t)(t0 + lane) * heads + h] = 1.f / (1.f + expf(-ds_input(proj + (size_t)(t0 + lane) * width + beta_at + h, splits, split_stride)));
  const float rate = expf(a_log[h]);
  for (int d = lane; d < dim; d += TS_WAVE) {
    const size_t channel = (size_t)h * dim + d;
    const T* w = a2 + channel * low;
    float z[DS_TOKENS];
#pragma unroll
    for (int tt = 0; tt < DS_TOKENS; ++tt) z[tt] = to_float(dt_bias[channel]);
    for (int r = 0; r < low; ++r) {
      const float wr = to_float(w[r]);
#pragma unroll
      for (int tt = 0; tt < DS_TOKENS; ++tt) z[tt] = fmaf(wr, lows[r][tt], z[tt]);
    }
#pragma unroll
    for (int tt = 0; tt < DS_TOKENS; ++tt) {
      if (tt < count) {
        const float step = z[tt] > 20.f ? z[tt] : log1pf(expf(z[tt]));
        decay[((size_t)(t0 + tt) * heads + h) * dim + d] = expf(-rate * step);
      }
    }
  }
}

// NR: state rows a thread holds; BATCH: tokens staged at a time.  DS_PARTS (8 or 16) neighbouring lanes
// share a value column; lane part p of them holds, of every stretch of 4 DS_PARTS rows, the four rows from
// 4 p on, so that the lanes of a column read neighbouring 16-byte pieces of a staged vector (rows from `dim`
// on are padding and stay zero); a workgroup owns DS_COLS columns.  A batch's k, q, decays, values, beta and k . q
// travel global memory -> registers -> LDS; the loads of the next batch are in flight while this one is
// walked, and LDS holds two batches so that one barrier a batch is enough.
//
// A token costs every wavefront the same chain of instructions whatever it owns, and every lane reads its
// rows of k, q and the decays from LDS, so what bounds a long walk is how thinly the state is spread: 16
// lanes a column and 8 columns a workgroup give a head of 128 x 128 to 16 workgroups of two wavefronts
// (prompt portions); single tokens, which read and write the state once, take 8 lanes a column and 32
// columns a workgroup, whose rows of the state are whole cache lines.
template <int NR, int BATCH, int DS_PARTS, int DS_COLS>
__global__ void __launch_bounds__(DS_PARTS * DS_COLS)
delta_scan_kernel(float* __restrict__ o, float* __restrict__ state, const float* __restrict__ qn, const float* __restrict__ kn,
                  const float* __restrict__ kq, const float* __restrict__ decay, const float* __restrict__ beta,
                  const float* __restrict__ u, const int* __restrict__ state_slots, const int* __restrict__ query_start_loc,
                  int first_seq, int heads, int kv_heads, int dim, int vdim) {
  constexpr int ROWS = DS_PARTS * NR;
  constexpr int THREADS = DS_PARTS * DS_COLS;
  constexpr int MINE = BATCH * ROWS / THREADS;          // elements of each of k, q, g a thread fetches
  constexpr int MINE_V = BATCH * DS_COLS / THREADS > 0 ? BATCH * DS_COLS / THREADS : 1;
  static_assert(BATCH * ROWS % THREADS == 0 && BATCH <= THREADS, "a batch is shared out evenly");
  __shared__ __attribute__((aligned(16))) float ks[2][BATCH][ROWS];
  __shared__ __attribute__((aligned(16))) float qs[2][BATCH][ROWS];
  __shared__ __attribute__((aligned(16))) float gs[2][BATCH][ROWS];
  __shared__ float vs[2][BATCH][DS_COLS];
  __shared__ float bs[2][BATCH], kqs[2][BATCH];
  __shared__ __attribute__((aligned(16))) float read_q_of[BATCH][THREADS];  // per token and lane: what the query reads of the lane's rows
  __shared__ float write_of[BATCH][DS_COLS];
  const int seq = first_seq + blockIdx.x, h = blockIdx.y;
  const int g = h / (heads / kv_heads);
  const int tid = threadIdx.x;
  const int part = tid % DS_PARTS, col_in = tid / DS_PARTS;
  const int c = blockIdx.z * DS_COLS + col_in;
  const bool live = c < vdim;
  const int row0 = query_start_loc[seq], count = query_start_loc[seq + 1] - row0;
  const size_t u_width = (size_t)2 * kv_heads * dim + (size_t)heads * vdim;
  float* held = state + ((size_t)state_slots[seq] * heads + h) * dim * vdim;
  // Row of the state that element i of this lane's registers holds.
  auto row_of = [&](int i) { return (i / 4) * (4 * DS_PARTS) + part * 4 + i % 4; };
  float s[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int d = row_of(i);
    s[i] = (live && d < dim) ? held[(size_t)d * vdim + c] : 0.f;
  }
  float pk[MINE], pq[MINE], pg[MINE], pv[MINE_V], pb = 0.f, pkq = 0.f;
  auto fetch = [&](int base) __attribute__((always_inline)) {
    const int batch = min(BATCH, count - base);
#pragma unroll
    for (int e = 0; e < MINE; ++e) {
      const int i = tid + e * THREADS;
      const int j = i / ROWS, d = i % ROWS;
      const bool in = j < batch && d < dim;
      const size_t t = (size_t)(row0 + base + (in ? j : 0));
      const int dd = in ? d : 0;
      const float a = kn[(t * kv_heads + g) * dim + dd], b = qn[(t * kv_heads + g) * dim + dd], cc = decay[(t * heads + h) * dim + dd];
      pk[e] = in ? a : 0.f;
      pq[e] = in ? b : 0.f;
      pg[e] = in ? cc : 0.f;
    }
#pragma unroll
    for (int e = 0; e < MINE_V; ++e) {
      const int i = tid + e * THREADS;
      const int j = i / DS_COLS, cc = blockIdx.z * DS_COLS + i % DS_COLS;
      const bool in = i < BATCH * DS_COLS && j < batch && cc < vdim;
      const float a = u[(size_t)(row0 + base + (in ? j : 0)) * u_width + (size_t)2 * kv_heads * dim + (size_t)h * vdim + (in ? cc : 0)];
      pv[e] = in ? a : 0.f;
    }
    const bool mine = tid < batch;
    const size_t t = (size_t)(row0 + base + (mine ? tid : 0));
    const float a = beta[t * heads + h], b = kq[t * kv_heads + g];
    pb = mine ? a : 0.f;
    pkq = mine ? b : 0.f;
  };
  auto stage = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int e = 0; e < MINE; ++e) {
      const int i = tid + e * THREADS;
      ks[buf][i / ROWS][i % ROWS] = pk[e];
      qs[buf][i / ROWS][i % ROWS] = pq[e];
      gs[buf][i / ROWS][i % ROWS] = pg[e];
    }
#pragma unroll
    for (int e = 0; e < MINE_V; ++e) {
      const int i = tid + e * THREADS;
      if (i < BATCH * DS_COLS) vs[buf][i / DS_COLS][i % DS_COLS] = pv[e];
    }
    if (tid < BATCH) {
      bs[buf][tid] = pb;
      kqs[buf][tid] = pkq;
    }
  };
  if (count > 0) fetch(0);
  int buf = 0;
  float* o_at = o + ((size_t)row0 * heads + h) * vdim + c;  // this column's output of the token being walked
  const size_t o_step = (size_t)heads * vdim;
  constexpr int Q = NR / 4;
  for (int base = 0; base < count; base += BATCH, buf ^= 1) {
    const int batch = min(BATCH, count - base);
    stage(buf);  // (the other buffer's readers were let go by the barrier of the batch before)
    __syncthreads();
    // In flight while this batch is walked; asked for unconditionally (behind the last batch: the last
    // token again, which nobody stages), so that no wait for it is placed inside the walk.
    fetch(min(base + BATCH, count - 1));
    // A token's vectors are read from LDS while the token before it is walked (two sets of registers in
    // turn).  What the query reads is left in LDS lane by lane and summed over a column's lanes behind the
    // batch, all tokens side by side: only the key's read-out, which the state's update waits for, crosses
    // lanes inside the walk.
    float4 ka[Q], qa[Q], ga[Q], kb[Q], qb[Q], gb[Q];
    float va, ba, vb, bb;
    auto read = [&](int j, float4* k4, float4* q4, float4* g4, float& v1, float& b1) __attribute__((always_inline)) {
#pragma unroll
      for (int x = 0; x < Q; ++x) {
        k4[x] = *reinterpret_cast<const float4*>(&ks[buf][j][x * 4 * DS_PARTS + part * 4]);
        q4[x] = *reinterpret_cast<const float4*>(&qs[buf][j][x * 4 * DS_PARTS + part * 4]);
        g4[x] = *reinterpret_cast<const float4*>(&gs[buf][j][x * 4 * DS_PARTS + part * 4]);
      }
      v1 = vs[buf][j][col_in];
      b1 = bs[buf][j];
    };
    auto token = [&](int j, const float4* kk, const float4* qq, const float4* gg, float vv, float beta_j) __attribute__((always_inline)) {
      // One pass decays the rows and forms what the key and the query read of the decayed state (four
      // running sums each, so that the additions do not wait for one another); the token's own write
      // reaches the read-out through k . q: o = (gS)^T q + w (k . q).
      float rk[4] = {0.f, 0.f, 0.f, 0.f}, rq[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int x = 0; x < Q; ++x) {
        const int i = 4 * x;
        s[i] *= gg[x].x; s[i + 1] *= gg[x].y; s[i + 2] *= gg[x].z; s[i + 3] *= gg[x].w;
        rk[0] = fmaf(s[i], kk[x].x, rk[0]); rk[1] = fmaf(s[i + 1], kk[x].y, rk[1]);
        rk[2] = fmaf(s[i + 2], kk[x].z, rk[2]); rk[3] = fmaf(s[i + 3], kk[x].w, rk[3]);
        rq[0] = fmaf(s[i], qq[x].x, rq[0]); rq[1] = fmaf(s[i + 1], qq[x].y, rq[1]);
        rq[2] = fmaf(s[i + 2], qq[x].z, rq[2]); rq[3] = fmaf(s[i + 3], qq[x].w, rq[3]);
      }
      float read_k = (rk[0] + rk[1]) + (rk[2] + rk[3]);
      read_q_of[j][tid] = (rq[0] + rq[1]) + (rq[2] + rq[3]);
      // Over the lanes of the column.
      read_k += lanes_moved<0xB1, 0xF>(0.f, read_k);
      read_k += lanes_moved<0x4E, 0xF>(0.f, read_k);
      read_k += lanes_moved<0x141, 0xF>(0.f, read_k);
      if (DS_PARTS == 16) read_k += lanes_moved<0x140, 0xF>(0.f, read_k);  // the two halves of a row of lanes
      const float write = beta_j * (vv - read_k);
      write_of[j][col_in] = write;  // (every lane of the column writes the same number)
#pragma unroll
      for (int x = 0; x < Q; ++x) {
        const int i = 4 * x;
        s[i] = fmaf(kk[x].x, write, s[i]); s[i + 1] = fmaf(kk[x].y, write, s[i + 1]);
        s[i + 2] = fmaf(kk[x].z, write, s[i + 2]); s[i + 3] = fmaf(kk[x].w, write, s[i + 3]);
      }
    };
    read(0, ka, qa, ga, va, ba);
    for (int j = 0; j < batch; j += 2) {
      read(min(j + 1, batch - 1), kb, qb, gb, vb, bb);
      token(j, ka, qa, ga, va, ba);
      if (j + 1 < batch) {
        read(min(j + 2, batch - 1), ka, qa, ga, va, ba);
        token(j + 1, kb, qb, gb, vb, bb);
      }
    }
    // The batch's outputs: lane `part` of a column sums what the column's lanes left for the tokens part,
    // part + DS_PARTS, ..  (A column's lanes are one wavefront's, whose LDS accesses keep their order.)
    for (int j = part; j < batch; j += DS_PARTS) {
      float sum = 0.f;
#pragma unroll
      for (int x = 0; x < DS_PARTS / 4; ++x) {
        const float4 piece = *reinterpret_cast<const float4*>(&read_q_of[j][col_in * DS_PARTS + 4 * x]);
        sum += (piece.x + piece.y) + (piece.z + piece.w);
      }
      if (live) o_at[(size_t)j * o_step] = fmaf(write_of[j][col_in], kqs[buf][j], sum);
    }
    o_at += (size_t)batch * o_step;
  }
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int d = row_of(i);
    if (live && d < dim) held[(size_t)d * vdim + c] = s[i];
  }
}

// Four wavefronts a workgroup, each with an item (tile of DS_TOKENS tokens, head) of its own.
template <typename T, typename P, int DS_TOKENS>
__global__ void __launch_bounds__(64 * DS_ITEMS)
delta_finish_kernel(T* __restrict__ y, const float* __restrict__ o, const P* __restrict__ proj, int splits, size_t split_stride,
                    int width, int low_at, int low, const T* __restrict__ g2, const T* __restrict__ gain, float eps, int tokens,
                    int heads, int vdim, float scale, size_t out_stride) {
  __shared__ __attribute__((aligned(16))) float lows_of[DS_ITEMS][DS_MAX_LOW][DS_TOKENS];
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x % TS_WAVE;
  const int tiles = (tokens + DS_TOKENS - 1) / DS_TOKENS;
  const long item = (long)blockIdx.x * DS_ITEMS + wave;
  const bool mine = item < (long)tiles * heads;
  const int h = mine ? (int)(item % heads) : 0;
  const int t0 = mine ? (int)(item / heads) * DS_TOKENS : 0;
  const int count = mine ? min(DS_TOKENS, tokens - t0) : 0;
  float (*lows)[DS_TOKENS] = lows_of[wave];
  for (int i = lane; i < DS_TOKENS * low; i += TS_WAVE) {
    const int tt = i / low, r = i % low;
    lows[r][tt] = tt < count ? ds_input(proj + (size_t)(t0 + tt) * width + low_at + r, splits, split_stride) : 0.f;
  }
  __syncthreads();
  if (!mine) return;
  float by[DS_TOKENS];
#pragma unroll
  for (int tt = 0; tt < DS_TOKENS; ++tt) {
    const float* mine_o = o + ((size_t)(t0 + min(tt, count - 1)) * heads + h) * vdim;
    float ss = 0.f;
    for (int c = lane; c < vdim; c += TS_WAVE) ss = fmaf(mine_o[c], mine_o[c], ss);
    ss = wave_sum(ss);
    by[tt] = rsqrtf(ss / (float)vdim + eps);
  }
  for (int c = lane; c < vdim; c += TS_WAVE) {
    const T* w = g2 + ((size_t)h * vdim + c) * low;
    float z[DS_TOKENS];
#pragma unroll
    for (int tt = 0; tt < DS_TOKENS; ++tt) z[tt] = 0.f;
    for (int r = 0; r < low; ++r) {
      const float wr = to_float(w[r]);
#pragma unroll
      for (int tt = 0; tt < DS_TOKENS; ++tt) z[tt] = fmaf(wr, lows[r][tt], z[tt]);
    }
    const float g = to_float(gain[c]);
#pragma unroll
    for (int tt = 0; tt < DS_TOKENS; ++tt) {
      if (tt < count) {
        const size_t at = ((size_t)(t0 + tt) * heads + h) * vdim + c;
        y[(size_t)(t0 + tt) * out_stride + (size_t)h * vdim + c] = from_float<T>(scale * o[at] * by[tt] * g / (1.f + expf(-z[tt])));
      }
    }
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
  // Eight tokens a tile over a prompt; one in a step of few tokens, whose workgroups are few anyway.
  const int per = tokens >= 64 ? 8 : 1;
  const int qk_blocks = (int)(((long)tokens * kv_heads + DS_ITEMS - 1) / DS_ITEMS);
  const long decay_items = (long)((tokens + per - 1) / per) * heads;
  const dim3 grid((unsigned)(qk_blocks + (decay_items + DS_ITEMS - 1) / DS_ITEMS)), block(64 * DS_ITEMS);
#define DS_ARGS(T, P)                                                                                                    \
  grid, block, 0, stream, qn, kn, kq, decay, beta, u, (const P*)proj, splits, (size_t)split_stride, width, beta_at, low_at, \
      low, (const T*)a2, (const T*)dt_bias, a_log, tokens, heads, kv_heads, dim, vdim, qk_blocks
#define DS_GO(T, P)                                                                                                      \
  if (per == 8)                                                                                                          \
    hipLaunchKernelGGL((delta_prepare_kernel<T, P, 8>), DS_ARGS(T, P));                                                  \
  else                                                                                                                   \
    hipLaunchKernelGGL((delta_prepare_kernel<T, P, 1>), DS_ARGS(T, P))
  if (dtype == TS_F32) DS_GO(float, float);
  else if (dtype == TS_BF16 && in_f32) DS_GO(bf16_t, float);
  else if (dtype == TS_BF16) DS_GO(bf16_t, bf16_t);
  else return TS_ERR_DTYPE;
#undef DS_GO
  return ts_launch_status();
}

extern "C" int ts_delta_scan(float* o, float* state, const float* qn, const float* kn, const float* kq, const float* decay, const float* beta,
                             const float* u, const int* state_slots, const int* query_start_loc, int first_seq, int num_seqs,
                             int heads, int kv_heads, int dim, int vdim, int spread, hipStream_t stream) {
  if (num_seqs == 0) return TS_OK;
  if (!o || !state || !qn || !kn || !kq || !decay || !beta || !u || !state_slots || !query_start_loc) return TS_ERR_ARG;
  if (heads < 1 || kv_heads < 1 || heads % kv_heads != 0 || heads > 65535 || dim < 1 || dim > 256 || vdim < 1) return TS_ERR_SHAPE;
  // `spread` (prompt portions): the state spread thinly; else whole cache lines of the state a workgroup.
#define DS_GO(NR, BATCH, PARTS, COLS)                                                                                 \
  do {                                                                                                                \
    const dim3 grid(num_seqs, heads, (vdim + COLS - 1) / COLS), block(PARTS * COLS);                                  \
    if (grid.z > 65535) return TS_ERR_SHAPE;                                                                          \
    hipLaunchKernelGGL((delta_scan_kernel<NR, BATCH, PARTS, COLS>), grid, block, 0, stream, o, state, qn, kn, kq,     \
                       decay, beta, u, state_slots, query_start_loc, first_seq, heads, kv_heads, dim, vdim);          \
  } while (0)
  if (spread) {
    if (dim <= 64) DS_GO(4, 16, 16, 8);
    else if (dim <= 128) DS_GO(8, 16, 16, 8);
    else DS_GO(16, 8, 16, 8);
  } else {
    if (dim <= 32) DS_GO(4, 8, 8, 32);
    else if (dim <= 64) DS_GO(8, 8, 8, 32);
    else if (dim <= 128) DS_GO(16, 8, 8, 32);
    else DS_GO(32, 8, 8, 32);
  }
#undef DS_GO
  return ts_launch_status();
}

extern "C" int ts_delta_finish(void* y, const float* o, const void* proj, int in_f32, int splits, long split_stride, int width,
                               int low_at, int low, const void* g2, const void* gain, float eps, int tokens, int heads, int vdim,
                               int dtype, float scale, long out_stride, hipStream_t stream) {
  if (tokens == 0) return TS_OK;
  if (!y || !o || !proj || !g2 || !gain || out_stride < (long)heads * vdim) return TS_ERR_ARG;
  if (heads < 1 || heads > 65535 || vdim < 1 || low < 1 || low > DS_MAX_LOW || splits < 1 || low_at < 0 || low_at + low > width)
    return TS_ERR_SHAPE;
  const int per = tokens >= 64 ? 8 : 1;
  const long items = (long)((tokens + per - 1) / per) * heads;
  const dim3 grid((unsigned)((items + DS_ITEMS - 1) / DS_ITEMS)), block(64 * DS_ITEMS);
#define DS_GO(T, P)                                                                                                   \
  if (per == 8)                                                                                                       \
    hipLaunchKernelGGL((delta_finish_kernel<T, P, 8>), grid, block, 0, stream, (T*)y, o, (const P*)proj, splits,       \
                       (size_t)split_stride, width, low_at, low, (const T*)g2, (const T*)gain, eps, tokens, heads, vdim, scale, (size_t)out_stride); \
  else                                                                                                                \
    hipLaunchKernelGGL((delta_finish_kernel<T, P, 1>), grid, block, 0, stream, (T*)y, o, (const P*)proj, splits,       \
                       (size_t)split_stride, width, low_at, low, (const T*)g2, (const T*)gain, eps, tokens, heads, vdim, scale, (size_t)out_stride)
  if (dtype == TS_F32) DS_GO(float, float);
  else if (dtype == TS_BF16 && in_f32) DS_GO(bf16_t, float);
  else if (dtype == TS_BF16) DS_GO(bf16_t, bf16_t);
  else return TS_ERR_DTYPE;
#undef DS_GO
  return ts_launch_status();
}
