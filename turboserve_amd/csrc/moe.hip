// Routed feed-forward ("mixture of experts"): the router with its selection rule, the experts'
// products for the (token, taken expert) pairs of a step, and the weighted sum.
//
// Router: z = R x comes from the engine's own product with a 32-bit result; here, all in 32-bit,
// s = sigmoid(z), or softmax(z) over all the router's outputs.  Experts are chosen by c = s +
// correction (a vector per layer; none: c = s).  The experts form `groups` equal groups of
// neighbours; a group's mark is the sum of its two largest c (its one c if it has one member);
// only experts of the `keep` groups with the largest marks can be taken; the `top` of them with
// the largest c are, with weights s / (sum of the taken s + 1e-20) * route_scale, or, not
// normalised, s * route_scale.  Equal values go to the lower index.  groups == 1 is plain top-k.
// An index at or above the number of experts that have matrices stands for the identity (the
// token itself): the products skip such pairs and the weighted sum reads the token's row.
#include "common.hpp"

#define MOE_MAX_EXPERTS 1024
#define MOE_MAX_TOP 32

// Index of the largest of the values the lanes hold (value, index pairs; index < 2^24), the
// lower index among equals; every lane returns it.  A lane without a candidate passes -inf.
__device__ __forceinline__ int wave_argmax(float value, int index, float& best) {
  best = wave_max(value);
  const float mine = (value == best) ? -(float)index : -16777216.f;
  return (int)(-wave_max(mine));
}

// One wavefront per token: the selection from the router's 32-bit outputs z [T, stride] (the
// first `experts` of a row; where extra_gate is asked for, element `experts` of the row is the
// gate's own output).
__global__ void __launch_bounds__(TS_WAVE)
moe_select_kernel(int* __restrict__ taken, float* __restrict__ weights, float* __restrict__ extra_gate,
                  const float* __restrict__ z, int stride, int experts, int top, int groups, int keep,
                  float route_scale, int softmax, const float* __restrict__ correction, int normalise, int mark_top) {
  __shared__ float weight_of[MOE_MAX_EXPERTS];  // s: what a taken expert is weighted with
  __shared__ float score[MOE_MAX_EXPERTS];      // c: what experts are chosen by
  __shared__ float mark[MOE_MAX_EXPERTS];   // per group
  __shared__ int open_group[MOE_MAX_EXPERTS];
  const int t = blockIdx.x;
  const int lane = threadIdx.x;
  const float* row = z + (size_t)t * stride;
  if (softmax) {
    float top_z = -INFINITY;
    for (int e = lane; e < experts; e += TS_WAVE) top_z = fmaxf(top_z, row[e]);
    top_z = wave_max(top_z);
    float sum = 0.f;
    for (int e = lane; e < experts; e += TS_WAVE) {
      const float v = expf(row[e] - top_z);
      weight_of[e] = v;
      sum += v;
    }
    sum = wave_sum(sum);
    for (int e = lane; e < experts; e += TS_WAVE) weight_of[e] = weight_of[e] / sum;  // each lane its own entries
  } else {
    for (int e = lane; e < experts; e += TS_WAVE) weight_of[e] = 1.f / (1.f + expf(-row[e]));
  }
  for (int e = lane; e < experts; e += TS_WAVE) score[e] = weight_of[e] + (correction ? correction[e] : 0.f);
  if (extra_gate && lane == 0) extra_gate[t] = 1.f / (1.f + expf(-row[experts]));
  __syncthreads();
  const int size = experts / groups;
  {
    for (int g = lane; g < groups; g += TS_WAVE) {
      float a = -INFINITY, b = -INFINITY;  // largest, second
      for (int i = 0; i < size; ++i) {
        const float s = score[g * size + i];
        if (s > a) { b = a; a = s; } else if (s > b) { b = s; }
      }
      mark[g] = (size > 1 && mark_top > 1) ? a + b : a;  // a group's mark: its two largest summed, or its largest
      open_group[g] = keep >= groups ? 1 : 0;
    }
  }
  __syncthreads();
  if (keep < groups) {
    for (int round = 0; round < keep; ++round) {
      {
        float mine = -INFINITY;
        int at = 0;
        for (int g = lane; g < groups; g += TS_WAVE)
          if (!open_group[g] && mark[g] > mine) { mine = mark[g]; at = g; }
        float best;
        const int g = wave_argmax(mine, at, best);
        if (lane == 0) open_group[g] = 1;
      }
      __syncthreads();
    }
  }
  float total = 0.f;
  float kept_score = 0.f;  // lane r holds the score of the r-th taken expert
  int kept_index = 0;
  for (int round = 0; round < top; ++round) {
    {
      float mine = -INFINITY;
      int at = 0;
      for (int e = lane; e < experts; e += TS_WAVE)
        if (open_group[e / size] && score[e] > mine) { mine = score[e]; at = e; }
      float best;
      const int e = wave_argmax(mine, at, best);
      const float s = weight_of[e];
      if (lane == round) { kept_score = s; kept_index = e; }
      total += s;
      if (lane == 0) score[e] = -INFINITY;  // taken
    }
    __syncthreads();
  }
  if (lane < top) {
    taken[(size_t)t * top + lane] = kept_index;
    weights[(size_t)t * top + lane] = (normalise ? kept_score / (total + 1e-20f) : kept_score) * route_scale;
  }
}

extern "C" int ts_moe_select(int* taken, float* weights, float* extra_gate, const float* z, int tokens, int stride,
                             int experts, int top, int groups, int keep, float route_scale, int softmax,
                             const float* correction, int normalise, int mark_top, hipStream_t stream) {
  if (tokens == 0) return TS_OK;
  if (!taken || !weights || !z || mark_top < 1 || mark_top > 2) return TS_ERR_ARG;
  if (experts < 1 || experts > MOE_MAX_EXPERTS || top < 1 || top > MOE_MAX_TOP || groups < 1 || experts % groups != 0 ||
      keep < 1 || keep > groups || top > (experts / groups) * keep || stride < experts + (extra_gate ? 1 : 0))
    return TS_ERR_SHAPE;
  hipLaunchKernelGGL(moe_select_kernel, dim3(tokens), dim3(TS_WAVE), 0, stream, taken, weights, extra_gate, z, stride,
                     experts, top, groups, keep, route_scale, softmax, correction, normalise, mark_top);
  return ts_launch_status();
}

// ---------------------------------------------------------------------------------------------
// The experts' products pair by pair: pair p = (token p / top, its (p % top)-th taken expert e).
// (Without a list of taken experts, pair p is with expert p mod E: the stacked matrices are then the
// heads of a per-head product, rows [T * E, K] head by head.)
// Weights are stacked over the experts, [E, N, K].  out[p, n] = W[e][n] . in[row(p)] with row(p) =
// p / in_share (the token's activations for the first product: in_share = top; the pair's own row
// for the second: in_share = 1).  GATED: N = 2 I rows alternate gate, up and the output is
// gated_unit(gate, up) of the run type, [P, I]; else the output is 32-bit, [P, N].  A block
// stages the input row in LDS as 32-bit and its wavefronts walk the rows of a slice of N: the
// weights stream once per pair, which is what a step of few tokens costs anyway.
// ---------------------------------------------------------------------------------------------
#define MOE_ROWS_PER_BLOCK 32

template <typename T>
__device__ __forceinline__ float row_dot_staged(const T* __restrict__ w, const float* __restrict__ xs, int k, int lane);

template <>
__device__ __forceinline__ float row_dot_staged<float>(const float* __restrict__ w, const float* __restrict__ xs, int k,
                                                       int lane) {
  float s = 0.f;
  for (int i = lane; i < k; i += TS_WAVE) s = fmaf(w[i], xs[i], s);
  return wave_sum(s);
}

template <>
__device__ __forceinline__ float row_dot_staged<bf16_t>(const bf16_t* __restrict__ w, const float* __restrict__ xs, int k,
                                                        int lane) {
  float s = 0.f;
  if ((k & 7) == 0 && ((uintptr_t)w & 15) == 0) {
    for (int i = lane * 8; i < k; i += TS_WAVE * 8) {
      const ts_u32x4 v = load_once16(w + i);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        s = fmaf(__uint_as_float(v[e] << 16), xs[i + 2 * e], s);
        s = fmaf(__uint_as_float(v[e] & 0xffff0000u), xs[i + 2 * e + 1], s);
      }
    }
  } else {
    for (int i = lane; i < k; i += TS_WAVE) s = fmaf(to_float(w[i]), xs[i], s);
  }
  return wave_sum(s);
}

template <typename T, bool GATED>
__global__ void __launch_bounds__(256)
moe_pair_rows_kernel(void* __restrict__ out_any, const T* __restrict__ in, const T* __restrict__ weight,
                     const int* __restrict__ taken, int in_share, int n, int k, int experts, GluRule rule) {
  extern __shared__ float xs[];
  const int pair = blockIdx.x;
  const int e = taken ? taken[pair] : pair % experts;  // no list: the experts in turn (pair p is with expert p mod E)
  const T* row = in + (size_t)(pair / in_share) * k;
  for (int i = threadIdx.x; i < k; i += blockDim.x) xs[i] = to_float(row[i]);
  __syncthreads();
  if (e < 0 || e >= experts) return;  // a host error; nothing is read out of bounds
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x % TS_WAVE, waves = blockDim.x / TS_WAVE;
  const T* w = weight + (size_t)e * n * k;
  if (GATED) {
    const int units = n / 2;
    T* out = (T*)out_any + (size_t)pair * units;
    const int first = blockIdx.y * MOE_ROWS_PER_BLOCK;
    for (int i = first + wave; i < min(first + MOE_ROWS_PER_BLOCK, units); i += waves) {
      const float g = row_dot_staged<T>(w + (size_t)(2 * i) * k, xs, k, lane);
      const float u = row_dot_staged<T>(w + (size_t)(2 * i + 1) * k, xs, k, lane);
      if (lane == 0) out[i] = from_float<T>(gated_unit(g, u, rule));
    }
  } else {
    float* out = (float*)out_any + (size_t)pair * n;
    const int first = blockIdx.y * MOE_ROWS_PER_BLOCK;
    for (int i = first + wave; i < min(first + MOE_ROWS_PER_BLOCK, n); i += waves) {
      const float y = row_dot_staged<T>(w + (size_t)i * k, xs, k, lane);
      if (lane == 0) out[i] = y;
    }
  }
}

extern "C" int ts_moe_pair_rows(void* out, const void* in, const void* weight, const int* taken, int pairs,
                                int in_share, int n, int k, int experts, int gated, float steepness, float limit,
                                float up_shift, float cubic, int dtype, hipStream_t stream) {
  if (pairs == 0) return TS_OK;
  if (!out || !in || !weight) return TS_ERR_ARG;
  if (n < 1 || k < 1 || k > 12288 || in_share < 1 || experts < 1 || (gated && (n & 1))) return TS_ERR_SHAPE;
  const GluRule rule = {steepness, limit, up_shift, cubic};
  const int outputs = gated ? n / 2 : n;
  const dim3 grid(pairs, (outputs + MOE_ROWS_PER_BLOCK - 1) / MOE_ROWS_PER_BLOCK), block(256);
  if (grid.y > 65535) return TS_ERR_SHAPE;
  const size_t lds = (size_t)k * sizeof(float);
  if (dtype == TS_F32 && gated)
    hipLaunchKernelGGL((moe_pair_rows_kernel<float, true>), grid, block, lds, stream, out, (const float*)in, (const float*)weight, taken, in_share, n, k, experts, rule);
  else if (dtype == TS_F32)
    hipLaunchKernelGGL((moe_pair_rows_kernel<float, false>), grid, block, lds, stream, out, (const float*)in, (const float*)weight, taken, in_share, n, k, experts, rule);
  else if (dtype == TS_BF16 && gated)
    hipLaunchKernelGGL((moe_pair_rows_kernel<bf16_t, true>), grid, block, lds, stream, out, (const bf16_t*)in, (const bf16_t*)weight, taken, in_share, n, k, experts, rule);
  else if (dtype == TS_BF16)
    hipLaunchKernelGGL((moe_pair_rows_kernel<bf16_t, false>), grid, block, lds, stream, out, (const bf16_t*)in, (const bf16_t*)weight, taken, in_share, n, k, experts, rule);
  else
    return TS_ERR_DTYPE;
  return ts_launch_status();
}

// ---------------------------------------------------------------------------------------------
// out[t, :] = sum_j weights[t, j] * pair_out[t * top + j, :]  (+ extra_gate[t] * extra[t, :]),
// 32-bit, summed in the order j = 0, 1, ..; `extra` (the shared expert's output) is of type P: T,
// or `splits` 32-bit partial sums `split_stride` elements apart.
// ---------------------------------------------------------------------------------------------
// Where `taken` is given, a pair whose index is at or above `experts` is the identity: its output
// is the token's own row of `rows` (type R), and pair_out holds nothing for it.
template <typename P, typename R>
__global__ void moe_combine_kernel(float* __restrict__ out, const float* __restrict__ pair_out,
                                   const float* __restrict__ weights, const P* __restrict__ extra, int splits,
                                   size_t split_stride, const float* __restrict__ extra_gate, int top, int width,
                                   const int* __restrict__ taken, int experts, const R* __restrict__ rows) {
  const int t = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= width) return;
  float s = 0.f;
  for (int j = 0; j < top; ++j) {
    const bool same = taken && taken[(size_t)t * top + j] >= experts;
    const float y = same ? to_float(rows[(size_t)t * width + i]) : pair_out[((size_t)t * top + j) * width + i];
    s = fmaf(weights[(size_t)t * top + j], y, s);
  }
  if (extra) {
    float x = 0.f;
    for (int sp = 0; sp < splits; ++sp) x += to_float(extra[(size_t)sp * split_stride + (size_t)t * width + i]);
    s = fmaf(extra_gate ? extra_gate[t] : 1.f, x, s);
  }
  out[(size_t)t * width + i] = s;
}

extern "C" int ts_moe_combine(float* out, const float* pair_out, const float* weights, const void* extra,
                              int extra_f32, int splits, long split_stride, const float* extra_gate, int tokens,
                              int top, int width, int dtype, const int* taken, int experts, const void* rows,
                              hipStream_t stream) {
  if (tokens == 0) return TS_OK;
  if (!out || !pair_out || !weights || top < 1 || width < 1 || splits < 1) return TS_ERR_ARG;
  if ((taken != nullptr) != (rows != nullptr)) return TS_ERR_ARG;
  const dim3 grid(tokens, (width + 255) / 256), block(256);
  if (grid.y > 65535) return TS_ERR_SHAPE;
  if (dtype != TS_F32 && dtype != TS_BF16) return TS_ERR_DTYPE;
  // `dtype` is the run's: that of `rows`, and of `extra` unless it is 32-bit partial sums.
  const bool extra32 = !extra || extra_f32 || dtype == TS_F32;
  if (dtype == TS_F32)
    hipLaunchKernelGGL((moe_combine_kernel<float, float>), grid, block, 0, stream, out, pair_out, weights, (const float*)extra, splits, (size_t)split_stride, extra_gate, top, width, taken, experts, (const float*)rows);
  else if (extra32)
    hipLaunchKernelGGL((moe_combine_kernel<float, bf16_t>), grid, block, 0, stream, out, pair_out, weights, (const float*)extra, splits, (size_t)split_stride, extra_gate, top, width, taken, experts, (const bf16_t*)rows);
  else
    hipLaunchKernelGGL((moe_combine_kernel<bf16_t, bf16_t>), grid, block, 0, stream, out, pair_out, weights, (const bf16_t*)extra, splits, (size_t)split_stride, extra_gate, top, width, taken, experts, (const bf16_t*)rows);
  return ts_launch_status();
}

// ---------------------------------------------------------------------------------------------
// Many tokens (prompt portions), bfloat16: the pairs are grouped by expert and every expert's
// rows go through the matrix cores in tiles, so an expert's matrices are read once per 64 rows
// instead of once per pair.
//
// ts_moe_group: order[P] = the pairs sorted by expert (within an expert in no fixed order: every
// row is computed alone, so the order changes nothing), tile_first[E + 1] = the running count of
// row tiles of MOE_TILE_ROWS (tile_first[E]: all of them), row_first[E + 1] = the running count of
// rows.  One block.
//
// ts_moe_grouped_rows: out[order[r], :] for every sorted row r, a block per (row tile, 128 output
// columns), found from tile_first; blocks beyond the last tile leave at once, so the grid is the
// upper bound P / MOE_TILE_ROWS + E.  K must be a multiple of 8.
// ---------------------------------------------------------------------------------------------
#define MOE_TILE_ROWS 128
#define MOE_TILE_COLS 128

__global__ void __launch_bounds__(1024)
moe_group_kernel(int* __restrict__ order, int* __restrict__ tile_first, int* __restrict__ row_first,
                 const int* __restrict__ taken, int pairs, int experts) {
  __shared__ int count[MOE_MAX_EXPERTS];
  __shared__ int cursor[MOE_MAX_EXPERTS];
  for (int e = threadIdx.x; e < experts; e += blockDim.x) count[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
    const int e = taken ? taken[p] : p % experts;
    if (e >= 0 && e < experts) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int rows = 0, tiles = 0;
    for (int e = 0; e < experts; ++e) {
      row_first[e] = rows;
      tile_first[e] = tiles;
      cursor[e] = rows;
      rows += count[e];
      tiles += (count[e] + MOE_TILE_ROWS - 1) / MOE_TILE_ROWS;
    }
    row_first[experts] = rows;
    tile_first[experts] = tiles;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
    const int e = taken ? taken[p] : p % experts;
    if (e >= 0 && e < experts) order[atomicAdd(&cursor[e], 1)] = p;
  }
}

extern "C" int ts_moe_group(int* order, int* tile_first, int* row_first, const int* taken, int pairs, int experts,
                            hipStream_t stream) {
  if (!order || !tile_first || !row_first || pairs < 1) return TS_ERR_ARG;
  if (experts < 1 || experts > MOE_MAX_EXPERTS) return TS_ERR_SHAPE;
  hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(1024), 0, stream, order, tile_first, row_first, taken, pairs, experts);
  return ts_launch_status();
}

typedef __bf16 moe_bf16x8 __attribute__((ext_vector_type(8)));
typedef float moe_f32x4 __attribute__((ext_vector_type(4)));

#define MOE_DEPTH 128                  // k per iteration
#define MOE_LDS_ROW (MOE_DEPTH + 8)    // elements; 272 bytes: sixteen rows' same piece lies in sixteen different banks' quads

// A block of four wavefronts owns 128 sorted rows x 128 columns; per iteration both operands go
// global memory -> registers (16-byte pieces, eight consecutive threads a row's 128 bytes) -> LDS ->
// matrix cores, 128 of K per iteration; the loads of the next iteration (sixteen 16-byte pieces a
// thread) are in flight while this one's products run: what an iteration waits for is a trip
// to memory, so it carries as many bytes as the registers hold.
// A wavefront computes 64 rows x 64 columns (4 x 4 tiles of 16 x 16: a fragment read from LDS
// serves four matrix instructions).
template <bool GATED>
__global__ void __launch_bounds__(256)
moe_grouped_rows_kernel(void* __restrict__ out_any, const bf16_t* __restrict__ in, const bf16_t* __restrict__ weight,
                        const int* __restrict__ order, const int* __restrict__ tile_first,
                        const int* __restrict__ row_first, int in_share, int n, int k, int experts, GluRule rule,
                        int tile_slots, int col_tiles) {
  extern __shared__ __attribute__((aligned(16))) uint16_t moe_tiles[];  // [rows of A, then rows of B][MOE_LDS_ROW]
  __shared__ int found;
  // Workgroup id -> (row tile, column tile): consecutive ids go to the eight dies in turn, so a
  // die's ids are id % 8 == die; of those, consecutive ones take consecutive row tiles under one
  // column tile, so the row tiles of an expert, which share their weights, meet in one die's L2.
  const int total = tile_slots * col_tiles;
  const int per_die = (total + 7) / 8;
  const int logical = (int)(blockIdx.x % 8) * per_die + (int)(blockIdx.x / 8);
  if (logical >= total) return;
  const int tile = logical % tile_slots;
  const int col_tile = logical / tile_slots;
  if (tile >= tile_first[experts]) return;  // the whole block leaves together
  if (threadIdx.x < TS_WAVE) {
    // The expert whose tiles hold this one.
    int best = -1;
    for (int e = threadIdx.x; e < experts; e += TS_WAVE)
      if (tile_first[e] <= tile && tile_first[e + 1] > tile) best = e;
    best = (int)wave_max((float)best);
    if (threadIdx.x == 0) found = best;
  }
  __syncthreads();
  const int e = found;
  const int tid = threadIdx.x;
  const int wave = tid / TS_WAVE, lane = tid % TS_WAVE;
  const int r16 = lane % 16, group = lane / 16;
  const int wm = wave / 2, wn = wave % 2;
  const int rows_begin = row_first[e] + (tile - tile_first[e]) * MOE_TILE_ROWS;
  const int rows_end = row_first[e + 1];
  const int col_begin = col_tile * MOE_TILE_COLS;
  const bf16_t* w = weight + (size_t)e * n * k;

  // What this thread fetches per iteration: pieces tid + 256 i of the tiles, piece = (row, 8 k).
  constexpr int ROW_PIECES = MOE_DEPTH / 8;     // 16-byte pieces of a row of an iteration
  constexpr int PASS_ROWS = 256 / ROW_PIECES;   // rows one pass of the threads covers
  constexpr int PASSES = MOE_TILE_ROWS / PASS_ROWS;
  static_assert(MOE_TILE_ROWS == MOE_TILE_COLS, "both tiles take the same passes");
  const int piece_k = 8 * (tid % ROW_PIECES);
  const int piece_row = tid / ROW_PIECES;  // + PASS_ROWS i
  const bf16_t* a_src[PASSES];
  const bf16_t* b_src[PASSES];
#pragma unroll
  for (int i = 0; i < PASSES; ++i) {
    const int r = min(rows_begin + piece_row + PASS_ROWS * i, rows_end - 1);
    a_src[i] = in + (size_t)(order[r] / in_share) * k;
  }
#pragma unroll
  for (int i = 0; i < PASSES; ++i) b_src[i] = w + (size_t)min(col_begin + piece_row + PASS_ROWS * i, n - 1) * k;
  ts_u32x4 a_reg[PASSES], b_reg[PASSES];
  auto fetch = [&](int k0) __attribute__((always_inline)) {
    const bool inside = k0 + piece_k < k;
    const int at = inside ? k0 + piece_k : 0;
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {
      a_reg[i] = *reinterpret_cast<const ts_u32x4*>(a_src[i] + at);
      if (!inside) a_reg[i] = ts_u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {
      b_reg[i] = *reinterpret_cast<const ts_u32x4*>(b_src[i] + at);  // plain: other row tiles read it again
      if (!inside) b_reg[i] = ts_u32x4{0u, 0u, 0u, 0u};
    }
  };
  uint16_t* a_tile = moe_tiles;
  uint16_t* b_tile = a_tile + MOE_TILE_ROWS * MOE_LDS_ROW;
  auto stage = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < PASSES; ++i)
      *reinterpret_cast<ts_u32x4*>(a_tile + (piece_row + PASS_ROWS * i) * MOE_LDS_ROW + piece_k) = a_reg[i];
#pragma unroll
    for (int i = 0; i < PASSES; ++i)
      *reinterpret_cast<ts_u32x4*>(b_tile + (piece_row + PASS_ROWS * i) * MOE_LDS_ROW + piece_k) = b_reg[i];
  };

  moe_f32x4 acc[4][4];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[a][b] = moe_f32x4{0.f, 0.f, 0.f, 0.f};
  fetch(0);
  for (int k0 = 0; k0 < k; k0 += MOE_DEPTH) {
    stage();
    __syncthreads();
    if (k0 + MOE_DEPTH < k) fetch(k0 + MOE_DEPTH);  // in flight while this iteration's products run
#pragma unroll
    for (int kk = 0; kk < MOE_DEPTH; kk += 32) {
      ts_u32x4 af[4], bf[4];
#pragma unroll
      for (int a = 0; a < 4; ++a)
        af[a] = *reinterpret_cast<const ts_u32x4*>(a_tile + (wm * 64 + 16 * a + r16) * MOE_LDS_ROW + kk + 8 * group);
#pragma unroll
      for (int b = 0; b < 4; ++b)
        bf[b] = *reinterpret_cast<const ts_u32x4*>(b_tile + (wn * 64 + 16 * b + r16) * MOE_LDS_ROW + kk + 8 * group);
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(moe_bf16x8, af[a]),
                                                              __builtin_bit_cast(moe_bf16x8, bf[b]), acc[a][b], 0, 0, 0);
    }
    __syncthreads();  // everyone has read this iteration's tiles before the next is staged
  }
  // acc[a][b][i] is row 16 a + 4 group + i, column 16 b + r16 of the wavefront's 64 x 64.
#pragma unroll
  for (int a = 0; a < 4; ++a) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = rows_begin + wm * 64 + 16 * a + 4 * group + i;
      const int pair = order[min(r, rows_end - 1)];
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int col = col_begin + wn * 64 + 16 * b + r16;
        const float v = acc[a][b][i];
        if (GATED) {
          const float other = __shfl_xor(v, 1, 64);  // columns alternate gate, up
          if ((r16 & 1) == 0 && r < rows_end && col + 1 < n)
            ((bf16_t*)out_any)[(size_t)pair * (n / 2) + col / 2] = from_float<bf16_t>(gated_unit(v, other, rule));
        } else if (r < rows_end && col < n) {
          ((float*)out_any)[(size_t)pair * n + col] = v;
        }
      }
    }
  }
}

extern "C" int ts_moe_grouped_rows(void* out, const void* in, const void* weight, const int* order,
                                   const int* tile_first, const int* row_first, int pairs, int in_share, int n, int k,
                                   int experts, int gated, float steepness, float limit, float up_shift, float cubic,
                                   hipStream_t stream) {
  if (pairs == 0) return TS_OK;
  if (!out || !in || !weight || !order || !tile_first || !row_first) return TS_ERR_ARG;
  if (n < 1 || k < 8 || k % 8 != 0 || in_share < 1 || experts < 1 || experts > MOE_MAX_EXPERTS || (gated && (n & 1)))
    return TS_ERR_SHAPE;
  if (((uintptr_t)in | (uintptr_t)weight) % 16 != 0) return TS_ERR_ARG;
  const GluRule rule = {steepness, limit, up_shift, cubic};
  const int tile_slots = pairs / MOE_TILE_ROWS + experts + 1, col_tiles = (n + MOE_TILE_COLS - 1) / MOE_TILE_COLS;
  if ((long)tile_slots * col_tiles + 8 > 2147483647L) return TS_ERR_SHAPE;
  const dim3 grid((unsigned)(((tile_slots * col_tiles + 7) / 8) * 8)), block(256);
  constexpr size_t lds = (size_t)(MOE_TILE_ROWS + MOE_TILE_COLS) * MOE_LDS_ROW * sizeof(uint16_t);
  static_assert(lds <= 80 * 1024, "two workgroups' buffers fit a compute unit's LDS");
  static bool raised = false;  // per process; the attribute belongs to the kernels
  if (!raised) {
    if (hipFuncSetAttribute((const void*)moe_grouped_rows_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess ||
        hipFuncSetAttribute((const void*)moe_grouped_rows_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return TS_ERR_LAUNCH;
    raised = true;
  }
  if (gated)
    hipLaunchKernelGGL(moe_grouped_rows_kernel<true>, grid, block, lds, stream, out, (const bf16_t*)in, (const bf16_t*)weight, order, tile_first, row_first, in_share, n, k, experts, rule, tile_slots, col_tiles);
  else
    hipLaunchKernelGGL(moe_grouped_rows_kernel<false>, grid, block, lds, stream, out, (const bf16_t*)in, (const bf16_t*)weight, order, tile_first, row_first, in_share, n, k, experts, rule, tile_slots, col_tiles);
  return ts_launch_status();
}
