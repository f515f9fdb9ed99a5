// A routed feed-forward (mixture of experts) for gfx950: every token goes through ``top`` of
// ``experts`` small gated feed-forwards, chosen by a router.
//
//   1. moe_route:  z = router x in float32, r = 1 / (1 + exp(-z)) (or softmax over the experts),
//                  the ``top`` largest r (the lower index first among equals), optionally
//                  divided by their sum. One workgroup a token.
//   2. moe_plan:   the (token, choice) pairs sorted by expert into rows; every expert's rows begin
//                  at a multiple of MOE_TILE_ROWS, so a tile of rows belongs to one expert. One
//                  workgroup; the tiles' experts and their number stay on the device, and the
//                  product kernels are launched for the most tiles there can be (a step's shape
//                  alone decides the grid, so a captured step replays).
//   3. moe_up:     per tile, inner = act(gate_e u) * (up_e u) with u = the pair's token row,
//                  multiplied by its score first when the score weighs the expert's input.
//   4. moe_down:   per tile, y[pair] = down_e inner (times the score when it weighs the output).
//   5. moe_combine: out[t] = sum over the token's pairs, in the order of the choices, float32.
//
// A row's sums run over K in an order that depends on K alone: where a pair lands among the rows
// changes nothing. T is the activation type; scores and sums are float32.
#include "common.h"

#define MOE_TILE_ROWS 16
#define MOE_MAX_EXPERTS 1024
#define MOE_ROUTER_SIGMOID 0
#define MOE_ROUTER_SOFTMAX 1

// ---------------------------------------------------------------- 1. router and choice
template <typename T>
__global__ __launch_bounds__(256) void moe_route_kernel(const T* __restrict__ x, const T* __restrict__ router, int H, int E,
                                                        int top, int kind, int* __restrict__ choice,
                                                        float* __restrict__ score) {
  __shared__ float r[MOE_MAX_EXPERTS];
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const T* xr = x + t * H;
  for (int e = wave; e < E; e += 4) {
    const T* w = router + (int64_t)e * H;
    float s = 0.0f;
    for (int j = lane; j < H; j += 64) s += cw_to_float(xr[j]) * cw_to_float(w[j]);
    s = cw_wave_sum(s);
    if (lane == 0) r[e] = s;
  }
  __syncthreads();
  if (wave != 0) return;
  if (kind == MOE_ROUTER_SOFTMAX) {
    float m = -3.0e38f;
    for (int e = lane; e < E; e += 64) m = fmaxf(m, r[e]);
    m = cw_wave_max(m);
    float sum = 0.0f;
    for (int e = lane; e < E; e += 64) sum += expf(r[e] - m);
    sum = cw_wave_sum(sum);
    for (int e = lane; e < E; e += 64) r[e] = expf(r[e] - m) / sum;
  } else {
    for (int e = lane; e < E; e += 64) r[e] = 1.0f / (1.0f + expf(-r[e]));
  }
  for (int k = 0; k < top; ++k) {
    // the largest score still there; among equals the lowest index
    float best = -1.0f;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += 64)
      if (r[e] > best) { best = r[e]; at = e; }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, 64);
      const int oa = __shfl_xor(at, off, 64);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    if (lane == 0) {
      choice[t * top + k] = at;
      score[t * top + k] = best;
      r[at] = -2.0f;  // scores are not negative: never chosen again
    }
  }
}

// the chosen scores of a token divided by their sum
__global__ __launch_bounds__(64) void moe_renorm_kernel(float* __restrict__ score, int top) {
  const int64_t t = blockIdx.x;
  float sum = 0.0f;
  for (int k = 0; k < top; ++k) sum += score[t * top + k];
  __syncthreads();
  for (int k = threadIdx.x; k < top; k += 64) score[t * top + k] /= sum;
}

// ---------------------------------------------------------------- 2. rows sorted by expert
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int* __restrict__ choice, int n_pairs, int E, int max_rows,
                                                        int* __restrict__ row_pair, int* __restrict__ tile_expert,
                                                        int* __restrict__ n_tiles) {
  __shared__ int counts[MOE_MAX_EXPERTS];
  __shared__ int first[MOE_MAX_EXPERTS + 1];
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += 1024) counts[e] = 0;
  for (int r = tid; r < max_rows; r += 1024) row_pair[r] = -1;
  __syncthreads();
  for (int p = tid; p < n_pairs; p += 1024) {
    const int e = choice[p];
    if (e >= 0 && e < E) atomicAdd(&counts[e], 1);
  }
  __syncthreads();
  if (tid == 0) {
    int rows = 0;
    for (int e = 0; e < E; ++e) {
      first[e] = rows;
      rows += (counts[e] + MOE_TILE_ROWS - 1) / MOE_TILE_ROWS * MOE_TILE_ROWS;
    }
    first[E] = rows;
    *n_tiles = rows / MOE_TILE_ROWS;
  }
  __syncthreads();
  for (int e = tid; e < E; e += 1024) {
    for (int tile = first[e] / MOE_TILE_ROWS; tile < first[e + 1] / MOE_TILE_ROWS; ++tile) tile_expert[tile] = e;
    counts[e] = 0;  // now the next free row of the expert
  }
  __syncthreads();
  for (int p = tid; p < n_pairs; p += 1024) {
    const int e = choice[p];
    if (e >= 0 && e < E) row_pair[first[e] + atomicAdd(&counts[e], 1)] = p;
  }
}

// ---------------------------------------------------------------- 3. / 4. the experts' products, plain arithmetic
// MODE 0: rows of x gathered by pair (token = pair / top), times the pair's score when
//         ``scale_input`` (rounded to the activation type), against the expert's gate and up
//         matrices [2 * N, K] (gate rows first); out[row, c] = act(gate) * up, [rows, N].
// MODE 1: rows of ``x`` as they lie ([rows, K]) against the expert's matrix [N, K]; the result goes to
//         out[pair, c], times the pair's score when ``scale_output``.
// A workgroup: 16 rows x 64 columns; K in steps of 32 through LDS.
#define MOE_KC 32
#define MOE_COLS 64
template <typename T, int MODE>
__global__ __launch_bounds__(256) void moe_expert_product_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                                 T* __restrict__ out, const int* __restrict__ row_pair,
                                                                 const int* __restrict__ tile_expert,
                                                                 const int* __restrict__ n_tiles,
                                                                 const float* __restrict__ score, int top, int K, int N,
                                                                 int use_score) {
  const int tile = blockIdx.y;
  if (tile >= *n_tiles) return;
  __shared__ float xs[MOE_TILE_ROWS][MOE_KC + 1];
  __shared__ float wa[MOE_COLS][MOE_KC + 1];
  __shared__ float wb[MODE == 0 ? MOE_COLS : 1][MOE_KC + 1];
  __shared__ int pair_of[MOE_TILE_ROWS];
  __shared__ float score_of[MOE_TILE_ROWS];
  const int tid = threadIdx.x;
  const int e = tile_expert[tile];
  const int r0 = tile * MOE_TILE_ROWS, c0 = blockIdx.x * MOE_COLS;
  if (tid < MOE_TILE_ROWS) {
    const int p = row_pair[r0 + tid];
    pair_of[tid] = p;
    score_of[tid] = (p >= 0 && use_score) ? score[p] : 1.0f;
  }
  __syncthreads();
  const T* we = w + (int64_t)e * (MODE == 0 ? 2 : 1) * N * K;
  const int r = tid >> 4, cq = tid & 15;
  float acc_a[4] = {0.0f, 0.0f, 0.0f, 0.0f}, acc_b[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int k0 = 0; k0 < K; k0 += MOE_KC) {
    for (int i = tid; i < MOE_TILE_ROWS * MOE_KC; i += 256) {
      const int rr = i / MOE_KC, kk = i % MOE_KC;
      const int p = pair_of[rr];
      float v = 0.0f;
      if (p >= 0 && k0 + kk < K) {
        if (MODE == 0) {
          v = cw_to_float(x[(int64_t)(p / top) * K + k0 + kk]);
          if (use_score) v = cw_to_float(cw_from_float<T>(v * score_of[rr]));
        } else {
          v = cw_to_float(x[(int64_t)(r0 + rr) * K + k0 + kk]);
        }
      }
      xs[rr][kk] = v;
    }
    for (int i = tid; i < MOE_COLS * MOE_KC; i += 256) {
      const int cc = i / MOE_KC, kk = i % MOE_KC;
      const bool in = c0 + cc < N && k0 + kk < K;
      wa[cc][kk] = in ? cw_to_float(we[(int64_t)(c0 + cc) * K + k0 + kk]) : 0.0f;
      if (MODE == 0) wb[cc][kk] = in ? cw_to_float(we[(int64_t)(N + c0 + cc) * K + k0 + kk]) : 0.0f;
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < MOE_KC; ++kk) {
      const float xv = xs[r][kk];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc_a[j] += xv * wa[cq + 16 * j][kk];
        if (MODE == 0) acc_b[j] += xv * wb[cq + 16 * j][kk];
      }
    }
    __syncthreads();
  }
  const int p = pair_of[r];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = c0 + cq + 16 * j;
    if (c >= N) continue;
    if (MODE == 0) {
      const float g = acc_a[j];
      out[(int64_t)(r0 + r) * N + c] = cw_from_float<T>(p >= 0 ? g / (1.0f + expf(-g)) * acc_b[j] : 0.0f);
    } else if (p >= 0) {
      out[(int64_t)p * N + c] = cw_from_float<T>(use_score ? acc_a[j] * score_of[r] : acc_a[j]);
    }
  }
}

// ---------------------------------------------------------------- 5. a token's pairs, added in their order
template <typename T>
__global__ void moe_combine_kernel(const T* __restrict__ y, T* __restrict__ out, int top, int H, int64_t total) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / H;
    const int j = (int)(i % H);
    float s = 0.0f;
    for (int k = 0; k < top; ++k) s += cw_to_float(y[(t * top + k) * H + j]);
    out[i] = cw_from_float<T>(s);
  }
}

// ---------------------------------------------------------------- entry points
CW_EXPORT int cw_moe_tile_rows() { return MOE_TILE_ROWS; }

// the most tiles and rows that ``n_pairs`` pairs over ``E`` experts can need
CW_EXPORT int cw_moe_max_tiles(int n_pairs, int E) {
  const int busy = n_pairs < E ? n_pairs : E;
  return n_pairs / MOE_TILE_ROWS + busy;
}

CW_EXPORT int cw_moe_route(const void* x, const void* router, int dtype, int T, int H, int E, int top, int kind, int renorm,
                           int* choice, float* score, hipStream_t stream) {
  if (T < 0 || H <= 0 || E <= 0 || top <= 0 || top > E || !x || !router || !choice || !score) return CW_ERR_ARG;
  if (kind != MOE_ROUTER_SIGMOID && kind != MOE_ROUTER_SOFTMAX) return CW_ERR_ARG;
  if (E > MOE_MAX_EXPERTS) return CW_ERR_SIZE;
  if (T == 0) return CW_OK;
  if (dtype == CW_F32)
    hipLaunchKernelGGL(moe_route_kernel<float>, dim3(T), dim3(256), 0, stream, (const float*)x, (const float*)router, H, E, top,
                       kind, choice, score);
  else if (dtype == CW_BF16)
    hipLaunchKernelGGL(moe_route_kernel<bf16_t>, dim3(T), dim3(256), 0, stream, (const bf16_t*)x, (const bf16_t*)router, H, E,
                       top, kind, choice, score);
  else return CW_ERR_DTYPE;
  if (renorm) hipLaunchKernelGGL(moe_renorm_kernel, dim3(T), dim3(64), 0, stream, score, top);
  return cw_launch_status();
}

CW_EXPORT int cw_moe_plan(const int* choice, int n_pairs, int E, int* row_pair, int max_rows, int* tile_expert, int max_tiles,
                          int* n_tiles, hipStream_t stream) {
  if (n_pairs < 0 || E <= 0 || !choice || !row_pair || !tile_expert || !n_tiles) return CW_ERR_ARG;
  if (E > MOE_MAX_EXPERTS) return CW_ERR_SIZE;
  if (max_tiles < cw_moe_max_tiles(n_pairs, E) || max_rows < max_tiles * MOE_TILE_ROWS) return CW_ERR_ARG;
  hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), 0, stream, choice, n_pairs, E, max_rows, row_pair, tile_expert,
                     n_tiles);
  return cw_launch_status();
}

// mode 0: the gate/up product with the activation (silu), mode 1: the down product
CW_EXPORT int cw_moe_expert_product(int mode, const void* x, const void* w, void* out, int dtype, const int* row_pair,
                                    const int* tile_expert, const int* n_tiles, int max_tiles, const float* score, int top,
                                    int K, int N, int use_score, hipStream_t stream) {
  if (max_tiles < 0 || K <= 0 || N <= 0 || top <= 0 || !x || !w || !out || !row_pair || !tile_expert || !n_tiles)
    return CW_ERR_ARG;
  if (use_score && !score) return CW_ERR_ARG;
  if (max_tiles > 65535) return CW_ERR_SIZE;
  if (max_tiles == 0) return CW_OK;
  dim3 grid((N + MOE_COLS - 1) / MOE_COLS, max_tiles), block(256);
#define CW_LAUNCH(T_, M_)                                                                                              \
  hipLaunchKernelGGL((moe_expert_product_kernel<T_, M_>), grid, block, 0, stream, (const T_*)x, (const T_*)w, (T_*)out, \
                     row_pair, tile_expert, n_tiles, score, top, K, N, use_score)
  if (dtype == CW_F32 && mode == 0) CW_LAUNCH(float, 0);
  else if (dtype == CW_F32 && mode == 1) CW_LAUNCH(float, 1);
  else if (dtype == CW_BF16 && mode == 0) CW_LAUNCH(bf16_t, 0);
  else if (dtype == CW_BF16 && mode == 1) CW_LAUNCH(bf16_t, 1);
  else return mode == 0 || mode == 1 ? CW_ERR_DTYPE : CW_ERR_ARG;
#undef CW_LAUNCH
  return cw_launch_status();
}

CW_EXPORT int cw_moe_combine(const void* y, void* out, int dtype, int T, int top, int H, hipStream_t stream) {
  if (T < 0 || top <= 0 || H <= 0 || !y || !out) return CW_ERR_ARG;
  if (T == 0) return CW_OK;
  const int64_t total = (int64_t)T * H;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 262144) blocks = 262144;
  dim3 grid((unsigned)blocks), block(256);
  if (dtype == CW_F32) hipLaunchKernelGGL(moe_combine_kernel<float>, grid, block, 0, stream, (const float*)y, (float*)out, top, H, total);
  else if (dtype == CW_BF16)
    hipLaunchKernelGGL(moe_combine_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)y, (bf16_t*)out, top, H, total);
  else return CW_ERR_DTYPE;
  return cw_launch_status();
}
