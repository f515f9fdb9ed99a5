// A routed feed-forward (mixture of experts) for gfx950: every token goes through ``top`` of
// ``experts`` small gated feed-forwards, chosen by a router.
//
//   1. moe_route:  z = router x in float32, r = 1 / (1 + exp(-z)) (or softmax over the experts),
//                  the ``top`` largest r, chosen by their z (the lower index first among equals), optionally
//                  divided by their sum. One workgroup a token. Options: a ``correction`` per
//                  expert joins r for the CHOICE only (the weights stay r); experts in ``groups``
//                  equal runs of neighbours, a run scored by the sum of its ``group_top`` largest
//                  choice scores, and only experts of the ``groups_kept`` best runs can be chosen;
//                  ``extra`` rows behind the router's (gates of the same input) leave their
//                  logistic values beside the choice.
//   2. moe_plan:   the (token, choice) pairs sorted by expert into rows; every expert's rows begin
//                  at a multiple of MOE_TILE_ROWS, so a tile of rows belongs to one expert. One
//                  workgroup; the tiles' experts and their number stay on the device, and the
//                  product kernels are launched for the most tiles there can be (a step's shape
//                  alone decides the grid, so a captured step replays).
//   3. moe_up:     per tile, inner = act(gate_e u) * (up_e u) with u = the pair's token row,
//                  multiplied by its score first when the score weighs the expert's input.
//   4. moe_down:   per tile, y[pair] = down_e inner (times the score when it weighs the output).
//   5. moe_combine: out[t] = sum over the token's pairs, in the order of the choices, float32;
//                  then, if there is one, the output of an expert that every token uses, times its gate.
//
// Steps 3 and 4 have three kernels. Plain arithmetic on the vector units (tiles of 16 rows): any
// type and size, and what float32 always runs. For bfloat16 with K a multiple of 8, on the matrix
// cores: few rows an expert (single tokens) take tiles of 16 rows and stream the expert's matrix
// once, K shared among the eight waves of a workgroup; many rows an expert (portions of prompts)
// take tiles of 128 rows against 128 matrix rows through LDS. The host chooses by the step's
// shape alone (pairs and experts), so a captured step replays.
//
// A row's sums run over K in an order that depends on K and the kernel alone: where a pair lands
// among the rows changes nothing. T is the activation type; scores and sums are float32.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;

#define MOE_TILE_ROWS 16    // of the plain and the streaming kernel
#define MOE_WIDE_ROWS 128   // of the LDS-tiled kernel
#define MOE_GROUPED_ROWS 256  // of the matrix product over row tiles with matrices of their own (another library's)
#define MOE_MAX_EXPERTS 1024
#define MOE_ROUTER_SIGMOID 0
#define MOE_ROUTER_SOFTMAX 1

// ---------------------------------------------------------------- 1. router and choice
#define MOE_MAX_EXTRA 8
#define MOE_MAX_GROUP_TOP 64
struct MoeRouteOptions {
  const float* correction;  // [E] or null
  int groups, groups_kept, group_top;   // groups <= 1: every expert can be chosen
  int extra;                // rows behind the router's E
  float* extra_out;         // [T, extra]
  int renorm;               // the chosen scores are divided by their sum plus renorm_eps
  float renorm_eps;
};

template <typename T>
__global__ __launch_bounds__(256) void moe_route_kernel(const T* __restrict__ x, const T* __restrict__ router, int H, int E,
                                                        int top, int kind, int* __restrict__ choice,
                                                        float* __restrict__ score, MoeRouteOptions opt) {
  __shared__ float r[MOE_MAX_EXPERTS + MOE_MAX_EXTRA];  // logits, then scores
  __shared__ float z[MOE_MAX_EXPERTS];  // what the choice compares
  __shared__ float run_score[MOE_MAX_EXPERTS];
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const T* xr = x + t * H;
  constexpr int V = 16 / (int)sizeof(T);
  const bool vec_ok = H % V == 0 && !((uintptr_t)x & 15) && !((uintptr_t)router & 15);
  for (int e = wave; e < E + opt.extra; e += 4) {
    const T* w = router + (int64_t)e * H;
    float s = 0.0f;
    if (vec_ok) {  // 16 bytes of each row a lane and step; the order of a lane's sums depends on H alone
      for (int j = lane * V; j < H; j += 64 * V) {
        if constexpr (sizeof(T) == 4) {
          const f32x4_t a = *reinterpret_cast<const f32x4_t*>(xr + j);
          const f32x4_t b = *reinterpret_cast<const f32x4_t*>(w + j);
#pragma unroll
          for (int i = 0; i < 4; ++i) s += a[i] * b[i];
        } else {
          const u32x4_t a = *reinterpret_cast<const u32x4_t*>(xr + j);
          const u32x4_t b = *reinterpret_cast<const u32x4_t*>(w + j);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            s += cw_bf16_bits_to_float((uint16_t)(a[i] & 0xffffu)) * cw_bf16_bits_to_float((uint16_t)(b[i] & 0xffffu));
            s += cw_bf16_bits_to_float((uint16_t)(a[i] >> 16)) * cw_bf16_bits_to_float((uint16_t)(b[i] >> 16));
          }
        }
      }
    } else {
      for (int j = lane; j < H; j += 64) s += cw_to_float(xr[j]) * cw_to_float(w[j]);
    }
    s = cw_wave_sum(s);
    if (lane == 0) r[e] = s;
  }
  __syncthreads();
  if (wave != 0) return;
  // the choice is made on the logits, which order the experts as the scores do and still tell
  // apart two experts whose scores both round to 1
  for (int e = lane; e < E; e += 64) z[e] = r[e];
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
  for (int x = lane; x < opt.extra; x += 64) opt.extra_out[t * opt.extra + x] = 1.0f / (1.0f + expf(-r[E + x]));
  if (opt.correction || opt.groups > 1) {
    // the choice is made on score + correction (which the logits no longer order), and runs are
    // compared by sums of scores
    for (int e = lane; e < E; e += 64) z[e] = r[e] + (opt.correction ? opt.correction[e] : 0.0f);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
  }
  if (opt.groups > 1) {
    const int per = E / opt.groups;
    for (int g = lane; g < opt.groups; g += 64) {
      // the sum of the run's largest choice scores, taken one after the other: the next one is
      // the largest that comes after the last in the order (score falling, index rising)
      float sum = 0.0f, prev = 3.4e38f;
      int prev_at = -1;
      for (int n = 0; n < opt.group_top && n < per; ++n) {
        float best = -3.4e38f;
        int at = -1;
        for (int e = g * per; e < (g + 1) * per; ++e) {
          const float c = z[e];
          const bool after = c < prev || (c == prev && e > prev_at);
          if (after && (at < 0 || c > best)) { best = c; at = e; }
        }
        if (at < 0) break;
        sum += best;
        prev = best;
        prev_at = at;
      }
      run_score[g] = sum;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
    // a run is kept if fewer than ``groups_kept`` runs come before it (a larger score, or an equal one and a lower index)
    for (int e = lane; e < E; e += 64) {
      const int g = e / per;
      int ahead = 0;
      for (int o = 0; o < opt.groups; ++o)
        ahead += (run_score[o] > run_score[g] || (run_score[o] == run_score[g] && o < g)) ? 1 : 0;
      if (ahead >= opt.groups_kept) z[e] = -3.4e38f;
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
  for (int k = 0; k < top; ++k) {
    // the largest logit still there; among equals the lowest index
    float best = -3.4e38f;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += 64)
      if (z[e] > best) { best = z[e]; at = e; }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, 64);
      const int oa = __shfl_xor(at, off, 64);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    if (lane == 0) {
      const bool found = at < E;   // not so if the logits are no numbers: a row that holds no token
      if (!found) at = k < E ? k : E - 1;
      choice[t * top + k] = at;
      score[t * top + k] = found ? r[at] : 0.0f;
      if (found) z[at] = -3.4e38f;  // never chosen again
    }
  }
  if (opt.renorm && lane == 0) {
    // the lane that wrote the chosen scores divides them by their sum, added in the order of the choices
    float sum = 0.0f;
    for (int k = 0; k < top; ++k) sum += score[t * top + k];
    sum += opt.renorm_eps;
    for (int k = 0; k < top; ++k) score[t * top + k] /= sum;
  }
}

// ---------------------------------------------------------------- 2. rows sorted by expert
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int* __restrict__ choice, int n_pairs, int E, int tile_rows,
                                                        int max_rows, int* __restrict__ row_pair,
                                                        int* __restrict__ tile_expert, int* __restrict__ n_tiles) {
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
      rows += (counts[e] + tile_rows - 1) / tile_rows * tile_rows;
    }
    first[E] = rows;
    *n_tiles = rows / tile_rows;
  }
  __syncthreads();
  for (int e = tid; e < E; e += 1024) {
    for (int tile = first[e] / tile_rows; tile < first[e + 1] / tile_rows; ++tile) tile_expert[tile] = e;
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

// ---------------------------------------------------------------- 3. / 4. on the matrix cores, few rows an expert
// A workgroup of eight waves owns a tile of 16 rows and 16 (MODE 0: gate and up) or 32 (MODE 1)
// output columns. The K loop, in steps of 64, is shared among the waves in runs that depend on K
// alone; a lane loads 32 contiguous bytes of its matrix row and of its x row a step (four lanes a
// 128-byte line), which feed two v_mfma_f32_16x16x32_bf16: the k values that lane quarter s holds
// are the same for both operands, which is all the instruction asks. The matrix is the first
// operand, so a lane ends with 4 neighbouring columns of one row. The waves' sums meet in LDS and
// are added in the waves' order. Loads are never conditional: a row or step outside the matrix
// reads a valid address and meets zeros in x.
#define MS_WAVES 8
template <int MODE>
__global__ __launch_bounds__(MS_WAVES * 64) void moe_stream_bf16_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                                        bf16_t* __restrict__ out, const int* __restrict__ row_pair,
                                                                        const int* __restrict__ tile_expert,
                                                                        const int* __restrict__ n_tiles,
                                                                        const float* __restrict__ score, int top, int K, int N,
                                                                        int use_score) {
  const int tile = blockIdx.y;
  if (tile >= *n_tiles) return;
  __shared__ float red[MS_WAVES][2][256];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, s = lane >> 4;
  const int e = tile_expert[tile];
  const int r0 = tile * MOE_TILE_ROWS;
  const int p = row_pair[r0 + c];
  const bool live = p >= 0;
  const bf16_t* xr = MODE == 0 ? x + (int64_t)(live ? p / top : 0) * K : x + (int64_t)(r0 + c) * K;
  const float sc = (MODE == 0 && use_score && live) ? score[p] : 1.0f;
  const int col0 = blockIdx.x * (MODE == 0 ? 16 : 32);
  const bf16_t* we = w + (int64_t)e * (MODE == 0 ? 2 : 1) * N * K;
  int64_t na, nb;
  if (MODE == 0) {
    const int64_t i = min((int64_t)col0 + c, (int64_t)N - 1);
    na = i;
    nb = N + i;
  } else {
    na = min((int64_t)col0 + c, (int64_t)N - 1);
    nb = min((int64_t)col0 + 16 + c, (int64_t)N - 1);
  }
  const bf16_t* wa = we + na * K;
  const bf16_t* wb = we + nb * K;
  const int steps = (K + 63) / 64;
  const int per = (steps + MS_WAVES - 1) / MS_WAVES;
  const int s_begin = wave * per, s_end = min(steps, s_begin + per);
  f32x4_t acc_a = (f32x4_t){0.0f, 0.0f, 0.0f, 0.0f}, acc_b = (f32x4_t){0.0f, 0.0f, 0.0f, 0.0f};
  bf16x8_t zero;
#pragma unroll
  for (int j = 0; j < 8; ++j) zero[j] = (__bf16)0.0f;
#pragma unroll 2
  for (int st = s_begin; st < s_end; ++st) {
    const int k = st * 64 + s * 16;
    const bool ok0 = k + 8 <= K, ok1 = k + 16 <= K;  // K is a multiple of 8
    const int k0 = ok0 ? k : 0, k1 = ok1 ? k + 8 : 0;
    const bf16x8_t a0 = *reinterpret_cast<const bf16x8_t*>(wa + k0);
    const bf16x8_t a1 = *reinterpret_cast<const bf16x8_t*>(wa + k1);
    const bf16x8_t b0 = *reinterpret_cast<const bf16x8_t*>(wb + k0);
    const bf16x8_t b1 = *reinterpret_cast<const bf16x8_t*>(wb + k1);
    bf16x8_t x0 = *reinterpret_cast<const bf16x8_t*>(xr + k0);
    bf16x8_t x1 = *reinterpret_cast<const bf16x8_t*>(xr + k1);
    if (!ok0 || !live) x0 = zero;
    if (!ok1 || !live) x1 = zero;
    if (MODE == 0 && use_score) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        x0[j] = (__bf16)((float)x0[j] * sc);
        x1[j] = (__bf16)((float)x1[j] * sc);
      }
    }
    acc_a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, x0, acc_a, 0, 0, 0);
    acc_b = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b0, x0, acc_b, 0, 0, 0);
    acc_a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, x1, acc_a, 0, 0, 0);
    acc_b = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b1, x1, acc_b, 0, 0, 0);
  }
  // lane (c, s) holds, for row c of the tile, columns 4 s .. 4 s + 3 of each set
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    red[wave][0][c * 16 + 4 * s + j] = acc_a[j];
    red[wave][1][c * 16 + 4 * s + j] = acc_b[j];
  }
  __syncthreads();
  const int tid = threadIdx.x;
  const int idx = tid & 255, set = tid >> 8;
  const int row = idx >> 4, j = idx & 15;
  const int pr = row_pair[r0 + row];
  if (MODE == 0) {
    if (set != 0) return;
    float g = 0.0f, u = 0.0f;
#pragma unroll
    for (int v = 0; v < MS_WAVES; ++v) {
      g += red[v][0][idx];
      u += red[v][1][idx];
    }
    const int col = col0 + j;
    if (col < N) out[(int64_t)(r0 + row) * N + col] = __float2bfloat16(pr >= 0 ? g / (1.0f + expf(-g)) * u : 0.0f);
  } else {
    float v = 0.0f;
#pragma unroll
    for (int q = 0; q < MS_WAVES; ++q) v += red[q][set][idx];
    const int col = col0 + set * 16 + j;
    if (pr >= 0 && col < N) out[(int64_t)pr * N + col] = __float2bfloat16(use_score ? v * score[pr] : v);
  }
}

// ---------------------------------------------------------------- 3. / 4. on the matrix cores, many rows an expert
// A workgroup of four waves owns a tile of 128 rows of one expert against 128 rows of its matrix
// (MODE 0: 64 gate rows and the 64 up rows that belong to them, a wave's 64 matrix rows being 32
// gate rows followed by their up rows, so that a lane holds both values of an output) and walks K
// in steps of 64: both tiles of a step go from global memory through registers into LDS, double
// buffered, the loads of the next step in flight while this one is multiplied. A wave owns a
// 64 x 64 quarter, 16 v_mfma_f32_16x16x32_bf16 for every 32 elements of K; LDS rows are padded by 16
// bytes. MODE 0 gathers its x rows by pair and multiplies them by the pair's score on their way
// into LDS; MODE 1 scatters its result rows to their pairs.
#define MW_BK 64
#define MW_ROW (MW_BK + 8)
#define MW_SMEM (2 * 2 * MOE_WIDE_ROWS * MW_ROW * 2)
template <int MODE>
__global__ __launch_bounds__(256, 2) void moe_wide_bf16_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                               bf16_t* __restrict__ out, const int* __restrict__ row_pair,
                                                               const int* __restrict__ tile_expert,
                                                               const int* __restrict__ n_tiles, const float* __restrict__ score,
                                                               int top, int K, int N, int use_score) {
  const int tile = blockIdx.y;
  if (tile >= *n_tiles) return;
  extern __shared__ __align__(16) unsigned char mw_smem[];
  bf16_t* As = reinterpret_cast<bf16_t*>(mw_smem);          // [2][128][MW_ROW]
  bf16_t* Bs = As + 2 * MOE_WIDE_ROWS * MW_ROW;              // [2][128][MW_ROW]
  __shared__ int pair_of[MOE_WIDE_ROWS];
  __shared__ float score_of[MOE_WIDE_ROWS];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int c = lane & 15, s = lane >> 4;
  const int tn = blockIdx.x;
  const int e = tile_expert[tile];
  const int r0 = tile * MOE_WIDE_ROWS;
  if (tid < MOE_WIDE_ROWS) {
    const int p = row_pair[r0 + tid];
    pair_of[tid] = p;
    score_of[tid] = (p >= 0 && use_score) ? score[p] : 1.0f;
  }
  __syncthreads();
  const bf16_t* we = w + (int64_t)e * (MODE == 0 ? 2 : 1) * N * K;

  // global -> registers -> LDS: thread -> 16-byte chunk (tid & 7) of rows (tid >> 3) + 32 i
  const int chunk = tid & 7, row0 = tid >> 3;
  const bf16_t* xp[4];
  const bf16_t* wp[4];
  bool xlive[4];
  float xs[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int rb = row0 + 32 * i;
    const int p = pair_of[rb];
    xlive[i] = p >= 0;
    xs[i] = score_of[rb];
    xp[i] = MODE == 0 ? x + (int64_t)(p >= 0 ? p / top : 0) * K : x + (int64_t)(r0 + rb) * K;
    int64_t n;
    if (MODE == 0) {
      const int q = rb & 63;
      const int64_t col = min((int64_t)tn * 64 + (rb >> 6) * 32 + (q & 31), (int64_t)N - 1);  // past the end: never stored
      n = q < 32 ? col : N + col;
    } else {
      n = min((int64_t)tn * 128 + rb, (int64_t)N - 1);
    }
    wp[i] = we + n * K;
  }
  u32x4_t gx[4], gw[4];
  const int k_tiles = (K + MW_BK - 1) / MW_BK;
  auto fetch = [&](int kt) __attribute__((always_inline)) {
    const int k = kt * MW_BK + chunk * 8;
    const bool ok = k + 8 <= K;        // K is a multiple of 8: a chunk is inside or outside
    const int at = ok ? k : 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      gx[i] = *reinterpret_cast<const u32x4_t*>(xp[i] + at);
      gw[i] = *reinterpret_cast<const u32x4_t*>(wp[i] + at);
      if (!ok || !xlive[i]) gx[i] = (u32x4_t){0u, 0u, 0u, 0u};
      if (!ok) gw[i] = (u32x4_t){0u, 0u, 0u, 0u};
    }
  };
  auto stash = [&](int stage) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (MODE == 0 && use_score) {  // u = score * x, rounded to bfloat16 as the other kernels round it
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float lo = cw_bf16_bits_to_float((uint16_t)(gx[i][j] & 0xffffu)) * xs[i];
          const float hi = cw_bf16_bits_to_float((uint16_t)(gx[i][j] >> 16)) * xs[i];
          gx[i][j] = (uint32_t)cw_float_to_bf16_bits(lo) | ((uint32_t)cw_float_to_bf16_bits(hi) << 16);
        }
      }
      *reinterpret_cast<u32x4_t*>(As + (stage * MOE_WIDE_ROWS + row0 + 32 * i) * MW_ROW + chunk * 8) = gx[i];
      *reinterpret_cast<u32x4_t*>(Bs + (stage * MOE_WIDE_ROWS + row0 + 32 * i) * MW_ROW + chunk * 8) = gw[i];
    }
  };

  f32x4_t acc[4][4];  // [block of 16 rows of x][block of 16 rows of the matrix]
#pragma unroll
  for (int mi = 0; mi < 4; ++mi)
#pragma unroll
    for (int ni = 0; ni < 4; ++ni) acc[mi][ni] = (f32x4_t){0.0f, 0.0f, 0.0f, 0.0f};
  auto multiply = [&](int stage) __attribute__((always_inline)) {
    const bf16_t* as = As + (stage * MOE_WIDE_ROWS + wm * 64 + c) * MW_ROW + s * 8;
    const bf16_t* bs = Bs + (stage * MOE_WIDE_ROWS + wn * 64 + c) * MW_ROW + s * 8;
#pragma unroll
    for (int kk = 0; kk < MW_BK / 32; ++kk) {
      bf16x8_t xf[4], wf[4];
#pragma unroll
      for (int mi = 0; mi < 4; ++mi) xf[mi] = *reinterpret_cast<const bf16x8_t*>(as + mi * 16 * MW_ROW + kk * 32);
#pragma unroll
      for (int ni = 0; ni < 4; ++ni) wf[ni] = *reinterpret_cast<const bf16x8_t*>(bs + ni * 16 * MW_ROW + kk * 32);
#pragma unroll
      for (int mi = 0; mi < 4; ++mi)
#pragma unroll
        for (int ni = 0; ni < 4; ++ni)
          acc[mi][ni] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[ni], xf[mi], acc[mi][ni], 0, 0, 0);
    }
  };
  fetch(0);
  stash(0);
  __syncthreads();
  for (int kt = 0; kt < k_tiles; ++kt) {
    if (kt + 1 < k_tiles) fetch(kt + 1);
    multiply(kt & 1);
    if (kt + 1 < k_tiles) stash((kt + 1) & 1);
    __syncthreads();
  }

  // lane (c, s) holds y[row wm * 64 + mi * 16 + c][columns 4 s + j of matrix block ni], j = 0..3
#pragma unroll
  for (int mi = 0; mi < 4; ++mi) {
    const int m = wm * 64 + mi * 16 + c;
    if (MODE == 0) {
#pragma unroll
      for (int ni = 0; ni < 2; ++ni) {
        const int64_t i0 = (int64_t)tn * 64 + wn * 32 + ni * 16 + 4 * s;
        if (i0 >= N) continue;
        uint16_t o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float g = acc[mi][ni][j], up = acc[mi][ni + 2][j];
          o[j] = cw_float_to_bf16_bits(g / (1.0f + expf(-g)) * up);  // a row without a pair met zeros: 0
        }
        bf16_t* dst = out + (int64_t)(r0 + m) * N + i0;
        if (i0 + 4 <= N && !(N & 3)) {
          uint2 pk;
          pk.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
          pk.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
          *reinterpret_cast<uint2*>(dst) = pk;
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (i0 + j < N) reinterpret_cast<uint16_t*>(dst)[j] = o[j];
        }
      }
    } else {
      const int p = pair_of[m];
      if (p < 0) continue;
      const float f = score_of[m];
#pragma unroll
      for (int ni = 0; ni < 4; ++ni) {
        const int64_t n0 = (int64_t)tn * 128 + wn * 64 + ni * 16 + 4 * s;
        if (n0 >= N) continue;
        uint16_t o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) o[j] = cw_float_to_bf16_bits(use_score ? acc[mi][ni][j] * f : acc[mi][ni][j]);
        bf16_t* dst = out + (int64_t)p * N + n0;
        if (n0 + 4 <= N && !(N & 3)) {
          uint2 pk;
          pk.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
          pk.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
          *reinterpret_cast<uint2*>(dst) = pk;
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (n0 + j < N) reinterpret_cast<uint16_t*>(dst)[j] = o[j];
        }
      }
    }
  }
}

// ---------------------------------------------------------------- 3a. the rows of the experts' tiles, laid out
// rows[r] = x[token of pair row_pair[r]] (times the pair's score with ``use_score``, rounded to
// bfloat16 as the other kernels round it), zeros where a row holds no pair; only the rows of the
// tiles that exist are written. For a matrix product that reads its rows as they lie (the grouped
// product of gemm_tile.hip). A workgroup takes rows in turn; 8 elements a thread.
__global__ __launch_bounds__(256) void moe_gather_bf16_kernel(const bf16_t* __restrict__ x, bf16_t* __restrict__ rows,
                                                              const int* __restrict__ row_pair,
                                                              const int* __restrict__ n_tiles, int tile_rows,
                                                              const float* __restrict__ score, int top, int K,
                                                              int use_score) {
  const int n_rows = *n_tiles * tile_rows;
  for (int r = blockIdx.x; r < n_rows; r += gridDim.x) {
    const int p = row_pair[r];
    const float f = (p >= 0 && use_score) ? score[p] : 1.0f;
    const bf16_t* src = x + (int64_t)(p >= 0 ? p / top : 0) * K;
    bf16_t* dst = rows + (int64_t)r * K;
    for (int k = threadIdx.x * 8; k < K; k += 256 * 8) {
      u32x4_t v = (u32x4_t){0u, 0u, 0u, 0u};
      if (p >= 0) {
        v = *reinterpret_cast<const u32x4_t*>(src + k);
        if (use_score) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float lo = cw_bf16_bits_to_float((uint16_t)(v[j] & 0xffffu)) * f;
            const float hi = cw_bf16_bits_to_float((uint16_t)(v[j] >> 16)) * f;
            v[j] = (uint32_t)cw_float_to_bf16_bits(lo) | ((uint32_t)cw_float_to_bf16_bits(hi) << 16);
          }
        }
      }
      *reinterpret_cast<u32x4_t*>(dst + k) = v;
    }
  }
}

// ---------------------------------------------------------------- 5. a token's pairs, added in their order
template <typename T>
__global__ void moe_combine_kernel(const T* __restrict__ y, T* __restrict__ out, int top, int H, int64_t total,
                                   const T* __restrict__ always, const float* __restrict__ always_gate, int gate_stride) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / H;
    const int j = (int)(i % H);
    float s = 0.0f;
    for (int k = 0; k < top; ++k) s += cw_to_float(y[(t * top + k) * H + j]);
    // an expert that every token uses joins last, times its gate if it has one
    if (always) s += cw_to_float(always[i]) * (always_gate ? always_gate[t * gate_stride] : 1.0f);
    out[i] = cw_from_float<T>(s);
  }
}

// ---------------------------------------------------------------- entry points
// rows of a tile by kernel: 0 plain arithmetic, 1 streaming (matrix cores), 2 wide tiles (matrix cores)
CW_EXPORT int cw_moe_tile_rows(int kernel) {
  return kernel == 3 ? MOE_GROUPED_ROWS : kernel == 2 ? MOE_WIDE_ROWS : MOE_TILE_ROWS;
}

// the most tiles that ``n_pairs`` pairs over ``E`` experts can need
CW_EXPORT int cw_moe_max_tiles(int n_pairs, int E, int tile_rows) {
  const int busy = n_pairs < E ? n_pairs : E;
  return n_pairs / tile_rows + busy;
}

CW_EXPORT int cw_moe_route(const void* x, const void* router, int dtype, int T, int H, int E, int top, int kind, int renorm,
                           int* choice, float* score, const float* correction, int groups, int groups_kept, int group_top,
                           int extra, float* extra_out, float renorm_eps, hipStream_t stream) {
  if (T < 0 || H <= 0 || E <= 0 || top <= 0 || top > E || !x || !router || !choice || !score) return CW_ERR_ARG;
  if (extra < 0 || extra > MOE_MAX_EXTRA || (extra > 0 && !extra_out)) return CW_ERR_ARG;
  if (groups > 1 && (E % groups || groups_kept < 1 || groups_kept > groups || group_top < 1 || group_top > MOE_MAX_GROUP_TOP ||
                     (E / groups) * groups_kept < top))
    return CW_ERR_ARG;
  const MoeRouteOptions opt = {correction, groups, groups_kept, group_top, extra, extra_out, renorm, renorm_eps};
  if (kind != MOE_ROUTER_SIGMOID && kind != MOE_ROUTER_SOFTMAX) return CW_ERR_ARG;
  if (E > MOE_MAX_EXPERTS) return CW_ERR_SIZE;
  if (T == 0) return CW_OK;
  if (dtype == CW_F32)
    hipLaunchKernelGGL(moe_route_kernel<float>, dim3(T), dim3(256), 0, stream, (const float*)x, (const float*)router, H, E, top,
                       kind, choice, score, opt);
  else if (dtype == CW_BF16)
    hipLaunchKernelGGL(moe_route_kernel<bf16_t>, dim3(T), dim3(256), 0, stream, (const bf16_t*)x, (const bf16_t*)router, H, E,
                       top, kind, choice, score, opt);
  else return CW_ERR_DTYPE;
  return cw_launch_status();
}

CW_EXPORT int cw_moe_plan(const int* choice, int n_pairs, int E, int tile_rows, int* row_pair, int max_rows, int* tile_expert,
                          int max_tiles, int* n_tiles, hipStream_t stream) {
  if (n_pairs < 0 || E <= 0 || !choice || !row_pair || !tile_expert || !n_tiles) return CW_ERR_ARG;
  if (tile_rows != MOE_TILE_ROWS && tile_rows != MOE_WIDE_ROWS && tile_rows != MOE_GROUPED_ROWS) return CW_ERR_ARG;
  if (E > MOE_MAX_EXPERTS) return CW_ERR_SIZE;
  if (max_tiles < cw_moe_max_tiles(n_pairs, E, tile_rows) || max_rows < max_tiles * tile_rows) return CW_ERR_ARG;
  hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), 0, stream, choice, n_pairs, E, tile_rows, max_rows, row_pair,
                     tile_expert, n_tiles);
  return cw_launch_status();
}

template <int MODE>
static int moe_wide_launch(dim3 grid, hipStream_t stream, const void* x, const void* w, void* out, const int* row_pair,
                           const int* tile_expert, const int* n_tiles, const float* score, int top, int K, int N, int use_score) {
  static bool raised = false;
  if (!raised) {
    if (hipFuncSetAttribute((const void*)moe_wide_bf16_kernel<MODE>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)MW_SMEM) != hipSuccess)
      return CW_ERR_LAUNCH;
    raised = true;
  }
  hipLaunchKernelGGL((moe_wide_bf16_kernel<MODE>), grid, dim3(256), MW_SMEM, stream, (const bf16_t*)x, (const bf16_t*)w,
                     (bf16_t*)out, row_pair, tile_expert, n_tiles, score, top, K, N, use_score);
  return cw_launch_status();
}

// mode 0: the gate/up product with the activation (silu), mode 1: the down product. ``kernel``: 0
// plain arithmetic (tiles of 16 rows, any type), 1 streaming and 2 wide tiles (bfloat16, K a
// multiple of 8; tiles of 16 and of 128 rows): the plan must have been made for the kernel's tile.
CW_EXPORT int cw_moe_expert_product(int mode, int kernel, const void* x, const void* w, void* out, int dtype,
                                    const int* row_pair, const int* tile_expert, const int* n_tiles, int max_tiles,
                                    const float* score, int top, int K, int N, int use_score, hipStream_t stream) {
  if (max_tiles < 0 || K <= 0 || N <= 0 || top <= 0 || !x || !w || !out || !row_pair || !tile_expert || !n_tiles)
    return CW_ERR_ARG;
  if (use_score && !score) return CW_ERR_ARG;
  if ((mode != 0 && mode != 1) || kernel < 0 || kernel > 2) return CW_ERR_ARG;
  if (max_tiles > 65535) return CW_ERR_SIZE;
  if (max_tiles == 0) return CW_OK;
  if (kernel != 0) {
    if (dtype != CW_BF16) return CW_ERR_DTYPE;
    if ((K & 7) || ((uintptr_t)x & 15) || ((uintptr_t)w & 15)) return CW_ERR_ARG;
    if (kernel == 1) {
      dim3 grid((N + (mode == 0 ? 15 : 31)) / (mode == 0 ? 16 : 32), max_tiles), block(MS_WAVES * 64);
      if (mode == 0)
        hipLaunchKernelGGL((moe_stream_bf16_kernel<0>), grid, block, 0, stream, (const bf16_t*)x, (const bf16_t*)w, (bf16_t*)out,
                           row_pair, tile_expert, n_tiles, score, top, K, N, use_score);
      else
        hipLaunchKernelGGL((moe_stream_bf16_kernel<1>), grid, block, 0, stream, (const bf16_t*)x, (const bf16_t*)w, (bf16_t*)out,
                           row_pair, tile_expert, n_tiles, score, top, K, N, use_score);
      return cw_launch_status();
    }
    dim3 grid((N + (mode == 0 ? 63 : 127)) / (mode == 0 ? 64 : 128), max_tiles);
    return mode == 0 ? moe_wide_launch<0>(grid, stream, x, w, out, row_pair, tile_expert, n_tiles, score, top, K, N, use_score)
                     : moe_wide_launch<1>(grid, stream, x, w, out, row_pair, tile_expert, n_tiles, score, top, K, N, use_score);
  }
  dim3 grid((N + MOE_COLS - 1) / MOE_COLS, max_tiles), block(256);
#define CW_LAUNCH(T_, M_)                                                                                              \
  hipLaunchKernelGGL((moe_expert_product_kernel<T_, M_>), grid, block, 0, stream, (const T_*)x, (const T_*)w, (T_*)out, \
                     row_pair, tile_expert, n_tiles, score, top, K, N, use_score)
  if (dtype == CW_F32 && mode == 0) CW_LAUNCH(float, 0);
  else if (dtype == CW_F32 && mode == 1) CW_LAUNCH(float, 1);
  else if (dtype == CW_BF16 && mode == 0) CW_LAUNCH(bf16_t, 0);
  else if (dtype == CW_BF16 && mode == 1) CW_LAUNCH(bf16_t, 1);
  else return CW_ERR_DTYPE;
#undef CW_LAUNCH
  return cw_launch_status();
}

// rows [max_tiles * tile_rows, K] bfloat16 = the plan's rows of x [tokens, K] as they lie, for a
// product that gathers nothing (K a multiple of 8)
CW_EXPORT int cw_moe_gather(const void* x, void* rows, int dtype, const int* row_pair, const int* n_tiles, int max_tiles,
                            int tile_rows, const float* score, int top, int K, int use_score, hipStream_t stream) {
  if (max_tiles < 0 || tile_rows <= 0 || K <= 0 || top <= 0 || !x || !rows || !row_pair || !n_tiles) return CW_ERR_ARG;
  if (use_score && !score) return CW_ERR_ARG;
  if (dtype != CW_BF16) return CW_ERR_DTYPE;
  if ((K & 7) || ((uintptr_t)x & 15) || ((uintptr_t)rows & 15)) return CW_ERR_ARG;
  if (max_tiles == 0) return CW_OK;
  int64_t blocks = (int64_t)max_tiles * tile_rows;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(moe_gather_bf16_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (const bf16_t*)x, (bf16_t*)rows,
                     row_pair, n_tiles, tile_rows, score, top, K, use_score);
  return cw_launch_status();
}

CW_EXPORT int cw_moe_combine(const void* y, void* out, int dtype, int T, int top, int H, const void* always,
                             const float* always_gate, int gate_stride, hipStream_t stream) {
  if (T < 0 || top <= 0 || H <= 0 || !y || !out || (always_gate && (!always || gate_stride < 1))) return CW_ERR_ARG;
  if (T == 0) return CW_OK;
  const int64_t total = (int64_t)T * H;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 262144) blocks = 262144;
  dim3 grid((unsigned)blocks), block(256);
  if (dtype == CW_F32) hipLaunchKernelGGL(moe_combine_kernel<float>, grid, block, 0, stream, (const float*)y, (float*)out, top, H, total,
                                           (const float*)always, always_gate, gate_stride);
  else if (dtype == CW_BF16)
    hipLaunchKernelGGL(moe_combine_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)y, (bf16_t*)out, top, H, total,
                       (const bf16_t*)always, always_gate, gate_stride);
  else return CW_ERR_DTYPE;
  return cw_launch_status();
}
