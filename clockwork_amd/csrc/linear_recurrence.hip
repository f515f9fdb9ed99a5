// A linear recurrence with a matrix state per head and a decay per key channel, for gfx950:
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T (q_scale * q_t),   S in float32 [dim, vdim],
// with the decay made inside from a low-rank projection: a_t = sigmoid(z_t)^(1/tau),
// z_t = A2 u_t + b (u_t the token's ``rank`` inputs). o_t is optionally RMS-normed over vdim
// with a weight shared by the heads and multiplied by silu(g_t).
//
// Variants (LinRecForm), for a recurrence of another family:
//   decay_kind 1:  a_t = exp(-exp(z_t)) with z_t = A2 u_t + b;  2: the same with z_t = A2 tanh(u_t) + b.
//   bonus [heads, dim]:  the output reads the state BEFORE the token joins it, and the token itself
//                  through the bonus:  o_t = (S_(t-1) + diag(bonus) k_t v_t^T)^T q_t,  then
//                  S_t = diag(a_t) S_(t-1) + k_t v_t^T.
//   norm_w_stride: vdim when every head has norm weights of its own ([heads, vdim]), else 0.
//   u, u_stride:   the decay input as rows of a tensor of its own (else columns of proj).
// q, k, v and the gate may also lie in planes one behind the other, [4][T, heads * dim]: then
// stride is the plane's row and an offset a multiple of the plane's size.
//
// A workgroup owns one (request, head): the state lives in registers for the whole portion (a
// thread holds a run of rows of one column), tokens are walked in order, sixteen at a time: their
// q, k, v and decays are staged in LDS, the walk itself has no barrier, the outputs' partial sums
// over the row runs are added, normed and gated once per sixteen tokens. Decays, their logarithms,
// the state and the norm are float32 whatever the activation type T is.
#include "common.h"

#define LR_TC 16  // tokens staged at a time

struct LinRecForm {
  int decay_kind;        // 0: sigmoid(z)^(1/tau); 1: exp(-exp(z)); 2: exp(-exp(z)) with tanh on the decay input
  const float* bonus;    // [heads, dim] or null
  int norm_w_stride;     // 0 or vdim
  const void* u;         // decay input rows, or null: columns u_off .. of proj
  int64_t u_stride;
  int state_stride;      // floats between two slots' states (>= heads * dim * vdim)
};

__device__ __forceinline__ float lr_decay(float z, int kind, float inv_tau) {
  if (kind >= 1) return expf(-expf(z));
  // log(sigmoid(z)) without cancellation, then the 1/tau-th power
  const float ls = z < 0.0f ? z - log1pf(expf(z)) : -log1pf(expf(-z));
  return expf(ls * inv_tau);
}

struct LinRecParams {
  const void* proj;   // [T, stride]: a token's q (heads * dim at q_off), k (k_off), v (heads * vdim at v_off),
  int64_t stride;     //   gate (heads * vdim at g_off, or g_off < 0) and decay input u (rank at u_off)
  int q_off, k_off, v_off, g_off, u_off;
  const void* a2;     // [heads * dim, rank], type T
  const float* a2b;   // [heads * dim] or null
  const float* norm_w;  // [vdim] or null: no norm
  float* state;       // [slots, heads, dim, vdim]
  const int* state_slots;  // [R]
  const int* cu_q;    // [R + 1]
  void* out;          // [T, heads * vdim]
  int heads, dim, vdim, rank, n_slots;
  float q_scale, inv_tau, eps;
};

template <typename T, int RPT>
__global__ __launch_bounds__(256) void linear_recurrence_kernel(LinRecParams p, LinRecForm f) {
  extern __shared__ __align__(16) float smem[];
  const int D = p.dim, V = p.vdim, Hn = p.heads;
  const int r = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int row0 = p.cu_q[r], q_len = p.cu_q[r + 1] - row0;
  const int slot = p.state_slots[r];
  if (q_len <= 0 || slot < 0 || slot >= p.n_slots) return;
  const int DS = min(256 / V, D);            // row runs: threads that share a column
  const int v = tid % V, s = tid / V;
  const bool active = s < DS;
  const int d0 = s * RPT;                    // this thread's rows d0 .. d0 + RPT - 1 (those below D)

  float* qs = smem;                 // [TC][D]
  float* ks = qs + LR_TC * D;       // [TC][D]
  float* as = ks + LR_TC * D;       // [TC][D] decays
  float* vs = as + LR_TC * D;       // [TC][V]
  float* part = vs + LR_TC * V;     // [TC][DS][V]

  float S[RPT];
  float* st = p.state + (int64_t)slot * f.state_stride + ((int64_t)h * D) * V;
  float bonus[RPT];
#pragma unroll
  for (int rr = 0; rr < RPT; ++rr) {
    S[rr] = (active && d0 + rr < D) ? st[(int64_t)(d0 + rr) * V + v] : 0.0f;
    bonus[rr] = (f.bonus && active && d0 + rr < D) ? f.bonus[h * D + d0 + rr] : 0.0f;
  }

  const T* proj = (const T*)p.proj;
  const T* a2 = (const T*)p.a2;
  T* out = (T*)p.out;
  for (int t0 = 0; t0 < q_len; t0 += LR_TC) {
    const int nt = min(LR_TC, q_len - t0);
    __syncthreads();
    for (int idx = tid; idx < nt * D; idx += 256) {
      const int t = idx / D, d = idx - t * D;
      const T* row = proj + (int64_t)(row0 + t0 + t) * p.stride;
      qs[idx] = cw_to_float(row[p.q_off + h * D + d]) * p.q_scale;
      ks[idx] = cw_to_float(row[p.k_off + h * D + d]);
      float z = p.a2b ? p.a2b[h * D + d] : 0.0f;
      const T* w = a2 + (int64_t)(h * D + d) * p.rank;
      const T* u = f.u ? (const T*)f.u + (int64_t)(row0 + t0 + t) * f.u_stride : row + p.u_off;
      if (f.decay_kind == 2) {
        for (int c = 0; c < p.rank; ++c) z += cw_to_float(w[c]) * tanhf(cw_to_float(u[c]));
      } else {
        for (int c = 0; c < p.rank; ++c) z += cw_to_float(w[c]) * cw_to_float(u[c]);
      }
      as[idx] = lr_decay(z, f.decay_kind, p.inv_tau);
    }
    for (int idx = tid; idx < nt * V; idx += 256) {
      const int t = idx / V, c = idx - t * V;
      vs[idx] = cw_to_float(proj[(int64_t)(row0 + t0 + t) * p.stride + p.v_off + h * V + c]);
    }
    __syncthreads();
    if (active) {
      for (int t = 0; t < nt; ++t) {
        const float vv = vs[t * V + v];
        float po = 0.0f;
#pragma unroll
        for (int rr = 0; rr < RPT; ++rr) {
          const int d = d0 + rr;
          if (d < D) {
            const float kv = ks[t * D + d] * vv;
            if (f.bonus) po += qs[t * D + d] * (S[rr] + bonus[rr] * kv);
            S[rr] = as[t * D + d] * S[rr] + kv;
            if (!f.bonus) po += qs[t * D + d] * S[rr];
          }
        }
        part[(t * DS + s) * V + v] = po;
      }
    }
    __syncthreads();
    // a wave per token: sum the partial outputs, norm over vdim, gate, store
    const int wave = tid >> 6, lane = tid & 63;
    for (int t = wave; t < nt; t += 4) {
      float o[4];  // vdim <= 256
      float ss = 0.0f;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = lane + u * 64;
        float sum = 0.0f;
        if (c < V)
          for (int q = 0; q < DS; ++q) sum += part[(t * DS + q) * V + c];
        o[u] = sum;
        ss += sum * sum;
      }
      float inv = 1.0f;
      if (p.norm_w) inv = 1.0f / sqrtf(cw_wave_sum(ss) / (float)V + p.eps);
      const int64_t trow = row0 + t0 + t;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = lane + u * 64;
        if (c < V) {
          float val = o[u] * inv;
          if (p.norm_w) val *= p.norm_w[h * f.norm_w_stride + c];
          if (p.g_off >= 0) {
            const float g = cw_to_float(proj[trow * p.stride + p.g_off + h * V + c]);
            val *= g / (1.0f + expf(-g));
          }
          out[trow * (int64_t)(Hn * V) + h * V + c] = cw_from_float<T>(val);
        }
      }
    }
  }
  if (active) {
#pragma unroll
    for (int rr = 0; rr < RPT; ++rr)
      if (d0 + rr < D) st[(int64_t)(d0 + rr) * V + v] = S[rr];
  }
}

// vdim up to 256; dim up to 128 rows a thread: dim <= 128 * min(256 / vdim, dim).
CW_EXPORT int cw_linear_recurrence_supported(int dim, int vdim) {
  if (dim <= 0 || vdim <= 0 || vdim > 256) return 0;
  const int ds = 256 / vdim < dim ? 256 / vdim : dim;
  return (dim + ds - 1) / ds <= 128 ? 1 : 0;
}

CW_EXPORT int cw_linear_recurrence(int dtype, const void* proj, int64_t stride, int q_off, int k_off, int v_off, int g_off,
                                   int u_off, const void* a2, const float* a2b, const float* norm_w, float* state,
                                   int n_slots, const int* state_slots, const int* cu_q, void* out, int n_requests,
                                   int heads, int dim, int vdim, int rank, float q_scale, float inv_tau, float eps,
                                   int decay_kind, const float* bonus, int norm_w_stride, const void* u, int64_t u_stride,
                                   int64_t state_stride, hipStream_t stream) {
  if (n_requests < 0 || !proj || !a2 || !state || !state_slots || !cu_q || !out) return CW_ERR_ARG;
  if (heads <= 0 || rank <= 0 || n_slots <= 0 || q_off < 0 || k_off < 0 || v_off < 0 || u_off < 0 || stride <= 0) return CW_ERR_ARG;
  if (q_off % stride + heads * dim > stride || k_off % stride + heads * dim > stride || v_off % stride + heads * vdim > stride ||
      (!u && u_off + rank > stride) || (g_off >= 0 && g_off % stride + heads * vdim > stride))
    return CW_ERR_ARG;
  if (decay_kind < 0 || decay_kind > 2 || (norm_w_stride != 0 && norm_w_stride != vdim) || (u && u_stride < rank) ||
      state_stride < (int64_t)heads * dim * vdim || state_stride > 0x7fffffff)
    return CW_ERR_ARG;
  if (!cw_linear_recurrence_supported(dim, vdim)) return CW_ERR_SIZE;
  const LinRecForm form = {decay_kind, bonus, norm_w_stride, u, u_stride, (int)state_stride};
  if (n_requests == 0) return CW_OK;
  if (heads > 65535) return CW_ERR_SIZE;
  LinRecParams p;
  p.proj = proj; p.stride = stride; p.q_off = q_off; p.k_off = k_off; p.v_off = v_off; p.g_off = g_off; p.u_off = u_off;
  p.a2 = a2; p.a2b = a2b; p.norm_w = norm_w; p.state = state; p.state_slots = state_slots; p.cu_q = cu_q; p.out = out;
  p.heads = heads; p.dim = dim; p.vdim = vdim; p.rank = rank; p.n_slots = n_slots;
  p.q_scale = q_scale; p.inv_tau = inv_tau; p.eps = eps;
  const int ds = 256 / vdim < dim ? 256 / vdim : dim;
  const int rpt = (dim + ds - 1) / ds;
  const size_t smem = ((size_t)LR_TC * (3 * dim + vdim) + (size_t)LR_TC * ds * vdim) * sizeof(float);
  dim3 grid(n_requests, heads), block(256);
#define CW_LAUNCH(T_, RPT_)                                                                                        \
  do {                                                                                                             \
    if (smem > 48 * 1024 && hipFuncSetAttribute((const void*)linear_recurrence_kernel<T_, RPT_>,                   \
                                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) \
      return CW_ERR_LAUNCH;                                                                                        \
    hipLaunchKernelGGL((linear_recurrence_kernel<T_, RPT_>), grid, block, smem, stream, p, form);                        \
  } while (0)
#define CW_BY_ROWS(T_)                         \
  do {                                         \
    if (rpt <= 2) CW_LAUNCH(T_, 2);            \
    else if (rpt <= 4) CW_LAUNCH(T_, 4);       \
    else if (rpt <= 8) CW_LAUNCH(T_, 8);       \
    else if (rpt <= 16) CW_LAUNCH(T_, 16);     \
    else if (rpt <= 32) CW_LAUNCH(T_, 32);     \
    else if (rpt <= 64) CW_LAUNCH(T_, 64);     \
    else CW_LAUNCH(T_, 128);                   \
  } while (0)
  if (dtype == CW_F32) CW_BY_ROWS(float);
  else if (dtype == CW_BF16) CW_BY_ROWS(bf16_t);
  else return CW_ERR_DTYPE;
#undef CW_BY_ROWS
#undef CW_LAUNCH
  return cw_launch_status();
}

// ======================================================================================
// The same recurrence for long portions, cut into segments of tokens that run side by side.
//
//   prepare:   per token and key channel the decay a (float32, through log-sigmoid), the scaled
//              query and the key as float32 rows [T, heads * dim]: the walks below read them
//              with addresses that do not depend on the lane, so they arrive in scalar registers.
//   segments:  every (segment, head) walks its tokens from a zero state: what the segment adds to
//              the state (float32 [dim, vdim]) and the product of its decays per channel.
//   carry:     per request and head, segment after segment: start(s + 1) = decay(s) * start(s) +
//              added(s), from the request's state slot; the last one is the slot's new state.
//   outputs:   every (segment, head) walks its tokens again from its start state: o_t = S_t^T q_t.
//   finish:    RMS norm over vdim, weight, silu(gate), cast: one wave per (token, head).
//
// In the walks a thread owns one column of the state with all its rows in registers (dim <= 128),
// a wave 64 columns; nothing is exchanged between threads. The sums are the same as in the
// token-by-token kernel but for the place of the parentheses: S_t = A S_start + (local sum).
// ======================================================================================
#define LRS_MAX_DIM 128

struct SegParams {
  const void* proj;
  int64_t stride;
  int q_off, k_off, v_off, g_off, u_off;
  const void* a2;
  const float* a2b;
  const float* norm_w;
  float* state;
  const int* state_slots;
  const int* cu_q;
  const int* seg_items;   // [n_segments, 4]: request, first token of the segment (in the portion), tokens, index of the segment in its request
  const int* req_first;   // [R + 1]: first segment of each request in seg_items
  float* dec;             // [T, heads * dim] decays
  float* qf;              // [T, heads * dim]
  float* kf;              // [T, heads * dim]
  float* added;           // [n_segments, heads, dim, vdim]
  float* seg_decay;       // [n_segments, heads, dim]
  float* raw;             // [T, heads * vdim] outputs before norm and gate
  void* out;
  int heads, dim, vdim, rank, n_slots, n_tokens;
  float q_scale, inv_tau, eps;
  int seg_tokens;         // the most tokens a segment has
  LinRecForm form;
};

template <typename T> struct LrVec;
template <> struct LrVec<float> {
  static constexpr int N = 4;
  __device__ static void load(const float* p, float* o) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
  }
};
template <> struct LrVec<bf16_t> {
  static constexpr int N = 8;
  __device__ static void load(const bf16_t* p, float* o) {
    const uint4 v = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) { o[2 * i] = __uint_as_float(w[i] << 16); o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u); }
  }
};

template <typename T>
__global__ __launch_bounds__(256) void lrs_prepare_kernel(SegParams p) {
  const int HD = p.heads * p.dim;
  const int64_t n = (int64_t)p.n_tokens * HD;
  const T* proj = (const T*)p.proj;
  const T* a2 = (const T*)p.a2;
  constexpr int N = LrVec<T>::N;
  const bool vec = p.rank % N == 0 && !((uintptr_t)a2 & 15) &&
                   (p.form.u ? p.form.u_stride % N == 0 && !((uintptr_t)p.form.u & 15)
                             : p.u_off % N == 0 && p.stride % N == 0 && !((uintptr_t)proj & 15));
  for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * 256) {
    const int64_t t = idx / HD;
    const int c = (int)(idx - t * HD);
    const T* row = proj + t * p.stride;
    float z = p.a2b ? p.a2b[c] : 0.0f;
    const T* w = a2 + (int64_t)c * p.rank;
    const T* u = p.form.u ? (const T*)p.form.u + t * p.form.u_stride : row + p.u_off;
    if (p.form.decay_kind == 2) {
      for (int e = 0; e < p.rank; ++e) z += cw_to_float(w[e]) * tanhf(cw_to_float(u[e]));
    } else if (vec) {  // 16 bytes of the decay matrix's row and of the token's decay input at a time
      for (int e = 0; e < p.rank; e += N) {
        float wv[N], uv[N];
        LrVec<T>::load(w + e, wv);
        LrVec<T>::load(u + e, uv);
#pragma unroll
        for (int i = 0; i < N; ++i) z += wv[i] * uv[i];
      }
    } else {
      for (int e = 0; e < p.rank; ++e) z += cw_to_float(w[e]) * cw_to_float(u[e]);
    }
    p.dec[idx] = lr_decay(z, p.form.decay_kind, p.inv_tau);
    p.qf[idx] = cw_to_float(row[p.q_off + c]) * p.q_scale;
    p.kf[idx] = cw_to_float(row[p.k_off + c]);
  }
}

// MODE 0: from zero, leaves ``added`` and ``seg_decay``; MODE 1: from the start state in ``added``
// (the carry kernel has turned it into that), writes the raw outputs.
template <typename T, int DIM, int MODE>
__global__ __launch_bounds__(256) void lrs_walk_kernel(SegParams p) {
  extern __shared__ __align__(16) float tile[];  // the segment's decays, keys and queries: [3][tokens][D]
  const int seg = blockIdx.x, h = blockIdx.y;
  const int v = blockIdx.z * blockDim.x + threadIdx.x;
  const int r = p.seg_items[4 * seg], tok0 = p.seg_items[4 * seg + 1], ntok = p.seg_items[4 * seg + 2];
  const int q_len = p.cu_q[r + 1] - p.cu_q[r];
  const int slot = p.state_slots[r];
  if (tok0 >= q_len || slot < 0 || slot >= p.n_slots) return;
  const int nt = min(ntok, q_len - tok0);
  const int64_t row0 = p.cu_q[r] + tok0;
  const int D = p.dim, V = p.vdim, HD = p.heads * p.dim;
  const bool live = v < V;
  const int vc = live ? v : V - 1;
  float S[DIM];
  float* mine = p.added + (((int64_t)seg * p.heads + h) * D) * V;
  if (MODE == 1) {
#pragma unroll
    for (int d = 0; d < DIM; ++d) S[d] = d < D ? mine[(int64_t)d * V + vc] : 0.0f;
  } else {
#pragma unroll
    for (int d = 0; d < DIM; ++d) S[d] = 0.0f;
  }
  float A[MODE == 0 ? DIM : 1];
  if (MODE == 0) {
#pragma unroll
    for (int d = 0; d < DIM; ++d) A[d] = 1.0f;
  }
  const T* proj = (const T*)p.proj;
  // the waves of the workgroup (each 64 columns of the same head's state) share the segment's
  // decays, keys and queries through LDS: fetched once, in whole rows, then read by every lane at
  // the same address (a broadcast) while the tokens are walked
  float* As = tile;
  float* Kt = As + p.seg_tokens * D;
  float* Qt = Kt + p.seg_tokens * D;
  for (int i = threadIdx.x; i < nt * D; i += blockDim.x) {
    const int t = i / D, d = i - t * D;
    const int64_t at = (row0 + t) * HD + h * D + d;
    As[i] = p.dec[at];
    Kt[i] = p.kf[at];
    if (MODE == 1) Qt[i] = p.qf[at];
  }
  __syncthreads();
  // with a bonus the token's own share of its output is one number a token whatever the state's
  // column, (sum over d of q_d bonus_d k_d) v: lane t of every wave sums token t's, once a segment,
  // and hands it to the others when the token's turn comes (a segment has at most 64 tokens)
  float own = 0.0f;
  if (MODE == 1 && p.form.bonus) {
    const int lane = threadIdx.x & 63;
    if (lane < nt) {
      const float* bn = p.form.bonus + h * D;
      for (int i = 0; i < D; ++i) {
        const int d = (i + lane) % D;   // every lane a bank of its own
        own += Qt[lane * D + d] * bn[d] * Kt[lane * D + d];
      }
    }
  }
  const bool reads_before = MODE == 1 && p.form.bonus != nullptr;   // the output reads the state before the token joins it
  for (int t = 0; t < nt; ++t) {
    const int64_t row = row0 + t;
    const float* a = As + t * D;
    const float* k = Kt + t * D;
    const float* q = Qt + t * D;
    const float vv = cw_to_float(proj[row * p.stride + p.v_off + h * V + vc]);
    float o0 = 0.0f, o1 = 0.0f, o2 = 0.0f, o3 = 0.0f;
    if (reads_before) {
      o0 = __shfl(own, t, 64) * vv;
#pragma unroll
      for (int d = 0; d < DIM; d += 4) {
        if (d < D) {
          o0 += q[d] * S[d];
          o1 += q[d + 1] * S[d + 1];
          o2 += q[d + 2] * S[d + 2];
          o3 += q[d + 3] * S[d + 3];
          S[d] = a[d] * S[d] + k[d] * vv;
          S[d + 1] = a[d + 1] * S[d + 1] + k[d + 1] * vv;
          S[d + 2] = a[d + 2] * S[d + 2] + k[d + 2] * vv;
          S[d + 3] = a[d + 3] * S[d + 3] + k[d + 3] * vv;
        }
      }
    } else {
#pragma unroll
      for (int d = 0; d < DIM; d += 4) {
        if (d < D) {  // D is a multiple of 4 here (the host sees to it)
          S[d] = a[d] * S[d] + k[d] * vv;
          S[d + 1] = a[d + 1] * S[d + 1] + k[d + 1] * vv;
          S[d + 2] = a[d + 2] * S[d + 2] + k[d + 2] * vv;
          S[d + 3] = a[d + 3] * S[d + 3] + k[d + 3] * vv;
          if (MODE == 1) {
            o0 += q[d] * S[d];
            o1 += q[d + 1] * S[d + 1];
            o2 += q[d + 2] * S[d + 2];
            o3 += q[d + 3] * S[d + 3];
          } else if (threadIdx.x == 0 && blockIdx.z == 0) {
            A[d] *= a[d]; A[d + 1] *= a[d + 1]; A[d + 2] *= a[d + 2]; A[d + 3] *= a[d + 3];
          }
        }
      }
    }
    if (MODE == 1 && live) p.raw[row * (int64_t)(p.heads * V) + h * V + v] = (o0 + o1) + (o2 + o3);
  }
  if (MODE == 0) {
    if (live) {
#pragma unroll
      for (int d = 0; d < DIM; ++d)
        if (d < D) mine[(int64_t)d * V + v] = S[d];
    }
    if (threadIdx.x == 0 && blockIdx.z == 0) {
      float* sd = p.seg_decay + ((int64_t)seg * p.heads + h) * D;
#pragma unroll
      for (int d = 0; d < DIM; ++d)
        if (d < D) sd[d] = A[d];
    }
  }
}

// per (request, head, 256 state elements): walk the request's segments in order
__global__ __launch_bounds__(256) void lrs_carry_kernel(SegParams p) {
  const int r = blockIdx.x, h = blockIdx.y;
  const int64_t e = (int64_t)blockIdx.z * 256 + threadIdx.x;  // element d * V + v
  const int D = p.dim, V = p.vdim;
  const int slot = p.state_slots[r];
  const int q_len = p.cu_q[r + 1] - p.cu_q[r];
  if (e >= (int64_t)D * V || slot < 0 || slot >= p.n_slots || q_len <= 0) return;
  const int d = (int)(e / V);
  float* st = p.state + (int64_t)slot * p.form.state_stride + ((int64_t)h * D) * V + e;
  float S = *st;
  for (int seg = p.req_first[r]; seg < p.req_first[r + 1]; ++seg) {
    if (p.seg_items[4 * seg + 1] >= q_len) break;  // segments past the request's tokens (a batch of fixed shape)
    float* mine = p.added + (((int64_t)seg * p.heads + h) * D) * V + e;
    const float add = *mine;
    *mine = S;  // the segment's start state, for the second walk
    S = p.seg_decay[((int64_t)seg * p.heads + h) * D + d] * S + add;
  }
  *st = S;
}

template <typename T>
__global__ __launch_bounds__(256) void lrs_finish_kernel(SegParams p) {
  const int V = p.vdim, Hn = p.heads;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * 4 + wave;  // (token, head)
  if (item >= (int64_t)p.n_tokens * Hn) return;
  const int64_t t = item / Hn;
  const int h = (int)(item - t * Hn);
  const float* o = p.raw + t * (int64_t)(Hn * V) + h * V;
  float ss = 0.0f;
  for (int c = lane; c < V; c += 64) ss += o[c] * o[c];
  float inv = 1.0f;
  if (p.norm_w) inv = 1.0f / sqrtf(cw_wave_sum(ss) / (float)V + p.eps);
  const T* proj = (const T*)p.proj;
  T* out = (T*)p.out;
  for (int c = lane; c < V; c += 64) {
    float val = o[c] * inv;
    if (p.norm_w) val *= p.norm_w[h * p.form.norm_w_stride + c];
    if (p.g_off >= 0) {
      const float g = cw_to_float(proj[t * p.stride + p.g_off + h * V + c]);
      val *= g / (1.0f + expf(-g));
    }
    out[t * (int64_t)(Hn * V) + h * V + c] = cw_from_float<T>(val);
  }
}

// dim a multiple of 4 up to 128
CW_EXPORT int cw_linear_recurrence_segments_supported(int dim, int vdim) {
  return dim > 0 && dim <= LRS_MAX_DIM && dim % 4 == 0 && vdim > 0 ? 1 : 0;
}

// floats of workspace: dec, qf, kf [T, heads * dim] each, added [segments, heads, dim, vdim],
// seg_decay [segments, heads, dim], raw [T, heads * vdim]
CW_EXPORT int64_t cw_linear_recurrence_segments_workspace_floats(int n_tokens, int n_segments, int heads, int dim, int vdim) {
  return 3 * (int64_t)n_tokens * heads * dim + (int64_t)n_segments * heads * dim * (vdim + 1) + (int64_t)n_tokens * heads * vdim;
}

CW_EXPORT int cw_linear_recurrence_segments(int dtype, const void* proj, int64_t stride, int q_off, int k_off, int v_off,
                                            int g_off, int u_off, const void* a2, const float* a2b, const float* norm_w,
                                            float* state, int n_slots, const int* state_slots, const int* cu_q,
                                            const int* seg_items, int n_segments, int seg_tokens, const int* req_first, float* workspace,
                                            void* out, int n_requests, int n_tokens, int heads, int dim, int vdim, int rank,
                                            float q_scale, float inv_tau, float eps, int decay_kind, const float* bonus,
                                            int norm_w_stride, const void* u, int64_t u_stride, int64_t state_stride,
                                            hipStream_t stream) {
  if (n_requests < 0 || n_tokens < 0 || n_segments < 0 || !proj || !a2 || !state || !state_slots || !cu_q || !seg_items ||
      !req_first || !workspace || !out)
    return CW_ERR_ARG;
  if (heads <= 0 || rank <= 0 || n_slots <= 0 || q_off < 0 || k_off < 0 || v_off < 0 || u_off < 0 || stride <= 0) return CW_ERR_ARG;
  if (q_off % stride + heads * dim > stride || k_off % stride + heads * dim > stride || v_off % stride + heads * vdim > stride ||
      (!u && u_off + rank > stride) || (g_off >= 0 && g_off % stride + heads * vdim > stride))
    return CW_ERR_ARG;
  if (decay_kind < 0 || decay_kind > 2 || (norm_w_stride != 0 && norm_w_stride != vdim) || (u && u_stride < rank) ||
      state_stride < (int64_t)heads * dim * vdim || state_stride > 0x7fffffff)
    return CW_ERR_ARG;
  if (!cw_linear_recurrence_segments_supported(dim, vdim)) return CW_ERR_SIZE;
  if (heads > 65535 || (vdim + 63) / 64 > 65535) return CW_ERR_SIZE;
  if (seg_tokens < 1 || (int64_t)3 * seg_tokens * dim * 4 > 48 * 1024 || (bonus && seg_tokens > 64)) return CW_ERR_SIZE;
  if (n_requests == 0 || n_tokens == 0 || n_segments == 0) return CW_OK;
  SegParams p;
  p.proj = proj; p.stride = stride; p.q_off = q_off; p.k_off = k_off; p.v_off = v_off; p.g_off = g_off; p.u_off = u_off;
  p.a2 = a2; p.a2b = a2b; p.norm_w = norm_w; p.state = state; p.state_slots = state_slots; p.cu_q = cu_q;
  p.seg_items = seg_items; p.req_first = req_first; p.out = out;
  p.heads = heads; p.dim = dim; p.vdim = vdim; p.rank = rank; p.n_slots = n_slots; p.n_tokens = n_tokens;
  p.q_scale = q_scale; p.inv_tau = inv_tau; p.eps = eps;
  p.form = LinRecForm{decay_kind, bonus, norm_w_stride, u, u_stride, (int)state_stride};
  const int64_t THD = (int64_t)n_tokens * heads * dim;
  p.dec = workspace; p.qf = p.dec + THD; p.kf = p.qf + THD;
  p.added = p.kf + THD;
  p.seg_decay = p.added + (int64_t)n_segments * heads * dim * vdim;
  p.raw = p.seg_decay + (int64_t)n_segments * heads * dim;
  int64_t pb = (THD + 255) / 256;
  if (pb > 65536) pb = 65536;
  p.seg_tokens = seg_tokens;
  const int walk_threads = vdim >= 256 ? 256 : 64 * ((vdim + 63) / 64);   // up to four waves share a segment's rows
  const dim3 walk_grid(n_segments, heads, (vdim + walk_threads - 1) / walk_threads);
  const size_t walk_lds = (size_t)3 * seg_tokens * dim * sizeof(float);
  const dim3 carry_grid(n_requests, heads, (unsigned)(((int64_t)dim * vdim + 255) / 256));
  const unsigned finish_blocks = (unsigned)(((int64_t)n_tokens * heads + 3) / 4);
#define CW_WALK(T_, DIM_)                                                                          \
  do {                                                                                             \
    hipLaunchKernelGGL((lrs_walk_kernel<T_, DIM_, 0>), walk_grid, dim3(walk_threads), walk_lds, stream, p); \
    hipLaunchKernelGGL(lrs_carry_kernel, carry_grid, dim3(256), 0, stream, p);                     \
    hipLaunchKernelGGL((lrs_walk_kernel<T_, DIM_, 1>), walk_grid, dim3(walk_threads), walk_lds, stream, p); \
  } while (0)
#define CW_ALL(T_)                                                                                 \
  do {                                                                                             \
    hipLaunchKernelGGL((lrs_prepare_kernel<T_>), dim3((unsigned)pb), dim3(256), 0, stream, p);     \
    if (dim <= 16) CW_WALK(T_, 16);                                                                \
    else if (dim <= 32) CW_WALK(T_, 32);                                                           \
    else if (dim <= 64) CW_WALK(T_, 64);                                                           \
    else CW_WALK(T_, 128);                                                                         \
    hipLaunchKernelGGL((lrs_finish_kernel<T_>), dim3(finish_blocks), dim3(256), 0, stream, p);     \
  } while (0)
  if (dtype == CW_F32) CW_ALL(float);
  else if (dtype == CW_BF16) CW_ALL(bf16_t);
  else return CW_ERR_DTYPE;
#undef CW_ALL
#undef CW_WALK
  return cw_launch_status();
}
