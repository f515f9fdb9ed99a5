// Softmax attention over paged rows whose keys and values have widths of their own, with the
// options that plain grouped attention lacks:
//
//   * maps:   a query head may carry M score maps (M = 1 or 2). Queries are laid out [head][map][dim],
//             a token's key row [kv head][map][dim], its value row [kv head][vdim]; every map is a
//             softmax of its own over the same values. With two maps the head's output is
//             A_0 - lambda * A_1 (lambda one float32 on the device).
//   * alias:  the values are the first vdim elements of the key row (a cached latent that serves
//             as key and as value); then there is one plane and M = 1.
//   * mask:   causal; a window of W positions (a token sees itself and the W - 1 before it); or
//             segments of C positions counted from position 0 (a token sees the earlier tokens of
//             its own segment). With a window, the first ``keep_first`` positions of a request
//             stay visible to every later token, at their true positions.
//   * cap:    scores are squashed before the softmax: cap * tanh(scale * q . k / cap).
//   * gate:   a head's output is multiplied by the logistic function of one number a token and head.
//   * sink:   exp(sink[head]) joins the softmax denominator (no key, no value, not scaled).
//   * norm:   the head's output is divided by its root mean square over vdim (eps inside the
//             root) and multiplied by a constant.
//
// Scores, softmax statistics, weights and the norm are float32 in both element types.
#include "common.h"

#define RA_ROWS 16          // (token, head, map) rows of a workgroup
#define RA_MAXC 32          // value columns a thread owns: vdim <= 16 * RA_MAXC
#define RA_MASK_CAUSAL 0
#define RA_MASK_WINDOW 1
#define RA_MASK_SEGMENTS 2

struct RowsAttnParams {
  const void* q;           // query (t, head, map, d) at t * q_stride + head * q_head_stride + map * dim + d
  int64_t q_stride, q_head_stride;
  void* out;               // output (t, head, c) at t * out_stride + head * out_head_stride + c
  int64_t out_stride, out_head_stride;
  const void* k_plane;     // [cache rows, k_row]
  const void* v_plane;     // [cache rows, v_row] (== k_plane with alias)
  int k_row, v_row;        // elements a token's row holds in each plane
  int64_t cache_rows;
  const int* block_tables; // [requests, table_width]
  int table_width;
  const int* ctx_lens;     // keys a request has after this step
  const int* cu_q;         // first token row of each request, [requests + 1]
  const int* items;        // (request, first token, tokens, 0)
  const float* sink;       // [heads] or nullptr
  const float* lambda;     // one float (maps == 2) or nullptr
  int heads, kv_heads, dim, vdim, maps;
  int heads_per_group;     // heads of a key/value head that one workgroup takes (<= RA_ROWS / maps)
  int tokens_per_item;     // RA_ROWS / (heads_per_group * maps)
  int key_chunk;           // keys a tile holds: 16, 32 or 64
  int block_size, mask_kind, mask_size;
  float scale;
  int head_norm;           // 0 / 1
  float norm_eps, post_mult;
  int keep_first;          // with a window: positions below this one are seen from anywhere later
  float softcap;           // > 0: score <- softcap * tanh(score / softcap)
  const void* gate;        // or nullptr: head h of token t is multiplied by logistic(gate[t * gate_stride + gate_off + h])
  int64_t gate_stride;
  int gate_off;
};

template <typename T>
__device__ __forceinline__ float ra_head_gate(const RowsAttnParams& p, int64_t token_row, int head) {
  if (!p.gate) return 1.0f;
  const float z = cw_to_float(((const T*)p.gate)[token_row * p.gate_stride + p.gate_off + head]);
  return 1.0f / (1.0f + expf(-z));
}

__host__ __device__ inline int ra_key_stride(int maps, int dim) { return maps * dim + 1; }

// floats of LDS: queries, key tile, value tile (none with alias), weights
static inline size_t ra_lds_floats(int maps, int dim, int vdim, int key_chunk, int alias) {
  return (size_t)RA_ROWS * dim + (size_t)key_chunk * ra_key_stride(maps, dim) + (alias ? 0 : (size_t)key_chunk * vdim) +
         (size_t)RA_ROWS * key_chunk;
}

template <typename T>
__global__ __launch_bounds__(256) void rows_attention_kernel(const RowsAttnParams p) {
  extern __shared__ __align__(16) float smem[];
  const int M = p.maps, D = p.dim, V = p.vdim, KC = p.key_chunk;
  const int kstride = ra_key_stride(M, D);
  const bool alias = p.v_plane == p.k_plane;
  float* qs = smem;                                   // [RA_ROWS][D]
  float* ks = qs + RA_ROWS * D;                       // [KC][kstride]
  float* vs = alias ? ks : ks + (size_t)KC * kstride; // [KC][V] (alias: the key tile, stride kstride)
  const int vstride = alias ? kstride : V;
  float* ps = (alias ? ks + (size_t)KC * kstride : vs + (size_t)KC * V);  // [RA_ROWS][KC]

  const int tid = threadIdx.x, row = tid >> 4, sub = tid & 15;
  const int* item = p.items + 4 * (int64_t)blockIdx.x;
  const int req = item[0], tok0 = item[1];
  const int g = blockIdx.y;                             // key/value head
  const int group = p.heads / p.kv_heads;
  const int HC = p.heads_per_group;
  const int h0 = blockIdx.z * HC;                       // first head of the group that this workgroup takes
  const int nh_here = min(HC, group - h0);
  const int rows_per_token = HC * M;
  const int ctx = p.ctx_lens[req];
  const int q_len = p.cu_q[req + 1] - p.cu_q[req];
  if (tok0 >= q_len) return;  // an item past the request's tokens (a batch of fixed shape)
  const int ntok = min(min(item[2], p.tokens_per_item), q_len - tok0);
  const int pos0 = ctx - q_len + tok0;                  // position of the item's first token
  // this thread's row
  const int tl = row / rows_per_token, hl = (row % rows_per_token) / M, m = row % M;
  const bool live = tl < ntok && hl < nh_here;
  const int head = g * group + h0 + (live ? hl : 0);
  const int64_t trow = (int64_t)p.cu_q[req] + tok0 + (live ? tl : 0);
  const int pos = pos0 + (live ? tl : 0);
  int lo = 0;
  if (p.mask_kind == RA_MASK_WINDOW) lo = max(0, pos - p.mask_size + 1);
  else if (p.mask_kind == RA_MASK_SEGMENTS) lo = (pos / p.mask_size) * p.mask_size;
  // the keys the workgroup walks: from the oldest that its first token sees to its last token
  int first = 0;
  if (p.mask_kind == RA_MASK_WINDOW) first = max(0, pos0 - p.mask_size + 1);
  else if (p.mask_kind == RA_MASK_SEGMENTS) first = (pos0 / p.mask_size) * p.mask_size;
  const int last = pos0 + ntok - 1;

  // queries into LDS as float32
  {
    const T* q = (const T*)p.q;
    for (int i = tid; i < RA_ROWS * D; i += 256) {
      const int r = i / D, d = i % D;
      const int rt = r / rows_per_token, rh = (r % rows_per_token) / M, rm = r % M;
      float v = 0.0f;
      if (rt < ntok && rh < nh_here)
        v = cw_to_float(q[((int64_t)p.cu_q[req] + tok0 + rt) * p.q_stride + (int64_t)(g * group + h0 + rh) * p.q_head_stride +
                          rm * D + d]);
      qs[i] = v;
    }
  }
  float run_max = -3.0e38f, run_sum = 0.0f;
  if (p.sink) { run_max = p.sink[head]; run_sum = 1.0f; }
  float acc[RA_MAXC];
#pragma unroll
  for (int i = 0; i < RA_MAXC; ++i) acc[i] = 0.0f;
  const int* table = p.block_tables + (int64_t)req * p.table_width;
  const T* kp = (const T*)p.k_plane;
  const T* vp = (const T*)p.v_plane;
  const int KI = KC >> 4;

  // the kept first positions that lie before the walk's oldest key are a stretch of their own
  const int kept_end = (p.mask_kind == RA_MASK_WINDOW && p.keep_first > 0) ? min(p.keep_first, first) : 0;
  const float inv_cap = p.softcap > 0.0f ? 1.0f / p.softcap : 0.0f;
  for (int stretch = kept_end > 0 ? 0 : 1; stretch < 2; ++stretch) {
  const int begin = stretch == 0 ? 0 : first, end = stretch == 0 ? kept_end - 1 : last;
  for (int k0 = begin; k0 <= end; k0 += KC) {
    __syncthreads();  // the tile of the round before has been read (and the queries are written)
    const int width = M * D;
    for (int i = tid; i < KC * width; i += 256) {
      const int j = i / width, d = i % width;
      const int key = k0 + j;
      float v = 0.0f;
      if (key <= end) {
        const int page = table[key / p.block_size];
        const int64_t slot = (int64_t)page * p.block_size + key % p.block_size;
        if (page >= 0 && slot < p.cache_rows) v = cw_to_float(kp[slot * p.k_row + (int64_t)g * width + d]);
      }
      ks[j * kstride + d] = v;
    }
    if (!alias) {
      for (int i = tid; i < KC * V; i += 256) {
        const int j = i / V, c = i % V;
        const int key = k0 + j;
        float v = 0.0f;
        if (key <= end) {
          const int page = table[key / p.block_size];
          const int64_t slot = (int64_t)page * p.block_size + key % p.block_size;
          if (page >= 0 && slot < p.cache_rows) v = cw_to_float(vp[slot * p.v_row + (int64_t)g * V + c]);
        }
        vs[j * V + c] = v;
      }
    }
    __syncthreads();
    // scores of this thread's row against keys sub, sub + 16, ...
    float s[4];
    float tile_max = -3.0e38f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      s[i] = -INFINITY;
      if (i < KI) {
        const int j = sub + 16 * i;
        const int key = k0 + j;
        const float* qrow = qs + row * D;
        const float* krow = ks + j * kstride + m * D;
        float dot = 0.0f;
        for (int d = 0; d < D; ++d) dot += qrow[d] * krow[d];
        if (live && key <= min(pos, end) && (key >= lo || key < p.keep_first)) {
          s[i] = dot * p.scale;
          if (p.softcap > 0.0f) s[i] = p.softcap * tanhf(s[i] * inv_cap);
          tile_max = fmaxf(tile_max, s[i]);
        }
      }
    }
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) tile_max = fmaxf(tile_max, __shfl_xor(tile_max, off, 64));
    const float new_max = fmaxf(run_max, tile_max);
    const float alpha = expf(run_max - new_max);
    float tile_sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (i < KI) {
        const float w = (s[i] == -INFINITY) ? 0.0f : expf(s[i] - new_max);
        tile_sum += w;
        ps[row * KC + sub + 16 * i] = w;
      }
    }
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) tile_sum += __shfl_xor(tile_sum, off, 64);
    run_sum = run_sum * alpha + tile_sum;
    run_max = new_max;
    __syncthreads();
    const float* prow = ps + row * KC;
#pragma unroll
    for (int i = 0; i < RA_MAXC; ++i) {
      const int c = sub + 16 * i;
      if (c < V) {
        float a = acc[i] * alpha;
        for (int j = 0; j < KC; ++j) a += prow[j] * vs[j * vstride + c];
        acc[i] = a;
      }
    }
  }
  }
  // a row that saw no key and has no sink cannot happen: every token sees itself
  const float inv = run_sum > 0.0f ? 1.0f / run_sum : 0.0f;
  const float lam = (M == 2 && p.lambda) ? p.lambda[0] : 0.0f;
  float sq = 0.0f;
#pragma unroll
  for (int i = 0; i < RA_MAXC; ++i) {
    const int c = sub + 16 * i;
    float o = acc[i] * inv;
    if (M == 2) {
      // rows of the two maps of one head are neighbours: 16 lanes apart
      const float other = __shfl_xor(o, 16, 64);
      o = o - lam * other;
    }
    if (c < V) sq += o * o;
    acc[i] = o;
  }
  float mult = 1.0f;
  if (p.head_norm) {
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) sq += __shfl_xor(sq, off, 64);
    mult = p.post_mult / sqrtf(sq / (float)V + p.norm_eps);
  }
  if (live && m == 0) {
    mult *= ra_head_gate<T>(p, trow, head);
    T* o = (T*)p.out + trow * p.out_stride + (int64_t)head * p.out_head_stride;
#pragma unroll
    for (int i = 0; i < RA_MAXC; ++i) {
      const int c = sub + 16 * i;
      if (c < V) o[c] = cw_from_float<T>(acc[i] * mult);
    }
  }
}

// The largest key tile (64, 32 or 16 keys) whose LDS fits; 0: the geometry is beyond the kernel.
CW_EXPORT int cw_rows_attention_key_chunk(int maps, int dim, int vdim, int alias) {
  if (maps < 1 || maps > 2 || dim < 1 || vdim < 1 || vdim > 16 * RA_MAXC) return 0;
  if (alias && (maps != 1 || vdim > dim)) return 0;
  for (int kc = 64; kc >= 16; kc >>= 1) {
    const size_t bytes = ra_lds_floats(maps, dim, vdim, kc, alias) * sizeof(float);
    // two workgroups a compute unit where that is to be had, else one
    if (bytes <= (kc == 16 ? 150u : 64u) * 1024u) return kc;
  }
  return 0;
}

// Heads of a key/value head that one workgroup takes, and from that the tokens of an item.
CW_EXPORT int cw_rows_attention_heads_per_group(int heads, int kv_heads, int maps) {
  if (heads < 1 || kv_heads < 1 || heads % kv_heads || maps < 1 || maps > 2) return 0;
  const int group = heads / kv_heads;
  return group < RA_ROWS / maps ? group : RA_ROWS / maps;
}
CW_EXPORT int cw_rows_attention_tokens_per_item(int heads, int kv_heads, int maps) {
  const int hc = cw_rows_attention_heads_per_group(heads, kv_heads, maps);
  return hc ? RA_ROWS / (hc * maps) : 0;
}

CW_EXPORT int cw_rows_attention(int dtype, const void* q, int64_t q_stride, int64_t q_head_stride, void* out,
                                int64_t out_stride, int64_t out_head_stride, const void* k_plane,
                                const void* v_plane, int k_row, int v_row, int64_t cache_rows,
                                const int* block_tables, int table_width, const int* ctx_lens, const int* cu_q,
                                const int* items, int n_items, const float* sink, const float* lambda, int heads,
                                int kv_heads, int dim, int vdim, int maps, int block_size, int mask_kind,
                                int mask_size, float scale, int head_norm, float norm_eps, float post_mult,
                                int keep_first, float softcap, const void* gate, int64_t gate_stride, int gate_off,
                                hipStream_t stream) {
  if (n_items < 0 || !q || !out || !k_plane || !v_plane || !block_tables || !ctx_lens || !cu_q || !items)
    return CW_ERR_ARG;
  if (block_size <= 0 || table_width <= 0 || mask_kind < 0 || mask_kind > 2 || (mask_kind != 0 && mask_size < 1))
    return CW_ERR_ARG;
  if (maps == 2 && !lambda) return CW_ERR_ARG;
  if (keep_first < 0 || (keep_first > 0 && mask_kind != RA_MASK_WINDOW) || softcap < 0.0f) return CW_ERR_ARG;
  const int alias = v_plane == k_plane;
  const int kc = cw_rows_attention_key_chunk(maps, dim, vdim, alias);
  const int hc = cw_rows_attention_heads_per_group(heads, kv_heads, maps);
  if (kc == 0 || hc == 0) return CW_ERR_SIZE;
  if (k_row < kv_heads * maps * dim || (!alias && v_row < kv_heads * vdim)) return CW_ERR_ARG;
  if (q_stride < 1 || q_head_stride < 1 || out_stride < 1 || out_head_stride < 1) return CW_ERR_ARG;
  if (n_items == 0) return CW_OK;
  RowsAttnParams p;
  p.q = q; p.q_stride = q_stride; p.q_head_stride = q_head_stride; p.out = out; p.out_stride = out_stride;
  p.out_head_stride = out_head_stride; p.k_plane = k_plane; p.v_plane = v_plane; p.k_row = k_row;
  p.v_row = alias ? k_row : v_row; p.cache_rows = cache_rows; p.block_tables = block_tables; p.table_width = table_width;
  p.ctx_lens = ctx_lens; p.cu_q = cu_q; p.items = items; p.sink = sink; p.lambda = lambda; p.heads = heads;
  p.kv_heads = kv_heads; p.dim = dim; p.vdim = vdim; p.maps = maps; p.heads_per_group = hc;
  p.tokens_per_item = RA_ROWS / (hc * maps); p.key_chunk = kc; p.block_size = block_size; p.mask_kind = mask_kind;
  p.mask_size = mask_size; p.scale = scale; p.head_norm = head_norm; p.norm_eps = norm_eps; p.post_mult = post_mult;
  p.keep_first = keep_first; p.softcap = softcap; p.gate = gate; p.gate_stride = gate_stride; p.gate_off = gate_off;
  if (gate && (gate_stride < 1 || gate_off < 0)) return CW_ERR_ARG;
  const size_t smem = ra_lds_floats(maps, dim, vdim, kc, alias) * sizeof(float);
  const int group = heads / kv_heads;
  dim3 grid(n_items, kv_heads, (group + hc - 1) / hc), block(256);
#define CW_LAUNCH(T_)                                                                                             \
  do {                                                                                                            \
    if (smem > 48 * 1024 && hipFuncSetAttribute((const void*)rows_attention_kernel<T_>,                           \
                                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) \
      return CW_ERR_LAUNCH;                                                                                       \
    hipLaunchKernelGGL((rows_attention_kernel<T_>), grid, block, smem, stream, p);                                \
  } while (0)
  if (dtype == CW_F32) CW_LAUNCH(float);
  else if (dtype == CW_BF16) CW_LAUNCH(bf16_t);
  else return CW_ERR_DTYPE;
#undef CW_LAUNCH
  return cw_launch_status();
}

// ======================================================================================
// bfloat16 on the matrix cores, for portions and single tokens alike.
//
// A workgroup takes up to 16 tokens of one request (the 16 columns of its score tiles), one
// key/value head, up to four (two maps) or 4 * UPW (one map) query heads of that head's group,
// VW = 16 * NT of the value columns, and one of gridDim.z runs of the keys. A wave holds UPW
// "units": with two maps the two maps of one head, else UPW heads. Keys come in chunks of 32
// through LDS (row-major for the scores, the values transposed for the value product); the next
// chunk is fetched into registers while this one is multiplied.
//
// Scores are made as K Q^T (v_mfma_f32_16x16x32_bf16): a lane then holds, for ITS query
// (lane % 16), the keys 4 * slot + e and 16 + 4 * slot + e of the chunk (slot = lane / 16), which is
// the A operand of the value product as it lies in the registers; the value fragments are read
// with the keys in that order. Softmax in units of log 2 with a running maximum per query, float32;
// the weights enter the value product rounded to bfloat16, sums are float32.
//
// With one run of keys the workgroup finishes its heads itself (denominator, the two maps'
// difference, the head norm); with several, every run leaves maximum, denominator and
// unnormalised sums in a workspace and rows_merge_kernel finishes.
// ======================================================================================
typedef __attribute__((ext_vector_type(8))) __bf16 ra_bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float ra_f32x4_t;
typedef __attribute__((ext_vector_type(4))) short ra_s16x4_t;
typedef __attribute__((address_space(3))) ra_s16x4_t ra_lds_s16x4_t;
#define RM_KT 32

__device__ __forceinline__ ra_bf16x8_t ra_load8(const bf16_t* p) { return *reinterpret_cast<const ra_bf16x8_t*>(p); }

struct RowsMfmaExtra {
  float* workspace;     // [items][gridDim.y][runs][4 waves][UPW][16 queries][2 + VW] when runs > 1
  int head_chunks;      // workgroups that share the heads of a key/value head's group
  int v_splits;         // workgroups that share the value columns
  int heads_per_wg;     // 4 (two maps) or 4 * UPW
};

__device__ __forceinline__ int ra_oldest_seen(int kind, int size, int pos) {
  if (kind == RA_MASK_WINDOW) return max(0, pos - size + 1);
  if (kind == RA_MASK_SEGMENTS) return (pos / size) * size;
  return 0;
}

// ALIAS: the values are columns of the key tile (one plane, one map): no value tile, no value loads.
template <int D32, int NT, int UPW, int MAPS, bool ALIAS>
__global__ __launch_bounds__(256) void rows_mfma_kernel(const RowsAttnParams p, const RowsMfmaExtra x) {
  extern __shared__ __align__(16) unsigned char ra_smem[];
  constexpr int D = D32 * 32, DA = D * MAPS, VW = NT * 16;
  // rows of both tiles are padded so that the 16-byte reads of key fragments and the 8-byte
  // transposing reads of value fragments spread over the banks
  constexpr int KROW = DA + 8, VROW = VW + 16;
  constexpr int KPR = DA / 8, VPR = VW / 8;
  constexpr int PFK = (RM_KT * KPR + 255) / 256, PFV = ALIAS ? 1 : (RM_KT * VPR + 255) / 256;
  static_assert(MAPS == 1 || UPW == 2, "two maps: a wave holds the two maps of one head");
  static_assert(!ALIAS || MAPS == 1, "values inside the key row: one map");
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int l16 = lane & 15, slot = lane >> 4;
  // items come with a request's tokens in order; the last ones see the most keys and go first
  const int* item = p.items + 4 * (int64_t)(gridDim.x - 1 - blockIdx.x);
  const int req = item[0], tok0 = item[1];
  const int q_len = p.cu_q[req + 1] - p.cu_q[req];
  if (tok0 >= q_len) return;  // an item past the request's tokens (a batch of fixed shape)
  const int nq = min(min(item[2], 16), q_len - tok0);
  const int pos0 = p.ctx_lens[req] - q_len + tok0;
  const int last = pos0 + nq - 1;
  const int first = ra_oldest_seen(p.mask_kind, p.mask_size, pos0);
  const int lo_last = ra_oldest_seen(p.mask_kind, p.mask_size, last);
  const int64_t row0 = (int64_t)p.cu_q[req] + tok0;
  const int* table = p.block_tables + (int64_t)req * p.table_width;

  const int vs = blockIdx.y % x.v_splits;
  const int hc = (blockIdx.y / x.v_splits) % x.head_chunks;
  const int g = blockIdx.y / (x.v_splits * x.head_chunks);
  const int group = p.heads / p.kv_heads;
  const int h0 = hc * x.heads_per_wg;
  const int nh_here = min(x.heads_per_wg, group - h0);
  const int v0 = vs * VW;

  bf16_t* Ks = reinterpret_cast<bf16_t*>(ra_smem);   // [RM_KT][KROW]
  bf16_t* Vs = Ks + RM_KT * KROW;                    // [RM_KT][VROW], row-major (not with ALIAS)
  const bf16_t* q = (const bf16_t*)p.q;
  const bf16_t* kc = (const bf16_t*)p.k_plane;
  const bf16_t* vc = (const bf16_t*)p.v_plane;

  // this wave's units: (head of the group, map)
  int unit_head[UPW];
  bool unit_ok[UPW];
  ra_bf16x8_t qf[UPW][D32];
  const int qi = min(l16, nq - 1);
#pragma unroll
  for (int a = 0; a < UPW; ++a) {
    const int hl = MAPS == 2 ? wave : wave + 4 * a;
    const int map = MAPS == 2 ? a : 0;
    unit_ok[a] = hl < nh_here;
    unit_head[a] = g * group + h0 + min(hl, nh_here - 1);
    const bf16_t* qrow = q + (row0 + qi) * p.q_stride + (int64_t)unit_head[a] * p.q_head_stride + map * D + slot * 8;
#pragma unroll
    for (int ks = 0; ks < D32; ++ks) qf[a][ks] = ra_load8(qrow + ks * 32);
  }

  // this workgroup's run of the key chunks. Behind a window that keeps a request's first
  // positions visible, those of them that lie before the window's oldest key are chunks of their own,
  // walked first; ``kept_end`` ends them.
  const int kept_end = (p.mask_kind == RA_MASK_WINDOW && p.keep_first > 0) ? min(p.keep_first, first) : 0;
  const int kept_chunks = (kept_end + RM_KT - 1) / RM_KT;
  const int n_chunks = kept_chunks + (last - first) / RM_KT + 1;
  const int runs = gridDim.z;
  const int per_run = (n_chunks + runs - 1) / runs;
  const int c_begin = blockIdx.z * per_run, c_end = min(n_chunks, c_begin + per_run);
  auto chunk_start = [&](int c) -> int { return c < kept_chunks ? c * RM_KT : first + (c - kept_chunks) * RM_KT; };
  auto chunk_limit = [&](int c) -> int { return c < kept_chunks ? kept_end - 1 : last; };

  uint4 kreg[PFK], vreg[PFV];
  // A chunk's cache rows are looked up once, by 32 threads, and wait in LDS (two chunks' worth):
  // a lookup inside the fetch would put a load of the page table before every load of a row, and
  // since loads come home in order each row's load would wait for all the loads before it.
  __shared__ int chunk_rows[2][RM_KT];
  auto row_of = [&](int c, int i) -> int {
    const int j = chunk_start(c) + i;
    if (j > chunk_limit(c)) return -1;
    const int b = j / p.block_size;
    const int page = b < p.table_width ? table[b] : -1;
    const int64_t row = (int64_t)page * p.block_size + j % p.block_size;
    return (page >= 0 && row < p.cache_rows) ? (int)row : -1;
  };
  auto fetch = [&](const int* rows_of_chunk) {
#pragma unroll
    for (int it = 0; it < PFK; ++it) {
      const int idx = tid + it * 256;
      const int at = min(idx, RM_KT * KPR - 1);
      const int e = at % KPR, jj = at / KPR;
      const int row = rows_of_chunk[jj];
      const uint4 v = *reinterpret_cast<const uint4*>(kc + (int64_t)(row >= 0 ? row : 0) * p.k_row + (int64_t)g * DA + e * 8);
      kreg[it] = (row >= 0 && idx == at) ? v : make_uint4(0, 0, 0, 0);
    }
    if constexpr (!ALIAS) {
#pragma unroll
      for (int it = 0; it < PFV; ++it) {
        const int idx = tid + it * 256;
        const int at = min(idx, RM_KT * VPR - 1);
        const int e = at % VPR, jj = at / VPR;
        const int row = rows_of_chunk[jj];
        const uint4 v = *reinterpret_cast<const uint4*>(vc + (int64_t)(row >= 0 ? row : 0) * p.v_row + (int64_t)g * p.vdim + v0 + e * 8);
        vreg[it] = (row >= 0 && idx == at) ? v : make_uint4(0, 0, 0, 0);
      }
    }
  };
  auto store = [&]() {
#pragma unroll
    for (int it = 0; it < PFK; ++it) {
      const int idx = tid + it * 256;
      if (idx < RM_KT * KPR) *reinterpret_cast<uint4*>(Ks + (idx / KPR) * KROW + (idx % KPR) * 8) = kreg[it];
    }
    if constexpr (!ALIAS) {
#pragma unroll
      for (int it = 0; it < PFV; ++it) {
        const int idx = tid + it * 256;
        if (idx < RM_KT * VPR) *reinterpret_cast<uint4*>(Vs + (idx / VPR) * VROW + (idx % VPR) * 8) = vreg[it];
      }
    }
  };

  constexpr float LOG2E = 1.4426950408889634f;
  const float scale2 = p.scale * LOG2E;
  // the cap in units of log 2 as well: cap * tanh(score / cap) * log2(e)
  const float cap2 = p.softcap * LOG2E, inv_cap2 = p.softcap > 0.0f ? 1.0f / cap2 : 0.0f;
  float m[UPW], l[UPW];
  ra_f32x4_t out[UPW][NT];
#pragma unroll
  for (int a = 0; a < UPW; ++a) {
    // the sink counts once: in the first run of the keys
    const bool sink_here = p.sink != nullptr && blockIdx.z == 0;
    m[a] = sink_here ? p.sink[unit_head[a]] * LOG2E : -3.0e38f;
    l[a] = (sink_here && slot == 0) ? 1.0f : 0.0f;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) out[a][nt] = ra_f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
  }
  // where this lane's value fragments begin: the transposing read (ds_read_b64_tr_b16) hands lane i
  // of a group of 16 element i % 4 of what lanes i / 4, 4 + i / 4, 8 + i / 4 and 12 + i / 4 address; with
  // lane i pointing at key 4 * slot + i / 4, columns 4 * (i % 4) .. + 4 of a 16-wide block, every lane
  // receives its column (i) of the keys 4 * slot .. + 4: the order in which it holds its weights
  const bf16_t* vlane = ALIAS ? Ks + (4 * slot + (l16 >> 2)) * KROW + v0 + 4 * (l16 & 3)
                              : Vs + (4 * slot + (l16 >> 2)) * VROW + 4 * (l16 & 3);
  constexpr int VSTRIDE = ALIAS ? KROW : VROW;

  if (c_begin < c_end) {
    if (tid < RM_KT) chunk_rows[0][tid] = row_of(c_begin, tid);
    if (tid >= 64 && tid < 64 + RM_KT && c_begin + 1 < c_end) chunk_rows[1][tid - 64] = row_of(c_begin + 1, tid - 64);
    __syncthreads();
    fetch(chunk_rows[0]);
  }
  for (int c = c_begin; c < c_end; ++c) {
    const int k0 = chunk_start(c), limit = chunk_limit(c);
    __syncthreads();   // the tiles of the chunk before have been read; the rows of the next chunk are written
    store();
    if (c + 1 < c_end) fetch(chunk_rows[(c + 1 - c_begin) & 1]);
    __syncthreads();
    // the rows of the chunk after the next: looked up now, written at the end of this round
    int later_row = -1;
    const bool looks_up = tid < RM_KT && c + 2 < c_end;
    if (looks_up) later_row = row_of(c + 2, tid);
    // a chunk whose keys every query of the item sees needs no tests
    const bool inside = nq == 16 && k0 + RM_KT - 1 <= min(pos0, limit) && (k0 >= lo_last || c < kept_chunks);
    ra_bf16x8_t pw[UPW];
#pragma unroll
    for (int a = 0; a < UPW; ++a) {
      const int map = MAPS == 2 ? a : 0;
      ra_f32x4_t acc0 = {0.0f, 0.0f, 0.0f, 0.0f}, acc1 = {0.0f, 0.0f, 0.0f, 0.0f};
      const bf16_t* kb = Ks + l16 * KROW + map * D + slot * 8;
#pragma unroll
      for (int ks = 0; ks < D32; ++ks) {
        acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ra_load8(kb + ks * 32), qf[a][ks], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ra_load8(kb + 16 * KROW + ks * 32), qf[a][ks], acc1, 0, 0, 0);
      }
      const int pos = pos0 + l16;
      const int lo = ra_oldest_seen(p.mask_kind, p.mask_size, pos);
      float s[8];
      float top = -INFINITY;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int j = k0 + (u >> 2) * 16 + slot * 4 + (u & 3);
        float v = (u < 4 ? acc0[u & 3] : acc1[u & 3]) * scale2;
        if (p.softcap > 0.0f) v = cap2 * tanhf(v * inv_cap2);
        if (!inside) v = (l16 < nq && j <= min(pos, limit) && (j >= lo || j < p.keep_first)) ? v : -INFINITY;
        s[u] = v;
        top = fmaxf(top, v);
      }
      top = cw_quad_max(top);
      const float mn = fmaxf(m[a], top);
      const float alpha = __builtin_amdgcn_exp2f(m[a] - mn);
      m[a] = mn;
      float sum = 0.0f;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const float w = __builtin_amdgcn_exp2f(s[u] - mn);
        sum += w;
        pw[a][u] = (__bf16)w;
      }
      l[a] = l[a] * alpha + sum;
      // the accumulators' rows are queries slot * 4 + e: each takes its own query's factor
      if (__ballot(alpha != 1.0f) != 0) {
        float ar[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) ar[e] = __shfl(alpha, slot * 4 + e, 64);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
          for (int e = 0; e < 4; ++e) out[a][nt][e] *= ar[e];
      }
    }
    // values: a fragment (16 value columns, 32 keys) serves all of the wave's units
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const bf16_t* vp = vlane + nt * 16;
      const ra_s16x4_t f0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((ra_lds_s16x4_t*)vp);
      const ra_s16x4_t f1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((ra_lds_s16x4_t*)(vp + 16 * VSTRIDE));
      const ra_bf16x8_t vf = __builtin_bit_cast(ra_bf16x8_t, __builtin_shufflevector(f0, f1, 0, 1, 2, 3, 4, 5, 6, 7));
#pragma unroll
      for (int a = 0; a < UPW; ++a) out[a][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pw[a], vf, out[a][nt], 0, 0, 0);
    }
    if (looks_up) chunk_rows[(c - c_begin) & 1][tid] = later_row;   // this chunk's rows were last read before this round's second barrier
  }

  if (runs > 1) {
    // maximum, denominator and unnormalised sums of this run, per unit and query
    const int64_t wg = ((int64_t)(gridDim.x - 1 - blockIdx.x) * gridDim.y + blockIdx.y) * runs + blockIdx.z;
    float* base = x.workspace + wg * (4 * UPW * 16 * (2 + VW));
#pragma unroll
    for (int a = 0; a < UPW; ++a) {
      const float total = cw_quad_sum(l[a]);
      float* u = base + (int64_t)(wave * UPW + a) * 16 * (2 + VW);
      if (slot == 0) { u[l16 * (2 + VW)] = m[a]; u[l16 * (2 + VW) + 1] = total; }
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int e = 0; e < 4; ++e) u[(slot * 4 + e) * (2 + VW) + 2 + nt * 16 + l16] = out[a][nt][e];
    }
    return;
  }

  // ---- finish: denominators, the two maps' difference, the head norm
  float inv_row[UPW][4];
#pragma unroll
  for (int a = 0; a < UPW; ++a) {
    const float total = cw_quad_sum(l[a]);
    const float inv = total > 0.0f ? 1.0f / total : 0.0f;
#pragma unroll
    for (int e = 0; e < 4; ++e) inv_row[a][e] = __shfl(inv, slot * 4 + e, 64);
  }
  const float lam = (MAPS == 2 && p.lambda) ? p.lambda[0] : 0.0f;
  constexpr int OUTS = MAPS == 2 ? 1 : UPW;
  bf16_t* o = (bf16_t*)p.out;
#pragma unroll
  for (int a = 0; a < OUTS; ++a) {
    float sq[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float v = out[a][nt][e] * inv_row[a][e];
        if (MAPS == 2) v -= lam * out[UPW - 1][nt][e] * inv_row[UPW - 1][e];
        out[a][nt][e] = v;
        sq[e] += v * v;
      }
    float mult[4] = {1.0f, 1.0f, 1.0f, 1.0f};
    if (p.head_norm) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
#pragma unroll
        for (int off = 8; off > 0; off >>= 1) sq[e] += __shfl_xor(sq[e], off, 64);
        mult[e] = p.post_mult / sqrtf(sq[e] / (float)p.vdim + p.norm_eps);
      }
    }
    if (unit_ok[a]) {
      if (p.gate) {
#pragma unroll
        for (int e = 0; e < 4; ++e) mult[e] *= ra_head_gate<bf16_t>(p, row0 + min(slot * 4 + e, nq - 1), unit_head[a]);
      }
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int i = slot * 4 + e;
          if (i < nq)
            o[(row0 + i) * p.out_stride + (int64_t)unit_head[a] * p.out_head_stride + v0 + nt * 16 + l16] =
                __float2bfloat16(out[a][nt][e] * mult[e]);
        }
    }
  }
}

// Puts the runs of rows_mfma_kernel together: one workgroup per (item, key/value head x head chunk x
// value split, head of the chunk); per query of the item a thread takes the value columns tid,
// tid + 256.
template <int MAPS>
__global__ __launch_bounds__(256) void rows_merge_kernel(const RowsAttnParams p, const RowsMfmaExtra x, int runs, int upw,
                                                         int vw) {
  __shared__ float scratch[4];
  const int tid = threadIdx.x;
  const int* item = p.items + 4 * (int64_t)blockIdx.x;
  const int req = item[0], tok0 = item[1];
  const int q_len = p.cu_q[req + 1] - p.cu_q[req];
  if (tok0 >= q_len) return;
  const int nq = min(min(item[2], 16), q_len - tok0);
  const int64_t row0 = (int64_t)p.cu_q[req] + tok0;
  const int vs = blockIdx.y % x.v_splits;
  const int hc = (blockIdx.y / x.v_splits) % x.head_chunks;
  const int g = blockIdx.y / (x.v_splits * x.head_chunks);
  const int group = p.heads / p.kv_heads;
  const int h0 = hc * x.heads_per_wg;
  const int hl = blockIdx.z;
  if (hl >= min(x.heads_per_wg, group - h0)) return;
  const int head = g * group + h0 + hl;
  const int v0 = vs * vw;
  const int stride_q = 2 + vw, stride_unit = 16 * stride_q;
  const int64_t stride_run = (int64_t)4 * upw * stride_unit;
  const float* base = x.workspace + ((int64_t)blockIdx.x * gridDim.y + blockIdx.y) * runs * stride_run;
  const float lam = (MAPS == 2 && p.lambda) ? p.lambda[0] : 0.0f;
  bf16_t* o = (bf16_t*)p.out;
  __shared__ float run_stats[2][64][2];   // per map and run: maximum (in units of log 2) and denominator
  for (int qi = 0; qi < nq; ++qi) {
    float val[2] = {0.0f, 0.0f};
    // every run's maximum and denominator, fetched side by side
    __syncthreads();
    if (tid < MAPS * runs) {
      const int map = tid / runs, r = tid % runs;
      const int unit = MAPS == 2 ? hl * upw + map : (hl % 4) * upw + hl / 4;
      const float* u = base + (int64_t)unit * stride_unit + qi * stride_q + r * stride_run;
      run_stats[map][r][0] = u[0];
      run_stats[map][r][1] = u[1];
    }
    __syncthreads();
#pragma unroll
    for (int map = 0; map < MAPS; ++map) {
      // the unit's place in a run's block: (wave, a)
      const int unit = MAPS == 2 ? hl * upw + map : (hl % 4) * upw + hl / 4;
      const float* u = base + (int64_t)unit * stride_unit + qi * stride_q;
      float top = -3.0e38f;
      for (int r = 0; r < runs; ++r) top = fmaxf(top, run_stats[map][r][0]);
      float den = 0.0f, part[2] = {0.0f, 0.0f};
#pragma unroll 4
      for (int r = 0; r < runs; ++r) {
        const float* ur = u + r * stride_run;
        const float f = __builtin_amdgcn_exp2f(run_stats[map][r][0] - top);
        den += run_stats[map][r][1] * f;
#pragma unroll
        for (int i = 0; i < 2; ++i)
          if (tid + 256 * i < vw) part[i] += ur[2 + tid + 256 * i] * f;
      }
      const float inv = den > 0.0f ? 1.0f / den : 0.0f;
#pragma unroll
      for (int i = 0; i < 2; ++i) val[i] += (map == 0 ? 1.0f : -lam) * part[i] * inv;
    }
    float mult = 1.0f;
    if (p.head_norm) {
      float sq = cw_wave_sum(val[0] * val[0] + val[1] * val[1]);   // columns past vw hold zeros
      __syncthreads();
      if ((tid & 63) == 0) scratch[tid >> 6] = sq;
      __syncthreads();
      sq = (scratch[0] + scratch[1]) + (scratch[2] + scratch[3]);
      mult = p.post_mult / sqrtf(sq / (float)p.vdim + p.norm_eps);
    }
    mult *= ra_head_gate<bf16_t>(p, row0 + qi, head);
#pragma unroll
    for (int i = 0; i < 2; ++i)
      if (tid + 256 * i < vw)
        o[(row0 + qi) * p.out_stride + (int64_t)head * p.out_head_stride + v0 + tid + 256 * i] = __float2bfloat16(val[i] * mult);
  }
}

// How the matrix-core kernel cuts a geometry: value columns a workgroup takes (16 * nt), how many
// workgroups share the columns, units a wave holds; 0 in *nt: not taken. Two maps: key rows of 64
// or 128 elements a map, value rows of 64, 128 or 256 (the head norm needs all columns in one
// workgroup). One map with values of their own: the same key and value sizes. One map with the values inside the key row: key rows of 160, 320 or 576 elements,
// values their first 128, 256 or 512.
static void ra_mfma_shape(int maps, int dim, int vdim, int alias, int* d32, int* nt, int* v_splits, int* upw) {
  *nt = 0; *v_splits = 1; *upw = maps == 2 ? 2 : 1; *d32 = dim / 32;
  if (dim % 32) return;
  if (maps == 2 && !alias) {
    if (*d32 != 2 && *d32 != 4) return;
    if (vdim == 64) *nt = 4; else if (vdim == 128) *nt = 8; else if (vdim == 256) *nt = 16;
  } else if (maps == 1 && !alias) {
    // a wave holds two heads: eight heads of a key/value head's group a workgroup
    if (*d32 != 2 && *d32 != 4) return;
    *upw = 2;
    if (vdim == 64) *nt = 4; else if (vdim == 128) *nt = 8; else if (vdim == 256) *nt = 16;
  } else if (maps == 1 && alias) {
    if (*d32 == 5 && vdim == 128) *nt = 8;
    else if (*d32 == 10 && vdim == 256) *nt = 16;
    else if (*d32 == 18 && vdim == 512) *nt = 32;
  }
}

CW_EXPORT int cw_rows_mfma_supported(int maps, int dim, int vdim, int alias) {
  int d32, nt, vsp, upw;
  ra_mfma_shape(maps, dim, vdim, alias, &d32, &nt, &vsp, &upw);
  return nt != 0;
}

// Workgroups of one run of keys: (items, y); and the floats of workspace that ``runs`` runs need.
CW_EXPORT int cw_rows_mfma_grid_y(int heads, int kv_heads, int maps, int dim, int vdim, int alias) {
  int d32, nt, vsp, upw;
  ra_mfma_shape(maps, dim, vdim, alias, &d32, &nt, &vsp, &upw);
  if (!nt || heads % kv_heads) return 0;
  const int per_wg = maps == 2 ? 4 : 4 * upw, group = heads / kv_heads;
  return kv_heads * ((group + per_wg - 1) / per_wg) * vsp;
}
CW_EXPORT int64_t cw_rows_mfma_workspace_floats(int n_items, int heads, int kv_heads, int maps, int dim, int vdim, int alias,
                                                int runs) {
  int d32, nt, vsp, upw;
  ra_mfma_shape(maps, dim, vdim, alias, &d32, &nt, &vsp, &upw);
  if (!nt || runs <= 1) return 0;
  return (int64_t)n_items * cw_rows_mfma_grid_y(heads, kv_heads, maps, dim, vdim, alias) * runs * 4 * upw * 16 * (2 + 16 * nt);
}

CW_EXPORT int cw_rows_attention_mfma(const void* q, int64_t q_stride, int64_t q_head_stride, void* out, int64_t out_stride,
                                     int64_t out_head_stride, const void* k_plane, const void* v_plane, int k_row, int v_row,
                                     int64_t cache_rows, const int* block_tables, int table_width, const int* ctx_lens,
                                     const int* cu_q, const int* items, int n_items, const float* sink, const float* lambda,
                                     int heads, int kv_heads, int dim, int vdim, int maps, int block_size, int mask_kind,
                                     int mask_size, float scale, int head_norm, float norm_eps, float post_mult, int runs,
                                     float* workspace, int64_t workspace_floats, int keep_first, float softcap,
                                     const void* gate, int64_t gate_stride, int gate_off, hipStream_t stream) {
  if (n_items < 0 || !q || !out || !k_plane || !v_plane || !block_tables || !ctx_lens || !cu_q || !items) return CW_ERR_ARG;
  if (block_size <= 0 || table_width <= 0 || mask_kind < 0 || mask_kind > 2 || (mask_kind != 0 && mask_size < 1)) return CW_ERR_ARG;
  if ((maps == 2 && !lambda) || runs < 1 || runs > 64) return CW_ERR_ARG;
  if (keep_first < 0 || (keep_first > 0 && mask_kind != RA_MASK_WINDOW) || softcap < 0.0f) return CW_ERR_ARG;
  const int alias = v_plane == k_plane;
  int d32, nt, vsp, upw;
  ra_mfma_shape(maps, dim, vdim, alias, &d32, &nt, &vsp, &upw);
  if (!nt || heads % kv_heads) return CW_ERR_SIZE;
  if (alias && (maps != 1 || kv_heads != 1 || vdim > dim)) return CW_ERR_ARG;
  if (head_norm && vsp != 1) return CW_ERR_ARG;
  // 16-byte loads: rows and heads begin at multiples of 8 elements
  if (q_stride % 8 || q_head_stride % 8 || k_row % 8 || (!alias && v_row % 8) || ((uintptr_t)q | (uintptr_t)k_plane | (uintptr_t)v_plane) % 16)
    return CW_ERR_ARG;
  if (k_row < kv_heads * maps * dim || (!alias && v_row < kv_heads * vdim)) return CW_ERR_ARG;
  if (runs > 1 && (!workspace || workspace_floats < cw_rows_mfma_workspace_floats(n_items, heads, kv_heads, maps, dim, vdim, alias, runs)))
    return CW_ERR_ARG;
  if (n_items == 0) return CW_OK;
  RowsAttnParams p;
  p.q = q; p.q_stride = q_stride; p.q_head_stride = q_head_stride; p.out = out; p.out_stride = out_stride;
  p.out_head_stride = out_head_stride; p.k_plane = k_plane; p.v_plane = v_plane; p.k_row = k_row;
  p.v_row = alias ? k_row : v_row; p.cache_rows = cache_rows; p.block_tables = block_tables; p.table_width = table_width;
  p.ctx_lens = ctx_lens; p.cu_q = cu_q; p.items = items; p.sink = sink; p.lambda = lambda; p.heads = heads;
  p.kv_heads = kv_heads; p.dim = dim; p.vdim = vdim; p.maps = maps; p.heads_per_group = 0; p.tokens_per_item = 16;
  p.key_chunk = RM_KT; p.block_size = block_size; p.mask_kind = mask_kind; p.mask_size = mask_size; p.scale = scale;
  p.head_norm = head_norm; p.norm_eps = norm_eps; p.post_mult = post_mult; p.keep_first = keep_first; p.softcap = softcap;
  p.gate = gate; p.gate_stride = gate_stride; p.gate_off = gate_off;
  if (gate && (gate_stride < 1 || gate_off < 0)) return CW_ERR_ARG;
  RowsMfmaExtra x;
  x.workspace = workspace; x.v_splits = vsp; x.heads_per_wg = maps == 2 ? 4 : 4 * upw;
  const int group = heads / kv_heads;
  x.head_chunks = (group + x.heads_per_wg - 1) / x.heads_per_wg;
  dim3 grid(n_items, kv_heads * x.head_chunks * vsp, runs), block(256);
  const size_t smem = ((size_t)RM_KT * (maps * dim + 8) + (alias ? 0 : (size_t)RM_KT * (16 * nt + 16))) * 2;
#define CW_LAUNCH(D32_, NT_, UPW_, MAPS_, ALIAS_)                                                                  \
  do {                                                                                                             \
    if (smem > 48 * 1024 && hipFuncSetAttribute((const void*)rows_mfma_kernel<D32_, NT_, UPW_, MAPS_, ALIAS_>,     \
                                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) \
      return CW_ERR_LAUNCH;                                                                                        \
    hipLaunchKernelGGL((rows_mfma_kernel<D32_, NT_, UPW_, MAPS_, ALIAS_>), grid, block, smem, stream, p, x);       \
  } while (0)
  if (maps == 2) {
    if (d32 == 2 && nt == 4) CW_LAUNCH(2, 4, 2, 2, false);
    else if (d32 == 2 && nt == 8) CW_LAUNCH(2, 8, 2, 2, false);
    else if (d32 == 2) CW_LAUNCH(2, 16, 2, 2, false);
    else if (nt == 4) CW_LAUNCH(4, 4, 2, 2, false);
    else if (nt == 8) CW_LAUNCH(4, 8, 2, 2, false);
    else CW_LAUNCH(4, 16, 2, 2, false);
  } else if (!alias) {
    if (d32 == 2 && nt == 4) CW_LAUNCH(2, 4, 2, 1, false);
    else if (d32 == 2 && nt == 8) CW_LAUNCH(2, 8, 2, 1, false);
    else if (d32 == 2) CW_LAUNCH(2, 16, 2, 1, false);
    else if (nt == 4) CW_LAUNCH(4, 4, 2, 1, false);
    else if (nt == 8) CW_LAUNCH(4, 8, 2, 1, false);
    else CW_LAUNCH(4, 16, 2, 1, false);
  } else {
    if (d32 == 5) CW_LAUNCH(5, 8, 1, 1, true);
    else if (d32 == 10) CW_LAUNCH(10, 16, 1, 1, true);
    else CW_LAUNCH(18, 32, 1, 1, true);
  }
#undef CW_LAUNCH
  if (hipGetLastError() != hipSuccess) return CW_ERR_LAUNCH;
  if (runs > 1) {
    dim3 mgrid(n_items, grid.y, x.heads_per_wg);
    if (maps == 2) hipLaunchKernelGGL(rows_merge_kernel<2>, mgrid, block, 0, stream, p, x, runs, upw, 16 * nt);
    else hipLaunchKernelGGL(rows_merge_kernel<1>, mgrid, block, 0, stream, p, x, runs, upw, 16 * nt);
  }
  return cw_launch_status();
}
