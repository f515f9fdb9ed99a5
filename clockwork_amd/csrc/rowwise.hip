// Row-wise kernels of blocks other than the pre-norm RMSNorm / SwiGLU one, for gfx950:
// embedding with a scale and a learned position table, residual add + LayerNorm (weight and
// bias), the sigmoid-gated residual add of two branches, act(gate) * up for the tanh form of GELU,
// the logit cap, the mean of two RMS-normed rows, the RMS norm of whole query / key
// projections fused with the cache write, residual add + Dynamic Tanh, the erf GELU, a sigmoid
// gate, biased projections into cache rows, the low-rank query step with the latent cache row,
// the rotation of one part of every head, the RMS norm of a branch's output as it joins the
// stream, the RMS norm of the stream with a weight kept as a distance from a constant, the RMS
// norm of every query / key vector with rotation and cache write, squared ReLU, and a scale.
// Statistics, gates and the residual stream are float32; T is the activation type.
#include "common.h"

// Sum over the workgroup (256 threads), the same value in every thread; ``scratch`` holds 4 floats.
// The order of the additions depends on the row's length alone.
__device__ __forceinline__ float block_sum_256(float v, float* scratch) {
  v = cw_wave_sum(v);
  __syncthreads();  // scratch may still be read from the sum before
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
  __syncthreads();
  return (scratch[0] + scratch[1]) + (scratch[2] + scratch[3]);
}

// ---------------------------------------------------------------- embedding, scaled, plus position
// resid[t, :] = scale * table[ids[t], :] + pos_table[positions[t], :] in float32. An id outside
// [0, V) gives a zero row, a position outside [0, P) adds nothing (the host checks both).
template <typename T>
__global__ void embedding_pos_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                                     const int* __restrict__ positions, const T* __restrict__ pos_table, float scale,
                                     float* __restrict__ resid, int H, int V, int P) {
  const int t = blockIdx.x;
  const int id = ids[t];
  const int p = pos_table ? positions[t] : -1;
  const bool ok = id >= 0 && id < V, pok = p >= 0 && p < P;
  const T* row = table + (int64_t)(ok ? id : 0) * H;
  const T* prow = pos_table + (int64_t)(pok ? p : 0) * H;
  float* out = resid + (int64_t)t * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = ok ? scale * cw_to_float(row[i]) : 0.0f;
    if (pok) v += cw_to_float(prow[i]);
    out[i] = v;
  }
}

CW_EXPORT int cw_embedding_pos(const void* table, int dtype, const int* ids, const int* positions, const void* pos_table,
                               float scale, float* resid, int T, int H, int V, int P, hipStream_t stream) {
  if (T < 0 || H <= 0 || V <= 0 || (pos_table && (P <= 0 || !positions))) return CW_ERR_ARG;
  if (T == 0) return CW_OK;
  dim3 grid(T), block(256);
  if (dtype == CW_F32)
    hipLaunchKernelGGL(embedding_pos_kernel<float>, grid, block, 0, stream, (const float*)table, ids, positions,
                       (const float*)pos_table, scale, resid, H, V, P);
  else if (dtype == CW_BF16)
    hipLaunchKernelGGL(embedding_pos_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)table, ids, positions,
                       (const bf16_t*)pos_table, scale, resid, H, V, P);
  else
    return CW_ERR_DTYPE;
  return cw_launch_status();
}

// ---------------------------------------------------------------- gated branches, as a value
// What a block with sigmoid gates on its branches adds to the residual stream of row t, element j:
//   s(z[t, j] + zb[j]) * a[t, j] + s(z[t, H + j] + zb[H + j]) * b[t, j]
// z [T, 2H] (or [T, H] when there is no second branch) are the gates' products, zb their biases;
// with z == nullptr the branches are added as they are. b may be absent.
template <typename T, typename BT>
struct GatedPair {
  const T* z;
  const BT* zb;
  const T* a;
  const T* b;
  int z_stride;
  __device__ __forceinline__ float at(int64_t t, int j, int H) const {
    float va = cw_to_float(a[t * H + j]);
    float vb = b ? cw_to_float(b[t * H + j]) : 0.0f;
    if (z) {
      float za = cw_to_float(z[t * z_stride + j]);
      if (zb) za += cw_to_float(zb[j]);
      va *= 1.0f / (1.0f + expf(-za));
      if (b) {
        float zz = cw_to_float(z[t * z_stride + H + j]);
        if (zb) zz += cw_to_float(zb[H + j]);
        vb *= 1.0f / (1.0f + expf(-zz));
      }
    }
    return va + vb;
  }
};

// ---------------------------------------------------------------- residual add + LayerNorm
// rows == nullptr: for every t < n: resid[t] += pending(t) (if any), out[t] = LN(resid[t]).
// rows != nullptr: for i < n: out[i] = LN(resid[rows[i]] + pending(rows[i])); resid untouched.
// LN(x) = (x - mean) / sqrt(mean((x - mean)^2) + eps) * weight + bias: the mean first, then the
// mean of the squared deviations, both float32. pending is a GatedPair (a == nullptr: nothing).
template <typename T, typename WT, typename BT>
__global__ __launch_bounds__(256) void add_layernorm_kernel(float* __restrict__ resid, GatedPair<T, BT> pend,
                                                            const WT* __restrict__ weight, const WT* __restrict__ bias,
                                                            float eps, T* __restrict__ out, const int* __restrict__ rows,
                                                            int H) {
  __shared__ float scratch[4];
  const int i = blockIdx.x;
  const int64_t t = rows ? rows[i] : i;
  float* x = resid + t * H;
  T* o = out + (int64_t)i * H;
  const bool has = pend.a != nullptr;
  const bool write_back = rows == nullptr && has;
  float s = 0.0f;
  for (int j = threadIdx.x; j < H; j += 256) {
    float v = x[j];
    if (has) v += pend.at(t, j, H);
    if (write_back) x[j] = v;
    s += v;
  }
  const float mean = block_sum_256(s, scratch) / (float)H;
  float ss = 0.0f;
  for (int j = threadIdx.x; j < H; j += 256) {
    float v = x[j];
    if (has && !write_back) v += pend.at(t, j, H);
    const float d = v - mean;
    ss += d * d;
  }
  const float inv = 1.0f / sqrtf(block_sum_256(ss, scratch) / (float)H + eps);
  for (int j = threadIdx.x; j < H; j += 256) {
    float v = x[j];
    if (has && !write_back) v += pend.at(t, j, H);
    o[j] = cw_from_float<T>((v - mean) * inv * cw_to_float(weight[j]) + (bias ? cw_to_float(bias[j]) : 0.0f));
  }
}

// z/zb/a/b: the pending gated branches (all nullptr: none); z_cols: columns of z (H or 2H).
CW_EXPORT int cw_add_layernorm(float* resid, const void* z, const void* zb, int zb_dtype, const void* a, const void* b,
                               int z_cols, const void* weight, const void* bias, int w_dtype, float eps, void* out,
                               int dtype, const int* rows, int n, int H, hipStream_t stream) {
  if (n < 0 || H <= 0 || !resid || !weight || !out) return CW_ERR_ARG;
  if (!a && (z || b)) return CW_ERR_ARG;
  if (z && z_cols != (b ? 2 * H : H) && z_cols != 2 * H) return CW_ERR_ARG;
  if (n == 0) return CW_OK;
  dim3 grid(n), block(256);
#define CW_LAUNCH(T, WT, BT)                                                                               \
  do {                                                                                                     \
    GatedPair<T, BT> pend{(const T*)z, (const BT*)zb, (const T*)a, (const T*)b, z_cols};                   \
    hipLaunchKernelGGL((add_layernorm_kernel<T, WT, BT>), grid, block, 0, stream, resid, pend,             \
                       (const WT*)weight, (const WT*)bias, eps, (T*)out, rows, H);                         \
  } while (0)
  const int zbt = zb ? zb_dtype : w_dtype;
  if (dtype == CW_F32 && w_dtype == CW_F32 && zbt == CW_F32) CW_LAUNCH(float, float, float);
  else if (dtype == CW_BF16 && w_dtype == CW_BF16 && zbt == CW_BF16) CW_LAUNCH(bf16_t, bf16_t, bf16_t);
  else if (dtype == CW_BF16 && w_dtype == CW_F32 && zbt == CW_F32) CW_LAUNCH(bf16_t, float, float);
  else if (dtype == CW_BF16 && w_dtype == CW_F32 && zbt == CW_BF16) CW_LAUNCH(bf16_t, float, bf16_t);
  else if (dtype == CW_BF16 && w_dtype == CW_BF16 && zbt == CW_F32) CW_LAUNCH(bf16_t, bf16_t, float);
  else return CW_ERR_DTYPE;
#undef CW_LAUNCH
  return cw_launch_status();
}

// ---------------------------------------------------------------- gated residual add
// resid[t, j] += the gated pair's value (see GatedPair), float32.
template <typename T, typename BT>
__global__ void gated_residual_add_kernel(float* __restrict__ resid, GatedPair<T, BT> pend, int64_t n, int H) {
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = idx / H;
    const int j = (int)(idx - t * H);
    resid[idx] += pend.at(t, j, H);
  }
}

CW_EXPORT int cw_gated_residual_add(float* resid, const void* z, const void* zb, int zb_dtype, const void* a,
                                    const void* b, int z_cols, int dtype, int T, int H, hipStream_t stream) {
  if (T < 0 || H <= 0 || !resid || !a) return CW_ERR_ARG;
  if (z && z_cols != H && z_cols != 2 * H) return CW_ERR_ARG;
  if (z && b && z_cols != 2 * H) return CW_ERR_ARG;
  if (T == 0) return CW_OK;
  const int64_t n = (int64_t)T * H;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 262144) blocks = 262144;
  dim3 grid((unsigned)blocks), block(256);
#define CW_LAUNCH(T_, BT_)                                                                     \
  do {                                                                                         \
    GatedPair<T_, BT_> pend{(const T_*)z, (const BT_*)zb, (const T_*)a, (const T_*)b, z_cols}; \
    hipLaunchKernelGGL((gated_residual_add_kernel<T_, BT_>), grid, block, 0, stream, resid, pend, n, H); \
  } while (0)
  const int zbt = zb ? zb_dtype : dtype;
  if (dtype == CW_F32 && zbt == CW_F32) CW_LAUNCH(float, float);
  else if (dtype == CW_BF16 && zbt == CW_BF16) CW_LAUNCH(bf16_t, bf16_t);
  else if (dtype == CW_BF16 && zbt == CW_F32) CW_LAUNCH(bf16_t, float);
  else return CW_ERR_DTYPE;
#undef CW_LAUNCH
  return cw_launch_status();
}

// ---------------------------------------------------------------- gelu_tanh(gate) * up
// gate_up: [T, 2*I] (gate columns first), out: [T, I];
// gelu_tanh(z) = 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))) in float32.
__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename T>
__global__ void gelu_mul_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int64_t n, int I) {
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = idx / I;
    const int i = (int)(idx - t * I);
    const float g = cw_to_float(gate_up[t * 2 * I + i]);
    const float u = cw_to_float(gate_up[t * 2 * I + I + i]);
    out[idx] = cw_from_float<T>(gelu_tanh_f(g) * u);
  }
}

CW_EXPORT int cw_gelu_tanh_mul(const void* gate_up, void* out, int dtype, int T, int I, hipStream_t stream) {
  if (T < 0 || I <= 0) return CW_ERR_ARG;
  if (T == 0) return CW_OK;
  const int64_t n = (int64_t)T * I;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 262144) blocks = 262144;
  dim3 grid((unsigned)blocks), block(256);
  if (dtype == CW_F32)
    hipLaunchKernelGGL(gelu_mul_kernel<float>, grid, block, 0, stream, (const float*)gate_up, (float*)out, n, I);
  else if (dtype == CW_BF16)
    hipLaunchKernelGGL(gelu_mul_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)gate_up, (bf16_t*)out, n, I);
  else
    return CW_ERR_DTYPE;
  return cw_launch_status();
}

// ---------------------------------------------------------------- logit cap
// x <- cap * tanh(x / cap), in place, float32.
__global__ void softcap_kernel(float* __restrict__ x, int64_t n, float cap, float inv_cap) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    x[i] = cap * tanhf(x[i] * inv_cap);
}

CW_EXPORT int cw_softcap(float* x, int64_t n, float cap, hipStream_t stream) {
  if (n < 0 || !(cap > 0.0f)) return CW_ERR_ARG;
  if (n == 0) return CW_OK;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(softcap_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, x, n, cap, 1.0f / cap);
  return cw_launch_status();
}

// ---------------------------------------------------------------- mean of RMS-normed rows
// out[t] = (rms(a[t]) * wa + rms(b[t]) * wb) / 2, rms(x) = x / sqrt(mean(x^2) + eps), float32 inside.
// b == nullptr: out[t] = rms(a[t]) * wa.
template <typename T, typename WT>
__global__ __launch_bounds__(256) void rms_mean2_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                        const WT* __restrict__ wa, const WT* __restrict__ wb, float eps,
                                                        T* __restrict__ out, int H) {
  __shared__ float scratch[4];
  const int64_t t = blockIdx.x;
  const T* xa = a + t * H;
  const T* xb = b ? b + t * H : nullptr;
  float sa = 0.0f, sb = 0.0f;
  for (int j = threadIdx.x; j < H; j += 256) {
    const float va = cw_to_float(xa[j]);
    sa += va * va;
    if (xb) { const float vb = cw_to_float(xb[j]); sb += vb * vb; }
  }
  const float ia = 1.0f / sqrtf(block_sum_256(sa, scratch) / (float)H + eps);
  const float ib = xb ? 1.0f / sqrtf(block_sum_256(sb, scratch) / (float)H + eps) : 0.0f;
  for (int j = threadIdx.x; j < H; j += 256) {
    float v = cw_to_float(xa[j]) * ia * cw_to_float(wa[j]);
    if (xb) v = 0.5f * (v + cw_to_float(xb[j]) * ib * cw_to_float(wb[j]));
    out[t * H + j] = cw_from_float<T>(v);
  }
}

CW_EXPORT int cw_rms_mean2(const void* a, const void* b, const void* wa, const void* wb, int w_dtype, float eps,
                           void* out, int dtype, int T, int H, hipStream_t stream) {
  if (T < 0 || H <= 0 || !a || !wa || !out || (b && !wb)) return CW_ERR_ARG;
  if (T == 0) return CW_OK;
  dim3 grid(T), block(256);
#define CW_LAUNCH(T_, WT_)                                                                                       \
  hipLaunchKernelGGL((rms_mean2_kernel<T_, WT_>), grid, block, 0, stream, (const T_*)a, (const T_*)b, (const WT_*)wa, \
                     (const WT_*)wb, eps, (T_*)out, H)
  if (dtype == CW_F32 && w_dtype == CW_F32) CW_LAUNCH(float, float);
  else if (dtype == CW_BF16 && w_dtype == CW_BF16) CW_LAUNCH(bf16_t, bf16_t);
  else if (dtype == CW_BF16 && w_dtype == CW_F32) CW_LAUNCH(bf16_t, float);
  else return CW_ERR_DTYPE;
#undef CW_LAUNCH
  return cw_launch_status();
}

// ---------------------------------------------------------------- whole-projection q/k norm + cache write
// proj: [T, stride], one row a token, holding the query projection (nq elements at column q_off),
// the key projection (nk at k_off) and the value projection (nv at v_off). The query projection is
// RMS-normed as one vector of nq elements with the weight qw (all heads at once) and rewritten in
// place; the key projection likewise with kw, written to the cache row k_cache[slot, nk]; the values
// are copied to v_cache[slot, nv]. A negative slot writes no cache row. qw / kw == nullptr: no norm.
template <typename T, typename WT>
__global__ __launch_bounds__(256) void qk_rownorm_store_kernel(T* __restrict__ proj, int64_t stride, int q_off, int k_off,
                                                               int v_off, int nq, int nk, int nv,
                                                               const WT* __restrict__ qw, const WT* __restrict__ kw,
                                                               float eps, const int* __restrict__ slots,
                                                               T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                               int64_t cache_rows) {
  __shared__ float scratch[4];
  const int64_t t = blockIdx.x;
  T* row = proj + t * stride;
  int64_t slot = slots ? (int64_t)slots[t] : -1;
  if (slot >= cache_rows) slot = -1;
  float sq = 0.0f, sk = 0.0f;
  if (qw)
    for (int j = threadIdx.x; j < nq; j += 256) { const float v = cw_to_float(row[q_off + j]); sq += v * v; }
  if (kw)
    for (int j = threadIdx.x; j < nk; j += 256) { const float v = cw_to_float(row[k_off + j]); sk += v * v; }
  const float iq = qw ? 1.0f / sqrtf(block_sum_256(sq, scratch) / (float)nq + eps) : 1.0f;
  const float ik = kw ? 1.0f / sqrtf(block_sum_256(sk, scratch) / (float)nk + eps) : 1.0f;
  if (qw)
    for (int j = threadIdx.x; j < nq; j += 256)
      row[q_off + j] = cw_from_float<T>(cw_to_float(row[q_off + j]) * iq * cw_to_float(qw[j]));
  if (slot >= 0) {
    T* kd = k_cache + slot * nk;
    for (int j = threadIdx.x; j < nk; j += 256)
      kd[j] = cw_from_float<T>(cw_to_float(row[k_off + j]) * ik * (kw ? cw_to_float(kw[j]) : 1.0f));
    T* vd = v_cache + slot * nv;
    for (int j = threadIdx.x; j < nv; j += 256) vd[j] = row[v_off + j];
  }
}

CW_EXPORT int cw_qk_rownorm_store(void* proj, int dtype, int64_t stride, int q_off, int k_off, int v_off, int nq, int nk,
                                  int nv, const void* qw, const void* kw, int w_dtype, float eps, const int* slots,
                                  void* k_cache, void* v_cache, int64_t cache_rows, int T, hipStream_t stream) {
  if (T < 0 || nq <= 0 || nk < 0 || nv < 0 || q_off < 0 || k_off < 0 || v_off < 0) return CW_ERR_ARG;
  if (q_off + nq > stride || (slots && (k_off + nk > stride || v_off + nv > stride))) return CW_ERR_ARG;
  if (slots && (!k_cache || !v_cache)) return CW_ERR_ARG;
  if (T == 0) return CW_OK;
  dim3 grid(T), block(256);
#define CW_LAUNCH(T_, WT_)                                                                                        \
  hipLaunchKernelGGL((qk_rownorm_store_kernel<T_, WT_>), grid, block, 0, stream, (T_*)proj, stride, q_off, k_off, \
                     v_off, nq, nk, nv, (const WT_*)qw, (const WT_*)kw, eps, slots, (T_*)k_cache, (T_*)v_cache,   \
                     cache_rows)
  const int wt = (qw || kw) ? w_dtype : dtype;
  if (dtype == CW_F32 && wt == CW_F32) CW_LAUNCH(float, float);
  else if (dtype == CW_BF16 && wt == CW_BF16) CW_LAUNCH(bf16_t, bf16_t);
  else if (dtype == CW_BF16 && wt == CW_F32) CW_LAUNCH(bf16_t, float);
  else return CW_ERR_DTYPE;
#undef CW_LAUNCH
  return cw_launch_status();
}

// ---------------------------------------------------------------- residual add + Dynamic Tanh
// resid[t, :] += scale * delta[t, :] (+ extra[t, :]), then out = tanh(alpha * resid) * w + b: a norm
// that takes no statistics of the row. ``extra`` is a float32 stream that joins the sum after the
// branch (the model's input, added again before a repeated run of layers). With ``rows`` only
// those rows are produced and resid is left alone. alpha is one element on the device.
template <typename DT, typename WT, typename OT>
__global__ __launch_bounds__(256) void add_dyt_kernel(float* __restrict__ resid, const DT* __restrict__ delta, float scale,
                                                      const float* __restrict__ extra, const WT* __restrict__ w,
                                                      const WT* __restrict__ b, const float* __restrict__ alpha,
                                                      OT* __restrict__ out, const int* __restrict__ rows, int H) {
  const int64_t i = blockIdx.x;
  const int64_t src = rows ? (int64_t)rows[i] : i;
  const float a = alpha[0];
  float* r = resid + src * H;
  for (int j = threadIdx.x; j < H; j += 256) {
    float x = r[j];
    if (delta) x += scale * cw_to_float(delta[src * H + j]);
    if (extra) x += extra[src * H + j];
    if (!rows && (delta || extra)) r[j] = x;
    float y = tanhf(a * x) * cw_to_float(w[j]);
    if (b) y += cw_to_float(b[j]);
    out[i * H + j] = cw_from_float<OT>(y);
  }
}

// The same for bfloat16 rows of a multiple of 4 elements: a thread takes 4 neighbours (16 bytes of
// the stream, 8 of the branch and of the output).
template <typename WT>
__global__ __launch_bounds__(256) void add_dyt_vec4_kernel(float* __restrict__ resid, const bf16_t* __restrict__ delta,
                                                           float scale, const float* __restrict__ extra,
                                                           const WT* __restrict__ w, const WT* __restrict__ b,
                                                           const float* __restrict__ alpha, bf16_t* __restrict__ out,
                                                           const int* __restrict__ rows, int H) {
  const int64_t i = blockIdx.x;
  const int64_t src = rows ? (int64_t)rows[i] : i;
  const float a = alpha[0];
  for (int j = 4 * threadIdx.x; j < H; j += 4 * 256) {
    float4 x = *reinterpret_cast<const float4*>(resid + src * H + j);
    if (delta) {
      const uint2 d = *reinterpret_cast<const uint2*>(delta + src * H + j);
      x.x += scale * cw_bf16_bits_to_float((uint16_t)(d.x & 0xffffu));
      x.y += scale * cw_bf16_bits_to_float((uint16_t)(d.x >> 16));
      x.z += scale * cw_bf16_bits_to_float((uint16_t)(d.y & 0xffffu));
      x.w += scale * cw_bf16_bits_to_float((uint16_t)(d.y >> 16));
    }
    if (extra) {
      const float4 e = *reinterpret_cast<const float4*>(extra + src * H + j);
      x.x += e.x; x.y += e.y; x.z += e.z; x.w += e.w;
    }
    if (!rows && (delta || extra)) *reinterpret_cast<float4*>(resid + src * H + j) = x;
    const float xs[4] = {x.x, x.y, x.z, x.w};
    uint16_t y[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      float v = tanhf(a * xs[u]) * cw_to_float(w[j + u]);
      if (b) v += cw_to_float(b[j + u]);
      y[u] = cw_float_to_bf16_bits(v);
    }
    *reinterpret_cast<uint2*>(out + i * H + j) = make_uint2((uint32_t)y[0] | ((uint32_t)y[1] << 16), (uint32_t)y[2] | ((uint32_t)y[3] << 16));
  }
}

CW_EXPORT int cw_add_dyt(float* resid, const void* delta, int delta_dtype, float scale, const float* extra, const void* w,
                         const void* b, int w_dtype, const float* alpha, void* out, int out_dtype, const int* rows, int n,
                         int H, hipStream_t stream) {
  if (n < 0 || H <= 0 || !resid || !w || !alpha || !out) return CW_ERR_ARG;
  if (n == 0) return CW_OK;
  dim3 grid(n), block(256);
#define CW_LAUNCH(DT_, WT_, OT_)                                                                                  \
  hipLaunchKernelGGL((add_dyt_kernel<DT_, WT_, OT_>), grid, block, 0, stream, resid, (const DT_*)delta, scale, extra, \
                     (const WT_*)w, (const WT_*)b, alpha, (OT_*)out, rows, H)
  const int dd = delta ? delta_dtype : out_dtype;
  const bool vec4 = H % 4 == 0 && dd == CW_BF16 && out_dtype == CW_BF16 &&
                    (((uintptr_t)resid | (uintptr_t)extra) % 16 == 0) && (((uintptr_t)delta | (uintptr_t)out) % 8 == 0);
  if (vec4 && w_dtype == CW_BF16)
    hipLaunchKernelGGL(add_dyt_vec4_kernel<bf16_t>, grid, block, 0, stream, resid, (const bf16_t*)delta, scale, extra,
                       (const bf16_t*)w, (const bf16_t*)b, alpha, (bf16_t*)out, rows, H);
  else if (vec4 && w_dtype == CW_F32)
    hipLaunchKernelGGL(add_dyt_vec4_kernel<float>, grid, block, 0, stream, resid, (const bf16_t*)delta, scale, extra,
                       (const float*)w, (const float*)b, alpha, (bf16_t*)out, rows, H);
  else if (dd == CW_F32 && w_dtype == CW_F32 && out_dtype == CW_F32) CW_LAUNCH(float, float, float);
  else if (dd == CW_BF16 && w_dtype == CW_BF16 && out_dtype == CW_BF16) CW_LAUNCH(bf16_t, bf16_t, bf16_t);
  else if (dd == CW_BF16 && w_dtype == CW_F32 && out_dtype == CW_BF16) CW_LAUNCH(bf16_t, float, bf16_t);
  else return CW_ERR_DTYPE;
#undef CW_LAUNCH
  return cw_launch_status();
}

// ---------------------------------------------------------------- erf GELU, in place
// x <- 0.5 x (1 + erf(x / sqrt 2)), float32 inside.
template <typename T>
__global__ void gelu_erf_kernel(T* __restrict__ x, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const float z = cw_to_float(x[i]);
    x[i] = cw_from_float<T>(0.5f * z * (1.0f + erff(z * 0.70710678118654752440f)));
  }
}

// bfloat16, 8 elements (16 bytes) a thread
__global__ void gelu_erf_vec8_kernel(uint4* __restrict__ x, int64_t n8) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8; i += (int64_t)gridDim.x * blockDim.x) {
    uint4 v = x[i];
    uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float a = cw_bf16_bits_to_float((uint16_t)(w[u] & 0xffffu)), b = cw_bf16_bits_to_float((uint16_t)(w[u] >> 16));
      const float ga = 0.5f * a * (1.0f + erff(a * 0.70710678118654752440f));
      const float gb = 0.5f * b * (1.0f + erff(b * 0.70710678118654752440f));
      w[u] = (uint32_t)cw_float_to_bf16_bits(ga) | ((uint32_t)cw_float_to_bf16_bits(gb) << 16);
    }
    x[i] = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

CW_EXPORT int cw_gelu_erf(void* x, int dtype, int64_t n, hipStream_t stream) {
  if (n < 0) return CW_ERR_ARG;
  if (n == 0) return CW_OK;
  if (dtype == CW_BF16 && n % 8 == 0 && (uintptr_t)x % 16 == 0) {
    int64_t blocks8 = (n / 8 + 255) / 256;
    if (blocks8 > 65536) blocks8 = 65536;
    hipLaunchKernelGGL(gelu_erf_vec8_kernel, dim3((unsigned)blocks8), dim3(256), 0, stream, (uint4*)x, n / 8);
    return cw_launch_status();
  }
  int64_t blocks = (n + 255) / 256;
  if (blocks > 262144) blocks = 262144;
  dim3 grid((unsigned)blocks), block(256);
  if (dtype == CW_F32) hipLaunchKernelGGL(gelu_erf_kernel<float>, grid, block, 0, stream, (float*)x, n);
  else if (dtype == CW_BF16) hipLaunchKernelGGL(gelu_erf_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)x, n);
  else return CW_ERR_DTYPE;
  return cw_launch_status();
}

// ---------------------------------------------------------------- a * sigmoid(z), in place on a
// a[t, j] <- a[t, j] / (1 + exp(-z[t, z_off + j / group])), j < n; z rows are z_stride elements
// apart. group 1: a gate an element; group g: one gate for every run of g elements (a head).
template <typename T>
__global__ void sigmoid_mul_kernel(T* __restrict__ a, const T* __restrict__ z, int64_t z_stride, int z_off, int n,
                                   int group, int64_t total) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / n;
    const int j = (int)(i % n) / group;
    const float g = 1.0f / (1.0f + expf(-cw_to_float(z[t * z_stride + z_off + j])));
    a[i] = cw_from_float<T>(cw_to_float(a[i]) * g);
  }
}

CW_EXPORT int cw_sigmoid_mul(void* a, const void* z, int dtype, int64_t z_stride, int z_off, int T, int n, int group,
                             hipStream_t stream) {
  if (T < 0 || n <= 0 || group <= 0 || n % group || z_off < 0 || z_off + n / group > z_stride) return CW_ERR_ARG;
  if (T == 0) return CW_OK;
  const int64_t total = (int64_t)T * n;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 262144) blocks = 262144;
  dim3 grid((unsigned)blocks), block(256);
  if (dtype == CW_F32)
    hipLaunchKernelGGL(sigmoid_mul_kernel<float>, grid, block, 0, stream, (float*)a, (const float*)z, z_stride, z_off, n, group, total);
  else if (dtype == CW_BF16)
    hipLaunchKernelGGL(sigmoid_mul_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)a, (const bf16_t*)z, z_stride, z_off, n, group, total);
  else return CW_ERR_DTYPE;
  return cw_launch_status();
}

// ---------------------------------------------------------------- biases and the cache write, no positions
// A row of proj holds a token's query, key and value projections at q_off / k_off / v_off. The
// bias (one element per column of proj, or nullptr) is added: the queries are rewritten in place,
// keys and values go to the rows k_plane[slot, nk] and v_plane[slot, nv]. A negative slot writes
// no cache row.
template <typename T, typename WT>
__global__ __launch_bounds__(256) void bias_store_kernel(T* __restrict__ proj, int64_t stride, int q_off, int k_off, int v_off,
                                                         int nq, int nk, int nv, const WT* __restrict__ bias,
                                                         const int* __restrict__ slots, T* __restrict__ k_plane,
                                                         T* __restrict__ v_plane, int64_t cache_rows) {
  const int64_t t = blockIdx.x;
  T* row = proj + t * stride;
  int64_t slot = slots ? (int64_t)slots[t] : -1;
  if (slot >= cache_rows) slot = -1;
  if (bias)
    for (int j = threadIdx.x; j < nq; j += 256)
      row[q_off + j] = cw_from_float<T>(cw_to_float(row[q_off + j]) + cw_to_float(bias[q_off + j]));
  if (slot >= 0) {
    T* kd = k_plane + slot * nk;
    for (int j = threadIdx.x; j < nk; j += 256)
      kd[j] = cw_from_float<T>(cw_to_float(row[k_off + j]) + (bias ? cw_to_float(bias[k_off + j]) : 0.0f));
    T* vd = v_plane + slot * nv;
    for (int j = threadIdx.x; j < nv; j += 256)
      vd[j] = cw_from_float<T>(cw_to_float(row[v_off + j]) + (bias ? cw_to_float(bias[v_off + j]) : 0.0f));
  }
}

CW_EXPORT int cw_bias_store(void* proj, int dtype, int64_t stride, int q_off, int k_off, int v_off, int nq, int nk, int nv,
                            const void* bias, int b_dtype, const int* slots, void* k_plane, void* v_plane,
                            int64_t cache_rows, int T, hipStream_t stream) {
  if (T < 0 || nq < 0 || nk < 0 || nv < 0 || q_off < 0 || k_off < 0 || v_off < 0) return CW_ERR_ARG;
  if (q_off + nq > stride || k_off + nk > stride || v_off + nv > stride) return CW_ERR_ARG;
  if (slots && (!k_plane || !v_plane)) return CW_ERR_ARG;
  if (T == 0) return CW_OK;
  dim3 grid(T), block(256);
#define CW_LAUNCH(T_, WT_)                                                                                         \
  hipLaunchKernelGGL((bias_store_kernel<T_, WT_>), grid, block, 0, stream, (T_*)proj, stride, q_off, k_off, v_off, nq, \
                     nk, nv, (const WT_*)bias, slots, (T_*)k_plane, (T_*)v_plane, cache_rows)
  const int wt = bias ? b_dtype : dtype;
  if (dtype == CW_F32 && wt == CW_F32) CW_LAUNCH(float, float);
  else if (dtype == CW_BF16 && wt == CW_BF16) CW_LAUNCH(bf16_t, bf16_t);
  else if (dtype == CW_BF16 && wt == CW_F32) CW_LAUNCH(bf16_t, float);
  else return CW_ERR_DTYPE;
#undef CW_LAUNCH
  return cw_launch_status();
}

// ---------------------------------------------------------------- low-rank queries and the latent cache row
// A row of proj holds, at dq_off, nq elements of a query's low-rank step and, at dkv_off,
// rank + rot elements of the key/value one. One workgroup a token:
//   cq[t, :]            = dq / rms(dq) * wq                      (T, [T, nq])
//   plane[slot, :rank]  = dkv[:rank] / rms(dkv[:rank]) * wkv     (the latent)
//   plane[slot, rank:]  = dkv[rank:] with its first rdims elements rotated by the token's position:
//                         pairs (i, i + rdims / 2), angle = float(position) * freq[i]
// rms(x) = sqrt(mean(x^2) + eps), float32.
template <typename T, typename WT>
__global__ __launch_bounds__(256) void latent_store_kernel(const T* __restrict__ proj, int64_t stride, int dq_off, int nq,
                                                           int dkv_off, int rank, int rot, int rdims,
                                                           const WT* __restrict__ wq, const WT* __restrict__ wkv, float eps,
                                                           const int* __restrict__ positions,
                                                           const float* __restrict__ freq, const int* __restrict__ slots,
                                                           T* __restrict__ cq, T* __restrict__ plane, int64_t cache_rows) {
  __shared__ float scratch[4];
  const int64_t t = blockIdx.x;
  const T* row = proj + t * stride;
  int64_t slot = slots ? (int64_t)slots[t] : -1;
  if (slot >= cache_rows) slot = -1;
  float sq = 0.0f, sk = 0.0f;
  for (int j = threadIdx.x; j < nq; j += 256) { const float v = cw_to_float(row[dq_off + j]); sq += v * v; }
  for (int j = threadIdx.x; j < rank; j += 256) { const float v = cw_to_float(row[dkv_off + j]); sk += v * v; }
  const float iq = 1.0f / sqrtf(block_sum_256(sq, scratch) / (float)nq + eps);
  const float ik = 1.0f / sqrtf(block_sum_256(sk, scratch) / (float)rank + eps);
  for (int j = threadIdx.x; j < nq; j += 256)
    cq[t * nq + j] = cw_from_float<T>(cw_to_float(row[dq_off + j]) * iq * cw_to_float(wq[j]));
  if (slot < 0) return;
  T* dst = plane + slot * (rank + rot);
  for (int j = threadIdx.x; j < rank; j += 256)
    dst[j] = cw_from_float<T>(cw_to_float(row[dkv_off + j]) * ik * cw_to_float(wkv[j]));
  const float pos = (float)positions[t];
  const int half = rdims / 2;
  const T* r = row + dkv_off + rank;
  for (int j = threadIdx.x; j < rot; j += 256) {
    float v = cw_to_float(r[j]);
    if (j < rdims) {
      const int i = j < half ? j : j - half;
      float s, c;
      sincosf(pos * freq[i], &s, &c);
      const float u = cw_to_float(r[i]), w = cw_to_float(r[i + half]);
      v = j < half ? u * c - w * s : w * c + u * s;
    }
    dst[rank + j] = cw_from_float<T>(v);
  }
}

CW_EXPORT int cw_latent_store(const void* proj, int dtype, int64_t stride, int dq_off, int nq, int dkv_off, int rank, int rot,
                              int rdims, const void* wq, const void* wkv, int w_dtype, float eps, const int* positions,
                              const float* freq, const int* slots, void* cq, void* plane, int64_t cache_rows, int T,
                              hipStream_t stream) {
  if (T < 0 || nq <= 0 || rank <= 0 || rot < 0 || rdims < 0 || rdims > rot || (rdims & 1)) return CW_ERR_ARG;
  if (dq_off < 0 || dkv_off < 0 || dq_off + nq > stride || dkv_off + rank + rot > stride) return CW_ERR_ARG;
  if (!proj || !wq || !wkv || !cq || !positions || (rdims && !freq) || (slots && !plane)) return CW_ERR_ARG;
  if (T == 0) return CW_OK;
  dim3 grid(T), block(256);
#define CW_LAUNCH(T_, WT_)                                                                                          \
  hipLaunchKernelGGL((latent_store_kernel<T_, WT_>), grid, block, 0, stream, (const T_*)proj, stride, dq_off, nq, dkv_off, \
                     rank, rot, rdims, (const WT_*)wq, (const WT_*)wkv, eps, positions, freq, slots, (T_*)cq, (T_*)plane,   \
                     cache_rows)
  if (dtype == CW_F32 && w_dtype == CW_F32) CW_LAUNCH(float, float);
  else if (dtype == CW_BF16 && w_dtype == CW_BF16) CW_LAUNCH(bf16_t, bf16_t);
  else if (dtype == CW_BF16 && w_dtype == CW_F32) CW_LAUNCH(bf16_t, float);
  else return CW_ERR_DTYPE;
#undef CW_LAUNCH
  return cw_launch_status();
}

// ---------------------------------------------------------------- rotate one part of every head, to another layout
// dst[t, h, dst_off + j] = src[t, h, src_off + j] for j < n, its first rdims elements rotated by
// the token's position (pairs (i, i + rdims / 2), angle = float(position) * freq[i]). Tokens of src
// and dst are src_stride / dst_stride elements apart, heads src_head / dst_head (token-major or
// head-major alike; the host checks that the strides stay inside the tensors).
template <typename T>
__global__ void rotate_part_kernel(const T* __restrict__ src, int64_t src_stride, int64_t src_head, int src_off,
                                   T* __restrict__ dst, int64_t dst_stride, int64_t dst_head, int dst_off, int heads, int n,
                                   int rdims, const int* __restrict__ positions, const float* __restrict__ freq) {
  const int64_t t = blockIdx.x;
  const float pos = (float)positions[t];
  const int half = rdims / 2;
  for (int e = threadIdx.x; e < heads * n; e += blockDim.x) {
    const int h = e / n, j = e % n;
    const T* s = src + t * src_stride + h * src_head + src_off;
    float v = cw_to_float(s[j]);
    if (j < rdims) {
      const int i = j < half ? j : j - half;
      float sn, cs;
      sincosf(pos * freq[i], &sn, &cs);
      const float u = cw_to_float(s[i]), w = cw_to_float(s[i + half]);
      v = j < half ? u * cs - w * sn : w * cs + u * sn;
    }
    dst[t * dst_stride + h * dst_head + dst_off + j] = cw_from_float<T>(v);
  }
}

CW_EXPORT int cw_rotate_part(const void* src, int dtype, int64_t src_stride, int64_t src_head, int src_off, void* dst,
                             int64_t dst_stride, int64_t dst_head, int dst_off, int heads, int n, int rdims,
                             const int* positions, const float* freq, int T, hipStream_t stream) {
  if (T < 0 || heads <= 0 || n < 0 || rdims < 0 || rdims > n || (rdims & 1)) return CW_ERR_ARG;
  if (src_off < 0 || dst_off < 0 || src_stride < 1 || dst_stride < 1 || src_head < 1 || dst_head < 1) return CW_ERR_ARG;
  if (!src || !dst || !positions || (rdims && !freq)) return CW_ERR_ARG;
  if (T == 0 || n == 0) return CW_OK;
  dim3 grid(T), block(256);
  if (dtype == CW_F32)
    hipLaunchKernelGGL(rotate_part_kernel<float>, grid, block, 0, stream, (const float*)src, src_stride, src_head, src_off,
                       (float*)dst, dst_stride, dst_head, dst_off, heads, n, rdims, positions, freq);
  else if (dtype == CW_BF16)
    hipLaunchKernelGGL(rotate_part_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)src, src_stride, src_head, src_off,
                       (bf16_t*)dst, dst_stride, dst_head, dst_off, heads, n, rdims, positions, freq);
  else return CW_ERR_DTYPE;
  return cw_launch_status();
}

// ---------------------------------------------------------------- a branch's output, normed, joins the stream
// For a block that norms what a sublayer gives back and not what it reads:
//   resid[t, :] += scale * branch[t, :] / sqrt(mean(branch[t, :]^2) + eps) * (w_offset + w)
// and image[t, :] = resid[t, :] in the activation type (what the next sublayer reads); image may be
// nullptr, and so may branch (then nothing is added and the image alone is made). float32 inside.
template <typename T, typename WT>
__global__ __launch_bounds__(256) void branch_norm_add_kernel(float* __restrict__ resid, const T* __restrict__ branch,
                                                              const WT* __restrict__ w, float w_offset, float eps, float scale,
                                                              T* __restrict__ image, int H) {
  __shared__ float scratch[4];
  const int64_t t = blockIdx.x;
  float* x = resid + t * H;
  const T* b = branch ? branch + t * H : nullptr;
  T* im = image ? image + t * H : nullptr;
  float inv = 0.0f;
  if (b) {
    float ss = 0.0f;
    for (int j = threadIdx.x; j < H; j += 256) { const float v = cw_to_float(b[j]); ss += v * v; }
    inv = scale / sqrtf(block_sum_256(ss, scratch) / (float)H + eps);
  }
  for (int j = threadIdx.x; j < H; j += 256) {
    float v = x[j];
    if (b) {
      v += cw_to_float(b[j]) * inv * (w_offset + cw_to_float(w[j]));
      x[j] = v;
    }
    if (im) im[j] = cw_from_float<T>(v);
  }
}

CW_EXPORT int cw_branch_norm_add(float* resid, const void* branch, const void* w, int w_dtype, float w_offset, float eps,
                                 float scale, void* image, int dtype, int T, int H, hipStream_t stream) {
  if (T < 0 || H <= 0 || !resid || (branch && !w)) return CW_ERR_ARG;
  if (T == 0 || (!branch && !image)) return CW_OK;
  dim3 grid(T), block(256);
#define CW_LAUNCH(T_, WT_)                                                                                           \
  hipLaunchKernelGGL((branch_norm_add_kernel<T_, WT_>), grid, block, 0, stream, resid, (const T_*)branch, (const WT_*)w, \
                     w_offset, eps, scale, (T_*)image, H)
  const int wt = branch ? w_dtype : dtype;
  if (dtype == CW_F32 && wt == CW_F32) CW_LAUNCH(float, float);
  else if (dtype == CW_BF16 && wt == CW_BF16) CW_LAUNCH(bf16_t, bf16_t);
  else if (dtype == CW_BF16 && wt == CW_F32) CW_LAUNCH(bf16_t, float);
  else return CW_ERR_DTYPE;
#undef CW_LAUNCH
  return cw_launch_status();
}

// ---------------------------------------------------------------- RMS norm of the stream, weight as an offset
// out[i, :] = resid[r, :] / sqrt(mean(resid[r, :]^2) + eps) * (w_offset + w), r = rows ? rows[i] : i;
// the product is made in float32 and rounded once. The stream is left as it is.
template <typename T, typename WT>
__global__ __launch_bounds__(256) void stream_norm_kernel(const float* __restrict__ resid, const WT* __restrict__ w,
                                                          float w_offset, float eps, T* __restrict__ out,
                                                          const int* __restrict__ rows, int H) {
  __shared__ float scratch[4];
  const int64_t i = blockIdx.x;
  const float* x = resid + (int64_t)(rows ? rows[i] : (int)i) * H;
  float ss = 0.0f;
  for (int j = threadIdx.x; j < H; j += 256) ss += x[j] * x[j];
  const float inv = 1.0f / sqrtf(block_sum_256(ss, scratch) / (float)H + eps);
  for (int j = threadIdx.x; j < H; j += 256) out[i * H + j] = cw_from_float<T>(x[j] * inv * (w_offset + cw_to_float(w[j])));
}

CW_EXPORT int cw_stream_norm(const float* resid, const void* w, int w_dtype, float w_offset, float eps, void* out, int dtype,
                             const int* rows, int n, int H, hipStream_t stream) {
  if (n < 0 || H <= 0 || !resid || !w || !out) return CW_ERR_ARG;
  if (n == 0) return CW_OK;
  dim3 grid(n), block(256);
#define CW_LAUNCH(T_, WT_)                                                                                          \
  hipLaunchKernelGGL((stream_norm_kernel<T_, WT_>), grid, block, 0, stream, resid, (const WT_*)w, w_offset, eps, (T_*)out, \
                     rows, H)
  if (dtype == CW_F32 && w_dtype == CW_F32) CW_LAUNCH(float, float);
  else if (dtype == CW_BF16 && w_dtype == CW_BF16) CW_LAUNCH(bf16_t, bf16_t);
  else if (dtype == CW_BF16 && w_dtype == CW_F32) CW_LAUNCH(bf16_t, float);
  else return CW_ERR_DTYPE;
#undef CW_LAUNCH
  return cw_launch_status();
}

// ---------------------------------------------------------------- per-vector q/k norm, rotation, cache write
// A row of proj holds a token's query projection (nqv vectors of dim elements from column q_off),
// its key projection (nkv vectors of dim from k_off) and, unless the values are the keys, its value
// projection (nv elements from v_off). bias (one element per column of proj, or nullptr) is added
// first. Every query and key vector by itself is then divided by its root mean square (eps inside
// the root) and multiplied by qw / kw (dim elements, shared by all vectors; nullptr: no norm), and
// its first rdims elements are rotated by the token's position: pairs (i, i + rdims / 2), angle =
// float(position) * freq[i]. Queries are rewritten in place, keys go to k_plane[slot, nkv * dim].
// Values go to v_plane[slot, nv]: the biased value projection, or with v_from_keys the biased key
// projection as it was before norm and rotation (nv == nkv * dim). A negative slot writes no
// cache row. One workgroup a token, one wave a vector at a time; float32 inside.
//
// Options (HeadNormOptions): ``pairing`` 1 rotates neighbours, (2i, 2i + 1) by freq[i], instead of
// halves. ``norm`` 0: no norm; 1: norm (and weight), then rotation; 2: rotation, then the rotated
// vector is divided by ITS root mean square (and multiplied by the weight). The weights may be
// absent with either norm. ``q_temp_every`` n > 0: every query is multiplied, last, by
// 1 + q_temp_coef * ln(floor((position + 1) / n) + 1).
#define HN_MAX_DIM 1024
struct HeadNormOptions {
  int pairing, norm, q_temp_every;
  float q_temp_coef;
};
__device__ __forceinline__ float hn_query_factor(const HeadNormOptions& o, int position) {
  return o.q_temp_every > 0 ? 1.0f + o.q_temp_coef * logf((float)((position + 1) / o.q_temp_every + 1)) : 1.0f;
}
template <typename T, typename WT, typename BT>
__global__ __launch_bounds__(1024) void headnorm_rope_store_kernel(
    T* __restrict__ proj, int64_t stride, int q_off, int k_off, int v_off, int nqv, int nkv, int dim, int nv,
    const BT* __restrict__ bias, const WT* __restrict__ qw, const WT* __restrict__ kw, float eps,
    const int* __restrict__ positions, const float* __restrict__ freq, int rdims, const int* __restrict__ slots,
    T* __restrict__ k_plane, T* __restrict__ v_plane, int v_from_keys, int64_t cache_rows, HeadNormOptions opt) {
  extern __shared__ float hn_vals[];  // [waves][dim], then the token's cosines and sines [2][rdims / 2]
  const int64_t t = blockIdx.x;
  T* row = proj + t * stride;
  int64_t slot = slots ? (int64_t)slots[t] : -1;
  if (slot >= cache_rows) slot = -1;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (slot >= 0 && v_plane) {
    const int src = v_from_keys ? k_off : v_off;
    T* vd = v_plane + slot * nv;
    for (int j = threadIdx.x; j < nv; j += blockDim.x)
      vd[j] = cw_from_float<T>(cw_to_float(row[src + j]) + (bias ? cw_to_float(bias[src + j]) : 0.0f));
  }
  const float pos = positions ? (float)positions[t] : 0.0f;
  const int half = rdims / 2, n_waves = blockDim.x >> 6;
  float* vals = hn_vals + wave * dim;
  // the angles are the same for every vector of the token: made once
  float* cosines = hn_vals + n_waves * dim;
  float* sines = cosines + half;
  for (int i = threadIdx.x; i < half; i += blockDim.x) sincosf(pos * freq[i], &sines[i], &cosines[i]);
  __syncthreads();
  const float q_factor = hn_query_factor(opt, positions ? positions[t] : 0);
  for (int vec = wave; vec < nqv + nkv; vec += n_waves) {
    const bool is_q = vec < nqv;
    if (!is_q && slot < 0) continue;
    const int base = is_q ? q_off + vec * dim : k_off + (vec - nqv) * dim;
    const WT* w = is_q ? qw : kw;
    float ss = 0.0f;
    for (int j = lane; j < dim; j += 64) {
      const float v = cw_to_float(row[base + j]) + (bias ? cw_to_float(bias[base + j]) : 0.0f);
      vals[j] = v;
      ss += v * v;
    }
    const float inv = opt.norm == 1 ? 1.0f / sqrtf(cw_wave_sum(ss) / (float)dim + eps) : 1.0f;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
    // element j after the norm that comes first (if that is the order) and the rotation
    auto turned = [&](int j) -> float {
      const bool pre = opt.norm == 1;
      if (j >= rdims) return vals[j] * (pre ? inv * (w ? cw_to_float(w[j]) : 1.0f) : 1.0f);
      const int i = opt.pairing ? j >> 1 : (j < half ? j : j - half);
      const int ja = opt.pairing ? 2 * i : i, jb = opt.pairing ? 2 * i + 1 : i + half;
      const float a = vals[ja] * (pre ? inv * (w ? cw_to_float(w[ja]) : 1.0f) : 1.0f);
      const float b = vals[jb] * (pre ? inv * (w ? cw_to_float(w[jb]) : 1.0f) : 1.0f);
      const float s = sines[i], c = cosines[i];
      return j == ja ? a * c - b * s : b * c + a * s;
    };
    float inv_after = 1.0f;
    if (opt.norm == 2) {
      float s2 = 0.0f;
      for (int j = lane; j < dim; j += 64) { const float r = turned(j); s2 += r * r; }
      inv_after = 1.0f / sqrtf(cw_wave_sum(s2) / (float)dim + eps);
    }
    T* dst = is_q ? row + base : k_plane + slot * ((int64_t)nkv * dim) + (int64_t)(vec - nqv) * dim;
    for (int j = lane; j < dim; j += 64) {
      float v = turned(j);
      if (opt.norm == 2) v *= inv_after * (w ? cw_to_float(w[j]) : 1.0f);
      dst[j] = cw_from_float<T>(is_q ? v * q_factor : v);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
  }
}

// The same for bfloat16 vectors of 8, 16, ... 512 elements whose rotated part is a multiple of 16:
// a lane holds 8 neighbouring elements of a vector (one 16-byte load and store), dim / 8 lanes a
// vector, several vectors a wave. The sum of squares meets over the vector's lanes by exchanges;
// a rotated element's partner, dims / 2 elements away, lies in the lane dims / 16 further.
// Element by element the arithmetic is the kernel's above.
typedef __attribute__((ext_vector_type(4))) unsigned int cw_u32x4_t;
template <typename WT, typename BT>
__global__ __launch_bounds__(256) void headnorm_rope_store_vec_kernel(
    bf16_t* __restrict__ proj, int64_t stride, int q_off, int k_off, int v_off, int nqv, int nkv, int dim, int nv,
    const BT* __restrict__ bias, const WT* __restrict__ qw, const WT* __restrict__ kw, float eps,
    const int* __restrict__ positions, const float* __restrict__ freq, int rdims, const int* __restrict__ slots,
    bf16_t* __restrict__ k_plane, bf16_t* __restrict__ v_plane, int v_from_keys, int64_t cache_rows, HeadNormOptions opt) {
  extern __shared__ float hn_vals[];  // the token's cosines and sines [2][rdims / 2]
  const int64_t t = blockIdx.x;
  bf16_t* row = proj + t * stride;
  int64_t slot = slots ? (int64_t)slots[t] : -1;
  if (slot >= cache_rows) slot = -1;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (slot >= 0 && v_plane) {
    const int src = v_from_keys ? k_off : v_off;
    bf16_t* vd = v_plane + slot * nv;
    for (int j = threadIdx.x; j < nv; j += 256)
      vd[j] = __float2bfloat16(__bfloat162float(row[src + j]) + (bias ? cw_to_float(bias[src + j]) : 0.0f));
  }
  const float pos = positions ? (float)positions[t] : 0.0f;
  const int half = rdims / 2;
  float* cosines = hn_vals;
  float* sines = cosines + half;
  for (int i = threadIdx.x; i < half; i += 256) sincosf(pos * freq[i], &sines[i], &cosines[i]);
  __syncthreads();
  const int lanes = dim >> 3, per_wave = 64 / lanes;   // lanes of a vector (a power of two), vectors of a wave
  const int sub = lane & (lanes - 1), j0 = sub * 8;
  // halves: a rotated element's partner lies dims / 2 elements away, in another lane; neighbours:
  // both elements of a pair lie in the lane itself
  const bool rotated = j0 < rdims, low = j0 < half;
  const int partner = (rotated && !opt.pairing) ? (low ? lane + (half >> 3) : lane - (half >> 3)) : lane;
  const int n_vec = nqv + nkv;
  const float q_factor = hn_query_factor(opt, positions ? positions[t] : 0);
  for (int first = 0; first < n_vec; first += 4 * per_wave) {  // every lane of a wave stays for the exchanges
    const int vec = first + wave * per_wave + lane / lanes;
    const bool is_q = vec < nqv;
    const bool live = vec < n_vec && (is_q || slot >= 0);
    const int base = (is_q ? q_off + vec * dim : k_off + (vec - nqv) * dim) + j0;
    const WT* w = is_q ? qw : kw;
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = 0.0f;
    if (live) {
      const cw_u32x4_t raw = *reinterpret_cast<const cw_u32x4_t*>(row + base);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[2 * i] = cw_bf16_bits_to_float((uint16_t)(raw[i] & 0xffffu));
        v[2 * i + 1] = cw_bf16_bits_to_float((uint16_t)(raw[i] >> 16));
      }
      if (bias) {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] += cw_to_float(bias[base + i]);
      }
    }
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) ss += v[i] * v[i];
    for (int off = 1; off < lanes; off <<= 1) ss += __shfl_xor(ss, off, 64);
    const bool pre = opt.norm == 1;
    const float inv = pre ? 1.0f / sqrtf(ss / (float)dim + eps) : 1.0f;
    float pv[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) pv[i] = opt.pairing ? v[i ^ 1] : __shfl(v[i], partner, 64);
    float r[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (rotated) {
        // ja, jb: the pair's two elements; ``mine_first``: this element is the pair's first
        const bool mine_first = opt.pairing ? !(i & 1) : low;
        const int idx = opt.pairing ? (j0 + i) >> 1 : (low ? j0 : j0 - half) + i;
        const int ja = opt.pairing ? 2 * idx : idx, jb = opt.pairing ? 2 * idx + 1 : idx + half;
        const float a = (mine_first ? v[i] : pv[i]) * (pre ? inv * (w ? cw_to_float(w[ja]) : 1.0f) : 1.0f);
        const float b = (mine_first ? pv[i] : v[i]) * (pre ? inv * (w ? cw_to_float(w[jb]) : 1.0f) : 1.0f);
        const float sn = live ? sines[idx] : 0.0f, c = live ? cosines[idx] : 0.0f;
        r[i] = mine_first ? a * c - b * sn : b * c + a * sn;
      } else {
        r[i] = v[i] * (pre ? inv * (w ? cw_to_float(w[j0 + i]) : 1.0f) : 1.0f);
      }
    }
    if (opt.norm == 2) {
      float s2 = 0.0f;
#pragma unroll
      for (int i = 0; i < 8; ++i) s2 += r[i] * r[i];
      for (int off = 1; off < lanes; off <<= 1) s2 += __shfl_xor(s2, off, 64);
      const float inv_after = 1.0f / sqrtf(s2 / (float)dim + eps);
#pragma unroll
      for (int i = 0; i < 8; ++i) r[i] *= inv_after * (w ? cw_to_float(w[j0 + i]) : 1.0f);
    }
    if (!live) continue;
    uint16_t o[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = cw_float_to_bf16_bits(is_q ? r[i] * q_factor : r[i]);
    cw_u32x4_t packed;
#pragma unroll
    for (int i = 0; i < 4; ++i) packed[i] = (uint32_t)o[2 * i] | ((uint32_t)o[2 * i + 1] << 16);
    bf16_t* dst = is_q ? row + base : k_plane + slot * ((int64_t)nkv * dim) + (int64_t)(vec - nqv) * dim + j0;
    *reinterpret_cast<cw_u32x4_t*>(dst) = packed;
  }
}

CW_EXPORT int cw_headnorm_rope_store(void* proj, int dtype, int64_t stride, int q_off, int k_off, int v_off, int nqv, int nkv,
                                     int dim, int nv, const void* bias, int b_dtype, const void* qw, const void* kw,
                                     int w_dtype, float eps, const int* positions, const float* freq, int rdims,
                                     const int* slots, void* k_plane, void* v_plane, int v_from_keys, int64_t cache_rows,
                                     int T, int pairing, int norm, float q_temp_coef, int q_temp_every,
                                     hipStream_t stream) {
  if (T < 0 || nqv < 0 || nkv < 0 || dim <= 0 || nv < 0 || rdims < 0 || rdims > dim || (rdims & 1)) return CW_ERR_ARG;
  if (pairing < 0 || pairing > 1 || norm < 0 || norm > 2 || q_temp_every < 0 || (q_temp_every > 0 && !positions)) return CW_ERR_ARG;
  const HeadNormOptions opt = {pairing, norm, q_temp_every, q_temp_coef};
  if (dim > HN_MAX_DIM) return CW_ERR_SIZE;
  if (q_off < 0 || k_off < 0 || v_off < 0 || q_off + (int64_t)nqv * dim > stride || k_off + (int64_t)nkv * dim > stride)
    return CW_ERR_ARG;
  if (v_from_keys ? nv != nkv * dim : v_off + (int64_t)nv > stride) return CW_ERR_ARG;
  if (!proj || (rdims && (!freq || !positions)) || (slots && nkv && !k_plane) || (slots && nv && !v_plane)) return CW_ERR_ARG;
  if ((qw == nullptr) != (kw == nullptr)) return CW_ERR_ARG;
  if (T == 0) return CW_OK;
  // bfloat16 vectors that lanes of 8 elements tile: the kernel of 16-byte accesses
  if (dtype == CW_BF16 && dim >= 8 && dim <= 512 && !(dim & (dim - 1)) && !(rdims & (pairing ? 7 : 15)) && !(q_off & 7) && !(k_off & 7) &&
      !(stride & 7) && !((uintptr_t)proj & 15) && !((uintptr_t)k_plane & 15)) {
    const size_t lds_vec = (size_t)(rdims ? rdims : 2) * sizeof(float);
#define CW_LAUNCH_VEC(WT_, BT_)                                                                                         \
  hipLaunchKernelGGL((headnorm_rope_store_vec_kernel<WT_, BT_>), dim3(T), dim3(256), lds_vec, stream, (bf16_t*)proj, stride, \
                     q_off, k_off, v_off, nqv, nkv, dim, nv, (const BT_*)bias, (const WT_*)qw, (const WT_*)kw, eps, positions, \
                     freq, rdims, slots, (bf16_t*)k_plane, (bf16_t*)v_plane, v_from_keys, cache_rows, opt)
    const int wt_v = qw ? w_dtype : CW_BF16, bt_v = bias ? b_dtype : CW_BF16;
    if (wt_v == CW_BF16 && bt_v == CW_BF16) CW_LAUNCH_VEC(bf16_t, bf16_t);
    else if (wt_v == CW_F32 && bt_v == CW_BF16) CW_LAUNCH_VEC(float, bf16_t);
    else if (wt_v == CW_BF16 && bt_v == CW_F32) CW_LAUNCH_VEC(bf16_t, float);
    else if (wt_v == CW_F32 && bt_v == CW_F32) CW_LAUNCH_VEC(float, float);
    else return CW_ERR_DTYPE;
#undef CW_LAUNCH_VEC
    return cw_launch_status();
  }
  // a wave a vector at a time: as many waves as there are vectors, 4 to 16
  const int n_vec = nqv + nkv;
  int waves = n_vec < 4 ? 4 : n_vec > 16 ? 16 : n_vec;
  while (waves > 4 && ((size_t)waves * dim + rdims) * sizeof(float) > 49152) --waves;  // their vectors share 48 KB of LDS
  dim3 grid(T), block(64 * waves);
  const size_t lds = ((size_t)waves * dim + rdims) * sizeof(float);
#define CW_LAUNCH(T_, WT_, BT_)                                                                                          \
  hipLaunchKernelGGL((headnorm_rope_store_kernel<T_, WT_, BT_>), grid, block, lds, stream, (T_*)proj, stride, q_off, k_off, \
                     v_off, nqv, nkv, dim, nv, (const BT_*)bias, (const WT_*)qw, (const WT_*)kw, eps, positions, freq, rdims, \
                     slots, (T_*)k_plane, (T_*)v_plane, v_from_keys, cache_rows, opt)
  const int wt = qw ? w_dtype : dtype, bt = bias ? b_dtype : dtype;
  if (dtype == CW_F32 && wt == CW_F32 && bt == CW_F32) CW_LAUNCH(float, float, float);
  else if (dtype == CW_BF16 && wt == CW_BF16 && bt == CW_BF16) CW_LAUNCH(bf16_t, bf16_t, bf16_t);
  else if (dtype == CW_BF16 && wt == CW_F32 && bt == CW_BF16) CW_LAUNCH(bf16_t, float, bf16_t);
  else if (dtype == CW_BF16 && wt == CW_BF16 && bt == CW_F32) CW_LAUNCH(bf16_t, bf16_t, float);
  else if (dtype == CW_BF16 && wt == CW_F32 && bt == CW_F32) CW_LAUNCH(bf16_t, float, float);
  else return CW_ERR_DTYPE;
#undef CW_LAUNCH
  return cw_launch_status();
}

// ---------------------------------------------------------------- squared ReLU, in place; a scale, in place
// x <- max(x, 0)^2, float32 inside.
template <typename T>
__global__ void relu_squared_kernel(T* __restrict__ x, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const float z = fmaxf(cw_to_float(x[i]), 0.0f);
    x[i] = cw_from_float<T>(z * z);
  }
}

CW_EXPORT int cw_relu_squared(void* x, int dtype, int64_t n, hipStream_t stream) {
  if (n < 0) return CW_ERR_ARG;
  if (n == 0) return CW_OK;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 262144) blocks = 262144;
  dim3 grid((unsigned)blocks), block(256);
  if (dtype == CW_F32) hipLaunchKernelGGL(relu_squared_kernel<float>, grid, block, 0, stream, (float*)x, n);
  else if (dtype == CW_BF16) hipLaunchKernelGGL(relu_squared_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)x, n);
  else return CW_ERR_DTYPE;
  return cw_launch_status();
}

// x <- x * s, float32 (logits).
__global__ void scale_kernel(float* __restrict__ x, int64_t n, float s) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) x[i] *= s;
}

CW_EXPORT int cw_scale(float* x, int64_t n, float s, hipStream_t stream) {
  if (n < 0) return CW_ERR_ARG;
  if (n == 0) return CW_OK;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 262144) blocks = 262144;
  hipLaunchKernelGGL(scale_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, x, n, s);
  return cw_launch_status();
}

// ---------------------------------------------------------------- tanh, in place
template <typename T>
__global__ void tanh_kernel(T* __restrict__ x, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    x[i] = cw_from_float<T>(tanhf(cw_to_float(x[i])));
}

CW_EXPORT int cw_tanh(void* x, int dtype, int64_t n, hipStream_t stream) {
  if (n < 0 || !x) return CW_ERR_ARG;
  if (n == 0) return CW_OK;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  if (dtype == CW_F32) hipLaunchKernelGGL(tanh_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, stream, (float*)x, n);
  else if (dtype == CW_BF16) hipLaunchKernelGGL(tanh_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, stream, (bf16_t*)x, n);
  else return CW_ERR_DTYPE;
  return cw_launch_status();
}

// ---------------------------------------------------------------- mixes of a token with the one before it
// out[s][t] = x[t] + (before[t] - x[t]) * mu[s], s < n_mix, float32 inside: ``before`` is the row
// of the request's token one position earlier: the row above in x, or for the first token of a
// request's portion what the request's state slot holds at ``prev_off`` (state rows are
// state_stride floats; a request's first token ever finds zeros there, its slot being fresh).
// items: (request, first token, tokens, 0), up to SHIFT_TOKENS tokens each. The workgroup of a
// request's first item then leaves the portion's last row in the slot, for the next step: it alone
// reads and writes the slot, in that order (a workgroup takes 256 columns of an item, a thread one).
#define SHIFT_TOKENS 16
#define SHIFT_MAX_MIXES 8
template <typename T, typename WT>
__global__ __launch_bounds__(256) void shift_mix_kernel(const T* __restrict__ x, const WT* __restrict__ mu, int n_mix,
                                                        float* __restrict__ state, int64_t state_stride, int64_t prev_off,
                                                        int n_slots, const int* __restrict__ state_slots,
                                                        const int* __restrict__ cu_q, const int* __restrict__ items,
                                                        T* __restrict__ out, int64_t n_tokens, int W) {
  const int* item = items + 4 * (int64_t)blockIdx.x;
  const int req = item[0], tok0 = item[1];
  const int row0 = cu_q[req], q_len = cu_q[req + 1] - row0;
  if (tok0 >= q_len) return;  // an item past the request's tokens (a batch of fixed shape)
  const int ntok = min(min(item[2], SHIFT_TOKENS), q_len - tok0);
  const int slot = state_slots[req];
  const bool has_slot = slot >= 0 && slot < n_slots;
  float* kept = has_slot ? state + (int64_t)slot * state_stride + prev_off : nullptr;
  // a thread owns one column of the item's tokens: what it reads of the slot it alone writes
  const int j = blockIdx.y * 256 + threadIdx.x;
  if (j >= W) return;
  float m[SHIFT_MAX_MIXES];
#pragma unroll
  for (int s = 0; s < SHIFT_MAX_MIXES; ++s) m[s] = s < n_mix ? cw_to_float(mu[(int64_t)s * W + j]) : 0.0f;
  float b = tok0 == 0 ? (kept ? kept[j] : 0.0f) : cw_to_float(x[((int64_t)row0 + tok0 - 1) * W + j]);
  for (int i = 0; i < ntok; ++i) {
    const int64_t row = (int64_t)row0 + tok0 + i;
    const float v = cw_to_float(x[row * W + j]);
#pragma unroll
    for (int s = 0; s < SHIFT_MAX_MIXES; ++s)
      if (s < n_mix) out[((int64_t)s * n_tokens + row) * W + j] = cw_from_float<T>(v + (b - v) * m[s]);
    b = v;
  }
  if (tok0 == 0 && kept) kept[j] = cw_to_float(x[((int64_t)row0 + q_len - 1) * W + j]);
}

CW_EXPORT int cw_shift_mix(const void* x, int dtype, const void* mu, int mu_dtype, int n_mix, float* state,
                           int64_t state_stride, int64_t prev_off, int n_slots, const int* state_slots, const int* cu_q,
                           const int* items, int n_items, void* out, int64_t n_tokens, int W, hipStream_t stream) {
  if (!x || !mu || !state || !state_slots || !cu_q || !items || !out) return CW_ERR_ARG;
  if (n_mix < 1 || n_mix > SHIFT_MAX_MIXES || n_items < 0 || n_tokens < 0 || W < 1 || n_slots < 1 || prev_off < 0 ||
      prev_off + W > state_stride)
    return CW_ERR_ARG;
  if (n_items == 0 || n_tokens == 0) return CW_OK;
#define CW_LAUNCH(T_, WT_)                                                                                          \
  hipLaunchKernelGGL((shift_mix_kernel<T_, WT_>), dim3(n_items, (W + 255) / 256), dim3(256), 0, stream, (const T_*)x, (const WT_*)mu, n_mix, \
                     state, state_stride, prev_off, n_slots, state_slots, cu_q, items, (T_*)out, n_tokens, W)
  if (dtype == CW_F32 && mu_dtype == CW_F32) CW_LAUNCH(float, float);
  else if (dtype == CW_BF16 && mu_dtype == CW_BF16) CW_LAUNCH(bf16_t, bf16_t);
  else if (dtype == CW_BF16 && mu_dtype == CW_F32) CW_LAUNCH(bf16_t, float);
  else return CW_ERR_DTYPE;
#undef CW_LAUNCH
  return cw_launch_status();
}

// ---------------------------------------------------------------- the stream beside the model's input
// resid[t] += a[t] + b[t] (what is still pending, either may be absent), then
// image[t] = [resid[t], input[t], e] in the activation type, e being ``extra`` columns that are 0
// but for a 1 in column ``hot``: the operand of a product that re-enters the stream from itself
// and the model's input, and picks one of ``extra`` learned rows on the way. float32 sums.
template <typename T>
__global__ __launch_bounds__(256) void stream_beside_input_kernel(float* __restrict__ resid, const T* __restrict__ a,
                                                                  const T* __restrict__ b, const float* __restrict__ input,
                                                                  T* __restrict__ image, int H, int extra, int hot) {
  const int64_t t = blockIdx.x;
  T* row = image + t * (2 * (int64_t)H + extra);
  for (int j = threadIdx.x; j < H; j += 256) {
    float v = resid[t * H + j];
    if (a) v += cw_to_float(a[t * H + j]);
    if (b) v += cw_to_float(b[t * H + j]);
    if (a || b) resid[t * H + j] = v;
    row[j] = cw_from_float<T>(v);
    row[H + j] = cw_from_float<T>(input[t * H + j]);
  }
  for (int e = threadIdx.x; e < extra; e += 256) row[2 * H + e] = cw_from_float<T>(e == hot ? 1.0f : 0.0f);
}

CW_EXPORT int cw_stream_beside_input(float* resid, const void* a, const void* b, const float* input, void* image, int dtype,
                                     int T, int H, int extra, int hot, hipStream_t stream) {
  if (T < 0 || H <= 0 || extra < 0 || hot < -1 || hot >= (extra ? extra : 1) || !resid || !input || !image) return CW_ERR_ARG;
  if (T == 0) return CW_OK;
  if (dtype == CW_F32)
    hipLaunchKernelGGL(stream_beside_input_kernel<float>, dim3(T), dim3(256), 0, stream, resid, (const float*)a, (const float*)b,
                       input, (float*)image, H, extra, hot);
  else if (dtype == CW_BF16)
    hipLaunchKernelGGL(stream_beside_input_kernel<bf16_t>, dim3(T), dim3(256), 0, stream, resid, (const bf16_t*)a,
                       (const bf16_t*)b, input, (bf16_t*)image, H, extra, hot);
  else return CW_ERR_DTYPE;
  return cw_launch_status();
}
