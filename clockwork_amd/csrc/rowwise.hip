// Row-wise kernels of blocks other than the pre-norm RMSNorm / SwiGLU one, for gfx950:
// embedding with a scale and a learned position table, residual add + LayerNorm (weight and
// bias), the sigmoid-gated residual add of two branches, act(gate) * up for the tanh form of GELU,
// the logit cap, the mean of two RMS-normed rows, and the RMS norm of whole query / key
// projections fused with the cache write.
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
