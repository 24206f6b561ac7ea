// A linear recurrence with a matrix state per head and a decay per key channel, for gfx950:
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T (q_scale * q_t),   S in float32 [dim, vdim],
// with the decay made inside from a low-rank projection: a_t = sigmoid(z_t)^(1/tau),
// z_t = A2 u_t + b (u_t the token's ``rank`` inputs). o_t is optionally RMS-normed over vdim
// with a weight shared by the heads and multiplied by silu(g_t).
//
// A workgroup owns one (request, head): the state lives in registers for the whole portion (a
// thread holds a run of rows of one column), tokens are walked in order, sixteen at a time: their
// q, k, v and decays are staged in LDS, the walk itself has no barrier, the outputs' partial sums
// over the row runs are added, normed and gated once per sixteen tokens. Decays, their logarithms,
// the state and the norm are float32 whatever the activation type T is.
#include "common.h"

#define LR_TC 16  // tokens staged at a time

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
__global__ __launch_bounds__(256) void linear_recurrence_kernel(LinRecParams p) {
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
  float* st = p.state + (((int64_t)slot * Hn + h) * D) * V;
#pragma unroll
  for (int rr = 0; rr < RPT; ++rr) S[rr] = (active && d0 + rr < D) ? st[(int64_t)(d0 + rr) * V + v] : 0.0f;

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
      for (int c = 0; c < p.rank; ++c) z += cw_to_float(w[c]) * cw_to_float(row[p.u_off + c]);
      // log(sigmoid(z)) without cancellation, then the 1/tau-th power
      const float ls = z < 0.0f ? z - log1pf(expf(z)) : -log1pf(expf(-z));
      as[idx] = expf(ls * p.inv_tau);
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
            S[rr] = as[t * D + d] * S[rr] + ks[t * D + d] * vv;
            po += qs[t * D + d] * S[rr];
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
          if (p.norm_w) val *= p.norm_w[c];
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
                                   hipStream_t stream) {
  if (n_requests < 0 || !proj || !a2 || !state || !state_slots || !cu_q || !out) return CW_ERR_ARG;
  if (heads <= 0 || rank <= 0 || n_slots <= 0 || q_off < 0 || k_off < 0 || v_off < 0 || u_off < 0) return CW_ERR_ARG;
  if (q_off + heads * dim > stride || k_off + heads * dim > stride || v_off + heads * vdim > stride ||
      u_off + rank > stride || (g_off >= 0 && g_off + heads * vdim > stride))
    return CW_ERR_ARG;
  if (!cw_linear_recurrence_supported(dim, vdim)) return CW_ERR_SIZE;
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
    hipLaunchKernelGGL((linear_recurrence_kernel<T_, RPT_>), grid, block, smem, stream, p);                        \
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
