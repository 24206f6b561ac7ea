// Softmax attention over a paged cache with four options that the plain kernels do not have, for
// gfx950: a key size that differs from the value size, a bias on the distance between query and
// key (score - r1[h] * log(1 + r2[h] * (i - j))), a learned extra term exp(sink[h]) in the softmax
// denominator, and a mixing of the normalised weights across heads before they meet the values
// (w'[h] = sum_g talk[h, g] * w[g]; head h applies w'[h] to the values of its own key/value head).
// Each option is off when its pointer is null.
//
// The mixing needs every head's normalised weight for a (query, key) pair at once, so a workgroup
// owns a run of up to BQ query tokens of one request with ALL heads, and walks the keys twice: the
// first walk finds every row's maximum and denominator, the second recomputes the scores, normalises,
// mixes across heads in LDS and multiplies with the values. Scores, weights and sums are float32.
// Keys and values come in chunks of KT keys, one key/value head at a time, through LDS.
#include "common.h"

#define SA_KT 32       // keys a chunk
#define SA_LANES 16    // lanes that share a (query, head) row of scores: 2 keys a lane and chunk
#define SA_MAX_ACC 32  // outputs a thread accumulates: BQ * heads * vdim <= 256 * SA_MAX_ACC

struct SinkAttnParams {
  const void* q;          // [T, q_stride]: a token's query heads, heads * dim elements
  int64_t q_stride;
  void* out;              // [T, heads * vdim]
  const void* k_cache;    // [rows, kv_heads, dim]
  const void* v_cache;    // [rows, kv_heads, vdim]
  const int* block_tables;  // [R, table_width]
  int table_width;
  const int* ctx_lens;    // [R] keys of each request once this step's tokens are cached
  const int* cu_q;        // [R + 1]
  const int* items;       // [n_items, 4]: request, first token of the run, tokens, unused
  const float* r1;        // [heads] or null
  const float* r2;        // [heads]
  const float* sink;      // [heads] or null
  const float* talk;      // [heads, heads] or null
  int heads, kv_heads, dim, vdim, block_size, window;
  float scale;
  int bq;                 // query tokens a workgroup takes at most
  int64_t cache_rows;
};

template <typename T>
__global__ __launch_bounds__(256) void sink_attention_kernel(SinkAttnParams p) {
  extern __shared__ __align__(16) float smem[];
  const int H = p.heads, G = p.kv_heads, D = p.dim, V = p.vdim, Hg = H / G, BQ = p.bq;
  const int tid = threadIdx.x;
  const int r = p.items[4 * blockIdx.x], tok0 = p.items[4 * blockIdx.x + 1];
  const int q_len = p.cu_q[r + 1] - p.cu_q[r];
  if (tok0 >= q_len) return;  // a run past the request's tokens (a batch of fixed shape)
  const int nq = min(min(p.items[4 * blockIdx.x + 2], BQ), q_len - tok0);
  const int pos0 = p.ctx_lens[r] - q_len + tok0;  // position of the run's first query
  const int last = pos0 + nq - 1;
  const int lo = p.window > 0 ? max(0, pos0 - p.window + 1) : 0;
  const int64_t row0 = p.cu_q[r] + tok0;
  const int* table = p.block_tables + (int64_t)r * p.table_width;

  float* Qs = smem;                      // [BQ][H * D]
  float* Ks = Qs + BQ * H * D;           // [KT][D + 1]
  float* Vs = Ks + SA_KT * (D + 1);      // [KT][V]
  float* Ss = Vs + SA_KT * V;            // [BQ * H][KT] normalised weights
  float* Ps = Ss + BQ * H * SA_KT;       // [BQ * H][KT] the same after the mixing
  float* Mx = Ps + BQ * H * SA_KT;       // [BQ * H]
  float* Lx = Mx + BQ * H;               // [BQ * H]
  float* Tk = Lx + BQ * H;               // [H * H]

  const T* q = (const T*)p.q;
  for (int idx = tid; idx < BQ * H * D; idx += 256) {
    const int i = idx / (H * D), c = idx - i * (H * D);
    Qs[idx] = i < nq ? cw_to_float(q[(row0 + i) * p.q_stride + c]) : 0.0f;
  }
  for (int idx = tid; idx < BQ * H; idx += 256) {
    const int g = idx % H;
    Mx[idx] = p.sink ? p.sink[g] : -3.0e38f;
    Lx[idx] = p.sink ? 1.0f : 0.0f;
  }
  if (p.talk)
    for (int idx = tid; idx < H * H; idx += 256) Tk[idx] = p.talk[idx];

  const T* kc = (const T*)p.k_cache;
  const T* vc = (const T*)p.v_cache;
  // one key/value head's rows of a chunk into LDS; keys past ``last`` or without a page are zeros
  auto load_rows = [&](const T* cache, int width, int c, int k0, float* dst, int dst_stride) {
    for (int idx = tid; idx < SA_KT * width; idx += 256) {
      const int jj = idx / width, e = idx - jj * width;
      const int j = k0 + jj;
      float v = 0.0f;
      if (j <= last) {
        const int page = table[j / p.block_size];
        const int64_t row = (int64_t)page * p.block_size + j % p.block_size;
        if (page >= 0 && row < p.cache_rows) v = cw_to_float(cache[(row * G + c) * width + e]);
      }
      dst[jj * dst_stride + e] = v;
    }
  };
  const int lane = tid % SA_LANES, rgroup = tid / SA_LANES;  // 16 groups of 16 lanes
  constexpr int KPL = SA_KT / SA_LANES;
  // the scores of row (i, g) against the chunk's keys lane, lane + 16: -inf where the key is not seen
  auto scores = [&](int i, int g, int k0, float* s) {
    const float* qv = Qs + (i * H + g) * D;
    const int pos = pos0 + i;
#pragma unroll
    for (int u = 0; u < KPL; ++u) {
      const int jj = lane + u * SA_LANES;
      const int j = k0 + jj;
      const float* kv = Ks + jj * (D + 1);
      float acc = 0.0f;
      for (int d = 0; d < D; ++d) acc += qv[d] * kv[d];
      acc *= p.scale;
      const int dist = pos - j;
      if (p.r1) acc -= p.r1[g] * log1pf(p.r2[g] * (float)max(dist, 0));
      const bool seen = i < nq && dist >= 0 && (p.window <= 0 || dist < p.window);
      s[u] = seen ? acc : -INFINITY;
    }
  };

  // ---- first walk: every row's maximum and denominator
  for (int k0 = lo; k0 <= last; k0 += SA_KT) {
    for (int c = 0; c < G; ++c) {
      __syncthreads();
      load_rows(kc, D, c, k0, Ks, D + 1);
      __syncthreads();
      for (int rw = rgroup; rw < BQ * Hg; rw += 256 / SA_LANES) {
        const int i = rw / Hg, g = c * Hg + rw % Hg;
        float s[KPL];
        scores(i, g, k0, s);
        float cm = s[0];
#pragma unroll
        for (int u = 1; u < KPL; ++u) cm = fmaxf(cm, s[u]);
#pragma unroll
        for (int off = SA_LANES / 2; off > 0; off >>= 1) cm = fmaxf(cm, __shfl_xor(cm, off, SA_LANES));
        const float m_old = Mx[i * H + g];
        const float m_new = fmaxf(m_old, cm);
        float sum = 0.0f;
#pragma unroll
        for (int u = 0; u < KPL; ++u) sum += expf(s[u] - m_new);
#pragma unroll
        for (int off = SA_LANES / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off, SA_LANES);
        if (lane == 0) {
          Lx[i * H + g] = Lx[i * H + g] * expf(m_old - m_new) + sum;
          Mx[i * H + g] = m_new;
        }
      }
    }
  }
  __syncthreads();

  // ---- second walk: normalised weights, mixed across heads, times the values
  const int per_head = BQ * Hg * V;               // outputs of the heads of one key/value head
  const int kpc = (per_head + 255) / 256;         // accumulators a thread holds for them
  const int n_acc = G * kpc;
  float acc[SA_MAX_ACC];
#pragma unroll
  for (int k = 0; k < SA_MAX_ACC; ++k) acc[k] = 0.0f;
  const float* Ws = p.talk ? Ps : Ss;
  for (int k0 = lo; k0 <= last; k0 += SA_KT) {
    for (int c = 0; c < G; ++c) {
      __syncthreads();
      load_rows(kc, D, c, k0, Ks, D + 1);
      __syncthreads();
      for (int rw = rgroup; rw < BQ * Hg; rw += 256 / SA_LANES) {
        const int i = rw / Hg, g = c * Hg + rw % Hg;
        float s[KPL];
        scores(i, g, k0, s);
        const float m = Mx[i * H + g], l = Lx[i * H + g], inv = l > 0.0f ? 1.0f / l : 0.0f;
#pragma unroll
        for (int u = 0; u < KPL; ++u) Ss[(i * H + g) * SA_KT + lane + u * SA_LANES] = expf(s[u] - m) * inv;
      }
    }
    __syncthreads();
    if (p.talk) {
      for (int idx = tid; idx < BQ * H * SA_KT; idx += 256) {
        const int jj = idx % SA_KT, row = idx / SA_KT, i = row / H, h = row - i * H;
        float v = 0.0f;
        for (int g = 0; g < H; ++g) v += Tk[h * H + g] * Ss[(i * H + g) * SA_KT + jj];
        Ps[idx] = v;
      }
    }
    int cur = -1;
#pragma unroll
    for (int kk = 0; kk < SA_MAX_ACC; ++kk) {
      const int c = kk / kpc, k = kk - c * kpc;
      if (kk < n_acc && c != cur) {  // the same for every thread
        __syncthreads();
        load_rows(vc, V, c, k0, Vs, V);
        __syncthreads();
        cur = c;
      }
      const int o = tid + k * 256;
      if (kk < n_acc && o < per_head) {
        const int dv = o % V, ih = o / V, i = ih / Hg, h = c * Hg + ih % Hg;
        const float* w = Ws + (i * H + h) * SA_KT;
        float a = acc[kk];
        for (int jj = 0; jj < SA_KT; ++jj) a += w[jj] * Vs[jj * V + dv];
        acc[kk] = a;
      }
    }
  }
  T* out = (T*)p.out;
#pragma unroll
  for (int kk = 0; kk < SA_MAX_ACC; ++kk) {
    const int c = kk / kpc, k = kk - c * kpc;
    const int o = tid + k * 256;
    if (kk < n_acc && o < per_head) {
      const int dv = o % V, ih = o / V, i = ih / Hg, h = c * Hg + ih % Hg;
      if (i < nq) out[(row0 + i) * (int64_t)(H * V) + h * V + dv] = cw_from_float<T>(acc[kk]);
    }
  }
}

static int64_t sink_attention_lds_floats(int bq, int H, int D, int V) {
  return (int64_t)bq * H * D + SA_KT * (D + 1) + SA_KT * V + 2 * (int64_t)bq * H * SA_KT + 2 * bq * H + H * H;
}

// The most query tokens a workgroup can take for heads of this geometry (a power of two up to 16;
// 0: the geometry is beyond the kernel: more than 8192 outputs a token, or no room in LDS).
CW_EXPORT int cw_sink_attention_max_bq(int heads, int kv_heads, int dim, int vdim) {
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || dim <= 0 || vdim <= 0) return 0;
  for (int bq = 16; bq >= 1; bq >>= 1) {
    const int64_t per_head = (int64_t)bq * (heads / kv_heads) * vdim;
    if (kv_heads * ((per_head + 255) / 256) > SA_MAX_ACC) continue;
    if (sink_attention_lds_floats(bq, heads, dim, vdim) * 4 > 150 * 1024) continue;
    return bq;
  }
  return 0;
}

CW_EXPORT int cw_sink_attention(int dtype, const void* q, int64_t q_stride, void* out, const void* k_cache,
                                const void* v_cache, int64_t cache_rows, const int* block_tables, int table_width,
                                const int* ctx_lens, const int* cu_q, const int* items, int n_items, int bq,
                                const float* r1, const float* r2, const float* sink, const float* talk, int heads,
                                int kv_heads, int dim, int vdim, int block_size, int window, float scale,
                                hipStream_t stream) {
  if (n_items < 0 || !q || !out || !k_cache || !v_cache || !block_tables || !ctx_lens || !cu_q || !items)
    return CW_ERR_ARG;
  if (block_size <= 0 || table_width <= 0 || window < 0 || (r1 && !r2)) return CW_ERR_ARG;
  const int most = cw_sink_attention_max_bq(heads, kv_heads, dim, vdim);
  if (most == 0) return CW_ERR_SIZE;
  if (bq < 1 || bq > most) return CW_ERR_ARG;
  if (n_items == 0) return CW_OK;
  SinkAttnParams p;
  p.q = q; p.q_stride = q_stride; p.out = out; p.k_cache = k_cache; p.v_cache = v_cache;
  p.block_tables = block_tables; p.table_width = table_width; p.ctx_lens = ctx_lens; p.cu_q = cu_q; p.items = items;
  p.r1 = r1; p.r2 = r2; p.sink = sink; p.talk = talk;
  p.heads = heads; p.kv_heads = kv_heads; p.dim = dim; p.vdim = vdim; p.block_size = block_size; p.window = window;
  p.scale = scale; p.bq = bq; p.cache_rows = cache_rows;
  const size_t smem = (size_t)sink_attention_lds_floats(bq, heads, dim, vdim) * sizeof(float);
  dim3 grid(n_items), block(256);
#define CW_LAUNCH(T_)                                                                                             \
  do {                                                                                                            \
    if (smem > 48 * 1024 && hipFuncSetAttribute((const void*)sink_attention_kernel<T_>,                           \
                                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) \
      return CW_ERR_LAUNCH;                                                                                       \
    hipLaunchKernelGGL((sink_attention_kernel<T_>), grid, block, smem, stream, p);                                \
  } while (0)
  if (dtype == CW_F32) CW_LAUNCH(float);
  else if (dtype == CW_BF16) CW_LAUNCH(bf16_t);
  else return CW_ERR_DTYPE;
#undef CW_LAUNCH
  return cw_launch_status();
}
