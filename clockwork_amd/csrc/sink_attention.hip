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
  int tb_len;             // matrix-core kernel: entries of the block table a workgroup keeps in LDS
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
      // the loads are unconditional (a key past ``last`` or without a page reads row 0 and is dropped
      // by a select): loads under conditions of their own would be waited for one by one
      const int j = min(k0 + jj, last);
      const int page = table[j / p.block_size];
      const int64_t row = (int64_t)page * p.block_size + j % p.block_size;
      const bool there = k0 + jj <= last && page >= 0 && row < p.cache_rows;
      const float v = cw_to_float(cache[((there ? row : 0) * G + c) * width + e]);
      dst[jj * dst_stride + e] = there ? v : 0.0f;
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
  p.scale = scale; p.bq = bq; p.cache_rows = cache_rows; p.tb_len = 0;
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

// ======================================================================================
// Single tokens (one query a request): three small kernels that share a request's keys among
// workgroups, since a request alone would leave all but one compute unit idle.
//
//   scores:  a workgroup per (request, run of ``sk`` keys): a thread takes one key of one
//            key/value head, reads its row once in 16-byte pieces and multiplies it with all query
//            heads of the group (the queries wait in LDS); scale, distance bias, mask. The scores
//            go to a float32 workspace, each head's maximum and sum of exponentials over the run
//            beside them.
//   values:  the same grid: every workgroup puts the runs' maxima and sums (and the sink)
//            together, so it knows each head's final denominator, normalises its run's scores,
//            mixes them across heads in LDS and multiplies with its run's values: a thread takes
//            one value column of one key/value head for all query heads of the group.
//   merge:   the runs' partial outputs are added in order.
// ======================================================================================
#define SD_MAX_SK 128
#define SD_HG 16      // query heads of a group that a thread handles at a time

struct SinkDecodeParams {
  const void* q;
  int64_t q_stride;
  void* out;
  const void* k_cache;
  const void* v_cache;
  const int* block_tables;
  int table_width;
  const int* ctx_lens;
  const int* cu_q;
  const float* r1;
  const float* r2;
  const float* sink;
  const float* talk;
  float* scores;   // [R, heads, n_runs * sk]
  float* stats;    // [R, n_runs, heads, 2]
  float* partial;  // [R, n_runs, heads * vdim]
  int heads, kv_heads, dim, vdim, block_size, window, sk, n_runs;
  float scale;
  int64_t cache_rows;
};

// keys that request r's single token sees: [lo, pos]; false if the request has another number of tokens
__device__ __forceinline__ bool sd_range(const SinkDecodeParams& p, int r, int& lo, int& pos) {
  if (p.cu_q[r + 1] - p.cu_q[r] != 1) return false;
  pos = p.ctx_lens[r] - 1;
  lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;
  return pos >= 0;
}

template <typename T> struct RowVec;
template <> struct RowVec<float> {
  static constexpr int N = 4;
  __device__ static void load(const float* p, float* o) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
  }
};
template <> struct RowVec<bf16_t> {
  static constexpr int N = 8;
  __device__ static void load(const bf16_t* p, float* o) {
    const uint4 v = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) { o[2 * i] = __uint_as_float(w[i] << 16); o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u); }
  }
};

template <typename T>
__global__ __launch_bounds__(256) void sink_decode_scores_kernel(SinkDecodeParams p) {
  extern __shared__ __align__(16) float smem[];
  const int H = p.heads, G = p.kv_heads, D = p.dim, Hg = H / G, SK = p.sk;
  const int r = blockIdx.x, run = blockIdx.y, tid = threadIdx.x;
  int lo, pos;
  if (!sd_range(p, r, lo, pos)) return;
  const int k0 = lo + run * SK;
  if (k0 > pos) return;
  float* qs = smem;            // [H * D]
  float* sc = qs + H * D;      // [H][SK]
  const T* q = (const T*)p.q + (int64_t)p.cu_q[r] * p.q_stride;
  for (int i = tid; i < H * D; i += 256) qs[i] = cw_to_float(q[i]);
  __syncthreads();
  const int* table = p.block_tables + (int64_t)r * p.table_width;
  const T* kc = (const T*)p.k_cache;
  constexpr int N = RowVec<T>::N;
  const bool vec = D % N == 0 && !((uintptr_t)kc & 15);
  // a run of few keys leaves threads over: 2, 4 or 8 neighbouring lanes then share a key's row
  // (each a run of its elements) and add their sums up with shuffles
  int tpk = 1;
  while (vec && tpk < 8 && SK * G * tpk * 2 <= 256 && D % (tpk * 2 * N) == 0) tpk *= 2;
  const int dpt = D / tpk;  // elements of a row that a thread takes
  for (int idx0 = tid; idx0 < SK * G * tpk; idx0 += 256) {
    const int idx = idx0 / tpk, piece = idx0 - idx * tpk;
    const int c = idx / SK, jj = idx - c * SK;
    const int j = k0 + jj;
    const bool seen = j <= pos;
    // a key that is not seen or has no page reads row 0 and its products are dropped: every
    // thread's loads are then the same instructions, asked for together
    const int jt = min(j, pos);
    const int page = table[jt / p.block_size];
    const int64_t row = (int64_t)page * p.block_size + jt % p.block_size;
    const bool there = seen && page >= 0 && row < p.cache_rows;
    const T* krow = kc + ((there ? row : 0) * G + c) * D;
    for (int h0 = 0; h0 < Hg; h0 += SD_HG) {
      float acc[SD_HG];
#pragma unroll
      for (int e = 0; e < SD_HG; ++e) acc[e] = 0.0f;
      {
        if (vec) {
          // four pieces of the row are asked for together: a trip to memory that waits for the one
          // before costs more than all the arithmetic of the row
          const int d_end = (piece + 1) * dpt;
          for (int d0 = piece * dpt; d0 < d_end; d0 += 4 * N) {
            float kv[4][N];
#pragma unroll
            for (int b = 0; b < 4; ++b)
              if (d0 + b * N < d_end) RowVec<T>::load(krow + d0 + b * N, kv[b]);
#pragma unroll
            for (int b = 0; b < 4; ++b) {
              if (d0 + b * N < d_end) {
#pragma unroll
                for (int e = 0; e < SD_HG; ++e) {
                  if (h0 + e < Hg) {
                    const float* qv = qs + (c * Hg + h0 + e) * D + d0 + b * N;
#pragma unroll
                    for (int u = 0; u < N; ++u) acc[e] += qv[u] * kv[b][u];
                  }
                }
              }
            }
          }
        } else {
          for (int d = piece * dpt; d < (piece + 1) * dpt; ++d) {
            const float kv = cw_to_float(krow[d]);
#pragma unroll
            for (int e = 0; e < SD_HG; ++e)
              if (h0 + e < Hg) acc[e] += qs[(c * Hg + h0 + e) * D + d] * kv;
          }
        }
      }
      for (int off = 1; off < tpk; off <<= 1) {
#pragma unroll
        for (int e = 0; e < SD_HG; ++e) acc[e] += __shfl_xor(acc[e], off, 64);
      }
#pragma unroll
      for (int e = 0; e < SD_HG; ++e) {
        if (h0 + e < Hg && piece == 0) {
          const int g = c * Hg + h0 + e;
          float s = there ? acc[e] * p.scale : 0.0f;
          if (p.r1) s -= p.r1[g] * log1pf(p.r2[g] * (float)max(pos - j, 0));
          sc[g * SK + jj] = seen ? s : -INFINITY;
        }
      }
    }
  }
  __syncthreads();
  const int wave = tid >> 6, lane = tid & 63;
  float* ws = p.scores + ((int64_t)r * H) * (p.n_runs * SK) + run * SK;
  for (int g = wave; g < H; g += 4) {
    float m = -INFINITY;
    for (int jj = lane; jj < SK; jj += 64) {
      const float s = sc[g * SK + jj];
      ws[(int64_t)g * (p.n_runs * SK) + jj] = s;
      m = fmaxf(m, s);
    }
    m = cw_wave_max(m);
    float l = 0.0f;
    for (int jj = lane; jj < SK; jj += 64) l += expf(sc[g * SK + jj] - m);
    l = cw_wave_sum(l);
    if (lane == 0) {
      float* st = p.stats + (((int64_t)r * p.n_runs + run) * H + g) * 2;
      st[0] = m;
      st[1] = l;
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void sink_decode_values_kernel(SinkDecodeParams p) {
  extern __shared__ __align__(16) float smem[];
  const int H = p.heads, G = p.kv_heads, V = p.vdim, Hg = H / G, SK = p.sk;
  const int r = blockIdx.x, run = blockIdx.y, tid = threadIdx.x;
  int lo, pos;
  if (!sd_range(p, r, lo, pos)) return;
  const int k0 = lo + run * SK;
  if (k0 > pos) return;
  const int runs = (pos - lo) / SK + 1;  // the runs that hold keys of this request
  float* Pn = smem;              // [H][SK] normalised weights
  float* Pm = Pn + H * SK;       // [H][SK] mixed
  float* mg = Pm + H * SK;       // [H] maxima
  float* il = mg + H;            // [H] 1 / denominators
  int* rows = (int*)(il + H);    // [SK] cache rows of the run's keys (-1: none)
  float* tk = (float*)(rows + SK);  // [H][H] the mixing matrix
  if (p.talk)
    for (int i = tid; i < H * H; i += 256) tk[i] = p.talk[i];
  // every head's final maximum and denominator from the runs' own: a wave per head, a lane per run
  for (int g = tid >> 6; g < H; g += 4) {
    const int ln = tid & 63;
    const float* st = p.stats + ((int64_t)r * p.n_runs * H + g) * 2;
    float m = p.sink ? p.sink[g] : -INFINITY;
    for (int s = ln; s < runs; s += 64) m = fmaxf(m, st[(int64_t)s * H * 2]);
    m = cw_wave_max(m);
    float l = 0.0f;
    for (int s = ln; s < runs; s += 64) l += st[(int64_t)s * H * 2 + 1] * expf(st[(int64_t)s * H * 2] - m);
    l = cw_wave_sum(l);
    if (p.sink) l += expf(p.sink[g] - m);
    if (ln == 0) {
      mg[g] = m;
      il[g] = l > 0.0f ? 1.0f / l : 0.0f;
    }
  }
  const int* table = p.block_tables + (int64_t)r * p.table_width;
  for (int jj = tid; jj < SK; jj += 256) {
    const int j = k0 + jj;
    int row = -1;
    if (j <= pos) {
      const int page = table[j / p.block_size];
      const int64_t at = (int64_t)page * p.block_size + j % p.block_size;
      if (page >= 0 && at < p.cache_rows) row = (int)at;
    }
    rows[jj] = row;
  }
  __syncthreads();
  const float* ws = p.scores + ((int64_t)r * H) * (p.n_runs * SK) + run * SK;
  for (int idx = tid; idx < H * SK; idx += 256) {
    const int g = idx / SK, jj = idx - g * SK;
    Pn[idx] = expf(ws[(int64_t)g * (p.n_runs * SK) + jj] - mg[g]) * il[g];
  }
  __syncthreads();
  const float* W = Pn;
  if (p.talk) {
    for (int idx = tid; idx < H * SK; idx += 256) {
      const int h = idx / SK, jj = idx - h * SK;
      float v = 0.0f;
      for (int g = 0; g < H; ++g) v += tk[h * H + g] * Pn[g * SK + jj];
      Pm[idx] = v;
    }
    __syncthreads();
    W = Pm;
  }
  const int nk = min(SK, pos - k0 + 1);
  const T* vc = (const T*)p.v_cache;
  float* part = p.partial + ((int64_t)r * p.n_runs + run) * (H * V);
  for (int idx = tid; idx < G * V; idx += 256) {
    const int c = idx / V, dv = idx - c * V;
    for (int h0 = 0; h0 < Hg; h0 += SD_HG) {
      float acc[SD_HG];
#pragma unroll
      for (int e = 0; e < SD_HG; ++e) acc[e] = 0.0f;
      // thirty-two keys' values are asked for together: the trips to memory run side by side
      for (int j0 = 0; j0 < nk; j0 += 32) {
        float v[32];
#pragma unroll
        for (int u = 0; u < 32; ++u) {
          // the load itself is unconditional (row 0 stands in, its value is dropped): a load under a
          // condition of its own is waited for before the next one is asked for
          const int row = j0 + u < nk ? rows[j0 + u] : -1;
          const float x = cw_to_float(vc[((int64_t)max(row, 0) * G + c) * V + dv]);
          v[u] = row >= 0 ? x : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 32; ++u) {
          if (j0 + u < nk) {
#pragma unroll
            for (int e = 0; e < SD_HG; ++e)
              if (h0 + e < Hg) acc[e] += W[(c * Hg + h0 + e) * SK + j0 + u] * v[u];
          }
        }
      }
#pragma unroll
      for (int e = 0; e < SD_HG; ++e)
        if (h0 + e < Hg) part[(c * Hg + h0 + e) * V + dv] = acc[e];
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void sink_decode_merge_kernel(SinkDecodeParams p) {
  const int r = blockIdx.x;
  int lo, pos;
  if (!sd_range(p, r, lo, pos)) return;
  const int runs = (pos - lo) / p.sk + 1;
  const int n = p.heads * p.vdim;
  T* out = (T*)p.out + (int64_t)p.cu_q[r] * n;
  const float* part = p.partial + (int64_t)r * p.n_runs * n;
  for (int i = blockIdx.y * 256 + threadIdx.x; i < n; i += gridDim.y * 256) {
    float v = part[i];
    for (int s = 1; s < runs; ++s) v += part[(int64_t)s * n + i];
    out[i] = cw_from_float<T>(v);
  }
}

// floats of workspace for R single tokens whose keys are cut into n_runs runs of sk keys
CW_EXPORT int64_t cw_sink_decode_workspace_floats(int n_requests, int n_runs, int sk, int heads, int vdim) {
  return (int64_t)n_requests * heads * n_runs * sk + (int64_t)n_requests * n_runs * heads * 2 +
         (int64_t)n_requests * n_runs * heads * vdim;
}

CW_EXPORT int cw_sink_decode_supported(int heads, int kv_heads, int dim, int vdim) {
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || dim <= 0 || vdim <= 0) return 0;
  const int64_t a = ((int64_t)heads * dim + (int64_t)heads * SD_MAX_SK) * 4;
  const int64_t b = (2 * (int64_t)heads * SD_MAX_SK + 2 * heads + SD_MAX_SK + (int64_t)heads * heads) * 4;
  return a <= 150 * 1024 && b <= 150 * 1024 ? 1 : 0;
}

// Every request of the step has one token (requests with another count are left alone). The keys a
// token sees ([max(0, pos - window + 1), pos]) are cut into runs of sk keys from their first;
// n_runs is the most runs any request has (the host knows the longest context).
CW_EXPORT int cw_sink_decode(int dtype, const void* q, int64_t q_stride, void* out, const void* k_cache,
                             const void* v_cache, int64_t cache_rows, const int* block_tables, int table_width,
                             const int* ctx_lens, const int* cu_q, int n_requests, int sk, int n_runs, float* workspace,
                             const float* r1, const float* r2, const float* sink, const float* talk, int heads,
                             int kv_heads, int dim, int vdim, int block_size, int window, float scale, hipStream_t stream) {
  if (n_requests < 0 || !q || !out || !k_cache || !v_cache || !block_tables || !ctx_lens || !cu_q || !workspace)
    return CW_ERR_ARG;
  if (block_size <= 0 || table_width <= 0 || window < 0 || (r1 && !r2) || sk < 1 || sk > SD_MAX_SK || n_runs < 1)
    return CW_ERR_ARG;
  if (!cw_sink_decode_supported(heads, kv_heads, dim, vdim)) return CW_ERR_SIZE;
  if (n_runs > 65535) return CW_ERR_SIZE;
  if (n_requests == 0) return CW_OK;
  SinkDecodeParams p;
  p.q = q; p.q_stride = q_stride; p.out = out; p.k_cache = k_cache; p.v_cache = v_cache;
  p.block_tables = block_tables; p.table_width = table_width; p.ctx_lens = ctx_lens; p.cu_q = cu_q;
  p.r1 = r1; p.r2 = r2; p.sink = sink; p.talk = talk;
  p.scores = workspace;
  p.stats = p.scores + (int64_t)n_requests * heads * n_runs * sk;
  p.partial = p.stats + (int64_t)n_requests * n_runs * heads * 2;
  p.heads = heads; p.kv_heads = kv_heads; p.dim = dim; p.vdim = vdim; p.block_size = block_size; p.window = window;
  p.sk = sk; p.n_runs = n_runs; p.scale = scale; p.cache_rows = cache_rows;
  const size_t smem1 = ((size_t)heads * dim + (size_t)heads * sk) * sizeof(float);
  const size_t smem2 = (2 * (size_t)heads * sk + 2 * heads + sk + (size_t)heads * heads) * sizeof(float);
  const dim3 grid(n_requests, n_runs), block(256);
  int my = (heads * vdim + 255) / 256;
  if (my > 64) my = 64;
#define CW_LAUNCH(T_)                                                                                                  \
  do {                                                                                                                 \
    if (smem1 > 48 * 1024 && hipFuncSetAttribute((const void*)sink_decode_scores_kernel<T_>,                           \
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem1) != hipSuccess)  \
      return CW_ERR_LAUNCH;                                                                                            \
    if (smem2 > 48 * 1024 && hipFuncSetAttribute((const void*)sink_decode_values_kernel<T_>,                           \
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem2) != hipSuccess)  \
      return CW_ERR_LAUNCH;                                                                                            \
    hipLaunchKernelGGL((sink_decode_scores_kernel<T_>), grid, block, smem1, stream, p);                                \
    hipLaunchKernelGGL((sink_decode_values_kernel<T_>), grid, block, smem2, stream, p);                                \
    hipLaunchKernelGGL((sink_decode_merge_kernel<T_>), dim3(n_requests, my), block, 0, stream, p);                     \
  } while (0)
  if (dtype == CW_F32) CW_LAUNCH(float);
  else if (dtype == CW_BF16) CW_LAUNCH(bf16_t);
  else return CW_ERR_DTYPE;
#undef CW_LAUNCH
  return cw_launch_status();
}

// ======================================================================================
// Portions in bfloat16 on the matrix cores. A workgroup owns 16 consecutive query tokens of one
// request with ALL heads (the mixing across heads needs them together); its 4 waves share the
// heads (wave w takes heads w, w + 4, ...). The keys are walked twice in chunks of 32, as in the
// kernel above: first each row's maximum and denominator, then normalised weights, their mixing
// across heads and the product with the values.
//
//   scores   S[16 q, 16 keys] = Q K^T     v_mfma_f32_16x16x32_bf16, Q fragments in registers for the
//                                         whole kernel, K from an LDS tile shared by the waves;
//   softmax  float32, on the lane's four rows of a tile; a row's statistics are finished across
//            the 16 lanes that share it once, after the first walk, and stay in registers;
//   mixing   the normalised weights of all heads meet in LDS as float32 [head][query][key]; a lane
//            then makes, for each of its wave's heads, the 8 mixed weights that are its part of the
//            next product's A operand;
//   values   O[16 q, 16 dv] += P' V       P' is float32: it is fed as two bfloat16 operands, its
//            leading 8 bits and the rounded rest, so the weights keep 16 bits of mantissa; V comes
//            from an LDS tile that holds the chunk transposed, [dv][key].
// ======================================================================================
typedef __attribute__((ext_vector_type(8))) __bf16 sa_bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float sa_f32x4_t;
#define SM_KT 32
#define SM_PROW 36   // floats a (head, query) row of weights takes in LDS: 32 and a pad against bank conflicts

__device__ __forceinline__ sa_bf16x8_t sm_load8(const bf16_t* p) {
  return *reinterpret_cast<const sa_bf16x8_t*>(p);
}

// HPW: heads a wave holds at most; D32: dim / 32; V16: vdim / 16; VS: workgroups that share a run's
// value columns (blockIdx.y: each makes all the weights and its own V16 / VS column tiles of the
// output; a launch of few runs fills the card that way)
template <int HPW, int D32, int V16, int VS>
__global__ __launch_bounds__(256) void sink_prefill_mfma_kernel(SinkAttnParams p) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  constexpr int D = D32 * 32, V = V16 * 16, NT = V16 / VS, VW = NT * 16;
  const int v0 = blockIdx.y * VW;   // this workgroup's first value column
  constexpr int KROW = D + 8;        // bf16 elements a key row takes in LDS
  constexpr int VROW = SM_KT + 8;    // bf16 elements a value column takes in LDS
  const int H = p.heads, G = p.kv_heads, Hg = H / G;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int l16 = lane & 15, slot = lane >> 4;
  const int r = p.items[4 * blockIdx.x], tok0 = p.items[4 * blockIdx.x + 1];
  const int q_len = p.cu_q[r + 1] - p.cu_q[r];
  if (tok0 >= q_len) return;
  const int nq = min(min(p.items[4 * blockIdx.x + 2], 16), q_len - tok0);
  const int pos0 = p.ctx_lens[r] - q_len + tok0;
  const int last = pos0 + nq - 1;
  const int lo = p.window > 0 ? max(0, pos0 - p.window + 1) : 0;
  const int64_t row0 = p.cu_q[r] + tok0;
  const int* table = p.block_tables + (int64_t)r * p.table_width;

  bf16_t* Ks = reinterpret_cast<bf16_t*>(smem_raw);              // [G][KT][KROW]
  bf16_t* Vt = Ks + G * SM_KT * KROW;                            // [G][VW][VROW]
  float* Pn = reinterpret_cast<float*>(Vt + G * VW * VROW);      // [H][16][SM_PROW]
  float* Tk = Pn + H * 16 * SM_PROW;                             // [H][H]
  int* Tb = reinterpret_cast<int*>(Tk + H * H);                  // [tb_len] pages of the keys this run sees

  const bf16_t* q = (const bf16_t*)p.q;
  const bf16_t* kc = (const bf16_t*)p.k_cache;
  const bf16_t* vc = (const bf16_t*)p.v_cache;
  if (p.talk)
    for (int i = tid; i < H * H; i += 256) Tk[i] = p.talk[i];
  // the pages of the keys in [lo, last]: looked up once, so a chunk's loads do not wait for the table
  const int tb0 = lo / p.block_size;
  for (int i = tid; i < p.tb_len; i += 256) Tb[i] = tb0 + i < p.table_width ? table[tb0 + i] : -1;
  __syncthreads();

  // this wave's heads and their query fragments: lane = query l16, 8 elements at slot
  sa_bf16x8_t qf[HPW][D32];
  const int qi = min(l16, nq - 1);
#pragma unroll
  for (int a = 0; a < HPW; ++a) {
    const int g = min(wave + 4 * a, H - 1);
#pragma unroll
    for (int ks = 0; ks < D32; ++ks) qf[a][ks] = sm_load8(q + (row0 + qi) * p.q_stride + g * D + ks * 32 + slot * 8);
  }

  // A chunk's keys (and values) of every key/value head travel in two steps: from the pages into
  // registers (asked for one chunk ahead, so the trip to memory runs beside the products of the
  // chunk before), then into LDS. Keys past ``last`` or without a page are zeros. A thread moves up
  // to PF pieces of 16 bytes of each (the host sees to it that this is enough).
  constexpr int PF = 4;
  uint4 kreg[PF], vreg[PF];
  auto row_of = [&](int j) -> int64_t {
    const int slot_ = min(max(j / p.block_size - tb0, 0), p.tb_len - 1);
    const int page = Tb[slot_];
    const int64_t row = (int64_t)page * p.block_size + j % p.block_size;
    return (j <= last && j / p.block_size - tb0 < p.tb_len && page >= 0 && row < p.cache_rows) ? row : -1;
  };
  auto fetch_keys = [&](int k0) {
    constexpr int PER_ROW = D / 8;
#pragma unroll
    for (int it = 0; it < PF; ++it) {
      const int idx = tid + it * 256;
      // every load is unconditional (a piece past the chunk or without a page reads row 0 and is
      // dropped): loads under conditions of their own would be waited for one by one
      const int at = min(idx, G * SM_KT * PER_ROW - 1);
      const int e = at % PER_ROW, jj = (at / PER_ROW) % SM_KT, c = at / (PER_ROW * SM_KT);
      const int64_t row = row_of(k0 + jj);
      const uint4 x = *reinterpret_cast<const uint4*>(kc + ((row >= 0 ? row : 0) * G + c) * D + e * 8);
      kreg[it] = (row >= 0 && idx == at) ? x : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_keys = [&]() {
    constexpr int PER_ROW = D / 8;
#pragma unroll
    for (int it = 0; it < PF; ++it) {
      const int idx = tid + it * 256;
      if (idx < G * SM_KT * PER_ROW) {
        const int e = idx % PER_ROW, jj = (idx / PER_ROW) % SM_KT, c = idx / (PER_ROW * SM_KT);
        *reinterpret_cast<uint4*>(Ks + (c * SM_KT + jj) * KROW + e * 8) = kreg[it];
      }
    }
  };
  auto fetch_values = [&](int k0) {
    constexpr int PER_ROW = VW / 8;
#pragma unroll
    for (int it = 0; it < PF; ++it) {
      const int idx = tid + it * 256;
      const int at = min(idx, G * SM_KT * PER_ROW - 1);
      const int e = at % PER_ROW, jj = (at / PER_ROW) % SM_KT, c = at / (PER_ROW * SM_KT);
      const int64_t row = row_of(k0 + jj);
      const uint4 x = *reinterpret_cast<const uint4*>(vc + ((row >= 0 ? row : 0) * G + c) * V + v0 + e * 8);
      vreg[it] = (row >= 0 && idx == at) ? x : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_values = [&]() {  // transposed: [dv][key]
    constexpr int PER_ROW = VW / 8;
#pragma unroll
    for (int it = 0; it < PF; ++it) {
      const int idx = tid + it * 256;
      if (idx < G * SM_KT * PER_ROW) {
        const int e = idx % PER_ROW, jj = (idx / PER_ROW) % SM_KT, c = idx / (PER_ROW * SM_KT);
        const uint32_t w[4] = {vreg[it].x, vreg[it].y, vreg[it].z, vreg[it].w};
        uint16_t* dst = reinterpret_cast<uint16_t*>(Vt) + (c * VW + e * 8) * VROW + jj;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          dst[(2 * u) * VROW] = (uint16_t)(w[u] & 0xffffu);
          dst[(2 * u + 1) * VROW] = (uint16_t)(w[u] >> 16);
        }
      }
    }
  };
  // the scores of head g against the chunk's 32 keys, in units of log 2 (so that the softmax takes
  // bare exp2 instructions): s[kt * 4 + e] is row slot * 4 + e, key 16 kt + l16; -inf where not
  // seen. The two tiles' products are issued in turn. ``inside``: every pair of the chunk is seen
  // (most chunks of a long window), so nothing is tested.
  constexpr float LOG2E = 1.4426950408889634f;
  const float scale2 = p.scale * LOG2E;
  auto scores = [&](int a, int g, int k0, bool inside, float* s) {
    const int c = g / Hg;
    sa_f32x4_t acc0 = {0.0f, 0.0f, 0.0f, 0.0f}, acc1 = {0.0f, 0.0f, 0.0f, 0.0f};
    const bf16_t* kb = Ks + (c * SM_KT + l16) * KROW + slot * 8;
#pragma unroll
    for (int ks = 0; ks < D32; ++ks) {
      acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[a][ks], sm_load8(kb + ks * 32), acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[a][ks], sm_load8(kb + 16 * KROW + ks * 32), acc1, 0, 0, 0);
    }
    // r1 * ln(1 + r2 d) in units of log 2 is r1 * log2(1 + r2 d)
    const float r1 = p.r1 ? p.r1[g] : 0.0f, r2 = p.r1 ? p.r2[g] : 0.0f;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      const int j = k0 + kt * 16 + l16;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int i = slot * 4 + e;
        const int dist = pos0 + i - j;
        float v = (kt == 0 ? acc0[e] : acc1[e]) * scale2;
        if (inside) {
          if (p.r1) v -= r1 * __builtin_amdgcn_logf(1.0f + r2 * (float)dist);
          s[kt * 4 + e] = v;
        } else {
          if (p.r1) v -= r1 * __builtin_amdgcn_logf(1.0f + r2 * (float)max(dist, 0));
          const bool seen = i < nq && dist >= 0 && (p.window <= 0 || dist < p.window);
          s[kt * 4 + e] = seen ? v : -INFINITY;
        }
      }
    }
  };
  // is every pair of (one of the run's 16 rows, one of the chunk's 32 keys) seen?
  auto all_seen = [&](int k0) {
    return nq == 16 && k0 + SM_KT - 1 <= pos0 && (p.window <= 0 || pos0 + 15 - k0 < p.window);
  };

  // ---- first walk: maxima and denominators, per lane, then across the 16 lanes of a row
  float m[HPW][4], l[HPW][4];
#pragma unroll
  for (int a = 0; a < HPW; ++a) {
    const int g = min(wave + 4 * a, H - 1);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      m[a][e] = p.sink ? p.sink[g] * LOG2E : -3.0e38f;
      l[a][e] = (p.sink && l16 == 0) ? 1.0f : 0.0f;
    }
  }
  fetch_keys(lo);
  for (int k0 = lo; k0 <= last; k0 += SM_KT) {
    __syncthreads();
    store_keys();
    if (k0 + SM_KT <= last) fetch_keys(k0 + SM_KT);
    __syncthreads();
    const bool inside = all_seen(k0);
#pragma unroll
    for (int a = 0; a < HPW; ++a) {
      const int g = wave + 4 * a;
      if (g < H) {
        float s[8];
        scores(a, g, k0, inside, s);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float mn = fmaxf(m[a][e], fmaxf(s[e], s[4 + e]));
          l[a][e] = l[a][e] * __builtin_amdgcn_exp2f(m[a][e] - mn) + __builtin_amdgcn_exp2f(s[e] - mn) +
                    __builtin_amdgcn_exp2f(s[4 + e] - mn);
          m[a][e] = mn;
        }
      }
    }
  }
#pragma unroll
  for (int a = 0; a < HPW; ++a)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
#pragma unroll
      for (int off = 8; off > 0; off >>= 1) {
        const float mo = __shfl_xor(m[a][e], off, 16), lo_ = __shfl_xor(l[a][e], off, 16);
        const float mn = fmaxf(m[a][e], mo);
        l[a][e] = l[a][e] * __builtin_amdgcn_exp2f(m[a][e] - mn) + lo_ * __builtin_amdgcn_exp2f(mo - mn);
        m[a][e] = mn;
      }
      l[a][e] = l[a][e] > 0.0f ? 1.0f / l[a][e] : 0.0f;  // from here on: 1 / denominator
    }

  // ---- second walk
  sa_f32x4_t out[HPW][NT];
#pragma unroll
  for (int a = 0; a < HPW; ++a)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) out[a][nt] = sa_f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
  fetch_keys(lo);
  fetch_values(lo);
  for (int k0 = lo; k0 <= last; k0 += SM_KT) {
    __syncthreads();
    store_keys();
    store_values();
    if (k0 + SM_KT <= last) {
      fetch_keys(k0 + SM_KT);
      fetch_values(k0 + SM_KT);
    }
    __syncthreads();
    const bool inside = all_seen(k0);
#pragma unroll
    for (int a = 0; a < HPW; ++a) {
      const int g = wave + 4 * a;
      if (g < H) {
        float s[8];
        scores(a, g, k0, inside, s);
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int e = 0; e < 4; ++e)
            Pn[(g * 16 + slot * 4 + e) * SM_PROW + kt * 16 + l16] =
                __builtin_amdgcn_exp2f(s[kt * 4 + e] - m[a][e]) * l[a][e];
      }
    }
    __syncthreads();
#pragma unroll
    for (int a = 0; a < HPW; ++a) {
      const int h = wave + 4 * a;
      if (h < H) {
        // this lane's part of the A operand: query l16, keys slot * 8 .. + 8 of the chunk
        float w[8];
        if (p.talk) {
#pragma unroll
          for (int u = 0; u < 8; ++u) w[u] = 0.0f;
          for (int g = 0; g < H; ++g) {
            const float t = Tk[h * H + g];
            const float4 x = *reinterpret_cast<const float4*>(Pn + (g * 16 + l16) * SM_PROW + slot * 8);
            const float4 y = *reinterpret_cast<const float4*>(Pn + (g * 16 + l16) * SM_PROW + slot * 8 + 4);
            w[0] += t * x.x; w[1] += t * x.y; w[2] += t * x.z; w[3] += t * x.w;
            w[4] += t * y.x; w[5] += t * y.y; w[6] += t * y.z; w[7] += t * y.w;
          }
        } else {
          const float4 x = *reinterpret_cast<const float4*>(Pn + (h * 16 + l16) * SM_PROW + slot * 8);
          const float4 y = *reinterpret_cast<const float4*>(Pn + (h * 16 + l16) * SM_PROW + slot * 8 + 4);
          w[0] = x.x; w[1] = x.y; w[2] = x.z; w[3] = x.w; w[4] = y.x; w[5] = y.y; w[6] = y.z; w[7] = y.w;
        }
        sa_bf16x8_t hi, lo8;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const __bf16 top = (__bf16)w[u];
          hi[u] = top;
          lo8[u] = (__bf16)(w[u] - (float)top);
        }
        const int c = h / Hg;
        const bf16_t* vb = Vt + (c * VW + l16) * VROW + slot * 8;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          const sa_bf16x8_t vf = sm_load8(vb + nt * 16 * VROW);
          out[a][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(hi, vf, out[a][nt], 0, 0, 0);
          out[a][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(lo8, vf, out[a][nt], 0, 0, 0);
        }
      }
    }
  }
  bf16_t* o = (bf16_t*)p.out;
#pragma unroll
  for (int a = 0; a < HPW; ++a) {
    const int h = wave + 4 * a;
    if (h < H) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int i = slot * 4 + e;
          if (i < nq) o[(row0 + i) * (int64_t)(H * V) + h * V + v0 + nt * 16 + l16] = __float2bfloat16(out[a][nt][e]);
        }
    }
  }
}

// ======================================================================================
// The same portions in ONE walk over the keys, for models of one or two key/value heads. The
// mixing across heads is linear: head h's output is
//   sum over g of talk[h, g] / denominator(g) * (unnormalised weights of head g) . V of h's key/value head,
// so a wave keeps, for each of its query heads, one accumulator per key/value head (with the
// usual running maximum), and the finished, normalised accumulators are mixed once at the end,
// through LDS. Scores are made as K Q^T: a lane then holds, for ITS query (l16), the chunk's keys
// 4 slot + e and 16 + 4 slot + e, which is the A operand of the value product as it lies in the
// registers (the value fragments are read with the keys in that order). Weights are float32 and
// fed as two bfloat16 operands, as in the kernel above.
// ======================================================================================
template <int HPW, int D32, int V16, int VS, int GC>
__global__ __launch_bounds__(256) void sink_prefill_onewalk_kernel(SinkAttnParams p) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  constexpr int D = D32 * 32, V = V16 * 16, NT = V16 / VS, VW = NT * 16;
  const int v0 = blockIdx.y * VW;
  constexpr int KROW = D + 8;
  constexpr int VROW = SM_KT + 8;
  const int H = p.heads, G = GC, Hg = H / G;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int l16 = lane & 15, slot = lane >> 4;
  const int r = p.items[4 * blockIdx.x], tok0 = p.items[4 * blockIdx.x + 1];
  const int q_len = p.cu_q[r + 1] - p.cu_q[r];
  if (tok0 >= q_len) return;
  const int nq = min(min(p.items[4 * blockIdx.x + 2], 16), q_len - tok0);
  const int pos0 = p.ctx_lens[r] - q_len + tok0;
  const int last = pos0 + nq - 1;
  const int lo = p.window > 0 ? max(0, pos0 - p.window + 1) : 0;
  const int64_t row0 = p.cu_q[r] + tok0;
  const int* table = p.block_tables + (int64_t)r * p.table_width;

  bf16_t* Ks = reinterpret_cast<bf16_t*>(smem_raw);              // [G][KT][KROW]
  bf16_t* Vt = Ks + G * SM_KT * KROW;                            // [G][VW][VROW]
  float* Ox = reinterpret_cast<float*>(smem_raw);                // at the end, over the tiles: [H][16][VW] finished outputs of one key/value head
  const int tile_bytes = (G * SM_KT * KROW + G * VW * VROW) * 2, finish_bytes = H * 16 * VW * 4;
  float* Tk = reinterpret_cast<float*>(smem_raw + max(tile_bytes, finish_bytes));  // [H][H], behind both
  int* Tb = reinterpret_cast<int*>(Tk + H * H);                  // [tb_len]

  const bf16_t* q = (const bf16_t*)p.q;
  const bf16_t* kc = (const bf16_t*)p.k_cache;
  const bf16_t* vc = (const bf16_t*)p.v_cache;
  for (int i = tid; i < H * H; i += 256) Tk[i] = p.talk ? p.talk[i] : (i / H == i % H ? 1.0f : 0.0f);
  const int tb0 = lo / p.block_size;
  for (int i = tid; i < p.tb_len; i += 256) Tb[i] = tb0 + i < p.table_width ? table[tb0 + i] : -1;
  __syncthreads();

  // query fragments as the B operand: lane = query l16, 8 elements at slot
  sa_bf16x8_t qf[HPW][D32];
  const int qi = min(l16, nq - 1);
#pragma unroll
  for (int a = 0; a < HPW; ++a) {
    const int g = min(wave + 4 * a, H - 1);
#pragma unroll
    for (int ks = 0; ks < D32; ++ks) qf[a][ks] = sm_load8(q + (row0 + qi) * p.q_stride + g * D + ks * 32 + slot * 8);
  }

  constexpr int PF = 4;
  uint4 kreg[PF], vreg[PF];
  auto row_of = [&](int j) -> int64_t {
    const int slot_ = min(max(j / p.block_size - tb0, 0), p.tb_len - 1);
    const int page = Tb[slot_];
    const int64_t row = (int64_t)page * p.block_size + j % p.block_size;
    return (j <= last && j / p.block_size - tb0 < p.tb_len && page >= 0 && row < p.cache_rows) ? row : -1;
  };
  auto fetch = [&](int k0) {
    constexpr int KPR = D / 8, VPR = VW / 8;
#pragma unroll
    for (int it = 0; it < PF; ++it) {
      const int idx = tid + it * 256;
      {
        const int at = min(idx, G * SM_KT * KPR - 1);
        const int e = at % KPR, jj = (at / KPR) % SM_KT, c = at / (KPR * SM_KT);
        const int64_t row = row_of(k0 + jj);
        const uint4 x = *reinterpret_cast<const uint4*>(kc + ((row >= 0 ? row : 0) * G + c) * D + e * 8);
        kreg[it] = (row >= 0 && idx == at) ? x : make_uint4(0, 0, 0, 0);
      }
      {
        const int at = min(idx, G * SM_KT * VPR - 1);
        const int e = at % VPR, jj = (at / VPR) % SM_KT, c = at / (VPR * SM_KT);
        const int64_t row = row_of(k0 + jj);
        const uint4 x = *reinterpret_cast<const uint4*>(vc + ((row >= 0 ? row : 0) * G + c) * V + v0 + e * 8);
        vreg[it] = (row >= 0 && idx == at) ? x : make_uint4(0, 0, 0, 0);
      }
    }
  };
  auto store = [&]() {
    constexpr int KPR = D / 8, VPR = VW / 8;
#pragma unroll
    for (int it = 0; it < PF; ++it) {
      const int idx = tid + it * 256;
      if (idx < G * SM_KT * KPR) {
        const int e = idx % KPR, jj = (idx / KPR) % SM_KT, c = idx / (KPR * SM_KT);
        *reinterpret_cast<uint4*>(Ks + (c * SM_KT + jj) * KROW + e * 8) = kreg[it];
      }
      if (idx < G * SM_KT * VPR) {
        const int e = idx % VPR, jj = (idx / VPR) % SM_KT, c = idx / (VPR * SM_KT);
        const uint32_t w[4] = {vreg[it].x, vreg[it].y, vreg[it].z, vreg[it].w};
        uint16_t* dst = reinterpret_cast<uint16_t*>(Vt) + (c * VW + e * 8) * VROW + jj;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          dst[(2 * u) * VROW] = (uint16_t)(w[u] & 0xffffu);
          dst[(2 * u + 1) * VROW] = (uint16_t)(w[u] >> 16);
        }
      }
    }
  };

  constexpr float LOG2E = 1.4426950408889634f;
  const float scale2 = p.scale * LOG2E;
  // per head: the query's running maximum (the same in the 4 lanes of a query), this lane's part
  // of its denominator, and the accumulators, one per key/value head
  float m[HPW], l[HPW];
  sa_f32x4_t out[HPW][GC][NT];
#pragma unroll
  for (int a = 0; a < HPW; ++a) {
    const int g = min(wave + 4 * a, H - 1);
    m[a] = p.sink ? p.sink[g] * LOG2E : -3.0e38f;
    l[a] = (p.sink && slot == 0) ? 1.0f : 0.0f;
#pragma unroll
    for (int c = 0; c < GC; ++c)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) out[a][c][nt] = sa_f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
  }

  fetch(lo);
  for (int k0 = lo; k0 <= last; k0 += SM_KT) {
    __syncthreads();
    store();
    if (k0 + SM_KT <= last) fetch(k0 + SM_KT);
    __syncthreads();
    const bool inside = nq == 16 && k0 + SM_KT - 1 <= pos0 && (p.window <= 0 || pos0 + 15 - k0 < p.window);
    sa_bf16x8_t ph[HPW], pl[HPW];
#pragma unroll
    for (int a = 0; a < HPW; ++a) {
      const int g = wave + 4 * a;
      if (g < H) {
        const int c = g / Hg;
        // S^T tiles: rows = keys 16 kt + 4 slot + e, column = this lane's query
        sa_f32x4_t acc0 = {0.0f, 0.0f, 0.0f, 0.0f}, acc1 = {0.0f, 0.0f, 0.0f, 0.0f};
        const bf16_t* kb = Ks + (c * SM_KT + l16) * KROW + slot * 8;
#pragma unroll
        for (int ks = 0; ks < D32; ++ks) {
          acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(sm_load8(kb + ks * 32), qf[a][ks], acc0, 0, 0, 0);
          acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(sm_load8(kb + 16 * KROW + ks * 32), qf[a][ks], acc1, 0, 0, 0);
        }
        const float r1 = p.r1 ? p.r1[g] : 0.0f, r2 = p.r1 ? p.r2[g] : 0.0f;
        float s[8];
        float top = -INFINITY;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int j = k0 + (u >> 2) * 16 + slot * 4 + (u & 3);
          const int dist = pos0 + l16 - j;
          float v = (u < 4 ? acc0[u & 3] : acc1[u & 3]) * scale2;
          if (p.r1) v -= r1 * __builtin_amdgcn_logf(1.0f + r2 * (float)max(dist, 0));
          if (!inside) {
            const bool seen = l16 < nq && dist >= 0 && (p.window <= 0 || dist < p.window);
            v = seen ? v : -INFINITY;
          }
          s[u] = v;
          top = fmaxf(top, v);
        }
        top = cw_quad_max(top);
        const float mn = fmaxf(m[a], top);
        const float alpha = __builtin_amdgcn_exp2f(m[a] - mn);
        m[a] = mn;
        float sum = 0.0f;
        float w[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          w[u] = __builtin_amdgcn_exp2f(s[u] - mn);
          sum += w[u];
        }
        l[a] = l[a] * alpha + sum;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const __bf16 t = (__bf16)w[u];
          ph[a][u] = t;
          pl[a][u] = (__bf16)(w[u] - (float)t);
        }
        // the accumulators' rows are queries slot * 4 + e: each takes its own query's factor
        if (__ballot(alpha != 1.0f) != 0) {
          float ar[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) ar[e] = __shfl(alpha, slot * 4 + e, 64);
#pragma unroll
          for (int cc = 0; cc < GC; ++cc)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
              for (int e = 0; e < 4; ++e) out[a][cc][nt][e] *= ar[e];
        }
      }
    }
    // values: a fragment (one key/value head, 16 value columns) serves all of the wave's heads
#pragma unroll
    for (int cc = 0; cc < GC; ++cc) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        // column l16 of the tile, keys 4 slot .. + 4 and 16 + 4 slot .. + 4: the order the weights lie in
        const bf16_t* vb = Vt + (cc * VW + nt * 16 + l16) * VROW + slot * 4;
        const uint2 lo4 = *reinterpret_cast<const uint2*>(vb), hi4 = *reinterpret_cast<const uint2*>(vb + 16);
        const uint4 both = make_uint4(lo4.x, lo4.y, hi4.x, hi4.y);
        const sa_bf16x8_t vf = *reinterpret_cast<const sa_bf16x8_t*>(&both);
#pragma unroll
        for (int a = 0; a < HPW; ++a) {
          if (wave + 4 * a < H) {
            out[a][cc][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ph[a], vf, out[a][cc][nt], 0, 0, 0);
            out[a][cc][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pl[a], vf, out[a][cc][nt], 0, 0, 0);
          }
        }
      }
    }
  }

  // ---- finish: denominators, then the mixing across heads, one key/value head at a time through LDS
  float inv_row[HPW][4];
#pragma unroll
  for (int a = 0; a < HPW; ++a) {
    const float total = cw_quad_sum(l[a]);
    const float inv = total > 0.0f ? 1.0f / total : 0.0f;
#pragma unroll
    for (int e = 0; e < 4; ++e) inv_row[a][e] = __shfl(inv, slot * 4 + e, 64);
  }
  bf16_t* o = (bf16_t*)p.out;
  for (int cc = 0; cc < GC; ++cc) {
    __syncthreads();  // the tiles (and the round before) are done with LDS
#pragma unroll
    for (int a = 0; a < HPW; ++a) {
      const int g = wave + 4 * a;
      if (g < H) {
#pragma unroll
        for (int c2 = 0; c2 < GC; ++c2) {
          if (c2 == cc) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
              for (int e = 0; e < 4; ++e)
                Ox[(g * 16 + slot * 4 + e) * VW + nt * 16 + l16] = out[a][c2][nt][e] * inv_row[a][e];
          }
        }
      }
    }
    __syncthreads();
    // heads of this key/value head: h = cc * Hg .. ; every thread takes outputs (h, query, column)
    const int n_out = Hg * 16 * VW;
    for (int idx = tid; idx < n_out; idx += 256) {
      const int col = idx % VW, i = (idx / VW) % 16, h = cc * Hg + idx / (VW * 16);
      float v = 0.0f;
      for (int g = 0; g < H; ++g) v += Tk[h * H + g] * Ox[(g * 16 + i) * VW + col];
      if (i < nq) o[(row0 + i) * (int64_t)(H * V) + h * V + v0 + col] = __float2bfloat16(v);
    }
  }
}

static int64_t sink_prefill_mfma_lds_bytes(int H, int G, int D, int V) {  // V: the value columns of one workgroup
  return (int64_t)G * SM_KT * (D + 8) * 2 + (int64_t)G * V * (SM_KT + 8) * 2 + (int64_t)H * 16 * SM_PROW * 4 + (int64_t)H * H * 4;
}
#define SM_MAX_TABLE 4096  // entries of the block table a workgroup keeps in LDS at most

// The geometries this kernel is built for: dim 64 or 128, vdim 64 or 128, up to 16 heads
// (4 a wave), and what of LDS they need.
CW_EXPORT int cw_sink_prefill_mfma_supported(int heads, int kv_heads, int dim, int vdim) {
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || heads > 16) return 0;
  if ((dim != 64 && dim != 128) || (vdim != 64 && vdim != 128)) return 0;
  // a thread moves up to four 16-byte pieces of a chunk's keys, and of its values
  if (kv_heads * SM_KT * (dim / 8) > 4 * 256 || kv_heads * SM_KT * (vdim / 8) > 4 * 256) return 0;
  return sink_prefill_mfma_lds_bytes(heads, kv_heads, dim, vdim) + SM_MAX_TABLE * 4 <= 150 * 1024 ? 1 : 0;
}

static int64_t sink_prefill_onewalk_lds_bytes(int H, int G, int D, int VW) {  // without the pages' table
  const int64_t tiles = (int64_t)G * SM_KT * (D + 8) * 2 + (int64_t)G * VW * (SM_KT + 8) * 2;
  const int64_t finish = (int64_t)H * 16 * VW * 4;   // laid over the tiles; the mixing matrix and the pages lie behind both
  return (tiles > finish ? tiles : finish) + (int64_t)H * H * 4;
}

// items: runs of up to 16 tokens. bfloat16 only. A launch of fewer than v_split_below runs gives
// every run two workgroups (the caller passes the number of compute units).
CW_EXPORT int cw_sink_prefill_mfma(const void* q, int64_t q_stride, void* out, const void* k_cache, const void* v_cache,
                                   int64_t cache_rows, const int* block_tables, int table_width, const int* ctx_lens,
                                   const int* cu_q, const int* items, int n_items, const float* r1, const float* r2,
                                   const float* sink, const float* talk, int heads, int kv_heads, int dim, int vdim,
                                   int block_size, int window, float scale, int v_split_below, hipStream_t stream) {
  if (n_items < 0 || !q || !out || !k_cache || !v_cache || !block_tables || !ctx_lens || !cu_q || !items) return CW_ERR_ARG;
  if (block_size <= 0 || table_width <= 0 || window < 0 || (r1 && !r2)) return CW_ERR_ARG;
  if (!cw_sink_prefill_mfma_supported(heads, kv_heads, dim, vdim)) return CW_ERR_SIZE;
  if (((uintptr_t)q & 15) || ((uintptr_t)k_cache & 15) || ((uintptr_t)v_cache & 15) || (q_stride % 8)) return CW_ERR_ARG;
  if (n_items == 0) return CW_OK;
  SinkAttnParams p;
  p.q = q; p.q_stride = q_stride; p.out = out; p.k_cache = k_cache; p.v_cache = v_cache;
  p.block_tables = block_tables; p.table_width = table_width; p.ctx_lens = ctx_lens; p.cu_q = cu_q; p.items = items;
  p.r1 = r1; p.r2 = r2; p.sink = sink; p.talk = talk;
  p.heads = heads; p.kv_heads = kv_heads; p.dim = dim; p.vdim = vdim; p.block_size = block_size; p.window = window;
  p.scale = scale; p.bq = 16; p.cache_rows = cache_rows;
  // few runs: two workgroups a run, each with half of the value columns
  const int vs = n_items < v_split_below ? 2 : 1;
  // the pages a run of 16 tokens can see: its window and itself, or the whole table
  int64_t tb_len = window > 0 ? (int64_t)(window + 16) / block_size + 2 : table_width;
  if (tb_len > table_width) tb_len = table_width;
  if (tb_len > SM_MAX_TABLE) return CW_ERR_SIZE;
  p.tb_len = (int)tb_len;
  const dim3 grid(n_items, vs), block(256);
  const int hpw = (heads + 3) / 4;
  // one or two key/value heads: the kernel that walks the keys once (two workgroups a run always:
  // its accumulators for all value columns would not fit the registers)
  if (kv_heads <= 2 && sink_prefill_onewalk_lds_bytes(heads, kv_heads, dim, vdim / 2) + tb_len * 4 <= 150 * 1024) {
    const size_t smem1 = (size_t)sink_prefill_onewalk_lds_bytes(heads, kv_heads, dim, vdim / 2) + (size_t)tb_len * 4;
    const dim3 grid1(n_items, 2);
#define CW_ONE(HPW_, D32_, V16_, GC_)                                                                                 \
  do {                                                                                                                \
    if (smem1 > 48 * 1024 && hipFuncSetAttribute((const void*)sink_prefill_onewalk_kernel<HPW_, D32_, V16_, 2, GC_>,  \
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem1) != hipSuccess) \
      return CW_ERR_LAUNCH;                                                                                           \
    hipLaunchKernelGGL((sink_prefill_onewalk_kernel<HPW_, D32_, V16_, 2, GC_>), grid1, block, smem1, stream, p);      \
  } while (0)
#define CW_ONE_HEADS(D32_, V16_, GC_)              \
  do {                                             \
    if (hpw <= 1) CW_ONE(1, D32_, V16_, GC_);      \
    else if (hpw == 2) CW_ONE(2, D32_, V16_, GC_); \
    else if (hpw == 3) CW_ONE(3, D32_, V16_, GC_); \
    else CW_ONE(4, D32_, V16_, GC_);               \
  } while (0)
#define CW_ONE_SIZES(GC_)                                        \
  do {                                                           \
    if (dim == 64 && vdim == 64) CW_ONE_HEADS(2, 4, GC_);        \
    else if (dim == 64 && vdim == 128) CW_ONE_HEADS(2, 8, GC_);  \
    else if (dim == 128 && vdim == 64) CW_ONE_HEADS(4, 4, GC_);  \
    else CW_ONE_HEADS(4, 8, GC_);                                \
  } while (0)
    if (kv_heads == 1) CW_ONE_SIZES(1);
    else CW_ONE_SIZES(2);
#undef CW_ONE_SIZES
#undef CW_ONE_HEADS
#undef CW_ONE
    return cw_launch_status();
  }
  const size_t smem = (size_t)sink_prefill_mfma_lds_bytes(heads, kv_heads, dim, vdim / vs) + (size_t)tb_len * 4;
#define CW_LAUNCH_VS(HPW_, D32_, V16_, VS_)                                                                           \
  do {                                                                                                                \
    if (smem > 48 * 1024 && hipFuncSetAttribute((const void*)sink_prefill_mfma_kernel<HPW_, D32_, V16_, VS_>,         \
                                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) \
      return CW_ERR_LAUNCH;                                                                                           \
    hipLaunchKernelGGL((sink_prefill_mfma_kernel<HPW_, D32_, V16_, VS_>), grid, block, smem, stream, p);              \
  } while (0)
#define CW_LAUNCH(HPW_, D32_, V16_)                 \
  do {                                              \
    if (vs == 2) CW_LAUNCH_VS(HPW_, D32_, V16_, 2); \
    else CW_LAUNCH_VS(HPW_, D32_, V16_, 1);         \
  } while (0)
#define CW_BY_HEADS(D32_, V16_)                \
  do {                                         \
    if (hpw <= 1) CW_LAUNCH(1, D32_, V16_);    \
    else if (hpw == 2) CW_LAUNCH(2, D32_, V16_); \
    else if (hpw == 3) CW_LAUNCH(3, D32_, V16_); \
    else CW_LAUNCH(4, D32_, V16_);             \
  } while (0)
  if (dim == 64 && vdim == 64) CW_BY_HEADS(2, 4);
  else if (dim == 64 && vdim == 128) CW_BY_HEADS(2, 8);
  else if (dim == 128 && vdim == 64) CW_BY_HEADS(4, 4);
  else CW_BY_HEADS(4, 8);
#undef CW_BY_HEADS
#undef CW_LAUNCH
#undef CW_LAUNCH_VS
  return cw_launch_status();
}
