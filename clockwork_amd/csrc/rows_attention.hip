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
//             its own segment).
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
};

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

  for (int k0 = first; k0 <= last; k0 += KC) {
    __syncthreads();  // the tile of the round before has been read (and the queries are written)
    const int width = M * D;
    for (int i = tid; i < KC * width; i += 256) {
      const int j = i / width, d = i % width;
      const int key = k0 + j;
      float v = 0.0f;
      if (key <= last) {
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
        if (key <= last) {
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
        if (live && key >= lo && key <= pos) {
          s[i] = dot * p.scale;
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
                                hipStream_t stream) {
  if (n_items < 0 || !q || !out || !k_plane || !v_plane || !block_tables || !ctx_lens || !cu_q || !items)
    return CW_ERR_ARG;
  if (block_size <= 0 || table_width <= 0 || mask_kind < 0 || mask_kind > 2 || (mask_kind != 0 && mask_size < 1))
    return CW_ERR_ARG;
  if (maps == 2 && !lambda) return CW_ERR_ARG;
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
