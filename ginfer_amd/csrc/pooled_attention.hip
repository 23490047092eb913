// Attention over a sliding window and, before the window, over the means of whole blocks of tokens, with a sigmoid in
// place of the softmax:
//   token i sees the tokens j with 0 <= i - j < size, and for every block b of `pool` tokens whose last token lies before
//   them (b pool + pool - 1 <= i - size) one key and one value, the means of the block's cached keys and values;
//   out[i, h] = sum over what i sees of sigmoid(scale q_i,h . k + bias_h) v          (no normalisation over keys)
// Keys and values live in pages, a token a row: [slot][kv head][dim] and [slot][kv head][vdim], in the cache's number
// format; the blocks' means live in pages of their own, a block a row, in 32-bit.
//
// prepare: behind the q | k | v | ... projection (32-bit rows): q and k are turned by position on their first rot_dims
//   coordinates (coordinate 2i pairs with 2i + 1; tables cos, sin float [positions, rot_dims / 2]), then each head's q and k
//   is divided by its root mean square (where `unit` says so); q goes out in 32-bit, k and v into their rows.
// pool: for every token of the step that ends a block, the means of the block's keys and values, added up in the order
//   of the positions, into the block's row.
// attend: a wavefront per (token, head); 64 keys at a time, a lane a key for the scores (one chain of multiply-adds over
//   the coordinates), then a lane a value column, the keys' weights added in the order of the keys: blocks first, then
//   tokens, each ascending.  The sums do not depend on how a request was cut into steps or on what else is in the batch.
//   The result is multiplied by sigmoid(gate) where a gate is given (32-bit rows with a stride).
#include "common.h"
#include "ginfer_amd.h"

#define PA_THREADS 64

__device__ __forceinline__ float pa_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }

// one wavefront per (token, unit): units 0 .. nh - 1 are the query heads, then nkv key heads, then nkv value heads
template <typename TC>
__global__ __launch_bounds__(PA_THREADS) void pwa_prepare_kernel(float* __restrict__ q_out, const float* __restrict__ proj,
                                                                 int64_t stride, const int32_t* __restrict__ positions,
                                                                 const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                                 const int64_t* __restrict__ slot_mapping, TC* __restrict__ k_rows,
                                                                 TC* __restrict__ v_rows, int nh, int nkv, int dim, int vdim,
                                                                 int rot_dims, int unit, float eps, int write) {
  const int64_t t = blockIdx.x;
  const int u = blockIdx.y, lane = threadIdx.x;
  const float* row = proj + t * stride;
  if (u >= nh + nkv) {                         // a value head: copied into its row
    if (!write) return;
    const int64_t slot = slot_mapping[t];
    if (slot < 0) return;
    const int g = u - nh - nkv;
    const float* src = row + (int64_t)(nh + nkv) * dim + (int64_t)g * vdim;
    TC* dst = v_rows + (slot * nkv + g) * (int64_t)vdim;
    for (int i = lane; i < vdim; i += PA_THREADS) Num<TC>::st(dst + i, src[i]);
    return;
  }
  const bool is_q = u < nh;
  const float* src = row + (int64_t)u * dim;   // q heads and k heads follow each other in the projection
  int64_t slot = -1;
  if (!is_q) {
    if (!write) return;
    slot = slot_mapping[t];
    if (slot < 0) return;
  }
  const int half = rot_dims / 2;
  const int64_t at = (int64_t)positions[t] * half;
  float ss = 0.f;
  // a lane keeps every 64th coordinate; heads of up to 256 coordinates
  float x[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int i = lane + r * PA_THREADS;
    float v = 0.f;
    if (i < dim) {
      v = src[i];
      if (i < rot_dims) {
        const float c = cos_t[at + (i >> 1)], sn = sin_t[at + (i >> 1)];
        const float o = src[i ^ 1];
        // the pair (even, odd) becomes (even c - odd s, odd c + even s)
        v = (i & 1) ? v * c + o * sn : v * c - o * sn;
      }
    }
    x[r] = v;
    ss += v * v;
  }
  float inv = 1.0f;
  if (unit) {
    ss = wave_sum(ss);
    inv = 1.0f / sqrtf(ss / (float)dim + eps);
  }
  if (is_q) {
    float* dst = q_out + (t * nh + u) * (int64_t)dim;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i = lane + r * PA_THREADS;
      if (i < dim) dst[i] = x[r] * inv;
    }
  } else {
    TC* dst = k_rows + (slot * nkv + (u - nh)) * (int64_t)dim;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i = lane + r * PA_THREADS;
      if (i < dim) Num<TC>::st(dst + i, x[r] * inv);
    }
  }
}

// the row of position p of entry e in a paged tensor, or -1 where the table has no page
__device__ __forceinline__ int64_t pa_row(const int32_t* __restrict__ table, int width, int e, int p, int page_size) {
  const int b = p / page_size;
  if (b >= width) return -1;
  const int page = table[(int64_t)e * width + b];
  return page < 0 ? -1 : (int64_t)page * page_size + (p - b * page_size);
}

// grid (tokens, 2 nkv): the keys' and the values' heads of the block that a token ends
template <typename TC>
__global__ __launch_bounds__(PA_THREADS) void pwa_pool_kernel(float* __restrict__ pk_rows, float* __restrict__ pv_rows,
                                                              const TC* __restrict__ k_rows, const TC* __restrict__ v_rows,
                                                              const int32_t* __restrict__ positions,
                                                              const int32_t* __restrict__ token_entry,
                                                              const int32_t* __restrict__ table, int width,
                                                              const int64_t* __restrict__ pool_slots, int nkv, int dim, int vdim,
                                                              int pool, int page_size) {
  const int64_t t = blockIdx.x;
  const int pos = positions[t];
  if ((pos + 1) % pool) return;
  const int64_t dst_row = pool_slots[t];
  if (dst_row < 0) return;
  const int e = token_entry[t];
  const bool keys = blockIdx.y < (unsigned)nkv;
  const int g = keys ? blockIdx.y : blockIdx.y - nkv, w = keys ? dim : vdim;
  const TC* src = keys ? k_rows : v_rows;
  float* dst = (keys ? pk_rows : pv_rows) + (dst_row * nkv + g) * (int64_t)w;
  const float inv = 1.0f / (float)pool;
  for (int c = threadIdx.x; c < w; c += PA_THREADS) {
    float sum = 0.f;
    for (int p = pos + 1 - pool; p <= pos; ++p) {
      const int64_t r = pa_row(table, width, e, p, page_size);
      if (r >= 0) sum += Num<TC>::ld(src + (r * nkv + g) * (int64_t)w + c);
    }
    dst[c] = sum * inv;
  }
}

// one wavefront per (token, head)
template <typename TC, typename TO>
__global__ __launch_bounds__(PA_THREADS) void pwa_attend_kernel(TO* __restrict__ out, const float* __restrict__ q,
                                                                const TC* __restrict__ k_rows, const TC* __restrict__ v_rows,
                                                                const float* __restrict__ pk_rows, const float* __restrict__ pv_rows,
                                                                const int32_t* __restrict__ positions,
                                                                const int32_t* __restrict__ token_entry,
                                                                const int32_t* __restrict__ table, int width,
                                                                const int32_t* __restrict__ pool_table, int pool_width,
                                                                const float* __restrict__ head_bias, const float* __restrict__ gate,
                                                                int64_t gate_stride, int nh, int nkv, int dim, int vdim,
                                                                int size, int pool, int page_size, float scale) {
  __shared__ float qs[256];
  __shared__ float ws[PA_THREADS];
  __shared__ int64_t rows[PA_THREADS];
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const int g = h / (nh / nkv);
  const int e = token_entry[t], i = positions[t];
  for (int d = lane; d < dim; d += PA_THREADS) qs[d] = q[(t * nh + h) * (int64_t)dim + d];
  const int lo = i - size + 1 > 0 ? i - size + 1 : 0;       // the first token of the window
  const int nb = pool > 0 ? lo / pool : 0;                  // blocks that end before the window
  const int n = nb + (i - lo + 1);
  const float bias = head_bias ? head_bias[h] : 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  __syncthreads();
  for (int x0 = 0; x0 < n; x0 += PA_THREADS) {
    const int cnt = n - x0 < PA_THREADS ? n - x0 : PA_THREADS;
    const int nblk = nb - x0 > 0 ? (nb - x0 < cnt ? nb - x0 : cnt) : 0;   // of this tile's keys, the first nblk are blocks
    const int x = x0 + lane;
    float w = 0.f;
    int64_t r = -1;
    if (x < n) {
      float s = 0.f;
      if (x < nb) {
        r = pa_row(pool_table, pool_width, e, x, page_size);
        if (r >= 0) {
          const float* kp = pk_rows + (r * nkv + g) * (int64_t)dim;
          for (int d = 0; d < dim; ++d) s = fmaf(qs[d], kp[d], s);
        }
      } else {
        r = pa_row(table, width, e, lo + (x - nb), page_size);
        if (r >= 0) {
          const TC* kp = k_rows + (r * nkv + g) * (int64_t)dim;
          for (int d = 0; d < dim; ++d) s = fmaf(qs[d], Num<TC>::ld(kp + d), s);
        }
      }
      w = r >= 0 ? pa_sigmoid(s * scale + bias) : 0.f;
    }
    __syncthreads();                                  // the tile before is read out
    ws[lane] = w;
    rows[lane] = r;
    __syncthreads();
#pragma unroll
    for (int c4 = 0; c4 < 4; ++c4) {
      const int c = lane + c4 * PA_THREADS;
      if (c < vdim) {
        float a = acc[c4];
        for (int l = 0; l < nblk; ++l)
          if (rows[l] >= 0) a = fmaf(ws[l], pv_rows[(rows[l] * nkv + g) * (int64_t)vdim + c], a);
        for (int l = nblk; l < cnt; ++l)
          if (rows[l] >= 0) a = fmaf(ws[l], Num<TC>::ld(v_rows + (rows[l] * nkv + g) * (int64_t)vdim + c), a);
        acc[c4] = a;
      }
    }
  }
#pragma unroll
  for (int c4 = 0; c4 < 4; ++c4) {
    const int c = lane + c4 * PA_THREADS;
    if (c < vdim) {
      float a = acc[c4];
      if (gate) a *= pa_sigmoid(gate[t * gate_stride + (int64_t)h * vdim + c]);
      Num<TO>::st(out + (t * nh + h) * (int64_t)vdim + c, a);
    }
  }
}

extern "C" int ga_pwa_prepare(void* q_out, const void* proj, int64_t stride, const void* positions, const void* cos_t,
                              const void* sin_t, const void* slot_mapping, void* k_rows, void* v_rows, int tokens, int nh,
                              int nkv, int dim, int vdim, int rot_dims, int unit, float eps, int write, int cache_bf16,
                              hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (nh <= 0 || nkv <= 0 || dim <= 0 || dim > 256 || vdim <= 0 || nh + 2 * nkv > 65535) return -1;
  if (rot_dims < 0 || rot_dims % 2 || rot_dims > dim || (rot_dims > 0 && (!cos_t || !sin_t))) return -2;
  dim3 grid(tokens, nh + 2 * nkv), block(PA_THREADS);
#define GO(T) hipLaunchKernelGGL(pwa_prepare_kernel<T>, grid, block, 0, stream, (float*)q_out, (const float*)proj, stride, \
                                 (const int32_t*)positions, (const float*)cos_t, (const float*)sin_t,                      \
                                 (const int64_t*)slot_mapping, (T*)k_rows, (T*)v_rows, nh, nkv, dim, vdim, rot_dims, unit, \
                                 eps, write)
  if (cache_bf16) GO(bf16_t); else GO(float);
#undef GO
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_pwa_pool(void* pk_rows, void* pv_rows, const void* k_rows, const void* v_rows, const void* positions,
                           const void* token_entry, const void* table, int width, const void* pool_slots, int tokens,
                           int nkv, int dim, int vdim, int pool, int page_size, int cache_bf16, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (nkv <= 0 || 2 * nkv > 65535 || dim <= 0 || vdim <= 0 || pool <= 0 || page_size <= 0 || width <= 0) return -1;
  dim3 grid(tokens, 2 * nkv), block(PA_THREADS);
#define GO(T) hipLaunchKernelGGL(pwa_pool_kernel<T>, grid, block, 0, stream, (float*)pk_rows, (float*)pv_rows,            \
                                 (const T*)k_rows, (const T*)v_rows, (const int32_t*)positions, (const int32_t*)token_entry, \
                                 (const int32_t*)table, width, (const int64_t*)pool_slots, nkv, dim, vdim, pool, page_size)
  if (cache_bf16) GO(bf16_t); else GO(float);
#undef GO
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_pwa_attend(void* out, const void* q, const void* k_rows, const void* v_rows, const void* pk_rows,
                             const void* pv_rows, const void* positions, const void* token_entry, const void* table,
                             int width, const void* pool_table, int pool_width, const void* head_bias, const void* gate,
                             int64_t gate_stride, int tokens, int nh, int nkv, int dim, int vdim, int size, int pool,
                             int page_size, float scale, int cache_bf16, int out_bf16, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (nh <= 0 || nkv <= 0 || nh % nkv || nh > 65535 || dim <= 0 || dim > 256 || vdim <= 0 || vdim > 256) return -1;
  if (size <= 0 || pool <= 0 || page_size <= 0 || width <= 0 || pool_width <= 0) return -2;
  dim3 grid(tokens, nh), block(PA_THREADS);
#define GO(T, O) hipLaunchKernelGGL((pwa_attend_kernel<T, O>), grid, block, 0, stream, (O*)out, (const float*)q,           \
                                    (const T*)k_rows, (const T*)v_rows, (const float*)pk_rows, (const float*)pv_rows,     \
                                    (const int32_t*)positions, (const int32_t*)token_entry, (const int32_t*)table, width, \
                                    (const int32_t*)pool_table, pool_width, (const float*)head_bias, (const float*)gate,  \
                                    gate_stride, nh, nkv, dim, vdim, size, pool, page_size, scale)
  if (cache_bf16) { if (out_bf16) GO(bf16_t, bf16_t); else GO(bf16_t, float); }
  else { if (out_bf16) GO(float, bf16_t); else GO(float, float); }
#undef GO
  return GA_CHECK_LAUNCH();
}
