// Attention over a sliding window and, before the window, over the means of whole blocks of tokens, with a sigmoid in
// place of the softmax:
//   token i sees the tokens j with 0 <= i - j < size, and for every block b of `pool` tokens whose last token lies before
//   them (b pool + pool - 1 <= i - size) one key and one value, the means of the block's cached keys and values;
//   out[i, h] = sum over what i sees of sigmoid(scale q_i,h . k + bias_h) v          (no normalisation over keys)
// Keys live in pages, a token a row: [page][slot][kv head][dim]; values transposed inside a page: [page][kv head][vdim][slot]
// (eight consecutive tokens of a value column are 16 bytes, an operand of the matrix cores), in the cache's number format; the
// blocks' means live in pages of their own, laid out alike with a block for a token, in 32-bit.
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

// where column c of kv head g of row `row` (page * page_size + place) lies in pages of transposed values
__device__ __forceinline__ int64_t pa_value_at(int64_t row, int g, int c, int nkv, int vdim, int page_size) {
  const int64_t page = row / page_size;
  return ((page * nkv + g) * (int64_t)vdim + c) * page_size + (row - page * page_size);
}

// one wavefront per (token, unit): units 0 .. nh - 1 are the query heads, then nkv key heads, then nkv value heads
template <typename TC>
__global__ __launch_bounds__(PA_THREADS) void pwa_prepare_kernel(float* __restrict__ q_out, const float* __restrict__ proj,
                                                                 int64_t stride, const int32_t* __restrict__ positions,
                                                                 const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                                 const int64_t* __restrict__ slot_mapping, TC* __restrict__ k_rows,
                                                                 TC* __restrict__ v_rows, int nh, int nkv, int dim, int vdim,
                                                                 int rot_dims, int unit, float eps, int write, int page_size) {
  const int64_t t = blockIdx.x;
  const int u = blockIdx.y, lane = threadIdx.x;
  const float* row = proj + t * stride;
  if (u >= nh + nkv) {                         // a value head: copied into its row
    if (!write) return;
    const int64_t slot = slot_mapping[t];
    if (slot < 0) return;
    const int g = u - nh - nkv;
    const float* src = row + (int64_t)(nh + nkv) * dim + (int64_t)g * vdim;
    for (int i = lane; i < vdim; i += PA_THREADS) Num<TC>::st(v_rows + pa_value_at(slot, g, i, nkv, vdim, page_size), src[i]);
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

// The mean over the block that ends at `pos` of one channel: eight rows are asked for at a time, without a branch in
// between (a row that is not there is read at row 0 and left out), and added in the order of the positions.
template <bool KEYS, typename TC>
__device__ __forceinline__ float pa_block_mean(const TC* __restrict__ rows, const int32_t* __restrict__ bt, int width, int pos,
                                               int pool, int page_size, int nkv, int g, int w, int c) {
  float sum = 0.f;
  for (int p0 = pos + 1 - pool; p0 <= pos; p0 += 8) {
    int page[8], at[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int p = p0 + j <= pos ? p0 + j : pos;
      const int b = p / page_size;
      at[j] = p - b * page_size;
      page[j] = bt[b < width ? b : width - 1];
      if (b >= width || p0 + j > pos) page[j] = -1;
    }
    float x[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int64_t pg = page[j] < 0 ? 0 : page[j];
      x[j] = KEYS ? Num<TC>::ld(rows + ((pg * page_size + at[j]) * nkv + g) * (int64_t)w + c)
                  : Num<TC>::ld(rows + ((pg * nkv + g) * (int64_t)w + c) * page_size + at[j]);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (page[j] >= 0) sum += x[j];
  }
  return sum / (float)pool;
}

// grid (tokens, 2 nkv): the keys' and the values' heads of the block that a token ends
template <typename TC>
__global__ __launch_bounds__(256) void pwa_pool_kernel(float* __restrict__ pk_rows, float* __restrict__ pv_rows,
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
  const int32_t* bt = table + (int64_t)token_entry[t] * width;
  if (blockIdx.y < (unsigned)nkv) {
    const int g = blockIdx.y;
    for (int c = threadIdx.x; c < dim; c += blockDim.x)
      pk_rows[(dst_row * nkv + g) * (int64_t)dim + c] = pa_block_mean<true, TC>(k_rows, bt, width, pos, pool, page_size, nkv, g, dim, c);
  } else {
    const int g = blockIdx.y - nkv;
    for (int c = threadIdx.x; c < vdim; c += blockDim.x)
      pv_rows[pa_value_at(dst_row, g, c, nkv, vdim, page_size)] =
          pa_block_mean<false, TC>(v_rows, bt, width, pos, pool, page_size, nkv, g, vdim, c);
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
          if (rows[l] >= 0) a = fmaf(ws[l], pv_rows[pa_value_at(rows[l], g, c, nkv, vdim, page_size)], a);
        for (int l = nblk; l < cnt; ++l)
          if (rows[l] >= 0) a = fmaf(ws[l], Num<TC>::ld(v_rows + pa_value_at(rows[l], g, c, nkv, vdim, page_size)), a);
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
                              int nkv, int dim, int vdim, int rot_dims, int unit, float eps, int write, int page_size, int cache_bf16,
                              hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (page_size <= 0) return -3;
  if (nh <= 0 || nkv <= 0 || dim <= 0 || dim > 256 || vdim <= 0 || nh + 2 * nkv > 65535) return -1;
  if (rot_dims < 0 || rot_dims % 2 || rot_dims > dim || (rot_dims > 0 && (!cos_t || !sin_t))) return -2;
  dim3 grid(tokens, nh + 2 * nkv), block(PA_THREADS);
#define GO(T) hipLaunchKernelGGL(pwa_prepare_kernel<T>, grid, block, 0, stream, (float*)q_out, (const float*)proj, stride, \
                                 (const int32_t*)positions, (const float*)cos_t, (const float*)sin_t,                      \
                                 (const int64_t*)slot_mapping, (T*)k_rows, (T*)v_rows, nh, nkv, dim, vdim, rot_dims, unit, \
                                 eps, write, page_size)
  if (cache_bf16) GO(bf16_t); else GO(float);
#undef GO
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_pwa_pool(void* pk_rows, void* pv_rows, const void* k_rows, const void* v_rows, const void* positions,
                           const void* token_entry, const void* table, int width, const void* pool_slots, int tokens,
                           int nkv, int dim, int vdim, int pool, int page_size, int cache_bf16, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (nkv <= 0 || 2 * nkv > 65535 || dim <= 0 || vdim <= 0 || pool <= 0 || page_size <= 0 || width <= 0) return -1;
  const int widest = dim > vdim ? dim : vdim;          // a thread a channel: the chains of a block's sum run side by side
  dim3 grid(tokens, 2 * nkv), block(widest <= 64 ? 64 : widest <= 128 ? 128 : 256);
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

// ---------------------------------------------------------------------------------------------------- matrix cores
// bfloat16 on v_mfma_f32_16x16x32_bf16 (D[m][n] += sum_k A[m][k] B[n][k]; lane l supplies row l % 16 and k-slots
// (l / 16) * 8 .. + 7 of both operands and receives D[(l / 16) * 4 + i][l % 16]).  The 16 columns n of a wavefront are 16
// (token, head) pairs that read the same request's pages and the same kv head:
//   rows   16 neighbouring tokens of a prompt portion for one head (the step's plan of tiles); a workgroup's 4 wavefronts
//          take 4 neighbouring heads.
//   heads  the heads of one kv group of one single token (at most 16); the token's tiles of keys are dealt to `splits`
//          workgroups, whose partial sums (there is no denominator: they simply add) a second kernel adds in order.
//   S^T = K Q^T    A = 16 keys x 32 coordinates, 16 bytes per lane from the key's row; row m of product t holds key
//                  8 (m / 4) + 4 t + m % 4 of the tile of 32, so a lane ends up with the scores of the 8 consecutive keys
//                  8 (l / 16) .. + 7 of its column, which is the k-slot layout of operand B for the weights:
//   O^T += V^T P^T A = 16 value columns x 8 consecutive keys from the transposed page, 16 bytes per lane.
// Tiles of 32 keys at absolute multiples of 32, first over the blocks' means (32-bit in memory, rounded to bfloat16 on the
// way into the operand), then over the tokens; keys a column does not see get the weight 0.  Weights in 32-bit.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

__device__ __forceinline__ bf16x8 pm_zero8() { return __builtin_bit_cast(bf16x8, make_uint4(0u, 0u, 0u, 0u)); }
__device__ __forceinline__ bf16x8 pm_pack8(const float* v) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = (uint32_t)f32_to_bf16(v[2 * i]) | ((uint32_t)f32_to_bf16(v[2 * i + 1]) << 16);
  return __builtin_bit_cast(bf16x8, make_uint4(w[0], w[1], w[2], w[3]));
}
__device__ __forceinline__ bf16x8 pm_load8(const bf16_t* p) { return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p)); }
__device__ __forceinline__ bf16x8 pm_load8(const float* p) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
  return pm_pack8(v);
}
__device__ __forceinline__ int pm_wave_min(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = min(v, __shfl_xor(v, o, WAVE));
  return v;
}
__device__ __forceinline__ int pm_wave_max(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = max(v, __shfl_xor(v, o, WAVE));
  return v;
}

// The walk over the tiles of keys [lo_min, hi_max] (every `step`-th tile from tile `first` on) for one set of 16 columns.
// qb: the columns' queries as B operands; [lo_c, hi_c]: the keys the lane's column sees (hi_c < lo_c: none); bt: the entry's
// block table over rows of TS (the tokens', or the blocks' means).  c = lane % 16, gq = lane / 16.
template <int DB, int VB, typename TS>
__device__ __forceinline__ void pm_walk(f32x4 (&acc)[VB], const bf16x8 (&qb)[DB], const TS* __restrict__ k_rows,
                                        const TS* __restrict__ v_pages, const int32_t* __restrict__ bt, int width, int nkv, int g,
                                        int dim, int vdim, int ps, int lo_c, int hi_c, int lo_min, int hi_max, int first, int step,
                                        float scale, float bias, int c, int gq) {
  for (int k0 = (lo_min & ~31) + 32 * first; k0 <= hi_max; k0 += 32 * step) {
    f32x4 s[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
    const TS* rowp[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int kp = k0 + 8 * (c >> 2) + 4 * t + (c & 3);
      rowp[t] = nullptr;
      if (kp >= lo_min && kp <= hi_max) {
        const int b = kp / ps;
        const int page = b < width ? bt[b] : -1;
        if (page >= 0) rowp[t] = k_rows + (((int64_t)page * ps + (kp - b * ps)) * nkv + g) * (int64_t)dim + 8 * gq;
      }
    }
    bf16x8 a[DB][2];
#pragma unroll
    for (int u = 0; u < DB; ++u)
#pragma unroll
      for (int t = 0; t < 2; ++t) a[u][t] = (rowp[t] != nullptr && 32 * u + 8 * gq < dim) ? pm_load8(rowp[t] + 32 * u) : pm_zero8();
#pragma unroll
    for (int u = 0; u < DB; ++u)
#pragma unroll
      for (int t = 0; t < 2; ++t) s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][t], qb[u], s[t], 0, 0, 0);
    float p[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int kp = k0 + 8 * gq + j;
      p[j] = (kp >= lo_c && kp <= hi_c) ? pa_sigmoid(s[j >> 2][j & 3] * scale + bias) : 0.f;
    }
    const bf16x8 pb = pm_pack8(p);
    const int gs = k0 + 8 * gq;                          // the lane's 8 consecutive keys, inside one page
    const TS* colp = nullptr;
    if (gs <= hi_max && gs + 7 >= lo_min) {
      const int b = gs / ps;
      const int page = b < width ? bt[b] : -1;
      if (page >= 0) colp = v_pages + ((int64_t)page * nkv + g) * (int64_t)vdim * ps + (gs - b * ps);
    }
    bf16x8 av[VB];
#pragma unroll
    for (int u = 0; u < VB; ++u) {
      const int r = 16 * u + c;
      av[u] = (colp != nullptr && r < vdim) ? pm_load8(colp + (int64_t)r * ps) : pm_zero8();
    }
#pragma unroll
    for (int u = 0; u < VB; ++u) acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[u], pb, acc[u], 0, 0, 0);
  }
}

template <int DB>
__device__ __forceinline__ void pm_load_query(bf16x8 (&qb)[DB], const float* __restrict__ q, int dim, int gq, bool ok) {
#pragma unroll
  for (int u = 0; u < DB; ++u) {
    const int d = 32 * u + 8 * gq;
    qb[u] = (ok && d < dim) ? pm_load8(q + d) : pm_zero8();
  }
}

// prompt portions: grid (tiles, ceil(nh / 4)); tiles int32 [n][4] = (entry, first row of the step, rows, first position)
template <int DB, int VB>
__global__ __launch_bounds__(256) void pwa_rows_kernel(bf16_t* __restrict__ out, const float* __restrict__ q,
                                                       const bf16_t* __restrict__ k_rows, const bf16_t* __restrict__ v_pages,
                                                       const float* __restrict__ pk_rows, const float* __restrict__ pv_pages,
                                                       const int32_t* __restrict__ tiles, const int32_t* __restrict__ table, int width,
                                                       const int32_t* __restrict__ pool_table, int pool_width,
                                                       const float* __restrict__ head_bias, const float* __restrict__ gate,
                                                       int64_t gate_stride, int nh, int nkv, int dim, int vdim, int size, int pool,
                                                       int ps, float scale) {
  const int h = blockIdx.y * 4 + threadIdx.x / WAVE;
  if (h >= nh) return;
  const int lane = threadIdx.x % WAVE, c = lane & 15, gq = lane >> 4;
  const int32_t* tile = tiles + 4 * (int64_t)blockIdx.x;
  const int e = tile[0], row0 = tile[1], nrows = tile[2], pos0 = tile[3];
  const int g = h / (nh / nkv);
  const bool ok = c < nrows;
  const int64_t row = row0 + (ok ? c : 0);
  const int i = pos0 + c;
  const int lo = ok ? (i - size + 1 > 0 ? i - size + 1 : 0) : 1, hi = ok ? i : 0;
  const int nb = ok ? lo / pool : 0;
  bf16x8 qb[DB];
  pm_load_query<DB>(qb, q + (row * nh + h) * (int64_t)dim, dim, gq, ok);
  f32x4 acc[VB];
#pragma unroll
  for (int u = 0; u < VB; ++u) acc[u] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float bias = head_bias ? head_bias[h] : 0.f;
  const int nb_max = pm_wave_max(nb);
  if (nb_max > 0)
    pm_walk<DB, VB, float>(acc, qb, pk_rows, pv_pages, pool_table + (int64_t)e * pool_width, pool_width, nkv, g, dim, vdim, ps, 0,
                           nb - 1, 0, nb_max - 1, 0, 1, scale, bias, c, gq);
  const int lo_min = pm_wave_min(ok ? lo : 0x3fffffff), hi_max = pos0 + nrows - 1;
  pm_walk<DB, VB, bf16_t>(acc, qb, k_rows, v_pages, table + (int64_t)e * width, width, nkv, g, dim, vdim, ps, lo, hi, lo_min, hi_max,
                          0, 1, scale, bias, c, gq);
  if (!ok) return;
#pragma unroll
  for (int u = 0; u < VB; ++u)
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int r = 16 * u + 4 * gq + k;
      if (r < vdim) {
        float a = acc[u][k];
        if (gate) a *= pa_sigmoid(gate[row * gate_stride + (int64_t)h * vdim + r]);
        out[(row * nh + h) * (int64_t)vdim + r] = f32_to_bf16(a);
      }
    }
}

// single tokens: grid (records, nkv, splits); info int32 [n][4] = (row of the step, position, entry, -)
template <int DB, int VB>
__global__ __launch_bounds__(WAVE) void pwa_heads_kernel(bf16_t* __restrict__ out, float* __restrict__ partial,
                                                         const float* __restrict__ q, const bf16_t* __restrict__ k_rows,
                                                         const bf16_t* __restrict__ v_pages, const float* __restrict__ pk_rows,
                                                         const float* __restrict__ pv_pages, const int32_t* __restrict__ info,
                                                         const int32_t* __restrict__ table, int width,
                                                         const int32_t* __restrict__ pool_table, int pool_width,
                                                         const float* __restrict__ head_bias, const float* __restrict__ gate,
                                                         int64_t gate_stride, int nh, int nkv, int dim, int vdim, int size, int pool,
                                                         int ps, float scale) {
  const int lane = threadIdx.x, c = lane & 15, gq = lane >> 4;
  const int32_t* rec = info + 4 * (int64_t)blockIdx.x;
  const int64_t row = rec[0];
  const int i = rec[1], e = rec[2];
  const int g = blockIdx.y, per = nh / nkv, splits = gridDim.z, split = blockIdx.z;
  const bool ok = c < per;
  const int h = g * per + (ok ? c : 0);
  const int lo = i - size + 1 > 0 ? i - size + 1 : 0;
  const int nb = lo / pool;
  bf16x8 qb[DB];
  pm_load_query<DB>(qb, q + (row * nh + h) * (int64_t)dim, dim, gq, ok);
  f32x4 acc[VB];
#pragma unroll
  for (int u = 0; u < VB; ++u) acc[u] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float bias = head_bias ? head_bias[h] : 0.f;
  if (nb > 0)
    pm_walk<DB, VB, float>(acc, qb, pk_rows, pv_pages, pool_table + (int64_t)e * pool_width, pool_width, nkv, g, dim, vdim, ps, 0,
                           nb - 1, 0, nb - 1, split, splits, scale, bias, c, gq);
  pm_walk<DB, VB, bf16_t>(acc, qb, k_rows, v_pages, table + (int64_t)e * width, width, nkv, g, dim, vdim, ps, lo, i, lo, i, split,
                          splits, scale, bias, c, gq);
  if (!ok) return;
#pragma unroll
  for (int u = 0; u < VB; ++u)
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int r = 16 * u + 4 * gq + k;
      if (r < vdim) {
        float a = acc[u][k];
        if (splits > 1) {
          partial[(((int64_t)split * gridDim.x + blockIdx.x) * nh + h) * vdim + r] = a;
        } else {
          if (gate) a *= pa_sigmoid(gate[row * gate_stride + (int64_t)h * vdim + r]);
          out[(row * nh + h) * (int64_t)vdim + r] = f32_to_bf16(a);
        }
      }
    }
}

// out[row, h, :] = gate * (partial[0] + partial[1] + ...): grid (records, pieces of a row)
__global__ __launch_bounds__(256) void pwa_merge_kernel(bf16_t* __restrict__ out, const float* __restrict__ partial,
                                                        const int32_t* __restrict__ info, const float* __restrict__ gate,
                                                        int64_t gate_stride, int records, int splits, int width) {
  const int64_t d = blockIdx.x, row = info[4 * d];
  for (int x = blockIdx.y * 256 + threadIdx.x; x < width; x += 256 * gridDim.y) {
    float a = 0.f;
    for (int s = 0; s < splits; ++s) a += partial[((int64_t)s * records + d) * width + x];
    if (gate) a *= pa_sigmoid(gate[row * gate_stride + x]);
    out[row * width + x] = f32_to_bf16(a);
  }
}

extern "C" int ga_pwa_attend_mfma(void* out, void* partial, const void* q, const void* k_rows, const void* v_pages,
                                  const void* pk_rows, const void* pv_pages, const void* tiles, int n_tiles, const void* info,
                                  int n_single, int splits, const void* table, int width, const void* pool_table, int pool_width,
                                  const void* head_bias, const void* gate, int64_t gate_stride, int nh, int nkv, int dim, int vdim,
                                  int size, int pool, int page_size, float scale, hipStream_t stream) {
  if (nh <= 0 || nkv <= 0 || nh % nkv || nh / nkv > 16 || dim <= 0 || dim > 256 || dim % 8 || vdim <= 0 || vdim > 256) return -1;
  if (size <= 0 || pool <= 0 || page_size <= 0 || page_size % 8 || width <= 0 || pool_width <= 0 || splits < 1) return -2;
  if (nkv > 65535 || splits > 65535 || (nh + 3) / 4 > 65535 || (splits > 1 && !partial)) return -3;
  const int db = dim <= 32 ? 1 : dim <= 64 ? 2 : dim <= 128 ? 4 : 8, vb = vdim <= 32 ? 2 : vdim <= 64 ? 4 : vdim <= 128 ? 8 : 16;
#define ARGS (const float*)q, (const bf16_t*)k_rows, (const bf16_t*)v_pages, (const float*)pk_rows, (const float*)pv_pages
#define TAIL (const int32_t*)table, width, (const int32_t*)pool_table, pool_width, (const float*)head_bias, (const float*)gate, \
             gate_stride, nh, nkv, dim, vdim, size, pool, page_size, scale
#define GO(DB, VB)                                                                                                              \
  if (db == DB && vb == VB) {                                                                                                   \
    if (n_tiles > 0)                                                                                                            \
      hipLaunchKernelGGL((pwa_rows_kernel<DB, VB>), dim3(n_tiles, (nh + 3) / 4), dim3(256), 0, stream, (bf16_t*)out, ARGS,      \
                         (const int32_t*)tiles, TAIL);                                                                          \
    if (n_single > 0)                                                                                                           \
      hipLaunchKernelGGL((pwa_heads_kernel<DB, VB>), dim3(n_single, nkv, splits), dim3(WAVE), 0, stream, (bf16_t*)out,          \
                         (float*)partial, ARGS, (const int32_t*)info, TAIL);                                                    \
  }
  GO(1, 2) GO(1, 4) GO(1, 8) GO(1, 16) GO(2, 2) GO(2, 4) GO(2, 8) GO(2, 16) GO(4, 2) GO(4, 4) GO(4, 8) GO(4, 16) GO(8, 2) GO(8, 4)
  GO(8, 8) GO(8, 16)
#undef GO
#undef TAIL
#undef ARGS
  if (n_single > 0 && splits > 1)
    hipLaunchKernelGGL(pwa_merge_kernel, dim3(n_single, (nh * vdim + 255) / 256 > 64 ? 64 : (nh * vdim + 255) / 256), dim3(256), 0, stream, (bf16_t*)out, (const float*)partial,
                       (const int32_t*)info, (const float*)gate, gate_stride, n_single, splits, nh * vdim);
  return GA_CHECK_LAUNCH();
}
