// Between a fused q|k|v projection and the attention kernels, for a mixer whose projections pass a short causal
// convolution over time: one launch does, for every token of the step,
// (a workgroup per token and head)
//   c[ch]  = sum_j w[ch, j] * u[t - taps + 1 + j, ch]     (u: the projection's rows; those before the step's tokens come
//                                                           from per-request state, zeros before the sequence's start)
//   q, k:    optionally divided by the root mean square of the token's whole q (k) projection, times a gain per channel
//   q, k:    the first rotary_dim coordinates of every head turned by the position's angle (pairs i, i + rotary_dim/2)
//   q   ->   out[t, head * padded + d]                      (heads padded with zeros to the width the attention takes)
//   k   ->   k_pages[page, kv head, place, d],   v -> v_pages[page, kv head, d, place]   (padded alike)
// Keys are head_dim wide, values value_dim; both are stored `padded` wide.  A second launch moves the state on by the
// step's tokens (a token of the first launch may read what the second overwrites).  The convolution, the rotation and
// the sums are 32-bit; the projection's rows come in 32-bit too (U = float; or in the compute dtype), so that what is
// cached is rounded once, at the end.  Every entry's numbers come from device arrays.
#include "common.h"
#include "ginfer_amd.h"

#define CR_THREADS 256
#define CR_HEAD_THREADS 256       // channels of a head (padded): the attention kernels take up to 256
#define CR_MAX_TAPS 16

// grid (tokens, nh + 2 nkv): a workgroup per token and head (q heads, then k heads, then v heads), a thread per channel
template <typename T, typename U>
__global__ __launch_bounds__(CR_HEAD_THREADS) void conv_rope_kv_kernel(
    T* __restrict__ q_out, const U* __restrict__ proj, const float* __restrict__ w, const float* __restrict__ state,
    const int64_t* __restrict__ slots, const int32_t* __restrict__ token_entry, const int32_t* __restrict__ cu,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ positions, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, const int64_t* __restrict__ slot_mapping, T* __restrict__ k_pages, T* __restrict__ v_pages,
    int nh, int nkv, int hd, int vd, int padded, int rotary_dim, int taps, int page_size, int write_kv,
    const float* __restrict__ row_scale, const float* __restrict__ gain) {
  __shared__ float head[CR_HEAD_THREADS];              // the head's convolved channels
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, d = threadIdx.x;
  const bool is_q = h < nh, is_k = !is_q && h < nh + nkv;
  const int g = is_q ? h : is_k ? h - nh : h - nh - nkv;                // the head among its kind
  const int own = (is_q || is_k) ? hd : vd;                             // its channels
  const int first = is_q ? g * hd : is_k ? (nh + g) * hd : (nh + nkv) * hd + g * vd;
  const int width = (nh + nkv) * hd + nkv * vd;
  const int64_t slot = (write_kv && !is_q) ? slot_mapping[t] : -1;
  if (!is_q && slot < 0) return;                       // nothing to write for this token
  float acc = 0.f;
  if (d < own) {
    const int c = first + d;
    if (w == nullptr) {
      acc = Num<U>::ld(proj + t * width + c);
    } else {
      const int e = token_entry[t];
      const int local = (int)t - cu[e];
      const bool fresh = q_start[e] == 0;
      const float* st = taps > 1 ? state + slots[e] * (int64_t)(taps - 1) * width : nullptr;
      for (int j = 0; j < taps; ++j) {
        const int back = taps - 1 - j;
        float v;
        if (local - back >= 0) v = Num<U>::ld(proj + (t - back) * width + c);
        else if (fresh) v = 0.f;
        else v = st[(int64_t)(taps - 1 + local - back) * width + c];
        acc += w[(int64_t)c * taps + j] * v;
      }
    }
  }
  // a norm over the whole projection of q (and of k): the row's factor from the launch before, a gain per channel
  if (row_scale != nullptr && !(!is_q && !is_k) && d < own) acc = acc * row_scale[t * 2 + (is_k ? 1 : 0)] * gain[first + d];
  const bool rotate = (is_q || is_k) && cos_t != nullptr;
  if (rotate) {
    head[d] = acc;
    __syncthreads();
    if (d < rotary_dim) {
      const int half = rotary_dim / 2, j = d < half ? d : d - half;
      const int64_t at = (int64_t)positions[t] * half + j;
      const float a = head[j], b = head[j + half], c = cos_t[at], s = sin_t[at];
      acc = d < half ? a * c - b * s : b * c + a * s;
    }
  }
  if (d >= padded) return;                             // (acc is zero from a head's own width on)
  if (is_q) {
    Num<T>::st(q_out + (t * nh + g) * (int64_t)padded + d, acc);
    return;
  }
  int64_t page, off;
  slot_page(slot, page_size, page, off);
  if (is_k) Num<T>::st(k_pages + ((page * nkv + g) * page_size + off) * padded + d, acc);
  else Num<T>::st(v_pages + ((page * nkv + g) * padded + d) * page_size + off, acc);
}

// row_scale[t, 0] = 1 / sqrt(mean(q[t, :]^2) + eps) over all nh * hd channels of the token's queries, row_scale[t, 1] the
// same over its nkv * hd key channels: the factors of a norm that runs over the whole projection before it is cut into
// heads.  A workgroup a token; every thread's partial sum and the workgroup's sum in an order that depends on the sizes alone.
template <typename U>
__global__ __launch_bounds__(CR_THREADS) void projection_rms_kernel(float* __restrict__ row_scale, const U* __restrict__ proj,
                                                                     int width, int q_width, int k_width, float eps) {
  __shared__ float scratch[CR_THREADS / WAVE];
  const int64_t t = blockIdx.x;
  const U* row = proj + t * width;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < q_width; i += CR_THREADS) { const float v = Num<U>::ld(row + i); sq = fmaf(v, v, sq); }
  for (int i = threadIdx.x; i < k_width; i += CR_THREADS) { const float v = Num<U>::ld(row + q_width + i); sk = fmaf(v, v, sk); }
  sq = block_sum<CR_THREADS / WAVE>(sq, scratch);
  sk = block_sum<CR_THREADS / WAVE>(sk, scratch);
  if (threadIdx.x == 0) {
    row_scale[t * 2] = 1.0f / sqrtf(sq / (float)q_width + eps);
    row_scale[t * 2 + 1] = 1.0f / sqrtf(sk / (float)k_width + eps);
  }
}

// one thread per (entry, channel): new state k <- the projection's row n - (taps - 1) + k of the entry's n tokens, or, where
// that lies before the step, old state n + k (read before it is written: it lies above k), or zero for a fresh request
template <typename T>
__global__ __launch_bounds__(CR_THREADS) void conv_state_update_kernel(float* __restrict__ state, const T* __restrict__ proj,
                                                                        const int64_t* __restrict__ slots,
                                                                        const int32_t* __restrict__ cu,
                                                                        const int32_t* __restrict__ q_start, int width, int taps) {
  const int e = blockIdx.x;
  const int first = cu[e], n = cu[e + 1] - first;
  if (n <= 0) return;
  const bool fresh = q_start[e] == 0;
  float* st = state + slots[e] * (int64_t)(taps - 1) * width;
  for (int c = blockIdx.y * CR_THREADS + threadIdx.x; c < width; c += gridDim.y * CR_THREADS) {
    for (int k = 0; k < taps - 1; ++k) {
      const int local = n - (taps - 1) + k;
      float v;
      if (local >= 0) v = Num<T>::ld(proj + (int64_t)(first + local) * width + c);
      else if (fresh) v = 0.f;
      else v = st[(int64_t)(n + k) * width + c];
      st[(int64_t)k * width + c] = v;
    }
  }
}

extern "C" int ga_conv_rope_kv(void* q_out, const void* proj, const void* w, void* state, const void* slots,
                               const void* token_entry, const void* cu, const void* q_start, const void* positions,
                               const void* cos_t, const void* sin_t, const void* slot_mapping, void* k_pages, void* v_pages,
                               int tokens, int entries, int nh, int nkv, int hd, int vd, int padded, int rotary_dim, int taps,
                               int page_size, int write_kv, int update_state, int is_bf16, int proj_bf16, void* row_scale,
                               const void* gain, float norm_eps, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (nh <= 0 || nkv <= 0 || hd <= 0 || vd <= 0 || padded < hd || padded < vd || page_size <= 0) return -1;
  if (taps < 1 || taps > CR_MAX_TAPS || (w == nullptr && taps != 1)) return -2;
  if (taps > 1 && (state == nullptr || slots == nullptr)) return -3;
  if (rotary_dim < 0 || rotary_dim % 2 || rotary_dim > hd || (rotary_dim > 0) != (cos_t != nullptr) || (cos_t == nullptr) != (sin_t == nullptr)) return -4;
  if (write_kv && (!slot_mapping || !k_pages || !v_pages)) return -5;
  const int width = (nh + nkv) * hd + nkv * vd;
  if (padded > CR_HEAD_THREADS) return -6;
  if ((row_scale != nullptr) != (gain != nullptr) || (row_scale != nullptr && taps != 1)) return -9;
  if (nh + 2 * nkv > 65535) return -7;
  int threads = 64;
  while (threads < padded) threads *= 2;
#define GO(T, U)                                                                                                       \
  do {                                                                                                                 \
    if (row_scale != nullptr)                                                                                          \
      hipLaunchKernelGGL(projection_rms_kernel<U>, dim3(tokens), dim3(CR_THREADS), 0, stream, (float*)row_scale,       \
                         (const U*)proj, width, nh * hd, nkv * hd, norm_eps);                                          \
    hipLaunchKernelGGL((conv_rope_kv_kernel<T, U>), dim3(tokens, nh + 2 * nkv), dim3(threads), 0, stream, (T*)q_out,   \
                       (const U*)proj, (const float*)w, (const float*)state, (const int64_t*)slots,                    \
                       (const int32_t*)token_entry, (const int32_t*)cu, (const int32_t*)q_start,                       \
                       (const int32_t*)positions, (const float*)cos_t, (const float*)sin_t,                            \
                       (const int64_t*)slot_mapping, (T*)k_pages, (T*)v_pages, nh, nkv, hd, vd, padded, rotary_dim,    \
                       taps, page_size, write_kv, (const float*)row_scale, (const float*)gain);                        \
    int rc = GA_CHECK_LAUNCH();                                                                                        \
    if (rc) return rc;                                                                                                 \
    if (update_state && taps > 1 && entries > 0) {                                                                     \
      int cols = (width + CR_THREADS - 1) / CR_THREADS;                                                                \
      if (cols > 64) cols = 64;                                                                                        \
      hipLaunchKernelGGL(conv_state_update_kernel<U>, dim3(entries, cols), dim3(CR_THREADS), 0, stream, (float*)state, \
                         (const U*)proj, (const int64_t*)slots, (const int32_t*)cu, (const int32_t*)q_start, width,    \
                         taps);                                                                                        \
    }                                                                                                                  \
  } while (0)
  if (!is_bf16 && proj_bf16) return -8;
  if (is_bf16 && proj_bf16) GO(bf16_t, bf16_t); else if (is_bf16) GO(bf16_t, float); else GO(float, float);
#undef GO
  return GA_CHECK_LAUNCH();
}
