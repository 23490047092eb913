// The real-gated linear recurrent unit (the recurrence of Griffin's recurrent block), over per-request state.
//   gates:  the channels fall into `blocks` equal parts; in part b, with u_b the part's channels of the token,
//             r = sigmoid(Ra[b] u_b + ra[b]),  i = sigmoid(Ri[b] u_b + ri[b])        (square matrices per part)
//             a = exp(-rate * r * softplus(lam)),  b = sqrt(1 - a^2) * i * u          (1 - a^2 taken as -expm1(2 log a))
//           written as two 32-bit tensors [tokens, channels].  The matrices come TRANSPOSED, [part][in][out], so that
//           neighbouring threads read neighbouring outputs; a sum runs over ascending `in` as one chain of fused
//           multiply-adds, whatever else is in the step.  A workgroup takes a few dozen tokens of one part.
//           The gates' launch also writes g = gelu_tanh(y) of the other branch (y: 32-bit rows of a projection, before their
//           activation), so that the walk over time below has nothing to work out but its own chain.
//   scan:   S_t = a_t S_(t-1) + b_t per channel, from S = 0 at a request's start; out[t] = S_t * g[t]; the state, float
//           [slots, channels], moves on in place.  Steps of single tokens: a thread a channel and entry.  Steps with prompt
//           portions: a workgroup owns RG_CH channels of an entry; all its wavefronts bring tiles of RG_TILE tokens of a, b
//           and g into LDS, a tile ahead of the one wavefront that walks the chain (the chain's own arithmetic is a few
//           instructions a token; what it would wait for is memory).  One chain of fused multiply-adds per channel either
//           way: the same bits however a prompt is cut.  Entries without tokens touch nothing.
// Everything is 32-bit; only `out` is written in the compute dtype.
#include "common.h"
#include "ginfer_amd.h"

#define RG_THREADS 256

__device__ __forceinline__ float rg_gelu_tanh(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// TOK tokens a thread; a workgroup holds `groups` such sets of tokens side by side where a part has fewer outputs than the
// workgroup has threads (thread = (set of tokens, output)), so that all threads work and a part's matrices are read once for
// groups * TOK tokens.  RG_BATCH elements of each matrix are asked for before the first is used: 16 in steps of many tokens,
// 64 in steps of few (a decode step waits for nothing but these loads, one round after the other).
template <int TOK, int RG_BATCH>
__global__ __launch_bounds__(RG_THREADS) void rglru_gates_kernel(float* __restrict__ a_out, float* __restrict__ b_out,
                                                                 const float* __restrict__ u, const float* __restrict__ ra_t,
                                                                 const float* __restrict__ ra_b, const float* __restrict__ ri_t,
                                                                 const float* __restrict__ ri_b, const float* __restrict__ lam,
                                                                 const float* __restrict__ y, int64_t y_stride,
                                                                 float* __restrict__ g_out, int tokens, int channels,
                                                                 int blocks, int groups, float rate) {
  extern __shared__ float us[];                        // [bw][groups * TOK]
  const int bw = channels / blocks, per = groups * TOK;
  const int t0 = blockIdx.x * per, nt = min(per, tokens - t0), b = blockIdx.y;
  for (int idx = threadIdx.x; idx < per * bw; idx += RG_THREADS) {
    const int tt = idx / bw, i = idx % bw;
    us[i * per + tt] = tt < nt ? u[(int64_t)(t0 + tt) * channels + b * bw + i] : 0.f;
  }
  __syncthreads();
  // a part's outputs may be dealt to several workgroups (gridDim.z: steps of few tokens, where a part's matrices are all
  // that is read and more compute units should pull them)
  const int os = (bw + gridDim.z - 1) / gridDim.z, o_begin = blockIdx.z * os, o_end = min(bw, o_begin + os);
  const int lanes = min(os, RG_THREADS);               // outputs side by side in a workgroup
  const int tg = threadIdx.x / lanes;                  // this thread's set of tokens
  if (tg >= groups) return;
  const float* wa = ra_t + (int64_t)b * bw * bw;
  const float* wi = ri_t + (int64_t)b * bw * bw;
  for (int o = o_begin + threadIdx.x % lanes; o < o_end; o += lanes) {
    float za[TOK], zi[TOK];
#pragma unroll
    for (int tt = 0; tt < TOK; ++tt) za[tt] = zi[tt] = 0.f;
    for (int i0 = 0; i0 < bw; i0 += RG_BATCH) {
      float wav[RG_BATCH], wiv[RG_BATCH];
#pragma unroll
      for (int j = 0; j < RG_BATCH; ++j) {
        const bool ok = i0 + j < bw;
        wav[j] = ok ? wa[(int64_t)(i0 + j) * bw + o] : 0.f;
        wiv[j] = ok ? wi[(int64_t)(i0 + j) * bw + o] : 0.f;
      }
#pragma unroll
      for (int j = 0; j < RG_BATCH; ++j) {
        if (i0 + j < bw) {
          const float* ui = us + (i0 + j) * per + tg * TOK;
#pragma unroll
          for (int tt = 0; tt < TOK; ++tt) {
            za[tt] = fmaf(wav[j], ui[tt], za[tt]);
            zi[tt] = fmaf(wiv[j], ui[tt], zi[tt]);
          }
        }
      }
    }
    const int c = b * bw + o;
    const float ba = ra_b[c], bi = ri_b[c], l = lam[c];
    const float sp = l > 30.f ? l : log1pf(expf(l));                  // softplus
#pragma unroll
    for (int tt = 0; tt < TOK; ++tt) {
      const int local = tg * TOK + tt;
      if (local < nt) {
        const float r = 1.0f / (1.0f + expf(-(za[tt] + ba)));
        const float g = 1.0f / (1.0f + expf(-(zi[tt] + bi)));
        const float log_a = -rate * r * sp;
        const int64_t at = (int64_t)(t0 + local) * channels + c;
        a_out[at] = expf(log_a);
        b_out[at] = sqrtf(-expm1f(2.0f * log_a)) * g * us[o * per + local];
        g_out[at] = rg_gelu_tanh(y[(int64_t)(t0 + local) * y_stride + c]);
      }
    }
  }
}

template <typename T>
__global__ __launch_bounds__(RG_THREADS) void rglru_scan_kernel(T* __restrict__ out, const float* __restrict__ a,
                                                                const float* __restrict__ b, const float* __restrict__ g,
                                                                float* __restrict__ state, const int64_t* __restrict__ slots,
                                                                const int32_t* __restrict__ cu, const int32_t* __restrict__ q_start,
                                                                int channels) {
  const int e = blockIdx.y;
  const int first = cu[e], n = cu[e + 1] - first;
  if (n <= 0) return;
  const int c = blockIdx.x * RG_THREADS + threadIdx.x;
  if (c >= channels) return;
  float* st = state + slots[e] * (int64_t)channels + c;
  float S = q_start[e] == 0 ? 0.f : *st;
  for (int t = 0; t < n; ++t) {
    const int64_t at = (int64_t)(first + t) * channels + c;
    S = fmaf(a[at], S, b[at]);
    Num<T>::st(out + at, S * g[at]);
  }
  *st = S;
}

#define RG_CH 16          // channels of a workgroup of the tiled walk
#define RG_TILE 64        // tokens of a tile
template <typename T>
__global__ __launch_bounds__(RG_THREADS) void rglru_scan_tiled_kernel(T* __restrict__ out, const float* __restrict__ a,
                                                                      const float* __restrict__ b, const float* __restrict__ g,
                                                                      float* __restrict__ state, const int64_t* __restrict__ slots,
                                                                      const int32_t* __restrict__ cu,
                                                                      const int32_t* __restrict__ q_start, int channels) {
  constexpr int PER = RG_TILE * RG_CH / RG_THREADS;        // elements of each of a, b, g that a thread brings per tile
  __shared__ float as[2][RG_TILE][RG_CH], bs[2][RG_TILE][RG_CH], gs[2][RG_TILE][RG_CH];
  const int e = blockIdx.y;
  const int first = cu[e], n = cu[e + 1] - first;
  if (n <= 0) return;
  const int c0 = blockIdx.x * RG_CH;
  float ra[PER], rb[PER], rg[PER];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int idx = threadIdx.x + k * RG_THREADS, tt = idx / RG_CH, ch = idx % RG_CH;
      const bool ok = t0 + tt < n && c0 + ch < channels;
      const int64_t at = (int64_t)(first + t0 + tt) * channels + c0 + ch;
      ra[k] = ok ? a[at] : 0.f;
      rb[k] = ok ? b[at] : 0.f;
      rg[k] = ok ? g[at] : 0.f;
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int idx = threadIdx.x + k * RG_THREADS, tt = idx / RG_CH, ch = idx % RG_CH;
      as[buf][tt][ch] = ra[k];
      bs[buf][tt][ch] = rb[k];
      gs[buf][tt][ch] = rg[k];
    }
  };
  const bool walker = threadIdx.x < RG_CH && c0 + threadIdx.x < channels;
  float* st = state + slots[e] * (int64_t)channels + c0 + threadIdx.x;
  float S = (walker && q_start[e] != 0) ? *st : 0.f;
  fetch(0);
  stage(0);
  __syncthreads();
  int buf = 0;
  for (int t0 = 0; t0 < n; t0 += RG_TILE) {
    const bool more = t0 + RG_TILE < n;
    if (more) fetch(t0 + RG_TILE);                       // on its way while the chain walks this tile
    if (walker) {
      const int nt = min(RG_TILE, n - t0);
      for (int tt = 0; tt < nt; ++tt) {
        S = fmaf(as[buf][tt][threadIdx.x], S, bs[buf][tt][threadIdx.x]);
        Num<T>::st(out + (int64_t)(first + t0 + tt) * channels + c0 + threadIdx.x, S * gs[buf][tt][threadIdx.x]);
      }
    }
    if (more) stage(buf ^ 1);                            // the other buffer: nobody reads it during this tile
    __syncthreads();
    buf ^= 1;
  }
  if (walker) *st = S;
}

extern "C" int ga_rglru_gates(void* a_out, void* b_out, const void* u, const void* ra_t, const void* ra_b, const void* ri_t,
                              const void* ri_b, const void* lam, const void* y, int64_t y_stride, void* g_out, int tokens,
                              int channels, int blocks, float rate, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (channels <= 0 || blocks <= 0 || channels % blocks || blocks > 65535) return -1;
  const int bw = channels / blocks;
  // sets of tokens side by side where a part is narrower than the workgroup (at most 8: the tile of u lies in LDS)
  // steps of few tokens: a part's outputs in slices of 32 to a workgroup (at most 16 slices)
  int slices = 1;
  if (tokens <= 64 && bw > 32) slices = (bw + 31) / 32 > 16 ? 16 : (bw + 31) / 32;
  const int os = (bw + slices - 1) / slices;
  int groups = os >= RG_THREADS ? 1 : RG_THREADS / os;
  if (groups > 8) groups = 8;
  int tok = 16;                                          // as many tokens a thread as leave the tile of u in 60 KB of LDS
  while (tok > 1 && (size_t)bw * groups * tok * sizeof(float) > 60 * 1024) tok = tok > 4 ? tok / 2 : 1;
  const size_t lds = (size_t)bw * groups * tok * sizeof(float);
  if (lds > 60 * 1024) return -2;
  while (groups > 1 && (groups - 1) * tok >= tokens) --groups;       // no more sets of tokens than the step has
  const size_t lds2 = (size_t)bw * groups * tok * sizeof(float);
  dim3 grid((tokens + groups * tok - 1) / (groups * tok), blocks, slices);
#define GO(TOK, B) hipLaunchKernelGGL((rglru_gates_kernel<TOK, B>), grid, dim3(RG_THREADS), lds2, stream, (float*)a_out, (float*)b_out, \
                                   (const float*)u, (const float*)ra_t, (const float*)ra_b, (const float*)ri_t,                \
                                   (const float*)ri_b, (const float*)lam, (const float*)y, y_stride, (float*)g_out, tokens,    \
                                   channels, blocks, groups, rate)
  if (tok == 16) { if (tokens <= 64) GO(16, 64); else GO(16, 16); }
  else if (tok == 8) { if (tokens <= 64) GO(8, 64); else GO(8, 16); }
  else if (tok == 4) GO(4, 16);
  else GO(1, 16);
#undef GO
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_rglru_scan(void* out, const void* a, const void* b, const void* g, void* state, const void* slots,
                             const void* cu, const void* q_start, int entries, int tokens, int channels, int out_bf16,
                             hipStream_t stream) {
  if (entries <= 0) return 0;
  if (channels <= 0 || entries > 65535) return -1;
  // a step of single tokens (as many entries as tokens, or more: padding) walks nothing: a thread a channel
  const bool single = tokens <= entries;
  dim3 grid(single ? (channels + RG_THREADS - 1) / RG_THREADS : (channels + RG_CH - 1) / RG_CH, entries);
#define GO(K, T) hipLaunchKernelGGL(K<T>, grid, dim3(RG_THREADS), 0, stream, (T*)out, (const float*)a, (const float*)b,  \
                                    (const float*)g, (float*)state, (const int64_t*)slots, (const int32_t*)cu,           \
                                    (const int32_t*)q_start, channels)
  if (single) { if (out_bf16) GO(rglru_scan_kernel, bf16_t); else GO(rglru_scan_kernel, float); }
  else { if (out_bf16) GO(rglru_scan_tiled_kernel, bf16_t); else GO(rglru_scan_tiled_kernel, float); }
#undef GO
  return GA_CHECK_LAUNCH();
}
