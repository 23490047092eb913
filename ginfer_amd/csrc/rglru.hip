// The real-gated linear recurrent unit (the recurrence of Griffin's recurrent block), over per-request state.
//   gates:  the channels fall into `blocks` equal parts; in part b, with u_b the part's channels of the token,
//             r = sigmoid(Ra[b] u_b + ra[b]),  i = sigmoid(Ri[b] u_b + ri[b])        (square matrices per part)
//             a = exp(-rate * r * softplus(lam)),  b = sqrt(1 - a^2) * i * u          (1 - a^2 taken as -expm1(2 log a))
//           written as two 32-bit tensors [tokens, channels].  The matrices come TRANSPOSED, [part][in][out], so that
//           neighbouring threads read neighbouring outputs; a sum runs over ascending `in` as one chain of fused
//           multiply-adds, whatever else is in the step.  A workgroup takes RG_TOKENS tokens of one part.
//   scan:   S_t = a_t S_(t-1) + b_t per channel, from S = 0 at a request's start; out[t] = S_t * gelu_tanh(y[t]) (y: 32-bit
//           rows of a projection, before their activation); the state, float [slots, channels], moves on in place.  A thread
//           a channel and entry; entries without tokens touch nothing.
// Everything is 32-bit; only `out` is written in the compute dtype.
#include "common.h"
#include "ginfer_amd.h"

#define RG_THREADS 256
#define RG_TOKENS 8

__global__ __launch_bounds__(RG_THREADS) void rglru_gates_kernel(float* __restrict__ a_out, float* __restrict__ b_out,
                                                                 const float* __restrict__ u, const float* __restrict__ ra_t,
                                                                 const float* __restrict__ ra_b, const float* __restrict__ ri_t,
                                                                 const float* __restrict__ ri_b, const float* __restrict__ lam,
                                                                 int tokens, int channels, int blocks, float rate) {
  extern __shared__ float us[];                        // [bw][RG_TOKENS]
  const int bw = channels / blocks;
  const int t0 = blockIdx.x * RG_TOKENS, nt = min(RG_TOKENS, tokens - t0), b = blockIdx.y;
  for (int idx = threadIdx.x; idx < RG_TOKENS * bw; idx += RG_THREADS) {
    const int tt = idx / bw, i = idx % bw;
    us[i * RG_TOKENS + tt] = tt < nt ? u[(int64_t)(t0 + tt) * channels + b * bw + i] : 0.f;
  }
  __syncthreads();
  const float* wa = ra_t + (int64_t)b * bw * bw;
  const float* wi = ri_t + (int64_t)b * bw * bw;
  for (int o = threadIdx.x; o < bw; o += RG_THREADS) {
    float za[RG_TOKENS], zi[RG_TOKENS];
#pragma unroll
    for (int tt = 0; tt < RG_TOKENS; ++tt) za[tt] = zi[tt] = 0.f;
    for (int i = 0; i < bw; ++i) {
      const float a = wa[(int64_t)i * bw + o], g = wi[(int64_t)i * bw + o];
      const float* ui = us + i * RG_TOKENS;
#pragma unroll
      for (int tt = 0; tt < RG_TOKENS; ++tt) {
        za[tt] = fmaf(a, ui[tt], za[tt]);
        zi[tt] = fmaf(g, ui[tt], zi[tt]);
      }
    }
    const int c = b * bw + o;
    const float ba = ra_b[c], bi = ri_b[c], l = lam[c];
    const float sp = l > 30.f ? l : log1pf(expf(l));                  // softplus
#pragma unroll
    for (int tt = 0; tt < RG_TOKENS; ++tt) {
      if (tt < nt) {
        const float r = 1.0f / (1.0f + expf(-(za[tt] + ba)));
        const float g = 1.0f / (1.0f + expf(-(zi[tt] + bi)));
        const float log_a = -rate * r * sp;
        const int64_t at = (int64_t)(t0 + tt) * channels + c;
        a_out[at] = expf(log_a);
        b_out[at] = sqrtf(-expm1f(2.0f * log_a)) * g * us[o * RG_TOKENS + tt];
      }
    }
  }
}

__device__ __forceinline__ float rg_gelu_tanh(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename T>
__global__ __launch_bounds__(RG_THREADS) void rglru_scan_kernel(T* __restrict__ out, const float* __restrict__ a,
                                                                const float* __restrict__ b, const float* __restrict__ y,
                                                                int64_t y_stride, float* __restrict__ state,
                                                                const int64_t* __restrict__ slots, const int32_t* __restrict__ cu,
                                                                const int32_t* __restrict__ q_start, int channels) {
  const int e = blockIdx.y;
  const int first = cu[e], n = cu[e + 1] - first;
  if (n <= 0) return;
  const int c = blockIdx.x * RG_THREADS + threadIdx.x;
  if (c >= channels) return;
  float* st = state + slots[e] * (int64_t)channels + c;
  float S = q_start[e] == 0 ? 0.f : *st;
  int t = 0;
  for (; t + 4 <= n; t += 4) {                         // four tokens' operands asked for before the chain uses them
    float av[4], bv[4], yv[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int64_t row = first + t + k;
      av[k] = a[row * channels + c];
      bv[k] = b[row * channels + c];
      yv[k] = y[row * y_stride + c];
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      S = fmaf(av[k], S, bv[k]);
      Num<T>::st(out + (int64_t)(first + t + k) * channels + c, S * rg_gelu_tanh(yv[k]));
    }
  }
  for (; t < n; ++t) {
    const int64_t row = first + t;
    S = fmaf(a[row * channels + c], S, b[row * channels + c]);
    Num<T>::st(out + row * channels + c, S * rg_gelu_tanh(y[row * y_stride + c]));
  }
  *st = S;
}

extern "C" int ga_rglru_gates(void* a_out, void* b_out, const void* u, const void* ra_t, const void* ra_b, const void* ri_t,
                              const void* ri_b, const void* lam, int tokens, int channels, int blocks, float rate,
                              hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (channels <= 0 || blocks <= 0 || channels % blocks || blocks > 65535) return -1;
  const int bw = channels / blocks;
  const size_t lds = (size_t)bw * RG_TOKENS * sizeof(float);
  if (lds > 60 * 1024) return -2;
  dim3 grid((tokens + RG_TOKENS - 1) / RG_TOKENS, blocks);
  hipLaunchKernelGGL(rglru_gates_kernel, grid, dim3(RG_THREADS), lds, stream, (float*)a_out, (float*)b_out, (const float*)u,
                     (const float*)ra_t, (const float*)ra_b, (const float*)ri_t, (const float*)ri_b, (const float*)lam, tokens,
                     channels, blocks, rate);
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_rglru_scan(void* out, const void* a, const void* b, const void* y, int64_t y_stride, void* state,
                             const void* slots, const void* cu, const void* q_start, int entries, int channels, int out_bf16,
                             hipStream_t stream) {
  if (entries <= 0) return 0;
  if (channels <= 0 || entries > 65535) return -1;
  dim3 grid((channels + RG_THREADS - 1) / RG_THREADS, entries);
  if (out_bf16)
    hipLaunchKernelGGL(rglru_scan_kernel<bf16_t>, grid, dim3(RG_THREADS), 0, stream, (bf16_t*)out, (const float*)a,
                       (const float*)b, (const float*)y, y_stride, (float*)state, (const int64_t*)slots, (const int32_t*)cu,
                       (const int32_t*)q_start, channels);
  else
    hipLaunchKernelGGL(rglru_scan_kernel<float>, grid, dim3(RG_THREADS), 0, stream, (float*)out, (const float*)a,
                       (const float*)b, (const float*)y, y_stride, (float*)state, (const int64_t*)slots, (const int32_t*)cu,
                       (const int32_t*)q_start, channels);
  return GA_CHECK_LAUNCH();
}
