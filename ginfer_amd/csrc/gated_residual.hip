// Sublayers that run side by side and enter the residual stream through gates of their own:
//   residual[t] += sigmoid(z1[t]) * y1[t] (+ sigmoid(z2[t]) * y2[t])         z: 32-bit rows [tokens, gates * hidden]
//   next[t]      = g * residual[t] / sqrt(mean(residual[t]^2) + eps)         (optional: the norm that is read next)
// The gated results are added to each other first and then to the stream.  All arithmetic in 32-bit; a row's sum of
// squares is taken in an order that depends on its length alone.  A workgroup a token.
#include "common.h"
#include "ginfer_amd.h"

#define GRS_THREADS 256

__device__ __forceinline__ float grs_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }

template <typename Y, typename C>
__global__ __launch_bounds__(GRS_THREADS) void gated_residual_add_kernel(float* __restrict__ residual, const float* __restrict__ z,
                                                                          const Y* __restrict__ y1, const Y* __restrict__ y2,
                                                                          const float* __restrict__ next_gain, float next_eps,
                                                                          C* __restrict__ next, int hidden) {
  __shared__ float scratch[GRS_THREADS / WAVE];
  const int64_t t = blockIdx.x;
  float* res = residual + t * hidden;
  const float* zr = z + t * (int64_t)hidden * (y2 ? 2 : 1);
  const Y* a = y1 + t * hidden;
  const Y* b = y2 ? y2 + t * hidden : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += GRS_THREADS) {
    float d = grs_sigmoid(zr[i]) * Num<Y>::ld(a + i);
    if (b) d += grs_sigmoid(zr[hidden + i]) * Num<Y>::ld(b + i);
    const float r = res[i] + d;
    res[i] = r;
    ss += r * r;
  }
  if (!next) return;
  ss = block_sum<GRS_THREADS / WAVE>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)hidden + next_eps);
  for (int i = threadIdx.x; i < hidden; i += GRS_THREADS) Num<C>::st(next + t * hidden + i, res[i] * inv * next_gain[i]);
}

extern "C" int ga_gated_residual_add(void* residual, const void* z, const void* y1, const void* y2, int tokens, int hidden,
                                     int y_bf16, const void* next_gain, float next_eps, void* next, int next_bf16,
                                     hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (hidden <= 0 || !z || !y1 || ((next != nullptr) != (next_gain != nullptr))) return -1;
  dim3 grid(tokens), block(GRS_THREADS);
#define GO(Y, C) hipLaunchKernelGGL((gated_residual_add_kernel<Y, C>), grid, block, 0, stream, (float*)residual,          \
                                    (const float*)z, (const Y*)y1, (const Y*)y2, (const float*)next_gain, next_eps, (C*)next, \
                                    hidden)
  if (y_bf16) { if (next_bf16) GO(bf16_t, bf16_t); else GO(bf16_t, float); }
  else { if (next_bf16) GO(float, bf16_t); else GO(float, float); }
#undef GO
  return GA_CHECK_LAUNCH();
}
