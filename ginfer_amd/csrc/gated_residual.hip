// Sublayers that run side by side and enter the residual stream through gates of their own:
//   residual[t] += sigmoid(z1[t]) * y1[t] (+ sigmoid(z2[t]) * y2[t])         z: 32-bit rows of gates * hidden numbers with a stride
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
                                                                          C* __restrict__ next, int hidden, int64_t z_stride) {
  __shared__ float scratch[GRS_THREADS / WAVE];
  const int64_t t = blockIdx.x;
  float* res = residual + t * hidden;
  const float* zr = z + t * z_stride;
  const Y* a = y1 + t * hidden;
  const Y* b = y2 ? y2 + t * hidden : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += GRS_THREADS) {
    float d = grs_sigmoid(zr[i]) * Num<Y>::ld(a + i);
    if (b) d = fmaf(grs_sigmoid(zr[hidden + i]), Num<Y>::ld(b + i), d);
    const float r = res[i] + d;
    res[i] = r;
    ss += r * r;
  }
  if (!next) return;
  ss = block_sum<GRS_THREADS / WAVE>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)hidden + next_eps);
  for (int i = threadIdx.x; i < hidden; i += GRS_THREADS) Num<C>::st(next + t * hidden + i, res[i] * inv * next_gain[i]);
}

// The same with four consecutive elements to a thread and access (16-byte loads of the 32-bit rows, 8 or 16 bytes of y), all
// of a row's operands asked for before the first is used, and the new row kept in registers for the norm: rows of a
// multiple of 4 up to GRS_THREADS * 4 * PER elements.
template <typename Y> struct Quad;
template <> struct Quad<float> {
  static __device__ __forceinline__ float4 ld(const float* p) { return *reinterpret_cast<const float4*>(p); }
  static __device__ __forceinline__ void st(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
};
template <> struct Quad<bf16_t> {
  static __device__ __forceinline__ float4 ld(const bf16_t* p) {
    const uint2 u = *reinterpret_cast<const uint2*>(p);
    return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                       __uint_as_float(u.y & 0xffff0000u));
  }
  static __device__ __forceinline__ void st(bf16_t* p, float4 v) {
    uint2 u;
    u.x = (uint32_t)f32_to_bf16(v.x) | ((uint32_t)f32_to_bf16(v.y) << 16);
    u.y = (uint32_t)f32_to_bf16(v.z) | ((uint32_t)f32_to_bf16(v.w) << 16);
    *reinterpret_cast<uint2*>(p) = u;
  }
};

template <typename Y, typename C, int PER>
__global__ __launch_bounds__(GRS_THREADS) void gated_residual_add_quad_kernel(float* __restrict__ residual, const float* __restrict__ z,
                                                                               const Y* __restrict__ y1, const Y* __restrict__ y2,
                                                                               const float* __restrict__ next_gain, float next_eps,
                                                                               C* __restrict__ next, int hidden, int64_t z_stride) {
  __shared__ float scratch[GRS_THREADS / WAVE];
  const int64_t t = blockIdx.x;
  float* res = residual + t * hidden;
  const float* zr = z + t * z_stride;
  const Y* a = y1 + t * hidden;
  const Y* b = y2 ? y2 + t * hidden : nullptr;
  float4 r[PER], za[PER], zb[PER], ya[PER], yb[PER];
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int i = 4 * (threadIdx.x + j * GRS_THREADS);
    if (i < hidden) {
      r[j] = Quad<float>::ld(res + i);
      za[j] = Quad<float>::ld(zr + i);
      ya[j] = Quad<Y>::ld(a + i);
      if (b) {
        zb[j] = Quad<float>::ld(zr + hidden + i);
        yb[j] = Quad<Y>::ld(b + i);
      }
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int i = 4 * (threadIdx.x + j * GRS_THREADS);
    if (i < hidden) {
      float4 d = make_float4(grs_sigmoid(za[j].x) * ya[j].x, grs_sigmoid(za[j].y) * ya[j].y, grs_sigmoid(za[j].z) * ya[j].z,
                             grs_sigmoid(za[j].w) * ya[j].w);
      if (b) {
        d.x = fmaf(grs_sigmoid(zb[j].x), yb[j].x, d.x);
        d.y = fmaf(grs_sigmoid(zb[j].y), yb[j].y, d.y);
        d.z = fmaf(grs_sigmoid(zb[j].z), yb[j].z, d.z);
        d.w = fmaf(grs_sigmoid(zb[j].w), yb[j].w, d.w);
      }
      r[j] = make_float4(r[j].x + d.x, r[j].y + d.y, r[j].z + d.z, r[j].w + d.w);
      Quad<float>::st(res + i, r[j]);
      ss += r[j].x * r[j].x + r[j].y * r[j].y + r[j].z * r[j].z + r[j].w * r[j].w;
    }
  }
  if (!next) return;
  ss = block_sum<GRS_THREADS / WAVE>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)hidden + next_eps);
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int i = 4 * (threadIdx.x + j * GRS_THREADS);
    if (i < hidden) {
      const float4 g = Quad<float>::ld(next_gain + i);
      Quad<C>::st(next + t * hidden + i, make_float4(r[j].x * inv * g.x, r[j].y * inv * g.y, r[j].z * inv * g.z, r[j].w * inv * g.w));
    }
  }
}

extern "C" int ga_gated_residual_add(void* residual, const void* z, int64_t z_stride, const void* y1, const void* y2, int tokens, int hidden,
                                     int y_bf16, const void* next_gain, float next_eps, void* next, int next_bf16,
                                     hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (hidden <= 0 || !z || !y1 || ((next != nullptr) != (next_gain != nullptr))) return -1;
  dim3 grid(tokens), block(GRS_THREADS);
  if (hidden % 4 == 0 && hidden <= GRS_THREADS * 4 * 8 && z_stride % 4 == 0 && ((uintptr_t)z & 15) == 0) {
#define GQ(Y, C, PER) hipLaunchKernelGGL((gated_residual_add_quad_kernel<Y, C, PER>), grid, block, 0, stream, (float*)residual,   \
                                         (const float*)z, (const Y*)y1, (const Y*)y2, (const float*)next_gain, next_eps, (C*)next, \
                                         hidden, z_stride)
#define GP(Y, C) do { if (hidden <= GRS_THREADS * 4) GQ(Y, C, 1); else if (hidden <= GRS_THREADS * 8) GQ(Y, C, 2);              \
                      else if (hidden <= GRS_THREADS * 16) GQ(Y, C, 4); else GQ(Y, C, 8); } while (0)
    if (y_bf16) { if (next_bf16) GP(bf16_t, bf16_t); else GP(bf16_t, float); }
    else { if (next_bf16) GP(float, bf16_t); else GP(float, float); }
#undef GP
#undef GQ
    return GA_CHECK_LAUNCH();
  }
#define GO(Y, C) hipLaunchKernelGGL((gated_residual_add_kernel<Y, C>), grid, block, 0, stream, (float*)residual,          \
                                    (const float*)z, (const Y*)y1, (const Y*)y2, (const float*)next_gain, next_eps, (C*)next, \
                                    hidden, z_stride)
  if (y_bf16) { if (next_bf16) GO(bf16_t, bf16_t); else GO(bf16_t, float); }
  else { if (next_bf16) GO(float, bf16_t); else GO(float, float); }
#undef GO
  return GA_CHECK_LAUNCH();
}
