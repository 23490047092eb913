// Hyper-connections: the residual stream kept as S streams side by side, X float [tokens, S, width], all 32-bit.
//   open:   X[t, s, :] = x[t, :]                                              (every stream starts as the embedding's output)
//   read:   u[t, :] = sum_s in[s] X[t, s, :];  rows[t, :] = gain * u / sqrt(mean(u^2) + eps)       (what a sublayer reads)
//   write:  X'[t, j, :] = sum_s mix[s, j] X[t, s, :] + out[j] * y[t, :]   for all j at once from the old streams; y may be
//           the 32-bit partial sums [parts, tokens, width] of a product whose K was split (added in order); and, where the
//           sublayer that runs next is known, its `read` of the new streams in the same launch
//   sum:    out[r, :] = sum_s X[rows[r], s, :]                                (the model's output reads the streams' sum)
// Sums over s run in ascending s as chains of fused multiply-adds; a row's sum of squares is taken in an order that
// depends on the width alone.  A workgroup a token.
#include "common.h"
#include "ginfer_amd.h"

#define HC_THREADS 256
#define HC_MAX_STREAMS 16

__global__ __launch_bounds__(HC_THREADS) void hc_open_kernel(float* __restrict__ X, const float* __restrict__ x, int width,
                                                             int streams) {
  const int64_t t = blockIdx.x;
  for (int c = threadIdx.x; c < width; c += HC_THREADS) {
    const float v = x[t * width + c];
    for (int s = 0; s < streams; ++s) X[(t * streams + s) * width + c] = v;
  }
}

// V consecutive elements to a thread and access: 1, or 4 where the width allows it (16-byte accesses of the 32-bit rows, 8 or
// 16 bytes of the compute dtype's)
template <typename T, int V> struct Pack;
template <> struct Pack<float, 1> {
  static __device__ __forceinline__ void ld(const float* p, float (&v)[1]) { v[0] = *p; }
  static __device__ __forceinline__ void st(float* p, const float (&v)[1]) { *p = v[0]; }
};
template <> struct Pack<bf16_t, 1> {
  static __device__ __forceinline__ void ld(const bf16_t* p, float (&v)[1]) { v[0] = bf16_to_f32(*p); }
  static __device__ __forceinline__ void st(bf16_t* p, const float (&v)[1]) { *p = f32_to_bf16(v[0]); }
};
template <> struct Pack<float, 4> {
  static __device__ __forceinline__ void ld(const float* p, float (&v)[4]) {
    const float4 f = *reinterpret_cast<const float4*>(p);
    v[0] = f.x; v[1] = f.y; v[2] = f.z; v[3] = f.w;
  }
  static __device__ __forceinline__ void st(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <> struct Pack<bf16_t, 4> {
  static __device__ __forceinline__ void ld(const bf16_t* p, float (&v)[4]) {
    const uint2 u = *reinterpret_cast<const uint2*>(p);
    v[0] = __uint_as_float(u.x << 16); v[1] = __uint_as_float(u.x & 0xffff0000u);
    v[2] = __uint_as_float(u.y << 16); v[3] = __uint_as_float(u.y & 0xffff0000u);
  }
  static __device__ __forceinline__ void st(bf16_t* p, const float (&v)[4]) {
    uint2 u;
    u.x = (uint32_t)f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16);
    u.y = (uint32_t)f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16);
    *reinterpret_cast<uint2*>(p) = u;
  }
};

// u of a token in LDS (dynamic, `width` floats), then the norm's rows
template <typename C, int V>
__device__ __forceinline__ void hc_norm_rows(C* __restrict__ rows, const float* u, float ss, const float* __restrict__ gain,
                                             float eps, int width, int64_t t, float* scratch) {
  ss = block_sum<HC_THREADS / WAVE>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  for (int c = threadIdx.x * V; c < width; c += HC_THREADS * V) {
    float g[V], r[V];
    Pack<float, V>::ld(gain + c, g);
#pragma unroll
    for (int k = 0; k < V; ++k) r[k] = u[c + k] * inv * g[k];
    Pack<C, V>::st(rows + t * width + c, r);
  }
}

template <typename C, int V>
__global__ __launch_bounds__(HC_THREADS) void hc_read_kernel(C* __restrict__ rows, const float* __restrict__ X,
                                                             const float* __restrict__ in_w, const float* __restrict__ gain,
                                                             float eps, int width, int streams) {
  extern __shared__ float u[];
  __shared__ float scratch[HC_THREADS / WAVE];
  const int64_t t = blockIdx.x;
  float ss = 0.f;
  for (int c = threadIdx.x * V; c < width; c += HC_THREADS * V) {
    float acc[V];
#pragma unroll
    for (int k = 0; k < V; ++k) acc[k] = 0.f;
    for (int s = 0; s < streams; ++s) {
      float x[V];
      Pack<float, V>::ld(X + (t * streams + s) * width + c, x);
      const float w = in_w[s];
#pragma unroll
      for (int k = 0; k < V; ++k) acc[k] = fmaf(w, x[k], acc[k]);
    }
#pragma unroll
    for (int k = 0; k < V; ++k) {
      u[c + k] = acc[k];
      ss = fmaf(acc[k], acc[k], ss);
    }
  }
  hc_norm_rows<C, V>(rows, u, ss, gain, eps, width, t, scratch);
}

template <typename Y, typename C, int V>
__global__ __launch_bounds__(HC_THREADS) void hc_write_kernel(float* __restrict__ X, const float* __restrict__ mix,
                                                              const float* __restrict__ out_w, const Y* __restrict__ y,
                                                              int parts, int64_t part_stride, const float* __restrict__ next_in,
                                                              const float* __restrict__ next_gain, float next_eps,
                                                              C* __restrict__ rows, int width, int streams) {
  extern __shared__ float u[];
  __shared__ float scratch[HC_THREADS / WAVE];
  __shared__ float m[HC_MAX_STREAMS * HC_MAX_STREAMS], o[HC_MAX_STREAMS], nin[HC_MAX_STREAMS];
  const int64_t t = blockIdx.x;
  if (threadIdx.x < streams * streams) m[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < streams) {
    o[threadIdx.x] = out_w[threadIdx.x];
    nin[threadIdx.x] = next_in ? next_in[threadIdx.x] : 0.f;
  }
  __syncthreads();
  float ss = 0.f;
  for (int c = threadIdx.x * V; c < width; c += HC_THREADS * V) {
    float old[HC_MAX_STREAMS][V];
#pragma unroll
    for (int s = 0; s < HC_MAX_STREAMS; ++s)
      if (s < streams) Pack<float, V>::ld(X + (t * streams + s) * width + c, old[s]);
    float yv[V];
    Pack<Y, V>::ld(y + t * width + c, yv);
    for (int p = 1; p < parts; ++p) {
      float more[V];
      Pack<Y, V>::ld(y + p * part_stride + t * width + c, more);
#pragma unroll
      for (int k = 0; k < V; ++k) yv[k] += more[k];
    }
    float acc[V];
#pragma unroll
    for (int k = 0; k < V; ++k) acc[k] = 0.f;
#pragma unroll
    for (int j = 0; j < HC_MAX_STREAMS; ++j) {
      if (j < streams) {
        float v[V];
#pragma unroll
        for (int k = 0; k < V; ++k) v[k] = 0.f;
#pragma unroll
        for (int s = 0; s < HC_MAX_STREAMS; ++s)
          if (s < streams) {
#pragma unroll
            for (int k = 0; k < V; ++k) v[k] = fmaf(m[s * streams + j], old[s][k], v[k]);
          }
#pragma unroll
        for (int k = 0; k < V; ++k) {
          v[k] = fmaf(o[j], yv[k], v[k]);
          acc[k] = fmaf(nin[j], v[k], acc[k]);
        }
        Pack<float, V>::st(X + (t * streams + j) * width + c, v);
      }
    }
    if (rows) {
#pragma unroll
      for (int k = 0; k < V; ++k) {
        u[c + k] = acc[k];
        ss = fmaf(acc[k], acc[k], ss);
      }
    }
  }
  if (rows) hc_norm_rows<C, V>(rows, u, ss, next_gain, next_eps, width, t, scratch);
}

// The same for rows of up to HC_THREADS * 4 * PER elements and S streams known when compiled: all of a token's operands are
// asked for before the first is used, the new u stays in registers, and the norm's gain is on its way during the sum through
// LDS.  Every sum in the order of the kernel above: the same bits.  (A decode step's launch is a few trips to memory; this
// one makes them two.)
template <typename Y, typename C, int S, int PER>
__global__ __launch_bounds__(HC_THREADS) void hc_write_rows_kernel(float* __restrict__ X, const float* __restrict__ mix,
                                                                   const float* __restrict__ out_w, const Y* __restrict__ y,
                                                                   int parts, int64_t part_stride,
                                                                   const float* __restrict__ next_in,
                                                                   const float* __restrict__ next_gain, float next_eps,
                                                                   C* __restrict__ rows, int width) {
  __shared__ float scratch[HC_THREADS / WAVE];
  __shared__ float m[S * S], o[S], nin[S];
  const int64_t t = blockIdx.x;
  float old[PER][S][4], yv[PER][4], gain[PER][4];
#pragma unroll
  for (int p = 0; p < PER; ++p) {
    const int c = 4 * (threadIdx.x + p * HC_THREADS);
    if (c < width) {
#pragma unroll
      for (int s = 0; s < S; ++s) Pack<float, 4>::ld(X + (t * S + s) * width + c, old[p][s]);
      Pack<Y, 4>::ld(y + t * width + c, yv[p]);
      if (rows) Pack<float, 4>::ld(next_gain + c, gain[p]);
    }
  }
  if (threadIdx.x < S * S) m[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < S) {
    o[threadIdx.x] = out_w[threadIdx.x];
    nin[threadIdx.x] = next_in ? next_in[threadIdx.x] : 0.f;
  }
  for (int q = 1; q < parts; ++q) {
#pragma unroll
    for (int p = 0; p < PER; ++p) {
      const int c = 4 * (threadIdx.x + p * HC_THREADS);
      if (c < width) {
        float more[4];
        Pack<Y, 4>::ld(y + q * part_stride + t * width + c, more);
#pragma unroll
        for (int k = 0; k < 4; ++k) yv[p][k] += more[k];
      }
    }
  }
  __syncthreads();
  float ss = 0.f, u[PER][4];
#pragma unroll
  for (int p = 0; p < PER; ++p) {
    const int c = 4 * (threadIdx.x + p * HC_THREADS);
    if (c < width) {
#pragma unroll
      for (int k = 0; k < 4; ++k) u[p][k] = 0.f;
#pragma unroll
      for (int j = 0; j < S; ++j) {
        float v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = 0.f;
#pragma unroll
        for (int s2 = 0; s2 < S; ++s2)
#pragma unroll
          for (int k = 0; k < 4; ++k) v[k] = fmaf(m[s2 * S + j], old[p][s2][k], v[k]);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          v[k] = fmaf(o[j], yv[p][k], v[k]);
          u[p][k] = fmaf(nin[j], v[k], u[p][k]);
        }
        Pack<float, 4>::st(X + (t * S + j) * width + c, v);
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) ss = fmaf(u[p][k], u[p][k], ss);
    }
  }
  if (!rows) return;
  ss = block_sum<HC_THREADS / WAVE>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + next_eps);
#pragma unroll
  for (int p = 0; p < PER; ++p) {
    const int c = 4 * (threadIdx.x + p * HC_THREADS);
    if (c < width) {
      float r[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) r[k] = u[p][k] * inv * gain[p][k];
      Pack<C, 4>::st(rows + t * width + c, r);
    }
  }
}

__global__ __launch_bounds__(HC_THREADS) void hc_sum_rows_kernel(float* __restrict__ out, const float* __restrict__ X,
                                                                 const int32_t* __restrict__ rows, int width, int streams) {
  const int64_t r = blockIdx.x;
  const int64_t t = rows ? rows[r] : r;
  for (int c = threadIdx.x; c < width; c += HC_THREADS) {
    float acc = 0.f;
    for (int s = 0; s < streams; ++s) acc += X[(t * streams + s) * width + c];
    out[r * width + c] = acc;
  }
}

static bool hc_sizes_ok(int width, int streams) {
  return width > 0 && streams >= 1 && streams <= HC_MAX_STREAMS && (size_t)width * sizeof(float) <= 60 * 1024;
}

extern "C" int ga_hc_max_streams() { return HC_MAX_STREAMS; }

extern "C" int ga_hc_open(void* X, const void* x, int tokens, int width, int streams, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (!hc_sizes_ok(width, streams)) return -1;
  hipLaunchKernelGGL(hc_open_kernel, dim3(tokens), dim3(HC_THREADS), 0, stream, (float*)X, (const float*)x, width, streams);
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_hc_read(void* rows, const void* X, const void* in_w, const void* gain, float eps, int tokens, int width,
                          int streams, int rows_bf16, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (!hc_sizes_ok(width, streams)) return -1;
  const size_t lds = (size_t)width * sizeof(float);
  const bool vec = width % 4 == 0 && (((uintptr_t)X | (uintptr_t)rows | (uintptr_t)gain) & 15) == 0;
#define GO(C, V) hipLaunchKernelGGL((hc_read_kernel<C, V>), dim3(tokens), dim3(HC_THREADS), lds, stream, (C*)rows,          \
                                    (const float*)X, (const float*)in_w, (const float*)gain, eps, width, streams)
  if (rows_bf16) { if (vec) GO(bf16_t, 4); else GO(bf16_t, 1); }
  else { if (vec) GO(float, 4); else GO(float, 1); }
#undef GO
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_hc_write(void* X, const void* mix, const void* out_w, const void* y, int y_bf16, int parts,
                           int64_t part_stride, const void* next_in, const void* next_gain, float next_eps, void* rows,
                           int rows_bf16, int tokens, int width, int streams, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (!hc_sizes_ok(width, streams) || parts < 1 || (parts > 1 && y_bf16)) return -1;
  if ((rows != nullptr) != (next_in != nullptr) || (rows != nullptr) != (next_gain != nullptr)) return -2;
  const size_t lds = rows ? (size_t)width * sizeof(float) : 0;
  const bool vec = width % 4 == 0 && (((uintptr_t)X | (uintptr_t)rows | (uintptr_t)next_gain | (uintptr_t)y) & 15) == 0 &&
                   (part_stride * (y_bf16 ? 2 : 4)) % 16 == 0;
#define GO(Y, C, V) hipLaunchKernelGGL((hc_write_kernel<Y, C, V>), dim3(tokens), dim3(HC_THREADS), lds, stream, (float*)X,  \
                                       (const float*)mix, (const float*)out_w, (const Y*)y, parts, part_stride,            \
                                       (const float*)next_in, (const float*)next_gain, next_eps, (C*)rows, width, streams)
#define GR(Y, C, S, PER) hipLaunchKernelGGL((hc_write_rows_kernel<Y, C, S, PER>), dim3(tokens), dim3(HC_THREADS), 0, stream,   \
                                            (float*)X, (const float*)mix, (const float*)out_w, (const Y*)y, parts, part_stride, \
                                            (const float*)next_in, (const float*)next_gain, next_eps, (C*)rows, width)
#define GP(Y, C, S) do { if (width <= HC_THREADS * 4) GR(Y, C, S, 1); else if (width <= HC_THREADS * 8) GR(Y, C, S, 2);         \
                         else GR(Y, C, S, 4); } while (0)
#define GV(Y, C) do { if (vec && width <= HC_THREADS * 16 && streams <= 4) {                                                   \
                        if (streams == 1) GP(Y, C, 1); else if (streams == 2) GP(Y, C, 2);                                     \
                        else if (streams == 3) GP(Y, C, 3); else GP(Y, C, 4);                                                  \
                      } else if (vec) GO(Y, C, 4); else GO(Y, C, 1); } while (0)
  if (y_bf16) { if (rows_bf16) GV(bf16_t, bf16_t); else GV(bf16_t, float); }
  else { if (rows_bf16) GV(float, bf16_t); else GV(float, float); }
#undef GV
#undef GP
#undef GR
#undef GO
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_hc_sum_rows(void* out, const void* X, const void* rows, int n_rows, int width, int streams,
                              hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (!hc_sizes_ok(width, streams)) return -1;
  hipLaunchKernelGGL(hc_sum_rows_kernel, dim3(n_rows), dim3(HC_THREADS), 0, stream, (float*)out, (const float*)X,
                     (const int32_t*)rows, width, streams);
  return GA_CHECK_LAUNCH();
}
