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
#define HC_MAX_STREAMS 8

__global__ __launch_bounds__(HC_THREADS) void hc_open_kernel(float* __restrict__ X, const float* __restrict__ x, int width,
                                                             int streams) {
  const int64_t t = blockIdx.x;
  for (int c = threadIdx.x; c < width; c += HC_THREADS) {
    const float v = x[t * width + c];
    for (int s = 0; s < streams; ++s) X[(t * streams + s) * width + c] = v;
  }
}

// u of a token in LDS (dynamic, `width` floats), then the norm's rows
template <typename C>
__device__ __forceinline__ void hc_norm_rows(C* __restrict__ rows, const float* u, float ss, const float* __restrict__ gain,
                                             float eps, int width, int64_t t, float* scratch) {
  ss = block_sum<HC_THREADS / WAVE>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  for (int c = threadIdx.x; c < width; c += HC_THREADS) Num<C>::st(rows + t * width + c, u[c] * inv * gain[c]);
}

template <typename C>
__global__ __launch_bounds__(HC_THREADS) void hc_read_kernel(C* __restrict__ rows, const float* __restrict__ X,
                                                             const float* __restrict__ in_w, const float* __restrict__ gain,
                                                             float eps, int width, int streams) {
  extern __shared__ float u[];
  __shared__ float scratch[HC_THREADS / WAVE];
  const int64_t t = blockIdx.x;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += HC_THREADS) {
    float acc = 0.f;
    for (int s = 0; s < streams; ++s) acc = fmaf(in_w[s], X[(t * streams + s) * width + c], acc);
    u[c] = acc;
    ss = fmaf(acc, acc, ss);
  }
  hc_norm_rows<C>(rows, u, ss, gain, eps, width, t, scratch);
}

template <typename Y, typename C>
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
  for (int c = threadIdx.x; c < width; c += HC_THREADS) {
    float old[HC_MAX_STREAMS];
#pragma unroll
    for (int s = 0; s < HC_MAX_STREAMS; ++s) old[s] = s < streams ? X[(t * streams + s) * width + c] : 0.f;
    float yv = Num<Y>::ld(y + t * width + c);
    for (int p = 1; p < parts; ++p) yv += Num<Y>::ld(y + p * part_stride + t * width + c);
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < HC_MAX_STREAMS; ++j) {
      if (j < streams) {
        float v = 0.f;
#pragma unroll
        for (int s = 0; s < HC_MAX_STREAMS; ++s)
          if (s < streams) v = fmaf(m[s * streams + j], old[s], v);
        v = fmaf(o[j], yv, v);
        X[(t * streams + j) * width + c] = v;
        acc = fmaf(nin[j], v, acc);
      }
    }
    if (rows) {
      u[c] = acc;
      ss = fmaf(acc, acc, ss);
    }
  }
  if (rows) hc_norm_rows<C>(rows, u, ss, next_gain, next_eps, width, t, scratch);
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
  if (rows_bf16)
    hipLaunchKernelGGL(hc_read_kernel<bf16_t>, dim3(tokens), dim3(HC_THREADS), lds, stream, (bf16_t*)rows, (const float*)X,
                       (const float*)in_w, (const float*)gain, eps, width, streams);
  else
    hipLaunchKernelGGL(hc_read_kernel<float>, dim3(tokens), dim3(HC_THREADS), lds, stream, (float*)rows, (const float*)X,
                       (const float*)in_w, (const float*)gain, eps, width, streams);
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_hc_write(void* X, const void* mix, const void* out_w, const void* y, int y_bf16, int parts,
                           int64_t part_stride, const void* next_in, const void* next_gain, float next_eps, void* rows,
                           int rows_bf16, int tokens, int width, int streams, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (!hc_sizes_ok(width, streams) || parts < 1 || (parts > 1 && y_bf16)) return -1;
  if ((rows != nullptr) != (next_in != nullptr) || (rows != nullptr) != (next_gain != nullptr)) return -2;
  const size_t lds = rows ? (size_t)width * sizeof(float) : 0;
#define GO(Y, C) hipLaunchKernelGGL((hc_write_kernel<Y, C>), dim3(tokens), dim3(HC_THREADS), lds, stream, (float*)X,        \
                                    (const float*)mix, (const float*)out_w, (const Y*)y, parts, part_stride,               \
                                    (const float*)next_in, (const float*)next_gain, next_eps, (C*)rows, width, streams)
  if (y_bf16) { if (rows_bf16) GO(bf16_t, bf16_t); else GO(bf16_t, float); }
  else { if (rows_bf16) GO(float, bf16_t); else GO(float, float); }
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
