// A short causal convolution over time on every channel of the 32-bit residual stream, with the inputs that lie before
// a step's tokens taken from per-request state:
//   h[t, c] = x[t, c] + sum_j w[c, j] * x[t - taps + 1 + j, c]            (zeros before the sequence's start)
// (without the x[t, c] in front where add_input is 0; plus bias[c] where a bias is given; x's rows may be columns of a
// wider tensor: x_stride)
// state[slot][k][c], k = 0 .. taps-2, holds the request's last taps-1 inputs (position len - (taps-1) + k, zeros for
// positions before 0).  `apply` reads x and the old state and writes h in the compute dtype; `update`, launched after
// it, moves the state on by the step's tokens.  A request whose q_start is 0 starts from zeros whatever its slot holds.
// Every entry reads its numbers (first row, length, tokens so far, slot) from device arrays, so the launches are the
// same for every batch of the same sizes.
#include "common.h"
#include "ginfer_amd.h"

#define SC_THREADS 256
#define SC_MAX_TAPS 16

template <typename T>
__global__ __launch_bounds__(SC_THREADS) void short_conv_apply_kernel(T* __restrict__ out, const float* __restrict__ x,
                                                                       const float* __restrict__ w, const float* __restrict__ state,
                                                                       const int64_t* __restrict__ slots,
                                                                       const int32_t* __restrict__ token_entry,
                                                                       const int32_t* __restrict__ cu, const int32_t* __restrict__ q_start,
                                                                       int width, int taps, int add_input, int64_t x_stride,
                                                                       const float* __restrict__ bias) {
  const int64_t t = blockIdx.x;
  const int e = token_entry[t];
  const int local = (int)t - cu[e];                 // place of the token among the entry's tokens of this step
  const bool fresh = q_start[e] == 0;
  // with one tap there is no state, and neither `state` nor `slots` is given
  const float* st = taps > 1 ? state + slots[e] * (int64_t)(taps - 1) * width : nullptr;
  for (int c = blockIdx.y * SC_THREADS + threadIdx.x; c < width; c += gridDim.y * SC_THREADS) {
    float acc = (add_input ? x[t * x_stride + c] : 0.f) + (bias ? bias[c] : 0.f);
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;               // how many tokens before t
      float v;
      if (local - back >= 0) v = x[(t - back) * x_stride + c];
      else if (fresh) v = 0.f;
      else v = st[(int64_t)(taps - 1 + local - back) * width + c];
      acc += w[(int64_t)c * taps + j] * v;
    }
    Num<T>::st(out + t * width + c, acc);
  }
}

// one thread per (entry, channel): it reads what it needs of the old state before it writes (new k reads old n + k, which
// lies above k for n >= 1; an entry without tokens changes nothing)
__global__ __launch_bounds__(SC_THREADS) void short_conv_update_kernel(float* __restrict__ state, const float* __restrict__ x,
                                                                        const int64_t* __restrict__ slots,
                                                                        const int32_t* __restrict__ cu,
                                                                        const int32_t* __restrict__ q_start, int width, int taps,
                                                                        int64_t x_stride) {
  const int e = blockIdx.x;
  const int first = cu[e], n = cu[e + 1] - first;
  if (n <= 0) return;
  const bool fresh = q_start[e] == 0;
  float* st = state + slots[e] * (int64_t)(taps - 1) * width;
  for (int c = blockIdx.y * SC_THREADS + threadIdx.x; c < width; c += gridDim.y * SC_THREADS) {
    for (int k = 0; k < taps - 1; ++k) {
      const int local = n - (taps - 1) + k;
      float v;
      if (local >= 0) v = x[(int64_t)(first + local) * x_stride + c];
      else if (fresh) v = 0.f;
      else v = st[(int64_t)(n + k) * width + c];
      st[(int64_t)k * width + c] = v;
    }
  }
}

extern "C" int ga_short_conv_apply(void* out, const void* x, const void* w, const void* state, const void* slots,
                                   const void* token_entry, const void* cu, const void* q_start, int tokens, int width,
                                   int taps, int add_input, int out_bf16, int64_t x_stride, const void* bias, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (width <= 0 || taps < 1 || taps > SC_MAX_TAPS) return -1;
  if (taps > 1 && (state == nullptr || slots == nullptr)) return -2;
  int cols = (width + SC_THREADS - 1) / SC_THREADS;
  if (cols > 64) cols = 64;
  dim3 grid(tokens, cols), block(SC_THREADS);
  if (out_bf16)
    hipLaunchKernelGGL(short_conv_apply_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)out, (const float*)x, (const float*)w,
                       (const float*)state, (const int64_t*)slots, (const int32_t*)token_entry, (const int32_t*)cu,
                       (const int32_t*)q_start, width, taps, add_input, x_stride, (const float*)bias);
  else
    hipLaunchKernelGGL(short_conv_apply_kernel<float>, grid, block, 0, stream, (float*)out, (const float*)x, (const float*)w,
                       (const float*)state, (const int64_t*)slots, (const int32_t*)token_entry, (const int32_t*)cu,
                       (const int32_t*)q_start, width, taps, add_input, x_stride, (const float*)bias);
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_short_conv_update(void* state, const void* x, const void* slots, const void* cu, const void* q_start,
                                    int entries, int width, int taps, int64_t x_stride, hipStream_t stream) {
  if (entries <= 0 || taps <= 1) return 0;
  if (width <= 0 || taps > SC_MAX_TAPS) return -1;
  int cols = (width + SC_THREADS - 1) / SC_THREADS;
  if (cols > 64) cols = 64;
  dim3 grid(entries, cols), block(SC_THREADS);
  hipLaunchKernelGGL(short_conv_update_kernel, grid, block, 0, stream, (float*)state, (const float*)x, (const int64_t*)slots,
                     (const int32_t*)cu, (const int32_t*)q_start, width, taps, x_stride);
  return GA_CHECK_LAUNCH();
}
