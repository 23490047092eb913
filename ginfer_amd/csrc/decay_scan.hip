// Linear attention with a decay, as a recurrence over per-request state (gated linear attention, retention):
//   per head:  S_t = diag(a_t) S_(t-1) + k_t v_t^T   (S is [dim, vdim]; a acts on the rows, which belong to the key channels),
//              o_t = S_t^T q_t
// a_t is one number per token and key channel (`decay`, float [tokens, heads * dim]) or one constant per head
// (`head_decay`, float [heads]).  q and k may be turned by position on their first rot_dims coordinates (coordinate i pairs
// with i + rot_dims / 2; angle tables cos, sin float [positions, rot_dims / 2]) and are then multiplied by q_scale and
// k_scale.  q, k and v are 32-bit rows of one projection (a common row stride).
// The state is 32-bit, [slot][head][dim][vdim]; a request whose q_start is 0 starts from zeros.  A workgroup owns one
// (entry, head, block of 16 value columns) and walks the entry's tokens in order, up to 16 at a time: the tile's q, k, a and v go
// through LDS (asked for from memory a tile ahead), every thread keeps the state of one column and every 16th row in registers, and the rows' partial
// outputs are added in a fixed order.  So a token's result does not depend on how the request's tokens were cut into
// steps, nor on what else is in the batch.
// gla_decay: a = sigmoid(z)^(1/tau), z = A2 (low) + b (A2 handed over transposed), `low` being the rows of a narrow projection (32-bit), as
//   exp(-softplus(-z) / tau), all in 32-bit.
// head_norm_gate: out[t, h, :] = o[t, h, :] / sqrt(mean(o[t, h, :]^2) + eps) (* weight[:]) (* silu(gate[t, h, :]), or * sigmoid of it).
// silu_inputs: the recurrence reads silu(q), silu(k), silu(v) in place of the projection's numbers.
#include "common.h"
#include "ginfer_amd.h"

#define DS_THREADS 256
#define DS_COLS 16        // value columns of a workgroup
#define DS_SLICES 16      // a column's rows are dealt to this many threads

template <int R, int TILE>   // R rows of the state per thread: dim <= 16 * R; TILE tokens per trip through LDS (<= 16)
__global__ __launch_bounds__(DS_THREADS) void decay_scan_kernel(
    float* __restrict__ out, const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v,
    int64_t stride, const float* __restrict__ decay, const float* __restrict__ head_decay, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, int rot_dims, float q_scale, float k_scale, float* __restrict__ state,
    const int64_t* __restrict__ slots, const int32_t* __restrict__ cu, const int32_t* __restrict__ q_start, int heads,
    int dim, int vdim, int silu_inputs) {
  constexpr int DP = DS_SLICES * R;
  __shared__ float qs[TILE][DP], ks[TILE][DP], as[TILE][DP], vs[TILE][DS_COLS];
  __shared__ float partial[TILE][DS_SLICES][DS_COLS];
  const int e = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * DS_COLS;
  const int first = cu[e], n = cu[e + 1] - first;
  if (n <= 0) return;
  const int j = threadIdx.x % DS_COLS, s = threadIdx.x / DS_COLS;
  const bool col_ok = v0 + j < vdim;
  float* st = state + ((slots[e] * heads + h) * (int64_t)dim) * vdim + v0 + j;
  float S[R];
  const int start = q_start[e];
  const bool fresh = start == 0;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = s + DS_SLICES * r;
    S[r] = (!fresh && col_ok && i < dim) ? st[(int64_t)i * vdim] : 0.f;
  }
  const int hd = heads * dim, half = rot_dims / 2;
  const float hdec = head_decay ? head_decay[h] : 0.f;
  // A thread's share of a tile's q, k and a (PER elements each) and one v: asked for a tile ahead, into registers, so
  // that the way to memory runs beside the walk over the tile before.
  constexpr int PER = TILE * DP / DS_THREADS;
  float rq[PER], rk[PER], ra[PER], rv;
  // q, k and v as the recurrence reads them: the projection's numbers, or their silu
  auto act = [&](float z) { return silu_inputs ? z / (1.0f + expf(-z)) : z; };
  // without a rotation, the activation (and the scales behind it) waits until a tile is stored to LDS: the fetch runs a tile
  // ahead, and nothing in it should use what its loads bring
  const bool late = silu_inputs && rot_dims == 0;
  auto fetch = [&](int t0) {
    const int nt = min(TILE, n - t0);
#pragma unroll
    for (int x = 0; x < PER; ++x) {
      const int idx = threadIdx.x + x * DS_THREADS;
      const int tt = idx / DP, i = idx % DP;
      float qv = 0.f, kv = 0.f, a = 0.f;
      if (tt < nt && i < dim) {
        const int64_t row = first + t0 + tt;
        const float* qp = q + row * stride + h * dim;
        const float* kp = k + row * stride + h * dim;
        qv = late ? qp[i] : act(qp[i]);
        kv = late ? kp[i] : act(kp[i]);
        if (i < rot_dims) {
          const int f = i < half ? i : i - half, other = i < half ? i + half : i - half;
          const int64_t at = (int64_t)(start + t0 + tt) * half + f;
          const float c = cos_t[at], sn = sin_t[at];
          const float qo = act(qp[other]), ko = act(kp[other]);
          // the pair (lo, hi) becomes (lo c - hi s, hi c + lo s)
          qv = i < half ? qv * c - qo * sn : qv * c + qo * sn;
          kv = i < half ? kv * c - ko * sn : kv * c + ko * sn;
        }
        if (!late) {
          qv *= q_scale;
          kv *= k_scale;
        }
        a = decay ? decay[row * hd + h * dim + i] : hdec;
      }
      rq[x] = qv;
      rk[x] = kv;
      ra[x] = a;
    }
    const int tt = threadIdx.x / DS_COLS, jj = threadIdx.x % DS_COLS;      // 16 * DS_COLS == DS_THREADS
    rv = (tt < nt && v0 + jj < vdim) ? v[(int64_t)(first + t0 + tt) * stride + h * vdim + v0 + jj] : 0.f;
  };
  fetch(0);
  for (int t0 = 0; t0 < n; t0 += TILE) {
    const int nt = min(TILE, n - t0);
    __syncthreads();                                   // the tile before is read out
#pragma unroll
    for (int x = 0; x < PER; ++x) {
      const int idx = threadIdx.x + x * DS_THREADS;
      qs[idx / DP][idx % DP] = late ? act(rq[x]) * q_scale : rq[x];
      ks[idx / DP][idx % DP] = late ? act(rk[x]) * k_scale : rk[x];
      as[idx / DP][idx % DP] = ra[x];
    }
    {
      const int tt = threadIdx.x / DS_COLS, jj = threadIdx.x % DS_COLS;
      if (tt < TILE) vs[tt][jj] = act(rv);
    }
    __syncthreads();
    if (t0 + TILE < n) fetch(t0 + TILE);
    for (int tt = 0; tt < nt; ++tt) {
      const float vv = vs[tt][j];
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int i = s + DS_SLICES * r;
        S[r] = as[tt][i] * S[r] + ks[tt][i] * vv;
        acc += S[r] * qs[tt][i];
      }
      partial[tt][s][j] = acc;
    }
    __syncthreads();
    {
      const int tt = threadIdx.x / DS_COLS, jj = threadIdx.x % DS_COLS;
      if (tt < nt && v0 + jj < vdim) {
        float o = 0.f;
#pragma unroll
        for (int p = 0; p < DS_SLICES; ++p) o += partial[tt][p][jj];
        out[((int64_t)(first + t0 + tt) * heads + h) * vdim + v0 + jj] = o;
      }
    }
  }
  if (col_ok) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int i = s + DS_SLICES * r;
      if (i < dim) st[(int64_t)i * vdim] = S[r];
    }
  }
}

// decay[t, c] = exp(-softplus(-z) / tau), z = sum_r a2t[r, c] * low[t, r] + bias[c], the sum in ascending r.  a2t is the
// widening matrix TRANSPOSED, [rank][channels]: neighbouring threads read neighbouring channels.  A workgroup takes GD_TOKENS
// tokens and 256 channels; the tokens' narrow rows go through LDS and every element of a2t is read once for all of them.
#define GD_TOKENS 16
#define GD_BATCH 32
__global__ __launch_bounds__(256) void gla_decay_kernel(float* __restrict__ decay, const float* __restrict__ low,
                                                        int64_t low_stride, const float* __restrict__ a2t,
                                                        const float* __restrict__ bias, int tokens, int channels, int rank,
                                                        float inv_tau) {
  extern __shared__ float lows[];                      // [rank][GD_TOKENS]
  const int t0 = blockIdx.x * GD_TOKENS, nt = min(GD_TOKENS, tokens - t0);
  for (int idx = threadIdx.x; idx < GD_TOKENS * rank; idx += 256) {
    const int tt = idx / rank, r = idx % rank;
    lows[r * GD_TOKENS + tt] = tt < nt ? low[(int64_t)(t0 + tt) * low_stride + r] : 0.f;
  }
  __syncthreads();
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= channels) return;
  float z[GD_TOKENS];
#pragma unroll
  for (int tt = 0; tt < GD_TOKENS; ++tt) z[tt] = 0.f;
  for (int r0 = 0; r0 < rank; r0 += GD_BATCH) {        // GD_BATCH elements of a2t are asked for at a time: in a decode step
    float w[GD_BATCH];                                 // every one comes from memory, a microsecond away
#pragma unroll
    for (int j = 0; j < GD_BATCH; ++j) w[j] = r0 + j < rank ? a2t[(int64_t)(r0 + j) * channels + c] : 0.f;
#pragma unroll
    for (int j = 0; j < GD_BATCH; ++j) {
      if (r0 + j < rank) {
        const float* lo = lows + (r0 + j) * GD_TOKENS;
#pragma unroll
        for (int tt = 0; tt < GD_TOKENS; ++tt) z[tt] = fmaf(w[j], lo[tt], z[tt]);
      }
    }
  }
  const float b = bias[c];
#pragma unroll
  for (int tt = 0; tt < GD_TOKENS; ++tt) {
    if (tt < nt) {
      const float v = z[tt] + b;
      // log(sigmoid(v)) = -softplus(-v); far out the softplus is its argument
      const float sp = -v > 30.f ? -v : log1pf(expf(-v));
      decay[(int64_t)(t0 + tt) * channels + c] = expf(-sp * inv_tau);
    }
  }
}

// one wavefront per (token, head)
template <typename T>
__global__ __launch_bounds__(DS_THREADS) void head_norm_gate_kernel(T* __restrict__ out, const float* __restrict__ x,
                                                                     const float* __restrict__ weight,
                                                                     const float* __restrict__ gate, int64_t gate_stride,
                                                                     int64_t rows, int heads, int vdim, float eps,
                                                                     int sigmoid_gate) {
  const int64_t row = (int64_t)blockIdx.x * (DS_THREADS / WAVE) + threadIdx.x / WAVE;
  if (row >= rows) return;
  const int lane = threadIdx.x % WAVE;
  const int64_t t = row / heads;
  const int h = (int)(row - t * heads);
  const float* p = x + row * vdim;
  float ss = 0.f;
  for (int i = lane; i < vdim; i += WAVE) ss += p[i] * p[i];
  ss = wave_sum(ss);
  const float rms = sqrtf(ss / (float)vdim + eps);
  const float* g = gate ? gate + t * gate_stride + (int64_t)h * vdim : nullptr;
  for (int i = lane; i < vdim; i += WAVE) {
    float y = p[i] / rms;
    if (weight) y *= weight[i];
    if (g) {
      const float z = g[i];
      y *= (sigmoid_gate ? 1.0f : z) / (1.0f + expf(-z));
    }
    Num<T>::st(out + row * vdim + i, y);
  }
}

// the same for rows as wide as all heads together (a norm over the whole row): a workgroup a row
template <typename T>
__global__ __launch_bounds__(DS_THREADS) void wide_norm_gate_kernel(T* __restrict__ out, const float* __restrict__ x,
                                                                     const float* __restrict__ weight,
                                                                     const float* __restrict__ gate, int64_t gate_stride,
                                                                     int width, float eps, int sigmoid_gate) {
  __shared__ float scratch[DS_THREADS / WAVE];
  const int64_t t = blockIdx.x;
  const float* p = x + t * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += DS_THREADS) ss = fmaf(p[i], p[i], ss);
  ss = block_sum<DS_THREADS / WAVE>(ss, scratch);
  const float rms = sqrtf(ss / (float)width + eps);
  const float* g = gate ? gate + t * gate_stride : nullptr;
  for (int i = threadIdx.x; i < width; i += DS_THREADS) {
    float y = p[i] / rms;
    if (weight) y *= weight[i];
    if (g) {
      const float z = g[i];
      y *= (sigmoid_gate ? 1.0f : z) / (1.0f + expf(-z));
    }
    Num<T>::st(out + t * width + i, y);
  }
}

// the same for rows of a multiple of 4 up to DS_THREADS * 4 * PER elements: four consecutive elements a thread and access, all
// of a row's operands asked for before the first is used; the sum of squares in the order of the kernel above (the same bits)
template <typename T, int PER>
__global__ __launch_bounds__(DS_THREADS) void wide_norm_gate_rows_kernel(T* __restrict__ out, const float* __restrict__ x,
                                                                          const float* __restrict__ weight,
                                                                          const float* __restrict__ gate, int64_t gate_stride,
                                                                          int width, float eps, int sigmoid_gate) {
  __shared__ float scratch[DS_THREADS / WAVE];
  const int64_t t = blockIdx.x;
  float4 xv[PER], wv[PER], gv[PER];
#pragma unroll
  for (int p = 0; p < PER; ++p) {
    const int i = 4 * (threadIdx.x + p * DS_THREADS);
    if (i < width) {
      xv[p] = *reinterpret_cast<const float4*>(x + t * width + i);
      if (weight) wv[p] = *reinterpret_cast<const float4*>(weight + i);
      if (gate) gv[p] = *reinterpret_cast<const float4*>(gate + t * gate_stride + i);
    }
  }
  // a thread of the kernel above adds the squares of elements tid, tid + 256, ...; here it holds other elements, so the
  // partial sums differ: rows of these widths always come here, never there
  float ss = 0.f;
#pragma unroll
  for (int p = 0; p < PER; ++p) {
    const int i = 4 * (threadIdx.x + p * DS_THREADS);
    if (i < width) {
      ss = fmaf(xv[p].x, xv[p].x, ss);
      ss = fmaf(xv[p].y, xv[p].y, ss);
      ss = fmaf(xv[p].z, xv[p].z, ss);
      ss = fmaf(xv[p].w, xv[p].w, ss);
    }
  }
  ss = block_sum<DS_THREADS / WAVE>(ss, scratch);
  const float rms = sqrtf(ss / (float)width + eps);
#pragma unroll
  for (int p = 0; p < PER; ++p) {
    const int i = 4 * (threadIdx.x + p * DS_THREADS);
    if (i < width) {
      float e[4] = {xv[p].x, xv[p].y, xv[p].z, xv[p].w};
      const float w4[4] = {wv[p].x, wv[p].y, wv[p].z, wv[p].w};
      const float g4[4] = {gv[p].x, gv[p].y, gv[p].z, gv[p].w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        float y = e[k] / rms;
        if (weight) y *= w4[k];
        if (gate) y *= (sigmoid_gate ? 1.0f : g4[k]) / (1.0f + expf(-g4[k]));
        Num<T>::st(out + t * width + i + k, y);
      }
    }
  }
}

extern "C" int ga_decay_scan(void* out, const void* q, const void* k, const void* v, int64_t stride, const void* decay,
                             const void* head_decay, const void* cos_t, const void* sin_t, int rot_dims, float q_scale,
                             float k_scale, void* state, const void* slots, const void* cu, const void* q_start, int entries,
                             int heads, int dim, int vdim, int silu_inputs, hipStream_t stream) {
  if (entries <= 0) return 0;
  if (heads <= 0 || dim <= 0 || vdim <= 0 || dim > 16 * DS_SLICES) return -1;
  if (heads > 65535 || (vdim + DS_COLS - 1) / DS_COLS > 65535) return -2;
  if ((decay == nullptr) == (head_decay == nullptr)) return -3;
  if (rot_dims < 0 || rot_dims % 2 || rot_dims > dim || (rot_dims > 0 && (!cos_t || !sin_t))) return -4;
  dim3 grid(entries, heads, (vdim + DS_COLS - 1) / DS_COLS), block(DS_THREADS);
  const int rows = (dim + DS_SLICES - 1) / DS_SLICES;
#define GO(R, T) hipLaunchKernelGGL((decay_scan_kernel<R, T>), grid, block, 0, stream, (float*)out, (const float*)q, (const float*)k, \
                                 (const float*)v, stride, (const float*)decay, (const float*)head_decay, (const float*)cos_t,  \
                                 (const float*)sin_t, rot_dims, q_scale, k_scale, (float*)state, (const int64_t*)slots,       \
                                 (const int32_t*)cu, (const int32_t*)q_start, heads, dim, vdim, silu_inputs)
  if (rows <= 1) GO(1, 16);
  else if (rows <= 2) GO(2, 16);
  else if (rows <= 3) GO(3, 16);
  else if (rows <= 4) GO(4, 16);
  else if (rows <= 6) GO(6, 16);
  else if (rows <= 8) GO(8, 16);
  else if (rows <= 12) GO(12, 16);
  else GO(16, 8);      // the widest heads take half the tokens a trip: the tile's operands fill the LDS
#undef GO
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_gla_decay(void* decay, const void* low, int64_t low_stride, const void* a2t, const void* bias, int tokens,
                            int channels, int rank, float tau, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (channels <= 0 || rank <= 0 || !(tau > 0.f)) return -1;
  if ((size_t)GD_TOKENS * rank * sizeof(float) > 48 * 1024) return -2;
  dim3 grid((tokens + GD_TOKENS - 1) / GD_TOKENS, (channels + 255) / 256);
  hipLaunchKernelGGL(gla_decay_kernel, grid, dim3(256), GD_TOKENS * rank * sizeof(float), stream, (float*)decay,
                     (const float*)low, low_stride, (const float*)a2t, (const float*)bias, tokens, channels, rank, 1.0f / tau);
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_head_norm_gate(void* out, const void* x, const void* weight, const void* gate, int64_t gate_stride,
                                 int64_t tokens, int heads, int vdim, float eps, int out_bf16, int sigmoid_gate,
                                 hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (vdim <= 0 || heads <= 0) return -1;
  if (heads == 1 && vdim >= 512 && vdim % 4 == 0 && vdim <= DS_THREADS * 16 && tokens < (1ll << 31) && gate_stride % 4 == 0 &&
      (((uintptr_t)x | (uintptr_t)weight | (uintptr_t)gate) & 15) == 0) {
#define GW(T, PER) hipLaunchKernelGGL((wide_norm_gate_rows_kernel<T, PER>), dim3((unsigned)tokens), dim3(DS_THREADS), 0, stream,  \
                                      (T*)out, (const float*)x, (const float*)weight, (const float*)gate, gate_stride, vdim, eps, \
                                      sigmoid_gate)
#define GT(T) do { if (vdim <= DS_THREADS * 4) GW(T, 1); else if (vdim <= DS_THREADS * 8) GW(T, 2); else GW(T, 4); } while (0)
    if (out_bf16) GT(bf16_t); else GT(float);
#undef GT
#undef GW
    return GA_CHECK_LAUNCH();
  }
  if (heads == 1 && vdim >= 512 && tokens < (1ll << 31)) {          // a row of a wavefront's 64 lanes would be a long walk
    if (out_bf16)
      hipLaunchKernelGGL(wide_norm_gate_kernel<bf16_t>, dim3((unsigned)tokens), dim3(DS_THREADS), 0, stream, (bf16_t*)out,
                         (const float*)x, (const float*)weight, (const float*)gate, gate_stride, vdim, eps, sigmoid_gate);
    else
      hipLaunchKernelGGL(wide_norm_gate_kernel<float>, dim3((unsigned)tokens), dim3(DS_THREADS), 0, stream, (float*)out,
                         (const float*)x, (const float*)weight, (const float*)gate, gate_stride, vdim, eps, sigmoid_gate);
    return GA_CHECK_LAUNCH();
  }
  const int64_t rows = tokens * heads;
  const int per = DS_THREADS / WAVE;
  dim3 grid((unsigned)((rows + per - 1) / per)), block(DS_THREADS);
  if (out_bf16)
    hipLaunchKernelGGL(head_norm_gate_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)out, (const float*)x,
                       (const float*)weight, (const float*)gate, gate_stride, rows, heads, vdim, eps, sigmoid_gate);
  else
    hipLaunchKernelGGL(head_norm_gate_kernel<float>, grid, block, 0, stream, (float*)out, (const float*)x,
                       (const float*)weight, (const float*)gate, gate_stride, rows, heads, vdim, eps, sigmoid_gate);
  return GA_CHECK_LAUNCH();
}
