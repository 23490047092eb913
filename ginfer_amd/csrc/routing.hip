// Routing of tokens to experts, and the gated activation of many experts side by side.
//   route:   from router scores z [T, E] (32-bit) the `top` largest of every row (the lowest index among equals), their
//            weights = softmax over the chosen scores alone; written as lists (ids, weights [T, top]) and as a row of E
//            weights with zeros at the experts not chosen.
//   weighted gated activation:  act[t, c] = w(t, c) * silu(gate[t, c]) * up[t, c] over the columns of all experts laid
//            side by side (expert e owns columns [e * ff, (e + 1) * ff)); columns behind the experts' (a shared expert that
//            every token uses) have the weight 1.  In the product that it reads, every expert's gate columns are followed
//            by that expert's up columns, so that one expert's part of the stacked matrix is one piece.  The product with the stacked down matrices then IS the weighted sum
//            of the chosen experts' outputs: the others enter with exact zeros.
#include "common.h"
#include "ginfer_amd.h"

#define ROUTE_MAX_EXPERTS 256
#define ROUTE_THREADS 64

// one wavefront per token; experts dealt to lanes, ROUTE_MAX_EXPERTS / 64 each
__global__ __launch_bounds__(ROUTE_THREADS) void route_topk_kernel(const float* __restrict__ scores, int32_t* __restrict__ ids,
                                                                   float* __restrict__ weights, float* __restrict__ dense,
                                                                   int experts, int top) {
  constexpr int PER = ROUTE_MAX_EXPERTS / ROUTE_THREADS;
  __shared__ float chosen_s[ROUTE_MAX_EXPERTS];
  __shared__ int32_t chosen_i[ROUTE_MAX_EXPERTS];
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x;
  float z[PER];
  bool taken[PER];
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int e = lane + j * ROUTE_THREADS;
    z[j] = e < experts ? scores[t * experts + e] : -INFINITY;
    // a score that is no number (the rows that pad a recorded step may hold anything) counts as the smallest: with
    // it no comparison below would hold, the lanes would come to different winners, each strike out its own, and the
    // next round would find no expert left
    if (!(z[j] == z[j])) z[j] = -INFINITY;
    taken[j] = e >= experts;
  }
  for (int k = 0; k < top; ++k) {
    // this lane's best that is still free, then the best over the lanes; equal scores go to the lowest index
    float best = -INFINITY;
    int at = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = lane + j * ROUTE_THREADS;
      if (!taken[j] && (at == 0x7fffffff || z[j] > best)) { best = z[j]; at = e; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, WAVE);
      const int oa = __shfl_xor(at, o, WAVE);
      if (oa != 0x7fffffff && (at == 0x7fffffff || ob > best || (ob == best && oa < at))) { best = ob; at = oa; }
    }
#pragma unroll
    for (int j = 0; j < PER; ++j)
      if (lane + j * ROUTE_THREADS == at) taken[j] = true;
    if (lane == 0) { chosen_s[k] = best; chosen_i[k] = at < experts ? at : 0; }   // top <= experts: one is always left
  }
  __syncthreads();
  // softmax over the chosen scores; chosen_s[0] is the largest
  const float top_score = chosen_s[0];
  float total = 0.f;
  for (int k = 0; k < top; ++k) total += expf(chosen_s[k] - top_score);
  for (int e = lane; e < experts; e += ROUTE_THREADS) dense[t * experts + e] = 0.f;
  __syncthreads();
  for (int k = lane; k < top; k += ROUTE_THREADS) {
    const float w = expf(chosen_s[k] - top_score) / total;
    ids[t * top + k] = chosen_i[k];
    weights[t * top + k] = w;
    dense[t * experts + chosen_i[k]] = w;
  }
}

// Routing by sigmoid scores with a correction and groups of experts (one wavefront per token):
//   s = sigmoid(z);  c = s + correction (the choice score; without a correction c = s)
//   the experts fall into `groups` equal groups of neighbours; a group's score is the sum of its `group_top` largest c; only
//   the experts of the `keep` best groups can be chosen (groups == 1: all of them)
//   the `top` experts with the largest c among those are chosen (the lowest index among equals)
//   weights: the chosen experts' s, divided by their sum + floor where `normalise`, times `scale`
// Written as route_topk_kernel writes them: ids and weights [T, top], and a row of weights over all experts.
#define ROUTE_GROUP_TOP_MAX 4
__global__ __launch_bounds__(ROUTE_THREADS) void route_sigmoid_groups_kernel(
    const float* __restrict__ logits, const float* __restrict__ correction, int32_t* __restrict__ ids,
    float* __restrict__ weights, float* __restrict__ dense, int experts, int top, int groups, int keep, int group_top,
    int normalise, float floor, float scale) {
  constexpr int PER = ROUTE_MAX_EXPERTS / ROUTE_THREADS;
  __shared__ float choice[ROUTE_MAX_EXPERTS], plain[ROUTE_MAX_EXPERTS], group_score[ROUTE_MAX_EXPERTS];
  __shared__ int32_t kept[ROUTE_MAX_EXPERTS], chosen_i[ROUTE_MAX_EXPERTS];
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x;
  float c[PER];
  bool taken[PER];
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int e = lane + j * ROUTE_THREADS;
    float z = e < experts ? logits[t * experts + e] : 0.f;
    float s = 1.0f / (1.0f + expf(-z));
    c[j] = e < experts ? s + (correction ? correction[e] : 0.f) : -INFINITY;
    // what is no number (the rows that pad a recorded step may hold anything) counts as the smallest
    if (!(c[j] == c[j])) { c[j] = -INFINITY; s = 0.f; }
    taken[j] = e >= experts;
    if (e < experts) { choice[e] = c[j]; plain[e] = s; }
  }
  __syncthreads();
  if (groups > 1) {
    const int n = experts / groups;
    for (int g = lane; g < groups; g += ROUTE_THREADS) {
      float best[ROUTE_GROUP_TOP_MAX];
#pragma unroll
      for (int k = 0; k < ROUTE_GROUP_TOP_MAX; ++k) best[k] = -INFINITY;
      for (int i = 0; i < n; ++i) {
        float v = choice[g * n + i];
#pragma unroll
        for (int k = 0; k < ROUTE_GROUP_TOP_MAX; ++k)
          if (k < group_top && v > best[k]) { const float o = best[k]; best[k] = v; v = o; }
      }
      float sum = 0.f;
#pragma unroll
      for (int k = 0; k < ROUTE_GROUP_TOP_MAX; ++k)
        if (k < group_top && k < n) sum += best[k];
      group_score[g] = sum;
      kept[g] = 0;
    }
    __syncthreads();
    if (lane == 0) {
      for (int k = 0; k < keep; ++k) {
        int at = -1;
        float best = -INFINITY;
        for (int g = 0; g < groups; ++g)
          if (!kept[g] && (at < 0 || group_score[g] > best)) { best = group_score[g]; at = g; }
        if (at >= 0) kept[at] = 1;
      }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = lane + j * ROUTE_THREADS;
      if (e < experts && !kept[e / n]) { taken[j] = true; c[j] = -INFINITY; }
    }
  }
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = lane + j * ROUTE_THREADS;
      if (!taken[j] && (at == 0x7fffffff || c[j] > best)) { best = c[j]; at = e; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, WAVE);
      const int oa = __shfl_xor(at, o, WAVE);
      if (oa != 0x7fffffff && (at == 0x7fffffff || ob > best || (ob == best && oa < at))) { best = ob; at = oa; }
    }
#pragma unroll
    for (int j = 0; j < PER; ++j)
      if (lane + j * ROUTE_THREADS == at) taken[j] = true;
    if (lane == 0) chosen_i[k] = at < experts ? at : 0;       // top <= the experts that can be chosen: one is always left
  }
  __syncthreads();
  float total = 0.f;
  for (int k = 0; k < top; ++k) total += plain[chosen_i[k]];             // in the order of the choice
  const float factor = normalise ? scale / (total + floor) : scale;
  for (int e = lane; e < experts; e += ROUTE_THREADS) dense[t * experts + e] = 0.f;
  __syncthreads();
  for (int k = lane; k < top; k += ROUTE_THREADS) {
    const float w = plain[chosen_i[k]] * factor;
    ids[t * top + k] = chosen_i[k];
    weights[t * top + k] = w;
    dense[t * experts + chosen_i[k]] = w;
  }
}

// gate_up [tokens, 2 * width]: for every expert its ff gate columns and then its ff up columns, the experts one after the
// other, and behind them the shared expert's (shared gates, then shared ups); out [tokens, width]: expert e's columns at
// [e * ff, (e + 1) * ff), the shared expert's behind.  V elements a thread in 16-byte accesses where the widths allow it.
template <typename T, int V>
__global__ __launch_bounds__(256) void weighted_silu_mul_kernel(T* __restrict__ out, const T* __restrict__ gate_up,
                                                                const float* __restrict__ dense, int64_t chunks_total,
                                                                int width, int experts, int ff) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= chunks_total) return;
  const int chunks = width / V;
  const int64_t t = i / chunks;
  const int c = (int)(i - t * chunks) * V;             // first column of the chunk; a chunk lies inside one expert
  const int e = c / ff;
  const int shared = width - experts * ff;
  float w = 1.f;
  int gate_at, up_at;
  if (e < experts) {
    w = dense[t * experts + e];
    gate_at = e * 2 * ff + (c - e * ff);
    up_at = gate_at + ff;
  } else {
    gate_at = experts * 2 * ff + (c - experts * ff);
    up_at = gate_at + shared;
  }
  union Pack { uint4 u; T e[16 / sizeof(T)]; };
  Pack res;
  if (w == 0.f) {                              // an expert that the token does not use: exact zeros, whatever it holds
#pragma unroll
    for (int j = 0; j < V; ++j) Num<T>::st(res.e + j, 0.f);
  } else {
    const T* gp = gate_up + t * 2 * width + gate_at;
    const T* up = gate_up + t * 2 * width + up_at;
    Pack g, u;
    if (V > 1) {
      g.u = *reinterpret_cast<const uint4*>(gp);
      u.u = *reinterpret_cast<const uint4*>(up);
    } else {
      g.e[0] = gp[0];
      u.e[0] = up[0];
    }
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const float gv = Num<T>::ld(g.e + j), uv = Num<T>::ld(u.e + j);
      Num<T>::st(res.e + j, w * (gv / (1.f + expf(-gv)) * uv));
    }
  }
  if (V > 1) *reinterpret_cast<uint4*>(out + t * width + c) = res.u;
  else out[t * width + c] = res.e[0];
}

// Router scores: z[t, e] = w[e] . x[t] + b[e] in 32-bit (x in the compute dtype or float, w and b float).  A wavefront per
// (token, expert): every lane a slice of the row, the lanes' sums added in the butterfly's order, so a score does not
// depend on what else is in the step.  The choice is route_topk_kernel's, launched behind.
template <typename T>
__global__ __launch_bounds__(256) void router_scores_kernel(float* __restrict__ scores, const T* __restrict__ x,
                                                            const float* __restrict__ w, const float* __restrict__ b,
                                                            int64_t pairs, int hidden, int experts) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int64_t p = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (p >= pairs) return;
  const int64_t t = p / experts;
  const int e = (int)(p - t * experts);
  const T* row = x + t * hidden;
  const float* we = w + (int64_t)e * hidden;
  // four sums a lane, so that four pairs of loads are under way at a time; added in a fixed order
  float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
  int k = lane;
  for (; k + 3 * WAVE < hidden; k += 4 * WAVE) {
    const float w0 = we[k], w1 = we[k + WAVE], w2 = we[k + 2 * WAVE], w3 = we[k + 3 * WAVE];
    const float x0 = Num<T>::ld(row + k), x1 = Num<T>::ld(row + k + WAVE), x2 = Num<T>::ld(row + k + 2 * WAVE),
                x3 = Num<T>::ld(row + k + 3 * WAVE);
    a0 += w0 * x0;
    a1 += w1 * x1;
    a2 += w2 * x2;
    a3 += w3 * x3;
  }
  for (; k < hidden; k += WAVE) a0 += we[k] * Num<T>::ld(row + k);
  float acc = wave_sum((a0 + a1) + (a2 + a3));
  if (lane == 0) scores[p] = acc + (b ? b[e] : 0.f);
}

// Rows of the token-expert pairs, grouped by expert, for steps whose experts run one after the other over their own
// rows: ids int32 [pairs] (pair p = token p / top, its choice p % top) -> offsets int32 [experts + 1], pair_of_row and
// row_of_pair int32 [pairs].  One workgroup; the order inside an expert's rows is whatever the counters give (no row's
// result depends on the rows beside it).
#define SORT_THREADS 1024
__global__ __launch_bounds__(SORT_THREADS) void route_sort_kernel(const int32_t* __restrict__ ids, int32_t* __restrict__ offsets,
                                                                   int32_t* __restrict__ pair_of_row,
                                                                   int32_t* __restrict__ row_of_pair, int pairs, int experts) {
  __shared__ int32_t count[ROUTE_MAX_EXPERTS], first[ROUTE_MAX_EXPERTS + 1];
  for (int e = threadIdx.x; e < experts; e += SORT_THREADS) count[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += SORT_THREADS) atomicAdd(&count[ids[p]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < experts; ++e) {
      first[e] = at;
      at += count[e];
    }
    first[experts] = at;
  }
  __syncthreads();
  for (int e = threadIdx.x; e <= experts; e += SORT_THREADS) offsets[e] = first[e];
  for (int e = threadIdx.x; e < experts; e += SORT_THREADS) count[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += SORT_THREADS) {
    const int e = ids[p];
    const int r = first[e] + atomicAdd(&count[e], 1);
    pair_of_row[r] = p;
    row_of_pair[p] = r;
  }
}

// The rows that the experts' products read, every expert's group `capacity` rows long (what lies behind a group's own
// rows is never read back): row r of the grouped order, which belongs to expert ids[pair_of_row[r]], goes to
// sorted[e * capacity + (r - offsets[e])] = x[pair_of_row[r] / top].  V elements per 16 bytes.
template <typename T>
__global__ __launch_bounds__(256) void gather_pair_rows_kernel(T* __restrict__ sorted, const T* __restrict__ x,
                                                               const int32_t* __restrict__ pair_of_row,
                                                               const int32_t* __restrict__ ids, const int32_t* __restrict__ offsets,
                                                               int capacity, int hidden, int top) {
  constexpr int V = 16 / sizeof(T);
  const int64_t r = blockIdx.x;
  const int pair = pair_of_row[r];
  const int e = ids[pair];
  const T* src = x + (int64_t)(pair / top) * hidden;
  T* dst = sorted + ((int64_t)e * capacity + (r - offsets[e])) * hidden;
  if (hidden % V == 0) {
    for (int k = threadIdx.x * V; k < hidden; k += 256 * V)
      *reinterpret_cast<uint4*>(dst + k) = *reinterpret_cast<const uint4*>(src + k);
  } else {
    for (int k = threadIdx.x; k < hidden; k += 256) dst[k] = src[k];
  }
}

// out[t] = sum_j weights[t, j] * y[place of pair t * top + j] (+ shared[t]): the chosen experts' results added up in the
// order of the choice, in 32-bit; y holds every expert's group `capacity` rows long, as the gather above laid them
template <typename T>
__global__ __launch_bounds__(256) void combine_pairs_kernel(T* __restrict__ out, const T* __restrict__ y,
                                                            const T* __restrict__ shared, const float* __restrict__ weights,
                                                            const int32_t* __restrict__ row_of_pair,
                                                            const int32_t* __restrict__ ids, const int32_t* __restrict__ offsets,
                                                            int capacity, int hidden, int top) {
  const int64_t t = blockIdx.x;
  for (int k = threadIdx.x; k < hidden; k += 256) {
    float acc = 0.f;
    for (int j = 0; j < top; ++j) {
      const int e = ids[t * top + j];
      const int64_t at = (int64_t)e * capacity + (row_of_pair[t * top + j] - offsets[e]);
      acc += weights[t * top + j] * Num<T>::ld(y + at * hidden + k);
    }
    if (shared) acc += Num<T>::ld(shared + t * hidden + k);
    Num<T>::st(out + t * hidden + k, acc);
  }
}

extern "C" int ga_route_topk(void* ids, void* weights, void* dense, const void* scores, int tokens, int experts, int top,
                             hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (experts <= 0 || experts > ROUTE_MAX_EXPERTS || top <= 0 || top > experts) return -1;
  hipLaunchKernelGGL(route_topk_kernel, dim3(tokens), dim3(ROUTE_THREADS), 0, stream, (const float*)scores, (int32_t*)ids,
                     (float*)weights, (float*)dense, experts, top);
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_route_sigmoid_groups(void* ids, void* weights, void* dense, const void* logits, const void* correction,
                                       int tokens, int experts, int top, int groups, int keep, int group_top, int normalise,
                                       float floor, float scale, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (experts <= 0 || experts > ROUTE_MAX_EXPERTS || top <= 0 || top > experts) return -1;
  if (groups < 1 || experts % groups || keep < 1 || keep > groups || top > keep * (experts / groups)) return -2;
  if (group_top < 1 || group_top > ROUTE_GROUP_TOP_MAX) return -3;
  hipLaunchKernelGGL(route_sigmoid_groups_kernel, dim3(tokens), dim3(ROUTE_THREADS), 0, stream, (const float*)logits,
                     (const float*)correction, (int32_t*)ids, (float*)weights, (float*)dense, experts, top, groups, keep,
                     group_top, normalise, floor, scale);
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_weighted_silu_mul(void* out, const void* gate_up, const void* dense, int tokens, int width, int experts,
                                    int ff, int is_bf16, hipStream_t stream) {
  if (tokens <= 0 || width <= 0) return 0;
  if (experts < 0 || ff <= 0 || (int64_t)experts * ff > width) return -1;
  const int v = is_bf16 ? 8 : 4;
  const int shared = width - experts * ff;
  const bool wide = ff % v == 0 && shared % v == 0 && ((uintptr_t)out | (uintptr_t)gate_up) % 16 == 0;
  const int64_t total = (int64_t)tokens * (wide ? width / v : width);
  dim3 grid((unsigned)((total + 255) / 256)), block(256);
#define GO(T, V) hipLaunchKernelGGL((weighted_silu_mul_kernel<T, V>), grid, block, 0, stream, (T*)out, (const T*)gate_up, \
                                    (const float*)dense, total, width, experts, ff)
  if (is_bf16) { if (wide) GO(bf16_t, 8); else GO(bf16_t, 1); }
  else { if (wide) GO(float, 4); else GO(float, 1); }
#undef GO
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_router_max_experts() { return ROUTE_MAX_EXPERTS; }

extern "C" int ga_router_scores(void* scores, const void* x, const void* w, const void* b, int tokens, int hidden, int experts,
                                int x_bf16, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (hidden <= 0 || experts <= 0 || experts > ROUTE_MAX_EXPERTS) return -1;
  const int64_t pairs = (int64_t)tokens * experts;
  dim3 grid((unsigned)((pairs + 3) / 4)), block(256);
  if (x_bf16)
    hipLaunchKernelGGL(router_scores_kernel<bf16_t>, grid, block, 0, stream, (float*)scores, (const bf16_t*)x, (const float*)w,
                       (const float*)b, pairs, hidden, experts);
  else
    hipLaunchKernelGGL(router_scores_kernel<float>, grid, block, 0, stream, (float*)scores, (const float*)x, (const float*)w,
                       (const float*)b, pairs, hidden, experts);
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_route_sort(const void* ids, void* offsets, void* pair_of_row, void* row_of_pair, int pairs, int experts,
                             hipStream_t stream) {
  if (experts <= 0 || experts > ROUTE_MAX_EXPERTS || pairs < 0) return -1;
  hipLaunchKernelGGL(route_sort_kernel, dim3(1), dim3(SORT_THREADS), 0, stream, (const int32_t*)ids, (int32_t*)offsets,
                     (int32_t*)pair_of_row, (int32_t*)row_of_pair, pairs, experts);
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_gather_pair_rows(void* sorted, const void* x, const void* pair_of_row, const void* ids, const void* offsets,
                                   int capacity, int pairs, int hidden, int top, int is_bf16, hipStream_t stream) {
  if (pairs <= 0) return 0;
  if (hidden <= 0 || top <= 0 || capacity <= 0 || ((uintptr_t)sorted | (uintptr_t)x) % 16) return -1;
  if (is_bf16)
    hipLaunchKernelGGL(gather_pair_rows_kernel<bf16_t>, dim3(pairs), dim3(256), 0, stream, (bf16_t*)sorted, (const bf16_t*)x,
                       (const int32_t*)pair_of_row, (const int32_t*)ids, (const int32_t*)offsets, capacity, hidden, top);
  else
    hipLaunchKernelGGL(gather_pair_rows_kernel<float>, dim3(pairs), dim3(256), 0, stream, (float*)sorted, (const float*)x,
                       (const int32_t*)pair_of_row, (const int32_t*)ids, (const int32_t*)offsets, capacity, hidden, top);
  return GA_CHECK_LAUNCH();
}

extern "C" int ga_combine_pairs(void* out, const void* y, const void* shared, const void* weights, const void* row_of_pair,
                                const void* ids, const void* offsets, int capacity, int tokens, int hidden, int top, int is_bf16,
                                hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (hidden <= 0 || top <= 0 || capacity <= 0) return -1;
  if (is_bf16)
    hipLaunchKernelGGL(combine_pairs_kernel<bf16_t>, dim3(tokens), dim3(256), 0, stream, (bf16_t*)out, (const bf16_t*)y,
                       (const bf16_t*)shared, (const float*)weights, (const int32_t*)row_of_pair, (const int32_t*)ids,
                       (const int32_t*)offsets, capacity, hidden, top);
  else
    hipLaunchKernelGGL(combine_pairs_kernel<float>, dim3(tokens), dim3(256), 0, stream, (float*)out, (const float*)y,
                       (const float*)shared, (const float*)weights, (const int32_t*)row_of_pair, (const int32_t*)ids,
                       (const int32_t*)offsets, capacity, hidden, top);
  return GA_CHECK_LAUNCH();
}
