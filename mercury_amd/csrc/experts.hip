// Routed experts, a gate activation with constants, and the scaled residual sum, in float32
// arithmetic.
//
//   mk_route_topk     softmax over a token's router logits (float32), the `top` largest
//                     scores (ties: the lower index), their weights score * scale, divided by
//                     the chosen scores' sum when `renormalize`.
//   mk_expert_gated   act[(t, j), :] = gate_act(Wg[e] x_t, Wu[e] x_t) for e = the j-th expert
//                     of token t: one row of activations per (token, chosen expert).
//   mk_expert_down    y[t, :] += sum_j weight[t, j] * Wd[e_j] act[(t, j), :], j in ascending
//                     order, so a token's sum is the same whatever else is in the batch.
//   mk_gate_act       the activation alone on [gate | up] rows.
//   mk_scaled_add     h += mult * (y + partial sums): the residual sum of a layer whose
//                     sublayers' outputs are scaled before they enter the stream.
//
// Gate activations (MK_ACT_*): SILU is round(silu(g)) * u as the SiLU-gated projection
// computes it; SWISH_CLAMP is g' * sigmoid(alpha * g') * (u' + beta) with g' = min(g, limit),
// u' = clamp(u, -limit, limit); GELU_TANH is 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))) * u.
//
//   mk_row_gate       act[t, :] *= sigmoid(x[t, :] . w): a feed-forward gated by one number a
//                     token.
#include "common.h"
#include "mercury_kernels.h"

template <typename T>
__device__ __forceinline__ float gate_act(float g, float u, int kind, float limit, float alpha,
                                          float beta) {
  if (kind == MK_ACT_SILU) return Elem<T>::round(g / (1.f + expf(-g))) * u;
  if (kind == MK_ACT_GELU_TANH) {
    const float inner = 0.7978845608028654f * (g + 0.044715f * g * g * g);
    return 0.5f * g * (1.f + tanhf(inner)) * u;
  }
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.f + expf(-alpha * g)) * (u + beta);
}

// ---------------------------------------------------------------------------------- routing

#define ROUTE_MAX_PER_LANE 16

__global__ __launch_bounds__(64) void route_topk_kernel(const float* __restrict__ logits,
                                                        int experts, int top, float scale,
                                                        int renormalize, int* __restrict__ ids,
                                                        float* __restrict__ weights) {
  const int t = blockIdx.x, lane = threadIdx.x;
  const float* z = logits + (size_t)t * experts;
  float s[ROUTE_MAX_PER_LANE];
  float m = -INFINITY;
#pragma unroll
  for (int c = 0; c < ROUTE_MAX_PER_LANE; ++c) {
    const int e = lane + c * MK_WAVE;
    s[c] = e < experts ? z[e] : -INFINITY;
    m = fmaxf(m, s[c]);
  }
  m = wave_max(m);
  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < ROUTE_MAX_PER_LANE; ++c) {
    const int e = lane + c * MK_WAVE;
    s[c] = e < experts ? expf(s[c] - m) : -1.f;   // taken or absent: below every score
    sum += e < experts ? s[c] : 0.f;
  }
  sum = wave_sum(sum);
  float chosen_sum = 0.f;
  float mine_w = 0.f;
  int mine_id = 0;
  for (int j = 0; j < top; ++j) {
    float best = -1.f;
    int best_e = 0x7fffffff;
#pragma unroll
    for (int c = 0; c < ROUTE_MAX_PER_LANE; ++c) {
      const int e = lane + c * MK_WAVE;
      if (s[c] > best) {   // ascending e within a lane: the first of equals stays
        best = s[c];
        best_e = e;
      }
    }
#pragma unroll
    for (int w = MK_WAVE / 2; w > 0; w >>= 1) {
      const float other = __shfl_xor(best, w, MK_WAVE);
      const int other_e = __shfl_xor(best_e, w, MK_WAVE);
      if (other > best || (other == best && other_e < best_e)) {
        best = other;
        best_e = other_e;
      }
    }
#pragma unroll
    for (int c = 0; c < ROUTE_MAX_PER_LANE; ++c)
      if (lane + c * MK_WAVE == best_e) s[c] = -1.f;
    const float score = best / sum;
    chosen_sum += score;
    if (lane == j) {
      mine_w = score;
      mine_id = best_e;
    }
  }
  if (lane < top) {
    ids[(size_t)t * top + lane] = mine_id;
    weights[(size_t)t * top + lane] = (renormalize ? mine_w / chosen_sum : mine_w) * scale;
  }
}

extern "C" int mk_route_topk(const float* logits, int experts, int top, float scale,
                             int renormalize, int* ids, float* weights, int tokens,
                             hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && experts > 0 && top > 0 && top <= experts, "route: bad sizes E=%d top=%d",
             experts, top);
  MK_REQUIRE(experts <= MK_WAVE * ROUTE_MAX_PER_LANE, "route: %d experts exceed the supported %d",
             experts, MK_WAVE * ROUTE_MAX_PER_LANE);
  MK_REQUIRE(top <= MK_WAVE, "route: top %d exceeds %d", top, MK_WAVE);
  if (tokens == 0) return 0;
  route_topk_kernel<<<tokens, MK_WAVE, 0, stream>>>(logits, experts, top, scale, renormalize, ids,
                                                    weights);
  MK_LAUNCH_CHECK("route_topk");
  return 0;
}

// Pairs grouped by expert, by one workgroup: a histogram in LDS, its prefix sums, and every
// pair placed at its expert's cursor.  The order within an expert is whatever the atomics
// give; nothing downstream depends on it (each pair's result goes to the pair's own row).
#define GROUP_MAX_EXPERTS 1024

__global__ __launch_bounds__(1024) void route_group_kernel(const int* __restrict__ ids, int pairs,
                                                           int experts, int* __restrict__ rows,
                                                           int* __restrict__ offsets) {
  __shared__ int counts[GROUP_MAX_EXPERTS];
  __shared__ int cursor[GROUP_MAX_EXPERTS];
  for (int e = threadIdx.x; e < experts; e += blockDim.x) counts[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) atomicAdd(&counts[ids[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < experts; ++e) {
      offsets[e] = at;
      cursor[e] = at;
      at += counts[e];
    }
    offsets[experts] = at;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) rows[atomicAdd(&cursor[ids[i]], 1)] = i;
}

extern "C" int mk_route_group(const int* ids, int pairs, int experts, int* rows, int* offsets,
                              hipStream_t stream) {
  MK_REQUIRE(pairs >= 0 && experts > 0 && experts <= GROUP_MAX_EXPERTS, "route_group: bad sizes");
  route_group_kernel<<<1, 1024, 0, stream>>>(ids, pairs, experts, rows, offsets);
  MK_LAUNCH_CHECK("route_group");
  return 0;
}

__global__ void expert_combine_kernel(const float* __restrict__ pairs_out, float* __restrict__ y,
                                      int top, int N, size_t total) {
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / N;
    const int n = (int)(idx - t * N);
    float v = 0.f;
    for (int j = 0; j < top; ++j) v += pairs_out[(t * top + j) * N + n];
    y[idx] += v;
  }
}

extern "C" int mk_expert_combine(const float* pairs_out, float* y, int tokens, int top, int N,
                                 hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && top > 0 && N > 0, "expert_combine: bad sizes");
  if (tokens == 0) return 0;
  const size_t total = (size_t)tokens * N;
  size_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  expert_combine_kernel<<<(int)blocks, 256, 0, stream>>>(pairs_out, y, top, N, total);
  MK_LAUNCH_CHECK("expert_combine");
  return 0;
}

// ------------------------------------------------------------------- experts, token by token

#define EXPERT_ROWS_PER_WAVE 4

// grid (tokens * top, ceil(ff / 16)); x [T, K]; w [E, 2 ff, K] = [gate | up]; act [T * top, ff].
template <typename T>
__global__ __launch_bounds__(256) void expert_gated_kernel(
    const T* __restrict__ x, const T* __restrict__ w, const int* __restrict__ ids,
    T* __restrict__ act, int top, int ff, int K, int kind, float limit, float alpha, float beta) {
  extern __shared__ float xs[];
  const int row = blockIdx.x, t = row / top;
  const T* xr = x + (size_t)t * K;
  for (int i = threadIdx.x; i < K; i += blockDim.x) xs[i] = Elem<T>::load(xr + i);
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* we = w + (size_t)ids[row] * 2 * ff * K;
#pragma unroll
  for (int r = 0; r < EXPERT_ROWS_PER_WAVE; ++r) {
    const int n = (blockIdx.y * 4 + wave) * EXPERT_ROWS_PER_WAVE + r;
    if (n >= ff) break;   // uniform within the wavefront
    const T* wg = we + (size_t)n * K;
    const T* wu = we + (size_t)(ff + n) * K;
    float g = 0.f, u = 0.f;
    for (int i = lane; i < K; i += MK_WAVE) {
      g = fmaf(xs[i], Elem<T>::load(wg + i), g);
      u = fmaf(xs[i], Elem<T>::load(wu + i), u);
    }
    g = wave_sum(g);
    u = wave_sum(u);
    if (lane == 0)
      Elem<T>::store(act + (size_t)row * ff + n, gate_act<T>(g, u, kind, limit, alpha, beta));
  }
}

// grid (tokens, ceil(N / 16)); act [T * top, ff]; w [E, N, ff]; y [T, N] float32, added into.
template <typename T>
__global__ __launch_bounds__(256) void expert_down_kernel(
    const T* __restrict__ act, const T* __restrict__ w, const int* __restrict__ ids,
    const float* __restrict__ weights, float* __restrict__ y, int top, int ff, int N) {
  extern __shared__ float as[];   // one row of the token's activations at a time
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float total[EXPERT_ROWS_PER_WAVE];
#pragma unroll
  for (int r = 0; r < EXPERT_ROWS_PER_WAVE; ++r) total[r] = 0.f;
  for (int j = 0; j < top; ++j) {
    const T* ar = act + ((size_t)t * top + j) * ff;
    __syncthreads();
    for (int i = threadIdx.x; i < ff; i += blockDim.x) as[i] = Elem<T>::load(ar + i);
    __syncthreads();
    const float weight = weights[(size_t)t * top + j];
    const T* we = w + (size_t)ids[(size_t)t * top + j] * N * ff;
#pragma unroll
    for (int r = 0; r < EXPERT_ROWS_PER_WAVE; ++r) {
      const int n = (blockIdx.y * 4 + wave) * EXPERT_ROWS_PER_WAVE + r;
      if (n >= N) break;
      const T* wr = we + (size_t)n * ff;
      float dot = 0.f;
      for (int i = lane; i < ff; i += MK_WAVE) dot = fmaf(as[i], Elem<T>::load(wr + i), dot);
      total[r] = fmaf(weight, wave_sum(dot), total[r]);
    }
  }
#pragma unroll
  for (int r = 0; r < EXPERT_ROWS_PER_WAVE; ++r) {
    const int n = (blockIdx.y * 4 + wave) * EXPERT_ROWS_PER_WAVE + r;
    if (n < N && lane == 0) y[(size_t)t * N + n] += total[r];
  }
}

extern "C" int mk_expert_gated(const void* x, const void* w, int dtype, const int* ids, void* act,
                               int tokens, int top, int ff, int K, int kind, float limit,
                               float alpha, float beta, hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && top > 0 && ff > 0 && K > 0, "expert_gated: bad sizes");
  MK_REQUIRE(kind == MK_ACT_SILU || kind == MK_ACT_SWISH_CLAMP || kind == MK_ACT_GELU_TANH,
             "expert_gated: activation %d", kind);
  MK_REQUIRE((size_t)K * 4 <= 64 * 1024, "expert_gated: rows of %d are too wide", K);
  MK_REQUIRE((long long)tokens * top < (1ll << 31), "expert_gated: too many rows");
  if (tokens == 0) return 0;
  const int per_block = 4 * EXPERT_ROWS_PER_WAVE;
  dim3 grid(tokens * top, (ff + per_block - 1) / per_block);
  MK_REQUIRE(grid.y <= 65535, "expert_gated: ff=%d too large for one launch", ff);
  if (dtype == MK_F32)
    expert_gated_kernel<float><<<grid, 256, (size_t)K * 4, stream>>>(
        (const float*)x, (const float*)w, ids, (float*)act, top, ff, K, kind, limit, alpha, beta);
  else if (dtype == MK_BF16)
    expert_gated_kernel<bf16_t><<<grid, 256, (size_t)K * 4, stream>>>(
        (const bf16_t*)x, (const bf16_t*)w, ids, (bf16_t*)act, top, ff, K, kind, limit, alpha, beta);
  else
    MK_REQUIRE(false, "expert_gated: unknown dtype %d", dtype);
  MK_LAUNCH_CHECK("expert_gated");
  return 0;
}

extern "C" int mk_expert_down(const void* act, const void* w, int dtype, const int* ids,
                              const float* weights, float* y, int tokens, int top, int ff, int N,
                              hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && top > 0 && ff > 0 && N > 0, "expert_down: bad sizes");
  MK_REQUIRE((size_t)ff * 4 <= 64 * 1024, "expert_down: rows of %d are too wide", ff);
  if (tokens == 0) return 0;
  const int per_block = 4 * EXPERT_ROWS_PER_WAVE;
  dim3 grid(tokens, (N + per_block - 1) / per_block);
  MK_REQUIRE(grid.y <= 65535, "expert_down: N=%d too large for one launch", N);
  const size_t lds = (size_t)ff * 4;
  if (dtype == MK_F32)
    expert_down_kernel<float><<<grid, 256, lds, stream>>>((const float*)act, (const float*)w, ids,
                                                          weights, y, top, ff, N);
  else if (dtype == MK_BF16)
    expert_down_kernel<bf16_t><<<grid, 256, lds, stream>>>((const bf16_t*)act, (const bf16_t*)w,
                                                           ids, weights, y, top, ff, N);
  else
    MK_REQUIRE(false, "expert_down: unknown dtype %d", dtype);
  MK_LAUNCH_CHECK("expert_down");
  return 0;
}

// ------------------------------------------------------------------ the activation by itself

template <typename T>
__global__ void gate_act_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int inter,
                                size_t total, int kind, float limit, float alpha, float beta) {
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / inter;
    const int i = (int)(idx - t * inter);
    const T* row = gate_up + t * 2 * (size_t)inter;
    Elem<T>::store(out + idx, gate_act<T>(Elem<T>::load(row + i), Elem<T>::load(row + inter + i),
                                          kind, limit, alpha, beta));
  }
}

extern "C" int mk_gate_act(const void* gate_up, void* out, int dtype, int tokens, int inter,
                           int kind, float limit, float alpha, float beta, hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && inter > 0, "gate_act: bad sizes T=%d I=%d", tokens, inter);
  MK_REQUIRE(kind == MK_ACT_SILU || kind == MK_ACT_SWISH_CLAMP || kind == MK_ACT_GELU_TANH,
             "gate_act: activation %d", kind);
  if (tokens == 0) return 0;
  const size_t total = (size_t)tokens * inter;
  size_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  if (dtype == MK_F32)
    gate_act_kernel<float><<<(int)blocks, 256, 0, stream>>>((const float*)gate_up, (float*)out,
                                                            inter, total, kind, limit, alpha, beta);
  else if (dtype == MK_BF16)
    gate_act_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>((const bf16_t*)gate_up, (bf16_t*)out,
                                                             inter, total, kind, limit, alpha, beta);
  else
    MK_REQUIRE(false, "gate_act: unknown dtype %d", dtype);
  MK_LAUNCH_CHECK("gate_act");
  return 0;
}

// ------------------------------------------------------------------- the scaled residual sum

// h[i] += mult * (y[i] + sum_k a[k * stride + i] + sum_k b[k * stride + i]), the partial sums
// in ascending k, a before b.  y may be null.
__global__ void scaled_add_kernel(float* __restrict__ h, const float* __restrict__ y,
                                  const float* __restrict__ a, int na, const float* __restrict__ b,
                                  int nb, size_t stride, float mult, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x) {
    float v = y ? y[i] : 0.f;
    for (int k = 0; k < na; ++k) v += a[(size_t)k * stride + i];
    for (int k = 0; k < nb; ++k) v += b[(size_t)k * stride + i];
    h[i] = fmaf(mult, v, h[i]);
  }
}

extern "C" int mk_scaled_add(float* h, const float* y, const float* a, int na, const float* b,
                             int nb, long long stride, float mult, long long n,
                             hipStream_t stream) {
  MK_REQUIRE(n >= 0 && na >= 0 && nb >= 0 && stride >= 0, "scaled_add: bad sizes");
  MK_REQUIRE((na == 0 || a) && (nb == 0 || b), "scaled_add: partial sums without a buffer");
  if (n == 0) return 0;
  long long blocks = (n + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  scaled_add_kernel<<<(int)blocks, 256, 0, stream>>>(h, y, a, na, b, nb, (size_t)stride, mult,
                                                     (size_t)n);
  MK_LAUNCH_CHECK("scaled_add");
  return 0;
}

__global__ void fill_zero_kernel(float* __restrict__ p, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x)
    p[i] = 0.f;
}

// A fill by a kernel, so that a step captured into a graph records no memset node.
extern "C" int mk_fill_zero(float* p, long long n, hipStream_t stream) {
  MK_REQUIRE(n >= 0, "fill_zero: negative count");
  if (n == 0) return 0;
  long long blocks = (n + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  fill_zero_kernel<<<(int)blocks, 256, 0, stream>>>(p, (size_t)n);
  MK_LAUNCH_CHECK("fill_zero");
  return 0;
}

// One workgroup per token: the dot product in float32, then the row scaled in place.
template <typename T>
__global__ __launch_bounds__(256) void row_gate_kernel(T* __restrict__ act, const T* __restrict__ x,
                                                       const T* __restrict__ w, int inter,
                                                       int hidden) {
  __shared__ float scratch[16];
  const size_t t = blockIdx.x;
  float dot = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x)
    dot = fmaf(Elem<T>::load(x + t * hidden + i), Elem<T>::load(w + i), dot);
  const float gate = 1.f / (1.f + expf(-block_sum(dot, scratch)));
  for (int i = threadIdx.x; i < inter; i += blockDim.x)
    Elem<T>::store(act + t * inter + i, Elem<T>::load(act + t * inter + i) * gate);
}

extern "C" int mk_row_gate(void* act, const void* x, const void* w, int dtype, int tokens,
                           int inter, int hidden, hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && inter > 0 && hidden > 0, "row_gate: bad sizes");
  if (tokens == 0) return 0;
  if (dtype == MK_F32)
    row_gate_kernel<float><<<tokens, 256, 0, stream>>>((float*)act, (const float*)x, (const float*)w, inter, hidden);
  else if (dtype == MK_BF16)
    row_gate_kernel<bf16_t><<<tokens, 256, 0, stream>>>((bf16_t*)act, (const bf16_t*)x, (const bf16_t*)w, inter, hidden);
  else
    MK_REQUIRE(false, "row_gate: unknown dtype %d", dtype);
  MK_LAUNCH_CHECK("row_gate");
  return 0;
}
