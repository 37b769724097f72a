// What mixers and feed-forwards of further makes need around their projections, in float32
// arithmetic for both storage types:
//
//   mk_qk_prepare      queries and keys between projection and cache: norms over the whole
//                      projection or over every head, a temperature that grows with the
//                      position, rotation of a head's first dims, the queries out, keys and
//                      values into the paged cache (the values may be the keys as projected, or
//                      mixed with the values an earlier layer left for the same tokens);
//   mk_unary_act       an activation of one operand (the square of relu, the tanh form of gelu);
//   mk_gate_mul        a sigmoid gate, column by column, on a mixer's output;
//   mk_stream_cast     the residual stream itself as a sublayer's input;
//   mk_normed_sum      h += mult * (rmsnorm(a) * wa + rmsnorm(b) * wb): mixers side by side;
//   mk_norm_scale_add  h += scale .* (rmsnorm(y) * w): a sublayer's output normed before it
//                      enters the stream, times a stored vector per channel; the new stream
//                      may go out once more in the compute dtype, for a sublayer that reads it;
//   mk_diff_heads      two attention maps per head combined, normed per head and gated;
//   mk_concat_cast     [a | b] row by row, in the compute dtype (the operand of a projection
//                      of two streams);
//   mk_copy_f32        a copy by a kernel (a captured graph records no memcpy node here).
#include <algorithm>

#include "common.h"
#include "mercury_kernels.h"

namespace {

template <typename TW>
__device__ __forceinline__ float weight_at(const void* w, int i) {
  return Elem<TW>::load((const TW*)w + i);
}

// One workgroup per token, or several that share its outputs.  The row of qkv is
// [q: n_q d | k: n_kv d | v: n_kv dv], the last part absent when the values are the keys.
#define QK_MAX_NORMED_HEADS 1024
template <typename T, typename TW>
__global__ __launch_bounds__(256) void qk_prepare_kernel(
    const float* __restrict__ qkv, int row_stride, T* __restrict__ q_out,
    const void* __restrict__ q_norm, const void* __restrict__ k_norm, float eps, float temp_coef,
    int temp_every, const float* __restrict__ cos_table, const float* __restrict__ sin_table,
    int rot, int interleaved, const int* __restrict__ positions,
    const int* __restrict__ token_seq, const int* __restrict__ block_table, int table_stride,
    T* __restrict__ k_cache, T* __restrict__ v_cache, int page_shift, int n_q, int n_kv, int d,
    int dv, int values_are_keys, int write_kv, int maps, int head_norm,
    float* __restrict__ v_carry, int v_mode, float v_lambda) {
  __shared__ float scratch[16];
  __shared__ float head_mult[QK_MAX_NORMED_HEADS];
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int half = rot / 2;
  const float* cs = cos_table + (size_t)pos * half;
  const float* sn = sin_table + (size_t)pos * half;
  const float* row = qkv + (size_t)t * row_stride;
  const int qw = n_q * d, kw = n_kv * d;
  const float* k_src = row + qw;

  float q_mult = 1.f, k_mult = 1.f;
  if (head_norm) {
    // a norm per head: the wavefronts take the heads of q, then of k, in turn
    const int lane = threadIdx.x & (MK_WAVE - 1);
    const int normed = n_q + (write_kv ? n_kv : 0);
    for (int head = threadIdx.x / MK_WAVE; head < normed; head += blockDim.x / MK_WAVE) {
      const float* src = row + (size_t)head * d;
      float sq = 0.f;
      for (int i = lane; i < d; i += MK_WAVE) sq += src[i] * src[i];
      sq = wave_sum(sq);
      if (lane == 0) head_mult[head] = rsqrtf(sq / (float)d + eps);
    }
    __syncthreads();
  } else if (q_norm) {
    float sq = 0.f;
    for (int i = threadIdx.x; i < qw; i += blockDim.x) sq += row[i] * row[i];
    q_mult = rsqrtf(block_sum(sq, scratch) / (float)qw + eps);
  }
  if (k_norm && write_kv && !head_norm) {
    float sq = 0.f;
    for (int i = threadIdx.x; i < kw; i += blockDim.x) sq += k_src[i] * k_src[i];
    k_mult = rsqrtf(block_sum(sq, scratch) / (float)kw + eps);
  }
  if (temp_every > 0) {
    q_mult *= 1.f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.f);
  }

  // the value of entry i of q (of k) before it turns
  auto q_at = [&](int i) {
    if (head_norm) return row[i] * head_mult[i / d] * q_mult * weight_at<TW>(q_norm, i % d);
    const float v = row[i] * q_mult;
    return q_norm ? v * weight_at<TW>(q_norm, i) : v;
  };
  auto k_at = [&](int i) {
    if (head_norm) return k_src[i] * head_mult[n_q + i / d] * weight_at<TW>(k_norm, i % d);
    const float v = k_src[i] * k_mult;
    return k_norm ? v * weight_at<TW>(k_norm, i) : v;
  };
  // entry j of a head after the turn: the partner is j ^ 1 (interleaved) or j -+ half; a head
  // of several score maps turns each map's first dims by itself
  const int map_dims = d / maps;
  auto turned = [&](auto at, int base, int j) {
    if (maps > 1) {
      const int map = j / map_dims;
      base += map * map_dims;
      j -= map * map_dims;
    }
    if (j >= rot) return at(base + j);
    if (interleaved) {
      const int pair = j >> 1;
      return (j & 1) ? at(base + j) * cs[pair] + at(base + j - 1) * sn[pair]
                     : at(base + j) * cs[pair] - at(base + j + 1) * sn[pair];
    }
    return j < half ? at(base + j) * cs[j] - at(base + j + half) * sn[j]
                    : at(base + j) * cs[j - half] + at(base + j - half) * sn[j - half];
  };

  // The outputs [q | k | v] are dealt over the workgroups of the token (blockIdx.y): with few
  // tokens each thread has one or two of them, and every workgroup has made the sums above
  // for itself.
  const int page_size = 1 << page_shift;
  const int page = write_kv ? block_table[(size_t)token_seq[t] * table_stride + (pos >> page_shift)] : -1;
  const int off = pos & (page_size - 1);
  // (the host never schedules a write into a page that was given back: page < 0 writes nothing)
  const int vw = n_kv * dv;
  const int qo = qw * maps;      // queries out: one per (head, map), a key row wide
  const int total = qo + (write_kv && page >= 0 ? kw + vw : 0);
  const float* v_src = values_are_keys ? k_src : k_src + kw;
  for (int idx = blockIdx.y * blockDim.x + threadIdx.x; idx < total; idx += gridDim.y * blockDim.x) {
    if (idx < qo) {
      const int query = idx / d, j = idx - query * d;
      const int head = query / maps, map = query - head * maps;
      const bool mine = maps == 1 || j / map_dims == map;
      Elem<T>::store(q_out + (size_t)t * qo + idx, mine ? turned(q_at, head * d, j) : 0.f);
    } else if (idx < qo + kw) {
      const int i = idx - qo;
      const int head = i / d, j = i - head * d;
      const size_t dst = (((size_t)page * n_kv + head) * page_size + off) * d + j;
      Elem<T>::store(k_cache + dst, turned(k_at, head * d, j));
    } else {
      const int i = idx - qo - kw;
      const int head = i / dv, j = i - head * dv;
      float value = v_src[i];
      // values mixed across layers: the first layer leaves its own, a later one blends them in
      if (v_mode == MK_VMIX_LEAVE) v_carry[(size_t)t * vw + i] = value;
      else if (v_mode == MK_VMIX_BLEND) value = (1.f - v_lambda) * value + v_lambda * v_carry[(size_t)t * vw + i];
      Elem<T>::store(v_cache + (((size_t)page * n_kv + head) * dv + j) * page_size + off, value);
    }
  }
}

template <typename TI, typename T>
__global__ void unary_act_kernel(const TI* __restrict__ x, T* __restrict__ out, long long n,
                                 int kind) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float v = Elem<TI>::load(x + i);
  float y = v;
  if (kind == MK_UNARY_RELU2) {
    const float r = fmaxf(v, 0.f);
    y = r * r;
  } else if (kind == MK_UNARY_GELU_TANH) {
    y = 0.5f * v * (1.f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
  }
  Elem<T>::store(out + i, y);
}

// A token's workgroups (blockIdx.y of them) each make the two rows' sums of squares for
// themselves, in the same order, and then write their own share of the weighted sum: with few
// tokens the row is spread over the chip, with many a token has one workgroup.
template <typename TW>
__global__ __launch_bounds__(256) void normed_sum_kernel(
    float* __restrict__ h, const float* __restrict__ ya, const float* __restrict__ pa, int na,
    const void* __restrict__ wa, const float* __restrict__ yb, const float* __restrict__ pb,
    int nb, const void* __restrict__ wb, float eps, float mult, size_t stride, int hidden) {
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * hidden;
  auto value = [&](const float* y, const float* p, int n, int i) {
    float v = y ? y[base + i] : 0.f;
    for (int k = 0; k < n; ++k) v += p[(size_t)k * stride + base + i];
    return v;
  };
  const bool has_b = yb != nullptr || nb > 0;
  float sa = 0.f, sb = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float a = value(ya, pa, na, i);
    sa += a * a;
    if (has_b) {
      const float b = value(yb, pb, nb, i);
      sb += b * b;
    }
  }
  const float ra = rsqrtf(block_sum(sa, scratch) / (float)hidden + eps);
  const float rb = has_b ? rsqrtf(block_sum(sb, scratch) / (float)hidden + eps) : 0.f;
  for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < hidden; i += gridDim.y * blockDim.x) {
    float sum = value(ya, pa, na, i) * ra * weight_at<TW>(wa, i);
    if (has_b) sum += value(yb, pb, nb, i) * rb * weight_at<TW>(wb, i);
    h[base + i] += mult * sum;
  }
}

// One workgroup per token (or several that share its outputs, each making the sum of squares
// for itself in the same order).
template <typename TW, typename TX>
__global__ __launch_bounds__(256) void norm_scale_add_kernel(
    float* __restrict__ h, const float* __restrict__ y, const float* __restrict__ partials,
    int count, size_t stride, const void* __restrict__ weight, const float* __restrict__ scale,
    float eps, int hidden, TX* __restrict__ x_out) {
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * hidden;
  auto value = [&](int i) {
    float v = y ? y[base + i] : 0.f;
    for (int k = 0; k < count; ++k) v += partials[(size_t)k * stride + base + i];
    return v;
  };
  float sq = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = value(i);
    sq += v * v;
  }
  const float r = rsqrtf(block_sum(sq, scratch) / (float)hidden + eps);
  for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < hidden; i += gridDim.y * blockDim.x) {
    const float normed = value(i) * r * weight_at<TW>(weight, i);
    const float sum = h[base + i] + (scale ? scale[i] * normed : normed);
    h[base + i] = sum;
    if (x_out) Elem<TX>::store(x_out + base + i, sum);
  }
}

// The same for rows of at most 256 NV entries, one workgroup per token: a thread keeps its
// entries in registers between the sum of squares and the output, and the partial sums of an
// entry are read side by side (in the same order of addition).
#define NSA_NV 16
template <typename TW, int NV, typename TX>
__global__ __launch_bounds__(256) void norm_scale_add_held_kernel(
    float* __restrict__ h, const float* __restrict__ y, const float* __restrict__ partials,
    int count, size_t stride, const void* __restrict__ weight, const float* __restrict__ scale,
    float eps, int hidden, TX* __restrict__ x_out) {
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * hidden;
  float vals[NV];
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = threadIdx.x + j * 256;
    vals[j] = y && i < hidden ? y[base + i] : 0.f;
  }
  // 64 / NV partial sums of every entry are asked for at a time and added in their order
  constexpr int KB = 64 / NV;
  for (int k0 = 0; k0 < count; k0 += KB) {
    float got[KB][NV];
#pragma unroll
    for (int kk = 0; kk < KB; ++kk) {
      const float* part = partials + (size_t)min(k0 + kk, count - 1) * stride + base;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int i = threadIdx.x + j * 256;
        got[kk][j] = i < hidden ? part[i] : 0.f;
      }
    }
#pragma unroll
    for (int kk = 0; kk < KB; ++kk)
      if (k0 + kk < count) {
#pragma unroll
        for (int j = 0; j < NV; ++j) vals[j] += got[kk][j];
      }
  }
  float sq = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) sq += vals[j] * vals[j];
  const float r = rsqrtf(block_sum(sq, scratch) / (float)hidden + eps);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = threadIdx.x + j * 256;
    if (i < hidden) {
      const float normed = vals[j] * r * weight_at<TW>(weight, i);
      const float sum = h[base + i] + (scale ? scale[i] * normed : normed);
      h[base + i] = sum;
      if (x_out) Elem<TX>::store(x_out + base + i, sum);
    }
  }
}

// One wavefront per (token, head).
template <typename T>
__global__ __launch_bounds__(64) void diff_heads_kernel(
    const T* __restrict__ a, T* __restrict__ out, const float* __restrict__ gate, int gate_stride,
    float lambda, float eps, float out_scale, int heads, int dv) {
  const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const T* a1 = a + ((size_t)t * heads + head) * 2 * dv;
  const T* a2 = a1 + dv;
  float sq = 0.f;
  for (int i = lane; i < dv; i += MK_WAVE) {
    const float o = Elem<T>::load(a1 + i) - lambda * Elem<T>::load(a2 + i);
    sq += o * o;
  }
  float mult = rsqrtf(wave_sum(sq) / (float)dv + eps) * out_scale;
  if (gate) mult *= 1.f / (1.f + expf(-gate[(size_t)t * gate_stride + head]));
  for (int i = lane; i < dv; i += MK_WAVE) {
    const float o = Elem<T>::load(a1 + i) - lambda * Elem<T>::load(a2 + i);
    Elem<T>::store(out + ((size_t)t * heads + head) * dv + i, o * mult);
  }
}

template <typename T>
__global__ void concat_cast_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                   T* __restrict__ out, int hidden) {
  const size_t t = blockIdx.x;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    Elem<T>::store(out + t * 2 * hidden + i, a[t * hidden + i]);
    Elem<T>::store(out + t * 2 * hidden + hidden + i, b[t * hidden + i]);
  }
}

__global__ void copy_f32_kernel(float* __restrict__ dst, const float* __restrict__ src,
                                long long n) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = src[i];
}

template <typename T>
__global__ void gate_mul_kernel(const T* __restrict__ a, const float* __restrict__ gate,
                                int gate_stride, T* __restrict__ out, int width, long long n) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const long long t = i / width;
  const float z = gate[t * gate_stride + (i - t * width)];
  Elem<T>::store(out + i, Elem<T>::load(a + i) / (1.f + expf(-z)));
}

// h += its partial sums, and the sum goes out in the compute dtype.
template <typename T>
__global__ void stream_cast_kernel(float* __restrict__ h, const float* __restrict__ partials,
                                   int count, size_t stride, T* __restrict__ out, long long n) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float v = h[i];
  if (count > 0) {
    for (int k = 0; k < count; ++k) v += partials[(size_t)k * stride + i];
    h[i] = v;
  }
  Elem<T>::store(out + i, v);
}

}  // namespace

extern "C" int mk_qk_prepare(const float* qkv, int row_stride, void* q_out, int dtype,
                             const void* q_norm, const void* k_norm, int norm_dtype, float eps,
                             float temp_coef, int temp_every, const float* cos_table,
                             const float* sin_table, int table_positions, int rot,
                             int interleaved, const int* positions, const int* token_seq,
                             const int* block_table, int table_stride, void* k_cache,
                             void* v_cache, int page_size, int n_q, int n_kv, int d, int dv,
                             int values_are_keys, int write_kv, int maps, int head_norm,
                             float* v_carry, int v_mode, float v_lambda, int tokens,
                             hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && n_q > 0 && n_kv >= 0 && d > 0 && dv > 0, "qk_prepare: bad sizes");
  MK_REQUIRE(!head_norm || (q_norm && (k_norm || !write_kv) && maps == 1),
             "qk_prepare: a norm per head needs its weights and one map a head");
  MK_REQUIRE(!head_norm || n_q + n_kv <= QK_MAX_NORMED_HEADS,
             "qk_prepare: %d heads to norm exceed the supported %d", n_q + n_kv, QK_MAX_NORMED_HEADS);
  MK_REQUIRE(v_mode == MK_VMIX_NONE || v_mode == MK_VMIX_LEAVE || v_mode == MK_VMIX_BLEND,
             "qk_prepare: unknown value mixing %d", v_mode);
  MK_REQUIRE(v_mode == MK_VMIX_NONE || (v_carry && write_kv && !values_are_keys),
             "qk_prepare: values mixed across layers need a buffer and a layer that writes its own");
  MK_REQUIRE(maps >= 1 && d % maps == 0, "qk_prepare: %d maps do not divide a head of %d", maps, d);
  MK_REQUIRE(rot >= 0 && rot <= d / maps && rot % 2 == 0,
             "qk_prepare: rotary width %d not in [0, %d] / even", rot, d / maps);
  MK_REQUIRE(maps == 1 || !interleaved, "qk_prepare: several maps turn in the half-split layout");
  MK_REQUIRE(rot == 0 || (table_positions > 0 && cos_table && sin_table),
             "qk_prepare: empty angle table");
  MK_REQUIRE(mk_is_pow2(page_size), "qk_prepare: page size %d is not a power of two", page_size);
  MK_REQUIRE(!values_are_keys || dv == d, "qk_prepare: values that are keys are as wide as keys");
  const int need = n_q * d + (write_kv ? n_kv * d + (values_are_keys ? 0 : n_kv * dv) : 0);
  MK_REQUIRE(row_stride >= need, "qk_prepare: row stride %d below the %d columns of q, k, v",
             row_stride, need);
  MK_REQUIRE((q_norm == nullptr) == (k_norm == nullptr) || !write_kv,
             "qk_prepare: a norm for queries and keys alike");
  MK_REQUIRE(temp_every >= 0, "qk_prepare: negative temperature period");
  MK_REQUIRE(!write_kv || (k_cache && v_cache && block_table), "qk_prepare: no cache to write");
  MK_REQUIRE(norm_dtype == MK_F32 || norm_dtype == MK_BF16, "qk_prepare: norm dtype %d", norm_dtype);
  if (tokens == 0) return 0;
  // few tokens: a token's outputs over several workgroups, so that the chip is not idle
  const int by_size = (need + n_q * d * (maps - 1) + 255) / 256;
  const int chunks = std::max(1, std::min(by_size, 1024 / tokens));
  const dim3 grid(tokens, chunks);
#define QK_LAUNCH(T, TW)                                                                         \
  qk_prepare_kernel<T, TW><<<grid, 256, 0, stream>>>(                                          \
      qkv, row_stride, (T*)q_out, q_norm, k_norm, eps, temp_coef, temp_every, cos_table,         \
      sin_table, rot, interleaved, positions, token_seq, block_table, table_stride, (T*)k_cache, \
      (T*)v_cache, mk_log2(page_size), n_q, n_kv, d, dv, values_are_keys, write_kv, maps,         \
      head_norm, v_carry, v_mode, v_lambda)
  if (dtype == MK_F32) {
    if (norm_dtype == MK_F32) QK_LAUNCH(float, float); else QK_LAUNCH(float, bf16_t);
  } else if (dtype == MK_BF16) {
    if (norm_dtype == MK_F32) QK_LAUNCH(bf16_t, float); else QK_LAUNCH(bf16_t, bf16_t);
  } else {
    MK_REQUIRE(false, "qk_prepare: unknown dtype %d", dtype);
  }
#undef QK_LAUNCH
  MK_LAUNCH_CHECK("qk_prepare");
  return 0;
}

extern "C" int mk_unary_act(const void* x, int in_dtype, void* out, int dtype, long long n,
                            int kind, hipStream_t stream) {
  MK_REQUIRE(n >= 0, "unary_act: negative count");
  MK_REQUIRE(kind == MK_UNARY_RELU2 || kind == MK_UNARY_GELU_TANH, "unary_act: unknown activation %d", kind);
  if (n == 0) return 0;
  const long long blocks = (n + 255) / 256;
  MK_REQUIRE(blocks < (1ll << 31), "unary_act: %lld elements are too many for one launch", n);
  if (in_dtype == MK_F32 && dtype == MK_F32)
    unary_act_kernel<float, float><<<(unsigned)blocks, 256, 0, stream>>>((const float*)x, (float*)out, n, kind);
  else if (in_dtype == MK_F32 && dtype == MK_BF16)
    unary_act_kernel<float, bf16_t><<<(unsigned)blocks, 256, 0, stream>>>((const float*)x, (bf16_t*)out, n, kind);
  else if (in_dtype == MK_BF16 && dtype == MK_BF16)
    unary_act_kernel<bf16_t, bf16_t><<<(unsigned)blocks, 256, 0, stream>>>((const bf16_t*)x, (bf16_t*)out, n, kind);
  else
    MK_REQUIRE(false, "unary_act: dtypes %d -> %d", in_dtype, dtype);
  MK_LAUNCH_CHECK("unary_act");
  return 0;
}

extern "C" int mk_normed_sum(float* h, const float* ya, const float* pa, int na, const void* wa,
                             const float* yb, const float* pb, int nb, const void* wb,
                             int weight_dtype, float eps, float mult, long long stride, int tokens,
                             int hidden, hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && hidden > 0, "normed_sum: bad sizes");
  MK_REQUIRE(na >= 0 && nb >= 0 && (na == 0 || pa) && (nb == 0 || pb),
             "normed_sum: partial sums without a buffer");
  MK_REQUIRE((ya || na) && wa, "normed_sum: no first operand");
  MK_REQUIRE(!(yb || nb) || wb, "normed_sum: a second operand without its weight");
  MK_REQUIRE(weight_dtype == MK_F32 || weight_dtype == MK_BF16, "normed_sum: weight dtype %d",
             weight_dtype);
  if (tokens == 0) return 0;
  const dim3 grid(tokens, std::max(1, std::min((hidden + 255) / 256, 512 / tokens)));
  if (weight_dtype == MK_F32)
    normed_sum_kernel<float><<<grid, 256, 0, stream>>>(h, ya, pa, na, wa, yb, pb, nb, wb, eps,
                                                          mult, (size_t)stride, hidden);
  else
    normed_sum_kernel<bf16_t><<<grid, 256, 0, stream>>>(h, ya, pa, na, wa, yb, pb, nb, wb, eps,
                                                           mult, (size_t)stride, hidden);
  MK_LAUNCH_CHECK("normed_sum");
  return 0;
}

extern "C" int mk_norm_scale_add(float* h, const float* y, const float* partials, int count,
                                 long long stride, const void* weight, int weight_dtype,
                                 const float* scale, float eps, int tokens, int hidden,
                                 void* x_out, int x_dtype, hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && hidden > 0, "norm_scale_add: bad sizes");
  MK_REQUIRE(!x_out || x_dtype == MK_F32 || x_dtype == MK_BF16, "norm_scale_add: x dtype %d", x_dtype);
  const bool x_bf16 = x_out && x_dtype == MK_BF16;
  MK_REQUIRE(count >= 0 && (count == 0 || partials), "norm_scale_add: partial sums without a buffer");
  MK_REQUIRE((y || count) && weight && h, "norm_scale_add: no operand");
  MK_REQUIRE(weight_dtype == MK_F32 || weight_dtype == MK_BF16, "norm_scale_add: weight dtype %d",
             weight_dtype);
  if (tokens == 0) return 0;
  if (hidden <= 256 * NSA_NV) {
#define NSA_LAUNCH(TW, NV)                                                                  \
  do {                                                                                      \
    if (x_bf16)                                                                             \
      norm_scale_add_held_kernel<TW, NV, bf16_t><<<tokens, 256, 0, stream>>>(               \
          h, y, partials, count, (size_t)stride, weight, scale, eps, hidden, (bf16_t*)x_out); \
    else                                                                                    \
      norm_scale_add_held_kernel<TW, NV, float><<<tokens, 256, 0, stream>>>(                \
          h, y, partials, count, (size_t)stride, weight, scale, eps, hidden, (float*)x_out); \
  } while (0)
    if (weight_dtype == MK_F32) {
      if (hidden <= 256 * 4) NSA_LAUNCH(float, 4);
      else if (hidden <= 256 * 8) NSA_LAUNCH(float, 8);
      else NSA_LAUNCH(float, NSA_NV);
    } else {
      if (hidden <= 256 * 4) NSA_LAUNCH(bf16_t, 4);
      else if (hidden <= 256 * 8) NSA_LAUNCH(bf16_t, 8);
      else NSA_LAUNCH(bf16_t, NSA_NV);
    }
#undef NSA_LAUNCH
    MK_LAUNCH_CHECK("norm_scale_add");
    return 0;
  }
  const dim3 grid(tokens, std::max(1, std::min((hidden + 255) / 256, 512 / tokens)));
#define NSA_WIDE(TW)                                                                           \
  do {                                                                                         \
    if (x_bf16)                                                                                \
      norm_scale_add_kernel<TW, bf16_t><<<grid, 256, 0, stream>>>(                             \
          h, y, partials, count, (size_t)stride, weight, scale, eps, hidden, (bf16_t*)x_out);  \
    else                                                                                       \
      norm_scale_add_kernel<TW, float><<<grid, 256, 0, stream>>>(                              \
          h, y, partials, count, (size_t)stride, weight, scale, eps, hidden, (float*)x_out);   \
  } while (0)
  if (weight_dtype == MK_F32) NSA_WIDE(float);
  else NSA_WIDE(bf16_t);
#undef NSA_WIDE
  MK_LAUNCH_CHECK("norm_scale_add");
  return 0;
}

extern "C" int mk_diff_heads(const void* a, void* out, int dtype, const float* gate,
                             int gate_stride, float lambda, float eps, float out_scale, int tokens,
                             int heads, int dv, hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && heads > 0 && dv > 0, "diff_heads: bad sizes");
  MK_REQUIRE(heads <= 65535, "diff_heads: too many heads (%d)", heads);
  MK_REQUIRE(!gate || gate_stride >= heads, "diff_heads: gate rows of %d for %d heads", gate_stride, heads);
  if (tokens == 0) return 0;
  const dim3 grid(tokens, heads);
  if (dtype == MK_F32)
    diff_heads_kernel<float><<<grid, MK_WAVE, 0, stream>>>((const float*)a, (float*)out, gate,
                                                             gate_stride, lambda, eps, out_scale, heads, dv);
  else if (dtype == MK_BF16)
    diff_heads_kernel<bf16_t><<<grid, MK_WAVE, 0, stream>>>((const bf16_t*)a, (bf16_t*)out, gate,
                                                              gate_stride, lambda, eps, out_scale, heads, dv);
  else
    MK_REQUIRE(false, "diff_heads: unknown dtype %d", dtype);
  MK_LAUNCH_CHECK("diff_heads");
  return 0;
}

extern "C" int mk_concat_cast(const float* a, const float* b, void* out, int dtype, int tokens,
                              int hidden, hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && hidden > 0, "concat_cast: bad sizes");
  if (tokens == 0) return 0;
  if (dtype == MK_F32)
    concat_cast_kernel<float><<<tokens, 256, 0, stream>>>(a, b, (float*)out, hidden);
  else if (dtype == MK_BF16)
    concat_cast_kernel<bf16_t><<<tokens, 256, 0, stream>>>(a, b, (bf16_t*)out, hidden);
  else
    MK_REQUIRE(false, "concat_cast: unknown dtype %d", dtype);
  MK_LAUNCH_CHECK("concat_cast");
  return 0;
}

extern "C" int mk_copy_f32(float* dst, const float* src, long long n, hipStream_t stream) {
  MK_REQUIRE(n >= 0, "copy: negative count");
  if (n == 0) return 0;
  const long long blocks = (n + 255) / 256;
  MK_REQUIRE(blocks < (1ll << 31), "copy: %lld elements are too many for one launch", n);
  copy_f32_kernel<<<(unsigned)blocks, 256, 0, stream>>>(dst, src, n);
  MK_LAUNCH_CHECK("copy");
  return 0;
}

extern "C" int mk_gate_mul(const void* a, int dtype, const float* gate, int gate_stride, void* out,
                           int tokens, int width, hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && width > 0, "gate_mul: bad sizes");
  MK_REQUIRE(gate_stride >= width, "gate_mul: gate rows of %d for %d columns", gate_stride, width);
  if (tokens == 0) return 0;
  MK_REQUIRE(a && gate && out, "gate_mul: null operand");
  const long long n = (long long)tokens * width, blocks = (n + 255) / 256;
  MK_REQUIRE(blocks < (1ll << 31), "gate_mul: %lld elements are too many for one launch", n);
  if (dtype == MK_F32)
    gate_mul_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>((const float*)a, gate, gate_stride, (float*)out, width, n);
  else if (dtype == MK_BF16)
    gate_mul_kernel<bf16_t><<<(unsigned)blocks, 256, 0, stream>>>((const bf16_t*)a, gate, gate_stride, (bf16_t*)out, width, n);
  else
    MK_REQUIRE(false, "gate_mul: unknown dtype %d", dtype);
  MK_LAUNCH_CHECK("gate_mul");
  return 0;
}

extern "C" int mk_stream_cast(float* h, const float* partials, int count, long long stride,
                              void* out, int dtype, long long n, hipStream_t stream) {
  MK_REQUIRE(n >= 0 && count >= 0 && (count == 0 || partials), "stream_cast: bad operands");
  if (n == 0) return 0;
  MK_REQUIRE(h && out, "stream_cast: null operand");
  const long long blocks = (n + 255) / 256;
  MK_REQUIRE(blocks < (1ll << 31), "stream_cast: %lld elements are too many for one launch", n);
  if (dtype == MK_F32)
    stream_cast_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>(h, partials, count, (size_t)stride, (float*)out, n);
  else if (dtype == MK_BF16)
    stream_cast_kernel<bf16_t><<<(unsigned)blocks, 256, 0, stream>>>(h, partials, count, (size_t)stride, (bf16_t*)out, n);
  else
    MK_REQUIRE(false, "stream_cast: unknown dtype %d", dtype);
  MK_LAUNCH_CHECK("stream_cast");
  return 0;
}
