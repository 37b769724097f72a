// Many small products in one launch on the matrix cores (bfloat16 in, float32 accumulate):
// y_b = x_b W_b^T for b < batch, x_b rows `lda` apart at x + b * x_batch, W_b [N, K] at
// w + b * w_batch, y_b rows `ldo` apart at out + b * o_batch.  What a mixer with a matrix of
// its own per head needs (x[t, head, :] W[head]^T), and, with a list of rows per product, what
// routed experts need (every expert's matrix over the tokens routed to it).
//
// A wavefront computes one or four tiles of 16 rows of x against 64 rows of W: W is the A
// operand (a lane holds 8 consecutive k of one row of W), x^T the B operand, so a lane ends up
// with four consecutive outputs of a row of x, and the row tiles share every piece of W the
// wavefront loads.  Operands go from memory straight into the products; the matrices are
// small enough (a head's, an expert's) to stay in the caches across the workgroups.
// K must be a multiple of 8 (a lane's 16 bytes); a last chunk of K short of 32 is padded with
// zeros in registers.
//
// Row lists (experts): product b takes the rows rows[offsets[b] .. offsets[b + 1]) instead of
// all M; entry i names source row rows[i] / gather_div of x and destination row rows[i] of
// out.  EPI_GATED: W_b is [gate rows | up rows] of N each and the output is the activation
// MK_ACT_* of the two; EPI_SCALED: the float32 output row is multiplied by row_scale[rows[i]].
#include "common.h"
#include "mercury_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

union BFrag {
  bf16x8 v;
  uint4 u;
};

enum { BEPI_BF16 = 0, BEPI_GATED = 1, BEPI_SCALED_F32 = 2 };

struct BatchedParams {
  const bf16_t* x;
  const bf16_t* w;
  void* out;
  int M, N, K, lda, ldo;
  long long x_batch, w_batch, o_batch;
  const int* rows;       // null: rows 0 .. M - 1 of every product
  const int* offsets;    // [batch + 1] into rows
  int gather_div;
  const float* row_scale;
  int act_kind;
  float limit, alpha, beta;
};

__device__ __forceinline__ float batched_act(float g, float u, const BatchedParams& p) {
  if (p.act_kind == MK_ACT_SILU) {
    const float s = g / (1.f + __expf(-g));
    return bf16_to_f32(f32_to_bf16(s)) * u;
  }
  if (p.act_kind == MK_ACT_GELU_TANH) {
    const float z = 0.7978845608028654f * (g + 0.044715f * g * g * g);
    return g / (1.f + __expf(-2.f * z)) * u;
  }
  g = fminf(g, p.limit);
  u = fminf(fmaxf(u, -p.limit), p.limit);
  return g / (1.f + __expf(-p.alpha * g)) * (u + p.beta);
}

// grid (ceil(N / 256), row tiles, batch); wavefront w of a workgroup takes 64 rows of W and
// RT tiles of 16 rows of x, which share every piece of W it loads (RT = 1 where a product has
// few rows: decoding).
template <int EPI, int RT>
__global__ __launch_bounds__(256) void gemm_batched_kernel(BatchedParams p) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g4 = lane >> 4;
  const int b = blockIdx.z;
  const int n0 = (blockIdx.x * 4 + wave) * 64;
  if (n0 >= p.N) return;
  int first = 0, count = p.M;
  if (p.rows) {
    first = p.offsets[b];
    count = p.offsets[b + 1] - first;
  }
  const int m0 = blockIdx.y * 16 * RT;
  if (m0 >= count) return;
  int dst_row[RT];
  const bf16_t* xr[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    const int mine = min(m0 + t * 16 + r, count - 1);
    dst_row[t] = p.rows ? p.rows[first + mine] : mine;
    const int src_row = p.rows ? dst_row[t] / p.gather_div : mine;
    xr[t] = p.x + (size_t)b * p.x_batch + (size_t)src_row * p.lda + g4 * 8;
  }
  const bf16_t* wb = p.w + (size_t)b * p.w_batch;
  constexpr int SETS = EPI == BEPI_GATED ? 2 : 1;   // gate rows and up rows
  const bf16_t* wr[SETS][4];
#pragma unroll
  for (int s = 0; s < SETS; ++s)
#pragma unroll
    for (int t = 0; t < 4; ++t)
      wr[s][t] = wb + (size_t)(s * p.N + min(n0 + t * 16 + r, p.N - 1)) * p.K + g4 * 8;
  f32x4 acc[SETS][4][RT];
#pragma unroll
  for (int s = 0; s < SETS; ++s)
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int u = 0; u < RT; ++u) acc[s][t][u] = (f32x4){0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < p.K; k0 += 32) {
    const bool live = k0 + g4 * 8 < p.K;   // K is a multiple of 8: a lane's chunk is whole or absent
    BFrag xf[RT];
#pragma unroll
    for (int u = 0; u < RT; ++u) xf[u].u = live ? *(const uint4*)(xr[u] + k0) : make_uint4(0, 0, 0, 0);
    BFrag wf[SETS][4];
#pragma unroll
    for (int s = 0; s < SETS; ++s)
#pragma unroll
      for (int t = 0; t < 4; ++t)
        wf[s][t].u = live ? *(const uint4*)(wr[s][t] + k0) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int s = 0; s < SETS; ++s)
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int u = 0; u < RT; ++u)
          acc[s][t][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[s][t].v, xf[u].v, acc[s][t][u], 0, 0, 0);
  }
  // the lane holds outputs n0 + t * 16 + g4 * 4 + i of its rows
#pragma unroll
  for (int u = 0; u < RT; ++u) {
    if (m0 + u * 16 + r >= count) continue;
    if (EPI == BEPI_SCALED_F32) {
      float* dst = (float*)p.out + (size_t)b * p.o_batch + (size_t)dst_row[u] * p.ldo;
      const float scale = p.row_scale ? p.row_scale[dst_row[u]] : 1.f;
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int n = n0 + t * 16 + g4 * 4 + i;
          if (n < p.N) dst[n] = acc[0][t][u][i] * scale;
        }
      continue;
    }
    bf16_t* dst = (bf16_t*)p.out + (size_t)b * p.o_batch + (size_t)dst_row[u] * p.ldo;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + t * 16 + g4 * 4 + i;
        if (n >= p.N) continue;
        const float v = EPI == BEPI_GATED ? batched_act(acc[0][t][u][i], acc[SETS - 1][t][u][i], p)
                                          : acc[0][t][u][i];
        dst[n] = f32_to_bf16(v);
      }
  }
}

// Row tiles per wavefront: four where a product has enough rows to fill them.
template <int EPI>
static void launch_batched(const BatchedParams& p, int max_rows, int batch, hipStream_t stream) {
  if (max_rows > 32) {
    dim3 grid((p.N + 255) / 256, (max_rows + 63) / 64, batch);
    gemm_batched_kernel<EPI, 4><<<grid, 256, 0, stream>>>(p);
  } else {
    dim3 grid((p.N + 255) / 256, (max_rows + 15) / 16, batch);
    gemm_batched_kernel<EPI, 1><<<grid, 256, 0, stream>>>(p);
  }
}

static int batched_check(const BatchedParams& p, int batch, int max_tiles) {
  MK_REQUIRE(p.N > 0 && p.K > 0 && batch > 0 && p.M >= 0, "batched product: bad sizes");
  MK_REQUIRE(p.K % 8 == 0 && p.lda % 8 == 0 && p.x_batch % 8 == 0 && p.w_batch % 8 == 0,
             "batched product: K=%d, lda=%d and the offsets must be multiples of 8", p.K, p.lda);
  MK_REQUIRE(((uintptr_t)p.x & 15) == 0 && ((uintptr_t)p.w & 15) == 0,
             "batched product: operands must be 16-byte aligned");
  MK_REQUIRE(batch <= 65535 && max_tiles <= 65535, "batched product: too large for one launch");
  return 0;
}

extern "C" int mk_linear_batched_mfma(const void* x, const void* w, void* out, int M, int N, int K,
                                      int lda, int ldo, int batch, long long x_batch,
                                      long long w_batch, long long o_batch, hipStream_t stream) {
  BatchedParams p = {};
  p.x = (const bf16_t*)x;
  p.w = (const bf16_t*)w;
  p.out = out;
  p.M = M; p.N = N; p.K = K; p.lda = lda; p.ldo = ldo;
  p.x_batch = x_batch; p.w_batch = w_batch; p.o_batch = o_batch;
  p.gather_div = 1;
  const int tiles = (M + 15) / 16;
  if (batched_check(p, batch, tiles)) return 1;
  MK_REQUIRE(lda >= K && ldo >= N, "batched product: leading dimensions too small");
  if (M == 0) return 0;
  launch_batched<BEPI_BF16>(p, M, batch, stream);
  MK_LAUNCH_CHECK("linear_batched_mfma");
  return 0;
}

// Experts over the tokens routed to them.  rows [T * top] lists the (token, choice) pairs
// grouped by expert, offsets [experts + 1] where each expert's group starts; max_rows bounds a
// group's size (the grid's row tiles; T * top always does).
//   gated: act[pair, :] = activation(Wg[e] x[pair / top], Wu[e] x[pair / top]), w [E, 2 ff, K]
//   down:  y[pair, :] = weight[pair] * Wd[e] act[pair, :], w [E, N, ff], float32
extern "C" int mk_expert_gated_mfma(const void* x, const void* w, void* act, const int* rows,
                                    const int* offsets, int experts, int max_rows, int top, int ff,
                                    int K, int kind, float limit, float alpha, float beta,
                                    hipStream_t stream) {
  BatchedParams p = {};
  p.x = (const bf16_t*)x;
  p.w = (const bf16_t*)w;
  p.out = act;
  p.M = max_rows; p.N = ff; p.K = K; p.lda = K; p.ldo = ff;
  p.w_batch = (long long)2 * ff * K;
  p.rows = rows;
  p.offsets = offsets;
  p.gather_div = top;
  p.act_kind = kind; p.limit = limit; p.alpha = alpha; p.beta = beta;
  MK_REQUIRE(kind == MK_ACT_SILU || kind == MK_ACT_SWISH_CLAMP || kind == MK_ACT_GELU_TANH,
             "expert_gated: activation %d", kind);
  MK_REQUIRE(rows && offsets && top > 0, "expert_gated: no row lists");
  const int tiles = (max_rows + 15) / 16;
  if (batched_check(p, experts, tiles)) return 1;
  if (max_rows == 0) return 0;
  launch_batched<BEPI_GATED>(p, max_rows, experts, stream);
  MK_LAUNCH_CHECK("expert_gated_mfma");
  return 0;
}

extern "C" int mk_expert_down_mfma(const void* act, const void* w, float* y, const int* rows,
                                   const int* offsets, const float* weights, int experts,
                                   int max_rows, int ff, int N, hipStream_t stream) {
  BatchedParams p = {};
  p.x = (const bf16_t*)act;
  p.w = (const bf16_t*)w;
  p.out = y;
  p.M = max_rows; p.N = N; p.K = ff; p.lda = ff; p.ldo = N;
  p.w_batch = (long long)N * ff;
  p.rows = rows;
  p.offsets = offsets;
  p.gather_div = 1;
  p.row_scale = weights;
  MK_REQUIRE(rows && offsets, "expert_down: no row lists");
  const int tiles = (max_rows + 15) / 16;
  if (batched_check(p, experts, tiles)) return 1;
  if (max_rows == 0) return 0;
  launch_batched<BEPI_SCALED_F32>(p, max_rows, experts, stream);
  MK_LAUNCH_CHECK("expert_down_mfma");
  return 0;
}
