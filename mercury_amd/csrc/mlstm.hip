// A matrix memory with an input gate, a forget gate and a running maximum that keeps its
// exponentials in range (the mLSTM cell), in float32 arithmetic whatever the model's storage
// type.  Per head, with log gates i_t and f_t:
//
//   m_t = max(f_t + m_(t-1), i_t)
//   S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T       (dim x vdim)
//   n_t = exp(f_t + m_(t-1) - m_t) n_(t-1) + exp(i_t - m_t) k_t             (dim)
//   o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
//
// with S, n and m zero before a sequence's first token (m starts at zero, not at minus
// infinity).  The gates come raw from a projection: i_t = cap tanh(a_t / cap),
// f_t = logsigmoid(cap tanh(b_t / cap)) (cap <= 0: a_t and logsigmoid(b_t)).
//
// The recurrence.  n is the state's column for a value that is always one, so it rides with
// S: a workgroup of four wavefronts owns 28 columns of one head of one sequence, a wavefront
// 7 of them and the n column once more, by 8 slices of the state's rows; a lane holds one
// column and R = ceil(dim / 8) consecutive rows in registers for the whole step.  The sum over
// rows is in-lane but for three exchanges across the slices, and n . q comes from the lanes of
// the wavefront's own n column.  Queries, keys, values and gates of 16 tokens at a time are
// staged in LDS; the running maximum of those tokens is made by 16 threads, each walking the
// tokens up to its own in the sequence's order, so that m, and with it every sum, is the same
// however the sequence was cut into steps and whatever else the step holds.
//
// A slot holds [heads, dim, vdim] floats of S, then n [heads, B, dim] and m [heads, B] once for
// each of the B = ceil(vdim / 28) workgroups of a head: a workgroup reads and writes a copy of
// its own (the copies are equal, made by the same operations in the same order), so none reads
// what another has already advanced.
#include "common.h"
#include "mercury_kernels.h"

#define ML_TOKENS 16       // tokens staged at a time
#define ML_WAVE_COLUMNS 7  // columns of S a wavefront owns beside its copy of n
#define ML_COLUMNS 28      // columns of a head per workgroup
#define ML_MAX_DIM 256

namespace {

__device__ __forceinline__ float log_sigmoid(float z) {
  // min(z, 0) - log(1 + exp(-|z|))
  return fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
}

template <int R>
__global__ __launch_bounds__(256) void mlstm_scan_kernel(
    const float* __restrict__ proj, int proj_stride, int q_col, int k_col, int v_col, int i_col,
    int f_col, float q_scale, float gate_cap, const int* __restrict__ cu_q,
    const int* __restrict__ slots, float* __restrict__ state, long long slot_stride, int heads,
    int dim, int vdim, float* __restrict__ out) {
  constexpr int DIM = R * 8;     // rows the lanes of a column hold between them (>= dim)
  constexpr int TOKENS = ML_TOKENS;
  __shared__ __align__(16) float q_s[TOKENS][DIM];
  __shared__ __align__(16) float k_s[TOKENS][DIM];
  __shared__ float v_s[TOKENS][ML_COLUMNS];
  __shared__ float gi_s[TOKENS], gf_s[TOKENS], keep_s[TOKENS], take_s[TOKENS], floor_s[TOKENS];
  __shared__ float m_s;
  const int seq = blockIdx.x, head = blockIdx.y, col0 = blockIdx.z * ML_COLUMNS;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int in_wave = lane & 7;
  const bool counts = in_wave == ML_WAVE_COLUMNS;       // this lane's column is n
  const int local = wave * ML_WAVE_COLUMNS + in_wave;   // among the workgroup's columns of S
  const int col = col0 + local;
  const int slice = lane >> 3, row0 = slice * R;
  const int t_begin = cu_q[seq], t_end = cu_q[seq + 1];
  if (t_begin >= t_end) return;
  const bool live = !counts && col < vdim;
  float* slot = state + (size_t)slots[seq] * slot_stride;
  float* s_at = slot + (size_t)head * dim * vdim;
  const size_t copy = (size_t)head * gridDim.z + blockIdx.z;
  float* n_at = slot + (size_t)heads * dim * vdim + copy * dim;
  float* m_at = slot + (size_t)heads * dim * vdim + (size_t)heads * gridDim.z * dim + copy;

  float s[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int row = row0 + i;
    float got = 0.f;
    if (row < dim) {
      if (counts) got = n_at[row];
      else if (live) got = s_at[(size_t)row * vdim + col];
    }
    s[i] = got;
  }
  float m_run = *m_at;

  for (int t0 = t_begin; t0 < t_end; t0 += TOKENS) {
    const int count = min(TOKENS, t_end - t0);
    __syncthreads();
    for (int e = tid; e < count * DIM; e += 256) {
      const int tt = e / DIM, row = e - tt * DIM;
      float qv = 0.f, kv = 0.f;
      if (row < dim) {
        const float* base = proj + (size_t)(t0 + tt) * proj_stride + head * dim + row;
        qv = base[q_col] * q_scale;
        kv = base[k_col];
      }
      q_s[tt][row] = qv;
      k_s[tt][row] = kv;
    }
    for (int e = tid; e < count * ML_COLUMNS; e += 256) {
      const int tt = e / ML_COLUMNS, c = e - tt * ML_COLUMNS;
      v_s[tt][c] = col0 + c < vdim
          ? proj[(size_t)(t0 + tt) * proj_stride + v_col + head * vdim + col0 + c] : 0.f;
    }
    if (tid < count) {
      const float* row = proj + (size_t)(t0 + tid) * proj_stride;
      float a = row[i_col + head], b = row[f_col + head];
      if (gate_cap > 0.f) {
        a = gate_cap * tanhf(a / gate_cap);
        b = gate_cap * tanhf(b / gate_cap);
      }
      gi_s[tid] = a;
      gf_s[tid] = log_sigmoid(b);
    }
    __syncthreads();
    if (tid < count) {
      float m = m_run, before = m_run;
      for (int j = 0; j <= tid; ++j) {
        before = m;
        m = fmaxf(gf_s[j] + m, gi_s[j]);
      }
      keep_s[tid] = expf(gf_s[tid] + before - m);
      take_s[tid] = expf(gi_s[tid] - m);
      floor_s[tid] = expf(-m);
      if (tid == count - 1) m_s = m;
    }
    __syncthreads();
    m_run = m_s;
    for (int tt = 0; tt < count; ++tt) {
      const float keep = keep_s[tt];
      const float tv = take_s[tt] * (counts ? 1.f : v_s[tt][min(local, ML_COLUMNS - 1)]);
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < R; i += 4) {
        const float4 q4 = *(const float4*)&q_s[tt][row0 + i];
        const float4 k4 = *(const float4*)&k_s[tt][row0 + i];
        s[i] = fmaf(k4.x, tv, keep * s[i]);
        s[i + 1] = fmaf(k4.y, tv, keep * s[i + 1]);
        s[i + 2] = fmaf(k4.z, tv, keep * s[i + 2]);
        s[i + 3] = fmaf(k4.w, tv, keep * s[i + 3]);
        o = fmaf(s[i], q4.x, o);
        o = fmaf(s[i + 1], q4.y, o);
        o = fmaf(s[i + 2], q4.z, o);
        o = fmaf(s[i + 3], q4.w, o);
      }
      o += __shfl_xor(o, 8, MK_WAVE);
      o += __shfl_xor(o, 16, MK_WAVE);
      o += __shfl_xor(o, 32, MK_WAVE);
      const float nq = __shfl(o, lane | 7, MK_WAVE);
      if (slice == 0 && live) {
        out[(size_t)(t0 + tt) * heads * vdim + head * vdim + col] =
            o / (fmaxf(fabsf(nq), floor_s[tt]) + 1e-6f);
      }
    }
  }
  // S by the lanes that own its columns; the workgroup's n by its first wavefront
  const bool keeps_n = counts && wave == 0;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int row = row0 + i;
    if (row >= dim) continue;
    if (live) s_at[(size_t)row * vdim + col] = s[i];
    else if (keeps_n) n_at[row] = s[i];
  }
  if (tid == 0) *m_at = m_run;
}

}  // namespace

extern "C" long long mk_mlstm_state_floats(int heads, int dim, int vdim) {
  if (heads <= 0 || dim <= 0 || vdim <= 0 || dim > ML_MAX_DIM) return -1;
  const long long copies = (vdim + ML_COLUMNS - 1) / ML_COLUMNS;
  return (long long)heads * ((long long)dim * vdim + copies * (dim + 1));
}

extern "C" int mk_mlstm_scan(const float* proj, int proj_stride, int q_col, int k_col, int v_col,
                             int i_col, int f_col, float q_scale, float gate_cap, const int* cu_q,
                             const int* slots, float* state, long long slot_stride, int heads,
                             int dim, int vdim, float* out, int tokens, int num_seqs,
                             hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && num_seqs >= 0 && heads > 0 && dim > 0 && vdim > 0, "mlstm: bad sizes");
  MK_REQUIRE(dim <= ML_MAX_DIM, "mlstm: heads of %d dims exceed the supported %d", dim, ML_MAX_DIM);
  MK_REQUIRE(slot_stride >= mk_mlstm_state_floats(heads, dim, vdim),
             "mlstm: a slot of %lld floats does not hold %d heads of %d x %d with n and m",
             slot_stride, heads, dim, vdim);
  MK_REQUIRE(q_col >= 0 && k_col >= 0 && v_col >= 0 && i_col >= 0 && f_col >= 0 &&
                 proj_stride >= q_col + heads * dim && proj_stride >= k_col + heads * dim &&
                 proj_stride >= v_col + heads * vdim && proj_stride >= i_col + heads &&
                 proj_stride >= f_col + heads,
             "mlstm: columns outside rows of %d", proj_stride);
  const int columns = (vdim + ML_COLUMNS - 1) / ML_COLUMNS;
  MK_REQUIRE(heads <= 65535 && columns <= 65535, "mlstm: too many heads or columns");
  if (tokens == 0 || num_seqs == 0) return 0;
  MK_REQUIRE(proj && cu_q && slots && state && out, "mlstm: null operand");
  const int per_lane = (dim + 7) / 8;
#define ML_LAUNCH(R)                                                                           \
  mlstm_scan_kernel<R><<<dim3(num_seqs, heads, columns), 256, 0, stream>>>(                    \
      proj, proj_stride, q_col, k_col, v_col, i_col, f_col, q_scale, gate_cap, cu_q, slots,    \
      state, slot_stride, heads, dim, vdim, out)
  if (per_lane <= 4) ML_LAUNCH(4);
  else if (per_lane <= 8) ML_LAUNCH(8);
  else if (per_lane <= 16) ML_LAUNCH(16);
  else ML_LAUNCH(32);
#undef ML_LAUNCH
  MK_LAUNCH_CHECK("mlstm_scan");
  return 0;
}
