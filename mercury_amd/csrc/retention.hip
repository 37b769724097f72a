// Retention: linear attention with a fixed decay per head and no softmax or denominator, in
// float32 arithmetic whatever the model's storage type.
//
//   mk_retention_scan   S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head, the state
//                       carried per request slot; queries and keys turn by their positions and
//                       the keys are scaled on the way in;
//   mk_head_norm_gate   a norm per head without a weight, then a gate of one number per column.
//
// The recurrence.  A workgroup of four wavefronts owns 32 columns of one head of one sequence;
// a wavefront 8 of them by 8 slices of the state's rows, a lane one column and R = ceil(dim / 8)
// consecutive rows, in registers for the whole step.  The sum over rows for o_t is in-lane but
// for three exchanges across the slices.  Queries, keys and values of 16 tokens at a time are
// staged in LDS, turned and scaled by the threads that stage them.  A sequence's tokens run in
// order, so the order of every sum depends on the sizes alone: a state is the same however
// the sequence was cut into steps and whatever else the step holds.
#include "common.h"
#include "mercury_kernels.h"

#define RT_TOKENS 16       // tokens staged at a time
#define RT_COLUMNS 32      // columns of a head per workgroup
#define RT_MAX_DIM 256

namespace {

template <int R>
__global__ __launch_bounds__(256) void retention_scan_kernel(
    const float* __restrict__ proj, int proj_stride, int q_col, int k_col, int v_col,
    const float* __restrict__ decay, float k_scale, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, int rot, const int* __restrict__ positions,
    const int* __restrict__ cu_q, const int* __restrict__ slots, float* __restrict__ state,
    long long slot_stride, int heads, int dim, int vdim, float* __restrict__ out) {
  constexpr int DIM = R * 8;     // rows the lanes of a column hold between them (>= dim)
  __shared__ __align__(16) float q_s[RT_TOKENS][DIM];
  __shared__ __align__(16) float k_s[RT_TOKENS][DIM];
  __shared__ float v_s[RT_TOKENS][RT_COLUMNS];
  const int seq = blockIdx.x, head = blockIdx.y, col0 = blockIdx.z * RT_COLUMNS;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int local = wave * 8 + (lane & 7), col = col0 + local;
  const int slice = lane >> 3, row0 = slice * R;
  const int t_begin = cu_q[seq], t_end = cu_q[seq + 1];
  if (t_begin >= t_end) return;
  const float g = decay[head];
  const int half = rot / 2;
  const bool live = col < vdim;
  float* mine = state + (size_t)slots[seq] * slot_stride + (size_t)head * dim * vdim;

  float s[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int row = row0 + i;
    s[i] = live && row < dim ? mine[(size_t)row * vdim + col] : 0.f;
  }

  for (int t0 = t_begin; t0 < t_end; t0 += RT_TOKENS) {
    const int count = min(RT_TOKENS, t_end - t0);
    __syncthreads();
    // stage: q and k turned (k scaled), rows past dim as zeros; v of this workgroup's columns
    for (int e = tid; e < count * DIM; e += 256) {
      const int tt = e / DIM, row = e - tt * DIM;
      float qv = 0.f, kv = 0.f;
      if (row < dim) {
        const float* base = proj + (size_t)(t0 + tt) * proj_stride + head * dim;
        const float* qp = base + q_col;
        const float* kp = base + k_col;
        if (row < rot) {
          const int pos = positions[t0 + tt];
          const int j = row < half ? row : row - half;
          const float c = cos_table[(size_t)pos * half + j], sn = sin_table[(size_t)pos * half + j];
          if (row < half) {
            qv = qp[row] * c - qp[row + half] * sn;
            kv = kp[row] * c - kp[row + half] * sn;
          } else {
            qv = qp[row] * c + qp[row - half] * sn;
            kv = kp[row] * c + kp[row - half] * sn;
          }
        } else {
          qv = qp[row];
          kv = kp[row];
        }
        kv *= k_scale;
      }
      q_s[tt][row] = qv;
      k_s[tt][row] = kv;
    }
    for (int e = tid; e < count * RT_COLUMNS; e += 256) {
      const int tt = e / RT_COLUMNS, c = e - tt * RT_COLUMNS;
      v_s[tt][c] = col0 + c < vdim
          ? proj[(size_t)(t0 + tt) * proj_stride + v_col + head * vdim + col0 + c] : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < count; ++tt) {
      const float v = v_s[tt][local];
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < R; i += 4) {
        const float4 k4 = *(const float4*)&k_s[tt][row0 + i];
        const float4 q4 = *(const float4*)&q_s[tt][row0 + i];
        s[i] = fmaf(k4.x, v, g * s[i]);
        s[i + 1] = fmaf(k4.y, v, g * s[i + 1]);
        s[i + 2] = fmaf(k4.z, v, g * s[i + 2]);
        s[i + 3] = fmaf(k4.w, v, g * s[i + 3]);
        o = fmaf(s[i], q4.x, o);
        o = fmaf(s[i + 1], q4.y, o);
        o = fmaf(s[i + 2], q4.z, o);
        o = fmaf(s[i + 3], q4.w, o);
      }
      o += __shfl_xor(o, 8, MK_WAVE);
      o += __shfl_xor(o, 16, MK_WAVE);
      o += __shfl_xor(o, 32, MK_WAVE);
      if (slice == 0 && live) out[(size_t)(t0 + tt) * heads * vdim + head * vdim + col] = o;
    }
  }
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int row = row0 + i;
    if (live && row < dim) mine[(size_t)row * vdim + col] = s[i];
  }
}

// One wavefront per (token, head).
template <typename T>
__global__ __launch_bounds__(64) void head_norm_gate_kernel(
    const float* __restrict__ y, T* __restrict__ out, const float* __restrict__ gate,
    int gate_stride, float eps, int heads, int dv) {
  const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const float* row = y + ((size_t)t * heads + head) * dv;
  float sq = 0.f;
  for (int i = lane; i < dv; i += MK_WAVE) sq += row[i] * row[i];
  const float r = rsqrtf(wave_sum(sq) / (float)dv + eps);
  for (int i = lane; i < dv; i += MK_WAVE) {
    float v = row[i] * r;
    if (gate) {
      const float z = gate[(size_t)t * gate_stride + head * dv + i];
      v *= z / (1.f + expf(-z));
    }
    Elem<T>::store(out + ((size_t)t * heads + head) * dv + i, v);
  }
}

}  // namespace

extern "C" int mk_retention_scan(const float* proj, int proj_stride, int q_col, int k_col,
                                 int v_col, const float* decay, float k_scale,
                                 const float* cos_table, const float* sin_table,
                                 int table_positions, int rot, const int* positions,
                                 const int* cu_q, const int* slots, float* state,
                                 long long slot_stride, int heads, int dim, int vdim, float* out,
                                 int tokens, int num_seqs, hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && num_seqs >= 0 && heads > 0 && dim > 0 && vdim > 0,
             "retention: bad sizes");
  MK_REQUIRE(dim <= RT_MAX_DIM, "retention: heads of %d dims exceed the supported %d", dim,
             RT_MAX_DIM);
  MK_REQUIRE(rot >= 0 && rot <= dim && rot % 2 == 0, "retention: rotary width %d not in [0, %d] / even",
             rot, dim);
  MK_REQUIRE(rot == 0 || (table_positions > 0 && cos_table && sin_table && positions),
             "retention: empty angle table");
  MK_REQUIRE(slot_stride >= (long long)heads * dim * vdim,
             "retention: a slot of %lld floats does not hold %d heads of %d x %d", slot_stride,
             heads, dim, vdim);
  MK_REQUIRE(q_col >= 0 && k_col >= 0 && v_col >= 0 && proj_stride >= q_col + heads * dim &&
                 proj_stride >= k_col + heads * dim && proj_stride >= v_col + heads * vdim,
             "retention: columns outside rows of %d", proj_stride);
  MK_REQUIRE(heads <= 65535 && (vdim + RT_COLUMNS - 1) / RT_COLUMNS <= 65535,
             "retention: too many heads or columns");
  if (tokens == 0 || num_seqs == 0) return 0;
  MK_REQUIRE(proj && decay && cu_q && slots && state && out, "retention: null operand");
  const dim3 grid(num_seqs, heads, (vdim + RT_COLUMNS - 1) / RT_COLUMNS);
  const int per_lane = (dim + 7) / 8;
#define RT_LAUNCH(R)                                                                            \
  retention_scan_kernel<R><<<grid, 256, 0, stream>>>(                                          \
      proj, proj_stride, q_col, k_col, v_col, decay, k_scale, cos_table, sin_table, rot,        \
      positions, cu_q, slots, state, slot_stride, heads, dim, vdim, out)
  if (per_lane <= 4) RT_LAUNCH(4);
  else if (per_lane <= 8) RT_LAUNCH(8);
  else if (per_lane <= 16) RT_LAUNCH(16);
  else RT_LAUNCH(32);
#undef RT_LAUNCH
  MK_LAUNCH_CHECK("retention_scan");
  return 0;
}

extern "C" int mk_head_norm_gate(const float* y, void* out, int dtype, const float* gate,
                                 int gate_stride, float eps, int tokens, int heads, int dv,
                                 hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && heads > 0 && dv > 0, "head_norm_gate: bad sizes");
  MK_REQUIRE(heads <= 65535, "head_norm_gate: too many heads (%d)", heads);
  MK_REQUIRE(!gate || gate_stride >= heads * dv, "head_norm_gate: gate rows of %d for %d columns",
             gate_stride, heads * dv);
  if (tokens == 0) return 0;
  const dim3 grid(tokens, heads);
  if (dtype == MK_F32)
    head_norm_gate_kernel<float><<<grid, MK_WAVE, 0, stream>>>(y, (float*)out, gate, gate_stride, eps, heads, dv);
  else if (dtype == MK_BF16)
    head_norm_gate_kernel<bf16_t><<<grid, MK_WAVE, 0, stream>>>(y, (bf16_t*)out, gate, gate_stride, eps, heads, dv);
  else
    MK_REQUIRE(false, "head_norm_gate: unknown dtype %d", dtype);
  MK_LAUNCH_CHECK("head_norm_gate");
  return 0;
}
