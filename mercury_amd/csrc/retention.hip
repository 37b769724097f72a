// Retention: linear attention with a fixed decay per head and no softmax or denominator, in
// float32 arithmetic whatever the model's storage type.
//
//   mk_retention_scan   S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head, the state
//                       carried per request slot; queries and keys turn by their positions and
//                       the keys are scaled on the way in;
//   mk_head_norm_gate   a norm per head, with or without a weight, then a gate of one number
//                       per column (silu or sigmoid).
//
// The recurrence.  A workgroup of four wavefronts owns 32 columns of one head of one sequence;
// a wavefront 8 of them by 8 slices of the state's rows, a lane one column and R = ceil(dim / 8)
// consecutive rows, in registers for the whole step.  The sum over rows for o_t is in-lane but
// for three exchanges across the slices.  Queries, keys and values of 16 tokens at a time are
// staged in LDS, turned and scaled by the threads that stage them (64 at a time were slower:
// a workgroup does not compute while it stages, and fewer workgroups fit beside it).  A
// sequence's tokens run in order, so the order of every sum depends on the sizes alone: a
// state is the same however the sequence was cut into steps and whatever else the step holds.
//
// A step with a sequence longer than RT_CHUNK tokens runs in chunks side by side, the decay
// being a constant: every chunk's recurrence from a zero state (pass 1, its last state into the
// workspace), the chunks' start states one after the other (the carry:
// S_start(c + 1) = decay^len(c) S_start(c) + S_local(c), the last into the slot), and
// decay^(n + 1) S_start^T q_t added to the n-th token of every chunk (pass 2).
#include "common.h"
#include "mercury_kernels.h"

#define RT_TOKENS 16       // tokens staged at a time
#define RT_COLUMNS 32      // columns of a head per workgroup
#define RT_MAX_DIM 256
#define RT_CHUNK 128       // tokens of a chunk when a step runs in chunks

namespace {

// The sequence and the tokens of chunk `c` of the step.
__device__ __forceinline__ void chunk_span(const int* __restrict__ cu_q, int num_seqs, int c,
                                           int& seq, int& t_begin, int& t_end) {
  int first = 0;
  for (seq = 0; seq < num_seqs; ++seq) {
    const int n = (cu_q[seq + 1] - cu_q[seq] + RT_CHUNK - 1) / RT_CHUNK;
    if (c < first + n) break;
    first += n;
  }
  if (seq >= num_seqs) {
    t_begin = t_end = 0;
    return;
  }
  t_begin = cu_q[seq] + (c - first) * RT_CHUNK;
  t_end = min(cu_q[seq + 1], t_begin + RT_CHUNK);
}

// MODE 0: a sequence's tokens from its slot's state, which is left for the next step.
// MODE 1: a chunk's tokens from a zero state; the chunk's last state goes to `chunks`.
// MODE 2: a chunk's start state (from `chunks`) read by its queries: out += decay^(n + 1) S^T q.
template <int R, int MODE>
__global__ __launch_bounds__(256) void retention_scan_kernel(
    const float* __restrict__ proj, int proj_stride, int q_col, int k_col, int v_col,
    const float* __restrict__ decay, float k_scale, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, int rot, const int* __restrict__ positions,
    const int* __restrict__ cu_q, const int* __restrict__ slots, float* __restrict__ state,
    long long slot_stride, int heads, int dim, int vdim, float* __restrict__ out,
    float* __restrict__ chunks, int num_seqs) {
  constexpr int DIM = R * 8;     // rows the lanes of a column hold between them (>= dim)
  constexpr int TOKENS = RT_TOKENS;
  __shared__ __align__(16) float q_s[TOKENS][DIM];
  __shared__ __align__(16) float k_s[TOKENS][DIM];
  __shared__ float v_s[TOKENS][RT_COLUMNS];
  const int head = blockIdx.y, col0 = blockIdx.z * RT_COLUMNS;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int local = wave * 8 + (lane & 7), col = col0 + local;
  const int slice = lane >> 3, row0 = slice * R;
  int seq = blockIdx.x, t_begin, t_end;
  if (MODE == 0) {
    t_begin = cu_q[seq];
    t_end = cu_q[seq + 1];
  } else {
    chunk_span(cu_q, num_seqs, blockIdx.x, seq, t_begin, t_end);
  }
  if (t_begin >= t_end) return;
  const float g = decay[head];
  const int half = rot / 2;
  const bool live = col < vdim;
  float* mine = MODE == 0
      ? state + (size_t)slots[seq] * slot_stride + (size_t)head * dim * vdim
      : chunks + ((size_t)blockIdx.x * heads + head) * dim * vdim;

  float s[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int row = row0 + i;
    s[i] = MODE != 1 && live && row < dim ? mine[(size_t)row * vdim + col] : 0.f;
  }
  float reach = g;     // MODE 2: decay^(n + 1) at the chunk's n-th token

  for (int t0 = t_begin; t0 < t_end; t0 += TOKENS) {
    const int count = min(TOKENS, t_end - t0);
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
    // the values; in pass 2, in their place, what pass 1 left in out for these columns
    for (int e = tid; e < count * RT_COLUMNS; e += 256) {
      const int tt = e / RT_COLUMNS, c = e - tt * RT_COLUMNS;
      float got = 0.f;
      if (col0 + c < vdim) {
        got = MODE == 2 ? out[(size_t)(t0 + tt) * heads * vdim + head * vdim + col0 + c]
                        : proj[(size_t)(t0 + tt) * proj_stride + v_col + head * vdim + col0 + c];
      }
      v_s[tt][c] = got;
    }
    __syncthreads();
    for (int tt = 0; tt < count; ++tt) {
      const float v = v_s[tt][local];
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < R; i += 4) {
        const float4 q4 = *(const float4*)&q_s[tt][row0 + i];
        if (MODE != 2) {
          const float4 k4 = *(const float4*)&k_s[tt][row0 + i];
          s[i] = fmaf(k4.x, v, g * s[i]);
          s[i + 1] = fmaf(k4.y, v, g * s[i + 1]);
          s[i + 2] = fmaf(k4.z, v, g * s[i + 2]);
          s[i + 3] = fmaf(k4.w, v, g * s[i + 3]);
        }
        o = fmaf(s[i], q4.x, o);
        o = fmaf(s[i + 1], q4.y, o);
        o = fmaf(s[i + 2], q4.z, o);
        o = fmaf(s[i + 3], q4.w, o);
      }
      o += __shfl_xor(o, 8, MK_WAVE);
      o += __shfl_xor(o, 16, MK_WAVE);
      o += __shfl_xor(o, 32, MK_WAVE);
      float* at = out + (size_t)(t0 + tt) * heads * vdim + head * vdim + col;
      if (slice == 0 && live) {
        *at = MODE == 2 ? fmaf(reach, o, v) : o;
      }
      reach *= g;
    }
  }
  if (MODE == 2) return;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int row = row0 + i;
    if (live && row < dim) mine[(size_t)row * vdim + col] = s[i];
  }
}

// The chunks' start states, one sequence's after the other: a thread owns one entry of a
// head's state, takes it from the slot, leaves in every chunk's place what the chunk starts
// from, and puts what the last chunk ends with back into the slot.
__global__ __launch_bounds__(256) void retention_carry_kernel(
    const int* __restrict__ cu_q, const int* __restrict__ slots, float* __restrict__ state,
    long long slot_stride, const float* __restrict__ decay, float* __restrict__ chunks, int heads,
    int entries) {
  const int seq = blockIdx.x, head = blockIdx.y, e = blockIdx.z * 256 + threadIdx.x;
  if (e >= entries) return;
  int first = 0;
  for (int i = 0; i < seq; ++i) first += (cu_q[i + 1] - cu_q[i] + RT_CHUNK - 1) / RT_CHUNK;
  const int tokens = cu_q[seq + 1] - cu_q[seq];
  if (tokens <= 0) return;
  const float g = decay[head];
  float whole = 1.f;     // the decay over a whole chunk
  for (int i = 0; i < RT_CHUNK; ++i) whole *= g;
  float* mine = state + (size_t)slots[seq] * slot_stride + (size_t)head * entries + e;
  float* at = chunks + ((size_t)first * heads + head) * entries + e;
  const size_t step = (size_t)heads * entries;
  const int count = (tokens + RT_CHUNK - 1) / RT_CHUNK;
  float s = *mine;
  // eight chunks' ends are asked for at a time, so that their ways to memory overlap
  for (int c0 = 0; c0 < count; c0 += 8) {
    float ended[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) ended[j] = c0 + j < count ? at[(size_t)(c0 + j) * step] : 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (c0 + j >= count) break;
      at[(size_t)(c0 + j) * step] = s;
      float reach = whole;
      if (c0 + j == count - 1) {
        const int len = tokens - (count - 1) * RT_CHUNK;
        reach = 1.f;
        for (int i = 0; i < len; ++i) reach *= g;
      }
      s = fmaf(reach, s, ended[j]);
    }
  }
  *mine = s;
}

// One wavefront per (token, head).
template <typename T>
__global__ __launch_bounds__(64) void head_norm_gate_kernel(
    const float* __restrict__ y, T* __restrict__ out, const float* __restrict__ gate,
    int gate_stride, float eps, int heads, int dv, const float* __restrict__ weight,
    int gate_kind) {
  const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const float* row = y + ((size_t)t * heads + head) * dv;
  float sq = 0.f;
  for (int i = lane; i < dv; i += MK_WAVE) sq += row[i] * row[i];
  const float r = rsqrtf(wave_sum(sq) / (float)dv + eps);
  for (int i = lane; i < dv; i += MK_WAVE) {
    float v = row[i] * r;
    if (weight) v *= weight[head * dv + i];
    if (gate) {
      const float z = gate[(size_t)t * gate_stride + head * dv + i];
      v *= (gate_kind == MK_GATE_SIGMOID ? 1.f : z) / (1.f + expf(-z));
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
                                 int tokens, int num_seqs, int total_chunks, float* workspace,
                                 hipStream_t stream) {
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
  MK_REQUIRE(total_chunks >= 0 && (total_chunks == 0 || workspace),
             "retention: chunks without a workspace");
  const int columns = (vdim + RT_COLUMNS - 1) / RT_COLUMNS;
  const int per_lane = (dim + 7) / 8;
#define RT_LAUNCH_R(R, MODE, first)                                                             \
  retention_scan_kernel<R, MODE><<<dim3(first, heads, columns), 256, 0, stream>>>(              \
      proj, proj_stride, q_col, k_col, v_col, decay, k_scale, cos_table, sin_table, rot,        \
      positions, cu_q, slots, state, slot_stride, heads, dim, vdim, out, workspace, num_seqs)
#define RT_LAUNCH(MODE, first)                                                                  \
  do {                                                                                          \
    if (per_lane <= 4) RT_LAUNCH_R(4, MODE, first);                                             \
    else if (per_lane <= 8) RT_LAUNCH_R(8, MODE, first);                                        \
    else if (per_lane <= 16) RT_LAUNCH_R(16, MODE, first);                                      \
    else RT_LAUNCH_R(32, MODE, first);                                                          \
  } while (0)
  if (total_chunks == 0) {
    RT_LAUNCH(0, num_seqs);
    MK_LAUNCH_CHECK("retention_scan");
    return 0;
  }
  RT_LAUNCH(1, total_chunks);
  MK_LAUNCH_CHECK("retention_scan (chunks)");
  const int entries = dim * vdim;
  retention_carry_kernel<<<dim3(num_seqs, heads, (entries + 255) / 256), 256, 0, stream>>>(
      cu_q, slots, state, slot_stride, decay, workspace, heads, entries);
  MK_LAUNCH_CHECK("retention_carry");
  RT_LAUNCH(2, total_chunks);
#undef RT_LAUNCH
#undef RT_LAUNCH_R
  MK_LAUNCH_CHECK("retention_scan (start states)");
  return 0;
}

extern "C" int mk_retention_chunk_tokens(void) { return RT_CHUNK; }

extern "C" long long mk_retention_scan_workspace(int total_chunks, int heads, int dim, int vdim) {
  if (total_chunks < 0 || heads <= 0 || dim <= 0 || vdim <= 0) return -1;
  return (long long)total_chunks * heads * dim * vdim;
}

extern "C" int mk_head_norm_gate(const float* y, void* out, int dtype, const float* gate,
                                 int gate_stride, float eps, int tokens, int heads, int dv,
                                 const float* weight, int gate_kind, hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && heads > 0 && dv > 0, "head_norm_gate: bad sizes");
  MK_REQUIRE(gate_kind == MK_GATE_SILU || gate_kind == MK_GATE_SIGMOID,
             "head_norm_gate: unknown gate %d", gate_kind);
  MK_REQUIRE(heads <= 65535, "head_norm_gate: too many heads (%d)", heads);
  MK_REQUIRE(!gate || gate_stride >= heads * dv, "head_norm_gate: gate rows of %d for %d columns",
             gate_stride, heads * dv);
  if (tokens == 0) return 0;
  const dim3 grid(tokens, heads);
  if (dtype == MK_F32)
    head_norm_gate_kernel<float><<<grid, MK_WAVE, 0, stream>>>(y, (float*)out, gate, gate_stride, eps, heads, dv, weight, gate_kind);
  else if (dtype == MK_BF16)
    head_norm_gate_kernel<bf16_t><<<grid, MK_WAVE, 0, stream>>>(y, (bf16_t*)out, gate, gate_stride, eps, heads, dv, weight, gate_kind);
  else
    MK_REQUIRE(false, "head_norm_gate: unknown dtype %d", dtype);
  MK_LAUNCH_CHECK("head_norm_gate");
  return 0;
}
