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
// A step with a sequence longer than ML_CHUNK tokens runs in chunks side by side.  With
// b_j the sum of the log forget gates from the chunk's first token to its j-th, m the running
// maximum of the whole sequence and m' the one of the chunk alone (from minus infinity):
//   gates     one wavefront a (chunk, head): b_j and m'_j = b_j + max_(s<=j)(i_s - b_s) of the
//             chunk's tokens by prefix sums and maxima, and with them the chunk's own
//             recurrence weights exp(f_j + m'_(j-1) - m'_j), exp(i_j - m'_j);
//   pass 1    every chunk's recurrence from a zero state under m' (its numerators and n . q
//             into `out` and a side buffer, its last state into the workspace);
//   carry     the chunks' start states one after the other, with the running maximum at
//             every chunk's start, m_start(c + 1) = max(m_start(c) + b_end(c), m'_end(c)):
//             S_start(c + 1) = exp(b_end + m_start - m_end) S_start(c) + exp(m'_end - m_end) S_own(c),
//             the last into the slot with the last m;
//   pass 2    S_start^T q_j of every token, and, with m_j = max(m_start + b_j, m'_j),
//             exp(b_j + m_start - m_j) (that) + exp(m'_j - m_j) (pass 1's) over the floored
//             denominator.
// Every exponent above is at most zero (to rounding): m_j >= b_j + m_start and m_j >= m'_j.  The
// running maximum only keeps the exponentials in range; made by prefix sums instead of step by
// step it differs in its last bits, which reach the result through the 1e-6 alone.
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
#define ML_CHUNK 128       // tokens of a chunk when a step runs in chunks
#define ML_GATE_FIELDS 4   // per (token, head): keep', take', b, m'
#define ML_CHUNK_FIELDS 4  // per (chunk, head): b_end, m'_end, m_start, the slot's m (a sequence's first chunk)

namespace {

__device__ __forceinline__ float log_sigmoid(float z) {
  // min(z, 0) - log(1 + exp(-|z|))
  return fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
}

__device__ __forceinline__ void activated_gates(const float* __restrict__ row, int i_col, int f_col,
                                                int head, float gate_cap, float& log_in,
                                                float& log_keep) {
  float a = row[i_col + head], b = row[f_col + head];
  if (gate_cap > 0.f) {
    a = gate_cap * tanhf(a / gate_cap);
    b = gate_cap * tanhf(b / gate_cap);
  }
  log_in = a;
  log_keep = log_sigmoid(b);
}

// The sequence and the tokens of chunk `c` of the step.
__device__ __forceinline__ void chunk_span(const int* __restrict__ cu_q, int num_seqs, int c,
                                           int& seq, int& t_begin, int& t_end) {
  int first = 0;
  for (seq = 0; seq < num_seqs; ++seq) {
    const int n = (cu_q[seq + 1] - cu_q[seq] + ML_CHUNK - 1) / ML_CHUNK;
    if (c < first + n) break;
    first += n;
  }
  if (seq >= num_seqs) {
    t_begin = t_end = 0;
    return;
  }
  t_begin = cu_q[seq] + (c - first) * ML_CHUNK;
  t_end = min(cu_q[seq + 1], t_begin + ML_CHUNK);
}

__device__ __forceinline__ float wave_prefix_sum(float v, int lane) {
#pragma unroll
  for (int d = 1; d < MK_WAVE; d <<= 1) {
    const float up = __shfl_up(v, d, MK_WAVE);
    if (lane >= d) v += up;
  }
  return v;
}

__device__ __forceinline__ float wave_prefix_max(float v, int lane) {
#pragma unroll
  for (int d = 1; d < MK_WAVE; d <<= 1) {
    const float up = __shfl_up(v, d, MK_WAVE);
    if (lane >= d) v = fmaxf(v, up);
  }
  return v;
}

// One wavefront a (chunk, head): gates [tokens, heads, ML_GATE_FIELDS], ends
// [chunks, heads, ML_CHUNK_FIELDS].
__global__ __launch_bounds__(64) void mlstm_gates_kernel(
    const float* __restrict__ proj, int proj_stride, int i_col, int f_col, float gate_cap,
    const int* __restrict__ cu_q, const int* __restrict__ slots, const float* __restrict__ state,
    long long slot_stride, int heads, int dim, int vdim, int copies, float* __restrict__ gates,
    float* __restrict__ ends, int num_seqs) {
  const int head = blockIdx.y, lane = threadIdx.x;
  int seq, t_begin, t_end;
  chunk_span(cu_q, num_seqs, blockIdx.x, seq, t_begin, t_end);
  if (t_begin >= t_end) return;
  float sum_before = 0.f, top_before = -INFINITY, own_last = -INFINITY;
  for (int t0 = t_begin; t0 < t_end; t0 += MK_WAVE) {
    const bool there = t0 + lane < t_end;
    float log_in = -INFINITY, log_keep = 0.f;
    if (there) {
      activated_gates(proj + (size_t)(t0 + lane) * proj_stride, i_col, f_col, head, gate_cap,
                      log_in, log_keep);
    }
    const float sum = sum_before + wave_prefix_sum(log_keep, lane);
    const float top = fmaxf(top_before, wave_prefix_max(log_in - sum, lane));
    const float own = sum + top;
    float own_before = __shfl_up(own, 1, MK_WAVE);
    if (lane == 0) own_before = own_last;
    if (there) {
      float* at = gates + ((size_t)(t0 + lane) * heads + head) * ML_GATE_FIELDS;
      at[0] = expf(fminf(log_keep + own_before - own, 0.f));     // 0 at a chunk's first token
      at[1] = expf(log_in - own);
      at[2] = sum;
      at[3] = own;
    }
    const int last = min(MK_WAVE, t_end - t0) - 1;
    sum_before = __shfl(sum, last, MK_WAVE);
    top_before = __shfl(top, last, MK_WAVE);
    own_last = __shfl(own, last, MK_WAVE);
  }
  if (lane == 0) {
    float* at = ends + ((size_t)blockIdx.x * heads + head) * ML_CHUNK_FIELDS;
    at[0] = sum_before;
    at[1] = own_last;
    if (t_begin == cu_q[seq]) {     // the sequence's first chunk keeps the m the slot holds
      at[3] = state[(size_t)slots[seq] * slot_stride + (size_t)heads * dim * vdim +
                    (size_t)heads * copies * dim + (size_t)head * copies];
    }
  }
}

// MODE 0: a sequence's tokens from its slot's state, which is left for the next step.
// MODE 1: a chunk's tokens from a zero state under the chunk's own running maximum; numerators
//         into out, n . q into side, the chunk's last state into `chunks`.
// MODE 2: a chunk's start state (from `chunks`) read by its queries and put together with what
//         MODE 1 left.
template <int R, int MODE>
__global__ __launch_bounds__(256) void mlstm_scan_kernel(
    const float* __restrict__ proj, int proj_stride, int q_col, int k_col, int v_col, int i_col,
    int f_col, float q_scale, float gate_cap, const int* __restrict__ cu_q,
    const int* __restrict__ slots, float* __restrict__ state, long long slot_stride, int heads,
    int dim, int vdim, float* __restrict__ out, const float* __restrict__ gates,
    float* __restrict__ side, float* __restrict__ chunks, const float* __restrict__ ends,
    int num_seqs) {
  constexpr int DIM = R * 8;     // rows the lanes of a column hold between them (>= dim)
  constexpr int TOKENS = ML_TOKENS;
  __shared__ __align__(16) float q_s[TOKENS][DIM];
  __shared__ __align__(16) float k_s[TOKENS][DIM];
  __shared__ float v_s[TOKENS][ML_COLUMNS];
  __shared__ float gi_s[TOKENS], gf_s[TOKENS], keep_s[TOKENS], take_s[TOKENS], floor_s[TOKENS];
  __shared__ float side_s[TOKENS];
  __shared__ float m_s;
  const int head = blockIdx.y, col0 = blockIdx.z * ML_COLUMNS;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int in_wave = lane & 7;
  const bool counts = in_wave == ML_WAVE_COLUMNS;       // this lane's column is n
  const int local = wave * ML_WAVE_COLUMNS + in_wave;   // among the workgroup's columns of S
  const int col = col0 + local;
  const int slice = lane >> 3, row0 = slice * R;
  int seq = blockIdx.x, t_begin, t_end;
  if (MODE == 0) {
    t_begin = cu_q[seq];
    t_end = cu_q[seq + 1];
  } else {
    chunk_span(cu_q, num_seqs, blockIdx.x, seq, t_begin, t_end);
  }
  if (t_begin >= t_end) return;
  const bool live = !counts && col < vdim;
  // MODE 0: the slot (a copy of n and m for every workgroup of the head); else the chunk's
  // place in the workspace: [dim, vdim] of S, then [dim] of n
  float* s_at;
  float* n_at;
  float* m_at = nullptr;
  if (MODE == 0) {
    float* slot = state + (size_t)slots[seq] * slot_stride;
    const size_t copy = (size_t)head * gridDim.z + blockIdx.z;
    s_at = slot + (size_t)head * dim * vdim;
    n_at = slot + (size_t)heads * dim * vdim + copy * dim;
    m_at = slot + (size_t)heads * dim * vdim + (size_t)heads * gridDim.z * dim + copy;
  } else {
    s_at = chunks + ((size_t)blockIdx.x * heads + head) * ((size_t)dim * vdim + dim);
    n_at = s_at + (size_t)dim * vdim;
  }

  float s[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int row = row0 + i;
    float got = 0.f;
    if (MODE != 1 && row < dim) {
      if (counts) got = n_at[row];
      else if (live) got = s_at[(size_t)row * vdim + col];
    }
    s[i] = got;
  }
  float m_run = MODE == 0 ? *m_at : 0.f;

  for (int t0 = t_begin; t0 < t_end; t0 += TOKENS) {
    const int count = min(TOKENS, t_end - t0);
    __syncthreads();
    for (int e = tid; e < count * DIM; e += 256) {
      const int tt = e / DIM, row = e - tt * DIM;
      float qv = 0.f, kv = 0.f;
      if (row < dim) {
        const float* base = proj + (size_t)(t0 + tt) * proj_stride + head * dim + row;
        qv = base[q_col] * q_scale;
        if (MODE != 2) kv = base[k_col];
      }
      q_s[tt][row] = qv;
      if (MODE != 2) k_s[tt][row] = kv;
    }
    // the values; in pass 2, in their place, what pass 1 left in out for these columns
    for (int e = tid; e < count * ML_COLUMNS; e += 256) {
      const int tt = e / ML_COLUMNS, c = e - tt * ML_COLUMNS;
      float got = 0.f;
      if (col0 + c < vdim) {
        got = MODE == 2 ? out[(size_t)(t0 + tt) * heads * vdim + head * vdim + col0 + c]
                        : proj[(size_t)(t0 + tt) * proj_stride + v_col + head * vdim + col0 + c];
      }
      v_s[tt][c] = got;
    }
    if (MODE == 0) {
      if (tid < count) {
        activated_gates(proj + (size_t)(t0 + tid) * proj_stride, i_col, f_col, head, gate_cap,
                        gi_s[tid], gf_s[tid]);
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
    } else if (tid < count) {
      const float* g = gates + ((size_t)(t0 + tid) * heads + head) * ML_GATE_FIELDS;
      if (MODE == 1) {
        keep_s[tid] = g[0];
        take_s[tid] = g[1];
      } else {     // pass 2: the weights of the start state and of the chunk's own part
        const float m_start = ends[((size_t)blockIdx.x * heads + head) * ML_CHUNK_FIELDS + 2];
        const float m = fmaxf(m_start + g[2], g[3]);
        keep_s[tid] = expf(fminf(g[2] + m_start - m, 0.f));
        take_s[tid] = expf(fminf(g[3] - m, 0.f));
        floor_s[tid] = expf(-m);
        side_s[tid] = side[(size_t)(t0 + tid) * heads + head];
      }
    }
    __syncthreads();
    if (MODE == 0) m_run = m_s;
    for (int tt = 0; tt < count; ++tt) {
      const float keep = keep_s[tt];
      const float held = counts ? 1.f : v_s[tt][min(local, ML_COLUMNS - 1)];
      const float tv = take_s[tt] * held;
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < R; i += 4) {
        const float4 q4 = *(const float4*)&q_s[tt][row0 + i];
        if (MODE != 2) {
          const float4 k4 = *(const float4*)&k_s[tt][row0 + i];
          s[i] = fmaf(k4.x, tv, keep * s[i]);
          s[i + 1] = fmaf(k4.y, tv, keep * s[i + 1]);
          s[i + 2] = fmaf(k4.z, tv, keep * s[i + 2]);
          s[i + 3] = fmaf(k4.w, tv, keep * s[i + 3]);
        }
        o = fmaf(s[i], q4.x, o);
        o = fmaf(s[i + 1], q4.y, o);
        o = fmaf(s[i + 2], q4.z, o);
        o = fmaf(s[i + 3], q4.w, o);
      }
      o += __shfl_xor(o, 8, MK_WAVE);
      o += __shfl_xor(o, 16, MK_WAVE);
      o += __shfl_xor(o, 32, MK_WAVE);
      float nq = __shfl(o, lane | 7, MK_WAVE);
      float* at = out + (size_t)(t0 + tt) * heads * vdim + head * vdim + col;
      if (MODE == 1) {
        if (slice == 0 && live) *at = o;
        if (blockIdx.z == 0 && tid == ML_WAVE_COLUMNS) side[(size_t)(t0 + tt) * heads + head] = nq;
        continue;
      }
      if (MODE == 2) {      // keep = w1, take = w2, held = pass 1's numerator
        o = fmaf(keep, o, tv);
        nq = fmaf(keep, nq, take_s[tt] * side_s[tt]);
      }
      if (slice == 0 && live) *at = o / (fmaxf(fabsf(nq), floor_s[tt]) + 1e-6f);
    }
  }
  if (MODE == 2) return;
  // S by the lanes that own its columns; n by the first wavefront (MODE 0: of every workgroup,
  // into its own copy; MODE 1: of the head's first workgroup)
  const bool keeps_n = counts && wave == 0 && (MODE == 0 || blockIdx.z == 0);
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int row = row0 + i;
    if (row >= dim) continue;
    if (live) s_at[(size_t)row * vdim + col] = s[i];
    else if (keeps_n) n_at[row] = s[i];
  }
  if (MODE == 0 && tid == 0) *m_at = m_run;
}

// The chunks' start states, one sequence's after the other: a thread owns one entry of a
// head's S or n, takes it from the slot, leaves in every chunk's place what the chunk starts
// from, and puts what the last chunk ends with back into the slot (n into every copy).  Every
// thread walks the running maximum along; the head's first thread leaves it at every chunk's
// start for pass 2 and puts the last one into the slot's copies.
__global__ __launch_bounds__(256) void mlstm_carry_kernel(
    const int* __restrict__ cu_q, const int* __restrict__ slots, float* __restrict__ state,
    long long slot_stride, float* __restrict__ ends, float* __restrict__ chunks, int heads,
    int dim, int vdim, int copies) {
  const int seq = blockIdx.x, head = blockIdx.y, e = blockIdx.z * 256 + threadIdx.x;
  const int entries = dim * vdim + dim;
  if (e >= entries) return;
  int first = 0;
  for (int i = 0; i < seq; ++i) first += (cu_q[i + 1] - cu_q[i] + ML_CHUNK - 1) / ML_CHUNK;
  const int tokens = cu_q[seq + 1] - cu_q[seq];
  if (tokens <= 0) return;
  float* slot = state + (size_t)slots[seq] * slot_stride;
  const bool of_n = e >= dim * vdim;
  float* mine = of_n ? slot + (size_t)heads * dim * vdim + (size_t)head * copies * dim + (e - dim * vdim)
                     : slot + (size_t)head * dim * vdim + e;
  float* at = chunks + ((size_t)first * heads + head) * entries + e;
  float* w = ends + ((size_t)first * heads + head) * ML_CHUNK_FIELDS;
  const size_t step = (size_t)heads * entries, w_step = (size_t)heads * ML_CHUNK_FIELDS;
  const int count = (tokens + ML_CHUNK - 1) / ML_CHUNK;
  float s = *mine;
  float m = w[3];
  // eight chunks' ends are asked for at a time, so that their ways to memory overlap
  for (int c0 = 0; c0 < count; c0 += 8) {
    float ended[8], sum[8], own[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const bool there = c0 + j < count;
      ended[j] = there ? at[(size_t)(c0 + j) * step] : 0.f;
      sum[j] = there ? w[(size_t)(c0 + j) * w_step] : 0.f;
      own[j] = there ? w[(size_t)(c0 + j) * w_step + 1] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (c0 + j >= count) break;
      at[(size_t)(c0 + j) * step] = s;
      if (e == 0) w[(size_t)(c0 + j) * w_step + 2] = m;
      const float m_end = fmaxf(m + sum[j], own[j]);
      s = fmaf(expf(fminf(sum[j] + m - m_end, 0.f)), s, expf(fminf(own[j] - m_end, 0.f)) * ended[j]);
      m = m_end;
    }
  }
  if (of_n) {
    for (int c = 0; c < copies; ++c) mine[(size_t)c * dim] = s;
  } else {
    *mine = s;
  }
  if (e == 0) {
    float* m_at = slot + (size_t)heads * dim * vdim + (size_t)heads * copies * dim + (size_t)head * copies;
    for (int c = 0; c < copies; ++c) m_at[c] = m;
  }
}

}  // namespace

extern "C" long long mk_mlstm_state_floats(int heads, int dim, int vdim) {
  if (heads <= 0 || dim <= 0 || vdim <= 0 || dim > ML_MAX_DIM) return -1;
  const long long copies = (vdim + ML_COLUMNS - 1) / ML_COLUMNS;
  return (long long)heads * ((long long)dim * vdim + copies * (dim + 1));
}

extern "C" int mk_mlstm_chunk_tokens(void) { return ML_CHUNK; }

extern "C" long long mk_mlstm_scan_workspace(int total_chunks, int tokens, int heads, int dim,
                                             int vdim) {
  if (total_chunks < 0 || tokens < 0 || heads <= 0 || dim <= 0 || vdim <= 0) return -1;
  // the chunks' states and scalars, the tokens' gates and n . q
  return (long long)total_chunks * heads * ((long long)dim * vdim + dim + ML_CHUNK_FIELDS) +
         (long long)tokens * heads * (ML_GATE_FIELDS + 1);
}

extern "C" int mk_mlstm_scan(const float* proj, int proj_stride, int q_col, int k_col, int v_col,
                             int i_col, int f_col, float q_scale, float gate_cap, const int* cu_q,
                             const int* slots, float* state, long long slot_stride, int heads,
                             int dim, int vdim, float* out, int tokens, int num_seqs,
                             int total_chunks, float* workspace, hipStream_t stream) {
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
  MK_REQUIRE(total_chunks >= 0 && (total_chunks == 0 || workspace),
             "mlstm: chunks without a workspace");
  const int per_lane = (dim + 7) / 8;
  float* chunk_states = workspace;
  float* ends = workspace ? chunk_states + (size_t)total_chunks * heads * ((size_t)dim * vdim + dim) : nullptr;
  float* gates = workspace ? ends + (size_t)total_chunks * heads * ML_CHUNK_FIELDS : nullptr;
  float* side = workspace ? gates + (size_t)tokens * heads * ML_GATE_FIELDS : nullptr;
#define ML_LAUNCH_R(R, MODE, first)                                                             \
  mlstm_scan_kernel<R, MODE><<<dim3(first, heads, columns), 256, 0, stream>>>(                  \
      proj, proj_stride, q_col, k_col, v_col, i_col, f_col, q_scale, gate_cap, cu_q, slots,     \
      state, slot_stride, heads, dim, vdim, out, gates, side, chunk_states, ends, num_seqs)
#define ML_LAUNCH(MODE, first)                                                                  \
  do {                                                                                          \
    if (per_lane <= 4) ML_LAUNCH_R(4, MODE, first);                                             \
    else if (per_lane <= 8) ML_LAUNCH_R(8, MODE, first);                                        \
    else if (per_lane <= 16) ML_LAUNCH_R(16, MODE, first);                                      \
    else ML_LAUNCH_R(32, MODE, first);                                                          \
  } while (0)
  if (total_chunks == 0) {
    ML_LAUNCH(0, num_seqs);
    MK_LAUNCH_CHECK("mlstm_scan");
    return 0;
  }
  mlstm_gates_kernel<<<dim3(total_chunks, heads), MK_WAVE, 0, stream>>>(
      proj, proj_stride, i_col, f_col, gate_cap, cu_q, slots, state, slot_stride, heads, dim, vdim,
      columns, gates, ends, num_seqs);
  MK_LAUNCH_CHECK("mlstm_gates");
  ML_LAUNCH(1, total_chunks);
  MK_LAUNCH_CHECK("mlstm_scan (chunks)");
  const int entries = dim * vdim + dim;
  mlstm_carry_kernel<<<dim3(num_seqs, heads, (entries + 255) / 256), 256, 0, stream>>>(
      cu_q, slots, state, slot_stride, ends, chunk_states, heads, dim, vdim, columns);
  MK_LAUNCH_CHECK("mlstm_carry");
  ML_LAUNCH(2, total_chunks);
#undef ML_LAUNCH
#undef ML_LAUNCH_R
  MK_LAUNCH_CHECK("mlstm_scan (start states)");
  return 0;
}
