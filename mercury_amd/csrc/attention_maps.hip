// Two-map (differential) attention over the paged cache on the matrix cores, bfloat16, with
// its tail fused: both maps of a head are softmax attentions over the same values,
//   o = a1 - lambda * a2,  o / sqrt(mean(o^2) + eps) * out_scale * sigmoid(gate[token, head]).
//
// A head's key row holds the two maps side by side (DM dims each); query (head, map) lies a
// key row wide in q with its own map's dims filled.  Keys lie as [page, kv head, slot, 2 DM],
// values transposed within the page as [page, kv head, DV, slot].
//
// A workgroup of four wavefronts owns 16 consecutive query rows of one sequence and one head.
// The keys any of its rows sees (the first `keep_first` of the sequence and the window's, or
// all up to the last row's position) are walked in blocks of 32; the wavefronts take the
// blocks in turn and merge their running maxima, sums and unnormalised results through LDS at
// the end, so a decoded token's keys are read by four wavefronts and a prompt's tiles spread
// over the chip whatever their lengths.  The products are transposed (S^T = K Q^T, then
// O^T = V^T P^T): a lane holds a query row's scores for eight keys, which is the operand
// layout the second product wants, and every per-row quantity (maximum, sum, the correction
// of the accumulators) lives in the lanes of that row.  Scores, softmax, the combination of
// the maps and the head's norm are float32; the weights enter the second product as
// bfloat16 like the values.
#include "common.h"
#include "mercury_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

namespace {

union MFrag {
  bf16x8 v;
  uint4 u;
  uint2 u2[2];
};

struct MapsParams {
  const bf16_t* q;        // [T, q_stride]: query (head, map) at (head * 2 + map) * 2 DM
  bf16_t* out;            // [T, heads, DV]
  const bf16_t* k_cache;
  const bf16_t* v_cache;
  const float* gate;      // [T, gate_stride] or null
  const int* positions;
  const int* cu_q;
  const int* block_table;
  int q_stride, gate_stride, table_stride, page_shift;
  int heads, kv_heads, window, keep_first;
  float scale_log2, lambda, eps, out_scale;
  int splits;             // workgroups that share a tile's key blocks (a step of single tokens)
  float* parts;           // [seq, head, split, map, 2 + DV]: maximum, sum, unnormalised result
};

#define AM_WAVES 4

// The tail for one row's lanes: o = a1 / l1 - lambda a2 / l2 over the head's DV values (this
// lane: 4 DVT of them), o / rms(o) * out_scale * sigmoid(gate), bfloat16 out.
template <int DVT>
__device__ __forceinline__ void finish_head(const MapsParams& p, f32x4 (&acc)[2][DVT],
                                            const float (&lsum)[2], int token, int head, int g4,
                                            bool row_ok) {
  constexpr int DV = DVT * 16;
  const float inv1 = lsum[0] > 0.f ? 1.f / lsum[0] : 0.f;
  const float inv2 = lsum[1] > 0.f ? p.lambda / lsum[1] : 0.f;
  float sq = 0.f;
#pragma unroll
  for (int t = 0; t < DVT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float o = acc[0][t][i] * inv1 - acc[1][t][i] * inv2;
      acc[0][t][i] = o;
      sq = __builtin_fmaf(o, o, sq);
    }
  sq += __shfl_xor(sq, 16, 64);
  sq += __shfl_xor(sq, 32, 64);
  if (!row_ok) return;
  float mult = rsqrtf(sq / (float)DV + p.eps) * p.out_scale;
  if (p.gate) mult *= 1.f / (1.f + expf(-p.gate[(size_t)token * p.gate_stride + head]));
  bf16_t* orow = p.out + ((size_t)token * p.heads + head) * DV + g4 * 4;
#pragma unroll
  for (int t = 0; t < DVT; ++t) {
    const uint2 packed = make_uint2(pack_bf16x2(acc[0][t][0] * mult, acc[0][t][1] * mult),
                                    pack_bf16x2(acc[0][t][2] * mult, acc[0][t][3] * mult));
    *(uint2*)(orow + t * 16) = packed;
  }
}

// DKC: 32-wide chunks of a map's dims; DVT: 16-wide tiles of the values.
template <int DKC, int DVT>
__global__ __launch_bounds__(256) void attn_maps_kernel(MapsParams p) {
  constexpr int DM = DKC * 32, DV = DVT * 16;
  // per wavefront but the first: maxima and sums [2][16], then accumulators [2][DVT][4][64]
  __shared__ float stat_s[AM_WAVES - 1][2][2][16];
  __shared__ float acc_s[AM_WAVES - 1][2][DVT][4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g4 = lane >> 4;
  const int seq = blockIdx.y, head = blockIdx.z;
  const int q0 = p.cu_q[seq], q_len = p.cu_q[seq + 1] - q0;
  const int split = blockIdx.x % p.splits;
  const int row0 = blockIdx.x / p.splits * 16;
  if (row0 >= q_len) return;                         // the whole workgroup
  const int rows = min(16, q_len - row0);
  const bool row_ok = r < rows;
  const int token = q0 + row0 + min(r, rows - 1);    // a row past the end repeats the last one
  const int pos = row_ok ? p.positions[token] : -1;  // sees nothing
  const int p_first = p.positions[q0 + row0], p_last = p.positions[q0 + row0 + rows - 1];
  const int kvh = head / (p.heads / p.kv_heads);
  const int ps = 1 << p.page_shift;
  const int* table = p.block_table + (size_t)seq * p.table_stride;

  // the blocks of 32 keys some row sees: [0, a_end) for the kept first keys, [b_begin, b_end)
  const int lo = p.window > 0 ? max(0, p_first - p.window + 1) : 0;
  const int b_begin = lo >> 5, b_end = (p_last >> 5) + 1;
  const int a_end = p.window > 0 && p.keep_first > 0 ? min((p.keep_first + 31) >> 5, b_begin) : 0;
  const int blocks = a_end + b_end - b_begin;

  MFrag qf[2][DKC];
  {
    const bf16_t* qrow = p.q + (size_t)token * p.q_stride + (size_t)head * 4 * DM + g4 * 8;
#pragma unroll
    for (int map = 0; map < 2; ++map)
#pragma unroll
      for (int c = 0; c < DKC; ++c)
        qf[map][c].u = *(const uint4*)(qrow + map * 3 * DM + c * 32);
  }
  f32x4 acc[2][DVT];
#pragma unroll
  for (int map = 0; map < 2; ++map)
#pragma unroll
    for (int t = 0; t < DVT; ++t) acc[map][t] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float m[2] = {-INFINITY, -INFINITY}, lsum[2] = {0.f, 0.f};
  const float c2 = p.scale_log2;

  for (int index = split * AM_WAVES + wave; index < blocks; index += AM_WAVES * p.splits) {
    const int key0 = (index < a_end ? index : b_begin + index - a_end) << 5;
    const bf16_t* kbase[2];
    const bf16_t* vbase[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int kh = key0 + h * 16;
      // a half no row sees (below the window and past the kept keys, or past the last row)
      // may lie on a page the sequence does not hold: page 0 exists, its keys are masked
      const bool seen = kh <= p_last && (p.window == 0 || kh + 15 >= lo || kh < p.keep_first);
      const int page = seen ? table[kh >> p.page_shift] : 0;
      const int off = kh & (ps - 1);
      kbase[h] = p.k_cache + (((size_t)page * p.kv_heads + kvh) * ps + off + r) * (2 * DM) + g4 * 8;
      vbase[h] = p.v_cache + (((size_t)page * p.kv_heads + kvh) * DV + r) * ps + off + g4 * 4;
    }
    MFrag vf[DVT];
#pragma unroll
    for (int t = 0; t < DVT; ++t) {
      vf[t].u2[0] = *(const uint2*)(vbase[0] + (size_t)t * 16 * ps);
      vf[t].u2[1] = *(const uint2*)(vbase[1] + (size_t)t * 16 * ps);
    }
    // which of this lane's eight keys its row sees
    bool see[8];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = key0 + h * 16 + g4 * 4 + i;
        see[h * 4 + i] = key <= pos && (p.window == 0 || pos - key < p.window || key < p.keep_first);
      }
#pragma unroll
    for (int map = 0; map < 2; ++map) {
      float s[8];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        MFrag kf[DKC];
#pragma unroll
        for (int c = 0; c < DKC; ++c) kf[c].u = *(const uint4*)(kbase[h] + map * DM + c * 32);
        f32x4 sc = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < DKC; ++c)
          sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[c].v, qf[map][c].v, sc, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) s[h * 4 + i] = see[h * 4 + i] ? sc[i] * c2 : -INFINITY;
      }
      float bm = fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])),
                       fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
      bm = fmaxf(bm, __shfl_xor(bm, 16, 64));
      bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
      const float m_new = fmaxf(m[map], bm);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      const float corr = __builtin_amdgcn_exp2f(m[map] - m_use);   // 0 while m is -inf
      lsum[map] *= corr;
#pragma unroll
      for (int t = 0; t < DVT; ++t) acc[map][t] *= corr;
      m[map] = m_new;
      float e[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) e[j] = __builtin_amdgcn_exp2f(s[j] - m_use);
      lsum[map] += ((e[0] + e[1]) + (e[2] + e[3])) + ((e[4] + e[5]) + (e[6] + e[7]));
      MFrag pf;
      pf.u = make_uint4(pack_bf16x2(e[0], e[1]), pack_bf16x2(e[2], e[3]), pack_bf16x2(e[4], e[5]),
                        pack_bf16x2(e[6], e[7]));
#pragma unroll
      for (int t = 0; t < DVT; ++t)
        acc[map][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[t].v, pf.v, acc[map][t], 0, 0, 0);
    }
  }
  // a row's sum lies in its four lanes
#pragma unroll
  for (int map = 0; map < 2; ++map) {
    lsum[map] += __shfl_xor(lsum[map], 16, 64);
    lsum[map] += __shfl_xor(lsum[map], 32, 64);
  }

  // the other wavefronts hand over what they hold; the first merges in their order
  if (wave > 0) {
#pragma unroll
    for (int map = 0; map < 2; ++map) {
      if (g4 == 0) {
        stat_s[wave - 1][map][0][r] = m[map];
        stat_s[wave - 1][map][1][r] = lsum[map];
      }
#pragma unroll
      for (int t = 0; t < DVT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc_s[wave - 1][map][t][i][lane] = acc[map][t][i];
    }
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int map = 0; map < 2; ++map) {
    float m_all = m[map];
#pragma unroll
    for (int w = 0; w < AM_WAVES - 1; ++w) m_all = fmaxf(m_all, stat_s[w][map][0][r]);
    const float m_use = m_all == -INFINITY ? 0.f : m_all;
    const float mine = __builtin_amdgcn_exp2f(m[map] - m_use);
    m[map] = m_all;
    lsum[map] *= mine;
#pragma unroll
    for (int t = 0; t < DVT; ++t) acc[map][t] *= mine;
#pragma unroll
    for (int w = 0; w < AM_WAVES - 1; ++w) {
      const float theirs = __builtin_amdgcn_exp2f(stat_s[w][map][0][r] - m_use);
      lsum[map] = __builtin_fmaf(stat_s[w][map][1][r], theirs, lsum[map]);
#pragma unroll
      for (int t = 0; t < DVT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          acc[map][t][i] = __builtin_fmaf(acc_s[w][map][t][i][lane], theirs, acc[map][t][i]);
    }
  }
  if (p.splits > 1) {
    // a step of single tokens: row 0 alone is live; its four lanes leave this split's part
    if (r != 0) return;
#pragma unroll
    for (int map = 0; map < 2; ++map) {
      float* part = p.parts + ((((size_t)seq * p.heads + head) * p.splits + split) * 2 + map) * (2 + DV);
      if (g4 == 0) {
        part[0] = m[map];
        part[1] = lsum[map];
      }
#pragma unroll
      for (int t = 0; t < DVT; ++t)
        *(f32x4*)(part + 2 + t * 16 + g4 * 4) = acc[map][t];
    }
    return;
  }
  finish_head<DVT>(p, acc, lsum, token, head, g4, row_ok);
}

// The splits of a step of single tokens merged in their order, and the head finished: one
// wavefront per (sequence, head), whose lanes 0, 16, 32, 48 hold the row as in the kernel above.
template <int DVT>
__global__ __launch_bounds__(64) void attn_maps_merge_kernel(MapsParams p) {
  constexpr int DV = DVT * 16;
  const int lane = threadIdx.x, r = lane & 15, g4 = lane >> 4;
  const int seq = blockIdx.x, head = blockIdx.y;
  const int token = p.cu_q[seq];
  const bool row_ok = r == 0 && p.cu_q[seq + 1] > token;
  f32x4 acc[2][DVT];
  float lsum[2];
#pragma unroll
  for (int map = 0; map < 2; ++map) {
    const float* base = p.parts + (((size_t)seq * p.heads + head) * p.splits * 2 + map) * (2 + DV);
    const size_t step = (size_t)2 * (2 + DV);
    float m_all = -INFINITY;
    for (int s = 0; s < p.splits; ++s) m_all = fmaxf(m_all, base[s * step]);
    const float m_use = m_all == -INFINITY ? 0.f : m_all;
    lsum[map] = 0.f;
#pragma unroll
    for (int t = 0; t < DVT; ++t) acc[map][t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < p.splits; ++s) {
      const float* part = base + s * step;
      const float w = __builtin_amdgcn_exp2f(part[0] - m_use);
      lsum[map] = __builtin_fmaf(part[1], w, lsum[map]);
#pragma unroll
      for (int t = 0; t < DVT; ++t) {
        const f32x4 theirs = *(const f32x4*)(part + 2 + t * 16 + g4 * 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[map][t][i] = __builtin_fmaf(theirs[i], w, acc[map][t][i]);
      }
    }
  }
  // the lanes of other rows hold copies of row 0's values, which leaves the shuffles alone
  finish_head<DVT>(p, acc, lsum, token, head, g4, row_ok);
}

#define AM_SHAPES(X) X(1, 2) X(1, 4) X(1, 8) X(2, 2) X(2, 4) X(2, 8) X(4, 4) X(4, 8)

}  // namespace

extern "C" int mk_attention_maps_supported(int map_dim, int dv, int page_size) {
  if (page_size < 16 || !mk_is_pow2(page_size)) return 0;
#define AM_HAS(DKC, DVT) \
  if (map_dim == DKC * 32 && dv == DVT * 16) return 1;
  AM_SHAPES(AM_HAS)
#undef AM_HAS
  return 0;
}

extern "C" int mk_attention_maps(const void* q, int q_stride, void* out, const void* k_cache,
                                 const void* v_cache, const float* gate, int gate_stride,
                                 const int* positions, const int* cu_q, const int* block_table,
                                 int table_stride, int page_size, int heads, int kv_heads,
                                 int map_dim, int dv, float scale, int window, int keep_first,
                                 float lambda, float eps, float out_scale, int num_seqs,
                                 int max_q_len, int splits, float* parts, hipStream_t stream) {
  MK_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0,
             "attention_maps: %d heads over %d kv heads", heads, kv_heads);
  MK_REQUIRE(mk_attention_maps_supported(map_dim, dv, page_size),
             "attention_maps: maps of %d dims over values of %d in pages of %d are not compiled",
             map_dim, dv, page_size);
  MK_REQUIRE(window >= 0 && keep_first >= 0, "attention_maps: negative window or kept keys");
  MK_REQUIRE(q_stride >= heads * 4 * map_dim, "attention_maps: query rows of %d for %d heads",
             q_stride, heads);
  MK_REQUIRE(!gate || gate_stride >= heads, "attention_maps: gate rows of %d for %d heads",
             gate_stride, heads);
  MK_REQUIRE(num_seqs >= 0 && max_q_len >= 0 && num_seqs <= 65535 && heads <= 65535,
             "attention_maps: bad step sizes");
  MK_REQUIRE(splits >= 1 && (splits == 1 || (max_q_len == 1 && parts)),
             "attention_maps: %d splits of the keys go with a step of single tokens and a buffer",
             splits);
  if (num_seqs == 0 || max_q_len == 0) return 0;
  MK_REQUIRE(q && out && k_cache && v_cache && positions && cu_q && block_table,
             "attention_maps: null operand");
  MapsParams p;
  p.q = (const bf16_t*)q;
  p.out = (bf16_t*)out;
  p.k_cache = (const bf16_t*)k_cache;
  p.v_cache = (const bf16_t*)v_cache;
  p.gate = gate;
  p.positions = positions;
  p.cu_q = cu_q;
  p.block_table = block_table;
  p.q_stride = q_stride;
  p.gate_stride = gate_stride;
  p.table_stride = table_stride;
  p.page_shift = mk_log2(page_size);
  p.heads = heads;
  p.kv_heads = kv_heads;
  p.window = window;
  p.keep_first = window > 0 ? keep_first : 0;
  p.scale_log2 = scale * 1.4426950408889634f;
  p.lambda = lambda;
  p.eps = eps;
  p.out_scale = out_scale;
  p.splits = splits;
  p.parts = parts;
  const dim3 grid((max_q_len + 15) / 16 * splits, num_seqs, heads);
#define AM_LAUNCH(DKC, DVT)                                                    \
  if (map_dim == DKC * 32 && dv == DVT * 16) {                                 \
    attn_maps_kernel<DKC, DVT><<<grid, 64 * AM_WAVES, 0, stream>>>(p);         \
  } else
  AM_SHAPES(AM_LAUNCH) {}
#undef AM_LAUNCH
  MK_LAUNCH_CHECK("attention_maps");
  if (splits > 1) {
    const dim3 merge(num_seqs, heads);
#define AM_MERGE(DVT)                                                   \
  if (dv == DVT * 16) attn_maps_merge_kernel<DVT><<<merge, 64, 0, stream>>>(p); else
    AM_MERGE(2) AM_MERGE(4) AM_MERGE(8) {}
#undef AM_MERGE
    MK_LAUNCH_CHECK("attention_maps (merge)");
  }
  return 0;
}

// Floats of the buffer a step of single tokens needs for `splits` > 1.
extern "C" long long mk_attention_maps_parts(int num_seqs, int heads, int dv, int splits) {
  if (num_seqs < 0 || heads <= 0 || dv <= 0 || splits < 1) return -1;
  return splits == 1 ? 0 : (long long)num_seqs * heads * splits * 2 * (2 + dv);
}
