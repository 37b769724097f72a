// Causal attention of many query heads over ONE shared key/value head whose keys are wider
// than its values, on the matrix cores (bfloat16 in, float32 accumulate): the attention of a
// mixer that caches a low-rank latent per token.  A cached token is a key row [c | r] of DK
// dims and the value c of DV dims, stored once more transposed within the page
// ([page, DV, slot]) because the value-side product wants the keys as its fast index.
//
// Work is cut into tiles of 16 rows, a row being a (token, head) pair of one sequence: row f
// stands for token f / H and head f % H, so a decoded token's heads share every load of the
// cache, and a prompt portion of n tokens is ceil(n H / 16) tiles.  A wavefront owns one
// (tile, part of the keys) and needs no shared memory:
//
//   S^T[key, row]  = K[key, :] . Q[row, :]        v_mfma_f32_16x16x32_bf16, A = K, B = Q^T
//   online softmax over keys in float32, base 2 (a lane holds 8 keys of one row)
//   O^T[dim, row] += V^T[dim, key] P^T[key, row]  A = V^T, B = P^T
//
// The first product leaves a lane with the probabilities the second wants from it as B.
// Widths are multiples of 32 (keys) and 16 (values) from a list of compiled shapes; the cache
// rows and the queries are padded with zeros up to the shape by whoever writes them, so every
// loop over a width has compile-time bounds and all loads of a block of keys are asked for
// before its first product.  With the keys split into parts, every part leaves an
// unnormalised result with its running maximum and sum, and a second kernel merges the parts
// in order.
//
// With a window a row sees the keys (pos - window, pos]: a tile starts at the block of the
// first key any of its rows sees, and the lower edge is masked like the upper one.  With
// sinks a head's exp(sink) is added to the denominator of its rows where the result is
// normalised (here, or in the merge of the parts).
#include "common.h"
#include "mercury_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

union LFrag {
  bf16x8 v;
  uint4 u;
  uint2 u2[2];
};

struct LatentAttnParams {
  const bf16_t* q;       // [T, heads, DKC * 32]
  bf16_t* out;           // [T, heads, DVT * 16]
  float* part_o;         // [tile, part, DVT * 16, 16]
  float* part_ml;        // [tile, part, 2, 16]
  const bf16_t* k_cache; // [pages, page, DKC * 32]
  const bf16_t* v_cache; // [pages, DVT * 16, page]
  const int* tile_seq;
  const int* tile_row0;
  const int* cu_q;
  const int* kv_len;
  const int* block_table;
  int table_stride;
  int page_shift;
  int heads;
  float scale_log2;      // scale * log2(e)
  int num_tiles;
  int num_parts;
  int dvt;               // for the merge kernel
  int window;            // > 0: a row at position p sees keys (p - window, p] only
  const float* sinks;    // [heads] or null: exp(sink) once more in a row's denominator
};

#define LOG2E 1.4426950408889634f

#define LAT_WAVES 4

// The shapes that are compiled: (32-wide key chunks, 16-wide value tiles).  A cache is laid
// out for the first of them that holds its widths (mk_attention_latent_widths).
#define LATENT_SHAPES(X) \
  X(2, 2) X(2, 4) X(3, 4) X(4, 4) X(4, 8) X(5, 8) X(6, 8) X(8, 16) X(10, 16) X(12, 16) X(18, 32) X(20, 32)

// The wavefronts of a workgroup are independent (tile, part) units; the block size is a
// launch parameter (one wavefront a workgroup when there are few units, so that they spread
// over the compute units).
// Whether a shape's registers hold a block's keys and values at once beside the queries and
// the accumulators.  The shapes that do not keep their queries in LDS (each wavefront its own
// 16 rows, written and read by the same lanes: no barrier), take a block's keys half by half
// and its values after them, and so fit two wavefronts a SIMD.
constexpr bool latent_early(int dkc, int dvt) { return dkc * 12 + dvt * 8 <= 320; }
constexpr int latent_q_stride(int dkc) { return dkc * 32 + 8; }   // elements; 16 bytes of padding

extern __shared__ __align__(16) unsigned char latent_lds[];

template <int DKC, int DVT>
__global__ __launch_bounds__(256, (latent_early(DKC, DVT) ? 1 : 2)) void attn_latent_kernel(LatentAttnParams p) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int unit = blockIdx.x * (blockDim.x >> 6) + wave;
  if (unit >= p.num_tiles * p.num_parts) return;   // a whole wavefront; nothing is shared
  // Tiles from the last: under a causal mask the later tiles of a prompt read the most keys.
  const int tile = p.num_tiles - 1 - unit / p.num_parts;
  const int part = unit % p.num_parts;
  const int r = lane & 15, g4 = lane >> 4;
  const int seq = p.tile_seq[tile], row0 = p.tile_row0[tile];
  const int q0 = p.cu_q[seq], q_len = p.cu_q[seq + 1] - q0;
  const int kv_len = p.kv_len[seq];
  const int rows = q_len * p.heads;
  const int f = min(row0 + r, rows - 1);            // a row past the end repeats the last one
  const bool row_ok = row0 + r < rows;
  const int token = q0 + f / p.heads, head = f % p.heads;
  const int pos = kv_len - q_len + f / p.heads;
  const int last_row = min(row0 + 15, rows - 1);
  const int kmax = kv_len - q_len + last_row / p.heads;       // the tile's last visible key
  const int all_see = kv_len - q_len + row0 / p.heads;         // keys every row of it sees
  const int blocks = (kmax >> 5) + 1;
  // the first key any row sees, and the first one all of them see
  const int lo_any = p.window > 0 ? max(0, all_see - p.window + 1) : 0;
  const int lo_all = p.window > 0 ? max(0, kmax - p.window + 1) : 0;
  const int b_first = lo_any >> 5;
  const int per = (blocks - b_first + p.num_parts - 1) / p.num_parts;
  const int b_begin = b_first + part * per, b_end = min(blocks, b_begin + per);
  const int ps = 1 << p.page_shift;
  constexpr int DK = DKC * 32, DV = DVT * 16;
  const int* table = p.block_table + (size_t)seq * p.table_stride;

  constexpr bool EARLY = latent_early(DKC, DVT);
  LFrag qf[EARLY ? DKC : 1];
  bf16_t* qs = (bf16_t*)latent_lds + ((size_t)wave * 16 + r) * latent_q_stride(DKC) + g4 * 8;
  {
    const bf16_t* qrow = p.q + ((size_t)token * p.heads + head) * DK + g4 * 8;
#pragma unroll
    for (int c = 0; c < DKC; ++c) {
      if constexpr (EARLY) qf[c].u = *(const uint4*)(qrow + c * 32);
      else *(uint4*)(qs + c * 32) = *(const uint4*)(qrow + c * 32);
    }
  }
  f32x4 acc[DVT];
#pragma unroll
  for (int t = 0; t < DVT; ++t) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, lsum = 0.f;
  const float c2 = p.scale_log2;

  for (int b = b_begin; b < b_end; ++b) {
    const int key0 = b << 5;
    const bf16_t* kbase[2];
    const bf16_t* vbase[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int kh = key0 + h * 16;
      const int index = kh >> p.page_shift;
      // a half past the sequence's pages reads page 0, which exists; its keys are masked
      const int page = index < p.table_stride ? max(table[index], 0) : 0;
      const int off = kh & (ps - 1);
      kbase[h] = p.k_cache + ((size_t)page * ps + off + r) * DK + g4 * 8;
      vbase[h] = p.v_cache + ((size_t)page * DV + r) * ps + off + g4 * 4;
    }
    // Everything the block needs is asked for before the first product where the registers
    // hold it all; the widest shapes take the keys half by half and the values after them.
    LFrag vf[DVT];
    float s[8];
    if constexpr (EARLY) {
      LFrag kf[2][DKC];
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int c = 0; c < DKC; ++c) kf[h][c].u = *(const uint4*)(kbase[h] + c * 32);
#pragma unroll
      for (int t = 0; t < DVT; ++t) {
        vf[t].u2[0] = *(const uint2*)(vbase[0] + (size_t)t * 16 * ps);
        vf[t].u2[1] = *(const uint2*)(vbase[1] + (size_t)t * 16 * ps);
      }
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        f32x4 sc = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < DKC; ++c)
          sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[h][c].v, qf[c].v, sc, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) s[h * 4 + i] = sc[i];
      }
    } else {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        LFrag kf[DKC];
#pragma unroll
        for (int c = 0; c < DKC; ++c) kf[c].u = *(const uint4*)(kbase[h] + c * 32);
        f32x4 sc = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < DKC; ++c) {
          LFrag qc;
          qc.u = *(const uint4*)(qs + c * 32);
          sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[c].v, qc.v, sc, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) s[h * 4 + i] = sc[i];
        __builtin_amdgcn_sched_barrier(0);   // the next loads stay behind these products
      }
      // (the values: half of them now, the other half behind the first half's products)
#pragma unroll
      for (int t = 0; t < DVT / 2; ++t) {
        vf[t].u2[0] = *(const uint2*)(vbase[0] + (size_t)t * 16 * ps);
        vf[t].u2[1] = *(const uint2*)(vbase[1] + (size_t)t * 16 * ps);
      }
    }
    if (key0 + 31 > all_see) {   // the block holds keys some row does not see
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (key0 + h * 16 + g4 * 4 + i > pos) s[h * 4 + i] = -INFINITY;
    }
    if (key0 < lo_all) {         // keys the window of some row has passed
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (key0 + h * 16 + g4 * 4 + i <= pos - p.window) s[h * 4 + i] = -INFINITY;
    }
    float bm = c2 * fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])),
                          fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
    if (__builtin_amdgcn_ballot_w64(bm > m) != 0) {
      bm = fmaxf(bm, __shfl_xor(bm, 16, 64));
      bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
      const float m_new = fmaxf(m, bm);
      const float corr = __builtin_amdgcn_exp2f(m - (m_new == -INFINITY ? 0.f : m_new));
      lsum *= corr;
#pragma unroll
      for (int t = 0; t < DVT; ++t) acc[t] *= corr;
      m = m_new;
    }
    const float m_use = m == -INFINITY ? 0.f : m;
    float e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) e[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[j], c2, -m_use));
    lsum += ((e[0] + e[1]) + (e[2] + e[3])) + ((e[4] + e[5]) + (e[6] + e[7]));
    LFrag pf;
    pf.u = make_uint4(pack_bf16x2(e[0], e[1]), pack_bf16x2(e[2], e[3]), pack_bf16x2(e[4], e[5]),
                      pack_bf16x2(e[6], e[7]));
    if constexpr (EARLY) {
#pragma unroll
      for (int t = 0; t < DVT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[t].v, pf.v, acc[t], 0, 0, 0);
    } else {
      static_assert(EARLY || DVT % 2 == 0, "the values of a wide shape go in two halves");
#pragma unroll
      for (int t = 0; t < DVT / 2; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[t].v, pf.v, acc[t], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < DVT / 2; ++t) {
        vf[t].u2[0] = *(const uint2*)(vbase[0] + (size_t)(t + DVT / 2) * 16 * ps);
        vf[t].u2[1] = *(const uint2*)(vbase[1] + (size_t)(t + DVT / 2) * 16 * ps);
      }
#pragma unroll
      for (int t = 0; t < DVT / 2; ++t)
        acc[t + DVT / 2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[t].v, pf.v, acc[t + DVT / 2], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  // a row's sum lies in its four lanes
  lsum += __shfl_xor(lsum, 16, 64);
  lsum += __shfl_xor(lsum, 32, 64);

  if (p.num_parts == 1) {
    if (!row_ok) return;
    if (p.sinks) lsum += __builtin_amdgcn_exp2f(p.sinks[head] * LOG2E - m);
    const float inv = 1.f / lsum;
    bf16_t* dst = p.out + ((size_t)token * p.heads + head) * DV + g4 * 4;
#pragma unroll
    for (int t = 0; t < DVT; ++t)
      *(uint2*)(dst + t * 16) = make_uint2(pack_bf16x2(acc[t][0] * inv, acc[t][1] * inv),
                                           pack_bf16x2(acc[t][2] * inv, acc[t][3] * inv));
    return;
  }
  // [tile, part, dim, row]: a lane's four dims of its row
  float* po = p.part_o + ((size_t)tile * p.num_parts + part) * DV * 16;
#pragma unroll
  for (int t = 0; t < DVT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) po[(size_t)(t * 16 + g4 * 4 + i) * 16 + r] = acc[t][i];
  if (g4 == 0) {
    float* ml = p.part_ml + ((size_t)tile * p.num_parts + part) * 32;
    ml[r] = m;
    ml[16 + r] = lsum;
  }
}

// The widest shapes with the keys split into parts (decoding: few tiles, long ranges of keys):
// the four wavefronts of a workgroup take one (tile, part) together.  Each computes all the
// scores (the keys' second to fourth reading comes from the caches) but only its quarter of
// the value tiles, so its registers hold a block's keys and its values at once and every load
// of a block is on its way before the first product: one trip to memory a block, where the
// kernel above, alone with all value tiles, makes four.
template <int DKC, int DVT>
__global__ __launch_bounds__(256) void attn_latent_split_values_kernel(LatentAttnParams p) {
  static_assert(DVT % 4 == 0, "four wavefronts share the value tiles");
  constexpr int MINE = DVT / 4;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int unit = blockIdx.x;
  const int tile = p.num_tiles - 1 - unit / p.num_parts;
  const int part = unit % p.num_parts;
  const int r = lane & 15, g4 = lane >> 4;
  const int seq = p.tile_seq[tile], row0 = p.tile_row0[tile];
  const int q0 = p.cu_q[seq], q_len = p.cu_q[seq + 1] - q0;
  const int kv_len = p.kv_len[seq];
  const int rows = q_len * p.heads;
  const int f = min(row0 + r, rows - 1);
  const int token = q0 + f / p.heads, head = f % p.heads;
  const int pos = kv_len - q_len + f / p.heads;
  const int last_row = min(row0 + 15, rows - 1);
  const int kmax = kv_len - q_len + last_row / p.heads;
  const int all_see = kv_len - q_len + row0 / p.heads;
  const int blocks = (kmax >> 5) + 1;
  // the first key any row sees, and the first one all of them see
  const int lo_any = p.window > 0 ? max(0, all_see - p.window + 1) : 0;
  const int lo_all = p.window > 0 ? max(0, kmax - p.window + 1) : 0;
  const int b_first = lo_any >> 5;
  const int per = (blocks - b_first + p.num_parts - 1) / p.num_parts;
  const int b_begin = b_first + part * per, b_end = min(blocks, b_begin + per);
  const int ps = 1 << p.page_shift;
  constexpr int DK = DKC * 32, DV = DVT * 16;
  const int* table = p.block_table + (size_t)seq * p.table_stride;

  LFrag qf[DKC];
  {
    const bf16_t* qrow = p.q + ((size_t)token * p.heads + head) * DK + g4 * 8;
#pragma unroll
    for (int c = 0; c < DKC; ++c) qf[c].u = *(const uint4*)(qrow + c * 32);
  }
  f32x4 acc[MINE];
#pragma unroll
  for (int t = 0; t < MINE; ++t) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, lsum = 0.f;
  const float c2 = p.scale_log2;

  for (int b = b_begin; b < b_end; ++b) {
    const int key0 = b << 5;
    const bf16_t* kbase[2];
    const bf16_t* vbase[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int kh = key0 + h * 16;
      const int index = kh >> p.page_shift;
      const int page = index < p.table_stride ? max(table[index], 0) : 0;
      const int off = kh & (ps - 1);
      kbase[h] = p.k_cache + ((size_t)page * ps + off + r) * DK + g4 * 8;
      vbase[h] = p.v_cache + ((size_t)page * DV + wave * MINE * 16 + r) * ps + off + g4 * 4;
    }
    LFrag kf[2][DKC];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int c = 0; c < DKC; ++c) kf[h][c].u = *(const uint4*)(kbase[h] + c * 32);
    LFrag vf[MINE];
#pragma unroll
    for (int t = 0; t < MINE; ++t) {
      vf[t].u2[0] = *(const uint2*)(vbase[0] + (size_t)t * 16 * ps);
      vf[t].u2[1] = *(const uint2*)(vbase[1] + (size_t)t * 16 * ps);
    }
    float s[8];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      f32x4 sc = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < DKC; ++c)
        sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[h][c].v, qf[c].v, sc, 0, 0, 0);
#pragma unroll
      for (int i = 0; i < 4; ++i) s[h * 4 + i] = sc[i];
    }
    if (key0 + 31 > all_see) {
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (key0 + h * 16 + g4 * 4 + i > pos) s[h * 4 + i] = -INFINITY;
    }
    if (key0 < lo_all) {         // keys the window of some row has passed
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (key0 + h * 16 + g4 * 4 + i <= pos - p.window) s[h * 4 + i] = -INFINITY;
    }
    float bm = c2 * fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])),
                          fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
    if (__builtin_amdgcn_ballot_w64(bm > m) != 0) {
      bm = fmaxf(bm, __shfl_xor(bm, 16, 64));
      bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
      const float m_new = fmaxf(m, bm);
      const float corr = __builtin_amdgcn_exp2f(m - (m_new == -INFINITY ? 0.f : m_new));
      lsum *= corr;
#pragma unroll
      for (int t = 0; t < MINE; ++t) acc[t] *= corr;
      m = m_new;
    }
    const float m_use = m == -INFINITY ? 0.f : m;
    float e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) e[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[j], c2, -m_use));
    lsum += ((e[0] + e[1]) + (e[2] + e[3])) + ((e[4] + e[5]) + (e[6] + e[7]));
    LFrag pf;
    pf.u = make_uint4(pack_bf16x2(e[0], e[1]), pack_bf16x2(e[2], e[3]), pack_bf16x2(e[4], e[5]),
                      pack_bf16x2(e[6], e[7]));
#pragma unroll
    for (int t = 0; t < MINE; ++t)
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[t].v, pf.v, acc[t], 0, 0, 0);
  }
  lsum += __shfl_xor(lsum, 16, 64);
  lsum += __shfl_xor(lsum, 32, 64);
  float* po = p.part_o + ((size_t)tile * p.num_parts + part) * DV * 16;
#pragma unroll
  for (int t = 0; t < MINE; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i)
      po[(size_t)((wave * MINE + t) * 16 + g4 * 4 + i) * 16 + r] = acc[t][i];
  if (wave == 0 && g4 == 0) {   // every wavefront has the same maxima and sums
    float* ml = p.part_ml + ((size_t)tile * p.num_parts + part) * 32;
    ml[r] = m;
    ml[16 + r] = lsum;
  }
}

// Prompt portions: a workgroup takes a tile of 64 rows of one sequence, 16 a wavefront, and
// walks the keys once for all four: every block of 32 keys and its transposed values are
// brought into LDS by the whole workgroup (through registers) and read from there by each
// wavefront as its operands, so a block costs the L2 one reading for 64 rows instead of four.
// One buffer; two workgroups a compute unit, one multiplying while the other loads.  Key rows
// lie 16 bytes, value rows 16 bytes further apart than their width, against bank conflicts.
template <int DKC, int DVT>
__global__ __launch_bounds__(256, (latent_early(DKC, DVT) ? 2 : 1)) void attn_latent_staged_kernel(LatentAttnParams p) {
  constexpr int DK = DKC * 32, DV = DVT * 16;
  constexpr int KS = DK + 8, VS = 40;                 // row pitches in elements
  __shared__ __align__(16) bf16_t ks[32 * KS];
  __shared__ __align__(16) bf16_t vs[DV * VS];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g4 = lane >> 4;
  const int tile = p.num_tiles - 1 - blockIdx.x;     // the longest walks start first
  const int seq = p.tile_seq[tile], row0 = p.tile_row0[tile];
  const int q0 = p.cu_q[seq], q_len = p.cu_q[seq + 1] - q0;
  const int kv_len = p.kv_len[seq];
  const int rows = q_len * p.heads;
  const int first_pos = kv_len - q_len;
  const int my_row0 = row0 + wave * 16;
  const bool wave_live = my_row0 < rows;             // a tile's last wavefronts may have no rows
  const int f = min(my_row0 + r, rows - 1);
  const bool row_ok = my_row0 + r < rows;
  const int token = q0 + f / p.heads, head = f % p.heads;
  const int pos = first_pos + f / p.heads;
  const int my_kmax = first_pos + min(my_row0 + 15, rows - 1) / p.heads;
  const int all_see = first_pos + min(my_row0, rows - 1) / p.heads;
  const int blocks = ((first_pos + min(row0 + 63, rows - 1) / p.heads) >> 5) + 1;
  // with a window: the first key any row of the wavefront sees, the first all of them see, and
  // the block the workgroup's walk starts at
  const int lo_any = p.window > 0 ? max(0, all_see - p.window + 1) : 0;
  const int lo_all = p.window > 0 ? max(0, my_kmax - p.window + 1) : 0;
  const int b_first = p.window > 0 ? max(0, first_pos + row0 / p.heads - p.window + 1) >> 5 : 0;
  const int ps = 1 << p.page_shift;
  const int* table = p.block_table + (size_t)seq * p.table_stride;

  LFrag qf[DKC];
  {
    const bf16_t* qrow = p.q + ((size_t)token * p.heads + head) * DK + g4 * 8;
#pragma unroll
    for (int c = 0; c < DKC; ++c) qf[c].u = *(const uint4*)(qrow + c * 32);
  }
  f32x4 acc[DVT];
#pragma unroll
  for (int t = 0; t < DVT; ++t) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, lsum = 0.f;
  const float c2 = p.scale_log2;
  constexpr int K_CHUNKS = 32 * (DK / 8), V_CHUNKS = DV * 4;   // 16-byte pieces of a block
  constexpr int K_MINE = (K_CHUNKS + 255) / 256, V_MINE = (V_CHUNKS + 255) / 256;

  for (int b = b_first; b < blocks; ++b) {
    const int key0 = b << 5;
    // the two halves' places in the cache (scalars: an array indexed by the half would live
    // in scratch memory)
    const int index0 = key0 >> p.page_shift, index1 = (key0 + 16) >> p.page_shift;
    const int page0 = index0 < p.table_stride ? max(table[index0], 0) : 0;
    const int page1 = index1 < p.table_stride ? max(table[index1], 0) : 0;
    const int off0 = key0 & (ps - 1), off1 = (key0 + 16) & (ps - 1);
    // (a thread past the last piece repeats it: loads and stores without conditions)
#define LAT_K_FROM(i, dst)                                                                        \
  {                                                                                               \
    const int idx_ = min(tid + (i) * 256, K_CHUNKS - 1);                                          \
    const int key_ = idx_ / (DK / 8), ch_ = idx_ % (DK / 8);                                      \
    const size_t slot_ = key_ < 16 ? (size_t)page0 * ps + off0 + key_                             \
                                   : (size_t)page1 * ps + off1 + key_ - 16;                       \
    dst = *(const uint4*)(p.k_cache + slot_ * DK + ch_ * 8);                                      \
  }
#define LAT_K_TO(i, src)                                                                          \
  {                                                                                               \
    const int idx_ = min(tid + (i) * 256, K_CHUNKS - 1);                                          \
    *(uint4*)(ks + (idx_ / (DK / 8)) * KS + (idx_ % (DK / 8)) * 8) = src;                         \
  }
#define LAT_V_FROM(i, dst)                                                                        \
  {                                                                                               \
    const int idx_ = min(tid + (i) * 256, V_CHUNKS - 1);                                          \
    const bool second_ = (idx_ >> 1) & 1;                                                         \
    dst = *(const uint4*)(p.v_cache + ((size_t)(second_ ? page1 : page0) * DV + (idx_ >> 2)) * ps + \
                          (second_ ? off1 : off0) + (idx_ & 1) * 8);                              \
  }
#define LAT_V_TO(i, src)                                                                          \
  {                                                                                               \
    const int idx_ = min(tid + (i) * 256, V_CHUNKS - 1);                                          \
    *(uint4*)(vs + (idx_ >> 2) * VS + ((idx_ >> 1) & 1) * 16 + (idx_ & 1) * 8) = src;             \
  }
    // (named registers, not arrays: the compiler keeps such arrays in scratch memory here)
    static_assert(K_MINE <= 10 && V_MINE <= 8, "more pieces a thread than it has names for");
    uint4 k0, k1, k2, k3, k4, k5, k6, k7, k8, k9, v0, v1, v2, v3, v4, v5, v6, v7;
#define LAT_EACH_K(DO) DO(0, k0) DO(1, k1) DO(2, k2) DO(3, k3) DO(4, k4) DO(5, k5) DO(6, k6) DO(7, k7) DO(8, k8) DO(9, k9)
#define LAT_EACH_V(DO) DO(0, v0) DO(1, v1) DO(2, v2) DO(3, v3) DO(4, v4) DO(5, v5) DO(6, v6) DO(7, v7)
#define LAT_KF(i, reg) if constexpr (i < K_MINE) LAT_K_FROM(i, reg)
#define LAT_KT(i, reg) if constexpr (i < K_MINE) LAT_K_TO(i, reg)
#define LAT_VF(i, reg) if constexpr (i < V_MINE) LAT_V_FROM(i, reg)
#define LAT_VT(i, reg) if constexpr (i < V_MINE) LAT_V_TO(i, reg)
    if constexpr (latent_early(DKC, DVT)) {
      LAT_EACH_K(LAT_KF)
      LAT_EACH_V(LAT_VF)
      __syncthreads();     // whoever still reads the block before has finished
      LAT_EACH_K(LAT_KT)
      LAT_EACH_V(LAT_VT)
    } else {               // the widest shapes: keys, then values, for the registers' sake
      LAT_EACH_K(LAT_KF)
      __syncthreads();
      LAT_EACH_K(LAT_KT)
      __builtin_amdgcn_sched_barrier(0);
      LAT_EACH_V(LAT_VF)
      LAT_EACH_V(LAT_VT)
    }
#undef LAT_EACH_K
#undef LAT_EACH_V
#undef LAT_KF
#undef LAT_KT
#undef LAT_VF
#undef LAT_VT
#undef LAT_K_FROM
#undef LAT_K_TO
#undef LAT_V_FROM
#undef LAT_V_TO
    __syncthreads();
    if (!wave_live || key0 > my_kmax || key0 + 31 < lo_any) continue;   // the wavefront's rows see nothing here
    float s[8];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      f32x4 sc = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < DKC; ++c) {
        LFrag kf;
        kf.u = *(const uint4*)(ks + (h * 16 + r) * KS + c * 32 + g4 * 8);
        sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf.v, qf[c].v, sc, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) s[h * 4 + i] = sc[i];
    }
    if (key0 + 31 > all_see) {
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (key0 + h * 16 + g4 * 4 + i > pos) s[h * 4 + i] = -INFINITY;
    }
    if (key0 < lo_all) {         // keys the window of some row has passed
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (key0 + h * 16 + g4 * 4 + i <= pos - p.window) s[h * 4 + i] = -INFINITY;
    }
    float bm = c2 * fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])),
                          fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
    if (__builtin_amdgcn_ballot_w64(bm > m) != 0) {
      bm = fmaxf(bm, __shfl_xor(bm, 16, 64));
      bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
      const float m_new = fmaxf(m, bm);
      const float corr = __builtin_amdgcn_exp2f(m - (m_new == -INFINITY ? 0.f : m_new));
      lsum *= corr;
#pragma unroll
      for (int t = 0; t < DVT; ++t) acc[t] *= corr;
      m = m_new;
    }
    const float m_use = m == -INFINITY ? 0.f : m;
    float e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) e[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[j], c2, -m_use));
    lsum += ((e[0] + e[1]) + (e[2] + e[3])) + ((e[4] + e[5]) + (e[6] + e[7]));
    LFrag pf;
    pf.u = make_uint4(pack_bf16x2(e[0], e[1]), pack_bf16x2(e[2], e[3]), pack_bf16x2(e[4], e[5]),
                      pack_bf16x2(e[6], e[7]));
#pragma unroll
    for (int t = 0; t < DVT; ++t) {
      LFrag vf;
      vf.u2[0] = *(const uint2*)(vs + (t * 16 + r) * VS + g4 * 4);
      vf.u2[1] = *(const uint2*)(vs + (t * 16 + r) * VS + 16 + g4 * 4);
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pf.v, acc[t], 0, 0, 0);
    }
  }
  if (!row_ok) return;
  lsum += __shfl_xor(lsum, 16, 64);
  lsum += __shfl_xor(lsum, 32, 64);
  if (p.sinks) lsum += __builtin_amdgcn_exp2f(p.sinks[head] * LOG2E - m);
  const float inv = 1.f / lsum;
  bf16_t* dst = p.out + ((size_t)token * p.heads + head) * DV + g4 * 4;
#pragma unroll
  for (int t = 0; t < DVT; ++t)
    *(uint2*)(dst + t * 16) = make_uint2(pack_bf16x2(acc[t][0] * inv, acc[t][1] * inv),
                                         pack_bf16x2(acc[t][2] * inv, acc[t][3] * inv));
}

#define LATENT_MAX_PARTS 64

// grid (tiles, value tiles / 4): a workgroup adds up the parts' results of 64 dims of a tile's
// rows, in part order.
__global__ __launch_bounds__(256) void attn_latent_merge_kernel(LatentAttnParams p) {
  __shared__ float weight[LATENT_MAX_PARTS][16];
  __shared__ float inv[16], top[16];
  const int tile = blockIdx.x;
  const int seq = p.tile_seq[tile], row0 = p.tile_row0[tile];
  const int q0 = p.cu_q[seq], q_len = p.cu_q[seq + 1] - q0;
  const int rows = q_len * p.heads;
  const int dv = p.dvt * 16;
  const float* ml = p.part_ml + (size_t)tile * p.num_parts * 32;
  // the parts' weights: thread (part, row) first, then one thread a row for the maximum
  for (int i = threadIdx.x; i < p.num_parts * 16; i += blockDim.x)
    weight[i >> 4][i & 15] = ml[(i >> 4) * 32 + (i & 15)];
  __syncthreads();
  if (threadIdx.x < 16) {
    const int r = threadIdx.x;
    float m = -INFINITY;
    for (int s = 0; s < p.num_parts; ++s) m = fmaxf(m, weight[s][r]);
    inv[r] = m;
    top[r] = m;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < p.num_parts * 16; i += blockDim.x) {
    const float ms = weight[i >> 4][i & 15];
    weight[i >> 4][i & 15] = ms == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms - inv[i & 15]);
  }
  __syncthreads();
  if (threadIdx.x < 16) {
    const int r = threadIdx.x;
    float total = 0.f;
    for (int s = 0; s < p.num_parts; ++s) total += weight[s][r] * ml[s * 32 + 16 + r];
    if (p.sinks && row0 + r < rows) {
      total += __builtin_amdgcn_exp2f(p.sinks[(row0 + r) % p.heads] * LOG2E - top[r]);
    }
    inv[r] = 1.f / total;
  }
  __syncthreads();
  // 64 dims x 16 rows = 1024 values a workgroup, four a thread, the parts' loads eight deep
  const float* po = p.part_o + (size_t)tile * p.num_parts * dv * 16;
  const size_t stride = (size_t)dv * 16;
  const int base = blockIdx.y * 1024 + threadIdx.x;
  float total[4] = {0.f, 0.f, 0.f, 0.f};
  int s = 0;
  for (; s + 8 <= p.num_parts; s += 8) {
    float v[8][4];
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int k = 0; k < 4; ++k)
        v[j][k] = base + k * 256 < dv * 16 ? po[(size_t)(s + j) * stride + base + k * 256] : 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int k = 0; k < 4; ++k) total[k] += weight[s + j][(base + k * 256) & 15] * v[j][k];
  }
  for (; s < p.num_parts; ++s)
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if (base + k * 256 < dv * 16)
        total[k] += weight[s][(base + k * 256) & 15] * po[(size_t)s * stride + base + k * 256];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int idx = base + k * 256;
    const int d = idx >> 4, r = idx & 15;
    if (idx >= dv * 16 || row0 + r >= rows) continue;
    const int f = row0 + r;
    p.out[((size_t)(q0 + f / p.heads) * p.heads + f % p.heads) * dv + d] = f32_to_bf16(total[k] * inv[r]);
  }
}

// The widths a cache must have for keys of at least `dk` and values of at least `dv` dims:
// the first compiled shape that holds them; 0 when none does.
extern "C" int mk_attention_latent_widths(int dk, int dv, int* key_width, int* value_width) {
#define LATENT_FITS(C, T)                                 \
  if (dk <= (C) * 32 && dv <= (T) * 16) {                 \
    if (key_width) *key_width = (C) * 32;                 \
    if (value_width) *value_width = (T) * 16;             \
    return 1;                                             \
  }
  LATENT_SHAPES(LATENT_FITS)
#undef LATENT_FITS
  return 0;
}

extern "C" int mk_attention_latent_supported(int dk, int dv, int page_size) {
  if (page_size < 16 || !mk_is_pow2(page_size)) return 0;
#define LATENT_IS(C, T) if (dk == (C) * 32 && dv == (T) * 16) return 1;
  LATENT_SHAPES(LATENT_IS)
#undef LATENT_IS
  return 0;
}

extern "C" int mk_attention_latent_max_parts(void) { return LATENT_MAX_PARTS; }

extern "C" int mk_attention_latent(const void* q, void* out, const void* k_cache,
                                   const void* v_cache, const int* tile_seq, const int* tile_row0,
                                   int num_tiles, int tile_rows, const int* cu_q, const int* kv_len,
                                   const int* block_table, int table_stride, int page_size,
                                   int heads, int dk, int dv, float scale, int num_parts,
                                   float* part_o, float* part_ml, int window, const float* sinks,
                                   hipStream_t stream) {
  MK_REQUIRE(window >= 0, "latent attention: negative window");
  MK_REQUIRE(tile_rows == 16 || (tile_rows == 64 && num_parts == 1),
             "latent attention: tiles of 16 rows, or of 64 with the keys unsplit");
  MK_REQUIRE(mk_attention_latent_supported(dk, dv, page_size),
             "latent attention: keys of %d, values of %d, pages of %d are not taken", dk, dv,
             page_size);
  MK_REQUIRE(heads > 0 && num_tiles >= 0 && table_stride > 0, "latent attention: bad sizes");
  MK_REQUIRE(num_parts >= 1 && num_parts <= LATENT_MAX_PARTS, "latent attention: %d parts", num_parts);
  MK_REQUIRE(num_parts == 1 || (part_o && part_ml), "latent attention: parts without a workspace");
  MK_REQUIRE(q && out && k_cache && v_cache && tile_seq && tile_row0 && cu_q && kv_len && block_table,
             "latent attention: null argument");
  MK_REQUIRE(scale > 0.f, "latent attention: the scale must be positive");
  if (num_tiles == 0) return 0;
  LatentAttnParams p;
  p.q = (const bf16_t*)q;
  p.out = (bf16_t*)out;
  p.part_o = part_o;
  p.part_ml = part_ml;
  p.k_cache = (const bf16_t*)k_cache;
  p.v_cache = (const bf16_t*)v_cache;
  p.tile_seq = tile_seq;
  p.tile_row0 = tile_row0;
  p.cu_q = cu_q;
  p.kv_len = kv_len;
  p.block_table = block_table;
  p.table_stride = table_stride;
  p.page_shift = mk_log2(page_size);
  p.heads = heads;
  p.scale_log2 = scale * 1.4426950408889634f;
  p.num_tiles = num_tiles;
  p.num_parts = num_parts;
  p.dvt = dv / 16;
  p.window = window;
  p.sinks = sinks;
  const long long units = (long long)num_tiles * num_parts;
  // few units: one wavefront a workgroup, so that they spread over the compute units
  const int waves = units >= 2048 ? LAT_WAVES : 1;
  MK_REQUIRE((units + waves - 1) / waves < (1ll << 31), "latent attention: too many tiles");
  const dim3 grid((unsigned)((units + waves - 1) / waves));
  if (tile_rows == 64) {
#define LATENT_STAGED(C, T)                                                \
  if (dk == (C) * 32 && dv == (T) * 16)                                    \
    attn_latent_staged_kernel<C, T><<<num_tiles, 256, 0, stream>>>(p);
    LATENT_SHAPES(LATENT_STAGED)
#undef LATENT_STAGED
    MK_LAUNCH_CHECK("attention_latent_staged");
    return 0;
  }
  if (num_parts > 1 && dv == 512 && (dk == 576 || dk == 640)) {
    if (dk == 576) attn_latent_split_values_kernel<18, 32><<<(unsigned)units, 256, 0, stream>>>(p);
    else attn_latent_split_values_kernel<20, 32><<<(unsigned)units, 256, 0, stream>>>(p);
    MK_LAUNCH_CHECK("attention_latent");
    attn_latent_merge_kernel<<<dim3(num_tiles, (p.dvt + 3) / 4), 256, 0, stream>>>(p);
    MK_LAUNCH_CHECK("attention_latent_merge");
    return 0;
  }
#define LATENT_LAUNCH(C, T)                                                                  \
  if (dk == (C) * 32 && dv == (T) * 16)                                                      \
    attn_latent_kernel<C, T><<<grid, 64 * waves,                                             \
                               latent_early(C, T) ? 0 : waves * 16 * latent_q_stride(C) * 2, \
                               stream>>>(p);
  LATENT_SHAPES(LATENT_LAUNCH)
#undef LATENT_LAUNCH
  MK_LAUNCH_CHECK("attention_latent");
  if (num_parts > 1) {
    attn_latent_merge_kernel<<<dim3(num_tiles, (p.dvt + 3) / 4), 256, 0, stream>>>(p);
    MK_LAUNCH_CHECK("attention_latent_merge");
  }
  return 0;
}
