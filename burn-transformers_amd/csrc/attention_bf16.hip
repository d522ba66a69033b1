// bfloat16 attention over the paged cache on the MFMA units of gfx950, compiled once per
// head size (-DBT_HEAD_DIM=N, N a multiple of 16).
//
// Both products use v_mfma_f32_16x16x32_bf16 and are arranged so that nothing has to be
// transposed through LDS:
//   scores^T [key][query] = K . Q^T : keys are the "A" rows (a lane loads 8 consecutive channels
//       of one key), queries the "B" columns.  A lane then holds, for ONE query (lane % 16), the
//       keys 4 * (lane / 16) + r of each 16-key sub-tile, so the softmax statistics of a query
//       are a reduction over registers and over the four lanes of that column.
//   out^T [channel][query] = V^T . P^T : the probabilities a lane holds are exactly the eight
//       keys its "B" operand needs; the matching "A" operand (one channel, those eight keys) is
//       two 8-byte loads because values are stored with four consecutive positions interleaved
//       per channel.
// Softmax is online (running maximum and sum in 32-bit); excluded scores are replaced by -inf
// and values of positions that hold no token are replaced by zero before they are multiplied.
//
//   attention_prefill  one work-group per (128 queries, head, sequence); each of four waves owns
//                      32 queries (two MFMA column tiles, which share every key and value load)
//                      and walks the keys up to its last query's position.  (Four column tiles
//                      per wave were measured and were slower: they leave one wave per SIMD.)
//   attention_decode   one token per sequence: one work-group per (key/value head, sequence);
//                      the query heads sharing that head are the MFMA columns; sixteen waves
//                      (eight for heads above 64) split the keys and meet in LDS.

#include "host.h"
#include "attention.h"

#ifndef BT_HEAD_DIM
#error "compile with -DBT_HEAD_DIM=<multiple of 16>"
#endif

constexpr int HD = BT_HEAD_DIM;
constexpr int NKS = (HD + 31) / 32;  // steps of 32 channels in q . k
constexpr int ND = HD / 16;          // blocks of 16 output channels
static_assert(HD % 16 == 0 && HD >= 16 && HD <= 256, "head size must be a multiple of 16 up to 256");

__device__ __forceinline__ bf16x8 load_bf16x8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }

// The operands of one tile of 32 keys, as the MFMA lanes hold them: keys for both 16-key
// sub-tiles and every step of 32 channels, values for every block of 16 output channels.
struct TileOperands {
  bf16x8 k[2][NKS];
  bf16x4 v[ND][2];
};

// Issues the loads of one tile (kb a multiple of 32); nothing waits on them here, so the caller
// can have the next tile's loads in flight while it works on the current one.
__device__ __forceinline__ void load_tile(TileOperands& t, const bf16_t* __restrict__ kplane,
                                          const bf16_t* __restrict__ vplane, int kb) {
  const int lane = threadIdx.x & 63, i16 = lane & 15, g = lane >> 4;
  const int kin = kb & (BT_KV_BLOCK - 1);
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      int channel = ks * 32 + g * 8;
      t.k[h][ks] = channel < HD ? load_bf16x8(kplane + (kin + 16 * h + i16) * HD + channel) : zero8;
    }
#pragma unroll
  for (int dt = 0; dt < ND; ++dt) {
    int channel = dt * 16 + i16;
    t.v[dt][0] = *reinterpret_cast<const bf16x4*>(vplane + ((kin / 4 + g) * HD + channel) * 4);
    t.v[dt][1] = *reinterpret_cast<const bf16x4*>(vplane + ((kin / 4 + 4 + g) * HD + channel) * 4);
  }
}

// One tile of 32 keys starting at position kb against NQ tiles of 16 queries.
//   qpos[nq]: position of the query in column lane % 16 of tile nq, -1 if there is none.
//   valid_end: positions >= valid_end hold no token (their values are replaced by zero).
template <int NQ>
__device__ __forceinline__ void attend_tile(const TileOperands& tile, int kb, int valid_end,
                                            const int (&qpos)[NQ], int window, float scale,
                                            const bf16x8 (&q)[NQ][NKS], floatx4 (&o)[NQ][ND],
                                            float (&m)[NQ], float (&l)[NQ]) {
  const int lane = threadIdx.x & 63, g = lane >> 4;
  floatx4 s[NQ][2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq) {
      floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(tile.k[t][ks], q[nq][ks], acc, 0, 0, 0);
      s[nq][t] = acc;
    }
  }
  bf16x8 pop[NQ];
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    const int qp = qpos[nq];
    float tile_max = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        int kp = kb + 16 * t + 4 * g + r;
        bool seen = kp <= qp && (window == 0 || kp > qp - window);
        float v = seen ? s[nq][t][r] * scale : -INFINITY;
        s[nq][t][r] = v;
        tile_max = fmaxf(tile_max, v);
      }
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, 64));
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, 64));
    float m_new = fmaxf(m[nq], tile_max);
    float m_safe = m_new == -INFINITY ? 0.f : m_new;
    float alpha = __expf(m[nq] - m_safe);
    float psum = 0.f;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float p = __expf(s[nq][t][r] - m_safe);
        psum += p;
        pop[nq][4 * t + r] = (bf16_t)p;
      }
    l[nq] = l[nq] * alpha + psum;  // per-lane part of the sum; the four lanes of a column meet at the end
    m[nq] = m_new;
#pragma unroll
    for (int dt = 0; dt < ND; ++dt)
#pragma unroll
      for (int r = 0; r < 4; ++r) o[nq][dt][r] *= alpha;
  }
  const bool ragged = kb + 32 > valid_end;
#pragma unroll
  for (int dt = 0; dt < ND; ++dt) {
    bf16x4 v0 = tile.v[dt][0], v1 = tile.v[dt][1];
    if (ragged) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (kb + 4 * g + r >= valid_end) v0[r] = (bf16_t)0.f;
        if (kb + 16 + 4 * g + r >= valid_end) v1[r] = (bf16_t)0.f;
      }
    }
    bf16x8 vop = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq)
      o[nq][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vop, pop[nq], o[nq][dt], 0, 0, 0);
  }
}

// Start of the (block, kv head) plane that holds position kb of a sequence.
__device__ __forceinline__ int64_t tile_plane(const AttnArgs& a, int seq, int kv_head, int kb) {
  int block = a.kv.blocks[(int64_t)seq * a.kv.max_blocks + kb / BT_KV_BLOCK];
  return ((int64_t)block * a.kv.kv_heads + kv_head) * (int64_t)(BT_KV_BLOCK * HD);
}

#define PREFILL_NQ 2
#define PREFILL_QUERIES_PER_WAVE (16 * PREFILL_NQ)
#define PREFILL_WAVES 4
#define PREFILL_QUERIES (PREFILL_QUERIES_PER_WAVE * PREFILL_WAVES)

__global__ void __launch_bounds__(PREFILL_WAVES * 64)
attention_prefill_kernel(AttnArgs a) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, i16 = lane & 15, g = lane >> 4;
  const int seq = blockIdx.z, head = blockIdx.y;
  const int q_tile = gridDim.x - 1 - blockIdx.x;  // the longest rows of the causal triangle first
  const int kv_head = head / (a.q_heads / a.kv.kv_heads);
  const int off = a.seq_off[seq], count = a.seq_off[seq + 1] - off, start = a.seq_start[seq];
  const int q0 = q_tile * PREFILL_QUERIES + wave * PREFILL_QUERIES_PER_WAVE;
  if (q0 >= count) return;
  const bf16_t* Q = static_cast<const bf16_t*>(a.q);
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  int qpos[PREFILL_NQ], tok[PREFILL_NQ];
  bf16x8 q[PREFILL_NQ][NKS];
  floatx4 o[PREFILL_NQ][ND];
  float m[PREFILL_NQ], l[PREFILL_NQ];
#pragma unroll
  for (int nq = 0; nq < PREFILL_NQ; ++nq) {
    int qi = q0 + nq * 16 + i16;
    bool exists = qi < count;
    qpos[nq] = exists ? start + qi : -1;
    tok[nq] = off + (exists ? qi : count - 1);
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      int channel = ks * 32 + g * 8;
      q[nq][ks] = channel < HD ? load_bf16x8(Q + (int64_t)tok[nq] * a.ldq + head * HD + channel) : zero8;
    }
#pragma unroll
    for (int dt = 0; dt < ND; ++dt) o[nq][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
    m[nq] = -INFINITY;
    l[nq] = 0.f;
  }
  const int last = q0 + PREFILL_QUERIES_PER_WAVE < count ? q0 + PREFILL_QUERIES_PER_WAVE : count;
  const int hi = start + last;  // one past the position of this wave's last query
  int lo = 0;
  if (a.window > 0 && start + q0 - a.window + 1 > 0) lo = (start + q0 - a.window + 1) & ~31;
  const int valid_end = start + count;
  const bf16_t* keys = static_cast<const bf16_t*>(a.kv.keys);
  const bf16_t* values = static_cast<const bf16_t*>(a.kv.values);
  TileOperands current, next;
  if (lo < hi) {
    int64_t plane = tile_plane(a, seq, kv_head, lo);
    load_tile(next, keys + plane, values + plane, lo);
  }
  for (int kb = lo; kb < hi; kb += 32) {
    current = next;
    if (kb + 32 < hi) {
      int64_t plane = tile_plane(a, seq, kv_head, kb + 32);
      load_tile(next, keys + plane, values + plane, kb + 32);
    }
    attend_tile<PREFILL_NQ>(current, kb, valid_end, qpos, a.window, a.scale, q, o, m, l);
  }
  bf16_t* out = static_cast<bf16_t*>(a.out);
#pragma unroll
  for (int nq = 0; nq < PREFILL_NQ; ++nq) {
    float total = l[nq];
    total += __shfl_xor(total, 16, 64);
    total += __shfl_xor(total, 32, 64);
    float inv = total > 0.f ? 1.0f / total : 0.f;
    if (qpos[nq] < 0) continue;
#pragma unroll
    for (int dt = 0; dt < ND; ++dt) {
      bf16x4 packed = {(bf16_t)(o[nq][dt][0] * inv), (bf16_t)(o[nq][dt][1] * inv), (bf16_t)(o[nq][dt][2] * inv),
                       (bf16_t)(o[nq][dt][3] * inv)};
      *reinterpret_cast<bf16x4*>(out + (int64_t)tok[nq] * a.ldo + head * HD + dt * 16 + 4 * g) = packed;
    }
  }
}

// sixteen waves leave each lane 128 registers, eight leave 256: large heads need the latter
#define DECODE_WAVES (HD <= 64 ? 16 : 8)

__global__ void __launch_bounds__(DECODE_WAVES * 64)
attention_decode_kernel(AttnArgs a) {
  // per wave: maximum and sum of each query column, and its output row; `group` columns are real
  extern __shared__ float sm[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, i16 = lane & 15, g = lane >> 4;
  const int seq = blockIdx.y, kv_head = blockIdx.x;
  const int group = a.q_heads / a.kv.kv_heads;
  float* sm_m = sm;                                   // [DECODE_WAVES][group]
  float* sm_l = sm + DECODE_WAVES * group;            // [DECODE_WAVES][group]
  float* sm_o = sm + 2 * DECODE_WAVES * group;        // [DECODE_WAVES][group][HD]
  // One token per sequence, in the order of the sequences: token `seq` belongs to sequence `seq`.
  // The query, the position and (without a window) the blocks of this wave's first two tiles do
  // not depend on each other, so their loads fly together; the keys and values then need one
  // more trip to memory, not two.
  const int tok = seq;
  const bf16_t* Q = static_cast<const bf16_t*>(a.q);
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const bool has_query = i16 < group;
  const int head = kv_head * group + (has_query ? i16 : 0);
  const int stride = 32 * DECODE_WAVES;
  const int* block_row = a.kv.blocks + (int64_t)seq * a.kv.max_blocks;
  const int last_entry = a.kv.max_blocks - 1;
  int early_block0 = 0, early_block1 = 0;
  if (a.window == 0) {
    int entry0 = (32 * wave) / BT_KV_BLOCK, entry1 = (32 * wave + stride) / BT_KV_BLOCK;
    early_block0 = block_row[entry0 < last_entry ? entry0 : last_entry];
    early_block1 = block_row[entry1 < last_entry ? entry1 : last_entry];
  }
  const int pos = a.seq_start[seq];
  bf16x8 q[1][NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) {
    int channel = ks * 32 + g * 8;
    q[0][ks] = (has_query && channel < HD) ? load_bf16x8(Q + (int64_t)tok * a.ldq + head * HD + channel) : zero8;
  }
  int qpos[1] = {has_query ? pos : -1};
  floatx4 o[1][ND];
  float m[1] = {-INFINITY}, l[1] = {0.f};
#pragma unroll
  for (int dt = 0; dt < ND; ++dt) o[0][dt] = floatx4{0.f, 0.f, 0.f, 0.f};

  int lo = 0;
  if (a.window > 0 && pos - a.window + 1 > 0) lo = (pos - a.window + 1) & ~31;
  const bf16_t* keys = static_cast<const bf16_t*>(a.kv.keys);
  const bf16_t* values = static_cast<const bf16_t*>(a.kv.values);
  const int first = lo + 32 * wave;
  // plane of the tile at kb: from the blocks fetched early where they apply, else from the table
  auto plane_of = [&](int kb, int j) {
    int block = (a.window == 0 && j < 2) ? (j == 0 ? early_block0 : early_block1) : block_row[kb / BT_KV_BLOCK];
    return ((int64_t)block * a.kv.kv_heads + kv_head) * (int64_t)(BT_KV_BLOCK * HD);
  };
  TileOperands current, next;
  if (first <= pos) {
    int64_t plane = plane_of(first, 0);
    load_tile(next, keys + plane, values + plane, first);
  }
  int j = 0;
  for (int kb = first; kb <= pos; kb += stride, ++j) {
    current = next;
    if (kb + stride <= pos) {
      int64_t plane = plane_of(kb + stride, j + 1);
      load_tile(next, keys + plane, values + plane, kb + stride);
    }
    attend_tile<1>(current, kb, pos + 1, qpos, a.window, a.scale, q, o, m, l);
  }
  float total = l[0];
  total += __shfl_xor(total, 16, 64);
  total += __shfl_xor(total, 32, 64);
  if (has_query) {
    if (g == 0) {
      sm_m[wave * group + i16] = m[0];
      sm_l[wave * group + i16] = total;
    }
#pragma unroll
    for (int dt = 0; dt < ND; ++dt)
#pragma unroll
      for (int r = 0; r < 4; ++r) sm_o[(wave * group + i16) * HD + dt * 16 + 4 * g + r] = o[0][dt][r];
  }
  __syncthreads();
  bf16_t* out = static_cast<bf16_t*>(a.out);
  for (int e = threadIdx.x; e < group * HD; e += DECODE_WAVES * 64) {
    int j = e / HD, channel = e % HD;
    float top = sm_m[j];
#pragma unroll
    for (int w = 1; w < DECODE_WAVES; ++w) top = fmaxf(top, sm_m[w * group + j]);
    float num = 0.f, den = 0.f;
    if (top != -INFINITY) {
#pragma unroll
      for (int w = 0; w < DECODE_WAVES; ++w) {
        float f = __expf(sm_m[w * group + j] - top);
        num += sm_o[(w * group + j) * HD + channel] * f;
        den += sm_l[w * group + j] * f;
      }
    }
    out[(int64_t)tok * a.ldo + (kv_head * group + j) * HD + channel] = (bf16_t)(den > 0.f ? num / den : 0.f);
  }
}

static int check_args(const AttnArgs& a, const char* who) {
  if (a.kv.head_dim != HD) BT_REFUSE("%s: built for head size %d, asked for %d", who, HD, a.kv.head_dim);
  if (a.kv.kv_heads <= 0 || a.q_heads <= 0 || a.q_heads % a.kv.kv_heads != 0)
    BT_REFUSE("%s: %d query heads cannot share %d key/value heads", who, a.q_heads, a.kv.kv_heads);
  if (a.window < 0) BT_REFUSE("%s: window %d must not be negative", who, a.window);
  if (!a.q || !a.out || !a.seq_off || !a.seq_start || !a.kv.blocks || !a.kv.keys || !a.kv.values)
    BT_REFUSE("%s: missing operand", who);
  if (a.ldq % 8 != 0 || a.ldo % 4 != 0 || ((uintptr_t)a.q & 15) || ((uintptr_t)a.out & 7))
    BT_REFUSE("%s: query rows must be 16-byte and output rows 8-byte aligned", who);
  return BT_OK;
}

BT_EXPORT int bt_head_dim() { return HD; }

BT_EXPORT int bt_attention_prefill_bf16(void* stream, const AttnArgs* args) {
  if (args->n_tokens <= 0 || args->n_seqs <= 0) return BT_OK;
  int rc = check_args(*args, "attention_prefill_bf16");
  if (rc) return rc;
  if (args->max_count <= 0) BT_REFUSE("attention_prefill_bf16: max_count %d must be positive", args->max_count);
  dim3 grid((args->max_count + PREFILL_QUERIES - 1) / PREFILL_QUERIES, args->q_heads, args->n_seqs);
  hipLaunchKernelGGL(attention_prefill_kernel, grid, dim3(PREFILL_WAVES * 64), 0, (hipStream_t)stream, *args);
  return bt_check_launch("attention_prefill_bf16");
}

BT_EXPORT int bt_attention_decode_bf16(void* stream, const AttnArgs* args) {
  if (args->n_tokens <= 0 || args->n_seqs <= 0) return BT_OK;
  int rc = check_args(*args, "attention_decode_bf16");
  if (rc) return rc;
  if (args->q_heads / args->kv.kv_heads > 16)
    BT_REFUSE("attention_decode_bf16: at most 16 query heads per key/value head, got %d",
              args->q_heads / args->kv.kv_heads);
  if (args->n_tokens != args->n_seqs) BT_REFUSE("attention_decode_bf16: needs exactly one token per sequence");
  dim3 grid(args->kv.kv_heads, args->n_seqs);
  int group = args->q_heads / args->kv.kv_heads;
  size_t lds = (size_t)DECODE_WAVES * group * (HD + 2) * sizeof(float);
  hipLaunchKernelGGL(attention_decode_kernel, grid, dim3(DECODE_WAVES * 64), lds, (hipStream_t)stream, *args);
  return bt_check_launch("attention_decode_bf16");
}
