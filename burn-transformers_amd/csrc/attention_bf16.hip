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
//                      Heads of 64 without a window: eight waves, keys and values through LDS
//                      (brought there by four waves that do nothing else), each block of keys
//                      taken by one of two sets of waves (attention_prefill_split_kernel).
//   attention_decode   one token per sequence: one work-group per (key/value head, sequence)
//                      and run of keys; the query heads sharing that head are the MFMA columns;
//                      eight waves split the keys and meet in LDS; the runs of a long context
//                      are joined by attention_join_kernel.

#include "host.h"
#include "attention.h"
#include "calls.h"

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

// The online softmax of both forms below works on exponents, x = score * c - (the query's running
// maximum, which may lag: RESCALE_SLACK), computed by the one FMA that the exponential needs
// anyway.  A lane looks at its OWN exponents only; the four lanes of a query compare notes, and
// every sum is rescaled, only when some lane of the wave has an exponent above RESCALE_SLACK (or
// a query meets its first key), which after a sequence's first tiles is rare.  (The maxima are
// taken of the FMA's results, not of the scores as the matrix unit leaves them: those the
// compiler would first pass through an instruction each to quieten a signalling NaN, and an
// instruction written by hand instead is not seen by the compiler's bookkeeping of the wait
// between a matrix instruction and the first read of its result: that was a real wrong result.)
//   m: the running maximum (-inf before the first key); top: the largest exponent of the tile
//   among the query's four lanes.  Returns what to take off the tile's exponents; `alpha` is what
//   the running sums are to be multiplied with.
__device__ __forceinline__ float raise_maximum(float& m, float top, float& alpha) {
  const bool fresh = m == -INFINITY;        // the exponents were taken against 0 then
  const bool nothing = top == -INFINITY;    // every key of the tile is excluded for this query
  const float delta = fresh ? (nothing ? 0.f : top) : fmaxf(top, 0.f);
  alpha = fresh ? 1.f : exp2f(-delta);      // (sums of a fresh query are zero)
  m = fresh ? (nothing ? -INFINITY : top) : m + delta;
  return delta;
}

// The running maximum of a query may lag behind the true one by up to this many powers of two
// before the sums are rescaled: probabilities then reach at most 2^RESCALE_SLACK instead of 1,
// which 32-bit sums and bfloat16 operands (a relative format) carry as well, and the rescaling
// of every output register, three instructions each, is skipped for nearly all tiles.
#define RESCALE_SLACK 8.0f

// One tile of 32 keys starting at position kb against NQ tiles of 16 queries.
//   qpos[nq]: position of the query in column lane % 16 of tile nq, -1 if there is none.
//   valid_end: positions >= valid_end hold no token (their values are replaced by zero).
//   c: the score scale times log2(e), positive; m[] is kept in those units (powers of two).
//   MASKED = false is for tiles every query of the wave sees whole (all keys at or before the
//   first query's position, no window): nothing is compared or replaced there.  Columns without
//   a query then hold numbers nobody reads.
template <int NQ, bool MASKED>
__device__ __forceinline__ void attend_tile(const TileOperands& tile, int kb, int valid_end,
                                            const int (&qpos)[NQ], int window, float c,
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
  float own[NQ];
  bool behind = false;
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    if (MASKED) {
      const int qp = qpos[nq];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          int kp = kb + 16 * t + 4 * g + r;
          bool seen = kp <= qp && (window == 0 || kp > qp - window);
          s[nq][t][r] = seen ? s[nq][t][r] : -INFINITY;
        }
    }
    const float m_use = m[nq] == -INFINITY ? 0.f : m[nq];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) s[nq][t][r] = fmaf(s[nq][t][r], c, -m_use);
    own[nq] = fmaxf(fmaxf(fmaxf(s[nq][0][0], s[nq][0][1]), fmaxf(s[nq][0][2], s[nq][0][3])),
                    fmaxf(fmaxf(s[nq][1][0], s[nq][1][1]), fmaxf(s[nq][1][2], s[nq][1][3])));
    behind = behind || own[nq] > (m[nq] == -INFINITY ? -INFINITY : RESCALE_SLACK);
  }
  if (__builtin_amdgcn_ballot_w64(behind) != 0) {   // the same for the whole wave: a scalar branch
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq) {
      float top = own[nq];
      top = fmaxf(top, __shfl_xor(top, 16, 64));
      top = fmaxf(top, __shfl_xor(top, 32, 64));
      float alpha;
      const float delta = raise_maximum(m[nq], top, alpha);
      l[nq] *= alpha;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) s[nq][t][r] -= delta;
#pragma unroll
      for (int dt = 0; dt < ND; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) o[nq][dt][r] *= alpha;
    }
  }
  bf16x8 pop[NQ];
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    float psum = 0.f;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float p = __builtin_amdgcn_exp2f(s[nq][t][r]);
        psum += p;
        pop[nq][4 * t + r] = (bf16_t)p;
      }
    l[nq] += psum;  // per-lane part of the sum; the four lanes of a column meet at the end
  }
  const bool ragged = MASKED && kb + 32 > valid_end;
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

#define LOG2_E 1.4426950408889634f

// Start of the (block, kv head) plane that holds position kb of a sequence.
__device__ __forceinline__ int64_t tile_plane(const AttnArgs& a, int seq, int kv_head, int kb) {
  int block = a.kv.blocks[(int64_t)seq * a.kv.max_blocks + kb / BT_KV_BLOCK];
  return kv_plane(a.kv, block, kv_head);
}

#ifndef PREFILL_NQ
#define PREFILL_NQ 2
#endif
#define PREFILL_QUERIES_PER_WAVE (16 * PREFILL_NQ)
#define PREFILL_WAVES 4
#define PREFILL_QUERIES (PREFILL_QUERIES_PER_WAVE * PREFILL_WAVES)

// Heads up to 64 fit two waves on a SIMD, so that two work-groups share a compute unit; larger
// heads would spill under that limit and are left one wave.
#if BT_HEAD_DIM <= 64
#define PREFILL_OCCUPANCY __attribute__((amdgpu_waves_per_eu(2)))
#else
#define PREFILL_OCCUPANCY
#endif

template <bool PAIRED>
__global__ void __launch_bounds__((PAIRED ? 2 : 1) * PREFILL_WAVES * 64) PREFILL_OCCUPANCY
attention_prefill_kernel(AttnArgs a) {
  // the wave's number is the same in all its lanes; saying so makes the walk over the keys scalar:
  // the block table is then read through the scalar cache and tests on the position are scalar
  // branches, neither of which waits for the tiles that are in flight
  const int lane = threadIdx.x & 63;
  int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int i16 = lane & 15, g = lane >> 4;
  // Work-groups go to the eight XCDs round-robin by their number, and each XCD has an L2 of its
  // own.  All work-groups that read one (sequence, key/value head), every query tile of every
  // query head that shares it, are therefore numbered so that they land on ONE XCD: its keys and
  // values come from memory once and from that L2 afterwards (spread over all eight, the keys and
  // values of a step were read from memory eight times over, and that set the kernel's time).
  //
  // PAIRED: a work-group is two query tiles of 128, four waves each: tile i from the end of the
  // causal triangle and tile i from its start.  A query at position p walks p / 32 tiles of keys,
  // so every SIMD of a compute unit gets one long and one short wave and all finish together;
  // with a work-group per tile, the units that drew two late tiles set the kernel's time.  It is
  // used when there are more tiles than compute units (otherwise a work-group per tile spreads
  // the work further) and for heads up to 64 (eight waves leave each 256 registers).
  const int group = a.q_heads / a.kv.kv_heads;
  const int q_tiles = (a.max_count + PREFILL_QUERIES - 1) / PREFILL_QUERIES;
  const int pairs = PAIRED ? (q_tiles + 1) / 2 : q_tiles;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int unit = (slot / (group * pairs)) * 8 + xcd;      // which (sequence, key/value head)
  if (unit >= a.n_seqs * a.kv.kv_heads) return;
  const int within = slot % (group * pairs);
  const int seq = unit / a.kv.kv_heads, kv_head = unit % a.kv.kv_heads;
  const int head = kv_head * group + within % group;
  const int pair = within / group, late = q_tiles - 1 - pair;
  const bool second = PAIRED && wave >= PREFILL_WAVES;   // the wave belongs to the early tile of the pair
  if (second && pair == late) return;                    // an odd number of tiles: the middle one is alone
  const int q_tile = second ? pair : late;
  wave &= PREFILL_WAVES - 1;
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
  // The tiles alternate between two sets of registers, each named at compile time, so nothing
  // is copied: while one is multiplied the other is in flight.  (A third set, two tiles ahead,
  // costs the registers that let two work-groups share a compute unit, and measured slower.)
  const float c = a.scale * LOG2_E;
  const int whole_until = a.window == 0 ? start + q0 + 1 : 0;   // tiles ending here or before are seen whole
  // A fetch beyond the last tile reads the first one again instead of being skipped: with the same
  // number of loads in flight on every path, the wait before a tile is for that tile only.
  TileOperands t0, t1;
  auto fetch = [&](TileOperands& into, int kb) {
    const int kf = kb < hi ? kb : lo;
    int64_t plane = tile_plane(a, seq, kv_head, kf);
    load_tile(into, keys + plane, values + plane, kf);
  };
  auto attend = [&](const TileOperands& tile, int kb) {
    if (kb + 32 <= whole_until)
      attend_tile<PREFILL_NQ, false>(tile, kb, valid_end, qpos, a.window, c, q, o, m, l);
    else
      attend_tile<PREFILL_NQ, true>(tile, kb, valid_end, qpos, a.window, c, q, o, m, l);
  };
  if (lo >= hi) return;   // (cannot happen: a wave with a query sees at least that query's key)
  fetch(t0, lo);
  fetch(t1, lo + 32);
  for (int kb = lo; kb < hi; kb += 64) {
    attend(t0, kb);
    fetch(t0, kb + 64);
    if (kb + 32 < hi) attend(t1, kb + 32);
    fetch(t1, kb + 96);
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

// A whole block of 64 keys at once, for the kernel that has it in LDS.  The softmax's own
// arithmetic sets that kernel's time, so this form spends as few vector instructions per score
// as it can:
//   * maxima per lane, lanes exchanging theirs only when sums are rescaled (raise_maximum);
//   * the sums of the probabilities come from the matrix unit: one more product with a tile of
//     ones adds, for every query, exactly the bfloat16 probabilities that the output rows are
//     made of, and leaves the whole sum in every lane of the query (rows[nq][*] all equal), so
//     nothing is added up lane by lane, during the walk or after it.
//   `masked` (the same for the whole wave) says that some query of the wave does not see the
//   whole block; both kinds of block run the same instructions but for the replacement of the
//   excluded scores, so the compiler keeps every running sum in one place.
struct BlockOperands {
  bf16x8 k[4][NKS];
  bf16x8 v[ND][2];   // [block of 16 channels][half of the block's positions]: see SHARED_V_BYTES
};

template <int NQ>
__device__ __forceinline__ void attend_block(const BlockOperands& blk, int kb, int valid_end, bool masked,
                                             const int (&qpos)[NQ], float c, const bf16x8 (&q)[NQ][NKS],
                                             floatx4 (&o)[NQ][ND], float (&m)[NQ], floatx4 (&rows)[NQ]) {
  const int lane = threadIdx.x & 63, g = lane >> 4;
  floatx4 s[NQ][4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq) {
      floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(blk.k[t][ks], q[nq][ks], acc, 0, 0, 0);
      s[nq][t] = acc;
    }
  }
  if (masked) {
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq) {
      const int qp = qpos[nq];
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) s[nq][t][r] = kb + 16 * t + 4 * g + r <= qp ? s[nq][t][r] : -INFINITY;
    }
  }
  float own[NQ];
  bool behind = false;
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    const float m_use = m[nq] == -INFINITY ? 0.f : m[nq];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) s[nq][t][r] = fmaf(s[nq][t][r], c, -m_use);
    float top = -INFINITY;
#pragma unroll
    for (int t = 0; t < 4; ++t)
      top = fmaxf(top, fmaxf(fmaxf(s[nq][t][0], s[nq][t][1]), fmaxf(s[nq][t][2], s[nq][t][3])));
    own[nq] = top;
    behind = behind || top > (m[nq] == -INFINITY ? -INFINITY : RESCALE_SLACK);
  }
  if (__builtin_amdgcn_ballot_w64(behind) != 0) {   // the same for the whole wave: a scalar branch
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq) {
      float top = own[nq];
      top = fmaxf(top, __shfl_xor(top, 16, 64));
      top = fmaxf(top, __shfl_xor(top, 32, 64));
      float alpha;
      const float delta = raise_maximum(m[nq], top, alpha);
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) s[nq][t][r] -= delta;
#pragma unroll
      for (int r = 0; r < 4; ++r) rows[nq][r] *= alpha;
#pragma unroll
      for (int dt = 0; dt < ND; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) o[nq][dt][r] *= alpha;
    }
  }
  bf16x8 pop[NQ][2];
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) pop[nq][t >> 1][4 * (t & 1) + r] = (bf16_t)__builtin_amdgcn_exp2f(s[nq][t][r]);
  }
  const bf16_t one = (bf16_t)1.0f;
  const bf16x8 ones = {one, one, one, one, one, one, one, one};
#pragma unroll
  for (int half = 0; half < 2; ++half)
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq)
      rows[nq] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pop[nq][half], rows[nq], 0, 0, 0);
  const bool ragged = masked && kb + 64 > valid_end;
#pragma unroll
  for (int dt = 0; dt < ND; ++dt) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      bf16x8 vop = blk.v[dt][half];
      if (ragged) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if (kb + 32 * half + 4 * g + r >= valid_end) vop[r] = (bf16_t)0.f;
          if (kb + 32 * half + 16 + 4 * g + r >= valid_end) vop[4 + r] = (bf16_t)0.f;
        }
      }
#pragma unroll
      for (int nq = 0; nq < NQ; ++nq)
        o[nq][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vop, pop[nq][half], o[nq][dt], 0, 0, 0);
    }
  }
}

#if BT_HEAD_DIM == 64
// The same for heads of 64 without a window, with the keys and values shared through LDS: a
// block of 64 positions (8 KiB of keys, 8 KiB of values, each one contiguous plane of the cache)
// is brought in ONCE per work-group, one 16-byte piece of each per thread, while the blocks
// before it are being multiplied; every wave then reads its MFMA operands from LDS.  With each
// wave loading its own operands from memory the kernel was bound by what one compute unit can
// pull (about 25 GB/s): the four or eight waves asked for the same bytes four or eight times.
//   keys:   row r (128 bytes) keeps its 16-byte chunk c at c ^ ((r >> 1) & 7): the 16 lanes of
//           a ds_read_b128 that read one chunk of 16 consecutive rows then hit different banks;
//   values: in the order of the MFMA operand.  A lane (channel i of a block of 16, group g of the
//           lanes) multiplies, for half h of the block's positions, the eight values of positions
//           32 h + 4 g + 0..3 and 32 h + 16 + 4 g + 0..3 of its channel: those 16 bytes lie
//           together at ((4 h + g) * 64 + channel) * 16, so an operand is ONE ds_read_b128 and
//           the 16 lanes of a group read 256 consecutive bytes.  (The cache keeps four
//           consecutive positions of a channel together, so a 16-byte piece of it, two channels
//           of one group of four positions, goes to the halves of two neighbouring operands,
//           eight bytes each.  Those writes collide in the banks, four lanes to a bank; bringing
//           one channel's two groups instead, eight bytes each, and writing 16 was measured and
//           was no faster.)
#define SHARED_K_BYTES (64 * 128)
#define SHARED_V_BYTES (64 * 128)
#define SHARED_STAGE (SHARED_K_BYTES + SHARED_V_BYTES)

// The KEYS of a tile are divided between two sets of four waves:
// a work-group takes ONE tile of 128 queries, both sets hold the same queries (a wave of each set
// the same 32), a turn brings two blocks of 64 keys in, the first set multiplies the even block
// and the second the odd one, and at the end the second set hands its running maxima, sums and
// output rows to the first through LDS, lane to lane.  Against a late and an early tile paired in
// one work-group (the form of attention_prefill_kernel, which this replaced here) the longest
// chain is half as long (a tile that ends at position 1,024 walks 8 turns, not 16 blocks), and
// every SIMD has two waves at work all the time instead of one for most of it.  The tiles are
// numbered latest first over the whole grid, so that the short ones fill in behind the long
// ones.  Measured at 25 heads: 2 x 1,024 tokens 29.3 -> 27.3 us, 2,048 tokens 50.2 -> 43.2 us,
// 4 chunks of 256 tokens behind 768 28.4 -> 21.8 us.  With the leaner softmax of attend_block
// (maxima per lane, sums from the matrix unit, values in LDS in operand order): 24.5, 38.5 and
// 20.3 us, and 8,192 tokens of one sequence 503 -> 445 us (480 TFLOP/s).  What the time goes to
// then, measured by leaving parts out at 8,192 tokens: with no loads from memory, no writes to
// LDS and no barrier 290 to 320 us are left, which is the waves' own instruction streams (two
// waves per SIMD, each issuing some 115 vector instructions, 32 exponentials at a quarter of
// the rate and 36 matrix instructions per block); the loads cost 80 us, the writes 28, the
// barrier 39.  Keeping three turns in LDS, so that operands are read a turn ahead and nobody
// waits at the barrier, and reading the block table a turn ahead were both tried and gained
// nothing: the cost of those parts is their instructions, not their waiting.  So the loads and
// the writes were given to waves of their own (below): 8,192 tokens 448 -> 349 us (616 TFLOP/s),
// 2,048 tokens 38.9 -> 34.6 us, 2 x 1,024 tokens 24.7 -> 23.7 us.
#define SPLIT_TURN (2 * SHARED_STAGE)
#define SPLIT_LDS_BYTES (2 * SPLIT_TURN)

// Four more waves do nothing but bring the blocks in (SPLIT_PRODUCERS): they ask memory for the
// turn after next, write the next turn's blocks from their registers into the LDS stage that
// everyone has left, and meet the others at the turn's barrier.  The time of the eight waves
// that multiply is their own instruction streams, so what they do not have to issue they do not
// pay for, and the bringers' streams run beside them on the same SIMDs (160 registers: three
// waves a SIMD).
#define SPLIT_PRODUCERS 4
#define SPLIT_THREADS ((2 * PREFILL_WAVES + SPLIT_PRODUCERS) * 64)

__global__ void __launch_bounds__(SPLIT_THREADS)
attention_prefill_split_kernel(AttnArgs a) {
  static_assert(2 * PREFILL_WAVES * 64 == 512 && SPLIT_PRODUCERS * 64 == 256,
                "two 16-byte pieces of a block's keys and two of its values per bringing thread");
  typedef __attribute__((__vector_size__(4 * sizeof(int)))) int int4v;
  extern __shared__ __attribute__((aligned(16))) unsigned char split_lds[];   // [2 turns][2 blocks][SHARED_STAGE]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave8 = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool brings = wave8 >= 2 * PREFILL_WAVES;           // (the same for a whole wave: a scalar branch)
  const int set = wave8 / PREFILL_WAVES, wave = wave8 % PREFILL_WAVES;
  const int i16 = lane & 15, g = lane >> 4;
  // work-groups that read the same keys and values lie on one XCD (as in attention_prefill_kernel);
  // within an XCD the tiles come latest first, all (sequence, head) pairs of a rank together
  // a.splits > 1: every tile's turns are cut into that many runs, a work-group each, which leave
  // (unnormalised output row, maximum, sum) per query and head for attention_join_kernel: a chunk
  // of a prompt behind a long context has few tiles of queries and many keys for each.  What
  // shares keys is then a run of a (sequence, head) pair, and those are what is dealt to the XCDs
  // (25 heads in 5 runs: 125 over 8, where whole pairs would give one XCD 4 x 5 and the others 3 x 5).
  const int runs = a.splits > 1 ? a.splits : 1;
  const int group = a.q_heads / a.kv.kv_heads;
  const int q_tiles = (a.max_count + PREFILL_QUERIES - 1) / PREFILL_QUERIES;
  const int units = a.n_seqs * a.kv.kv_heads * runs, units_per_xcd = (units + 7) / 8;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int per_rank = units_per_xcd * group;
  const int rank = slot / per_rank, inside = slot % per_rank;
  const int unit = (inside / group) * 8 + xcd;
  if (unit >= units) return;                                // the whole work-group
  const int pair = unit / runs, run = unit % runs;
  const int seq = pair / a.kv.kv_heads, kv_head = pair % a.kv.kv_heads;
  const int head = kv_head * group + inside % group;
  const int q_tile = q_tiles - 1 - rank;
  const int off = a.seq_off[seq], count = a.seq_off[seq + 1] - off, start = a.seq_start[seq];
  if (q_tile * PREFILL_QUERIES >= count) return;            // the whole work-group: this sequence is shorter
  const int reach = (q_tile + 1) * PREFILL_QUERIES < count ? (q_tile + 1) * PREFILL_QUERIES : count;
  const int n_blocks = (start + reach + BT_KV_BLOCK - 1) / BT_KV_BLOCK;
  const int n_turns = (n_blocks + 1) / 2;
  const int per_run = (n_turns + runs - 1) / runs;
  const int t_begin = run * per_run;
  const int t_end = t_begin + per_run < n_turns ? t_begin + per_run : n_turns;
  const bool empty_run = t_begin >= t_end;                  // (the same for the whole work-group)
  // Every wave meets the others at the same barriers: one when the first turn is in place, one at
  // the end of every turn, one before the second set's results are read.

  if (brings) {
    if (empty_run) return;
    const bf16_t* keys = static_cast<const bf16_t*>(a.kv.keys);
    const bf16_t* values = static_cast<const bf16_t*>(a.kv.values);
    typedef __attribute__((__vector_size__(2 * sizeof(int)))) int int2v;
    const int mine = tid - 2 * PREFILL_WAVES * 64;           // 0 .. 255: pieces mine and mine + 256 of each plane
    int4v kreg[2][2], vreg[2][2];
    auto fetch = [&](int turn) {
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        int block_index = 2 * turn + b;
        if (block_index >= n_blocks) block_index = n_blocks - 1;     // (read again, never multiplied)
        int64_t plane = tile_plane(a, seq, kv_head, block_index * BT_KV_BLOCK);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          kreg[b][h] = *reinterpret_cast<const int4v*>(keys + plane + (mine + 256 * h) * 8);
          vreg[b][h] = *reinterpret_cast<const int4v*>(values + plane + (mine + 256 * h) * 8);
        }
      }
    };
    auto stash = [&](unsigned char* turn_base) {
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        unsigned char* stage = turn_base + b * SHARED_STAGE;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int piece = mine + 256 * h;
          const int row = piece >> 3, chunk = piece & 7;
          *reinterpret_cast<int4v*>(stage + row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4)) = kreg[b][h];
          // a piece of the values: positions 4 * four .. + 3 of channels 2 * pair and 2 * pair + 1,
          // eight bytes each, to the halves of two neighbouring operands
          const int four = piece >> 5, pair = piece & 31;
          unsigned char* place = stage + SHARED_K_BYTES + (((four >> 3) * 4 + (four & 3)) * 64 + 2 * pair) * 16 +
                                 ((four >> 2) & 1) * 8;
          *reinterpret_cast<int2v*>(place) = int2v{vreg[b][h][0], vreg[b][h][1]};
          *reinterpret_cast<int2v*>(place + 16) = int2v{vreg[b][h][2], vreg[b][h][3]};
        }
      }
    };
    fetch(t_begin);
    stash(split_lds);
    if (t_begin + 1 < t_end) fetch(t_begin + 1);
    __syncthreads();                                         // the first turn is in place
    for (int t = t_begin; t < t_end; ++t) {
      // the place of turn t + 1 was read in turn t - 1, which everyone has left
      if (t + 1 < t_end) stash(split_lds + ((t + 1 - t_begin) & 1) * SPLIT_TURN);
      if (t + 2 < t_end) fetch(t + 2);
      __syncthreads();                                       // the end of turn t
    }
    __syncthreads();                                         // (before the second set's results are read)
    return;
  }

  const int q0 = q_tile * PREFILL_QUERIES + wave * PREFILL_QUERIES_PER_WAVE;
  const bool active = q0 < count;
  const bf16_t* Q = static_cast<const bf16_t*>(a.q);

  int qpos[PREFILL_NQ], tok[PREFILL_NQ];
  bf16x8 q[PREFILL_NQ][NKS];
  floatx4 o[PREFILL_NQ][ND], rows[PREFILL_NQ];   // rows[nq][*]: the sum of query nq's probabilities
  float m[PREFILL_NQ];
#pragma unroll
  for (int nq = 0; nq < PREFILL_NQ; ++nq) {
    int qi = q0 + nq * 16 + i16;
    bool exists = active && qi < count;
    qpos[nq] = exists ? start + qi : -1;
    tok[nq] = off + (exists ? qi : count - 1);
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks)
      q[nq][ks] = load_bf16x8(Q + (int64_t)tok[nq] * a.ldq + head * HD + ks * 32 + g * 8);
#pragma unroll
    for (int dt = 0; dt < ND; ++dt) o[nq][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
    rows[nq] = floatx4{0.f, 0.f, 0.f, 0.f};
    m[nq] = -INFINITY;
  }
  const int last = q0 + PREFILL_QUERIES_PER_WAVE < count ? q0 + PREFILL_QUERIES_PER_WAVE : count;
  const int hi = active ? start + last : 0;     // one past the position of this wave's last query
  const int valid_end = start + count;
  const float c = a.scale * LOG2_E;
  const int whole_until = start + q0 + 1;       // blocks ending here or before are seen whole

  if (empty_run) {       // a run beyond the tile's last turn: its records say that it saw no key
    if (set == 0 && g == 0) {
#pragma unroll
      for (int nq = 0; nq < PREFILL_NQ; ++nq)
        if (qpos[nq] >= 0) {
          float* record = a.partial + (((int64_t)tok[nq] * a.q_heads + head) * runs + run) * (HD + 2);
          record[HD] = -INFINITY;
          record[HD + 1] = 0.f;
        }
    }
    return;
  }
  __syncthreads();                              // the first turn is in place
  for (int t = t_begin; t < t_end; ++t) {
    const int block_index = 2 * t + set;
    const int kb = block_index * BT_KV_BLOCK;
    if (block_index < n_blocks && kb < hi) {
      const unsigned char* stage = split_lds + ((t - t_begin) & 1) * SPLIT_TURN + set * SHARED_STAGE;
      BlockOperands blk;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          int row = 16 * kt + i16, chunk = ks * 4 + g;
          blk.k[kt][ks] = *reinterpret_cast<const bf16x8*>(stage + row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4));
        }
#pragma unroll
      for (int dt = 0; dt < ND; ++dt)
#pragma unroll
        for (int half = 0; half < 2; ++half)
          blk.v[dt][half] = *reinterpret_cast<const bf16x8*>(stage + SHARED_K_BYTES +
                                                             ((4 * half + g) * 64 + dt * 16 + i16) * 16);
      attend_block<PREFILL_NQ>(blk, kb, valid_end, kb + 64 > whole_until, qpos, c, q, o, m, rows);
    }
    __syncthreads();   // turn t + 1 is in place, and everyone is done with turn t before it is overwritten
  }
  // The second set's results go to the first, lane to lane: value k of lane `lane` of wave `wave`
  // at float (k * PREFILL_WAVES + wave) * 64 + lane (everyone is past the last turn's barrier).
  float* hand = reinterpret_cast<float*>(split_lds);
  constexpr int PER_QUERY = 2 + 4 * ND;
  if (set == 1) {
#pragma unroll
    for (int nq = 0; nq < PREFILL_NQ; ++nq) {
      const int k0 = nq * PER_QUERY;
      hand[((k0 + 0) * PREFILL_WAVES + wave) * 64 + lane] = m[nq];
      hand[((k0 + 1) * PREFILL_WAVES + wave) * 64 + lane] = rows[nq][0];
#pragma unroll
      for (int dt = 0; dt < ND; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) hand[((k0 + 2 + 4 * dt + r) * PREFILL_WAVES + wave) * 64 + lane] = o[nq][dt][r];
    }
  }
  __syncthreads();
  if (set == 1 || !active) return;
  bf16_t* out = static_cast<bf16_t*>(a.out);
#pragma unroll
  for (int nq = 0; nq < PREFILL_NQ; ++nq) {
    const int k0 = nq * PER_QUERY;
    const float m_other = hand[((k0 + 0) * PREFILL_WAVES + wave) * 64 + lane];
    const float l_other = hand[((k0 + 1) * PREFILL_WAVES + wave) * 64 + lane];
    const float top = fmaxf(m[nq], m_other);                       // (the maxima are kept in powers of two)
    const float mine = m[nq] == -INFINITY ? 0.f : exp2f(m[nq] - top);
    const float theirs = m_other == -INFINITY ? 0.f : exp2f(m_other - top);
    const float total = rows[nq][0] * mine + l_other * theirs;   // (whole sums: see attend_block)
    float inv = total > 0.f ? 1.0f / total : 0.f;
    if (qpos[nq] < 0) continue;
    if (runs > 1) {      // this run's share of the query's row, relative to its own maximum
      typedef __attribute__((__vector_size__(2 * sizeof(float)))) float float2v;
      float* record = a.partial + (((int64_t)tok[nq] * a.q_heads + head) * runs + run) * (HD + 2);
#pragma unroll
      for (int dt = 0; dt < ND; ++dt) {
        float joined[4];
#pragma unroll
        for (int r = 0; r < 4; ++r)
          joined[r] = o[nq][dt][r] * mine + hand[((k0 + 2 + 4 * dt + r) * PREFILL_WAVES + wave) * 64 + lane] * theirs;
        *reinterpret_cast<float2v*>(record + dt * 16 + 4 * g) = float2v{joined[0], joined[1]};
        *reinterpret_cast<float2v*>(record + dt * 16 + 4 * g + 2) = float2v{joined[2], joined[3]};
      }
      if (g == 0) {
        record[HD] = top;
        record[HD + 1] = total;
      }
      continue;
    }
#pragma unroll
    for (int dt = 0; dt < ND; ++dt) {
      float joined[4];
#pragma unroll
      for (int r = 0; r < 4; ++r)
        joined[r] = (o[nq][dt][r] * mine + hand[((k0 + 2 + 4 * dt + r) * PREFILL_WAVES + wave) * 64 + lane] * theirs) * inv;
      bf16x4 packed = {(bf16_t)joined[0], (bf16_t)joined[1], (bf16_t)joined[2], (bf16_t)joined[3]};
      *reinterpret_cast<bf16x4*>(out + (int64_t)tok[nq] * a.ldo + head * HD + dt * 16 + 4 * g) = packed;
    }
  }
}
#endif  // BT_HEAD_DIM == 64

// Eight waves: measured against sixteen and four at batches 1 to 64 (contexts of 500 to 900), eight
// are never slower, and at batch 64 a compute unit then holds two work-groups, so that one's
// reduction overlaps the other's loads (57 -> 42 us).
#define DECODE_WAVES 8

__global__ void __launch_bounds__(DECODE_WAVES * 64)
attention_decode_kernel(AttnArgs a) {
  // per wave: maximum and sum of each query column, and its output row; `group` columns are real
  extern __shared__ float sm[];
  // (the wave's number is said to be the same in all lanes, so that tests on it are scalar branches)
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int i16 = lane & 15, g = lane >> 4;
  const int seq = blockIdx.y, kv_head = blockIdx.x;
  const int splits = a.splits > 1 ? a.splits : 1, split = blockIdx.z;
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
  const bool early = a.window == 0 && splits == 1;    // (a later run's first tiles depend on the position)
  if (early) {
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
  // the tiles of 32 keys from `lo` through the query's own position, cut into `splits` runs
  const int tiles = (pos - lo) / 32 + 1, per_split = (tiles + splits - 1) / splits;
  const int tile_begin = split * per_split;
  const int tile_end = tile_begin + per_split < tiles ? tile_begin + per_split : tiles;
  const int first = lo + 32 * (tile_begin + wave), end = lo + 32 * tile_end;
  // plane of the tile at kb: from the blocks fetched early where they apply, else from the table
  auto plane_of = [&](int kb, int j) {
    int block = (early && j < 2) ? (j == 0 ? early_block0 : early_block1) : block_row[kb / BT_KV_BLOCK];
    return kv_plane(a.kv, block, kv_head);
  };
  const float c = a.scale * LOG2_E;
  auto fetch = [&](TileOperands& into, int kb, int j) {
    if (kb < end) {
      int64_t plane = plane_of(kb, j);
      load_tile(into, keys + plane, values + plane, kb);
    }
  };
  auto attend = [&](const TileOperands& tile, int kb) {   // one form: this kernel waits for memory, not for the ALU
    attend_tile<1, true>(tile, kb, pos + 1, qpos, a.window, c, q, o, m, l);
  };
  TileOperands current, next;
  fetch(next, first, 0);
  int j = 0;
  for (int kb = first; kb < end; kb += stride, ++j) {
    current = next;
    fetch(next, kb + stride, j + 1);
    attend(current, kb);
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
        float f = exp2f(sm_m[w * group + j] - top);   // the maxima are kept in powers of two
        num += sm_o[(w * group + j) * HD + channel] * f;
        den += sm_l[w * group + j] * f;
      }
    }
    if (splits == 1) {
      out[activation_offset<bf16_t>(a.out_rows, a.ldo, tok, (kv_head * group + j) * HD + channel)] =
          (bf16_t)(den > 0.f ? num / den : 0.f);
    } else {     // this run's share, for attention_join_kernel
      float* mine = a.partial + (((int64_t)seq * a.q_heads + kv_head * group + j) * splits + split) * (HD + 2);
      mine[channel] = num;
      if (channel == 0) {
        mine[HD] = top;
        mine[HD + 1] = den;
      }
    }
  }
}

// Joins the runs of attention_decode_kernel (a row is a sequence's one token) or of
// attention_prefill_split_kernel (a row is a token of the step): a wave per (row, query head),
// four to a work-group.  A run that saw no key has the maximum -inf and whatever else in its
// record.  The records of eight runs are asked for together (one trip to memory for up to eight
// runs; with a load per run and loop the kernel took 6 us for 6,400 pairs in five runs).
__global__ void __launch_bounds__(256)
attention_join_kernel(AttnArgs a, int n_rows) {
  constexpr int NCH = (HD + 63) / 64;          // channels per lane
  const int lane = threadIdx.x & 63;
  const int pair = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (pair >= n_rows * a.q_heads) return;      // (a whole wave; there is no barrier)
  const int row = pair / a.q_heads, head = pair % a.q_heads;
  const float* runs = a.partial + (int64_t)pair * a.splits * (HD + 2);
  float top = -INFINITY, den = 0.f, num[NCH];
#pragma unroll
  for (int c = 0; c < NCH; ++c) num[c] = 0.f;
  for (int s0 = 0; s0 < a.splits; s0 += 8) {
    float m[8], l[8], o[8][NCH];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const bool there = s0 + j < a.splits;
      const float* record = runs + (there ? s0 + j : s0) * (HD + 2);
      m[j] = record[HD];
      l[j] = record[HD + 1];
#pragma unroll
      for (int c = 0; c < NCH; ++c) o[j][c] = record[lane + 64 * c < HD ? lane + 64 * c : 0];
      if (!there) m[j] = -INFINITY;
    }
    float batch_top = m[0];
#pragma unroll
    for (int j = 1; j < 8; ++j) batch_top = fmaxf(batch_top, m[j]);
    const float new_top = fmaxf(top, batch_top);
    if (new_top == -INFINITY) continue;        // (the same for the whole wave)
    const float keep = top == -INFINITY ? 0.f : exp2f(top - new_top);      // (the maxima are kept in powers of two)
    den *= keep;
#pragma unroll
    for (int c = 0; c < NCH; ++c) num[c] *= keep;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (m[j] == -INFINITY) continue;
      const float f = exp2f(m[j] - new_top);
      den += l[j] * f;
#pragma unroll
      for (int c = 0; c < NCH; ++c) num[c] += o[j][c] * f;
    }
    top = new_top;
  }
  bf16_t* out = static_cast<bf16_t*>(a.out);
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int channel = lane + 64 * c;
    if (channel < HD)
      out[activation_offset<bf16_t>(a.out_rows, a.ldo, row, head * HD + channel)] = (bf16_t)(den > 0.f ? num[c] / den : 0.f);
  }
}

static int check_args(const AttnArgs& a, const char* who) {
  if (a.kv.head_dim != HD) BT_REFUSE("%s: built for head size %d, asked for %d", who, HD, a.kv.head_dim);
  if (a.kv.kv_heads <= 0 || a.q_heads <= 0 || a.q_heads % a.kv.kv_heads != 0)
    BT_REFUSE("%s: %d query heads cannot share %d key/value heads", who, a.q_heads, a.kv.kv_heads);
  if (a.window < 0) BT_REFUSE("%s: window %d must not be negative", who, a.window);
  if (!(a.scale > 0.f)) BT_REFUSE("%s: the score scale %g must be positive (the maximum is taken before scaling)", who, a.scale);
  if (!a.q || !a.out || !a.seq_off || !a.seq_start || !a.kv.blocks || !a.kv.keys || !a.kv.values)
    BT_REFUSE("%s: missing operand", who);
  if (a.ldq % 8 != 0 || a.ldo % 4 != 0 || ((uintptr_t)a.q & 15) || ((uintptr_t)a.out & 7))
    BT_REFUSE("%s: query rows must be 16-byte and output rows 8-byte aligned", who);
  return BT_OK;
}

BT_EXPORT int bt_head_dim() { return HD; }

BT_EXPORT int bt_attention_prefill_bf16(void* stream, const AttnArgs* args) {
  if (args->out_rows != 0) BT_REFUSE("attention_prefill_bf16: a chunk-major output is written by the bfloat16 decode kernel only");
  if (args->n_tokens <= 0 || args->n_seqs <= 0) return BT_OK;
  int rc = check_args(*args, "attention_prefill_bf16");
  if (rc) return rc;
  if (args->max_count <= 0) BT_REFUSE("attention_prefill_bf16: max_count %d must be positive", args->max_count);
  const int runs = args->splits > 1 ? args->splits : 1;
  if (runs > 1 && (HD != 64 || args->window != 0 || !args->partial || runs > 64))
    BT_REFUSE("attention_prefill_bf16: runs of keys (%d) are for heads of 64 without a window, at most 64, and need a place "
              "for their partial results", runs);
  const int q_tiles = (args->max_count + PREFILL_QUERIES - 1) / PREFILL_QUERIES;
  const int group = args->q_heads / args->kv.kv_heads;
  const int64_t units = (int64_t)args->n_seqs * args->kv.kv_heads;
  const int64_t units_per_xcd = (units + 7) / 8;
  static int compute_units = 0;
  if (compute_units == 0) {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&compute_units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess)
      compute_units = 256;
  }
  const bool paired = HD <= 64 && units * group * q_tiles > compute_units;
  const int64_t groups = 8 * units_per_xcd * group * (paired ? (q_tiles + 1) / 2 : q_tiles);
  if (groups > 0x7fffffff) BT_REFUSE("attention_prefill_bf16: %lld work-groups are too many", (long long)groups);
  dim3 grid((unsigned)groups);
#if BT_HEAD_DIM == 64
  if (args->window == 0) {   // keys and values shared through LDS, a tile's keys on two sets of waves
    static bool raised = false;                 // 72 KB: beyond what a kernel gets without asking
    if (!raised) {
      hipError_t err = hipFuncSetAttribute((const void*)attention_prefill_split_kernel,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)SPLIT_LDS_BYTES);
      if (err != hipSuccess) BT_REFUSE("attention_prefill_bf16: cannot get %d bytes of LDS: %s", (int)SPLIT_LDS_BYTES, hipGetErrorString(err));
      raised = true;
    }
    const int64_t split_groups = 8 * ((units * runs + 7) / 8) * group * q_tiles;
    if (split_groups > 0x7fffffff) BT_REFUSE("attention_prefill_bf16: %lld work-groups are too many", (long long)split_groups);
    hipLaunchKernelGGL(attention_prefill_split_kernel, dim3((unsigned)split_groups), dim3(SPLIT_THREADS), SPLIT_LDS_BYTES,
                       (hipStream_t)stream, *args);
    if (runs > 1) {
      rc = bt_check_launch("attention_prefill_bf16");
      if (rc) return rc;
      if ((int64_t)args->n_tokens * args->q_heads > 0x7fffffff) BT_REFUSE("attention_prefill_bf16: too many rows to join");
      hipLaunchKernelGGL(attention_join_kernel, dim3((unsigned)(((int64_t)args->n_tokens * args->q_heads + 3) / 4)), dim3(256), 0,
                         (hipStream_t)stream, *args, args->n_tokens);
    }
    return bt_check_launch("attention_prefill_bf16");
  }
#endif
  if constexpr (HD <= 64) {   // (the paired form is not even built for larger heads)
    if (paired) {
      hipLaunchKernelGGL(attention_prefill_kernel<true>, grid, dim3(2 * PREFILL_WAVES * 64), 0, (hipStream_t)stream, *args);
      return bt_check_launch("attention_prefill_bf16");
    }
  }
  hipLaunchKernelGGL(attention_prefill_kernel<false>, grid, dim3(PREFILL_WAVES * 64), 0, (hipStream_t)stream, *args);
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
  if (args->out_rows != 0 && args->out_rows < args->n_tokens)
    BT_REFUSE("attention_decode_bf16: a chunk-major output of %d rows for %d tokens", args->out_rows, args->n_tokens);
  const int splits = args->splits > 1 ? args->splits : 1;
  if (splits > 1 && !args->partial) BT_REFUSE("attention_decode_bf16: %d runs of keys need a place for their partial results", splits);
  if (splits > 65535 || args->n_seqs > 65535) BT_REFUSE("attention_decode_bf16: %d sequences in %d runs are too many", args->n_seqs, splits);
  dim3 grid(args->kv.kv_heads, args->n_seqs, splits);
  int group = args->q_heads / args->kv.kv_heads;
  size_t lds = (size_t)DECODE_WAVES * group * (HD + 2) * sizeof(float);
  hipLaunchKernelGGL(attention_decode_kernel, grid, dim3(DECODE_WAVES * 64), lds, (hipStream_t)stream, *args);
  if (splits > 1) {
    rc = bt_check_launch("attention_decode_bf16");
    if (rc) return rc;
    hipLaunchKernelGGL(attention_join_kernel, dim3((unsigned)(((int64_t)args->n_seqs * args->q_heads + 3) / 4)), dim3(256), 0,
                       (hipStream_t)stream, *args, args->n_seqs);
  }
  return bt_check_launch("attention_decode_bf16");
}

// The same entry points with their arguments as one structure (calls.h), for launch lists.
BT_EXPORT int bt_attention_prefill_bf16_call(void* stream, const AttentionCall* c) { return bt_attention_prefill_bf16(stream, &c->args); }
BT_EXPORT int bt_attention_decode_bf16_call(void* stream, const AttentionCall* c) { return bt_attention_decode_bf16(stream, &c->args); }
