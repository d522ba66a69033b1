// Attention over the paged cache in true 32-bit: the float path's kernel for prompts and for
// decoding.  Plain FMA arithmetic (no matrix cores: the float MFMA instructions would want the
// probabilities moved between lanes, and this path is the check, not the product), but tiled so
// that keys and values are read once per 32 queries instead of once per query.
//
// A work-group of four waves takes 32 consecutive queries of one sequence and one head, and walks
// the sequence's blocks of 64 keys in order:
//   * the block's keys [64][hd] and values [16][hd][4] are copied into LDS as they lie in the
//     cache (the next block's are already in flight into registers meanwhile);
//   * scores: lane = key, wave = eight of the queries; a lane reads its key row 16 bytes at a
//     time (rows padded by 16 bytes: conflict-free) against the queries' rows (broadcast reads);
//   * online softmax: a query's 64 scores lie across the lanes of one wave, so maximum and sum
//     are wave reductions in registers; excluded scores are replaced by -inf, a block that a
//     query sees nothing of changes nothing for it (exactly), and a query that sees no key at
//     all gets zeros;
//   * values: lane = channel (two channels per lane beyond 64), the same eight queries; the
//     cache's value layout (four positions interleaved per channel) makes a lane's read of four
//     keys one 16-byte LDS read, against the probabilities (broadcast reads).
// A query's result depends on its own keys and on the block boundaries only, which lie at
// multiples of 64 positions whatever the step: the same arithmetic in the same order whatever
// else the step holds.  (Steps of one token per sequence have a kernel of their own, below.)
//
// Head sizes: multiples of 16 up to 128.

#include <type_traits>

#include "host.h"
#include "attention.h"
#include "calls.h"

#define F32_QUERIES 32
#define F32_WAVE_QUERIES 8

template <int CPT>   // channels per lane: 1 (head sizes up to 64) or 2 (up to 128)
__global__ void __launch_bounds__(256)
attention_f32_kernel(AttnArgs a) {
  constexpr int MAX_HD = 64 * CPT;
  constexpr int LOADS = BT_KV_BLOCK * MAX_HD / 4 / 256;      // 16-byte pieces of a block per thread
  extern __shared__ __attribute__((aligned(16))) float lds[];  // sized for MAX_HD (lds_bytes below)
  float* qs = lds;                                             // [32][hd]
  float* ks = qs + F32_QUERIES * MAX_HD;                       // [64][hd + 4]
  float* vs = ks + BT_KV_BLOCK * (MAX_HD + 4);                 // [16][hd][4], as in the cache
  float* ps = vs + BT_KV_BLOCK * MAX_HD;                       // [32][64]

  const int hd = a.kv.head_dim;
  const int q_tiles = (a.max_count + F32_QUERIES - 1) / F32_QUERIES;
  const int seq = blockIdx.x / q_tiles, tile = blockIdx.x % q_tiles;
  const int head = blockIdx.y, kv_head = head / (a.q_heads / a.kv.kv_heads);
  const int off = a.seq_off[seq], count = a.seq_off[seq + 1] - off, start = a.seq_start[seq];
  const int q0 = tile * F32_QUERIES;
  if (q0 >= count) return;                                    // the whole work-group: no barrier is left waiting
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n_queries = count - q0 < F32_QUERIES ? count - q0 : F32_QUERIES;
  const int first_pos = start + q0, last_pos = first_pos + n_queries - 1;
  const int lo_pos = (a.window > 0 && first_pos - a.window + 1 > 0) ? first_pos - a.window + 1 : 0;
  const int first_block = lo_pos / BT_KV_BLOCK, last_block = last_pos / BT_KV_BLOCK;
  const bool wave_active = wave * F32_WAVE_QUERIES < n_queries;   // else its eight queries do not exist

  // the queries' rows; rows that do not exist stay zero and are never stored
  const float* q = static_cast<const float*>(a.q);
  for (int i = tid; i < F32_QUERIES * (hd / 4); i += 256) {
    int row = i / (hd / 4), c4 = i % (hd / 4);
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (row < n_queries) v = *reinterpret_cast<const float4*>(q + (int64_t)(off + q0 + row) * a.ldq + head * hd + c4 * 4);
    *reinterpret_cast<float4*>(qs + row * hd + c4 * 4) = v;
  }

  const float* keys = static_cast<const float*>(a.kv.keys);
  const float* values = static_cast<const float*>(a.kv.values);
  const int pieces = BT_KV_BLOCK * hd / 4;                   // 16-byte pieces of a block's keys (and of its values)
  floatx4 kreg[LOADS], vreg[LOADS];
  auto fetch = [&](int block) __attribute__((always_inline)) {
    int physical = a.kv.blocks[(int64_t)seq * a.kv.max_blocks + block];
    int64_t base = kv_plane(a.kv, physical, kv_head);
#pragma unroll
    for (int j = 0; j < LOADS; ++j) {
      int piece = tid + 256 * j;
      int at = piece < pieces ? piece : 0;                    // pieces beyond a smaller head size: read the first, keep none
      kreg[j] = *reinterpret_cast<const floatx4*>(keys + base + (int64_t)at * 4);
      vreg[j] = *reinterpret_cast<const floatx4*>(values + base + (int64_t)at * 4);
    }
  };
  // Positions behind the tile's last query hold no token of this step and may hold anything, NaN
  // included (a block that another sequence used before), and 0 * NaN is NaN: their values are
  // replaced by zero here, once per block and only in the sequence's last block, so that the
  // multiplications below need no test of their own (a select beside every FMA cost the value
  // phase half its time).  Everything at or before the last query is a token of this sequence.
  auto stage = [&](int block) __attribute__((always_inline)) {
    const int beyond = last_pos - block * BT_KV_BLOCK;        // positions of the block above this hold no token
#pragma unroll
    for (int j = 0; j < LOADS; ++j) {
      int piece = tid + 256 * j;
      if (piece < pieces) {
        int row = piece / (hd / 4), c4 = piece % (hd / 4);
        *reinterpret_cast<floatx4*>(ks + row * (hd + 4) + c4 * 4) = kreg[j];
        floatx4 v = vreg[j];
        if (beyond < BT_KV_BLOCK - 1) {                       // (the same for the whole work-group)
          int first = (piece / hd) * 4;                       // the piece holds positions first .. first + 3 of one channel
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (first + r > beyond) v[r] = 0.f;
        }
        *reinterpret_cast<floatx4*>(vs + piece * 4) = v;
      }
    }
  };

  float run_max[F32_WAVE_QUERIES], run_sum[F32_WAVE_QUERIES], acc[F32_WAVE_QUERIES][CPT];
#pragma unroll
  for (int i = 0; i < F32_WAVE_QUERIES; ++i) {
    run_max[i] = -INFINITY;
    run_sum[i] = 0.f;
#pragma unroll
    for (int j = 0; j < CPT; ++j) acc[i][j] = 0.f;
  }
  const int my_q = wave * F32_WAVE_QUERIES;                   // first of the wave's queries in the tile
  // how many of the wave's eight queries exist (one, when decoding): the same in all lanes, so
  // the tests on it below are scalar branches around work nobody needs
  const int nq = __builtin_amdgcn_readfirstlane(n_queries - my_q < F32_WAVE_QUERIES ? n_queries - my_q : F32_WAVE_QUERIES);

  fetch(first_block);
  for (int block = first_block; block <= last_block; ++block) {
    __syncthreads();                                          // the previous block's LDS is no longer read
    stage(block);
    if (block < last_block) fetch(block + 1);                 // in flight while this block is worked on
    __syncthreads();
    float rescale[F32_WAVE_QUERIES];
    // ALL: the wave's eight queries all exist (a prompt's interior): no tests in the loops
    auto score_phase = [&](auto all) __attribute__((always_inline)) {
      constexpr bool ALL = decltype(all)::value;
      // scores of key `lane` of the block for the wave's eight queries
      float s[F32_WAVE_QUERIES];
#pragma unroll
      for (int i = 0; i < F32_WAVE_QUERIES; ++i) s[i] = 0.f;
      const float* krow = ks + lane * (hd + 4);
      for (int c = 0; c < hd; c += 4) {
        float4 kv4 = *reinterpret_cast<const float4*>(krow + c);
#pragma unroll
        for (int i = 0; i < F32_WAVE_QUERIES; ++i) {
          if (!ALL && i >= nq) continue;
          float4 q4 = *reinterpret_cast<const float4*>(qs + (my_q + i) * hd + c);
          s[i] = fmaf(q4.x, kv4.x, s[i]);
          s[i] = fmaf(q4.y, kv4.y, s[i]);
          s[i] = fmaf(q4.z, kv4.z, s[i]);
          s[i] = fmaf(q4.w, kv4.w, s[i]);
        }
      }
      const int key_pos = block * BT_KV_BLOCK + lane;
#pragma unroll
      for (int i = 0; i < F32_WAVE_QUERIES; ++i) {
        rescale[i] = 1.f;
        if (!ALL && i >= nq) continue;
        int pos = first_pos + my_q + i;
        bool seen = key_pos <= pos && (a.window <= 0 || key_pos > pos - a.window);
        float score = seen ? s[i] * a.scale : -INFINITY;
        float new_max = fmaxf(run_max[i], wave_max(score));
        // nothing seen so far, this block included: everything stays at its start
        float p = new_max == -INFINITY ? 0.f : expf(score - new_max);
        rescale[i] = new_max == -INFINITY ? 1.f : expf(run_max[i] - new_max);    // exp(-inf) = 0 at the first block seen
        run_sum[i] = fmaf(run_sum[i], rescale[i], wave_sum(p));     // spelled out: the same in both forms
        run_max[i] = new_max;
        ps[(my_q + i) * BT_KV_BLOCK + lane] = p;
      }
    };
    if (wave_active) {
      if (nq == F32_WAVE_QUERIES) score_phase(std::true_type{}); else score_phase(std::false_type{});
    }
    __syncthreads();                                          // the probabilities are in LDS
    auto value_phase = [&](auto all) __attribute__((always_inline)) {
      constexpr bool ALL = decltype(all)::value;
#pragma unroll
      for (int i = 0; i < F32_WAVE_QUERIES; ++i)
#pragma unroll
        for (int j = 0; j < CPT; ++j) acc[i][j] *= rescale[i];
      // values: channel lane (+ 64) of four keys at a time.  Unrolled by two: measured at 2 x 1,024
      // tokens of 25 heads of 64, 461 / 445 / 546 us a layer unrolled by 1 / 2 / 4 (whole, the
      // compiler hoists every read above the arithmetic and spills: 1,900 us)
#pragma unroll 2
      for (int k4 = 0; k4 < BT_KV_BLOCK / 4; ++k4) {
        float4 v4[CPT];
#pragma unroll
        for (int j = 0; j < CPT; ++j) {
          int channel = lane + 64 * j;
          v4[j] = channel < hd ? *reinterpret_cast<const float4*>(vs + (k4 * hd + channel) * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int i = 0; i < F32_WAVE_QUERIES; ++i) {
          if (!ALL && i >= nq) continue;
          float4 p4 = *reinterpret_cast<const float4*>(ps + (my_q + i) * BT_KV_BLOCK + k4 * 4);
#pragma unroll
          for (int j = 0; j < CPT; ++j) {
            // (values of positions that hold no token were zeroed when the block was staged)
            acc[i][j] = fmaf(p4.x, v4[j].x, acc[i][j]);
            acc[i][j] = fmaf(p4.y, v4[j].y, acc[i][j]);
            acc[i][j] = fmaf(p4.z, v4[j].z, acc[i][j]);
            acc[i][j] = fmaf(p4.w, v4[j].w, acc[i][j]);
          }
        }
      }
    };
    if (wave_active) {
      if (nq == F32_WAVE_QUERIES) value_phase(std::true_type{}); else value_phase(std::false_type{});
    }
  }
  if (wave_active) {
    float* out = static_cast<float*>(a.out);
#pragma unroll
    for (int i = 0; i < F32_WAVE_QUERIES; ++i) {
#pragma unroll
      for (int j = 0; j < CPT; ++j) {
        int channel = lane + 64 * j;
        if (my_q + i < n_queries && channel < hd)
          out[(int64_t)(off + q0 + my_q + i) * a.ldo + head * hd + channel] = run_sum[i] > 0.f ? acc[i][j] / run_sum[i] : 0.f;
      }
    }
  }
}

// One token per sequence (a decode step): the tiled kernel above would give each work-group a
// single query and leave three of its four waves only the staging.  Here a work-group still
// takes one (sequence, head), but its four waves take the blocks of 64 keys in turn and read them
// straight from the cache: scores with lane = key (a lane reads its own key's row, the query comes
// from LDS as a broadcast), the block's softmax statistics as wave reductions, values with lane =
// channel (four keys per 16-byte read, as the cache lays them out; the probabilities come back
// from LDS as broadcasts).  The four waves' running results meet in LDS at the end.
template <int CPT>
__global__ void __launch_bounds__(256)
attention_f32_decode_kernel(AttnArgs a) {
  constexpr int MAX_HD = 64 * CPT;
  __shared__ __attribute__((aligned(16))) float qs[MAX_HD];
  __shared__ __attribute__((aligned(16))) float ps[4][BT_KV_BLOCK];
  __shared__ float part_max[4], part_sum[4];
  __shared__ __attribute__((aligned(16))) float part_acc[4][MAX_HD];
  const int hd = a.kv.head_dim;
  const int seq = blockIdx.x, head = blockIdx.y, kv_head = head / (a.q_heads / a.kv.kv_heads);
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pos = a.seq_start[seq];                     // the query's position: token `seq` of the step
  const float* q = static_cast<const float*>(a.q) + (int64_t)seq * a.ldq + head * hd;
  if (tid < hd) qs[tid] = q[tid];
  __syncthreads();
  const int lo = (a.window > 0 && pos - a.window + 1 > 0) ? pos - a.window + 1 : 0;
  int first_block = lo / BT_KV_BLOCK, last_block = pos / BT_KV_BLOCK;
  const int splits = a.splits > 1 ? a.splits : 1, split = blockIdx.z;
  if (splits > 1) {       // this work-group's run of the blocks (it may be empty)
    const int per_split = (last_block - first_block + splits) / splits;
    first_block += split * per_split;
    last_block = first_block + per_split - 1 < last_block ? first_block + per_split - 1 : last_block;
  }
  const float* keys = static_cast<const float*>(a.kv.keys);
  const float* values = static_cast<const float*>(a.kv.values);
  float run_max = -INFINITY, run_sum = 0.f, acc[CPT];
#pragma unroll
  for (int j = 0; j < CPT; ++j) acc[j] = 0.f;
  for (int block = first_block + wave; block <= last_block; block += 4) {
    int physical = a.kv.blocks[(int64_t)seq * a.kv.max_blocks + block];
    int64_t base = kv_plane(a.kv, physical, kv_head);
    // this lane's key: row `lane` of the block
    const float4* krow = reinterpret_cast<const float4*>(keys + base + (int64_t)lane * hd);
    const int quads = hd >> 2;
    float4 kreg[16 * CPT];                     // the whole row in flight at once: one trip to memory, not sixteen
#pragma unroll
    for (int c4 = 0; c4 < 16 * CPT; ++c4) kreg[c4] = krow[c4 < quads ? c4 : 0];
    float s = 0.f;
#pragma unroll
    for (int c4 = 0; c4 < 16 * CPT; ++c4) {
      if (c4 < quads) {
        float4 q4 = *reinterpret_cast<const float4*>(qs + c4 * 4);
        s = fmaf(q4.x, kreg[c4].x, s);
        s = fmaf(q4.y, kreg[c4].y, s);
        s = fmaf(q4.z, kreg[c4].z, s);
        s = fmaf(q4.w, kreg[c4].w, s);
      }
    }
    const int key_pos = block * BT_KV_BLOCK + lane;
    const bool seen = key_pos <= pos && key_pos >= lo;
    const float score = seen ? s * a.scale : -INFINITY;
    const float new_max = fmaxf(run_max, wave_max(score));          // finite: the block holds at least one seen key
    const float p = expf(score - new_max);
    const float rescale = expf(run_max - new_max);                  // exp(-inf) = 0 at the wave's first block
    run_sum = fmaf(run_sum, rescale, wave_sum(p));
    run_max = new_max;
    ps[wave][lane] = p;                                             // read back below by this wave only
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int j = 0; j < CPT; ++j) acc[j] *= rescale;
#pragma unroll
    for (int j = 0; j < CPT; ++j) {
      const int channel = lane + 64 * j;
      const int cc = channel < hd ? channel : 0;
      float4 vreg[BT_KV_BLOCK / 4];            // the channel's 64 values in flight at once
#pragma unroll
      for (int k4 = 0; k4 < BT_KV_BLOCK / 4; ++k4)
        vreg[k4] = *reinterpret_cast<const float4*>(values + base + (int64_t)(k4 * hd + cc) * 4);
#pragma unroll
      for (int k4 = 0; k4 < BT_KV_BLOCK / 4; ++k4) {
        float4 p4 = *reinterpret_cast<const float4*>(&ps[wave][k4 * 4]);
        // a position that holds no token yet may hold anything (0 * NaN is NaN): not multiplied
        acc[j] = p4.x != 0.f ? fmaf(p4.x, vreg[k4].x, acc[j]) : acc[j];
        acc[j] = p4.y != 0.f ? fmaf(p4.y, vreg[k4].y, acc[j]) : acc[j];
        acc[j] = p4.z != 0.f ? fmaf(p4.z, vreg[k4].z, acc[j]) : acc[j];
        acc[j] = p4.w != 0.f ? fmaf(p4.w, vreg[k4].w, acc[j]) : acc[j];
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");          // the probabilities are overwritten next turn
    __builtin_amdgcn_wave_barrier();
  }
  if (lane == 0) {
    part_max[wave] = run_max;
    part_sum[wave] = run_sum;
  }
#pragma unroll
  for (int j = 0; j < CPT; ++j)
    if (lane + 64 * j < hd) part_acc[wave][lane + 64 * j] = acc[j];
  __syncthreads();
  if (wave == 0) {
    float top = fmaxf(fmaxf(part_max[0], part_max[1]), fmaxf(part_max[2], part_max[3]));
    float* out = static_cast<float*>(a.out) + (int64_t)seq * a.ldo + head * hd;
    float* mine = splits > 1 ? a.partial + (((int64_t)seq * a.q_heads + head) * splits + split) * (hd + 2) : nullptr;
#pragma unroll
    for (int j = 0; j < CPT; ++j) {
      int channel = lane + 64 * j;
      if (channel >= hd) continue;
      float num = 0.f, den = 0.f;
#pragma unroll
      for (int w = 0; w < 4; ++w) {                                 // a wave that had no block: maximum -inf, weight 0
        float f = part_max[w] == -INFINITY ? 0.f : expf(part_max[w] - top);
        num = fmaf(part_acc[w][channel], f, num);
        den = fmaf(part_sum[w], f, den);
      }
      if (splits == 1) {
        out[channel] = den > 0.f ? num / den : 0.f;
      } else {                                                      // this run's share, for attention_f32_join_kernel
        mine[channel] = num;
        if (channel == 0) {
          mine[hd] = top;
          mine[hd + 1] = den;
        }
      }
    }
  }
}

// Joins the runs of attention_f32_decode_kernel: a work-group of one wave per (sequence, head).
__global__ void __launch_bounds__(64)
attention_f32_join_kernel(AttnArgs a) {
  const int hd = a.kv.head_dim;
  const int seq = blockIdx.x / a.q_heads, head = blockIdx.x % a.q_heads;
  const float* runs = a.partial + ((int64_t)seq * a.q_heads + head) * a.splits * (hd + 2);
  float top = -INFINITY;
  for (int s = 0; s < a.splits; ++s) top = fmaxf(top, runs[s * (hd + 2) + hd]);
  float* out = static_cast<float*>(a.out) + (int64_t)seq * a.ldo + head * hd;
  for (int channel = threadIdx.x; channel < hd; channel += 64) {
    float num = 0.f, den = 0.f;
    for (int s = 0; s < a.splits; ++s) {                            // an empty run: maximum -inf, weight 0
      float run_top = runs[s * (hd + 2) + hd];
      float f = run_top == -INFINITY ? 0.f : expf(run_top - top);
      num = fmaf(runs[s * (hd + 2) + channel], f, num);
      den = fmaf(runs[s * (hd + 2) + hd + 1], f, den);
    }
    out[channel] = den > 0.f ? num / den : 0.f;
  }
}

BT_EXPORT int bt_attention_f32(void* stream, const AttnArgs* args) {
  if (args->out_rows != 0) BT_REFUSE("attention_f32: a chunk-major output is written by the bfloat16 decode kernel only");
  const AttnArgs& a = *args;
  if (a.n_tokens <= 0 || a.n_seqs <= 0) return BT_OK;
  const int hd = a.kv.head_dim;
  if (hd <= 0 || hd % 16 != 0 || hd > 128) BT_REFUSE("attention_f32: head size %d must be a multiple of 16 up to 128", hd);
  if (a.kv.kv_heads <= 0 || a.q_heads <= 0 || a.q_heads % a.kv.kv_heads != 0)
    BT_REFUSE("attention_f32: %d query heads cannot share %d key/value heads", a.q_heads, a.kv.kv_heads);
  if (a.window < 0) BT_REFUSE("attention_f32: window %d must not be negative", a.window);
  if (a.max_count <= 0) BT_REFUSE("attention_f32: max_count %d must be positive", a.max_count);
  if (!(a.scale > 0.f)) BT_REFUSE("attention_f32: scale %g must be positive", (double)a.scale);
  if (!a.q || !a.out || !a.seq_off || !a.seq_start || !a.kv.blocks || !a.kv.keys || !a.kv.values)
    BT_REFUSE("attention_f32: missing operand");
  if (a.ldq % 4 != 0 || ((uintptr_t)a.q & 15) || ((uintptr_t)a.kv.keys & 15) || ((uintptr_t)a.kv.values & 15))
    BT_REFUSE("attention_f32: queries, keys and values are read 16 bytes at a time (row pitch %lld)", (long long)a.ldq);
  if (a.max_count == 1 && a.n_tokens == a.n_seqs) {      // a decode step: one token per sequence, in their order
    const int splits = a.splits > 1 ? a.splits : 1;
    if (splits > 1 && !a.partial) BT_REFUSE("attention_f32: %d runs of keys need a place for their partial results", splits);
    if (splits > 65535 || a.q_heads > 65535) BT_REFUSE("attention_f32: %d heads in %d runs are too many", a.q_heads, splits);
    dim3 grid(a.n_seqs, a.q_heads, splits);
    if (hd <= 64)
      hipLaunchKernelGGL(attention_f32_decode_kernel<1>, grid, dim3(256), 0, (hipStream_t)stream, a);
    else
      hipLaunchKernelGGL(attention_f32_decode_kernel<2>, grid, dim3(256), 0, (hipStream_t)stream, a);
    if (splits > 1) {
      int rc = bt_check_launch("attention_f32");
      if (rc) return rc;
      hipLaunchKernelGGL(attention_f32_join_kernel, dim3((unsigned)a.n_seqs * a.q_heads), dim3(64), 0, (hipStream_t)stream, a);
    }
    return bt_check_launch("attention_f32");
  }
  const int q_tiles = (a.max_count + F32_QUERIES - 1) / F32_QUERIES;
  dim3 grid(a.n_seqs * q_tiles, a.q_heads), block(256);
  auto lds_bytes = [](int max_hd) {
    return sizeof(float) * (size_t)(F32_QUERIES * max_hd + BT_KV_BLOCK * (max_hd + 4) + BT_KV_BLOCK * max_hd +
                                    F32_QUERIES * BT_KV_BLOCK);
  };
  if (hd <= 64) {
    hipLaunchKernelGGL(attention_f32_kernel<1>, grid, block, lds_bytes(64), (hipStream_t)stream, a);
  } else {
    static bool raised = false;                 // 90 KB: beyond what a kernel gets without asking
    if (!raised) {
      hipError_t err = hipFuncSetAttribute((const void*)attention_f32_kernel<2>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes(128));
      if (err != hipSuccess) BT_REFUSE("attention_f32: cannot get %zu bytes of LDS: %s", lds_bytes(128), hipGetErrorString(err));
      raised = true;
    }
    hipLaunchKernelGGL(attention_f32_kernel<2>, grid, block, lds_bytes(128), (hipStream_t)stream, a);
  }
  return bt_check_launch("attention_f32");
}

// The same entry points with their arguments as one structure (calls.h), for launch lists.
BT_EXPORT int bt_attention_f32_call(void* stream, const AttentionCall* c) { return bt_attention_f32(stream, &c->args); }
