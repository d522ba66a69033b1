// Attention over the paged cache in true 32-bit: the float path's kernels for prompts and for
// decoding.  Head sizes: multiples of 16 up to 128 (others take the plain kernel).
//
// Prompts and chunks run on the matrix units.  v_mfma_f32_16x16x4_f32 multiplies and adds in full
// 32-bit (no reduced-precision mode exists in it), and the arrangement of the bfloat16 kernels
// needs no probabilities moved between lanes here either:
//   scores^T [key][query] = K . Q^T: keys are the "A" rows, queries the "B" columns, and a lane
//       (column lane % 16, group g = lane / 16) ends up with keys 4 g + r (r = 0..3) of each tile
//       of 16 keys for ONE query.  A 16-byte read gives a lane four channels; the four
//       instructions that take them multiply channel 16 c + 4 g + r in K index g of step r, the
//       same for both operands, so every channel is taken exactly once.
//   out^T [channel][query] = V^T . P^T: in step r of a tile of 16 keys the K index g stands for
//       key 4 g + r, so the "B" operand is the lane's OWN probability r, and the "A" operand
//       (channel lane % 16 of a block of 16 channels, key 4 g + r) is element r of ONE 16-byte
//       read, because the cache keeps four consecutive positions of a channel together.
// A work-group of four waves takes 64 consecutive queries of one sequence and head, 16 per wave,
// and walks the sequence's blocks of 64 keys up to its last query:
//   * the block's keys [64][hd] (rows 16 bytes apart in the banks) and values [16][hd][4] are
//     copied into LDS as they lie in the cache, once per work-group (the next block's are already
//     in flight into registers meanwhile);
//   * the softmax is per query and per block of 64 keys: maximum, rescaling and sum are taken
//     anew at every block, nothing lags; excluded scores are replaced by -inf, a block that a
//     query sees nothing of changes nothing for it (exactly), and a query that sees no key at all
//     gets zeros;
//   * values of positions behind the tile's last query (which may hold anything, NaN included,
//     and 0 * NaN is NaN) are replaced by zero once, when the block is staged.
// A query's result depends on its own keys and on the block boundaries only, which lie at
// multiples of 64 positions whatever the step: the same arithmetic in the same order whatever
// else the step holds.  (Steps of one token per sequence have a kernel of their own, below.)
// Measured at 25 heads of 64, 2 x 1,024 tokens: 87 us a layer, 77 TFLOP/s, half of the float
// MFMA peak; the FMA kernel this replaced (lane = key for the scores, lane = channel for the
// values, probabilities through LDS) took 445 us.
#include "host.h"
#include "attention.h"
#include "calls.h"

#define F32M_QUERIES 64

template <int HD>
__global__ void __launch_bounds__(256)
attention_f32_mfma_kernel(AttnArgs a) {
  constexpr int KS = HD / 16;                                // 16-byte reads of a row per lane; blocks of 16 channels
  constexpr int LOADS = BT_KV_BLOCK * HD / 4 / 256;          // 16-byte pieces of a block per thread
  constexpr int K_ROW = HD + 4;                              // floats: rows 16 bytes apart in the banks
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* ks = lds;                                           // [64][HD + 4]
  float* vs = ks + BT_KV_BLOCK * K_ROW;                      // [16][HD][4], as in the cache

  // The tiles are numbered latest first over the whole grid: a tile's walk is as long as its
  // position, nearly all work-groups are resident at once, and a compute unit is given every
  // 256th of them, so that each gets long and short ones.  (Numbered sequence by sequence, a
  // unit drew tiles of one length: 152 -> 87 us a layer at 2 x 1,024 tokens of 25 heads.)
  const int q_tiles = (a.max_count + F32M_QUERIES - 1) / F32M_QUERIES;
  const int units = a.n_seqs * a.q_heads;
  const int tile = q_tiles - 1 - blockIdx.x / units, unit = blockIdx.x % units;
  const int seq = unit / a.q_heads, head = unit % a.q_heads, kv_head = head / (a.q_heads / a.kv.kv_heads);
  const int off = a.seq_off[seq], count = a.seq_off[seq + 1] - off, start = a.seq_start[seq];
  const int q0 = tile * F32M_QUERIES;
  if (q0 >= count) return;                                   // the whole work-group: no barrier is left waiting
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int i16 = lane & 15, g = lane >> 4;
  const int n_queries = count - q0 < F32M_QUERIES ? count - q0 : F32M_QUERIES;
  const int first_pos = start + q0, last_pos = first_pos + n_queries - 1;
  const int lo_pos = (a.window > 0 && first_pos - a.window + 1 > 0) ? first_pos - a.window + 1 : 0;
  const int first_block = lo_pos / BT_KV_BLOCK, last_block = last_pos / BT_KV_BLOCK;
  const bool wave_active = wave * 16 < n_queries;
  // what the wave's queries can see at all: positions wave_lo .. wave_hi
  const int wave_first = first_pos + wave * 16;
  const int wave_hi = wave_first + 15 < last_pos ? wave_first + 15 : last_pos;
  const int wave_lo = (a.window > 0 && wave_first - a.window + 1 > 0) ? wave_first - a.window + 1 : 0;
  const int mine = wave * 16 + i16;                          // the lane's query within the tile
  const bool exists = wave_active && mine < n_queries;
  const int qpos = exists ? first_pos + mine : -1;           // (a column without a query sees no key and is never stored)

  const float* q = static_cast<const float*>(a.q);
  floatx4 qreg[KS];
  {
    const float* row = q + (int64_t)(off + q0 + (exists ? mine : 0)) * a.ldq + head * HD;
#pragma unroll
    for (int c = 0; c < KS; ++c) qreg[c] = *reinterpret_cast<const floatx4*>(row + 16 * c + 4 * g);
  }

  const float* keys = static_cast<const float*>(a.kv.keys);
  const float* values = static_cast<const float*>(a.kv.values);
  floatx4 kreg[LOADS], vreg[LOADS];
  auto fetch = [&](int block) __attribute__((always_inline)) {
    int physical = a.kv.blocks[(int64_t)seq * a.kv.max_blocks + block];
    int64_t base = kv_plane(a.kv, physical, kv_head);
#pragma unroll
    for (int j = 0; j < LOADS; ++j) {
      int piece = tid + 256 * j;
      kreg[j] = *reinterpret_cast<const floatx4*>(keys + base + (int64_t)piece * 4);
      vreg[j] = *reinterpret_cast<const floatx4*>(values + base + (int64_t)piece * 4);
    }
  };
  // (values of positions behind the tile's last query become zero here, once per block and only
  // in the sequence's last block, so that the multiplications need no test of their own)
  auto stage = [&](int block) __attribute__((always_inline)) {
    const int beyond = last_pos - block * BT_KV_BLOCK;
#pragma unroll
    for (int j = 0; j < LOADS; ++j) {
      int piece = tid + 256 * j;
      int row = piece / (HD / 4), c4 = piece % (HD / 4);
      *reinterpret_cast<floatx4*>(ks + row * K_ROW + c4 * 4) = kreg[j];
      floatx4 v = vreg[j];
      if (beyond < BT_KV_BLOCK - 1) {                        // (the same for the whole work-group)
        int first = (piece / HD) * 4;                        // the piece holds positions first .. first + 3 of one channel
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (first + r > beyond) v[r] = 0.f;
      }
      *reinterpret_cast<floatx4*>(vs + piece * 4) = v;
    }
  };

  const float c2 = a.scale * 1.4426950408889634f;            // scores to powers of two
  float run_max = -INFINITY, run_sum = 0.f;                  // run_sum: the lane's share; the four lanes of a query meet at the end
  floatx4 o[KS];
#pragma unroll
  for (int dt = 0; dt < KS; ++dt) o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};

  fetch(first_block);
  for (int block = first_block; block <= last_block; ++block) {
    __syncthreads();                                         // the previous block's LDS is no longer read
    stage(block);
    if (block < last_block) fetch(block + 1);                // in flight while this block is worked on
    __syncthreads();
    const int kb = block * BT_KV_BLOCK;
    if (!wave_active || kb > wave_hi || kb + BT_KV_BLOCK <= wave_lo) continue;   // (the same for the whole wave)
    // Operands are asked for a step before they are multiplied (two sets of registers, named at
    // compile time), and the four tiles' sums (then the blocks of output channels) take turns, so
    // that neither an LDS read nor a matrix instruction waits for the one before it.
    floatx4 s[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) s[t] = floatx4{0.f, 0.f, 0.f, 0.f};
    const float* krow = ks + i16 * K_ROW + 4 * g;
    floatx4 k4[2][4];
#pragma unroll
    for (int t = 0; t < 4; ++t) k4[0][t] = *reinterpret_cast<const floatx4*>(krow + 16 * t * K_ROW);
#pragma unroll
    for (int c = 0; c < KS; ++c) {
      if (c + 1 < KS) {
#pragma unroll
        for (int t = 0; t < 4; ++t) k4[(c + 1) & 1][t] = *reinterpret_cast<const floatx4*>(krow + 16 * t * K_ROW + 16 * (c + 1));
      }
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int t = 0; t < 4; ++t) s[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(k4[c & 1][t][r], qreg[c][r], s[t], 0, 0, 0);
    }
    const float* vcol = vs + (g * HD + i16) * 4;
    floatx4 v4[2][KS];
#pragma unroll
    for (int dt = 0; dt < KS; ++dt) v4[0][dt] = *reinterpret_cast<const floatx4*>(vcol + 64 * dt);
    // a block that every query of the wave sees whole needs no comparisons
    const bool whole = kb + BT_KV_BLOCK - 1 <= wave_first && (a.window <= 0 || kb > wave_hi - a.window);
    if (!whole) {
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int key_pos = kb + 16 * t + 4 * g + r;
          const bool seen = key_pos <= qpos && (a.window <= 0 || key_pos > qpos - a.window);
          s[t][r] = seen ? s[t][r] : -INFINITY;
        }
    }
    float top = -INFINITY;
#pragma unroll
    for (int t = 0; t < 4; ++t) top = fmaxf(top, fmaxf(fmaxf(s[t][0], s[t][1]), fmaxf(s[t][2], s[t][3])));
    top = fmaxf(top, __shfl_xor(top, 16, 64));
    top = fmaxf(top, __shfl_xor(top, 32, 64));
    const float new_max = fmaxf(run_max, top * c2);          // in powers of two
    // nothing seen so far, this block included: everything stays at its start
    const float rescale = new_max == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(run_max - new_max);   // 2^-inf = 0 at the first block seen
    const float m_use = new_max == -INFINITY ? 0.f : new_max;
    float block_sum = 0.f;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        s[t][r] = __builtin_amdgcn_exp2f(fmaf(s[t][r], c2, -m_use));
        block_sum += s[t][r];
      }
    run_sum = fmaf(run_sum, rescale, block_sum);
    run_max = new_max;
#pragma unroll
    for (int dt = 0; dt < KS; ++dt)
#pragma unroll
      for (int r = 0; r < 4; ++r) o[dt][r] *= rescale;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      if (t + 1 < 4) {
#pragma unroll
        for (int dt = 0; dt < KS; ++dt) v4[(t + 1) & 1][dt] = *reinterpret_cast<const floatx4*>(vcol + 16 * (t + 1) * HD + 64 * dt);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int dt = 0; dt < KS; ++dt) o[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(v4[t & 1][dt][r], s[t][r], o[dt], 0, 0, 0);
    }
  }
  float total = run_sum;
  total += __shfl_xor(total, 16, 64);
  total += __shfl_xor(total, 32, 64);
  if (exists) {
    float* out = static_cast<float*>(a.out) + (int64_t)(off + q0 + mine) * a.ldo + head * HD;
#pragma unroll
    for (int dt = 0; dt < KS; ++dt) {
      floatx4 r4;
#pragma unroll
      for (int r = 0; r < 4; ++r) r4[r] = total > 0.f ? o[dt][r] / total : 0.f;
      *reinterpret_cast<floatx4*>(out + 16 * dt + 4 * g) = r4;
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

template <int HD>
static int launch_prompt(hipStream_t stream, const AttnArgs& a) {
  const int q_tiles = (a.max_count + F32M_QUERIES - 1) / F32M_QUERIES;
  const size_t lds = sizeof(float) * (size_t)(BT_KV_BLOCK * (HD + 4) + BT_KV_BLOCK * HD);
  if (lds > 64 * 1024) {                        // beyond what a kernel gets without asking
    static bool raised = false;
    if (!raised) {
      hipError_t err = hipFuncSetAttribute((const void*)attention_f32_mfma_kernel<HD>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (err != hipSuccess) BT_REFUSE("attention_f32: cannot get %zu bytes of LDS: %s", lds, hipGetErrorString(err));
      raised = true;
    }
  }
  const int64_t groups = (int64_t)a.n_seqs * a.q_heads * q_tiles;
  if (groups > 0x7fffffff) BT_REFUSE("attention_f32: %lld work-groups are too many", (long long)groups);
  hipLaunchKernelGGL(attention_f32_mfma_kernel<HD>, dim3((unsigned)groups), dim3(256), lds, stream, a);
  return bt_check_launch("attention_f32");
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
  if (a.ldo % 4 != 0 || ((uintptr_t)a.out & 15))
    BT_REFUSE("attention_f32: output rows are written 16 bytes at a time (row pitch %lld)", (long long)a.ldo);
  switch (hd) {
    case 16: return launch_prompt<16>((hipStream_t)stream, a);
    case 32: return launch_prompt<32>((hipStream_t)stream, a);
    case 48: return launch_prompt<48>((hipStream_t)stream, a);
    case 64: return launch_prompt<64>((hipStream_t)stream, a);
    case 80: return launch_prompt<80>((hipStream_t)stream, a);
    case 96: return launch_prompt<96>((hipStream_t)stream, a);
    case 112: return launch_prompt<112>((hipStream_t)stream, a);
    default: return launch_prompt<128>((hipStream_t)stream, a);
  }
}

// The same entry points with their arguments as one structure (calls.h), for launch lists.
BT_EXPORT int bt_attention_f32_call(void* stream, const AttentionCall* c) { return bt_attention_f32(stream, &c->args); }
