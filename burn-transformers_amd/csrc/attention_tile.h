// The bfloat16 attention tile on the MFMA units of gfx950: the operands of 32 keys as the lanes hold
// them, and one online-softmax step over them.  Compiled per head size (-DBT_HEAD_DIM=N).
#pragma once

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
  float m_new[NQ];
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
    float tile_max = fmaxf(fmaxf(fmaxf(s[nq][0][0], s[nq][0][1]), fmaxf(s[nq][0][2], s[nq][0][3])),
                           fmaxf(fmaxf(s[nq][1][0], s[nq][1][1]), fmaxf(s[nq][1][2], s[nq][1][3])));
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, 64));
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, 64));
    m_new[nq] = fmaxf(m[nq], tile_max * c);
    behind = behind || m_new[nq] > m[nq] + RESCALE_SLACK;   // true for the first tile: m starts at -inf
  }
  if (__builtin_amdgcn_ballot_w64(behind) != 0) {   // the same for the whole wave: a scalar branch
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq) {
      float alpha = m_new[nq] == -INFINITY ? 1.f : exp2f(m[nq] - m_new[nq]);
      m[nq] = m_new[nq];
      l[nq] *= alpha;
#pragma unroll
      for (int dt = 0; dt < ND; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) o[nq][dt][r] *= alpha;
    }
  }
  bf16x8 pop[NQ];
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    const float m_use = m[nq] == -INFINITY ? 0.f : m[nq];
    float psum = 0.f;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float p = __builtin_amdgcn_exp2f(fmaf(s[nq][t][r], c, -m_use));
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
