// Matrix products on the MFMA units of gfx950, C[M,N] = A[M,K] . W[N,K]^T with 32-bit
// accumulation, in bfloat16 and in float (the float instructions multiply and add in full
// 32-bit: no reduced-precision mode exists in them).  Both operands are K-contiguous, which is
// what an MFMA lane wants: consecutive K values in one 16-byte load.
//
//   gemm_tile    128 x 128 x 64 tiles for many rows (prefill).  Four waves, each a quarter of the
//                tile as 2 x 2 blocks of v_mfma_f32_32x32x16_bf16; operands staged through LDS
//                with an XOR swizzle of the 16-byte chunks, the next tile's global loads in
//                flight during the multiplication, tiles numbered so that each XCD's L2 sees
//                neighbours.  (The kernel is a template over the tile and the prefetch depth;
//                larger tiles and deeper prefetch were measured and lost to this one: they
//                leave room for one work-group per compute unit only.)
//   gemm_skinny  up to 64 rows (decode).  The product is bound by streaming W once from HBM:
//                a work-group owns 16 columns, its eight waves split K, every lane keeps several
//                16-byte loads of W in flight, v_mfma_f32_16x16x32_bf16 does the arithmetic and
//                the waves' partial sums meet in LDS.  K can also be split across work-groups
//                into 32-bit partial sums that the consumer adds up.
//
// The weights are the MFMA "A" operand (rows = output columns n), the activations the "B"
// operand (columns = rows m), so a lane ends up with four consecutive n of one m.
//
// The tile kernel's general form and the skinny kernel are templates over the element type; the
// two leaner forms of the tile kernel are bfloat16 only.

#include "host.h"
#include "epilogue.h"
#include "calls.h"

#define TILE_K 64            // bfloat16 values in a 128-byte row of an LDS tile
#define TILE_ROW_BYTES 128

typedef __attribute__((__vector_size__(4 * sizeof(int)))) int int4v;

// What a lane's 16-byte operand read is to the matrix cores.  bfloat16: eight K values, one
// instruction of depth 32 (16-wide blocks; the lane's K group is lane / 16) or 16 (32-wide
// blocks; lane / 32).  float: four K values, taken by four instructions of depth 4 (or 2), the
// i-th multiplying element i of both operands: a lane's K group is the same for both operands,
// so the four instructions cover 16 (or 8) distinct K values exactly once.  The result lies in
// the lanes the same way for both types.
template <typename T>
struct Mma;
template <>
struct Mma<bf16_t> {
  static constexpr int ELEMS = 8;
  static __device__ __forceinline__ void block16(floatx4& acc, int4v w, int4v a) {
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, w), __builtin_bit_cast(bf16x8, a), acc, 0, 0, 0);
  }
  static __device__ __forceinline__ void block32(floatx16& acc, int4v w, int4v a) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, w), __builtin_bit_cast(bf16x8, a), acc, 0, 0, 0);
  }
};
template <>
struct Mma<float> {
  static constexpr int ELEMS = 4;
  static __device__ __forceinline__ void block16(floatx4& acc, int4v w, int4v a) {
    floatx4 wf = __builtin_bit_cast(floatx4, w), af = __builtin_bit_cast(floatx4, a);
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wf[i], af[i], acc, 0, 0, 0);
  }
  static __device__ __forceinline__ void block32(floatx16& acc, int4v w, int4v a) {
    floatx4 wf = __builtin_bit_cast(floatx4, w), af = __builtin_bit_cast(floatx4, a);
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(wf[i], af[i], acc, 0, 0, 0);
  }
};

// 16-byte chunk `chunk` of row `row` of an LDS tile with 128-byte rows.  LDS has 64 banks of four
// bytes and serves 16 lanes of a 16-byte access at a time, so two rows span the banks once and
// the 16 consecutive rows that read the same chunk for an MFMA operand must land in 16 different
// 16-byte slots: the chunk is XORed with bits 1..3 of the row (rows 2j and 2j + 1 share a value
// and differ in the half of the banks they occupy).  Measured with SQ_LDS_BANK_CONFLICT: a third
// of the LDS cycles were conflicts with the XOR taken from bits 0..2.
__device__ __forceinline__ int swizzled(int row, int chunk) {
  return row * TILE_ROW_BYTES + ((chunk ^ ((row >> 1) & 7)) << 4);
}

// Work-groups are handed to the eight XCDs in turn and each XCD has an L2 of its own, so the
// tiles are renumbered to give every XCD one contiguous range of them; inside a range, tiles
// that share a block of W's rows come first.
__device__ __forceinline__ int xcd_contiguous(int bid, int blocks) {
  int xcd = bid & 7, local = bid >> 3;
  int q = blocks >> 3, r = blocks & 7;
  return xcd * q + (xcd < r ? xcd : r) + local;
}

// BM x BN tiles of 128-byte rows (64 bfloat16 or 32 float K values), WM x WN waves, each wave
// (BM / WM) x (BN / WN) as 32-wide MFMA blocks; LDS holds two stages.  PF register sets hold tiles on their way
// from memory to LDS: with one, the loads of tile i + 1 fly while tile i is multiplied; with
// two, tile i + 1 waits in registers and the loads of tile i + 2 fly.
template <typename T, int BM, int BN, int WM, int WN, int PF>
__global__ void __launch_bounds__(WM * WN * 64)
gemm_tile_kernel(const T* __restrict__ A, int64_t lda, const T* __restrict__ W, int M, int N,
                 int K, Epilogue epi, int tiles_m, int tiles_n) {
  constexpr int ELEMS = Mma<T>::ELEMS;          // K values in a 16-byte chunk
  constexpr int ROW_K = 8 * ELEMS;              // K values in a 128-byte row of a tile
  constexpr int THREADS = WM * WN * 64;
  constexpr int ROWS = BM + BN;                 // rows of a stage: A's, then W's
  constexpr int PER_THREAD = ROWS * 8 / THREADS;  // 16-byte chunks a thread moves per tile
  constexpr int ROW_STEP = THREADS / 8;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  static_assert(ROWS * 8 % THREADS == 0 && BM % ROW_STEP == 0, "tile does not divide among the threads");
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];   // [2][ROWS * 128]
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int wm = wave % WM, wn = wave / WM;
  const int l32 = lane & 31, g = lane >> 5;
  const int tile = xcd_contiguous(blockIdx.x, tiles_m * tiles_n);
  const int m_base = (tile % tiles_m) * BM, n_base = (tile / tiles_m) * BN;
  const int split = blockIdx.z, splits = gridDim.z;
  const int k_tiles = (K + ROW_K - 1) / ROW_K;
  const int kt_begin = (int)((int64_t)k_tiles * split / splits);
  const int kt_end = (int)((int64_t)k_tiles * (split + 1) / splits);

  // chunk c of rows r0, r0 + ROW_STEP, ... of the stage: A's rows first, then W's.  Addresses
  // are rebuilt from the two bases for every load; keeping one pointer per row would not fit
  // the registers of the larger tiles.
  const int c = tid & 7, r0 = tid >> 3;
  constexpr int A_CHUNKS = BM / ROW_STEP;
  int4v regs[PF][PER_THREAD];
  auto load_tile = [&](int set, int kt) {
    // a chunk beyond K (a multiple of the chunk) reads the row's last chunk and is cleared when stored
    int k = kt * ROW_K + c * ELEMS;
    int kc = k < K ? k : K - ELEMS;
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      int row = r0 + ROW_STEP * i;
      const T* src;
      if (i < A_CHUNKS) {
        int m = m_base + row;
        src = A + (int64_t)(m < M ? m : M - 1) * lda;
      } else {
        int n = n_base + row - BM;
        src = W + (int64_t)(n < N ? n : N - 1) * K;
      }
      regs[set][i] = *reinterpret_cast<const int4v*>(src + kc);
    }
  };
  auto store_tile = [&](int set, int kt, int stage) {
    int keep = kt * ROW_K + c * ELEMS < K ? -1 : 0;
    unsigned char* base = lds + stage * (ROWS * TILE_ROW_BYTES);
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i)
      *reinterpret_cast<int4v*>(base + swizzled(r0 + ROW_STEP * i, c)) = regs[set][i] & keep;
  };

  floatx16 acc[TN][TM];
#pragma unroll
  for (int bn = 0; bn < TN; ++bn)
#pragma unroll
    for (int bm = 0; bm < TM; ++bm)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[bn][bm][r] = 0.f;

  auto multiply = [&](int stage) {
    // all operands of the tile are read before the first multiplication: LDS latency is paid once
    // per tile, and the reads of later steps return while earlier steps multiply
    const unsigned char* a_lds = lds + stage * (ROWS * TILE_ROW_BYTES);
    const unsigned char* w_lds = a_lds + BM * TILE_ROW_BYTES;
    constexpr int STEPS = TILE_ROW_BYTES / 32;      // a step: the two K groups' chunks
    int4v wop[STEPS][TN], aop[STEPS][TM];
#pragma unroll
    for (int kk = 0; kk < STEPS; ++kk) {
#pragma unroll
      for (int b = 0; b < TN; ++b)
        wop[kk][b] = *reinterpret_cast<const int4v*>(w_lds + swizzled(wn * (BN / WN) + b * 32 + l32, 2 * kk + g));
#pragma unroll
      for (int b = 0; b < TM; ++b)
        aop[kk][b] = *reinterpret_cast<const int4v*>(a_lds + swizzled(wm * (BM / WM) + b * 32 + l32, 2 * kk + g));
    }
#pragma unroll
    for (int kk = 0; kk < STEPS; ++kk)
#pragma unroll
      for (int bn = 0; bn < TN; ++bn)
#pragma unroll
        for (int bm = 0; bm < TM; ++bm)
          Mma<T>::block32(acc[bn][bm], wop[kk][bn], aop[kk][bm]);
  };

  const int count = kt_end - kt_begin;
  if (PF == 1) {
    // tile i is multiplied from stage i % 2 while the loads of tile i + 1 fly into the registers
    if (count > 0) {
      load_tile(0, kt_begin);
      store_tile(0, kt_begin, 0);
    }
    __syncthreads();
    for (int i = 0; i < count; ++i) {
      if (i + 1 < count) load_tile(0, kt_begin + i + 1);
      multiply(i & 1);
      if (i + 1 < count) store_tile(0, kt_begin + i + 1, (i + 1) & 1);
      __syncthreads();
    }
  } else {
    // tile i is multiplied from stage i % 2 while tile i + 1 sits in register set (i + 1) % 2 and
    // the loads of tile i + 2 fly into the other set
    if (count > 0) {
      load_tile(0, kt_begin);
      if (count > 1) load_tile(PF - 1, kt_begin + 1);
      store_tile(0, kt_begin, 0);
    }
    __syncthreads();
    for (int i = 0; i < count; i += 2) {
      if (i + 2 < count) load_tile(0, kt_begin + i + 2);
      multiply(0);
      if (i + 1 < count) store_tile(PF - 1, kt_begin + i + 1, 1);
      __syncthreads();
      if (i + 1 >= count) break;
      if (i + 3 < count) load_tile(PF - 1, kt_begin + i + 3);
      multiply(1);
      if (i + 2 < count) store_tile(0, kt_begin + i + 2, 0);
      __syncthreads();
    }
  }

  // lane holds D[i][j]: i = 8 * (r / 4) + 4 * g + r % 4 (column n), j = lane % 32 (row m)
#pragma unroll
  for (int bm = 0; bm < TM; ++bm) {
    const int m = m_base + wm * (BM / WM) + bm * 32 + l32;
#pragma unroll
    for (int bn = 0; bn < TN; ++bn) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float v[4] = {acc[bn][bm][4 * q], acc[bn][bm][4 * q + 1], acc[bn][bm][4 * q + 2], acc[bn][bm][4 * q + 3]};
        int n0 = n_base + wn * (BN / WN) + bn * 32 + q * 8 + g * 4;
        if (m < M) epilogue4<T>(epi, N, m, n0, v, split);
      }
    }
  }
}

// The same 128 x 128 x 64 tiling for K a multiple of 64 and operands below 4 GiB, written so that
// the loop over K holds almost nothing but loads, LDS traffic and MFMAs.  Counters
// (SQ_INSTS_VALU against SQ_INSTS_VALU_MFMA_MOPS) showed five ordinary vector instructions per
// MFMA in the template above, nearly all of them address arithmetic.  Here every address is a
// uniform base that a scalar add advances, plus a per-lane offset computed once: global loads
// take a 32-bit lane offset, LDS accesses one lane offset plus an immediate (rows 32 apart share
// their swizzle and lie 4096 bytes apart; the two stages are 32 KiB apart).
#define FAST_STAGE_BYTES (256 * TILE_ROW_BYTES)
#define FAST_W_BYTES (128 * TILE_ROW_BYTES)

__global__ void __launch_bounds__(256)
gemm_tile_fast_kernel(const bf16_t* __restrict__ A, int64_t lda, const bf16_t* __restrict__ W, int M, int N,
                      int K, Epilogue epi, int tiles_m, int tiles_n) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[2 * FAST_STAGE_BYTES];
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int wm = wave & 1, wn = wave >> 1;
  const int l32 = lane & 31, g = lane >> 5;
  const int tile = xcd_contiguous(blockIdx.x, tiles_m * tiles_n);
  const int m_base = (tile % tiles_m) * 128, n_base = (tile / tiles_m) * 128;
  const int split = blockIdx.z, splits = gridDim.z;
  const int k_tiles = K / TILE_K;
  const int kt_begin = (int)((int64_t)k_tiles * split / splits);
  const int count = (int)((int64_t)k_tiles * (split + 1) / splits) - kt_begin;

  const int c = tid & 7, r0 = tid >> 3;
  unsigned a_off[4], w_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int m = m_base + r0 + 32 * i, n = n_base + r0 + 32 * i;
    m = m < M ? m : M - 1;
    n = n < N ? n : N - 1;
    a_off[i] = (unsigned)(((int64_t)m * lda + c * 8) * 2);
    w_off[i] = (unsigned)(((int64_t)n * K + c * 8) * 2);
  }
  const unsigned char* a_k = reinterpret_cast<const unsigned char*>(A) + (int64_t)kt_begin * (TILE_K * 2);
  const unsigned char* w_k = reinterpret_cast<const unsigned char*>(W) + (int64_t)kt_begin * (TILE_K * 2);
  const int st_off = swizzled(r0, c);
  int w_rd[4], a_rd[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) {
    w_rd[kk] = FAST_W_BYTES + swizzled(wn * 64 + l32, 2 * kk + g);
    a_rd[kk] = swizzled(wm * 64 + l32, 2 * kk + g);
  }

  int4v ra[4], rw[4];
  auto load_tile = [&]() {     // the tile a_k, w_k point at; then advance them
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ra[i] = *reinterpret_cast<const int4v*>(a_k + a_off[i]);
      rw[i] = *reinterpret_cast<const int4v*>(w_k + w_off[i]);
    }
    a_k += TILE_K * 2;
    w_k += TILE_K * 2;
  };
  auto store_tile = [&](int stage_bytes) {
    unsigned char* base = lds + stage_bytes + st_off;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      *reinterpret_cast<int4v*>(base + i * 4096) = ra[i];
      *reinterpret_cast<int4v*>(base + FAST_W_BYTES + i * 4096) = rw[i];
    }
  };
  floatx16 acc[2][2];
#pragma unroll
  for (int bn = 0; bn < 2; ++bn)
#pragma unroll
    for (int bm = 0; bm < 2; ++bm)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[bn][bm][r] = 0.f;

  if (count > 0) {
    load_tile();
    store_tile(0);
  }
  __syncthreads();
  // one loop body, no exit in its middle: the accumulators then stay where the MFMAs want them
  // (with the loop unrolled by two and left from its middle, the compiler copied all of them
  // between register files in every iteration)
  int stage_bytes = 0;
  for (int i = 0; i < count; ++i) {
    const bool more = i + 1 < count;
    if (more) load_tile();
    const unsigned char* base = lds + stage_bytes;
    bf16x8 wop[4][2], aop[4][2];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        wop[kk][b] = *reinterpret_cast<const bf16x8*>(base + w_rd[kk] + b * 4096);
        aop[kk][b] = *reinterpret_cast<const bf16x8*>(base + a_rd[kk] + b * 4096);
      }
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
#pragma unroll
      for (int bn = 0; bn < 2; ++bn)
#pragma unroll
        for (int bm = 0; bm < 2; ++bm)
          acc[bn][bm] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wop[kk][bn], aop[kk][bm], acc[bn][bm], 0, 0, 0);
    stage_bytes ^= FAST_STAGE_BYTES;
    if (more) store_tile(stage_bytes);
    __syncthreads();
  }

  // lane holds D[i][j]: i = 8 * (r / 4) + 4 * g + r % 4 (column n), j = lane % 32 (row m)
#pragma unroll
  for (int bm = 0; bm < 2; ++bm) {
    const int m = m_base + wm * 64 + bm * 32 + l32;
#pragma unroll
    for (int bn = 0; bn < 2; ++bn) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float v[4] = {acc[bn][bm][4 * q], acc[bn][bm][4 * q + 1], acc[bn][bm][4 * q + 2], acc[bn][bm][4 * q + 3]};
        int n0 = n_base + wn * 64 + bn * 32 + q * 8 + g * 4;
        if (m < M) epilogue4<bf16_t>(epi, N, m, n0, v, split);
      }
    }
  }
}

// The third form of the same tiling moves the operands from memory straight into LDS
// (global_load_lds_dwordx4: every lane names 16 bytes in memory, the wave's 64 pieces land in one
// contiguous KiB of LDS), which frees the staging registers and, more to the point, lets
// DMA_STAGES - 1 tiles be in flight while one is multiplied: the products above are bound by
// memory latency (one tile in flight per work-group, two work-groups per compute unit), not by
// MFMA or LDS throughput.  The compiler's own bookkeeping would wait for ALL such loads before any
// LDS read, so the waits are written by hand (s_waitcnt vmcnt(n) with n = loads of the tiles that
// may still be in flight) and the work-group meets at a bare s_barrier:
//     wait for my loads of tile i | barrier | start the loads of tile i + STAGES - 1 into the
//     stage tile i - 1 was read from | read tile i from LDS | multiply
// The swizzle is applied on the memory side: lane l of the load that fills rows 8 s .. 8 s + 7
// writes physical chunk l % 8 of row 8 s + l / 8, so it fetches the logical chunk that belongs
// there.  K must be a multiple of 64, operands below 4 GiB.
#define DMA_STAGES 4
#define DMA_LOADS 8   // global_load_lds instructions per wave and tile

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__global__ void __launch_bounds__(256)
gemm_tile_dma_kernel(const bf16_t* __restrict__ A, int64_t lda, const bf16_t* __restrict__ W, int M, int N,
                     int K, Epilogue epi, int tiles_m, int tiles_n) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];   // [DMA_STAGES][256 rows][128 bytes]
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int wm = wave & 1, wn = wave >> 1;
  const int l32 = lane & 31, g = lane >> 5;
  const int tile = xcd_contiguous(blockIdx.x, tiles_m * tiles_n);
  const int m_base = (tile % tiles_m) * 128, n_base = (tile / tiles_m) * 128;
  const int split = blockIdx.z, splits = gridDim.z;
  const int k_tiles = K / TILE_K;
  const int kt_begin = (int)((int64_t)k_tiles * split / splits);
  const int count = (int)((int64_t)k_tiles * (split + 1) / splits) - kt_begin;

  // waves 0 and 1 fetch A's 128 rows, waves 2 and 3 W's: load j of a wave fills stage rows
  // 64 * wave + 8 j .. + 7 (rows 128 .. 255 of a stage are W's)
  const bool fetch_w = wave >= 2;
  const unsigned char* src = reinterpret_cast<const unsigned char*>(fetch_w ? W : A) +
                             (int64_t)kt_begin * (TILE_K * 2);
  unsigned off[DMA_LOADS];
#pragma unroll
  for (int j = 0; j < DMA_LOADS; ++j) {
    int stage_row = 64 * wave + 8 * j + (lane >> 3);
    int chunk = (lane & 7) ^ ((stage_row >> 1) & 7);
    int row = (stage_row & 127) + (fetch_w ? n_base : m_base);
    int limit = fetch_w ? N : M;
    row = row < limit ? row : limit - 1;
    off[j] = (unsigned)(((int64_t)row * (fetch_w ? (int64_t)K : lda) + chunk * 8) * 2);
  }
  auto issue = [&](int stage) {   // the tile `src` points at, into `stage`; then advance
#pragma unroll
    for (int j = 0; j < DMA_LOADS; ++j)
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)(src + off[j]),
          (__attribute__((address_space(3))) void*)(lds + stage * FAST_STAGE_BYTES + (64 * wave + 8 * j) * TILE_ROW_BYTES),
          16, 0, 0);
    src += TILE_K * 2;
  };
  int w_rd[4], a_rd[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) {
    w_rd[kk] = FAST_W_BYTES + swizzled(wn * 64 + l32, 2 * kk + g);
    a_rd[kk] = swizzled(wm * 64 + l32, 2 * kk + g);
  }
  floatx16 acc[2][2];
#pragma unroll
  for (int bn = 0; bn < 2; ++bn)
#pragma unroll
    for (int bm = 0; bm < 2; ++bm)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[bn][bm][r] = 0.f;

#pragma unroll
  for (int t = 0; t < DMA_STAGES - 1; ++t)
    if (t < count) issue(t);
  int stage = 0, next_stage = DMA_STAGES - 1;
  for (int i = 0; i < count; ++i) {
    // tiles i + 1 .. i + STAGES - 2 (those that exist) may still be in flight
    int newer = count - 1 - i;
    if (newer >= DMA_STAGES - 2) wait_vmcnt<DMA_LOADS * (DMA_STAGES - 2)>();
    else if (newer == 1) wait_vmcnt<DMA_LOADS>();
    else wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (i + DMA_STAGES - 1 < count) issue(next_stage);
    const unsigned char* base = lds + stage * FAST_STAGE_BYTES;
    bf16x8 wop[4][2], aop[4][2];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        wop[kk][b] = *reinterpret_cast<const bf16x8*>(base + w_rd[kk] + b * 4096);
        aop[kk][b] = *reinterpret_cast<const bf16x8*>(base + a_rd[kk] + b * 4096);
      }
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
#pragma unroll
      for (int bn = 0; bn < 2; ++bn)
#pragma unroll
        for (int bm = 0; bm < 2; ++bm)
          acc[bn][bm] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wop[kk][bn], aop[kk][bm], acc[bn][bm], 0, 0, 0);
    stage = stage + 1 == DMA_STAGES ? 0 : stage + 1;
    next_stage = next_stage + 1 == DMA_STAGES ? 0 : next_stage + 1;
  }

  // lane holds D[i][j]: i = 8 * (r / 4) + 4 * g + r % 4 (column n), j = lane % 32 (row m)
#pragma unroll
  for (int bm = 0; bm < 2; ++bm) {
    const int m = m_base + wm * 64 + bm * 32 + l32;
#pragma unroll
    for (int bn = 0; bn < 2; ++bn) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float v[4] = {acc[bn][bm][4 * q], acc[bn][bm][4 * q + 1], acc[bn][bm][4 * q + 2], acc[bn][bm][4 * q + 3]};
        int n0 = n_base + wn * 64 + bn * 32 + q * 8 + g * 4;
        if (m < M) epilogue4<bf16_t>(epi, N, m, n0, v, split);
      }
    }
  }
}

// The direct-to-LDS form again, for products of some tens to some hundreds of rows (short prompts,
// chunks of prompts): a template over the tile (BM x BN, 64 or 128 each, four waves as 2 x 2) and
// the number of stages.  Such a product has too few tiles of 128 x 128 to fill the chip, and with
// smaller tiles a work-group has less arithmetic per byte it pulls, so that its time is the 25 (or
// 100) trips to memory of its loop over K unless several of them are in flight at once.  Same layout
// of a stage as above (A's rows, then W's, 128 bytes each, the swizzle applied on the memory side),
// same waits written by hand.  K a multiple of 64, operands below 4 GiB.
// Measured at 128 rows (us; the vendor's library beside it): tiles of 64 x 64 in four stages 4800 x
// 1600 12.0 (17.3), 6400 x 1600 13.6 (18.2), and with K cut into four slices of pending partial sums
// 1600 x 1600 5.9 (11.2), 1600 x 6400 12.1 (18.4); at 256 rows tiles of 128 x 64 take 17.4 (20.0) and
// 20.0 (21.4), two slices of 64 x 64 7.4 (11.7) and 19.2 (23.9); sliced products win up to 512 rows
// (9.5 and 30.7 against 12.1 and 32.4), the others lose to the library from 512 rows on.  Four stages
// (64 KiB, two work-groups to a compute unit) do as well as eight or better.
// What bounds these forms is what the compute units pull, not what they multiply: a work-group
// gets a tile of 64 x 64 (16 KiB) about every 0.4 us, one of 128 x 64 every 0.6 us and one of 128 x
// 128 every 0.85 us, whatever the number of stages; with the matrix instructions and the LDS reads
// taken out the times stay.  Measured and not taken, all at 128 rows and within 10 % of the above:
// a ring of register sets in place of the direct loads (slower), waves that do nothing but issue the
// loads (2, 4 or 8 loads a wave and tile: the same times), all rows of the step against 32 columns
// with the weights in a ring of their own, 8 or 16 tiles deep, filled by a wave of its own (the
// same), each work-group starting its walk over K at another tile (the same).  All work-groups
// together pull at 6 to 12 TB/s through the L2s, more the more of them share a compute unit; a
// kernel that only reads as much without a loop does 27 TB/s from the L2 and 6.6 from memory.
// For prompts of thousands of rows a tile of 256 x 256 on eight waves (twice the multiplications
// per byte pulled) was measured too, in two forms.  With K in steps of 64 its two stages of 64 KiB
// are all that the LDS holds, so one tile is in flight at a time and its latency is not hidden:
// 2048 x 4800 x 1600 took 86 us where the lean form takes 70 and the vendor's library 39.  With K in
// steps of 32 and four stages of 32 KiB (rows two to a 128-byte line, swizzled free of bank
// conflicts) three tiles are in flight, but a wave's load then asks for sixteen half cache lines
// where it asked for eight whole ones, and a compute unit pulls half the bytes: 88 us.  What a
// compute unit pulls is a number of cache lines a microsecond (about 300), not of bytes.
template <int NEWER, int LOADS>
__device__ __forceinline__ void wait_for_all_but(int newer) {
  // waits until at most `newer` tiles' loads (LOADS instructions each) of this wave are in flight
  if constexpr (NEWER == 0) {
    wait_vmcnt<0>();
  } else {
    if (newer >= NEWER) wait_vmcnt<NEWER * LOADS>();
    else wait_for_all_but<NEWER - 1, LOADS>(newer);
  }
}

template <int BM, int BN, int STAGES>
__global__ void __launch_bounds__(256)
gemm_tile_deep_kernel(const bf16_t* __restrict__ A, int64_t lda, const bf16_t* __restrict__ W, int M, int N,
                      int K, Epilogue epi, int tiles_m, int tiles_n) {
  constexpr int ROWS = BM + BN;                   // rows of a stage
  constexpr int STAGE_BYTES = ROWS * TILE_ROW_BYTES;
  constexpr int LOADS = ROWS / 32;                // global_load_lds instructions per wave and tile (8 rows each)
  constexpr int TM = BM / 64, TN = BN / 64;       // 32-wide MFMA blocks of a wave's (BM / 2) x (BN / 2)
  static_assert((BM == 64 || BM == 128) && (BN == 64 || BN == 128) && STAGES >= 3 && LOADS * (STAGES - 2) < 64,
                "tiles of 64 or 128, and no more loads in flight than the wave's counter holds");
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];   // [STAGES][ROWS][128 bytes]
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int wm = wave & 1, wn = wave >> 1;
  const int l32 = lane & 31, g = lane >> 5;
  const int tile = xcd_contiguous(blockIdx.x, tiles_m * tiles_n);
  const int m_base = (tile % tiles_m) * BM, n_base = (tile / tiles_m) * BN;
  const int split = blockIdx.z, splits = gridDim.z;
  const int k_tiles = K / TILE_K;
  const int kt_begin = (int)((int64_t)k_tiles * split / splits);
  const int count = (int)((int64_t)k_tiles * (split + 1) / splits) - kt_begin;

  // load j of wave w fills stage rows 8 (LOADS w + j) .. + 7: A's rows below BM, W's from there on
  const unsigned char* a_bytes = reinterpret_cast<const unsigned char*>(A) + (int64_t)kt_begin * (TILE_K * 2);
  const unsigned char* w_bytes = reinterpret_cast<const unsigned char*>(W) + (int64_t)kt_begin * (TILE_K * 2);
  unsigned off[LOADS];
  bool from_w[LOADS];
#pragma unroll
  for (int j = 0; j < LOADS; ++j) {
    int first_row = __builtin_amdgcn_readfirstlane(8 * (LOADS * wave + j));
    from_w[j] = first_row >= BM;                  // (the same for the whole wave: eight rows never straddle BM)
    int stage_row = first_row + (lane >> 3);
    int chunk = (lane & 7) ^ ((stage_row >> 1) & 7);
    int row = from_w[j] ? n_base + stage_row - BM : m_base + stage_row;
    int limit = from_w[j] ? N : M;
    row = row < limit ? row : limit - 1;
    off[j] = (unsigned)(((int64_t)row * (from_w[j] ? (int64_t)K : lda) + chunk * 8) * 2);
  }
  auto issue = [&](int stage) {   // the tile a_bytes / w_bytes point at, into `stage`; then advance
#pragma unroll
    for (int j = 0; j < LOADS; ++j)
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)((from_w[j] ? w_bytes : a_bytes) + off[j]),
          (__attribute__((address_space(3))) void*)(lds + stage * STAGE_BYTES + 8 * (LOADS * wave + j) * TILE_ROW_BYTES),
          16, 0, 0);
    a_bytes += TILE_K * 2;
    w_bytes += TILE_K * 2;
  };
  int w_rd[4], a_rd[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) {
    w_rd[kk] = BM * TILE_ROW_BYTES + swizzled(wn * (BN / 2) + l32, 2 * kk + g);
    a_rd[kk] = swizzled(wm * (BM / 2) + l32, 2 * kk + g);
  }
  floatx16 acc[TN][TM];
#pragma unroll
  for (int bn = 0; bn < TN; ++bn)
#pragma unroll
    for (int bm = 0; bm < TM; ++bm)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[bn][bm][r] = 0.f;

#pragma unroll
  for (int t = 0; t < STAGES - 1; ++t)
    if (t < count) issue(t);
  int stage = 0, next_stage = STAGES - 1;
  for (int i = 0; i < count; ++i) {
    // tiles i + 1 .. i + STAGES - 2 (those that exist) may still be in flight
    wait_for_all_but<STAGES - 2, LOADS>(count - 1 - i);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (i + STAGES - 1 < count) issue(next_stage);
    const unsigned char* base = lds + stage * STAGE_BYTES;
    bf16x8 wop[4][TN], aop[4][TM];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
#pragma unroll
      for (int b = 0; b < TN; ++b) wop[kk][b] = *reinterpret_cast<const bf16x8*>(base + w_rd[kk] + b * 4096);
#pragma unroll
      for (int b = 0; b < TM; ++b) aop[kk][b] = *reinterpret_cast<const bf16x8*>(base + a_rd[kk] + b * 4096);
    }
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
#pragma unroll
      for (int bn = 0; bn < TN; ++bn)
#pragma unroll
        for (int bm = 0; bm < TM; ++bm)
          acc[bn][bm] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wop[kk][bn], aop[kk][bm], acc[bn][bm], 0, 0, 0);
    stage = stage + 1 == STAGES ? 0 : stage + 1;
    next_stage = next_stage + 1 == STAGES ? 0 : next_stage + 1;
  }

  // lane holds D[i][j]: i = 8 * (r / 4) + 4 * g + r % 4 (column n), j = lane % 32 (row m)
#pragma unroll
  for (int bm = 0; bm < TM; ++bm) {
    const int m = m_base + wm * (BM / 2) + bm * 32 + l32;
#pragma unroll
    for (int bn = 0; bn < TN; ++bn) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float v[4] = {acc[bn][bm][4 * q], acc[bn][bm][4 * q + 1], acc[bn][bm][4 * q + 2], acc[bn][bm][4 * q + 3]};
        int n0 = n_base + wn * (BN / 2) + bn * 32 + q * 8 + g * 4;
        if (m < M) epilogue4<bf16_t>(epi, N, m, n0, v, split);
      }
    }
  }
}

// Memory latency on this GPU is about a microsecond and one compute unit alone pulls only a few
// per cent of the HBM bandwidth, while a decode step is hundreds of short kernels.  So the
// skinny kernel (a) wants at least as many work-groups as there are compute units, which is
// what splitting K is for when there are few output columns, and (b) has ONE round trip to
// memory on its critical path: everything the epilogue needs (bias, old residual, cache
// addresses) is fetched together with the first batch of weights, without a branch in between.
// MT row blocks of 16 (activations) by NT column blocks of 16 (weights) per work-group.  With
// more than 16 rows the activations a work-group reads (all rows, its whole K range) outweigh its
// weights, and they are read once per work-group: two column blocks halve that traffic.
//
// QPL > 0 (bfloat16, up to 16 rows): the activations are not read from memory but made here, as
// the normalised rows of the float32 residual stream (NormOperand): the norm that would
// otherwise be a kernel of its own in front of this one.  Every work-group normalises all rows
// (a wave takes rows w and w + 8: the row in its registers, QPL quads of four floats per lane,
// statistics as wave reductions) and leaves them in LDS as bfloat16, where the multiplication
// reads its operand.  The rows' loads are issued before the first batch of weights, so the
// statistics are computed while the weights are on their way.
__device__ float bt_norm_zeros[4] = {0.f, 0.f, 0.f, 0.f};

template <typename T, int MT, int NT, int U, int WAVES, int QPL = 0, bool CHUNKED = false>
__global__ void __launch_bounds__(WAVES * 64)
gemm_skinny_kernel(const T* __restrict__ A, int64_t lda, const T* __restrict__ W, int M, int N,
                   int K, Epilogue epi, int tile_columns, NormOperand norm, int packed, int a_rows) {
  constexpr int ELEMS = Mma<T>::ELEMS;      // K values in a lane's 16-byte load
  constexpr int CHUNK = 4 * ELEMS;          // K values the wave's four K groups cover together
  constexpr bool NORM = QPL > 0;
  static_assert(!NORM || (MT == 1 && sizeof(T) == 2), "the fused norm is for bfloat16 and up to 16 rows");
  extern __shared__ __attribute__((aligned(16))) unsigned char normed[];   // NORM: [16][K * 2 + 16] bytes
  const int normed_pitch = K * 2 + 16;      // the 16 bytes spread the rows over the LDS banks
  // tile_columns: how many of its 16 * NT output columns a work-group really owns (a multiple of
  // four).  Fewer than all of them is for balance: 300 work-groups of 16 columns leave 44 of 256
  // compute units with twice the bytes of the others, 400 of 12 columns leave every unit at most
  // 24 columns.  The lanes of the columns left out repeat the last real one and store nothing.
  __shared__ __attribute__((aligned(16))) float red[WAVES][MT * NT][64][4];
  static_assert(MT * NT <= WAVES, "one wave finishes each block of the work-group's output");
  // the wave's number is the same in all its lanes: saying so keeps every test on it a scalar
  // branch, which costs no wait for loads in flight (a divergent one does)
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int i16 = lane & 15, g = lane >> 4;
  const int n_base = blockIdx.x * tile_columns;
  const int n_end = n_base + tile_columns < N ? n_base + tile_columns : N;   // one past this work-group's last column
  const int split = blockIdx.y, splits = gridDim.y;
  // packed: W is not [N][K] but, for each work-group's `tile_columns` columns, the chunks of K one
  // after the other, [group][chunk][tile_columns][CHUNK], K and the last group padded with zeros:
  // a wave's load of a chunk is then one contiguous run of bytes and a work-group reads one
  // contiguous block front to back.
  const int w_chunk_pitch = packed ? tile_columns * CHUNK : CHUNK;     // elements from one chunk to the next
  const T* w_row[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    int n = n_base + nt * 16 + i16;
    n = n < n_end ? n : n_end - 1;
    w_row[nt] = packed ? W + ((int64_t)blockIdx.x * ((K + CHUNK - 1) / CHUNK) * tile_columns + (n - n_base)) * CHUNK
                       : W + (int64_t)n * K;
  }
  // CHUNKED: the activations are chunk-major (activation_offset in common.h) with a_rows rows: the
  // 64 lanes of an operand load then read one contiguous KiB.  (A form of the kernel of its own, so
  // that the row-major form keeps its loads free of anything computed per lane between them.)
  const int a_chunk_pitch = CHUNKED ? a_rows * CHUNK : CHUNK;      // elements from one chunk of a row to its next
  const T* a_row[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int m = mt * 16 + i16;
    a_row[mt] = CHUNKED ? A + (int64_t)(m < M ? m : M - 1) * CHUNK : A + (int64_t)(m < M ? m : M - 1) * lda;
  }
  // A batch is two phases.  First every load of the batch is issued: a chunk beyond K is
  // skipped by a scalar branch, a group beyond K (a multiple of the group) inside the last chunk
  // reads the row's last group instead.  Only then are the weights of such a group cleared (with
  // a bit mask) and multiplied.  Nothing that depends on a lane or on loaded data stands between
  // the loads, so the compiler has no reason to wait for one before it issues the next.
  // Rows beyond M repeat row M - 1; their results are dropped by the epilogue.
  const int chunks = (K + CHUNK - 1) / CHUNK;
  const int stride = splits * WAVES;
  floatx4 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = floatx4{0.f, 0.f, 0.f, 0.f};
  int4v wv[U][NT], av[U][MT];
  auto issue = [&](int c0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int cc = c0 + u * stride;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) wv[u][nt] = int4v{0, 0, 0, 0};
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) av[u][mt] = int4v{0, 0, 0, 0};
      if (cc < chunks) {
        int k = cc * CHUNK + g * ELEMS;
        int kc = k < K ? k : K - ELEMS;
        int wc = packed ? cc * w_chunk_pitch + g * ELEMS : kc;      // (the packed chunks are whole: zeros beyond K)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) wv[u][nt] = *reinterpret_cast<const int4v*>(w_row[nt] + wc);
        if constexpr (!NORM) {
          // (kc is a multiple of ELEMS inside one chunk: chunk kc / CHUNK, offset kc % CHUNK)
          int ac = CHUNKED ? (kc / CHUNK) * a_chunk_pitch + kc % CHUNK : kc;
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) av[u][mt] = *reinterpret_cast<const int4v*>(a_row[mt] + ac);
        }
      }
    }
  };
  auto multiply = [&](int c0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int keep = (c0 + u * stride) * CHUNK + g * ELEMS < K ? -1 : 0;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        int4v w = wv[u][nt] & keep;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) Mma<T>::block16(acc[mt][nt], w, av[u][mt]);
      }
    }
  };
  // NORM: the operand of every chunk of the batch from LDS (a chunk beyond K reads the row's last
  // group, as the loads from memory do; its weights are cleared)
  auto operands_from_lds = [&](int c0) {
    const int row = i16 < M ? i16 : M - 1;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int k = (c0 + u * stride) * CHUNK + g * ELEMS;
      int kc = k < K ? k : K - ELEMS;
      av[u][0] = *reinterpret_cast<const int4v*>(normed + row * normed_pitch + kc * 2);
    }
  };
  int c0 = split * WAVES + wave;
  if constexpr (NORM) {
    const int quads = K >> 2;
    const float4* g4 = reinterpret_cast<const float4*>(norm.gamma);
    const float4* b4 = reinterpret_cast<const float4*>(norm.beta);
    const float4* z4 = reinterpret_cast<const float4*>(bt_norm_zeros);
    float4 xv[QPL], gv[QPL], bv[QPL];
    auto load_row = [&](int r) {
      const float4* xr = reinterpret_cast<const float4*>(norm.x + (int64_t)r * norm.ldx);
#pragma unroll
      for (int q = 0; q < QPL; ++q) {
        int c = lane + 64 * q;
        int cc = c < quads ? c : 0;          // lanes beyond the row read its start; the result is never used
        xv[q] = xr[cc];
        gv[q] = g4[cc];
        bv[q] = norm.beta ? b4[cc] : z4[0];
      }
    };
    auto normalise_row = [&](int r) {
      float part = 0.f;
#pragma unroll
      for (int q = 0; q < QPL; ++q)
        if (lane + 64 * q < quads)
          part += norm.kind == 0 ? (xv[q].x + xv[q].y + xv[q].z + xv[q].w)
                                 : (xv[q].x * xv[q].x + xv[q].y * xv[q].y + xv[q].z * xv[q].z + xv[q].w * xv[q].w);
      float total = wave_sum(part);
      float mean = 0.f, rstd;
      if (norm.kind == 0) {
        mean = total / (float)K;
        float sq = 0.f;
#pragma unroll
        for (int q = 0; q < QPL; ++q)
          if (lane + 64 * q < quads) {
            float a0 = xv[q].x - mean, a1 = xv[q].y - mean, a2 = xv[q].z - mean, a3 = xv[q].w - mean;
            sq += a0 * a0 + a1 * a1 + a2 * a2 + a3 * a3;
          }
        rstd = 1.0f / sqrtf(wave_sum(sq) / (float)K + norm.eps);
      } else {
        rstd = 1.0f / sqrtf(total / (float)K + norm.eps);
      }
#pragma unroll
      for (int q = 0; q < QPL; ++q) {
        int c = lane + 64 * q;
        if (c < quads) {
          bf16x4 y = {(bf16_t)((xv[q].x - mean) * rstd * gv[q].x + bv[q].x), (bf16_t)((xv[q].y - mean) * rstd * gv[q].y + bv[q].y),
                      (bf16_t)((xv[q].z - mean) * rstd * gv[q].z + bv[q].z), (bf16_t)((xv[q].w - mean) * rstd * gv[q].w + bv[q].w)};
          *reinterpret_cast<bf16x4*>(normed + r * normed_pitch + c * 8) = y;
        }
      }
    };
    if (wave < M) load_row(wave);            // (the wave's number is scalar: no lane-dependent branch)
    issue(c0);                               // the weights of the first batch, behind the row
    if (wave < M) normalise_row(wave);
    if (wave + WAVES < M) {
      load_row(wave + WAVES);
      normalise_row(wave + WAVES);
    }
    __syncthreads();
    operands_from_lds(c0);
  } else {
    issue(c0);
  }
  // wave w < MT * NT finishes row block w / NT of column block w % NT: lane holds D[i][j],
  // i = 4 * (lane / 16) + r (column n), j = lane % 16 (row m); what its epilogue needs is
  // fetched now, behind the first batch
  const int blocks = MT * NT;
  const int mine = wave < blocks ? wave : 0;
  const int out_m = (mine / NT) * 16 + i16, out_n0 = n_base + (mine % NT) * 16 + g * 4;
  EpiloguePrefetch pre = {};
  if (wave < blocks) pre = epilogue_prefetch(epi, M, n_end, out_m, out_n0, split);
  multiply(c0);
  for (c0 += stride * U; c0 < chunks; c0 += stride * U) {
    issue(c0);
    if constexpr (NORM) operands_from_lds(c0);
    multiply(c0);
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
      *reinterpret_cast<floatx4*>(&red[wave][mt * NT + nt][lane][0]) = acc[mt][nt];
  __syncthreads();
  if (wave < blocks) {
    float v[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < WAVES; ++w)
#pragma unroll
      for (int r = 0; r < 4; ++r) v[r] += red[w][wave][lane][r];
    if (out_m < M) epilogue4_prefetched<T>(epi, n_end, out_m, out_n0, v, split, pre);   // nothing beyond n_end
  }
}

static int check_operands(const char* who, int elems, const void* A, int64_t lda, const void* W, int M, int N,
                          int K, const Epilogue& e, int splits) {
  if (N <= 0 || K <= 0) BT_REFUSE("%s: N %d and K %d must be positive", who, N, K);
  if (K % elems != 0 || lda % elems != 0)
    BT_REFUSE("%s: K %d and the row pitch %lld must be multiples of %d (16-byte loads)", who, K, (long long)lda, elems);
  if (((uintptr_t)A & 15) || ((uintptr_t)W & 15)) BT_REFUSE("%s: operands must be 16-byte aligned", who);
  if (e.mode < 0 || e.mode > 4 || e.out == nullptr) BT_REFUSE("%s: bad epilogue", who);
  if (splits < 1 || (splits > 1 && e.mode != EPI_F32))
    BT_REFUSE("%s: K can be split %d ways only into 32-bit partial sums", who, splits);
  if (e.out_rows != 0 && ((e.mode != EPI_STORE && e.mode != EPI_ACT) || e.out_rows < M))
    BT_REFUSE("%s: a chunk-major output of %d rows for %d rows (stored or activated results only)", who, e.out_rows, M);
  if (e.mode == EPI_QKV) {
    if (e.kv.head_dim <= 0 || e.kv.head_dim % 16 != 0)
      BT_REFUSE("%s: head size %d must be a multiple of 16", who, e.kv.head_dim);
    if (e.n_q % 16 != 0 || e.n_kv != e.kv.kv_heads * e.kv.head_dim || e.n_q + 2 * e.n_kv != N)
      BT_REFUSE("%s: fused projection of %d columns does not split into %d query and 2 x %d key/value columns",
                who, N, e.n_q, e.n_kv);
    if (!e.tok_seq || !e.tok_pos || !e.kv.blocks || !e.kv.keys || !e.kv.values)
      BT_REFUSE("%s: the key/value scatter needs token and cache tables", who);
  }
  return BT_OK;
}

template <typename T, int BM, int BN, int WM, int WN, int PF>
static void launch_tile(hipStream_t stream, const T* A, int64_t lda, const T* W, int M, int N, int K,
                        const Epilogue& epi, int splits) {
  int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  size_t lds = (size_t)2 * (BM + BN) * TILE_ROW_BYTES;
  auto kernel = gemm_tile_kernel<T, BM, BN, WM, WN, PF>;
  if (lds > 64 * 1024)
    (void)hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n, 1, splits), dim3(WM * WN * 64), lds, stream, A, lda, W, M, N,
                     K, epi, tiles_m, tiles_n);
}

template <int BM, int BN, int STAGES>
static int launch_deep_form(hipStream_t s, const bf16_t* a, int64_t lda, const bf16_t* w, int M, int N, int K,
                            const Epilogue& epi, int splits) {
  auto kernel = gemm_tile_deep_kernel<BM, BN, STAGES>;
  const size_t lds = (size_t)STAGES * (BM + BN) * TILE_ROW_BYTES;
  static bool raised = false;
  if (!raised) {
    hipError_t err = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (err != hipSuccess) BT_REFUSE("gemm_tile: cannot get %zu bytes of LDS: %s", lds, hipGetErrorString(err));
    raised = true;
  }
  int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n, 1, splits), dim3(256), lds, s, a, lda, w, M, N, K, epi, tiles_m, tiles_n);
  return bt_check_launch("gemm_tile");
}

// variants 4 .. 7: the deep forms (64 x 64 with 8 or 4 stages, 128 x 64 with 6 or 3)
static int launch_deep(hipStream_t s, int variant, const bf16_t* a, int64_t lda, const bf16_t* w, int M, int N, int K,
                       const Epilogue& epi, int splits) {
  switch (variant) {
    case 4: return launch_deep_form<64, 64, 8>(s, a, lda, w, M, N, K, epi, splits);
    case 5: return launch_deep_form<64, 64, 4>(s, a, lda, w, M, N, K, epi, splits);
    case 6: return launch_deep_form<128, 64, 6>(s, a, lda, w, M, N, K, epi, splits);
    case 7: return launch_deep_form<128, 64, 3>(s, a, lda, w, M, N, K, epi, splits);
  }
  BT_REFUSE("gemm_tile: unknown form %d", variant);
}

// dtype: 0 float, 1 bfloat16 (the codes of every entry point that takes both).
// variant: 0 = the fastest form the operands allow; 1 = template, 2 = lean, 3 = direct to LDS,
// 4 .. 7 = direct to LDS with smaller tiles and more stages (asked for by tests, by measurements
// and, for steps of some tens to some hundreds of rows, by the caller; a form that cannot take
// the operands is refused; float has the template only)
BT_EXPORT int bt_gemm_tile(void* stream, int dtype, const void* A, int64_t lda, const void* W, int M, int N, int K,
                           const Epilogue* epi, int splits, int variant) {
  if (M <= 0) return BT_OK;
  if (dtype != 0 && dtype != 1) BT_REFUSE("gemm_tile: element type %d is neither float nor bfloat16", dtype);
  int rc = check_operands("gemm_tile", dtype == 0 ? 4 : 8, A, lda, W, M, N, K, *epi, splits);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == 0) {
    if (variant > 1) BT_REFUSE("gemm_tile: float products have the general form only, not variant %d", variant);
    launch_tile<float, 128, 128, 2, 2, 1>(s, (const float*)A, lda, (const float*)W, M, N, K, *epi, splits);
    return bt_check_launch("gemm_tile");
  }
  const bf16_t* a = (const bf16_t*)A;
  const bf16_t* w = (const bf16_t*)W;
  const int64_t four_gib = (int64_t)1 << 32;
  const bool lean_ok = K % TILE_K == 0 && (int64_t)M * lda * 2 < four_gib && (int64_t)N * K * 2 < four_gib;
  // Direct to LDS keeps three tiles in flight but leaves room for one work-group per compute
  // unit; it wins when there is at most one tile per compute unit anyway, the lean form (two
  // work-groups per unit) when there are more.
  if (variant == 0) variant = !lean_ok ? 1 : ((int64_t)((M + 127) / 128) * ((N + 127) / 128) * splits <= 256 ? 3 : 2);
  if (variant != 1 && !lean_ok)
    BT_REFUSE("gemm_tile: this form needs K %d to be a multiple of 64 and operands below 4 GiB", K);
  if (variant >= 4) return launch_deep(s, variant, a, lda, w, M, N, K, *epi, splits);
  int tiles_m = (M + 127) / 128, tiles_n = (N + 127) / 128;
  dim3 grid(tiles_m * tiles_n, 1, splits);
  if (variant == 3) {
    size_t lds = (size_t)DMA_STAGES * FAST_STAGE_BYTES;
    static bool raised = false;
    if (!raised) {
      hipError_t err = hipFuncSetAttribute((const void*)gemm_tile_dma_kernel,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (err != hipSuccess) BT_REFUSE("gemm_tile: cannot get %zu bytes of LDS: %s", lds, hipGetErrorString(err));
      raised = true;
    }
    hipLaunchKernelGGL(gemm_tile_dma_kernel, grid, dim3(256), lds, s, a, lda, w, M, N, K, *epi, tiles_m, tiles_n);
  } else if (variant == 2) {
    hipLaunchKernelGGL(gemm_tile_fast_kernel, grid, dim3(256), 0, s, a, lda, w, M, N, K, *epi, tiles_m, tiles_n);
  } else {
    launch_tile<bf16_t, 128, 128, 2, 2, 1>(s, a, lda, w, M, N, K, *epi, splits);
  }
  return bt_check_launch("gemm_tile");
}

template <typename T>
static void launch_skinny(hipStream_t s, const T* a, int64_t lda, const T* w, int M, int N, int K, const Epilogue& epi,
                          int splits, int columns, int packed, int a_rows) {
  dim3 grid((N + columns - 1) / columns, splits), block(512);
  const NormOperand none = {};
#define LAUNCH_SKINNY(MT, NT, U)                                                                                   \
  do {                                                                                                             \
    if (a_rows > 0)                                                                                                \
      hipLaunchKernelGGL((gemm_skinny_kernel<T, MT, NT, U, 8, 0, true>), grid, block, 0, s, a, lda, w, M, N, K, epi, \
                         columns, none, packed, a_rows);                                                           \
    else                                                                                                           \
      hipLaunchKernelGGL((gemm_skinny_kernel<T, MT, NT, U, 8>), grid, block, 0, s, a, lda, w, M, N, K, epi, columns, \
                         none, packed, 0);                                                                         \
  } while (0)
  if (M <= 16) {
    if (columns <= 16) LAUNCH_SKINNY(1, 1, 8); else LAUNCH_SKINNY(1, 2, 8);
  } else if (M <= 32) {
    // eight loads in flight where a wave has more than four chunks of K to go through (measured at
    // 17 and 32 rows: 6.4 -> 6.1 us and 6.6 -> 6.4 us for 4800 x 1600; with four chunks or fewer
    // the longer batch only adds loads that are skipped, 4.2 -> 4.4 us for 1600 x 1600 in two slices)
    constexpr int chunk = 4 * Mma<T>::ELEMS;
    const int per_wave = (((K + chunk - 1) / chunk + splits - 1) / splits + 7) / 8;
    if (per_wave > 4) {
      if (columns <= 16) LAUNCH_SKINNY(2, 1, 8); else LAUNCH_SKINNY(2, 2, 8);
    } else {
      if (columns <= 16) LAUNCH_SKINNY(2, 1, 4); else LAUNCH_SKINNY(2, 2, 4);
    }
  } else {
    if (columns <= 16) LAUNCH_SKINNY(4, 1, 2); else LAUNCH_SKINNY(4, 2, 2);
  }
#undef LAUNCH_SKINNY
}

// The product of the normalised rows of a float32 residual stream (see NormOperand): bfloat16
// weights, up to 16 rows, K up to 2048 and a multiple of 8.
static int launch_skinny_norm(hipStream_t s, const NormOperand& norm, const bf16_t* w, int M, int N, int K,
                              const Epilogue& epi, int splits, int columns, int packed) {
  dim3 grid((N + columns - 1) / columns, splits), block(512);
  size_t lds = (size_t)16 * (K * 2 + 16);
#define LAUNCH_NORM(NT, QPL)                                                                                   \
  do {                                                                                                         \
    auto kernel = gemm_skinny_kernel<bf16_t, 1, NT, 8, 8, QPL>;                                                \
    static size_t granted = 0;    /* statically allocated LDS comes on top: ask for room beyond the default */ \
    if (lds > granted) {                                                                                       \
      hipError_t err = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
      if (err != hipSuccess) BT_REFUSE("gemm_skinny: cannot get %zu bytes of LDS: %s", lds, hipGetErrorString(err));   \
      granted = lds;                                                                                           \
    }                                                                                                          \
    hipLaunchKernelGGL(kernel, grid, block, lds, s, (const bf16_t*)nullptr, (int64_t)0, w, M, N, K, epi, columns, norm, packed, 0); \
  } while (0)
  if (K <= 1024) {
    if (columns <= 16) LAUNCH_NORM(1, 4); else LAUNCH_NORM(2, 4);
  } else {
    if (columns <= 16) LAUNCH_NORM(1, 8); else LAUNCH_NORM(2, 8);
  }
#undef LAUNCH_NORM
  return BT_OK;
}

// norm: null, or the activations are the normalised rows it describes (then A and lda are ignored)
// a_rows: 0, or A is chunk-major with that many rows (activation_offset in common.h; lda is not used).
// packed_columns: 0, or W is the packed form of the matrix for that many columns per work-group (see
// the kernel), which then is the number of columns a work-group takes.
BT_EXPORT int bt_gemm_skinny(void* stream, int dtype, const void* A, int64_t lda, const void* W, int M, int N, int K,
                             const Epilogue* epi, int splits, int variant, const NormOperand* norm, int packed_columns,
                             int a_rows) {
  if (M <= 0) return BT_OK;
  if (M > 64) BT_REFUSE("gemm_skinny: %d rows, at most 64", M);
  if (dtype != 0 && dtype != 1) BT_REFUSE("gemm_skinny: element type %d is neither float nor bfloat16", dtype);
  const int elems = dtype == 0 ? 4 : 8;
  if (a_rows != 0 && (norm != nullptr || a_rows < M))
    BT_REFUSE("gemm_skinny: chunk-major activations of %d rows for a product of %d rows%s", a_rows, M,
              norm != nullptr ? " that normalises its rows itself" : "");
  if (norm != nullptr) {
    if (dtype != 1 || M > 16 || K > 2048)
      BT_REFUSE("gemm_skinny: the fused norm takes bfloat16 weights, up to 16 rows and K up to 2048 (got %d rows, K %d)", M, K);
    if (!norm->x || !norm->gamma || norm->ldx < K || norm->ldx % 4 != 0 || ((uintptr_t)norm->x & 15) ||
        ((uintptr_t)norm->gamma & 15) || ((uintptr_t)norm->beta & 15) || (norm->kind != 0 && norm->kind != 1))
      BT_REFUSE("gemm_skinny: the rows to normalise, their scale and shift must be 16-byte aligned float32");
    A = W;            // (only its alignment is looked at below)
    lda = K;
  }
  if (a_rows != 0) lda = K;          // (chunk-major rows have no pitch; K itself is checked)
  int rc = check_operands("gemm_skinny", elems, A, lda, W, M, N, K, *epi, splits);
  if (rc) return rc;
  // 8 to 32 columns per work-group in steps of four (one or two column blocks of the kernel),
  // whichever leaves the busiest compute unit the least to pull: work-groups land on the units in
  // whole rounds.  Variants 8, 12, ... 32 (measurements and tests) force that many.
  static int compute_units = 0;
  if (compute_units == 0) {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&compute_units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess)
      compute_units = 256;
  }
  // columns per work-group: the cost of a work-group is what it pulls for one chunk of K (its
  // columns of the weights and the step's rows of the activations) times its chunks, plus a fixed part
  int columns = M <= 16 ? 16 : 32;
  const int packed = packed_columns != 0;
  if (packed) {
    if (packed_columns < 8 || packed_columns > 32 || packed_columns % 4 != 0)
      BT_REFUSE("gemm_skinny: a matrix packed for %d columns per work-group (8, 12, ... 32 are possible)", packed_columns);
    columns = packed_columns;
  } else if (variant >= 8 && variant <= 32 && variant % 4 == 0) {
    columns = variant;
  } else if (variant == 0) {
    const int chunk = 4 * elems;
    const int64_t per = ((K + chunk - 1) / chunk + splits - 1) / splits;
    int64_t best = -1;
    for (int c = 32; c >= 8; c -= 4) {
      int64_t groups = (int64_t)((N + c - 1) / c) * splits;
      int64_t cost = ((groups + compute_units - 1) / compute_units) * (per * (c + M) + 160);
      if (best < 0 || cost < best) { best = cost; columns = c; }
    }
  }
  if (norm != nullptr) {
    rc = launch_skinny_norm((hipStream_t)stream, *norm, (const bf16_t*)W, M, N, K, *epi, splits, columns, packed);
    if (rc) return rc;
  } else if (dtype == 0) {
    launch_skinny<float>((hipStream_t)stream, (const float*)A, lda, (const float*)W, M, N, K, *epi, splits, columns, packed, a_rows);
  } else {
    launch_skinny<bf16_t>((hipStream_t)stream, (const bf16_t*)A, lda, (const bf16_t*)W, M, N, K, *epi, splits, columns, packed, a_rows);
  }
  return bt_check_launch("gemm_skinny");
}

// The same entry points with their arguments as one structure (calls.h), for launch lists.
BT_EXPORT int bt_gemm_tile_call(void* stream, const GemmCall* c) {
  if (c->has_norm || c->a_rows || c->packed_columns)
    BT_REFUSE("gemm_tile: no rows to normalise, no chunk-major rows and no packed weights");
  return bt_gemm_tile(stream, c->dtype, c->A, c->lda, c->W, c->M, c->N, c->K, &c->epi, c->splits, c->variant);
}
BT_EXPORT int bt_gemm_skinny_call(void* stream, const GemmCall* c) {
  return bt_gemm_skinny(stream, c->dtype, c->A, c->lda, c->W, c->M, c->N, c->K, &c->epi, c->splits, c->variant,
                        c->has_norm ? &c->norm : nullptr, c->packed_columns, c->a_rows);
}
