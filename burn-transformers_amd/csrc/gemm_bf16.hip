// bfloat16 matrix products on the MFMA units of gfx950, C[M,N] = A[M,K] . W[N,K]^T with 32-bit
// accumulation.  Both operands are K-contiguous, which is what an MFMA lane wants: eight
// consecutive K values in one 16-byte load.
//
//   gemm_tile    128 x 128 x 64 tiles for many rows (prefill).  Four waves, each 64 x 64 as
//                2 x 2 blocks of v_mfma_f32_32x32x16_bf16; operands staged through LDS with an
//                XOR swizzle of the 16-byte chunks, global loads of the next tile in flight
//                while the current one is multiplied.
//   gemm_skinny  up to 64 rows (decode).  The product is bound by streaming W once from HBM:
//                a work-group owns 16 columns, its eight waves split K, every lane keeps several
//                16-byte loads of W in flight, v_mfma_f32_16x16x32_bf16 does the arithmetic and
//                the waves' partial sums meet in LDS.  K can also be split across work-groups
//                into 32-bit partial sums that the consumer adds up.
//
// The weights are the MFMA "A" operand (rows = output columns n), the activations the "B"
// operand (columns = rows m), so a lane ends up with four consecutive n of one m.

#include "host.h"
#include "epilogue.h"

#define TILE_M 128
#define TILE_N 128
#define TILE_K 64
#define TILE_ROW_BYTES 128

__device__ __forceinline__ int chunks_of(int K) { return (K + 31) / 32; }

__device__ __forceinline__ int swizzled(int row, int chunk) {
  return row * TILE_ROW_BYTES + ((chunk ^ (row & 7)) << 4);
}

__global__ void __launch_bounds__(256)
gemm_tile_kernel(const bf16_t* __restrict__ A, int64_t lda, const bf16_t* __restrict__ W, int M, int N,
                 int K, Epilogue epi) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[2][2][TILE_M * TILE_ROW_BYTES];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wm = wave & 1, wn = wave >> 1;
  const int l32 = lane & 31, g = lane >> 5;
  const int m_base = blockIdx.y * TILE_M, n_base = blockIdx.x * TILE_N;
  const int split = blockIdx.z, splits = gridDim.z;
  const int k_tiles = (K + TILE_K - 1) / TILE_K;
  const int kt_begin = (int)((int64_t)k_tiles * split / splits);
  const int kt_end = (int)((int64_t)k_tiles * (split + 1) / splits);

  // global -> register staging: chunk c of rows r0, r0+32, r0+64, r0+96 of both operands
  const int c = tid & 7, r0 = tid >> 3;
  const bf16_t* a_src[4];
  const bf16_t* w_src[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int m = m_base + r0 + 32 * i, n = n_base + r0 + 32 * i;
    m = m < M ? m : M - 1;
    n = n < N ? n : N - 1;
    a_src[i] = A + (int64_t)m * lda + c * 8;
    w_src[i] = W + (int64_t)n * K + c * 8;
  }
  uint4 ra[4], rw[4];
  auto load_tile = [&](int kt) {
    int k = kt * TILE_K + c * 8;
    bool inside = k < K;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ra[i] = inside ? *reinterpret_cast<const uint4*>(a_src[i] + kt * TILE_K) : make_uint4(0, 0, 0, 0);
      rw[i] = inside ? *reinterpret_cast<const uint4*>(w_src[i] + kt * TILE_K) : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int row = r0 + 32 * i;
      *reinterpret_cast<uint4*>(&lds[buf][0][swizzled(row, c)]) = ra[i];
      *reinterpret_cast<uint4*>(&lds[buf][1][swizzled(row, c)]) = rw[i];
    }
  };

  floatx16 acc[2][2];
#pragma unroll
  for (int bn = 0; bn < 2; ++bn)
#pragma unroll
    for (int bm = 0; bm < 2; ++bm)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[bn][bm][r] = 0.f;

  if (kt_begin < kt_end) {
    load_tile(kt_begin);
    store_tile(0);
  }
  __syncthreads();
  for (int kt = kt_begin; kt < kt_end; ++kt) {
    int buf = (kt - kt_begin) & 1;
    bool more = kt + 1 < kt_end;
    if (more) load_tile(kt + 1);
#pragma unroll
    for (int kk = 0; kk < TILE_K / 16; ++kk) {
      bf16x8 wop[2], aop[2];
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        int wrow = wn * 64 + b * 32 + l32, arow = wm * 64 + b * 32 + l32;
        wop[b] = *reinterpret_cast<const bf16x8*>(&lds[buf][1][swizzled(wrow, 2 * kk + g)]);
        aop[b] = *reinterpret_cast<const bf16x8*>(&lds[buf][0][swizzled(arow, 2 * kk + g)]);
      }
#pragma unroll
      for (int bn = 0; bn < 2; ++bn)
#pragma unroll
        for (int bm = 0; bm < 2; ++bm)
          acc[bn][bm] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wop[bn], aop[bm], acc[bn][bm], 0, 0, 0);
    }
    if (more) store_tile(buf ^ 1);
    __syncthreads();
  }

  // lane holds D[i][j]: i = 8 * (r / 4) + 4 * g + r % 4 (column n), j = lane % 32 (row m)
#pragma unroll
  for (int bm = 0; bm < 2; ++bm) {
    int m = m_base + wm * 64 + bm * 32 + l32;
    if (m >= M) continue;
#pragma unroll
    for (int bn = 0; bn < 2; ++bn) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float v[4] = {acc[bn][bm][4 * q], acc[bn][bm][4 * q + 1], acc[bn][bm][4 * q + 2], acc[bn][bm][4 * q + 3]};
        int n0 = n_base + wn * 64 + bn * 32 + q * 8 + g * 4;
        epilogue4<bf16_t>(epi, N, m, n0, v, split);
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
template <int MT, int U, int WAVES>
__global__ void __launch_bounds__(WAVES * 64)
gemm_skinny_kernel(const bf16_t* __restrict__ A, int64_t lda, const bf16_t* __restrict__ W, int M, int N,
                   int K, Epilogue epi) {
  __shared__ __attribute__((aligned(16))) float red[WAVES][MT][64][4];
  // the wave's number is the same in all its lanes: saying so keeps every test on it a scalar
  // branch, which costs no wait for loads in flight (a divergent one does)
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int i16 = lane & 15, g = lane >> 4;
  const int n_base = blockIdx.x * 16;
  const int split = blockIdx.y, splits = gridDim.y;
  int n = n_base + i16;
  n = n < N ? n : N - 1;
  const bf16_t* w_row = W + (int64_t)n * K;
  const bf16_t* a_row[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int m = mt * 16 + i16;
    a_row[mt] = A + (int64_t)(m < M ? m : M - 1) * lda;
  }
  // A batch is two phases.  First every load of the batch is issued: a chunk of 32 beyond K is
  // skipped by a scalar branch, a group of eight beyond K (a multiple of 8) inside the last chunk
  // reads the row's last group instead.  Only then are the weights of such a group cleared (with
  // a bit mask) and multiplied.  Nothing that depends on a lane or on loaded data stands between
  // the loads, so the compiler has no reason to wait for one before it issues the next.
  // Rows beyond M repeat row M - 1; their results are dropped by the epilogue.
  typedef __attribute__((__vector_size__(4 * sizeof(int)))) int int4v;
  const int chunks = chunks_of(K);
  const int stride = splits * WAVES;
  floatx4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = floatx4{0.f, 0.f, 0.f, 0.f};
  int4v wv[U], av[U][MT];
  auto issue = [&](int c0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int cc = c0 + u * stride;
      wv[u] = int4v{0, 0, 0, 0};
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) av[u][mt] = int4v{0, 0, 0, 0};
      if (cc < chunks) {
        int k = cc * 32 + g * 8;
        int kc = k < K ? k : K - 8;
        wv[u] = *reinterpret_cast<const int4v*>(w_row + kc);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) av[u][mt] = *reinterpret_cast<const int4v*>(a_row[mt] + kc);
      }
    }
  };
  auto multiply = [&](int c0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int keep = (c0 + u * stride) * 32 + g * 8 < K ? -1 : 0;
      bf16x8 w = __builtin_bit_cast(bf16x8, wv[u] & keep);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w, __builtin_bit_cast(bf16x8, av[u][mt]), acc[mt], 0, 0, 0);
    }
  };
  int c0 = split * WAVES + wave;
  issue(c0);
  // wave w < MT finishes row block w: lane holds D[i][j], i = 4 * (lane / 16) + r (column n),
  // j = lane % 16 (row m); what its epilogue needs is fetched now, behind the first batch
  const int out_m = (wave < MT ? wave : 0) * 16 + i16, out_n0 = n_base + g * 4;
  EpiloguePrefetch pre = {};
  if (wave < MT) pre = epilogue_prefetch(epi, M, N, out_m, out_n0, split);
  multiply(c0);
  for (c0 += stride * U; c0 < chunks; c0 += stride * U) {
    issue(c0);
    multiply(c0);
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
    *reinterpret_cast<floatx4*>(&red[wave][mt][lane][0]) = acc[mt];
  __syncthreads();
  if (wave < MT) {
    float v[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < WAVES; ++w)
#pragma unroll
      for (int r = 0; r < 4; ++r) v[r] += red[w][wave][lane][r];
    if (out_m < M) epilogue4_prefetched<bf16_t>(epi, N, out_m, out_n0, v, split, pre);
  }
}

static int check_operands(const char* who, const void* A, int64_t lda, const void* W, int M, int N, int K,
                          const Epilogue& e, int splits) {
  if (N <= 0 || K <= 0) BT_REFUSE("%s: N %d and K %d must be positive", who, N, K);
  if (K % 8 != 0 || lda % 8 != 0)
    BT_REFUSE("%s: K %d and the row pitch %lld must be multiples of 8 (16-byte loads)", who, K, (long long)lda);
  if (((uintptr_t)A & 15) || ((uintptr_t)W & 15)) BT_REFUSE("%s: operands must be 16-byte aligned", who);
  if (e.mode < 0 || e.mode > 4 || e.out == nullptr) BT_REFUSE("%s: bad epilogue", who);
  if (splits < 1 || (splits > 1 && e.mode != EPI_F32))
    BT_REFUSE("%s: K can be split %d ways only into 32-bit partial sums", who, splits);
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

BT_EXPORT int bt_gemm_tile_bf16(void* stream, const void* A, int64_t lda, const void* W, int M, int N, int K,
                                const Epilogue* epi, int splits) {
  if (M <= 0) return BT_OK;
  int rc = check_operands("gemm_tile_bf16", A, lda, W, M, N, K, *epi, splits);
  if (rc) return rc;
  dim3 grid((N + TILE_N - 1) / TILE_N, (M + TILE_M - 1) / TILE_M, splits), block(256);
  hipLaunchKernelGGL(gemm_tile_kernel, grid, block, 0, (hipStream_t)stream, (const bf16_t*)A, lda,
                     (const bf16_t*)W, M, N, K, *epi);
  return bt_check_launch("gemm_tile_bf16");
}

BT_EXPORT int bt_gemm_skinny_bf16(void* stream, const void* A, int64_t lda, const void* W, int M, int N, int K,
                                  const Epilogue* epi, int splits) {
  if (M <= 0) return BT_OK;
  if (M > 64) BT_REFUSE("gemm_skinny_bf16: %d rows, at most 64", M);
  int rc = check_operands("gemm_skinny_bf16", A, lda, W, M, N, K, *epi, splits);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  const bf16_t* a = (const bf16_t*)A;
  const bf16_t* w = (const bf16_t*)W;
  dim3 grid((N + 15) / 16, splits);
  if (M <= 16)
    hipLaunchKernelGGL((gemm_skinny_kernel<1, 8, 8>), grid, dim3(512), 0, s, a, lda, w, M, N, K, *epi);
  else if (M <= 32)
    hipLaunchKernelGGL((gemm_skinny_kernel<2, 4, 8>), grid, dim3(512), 0, s, a, lda, w, M, N, K, *epi);
  else
    hipLaunchKernelGGL((gemm_skinny_kernel<4, 2, 8>), grid, dim3(512), 0, s, a, lda, w, M, N, K, *epi);
  return bt_check_launch("gemm_skinny_bf16");
}
