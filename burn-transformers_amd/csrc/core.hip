// Core kernel module: the kernels every run needs, in plain form.
//   * embedding gather (+ learned position table)
//   * residual add + normalisation (32-bit statistics)
//   * a plain tiled matrix product with true 32-bit multiply-accumulate
//   * plain attention over the paged cache (one work-group per query row and head)
//   * greedy and temperature sampling with log-probabilities
// The 32-bit path of the model runs entirely on these; the bfloat16 path uses them for
// everything that is not an MFMA kernel, and the tests use the matrix product and the
// attention here as the slow twins of the MFMA kernels.

#include <float.h>

#include <mutex>

#define BT_EPILOGUE_ANY_HEAD_SIZE      // the plain product takes fused projections of any head size
#include "host.h"
#include "epilogue.h"
#include "attention.h"
#include "calls.h"
#include "no_alloc.h"

// ---------------------------------------------------------------------------------------------
// Embedding: x[t] = table[ids[t]] (+ positions[pos[t]]), written as 32-bit residual stream.
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(const int* __restrict__ ids, const int* __restrict__ pos,
                             const T* __restrict__ table, const T* __restrict__ positions,
                             float* __restrict__ out, int width) {
  int t = blockIdx.x;
  const T* row = table + (int64_t)ids[t] * width;
  const T* prow = positions ? positions + (int64_t)pos[t] * width : nullptr;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float v = to_float(row[c]);
    if (prow) v += to_float(prow[c]);
    out[(int64_t)t * width + c] = v;
  }
}

BT_EXPORT int bt_embed(void* stream, int dtype, const int* ids, const int* pos, const void* table,
                       const void* positions, float* out, int tokens, int width) {
  if (tokens <= 0) return BT_OK;
  if (width <= 0) BT_REFUSE("embed: width %d must be positive", width);
  dim3 grid(tokens), block(256);
  if (dtype == 0)
    hipLaunchKernelGGL(embed_kernel<float>, grid, block, 0, (hipStream_t)stream, ids, pos,
                       (const float*)table, (const float*)positions, out, width);
  else
    hipLaunchKernelGGL(embed_kernel<bf16_t>, grid, block, 0, (hipStream_t)stream, ids, pos,
                       (const bf16_t*)table, (const bf16_t*)positions, out, width);
  return bt_check_launch("embed");
}

// ---------------------------------------------------------------------------------------------
// Residual add + normalisation.
//   v = x[t] + sum_s delta[s][t] + bias          (t = rows ? rows[r] : r)
//   x[t] = v                                     (if write_back)
//   out[r] = norm(v) * gamma + beta              kind 0: (v - mean) / sqrt(var + eps)
//                                                kind 1: v / sqrt(mean(v^2) + eps), no beta
// Statistics in 32-bit with two passes over the row kept in LDS.
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void add_norm_kernel(float* __restrict__ x, const float* __restrict__ delta, int n_delta,
                                int64_t delta_stride, const float* __restrict__ bias,
                                const float* __restrict__ gamma, const float* __restrict__ beta,
                                float eps, int kind, T* __restrict__ out, const int* __restrict__ rows,
                                int width, int write_back, int out_rows) {
  extern __shared__ float row_buf[];
  __shared__ float scratch[32];
  int r = blockIdx.x;
  int t = rows ? rows[r] : r;
  float* xr = x + (int64_t)t * width;
  float partial = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float v = xr[c];
    for (int s = 0; s < n_delta; ++s) v += delta[s * delta_stride + (int64_t)t * width + c];
    if (bias) v += bias[c];
    row_buf[c] = v;
    if (write_back) xr[c] = v;
    partial += (kind == 0) ? v : v * v;
  }
  float total = block_sum(partial, scratch);
  float mean = 0.f, rstd;
  if (kind == 0) {
    mean = total / (float)width;
    float sq = 0.f;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
      float dlt = row_buf[c] - mean;
      sq += dlt * dlt;
    }
    float var = block_sum(sq, scratch) / (float)width;
    rstd = 1.0f / sqrtf(var + eps);
  } else {
    rstd = 1.0f / sqrtf(total / (float)width + eps);
  }
  if (out == nullptr) return;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float y = (row_buf[c] - mean) * rstd * gamma[c];
    if (beta) y += beta[c];
    out[activation_offset<T>(out_rows, width, r, c)] = from_float<T>(y);
  }
}

// The same for rows whose width is a multiple of four and at most 1024 * VPT (VPT up to 4), with
// exactly NS partial sums: the row lives in registers and the code is straight-line, so every
// load of a thread (stream, each partial sum, bias, scale, shift) is a 16-byte load that is in
// flight together with all the others.  A decode step has few rows: one row's latency counts.
// Zeros to read where a bias or a shift is absent: selecting the pointer keeps the loads
// unconditional (a test of the pointer around each load would split them into pieces).
__device__ float bt_zero_row[4096];

template <typename T, int VPT, int NS>
__global__ void __launch_bounds__(256)
add_norm_vec_kernel(float* __restrict__ x, const float* __restrict__ delta, int64_t delta_stride,
                    const float* __restrict__ bias, const float* __restrict__ gamma,
                    const float* __restrict__ beta, float eps, int kind, T* __restrict__ out,
                    const int* __restrict__ rows, int width, int write_back, int out_rows) {
  __shared__ float scratch[32];
  const int r = blockIdx.x;
  const int t = rows ? rows[r] : r;
  const int quads = width >> 2;
  float4* xr = reinterpret_cast<float4*>(x) + (int64_t)t * quads;
  const float4* dr = reinterpret_cast<const float4*>(delta) + (int64_t)t * quads;
  const int64_t dstride = delta_stride >> 2;
  const float4* z4 = reinterpret_cast<const float4*>(bt_zero_row);
  const float4* b4 = bias ? reinterpret_cast<const float4*>(bias) : z4;
  const float4* g4 = gamma ? reinterpret_cast<const float4*>(gamma) : z4;
  const float4* be4 = beta ? reinterpret_cast<const float4*>(beta) : z4;
  float4 v[VPT], part[VPT][NS > 0 ? NS : 1], b[VPT], g[VPT], be[VPT];
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    int c = threadIdx.x + i * 256;
    int cc = c < quads ? c : 0;     // lanes beyond the row read column 0; the result is never used
    v[i] = xr[cc];
#pragma unroll
    for (int s = 0; s < NS; ++s) part[i][s] = dr[s * dstride + cc];
    b[i] = b4[cc];
    g[i] = g4[cc];
    be[i] = be4[cc];
  }
  float partial = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
#pragma unroll
    for (int s = 0; s < NS; ++s) {   // same order of additions as the plain kernel
      v[i].x += part[i][s].x; v[i].y += part[i][s].y; v[i].z += part[i][s].z; v[i].w += part[i][s].w;
    }
    v[i].x += b[i].x; v[i].y += b[i].y; v[i].z += b[i].z; v[i].w += b[i].w;
    int c = threadIdx.x + i * 256;
    if (c < quads) {
      if (write_back) xr[c] = v[i];
      partial += (kind == 0) ? (v[i].x + v[i].y + v[i].z + v[i].w)
                             : (v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w);
    }
  }
  if (out == nullptr) return;
  float total = block_sum(partial, scratch);
  float mean = 0.f, rstd;
  if (kind == 0) {
    mean = total / (float)width;
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      if (threadIdx.x + i * 256 < quads) {
        float a0 = v[i].x - mean, a1 = v[i].y - mean, a2 = v[i].z - mean, a3 = v[i].w - mean;
        sq += a0 * a0 + a1 * a1 + a2 * a2 + a3 * a3;
      }
    }
    float var = block_sum(sq, scratch) / (float)width;
    rstd = 1.0f / sqrtf(var + eps);
  } else {
    rstd = 1.0f / sqrtf(total / (float)width + eps);
  }
  T* orow = out + (int64_t)r * width;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    int c = threadIdx.x + i * 256;
    if (c >= quads) continue;
    float y[4] = {(v[i].x - mean) * rstd * g[i].x + be[i].x, (v[i].y - mean) * rstd * g[i].y + be[i].y,
                  (v[i].z - mean) * rstd * g[i].z + be[i].z, (v[i].w - mean) * rstd * g[i].w + be[i].w};
    if (out_rows == 0) store4<T>(orow + 4 * c, y, 4, true);        // (the same branch for every thread)
    else store4<T>(out + activation_offset<T>(out_rows, width, r, 4 * c), y, 4, true);
  }
}

// The same for steps with many rows (a prefill): one WAVE per row, four rows per work-group.  The
// row lives in the wave's registers (QPL quads of four floats per lane, so width <= 256 * QPL),
// statistics are wave reductions with no barrier, and a compute unit has many rows in flight;
// with one work-group per row the two block-wide reductions leave the memory system idle.
// NS: the number of pending partial sums (n_delta), so that they are all asked for together with
// the row, or -1 for any number, one trip to memory after the other (512 rows with two sums
// pending: 9.2 us that way).
template <typename T, int QPL, int NS>
__global__ void __launch_bounds__(256)
add_norm_rows_kernel(float* __restrict__ x, const float* __restrict__ delta, int n_delta, int64_t delta_stride,
                     const float* __restrict__ bias, const float* __restrict__ gamma,
                     const float* __restrict__ beta, float eps, int kind, T* __restrict__ out,
                     const int* __restrict__ rows, int n_rows, int width, int write_back) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = blockIdx.x * 4 + wave;
  if (r >= n_rows) return;                     // a whole wave leaves; there is no barrier below
  const int t = rows ? rows[r] : r;
  const int quads = width >> 2;
  float4* xr = reinterpret_cast<float4*>(x) + (int64_t)t * quads;
  const float4* dr = reinterpret_cast<const float4*>(delta) + (int64_t)t * quads;
  const int64_t dstride = delta_stride >> 2;
  const float4* z4 = reinterpret_cast<const float4*>(bt_zero_row);
  const float4* b4 = bias ? reinterpret_cast<const float4*>(bias) : z4;
  const float4* g4 = gamma ? reinterpret_cast<const float4*>(gamma) : z4;
  const float4* be4 = beta ? reinterpret_cast<const float4*>(beta) : z4;
  // every vector a lane needs is asked for before anything is added: one trip to memory
  float4 v[QPL], b[QPL], g[QPL], be[QPL];
#pragma unroll
  for (int i = 0; i < QPL; ++i) {
    int c = lane + i * 64;
    int cc = c < quads ? c : 0;
    v[i] = xr[cc];
    b[i] = b4[cc];
    g[i] = g4[cc];
    be[i] = be4[cc];
  }
  if constexpr (NS >= 0) {                     // same order of additions as the plain kernel
    float4 d[NS > 0 ? NS : 1][QPL];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
      for (int i = 0; i < QPL; ++i) {
        int c = lane + i * 64;
        d[s][i] = dr[s * dstride + (c < quads ? c : 0)];
      }
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
      for (int i = 0; i < QPL; ++i) {
        v[i].x += d[s][i].x; v[i].y += d[s][i].y; v[i].z += d[s][i].z; v[i].w += d[s][i].w;
      }
  } else {
    for (int s = 0; s < n_delta; ++s) {
#pragma unroll
      for (int i = 0; i < QPL; ++i) {
        int c = lane + i * 64;
        float4 d = dr[s * dstride + (c < quads ? c : 0)];
        v[i].x += d.x; v[i].y += d.y; v[i].z += d.z; v[i].w += d.w;
      }
    }
  }
  float partial = 0.f;
#pragma unroll
  for (int i = 0; i < QPL; ++i) {
    int c = lane + i * 64;
    v[i].x += b[i].x; v[i].y += b[i].y; v[i].z += b[i].z; v[i].w += b[i].w;
    if (c < quads) {
      if (write_back) xr[c] = v[i];
      partial += (kind == 0) ? (v[i].x + v[i].y + v[i].z + v[i].w)
                             : (v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w);
    }
  }
  if (out == nullptr) return;
  float total = wave_sum(partial);
  float mean = 0.f, rstd;
  if (kind == 0) {
    mean = total / (float)width;
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < QPL; ++i) {
      if (lane + i * 64 < quads) {
        float a0 = v[i].x - mean, a1 = v[i].y - mean, a2 = v[i].z - mean, a3 = v[i].w - mean;
        sq += a0 * a0 + a1 * a1 + a2 * a2 + a3 * a3;
      }
    }
    rstd = 1.0f / sqrtf(wave_sum(sq) / (float)width + eps);
  } else {
    rstd = 1.0f / sqrtf(total / (float)width + eps);
  }
  T* orow = out + (int64_t)r * width;
#pragma unroll
  for (int i = 0; i < QPL; ++i) {
    int c = lane + i * 64;
    if (c < quads) {
      float y[4] = {(v[i].x - mean) * rstd * g[i].x + be[i].x, (v[i].y - mean) * rstd * g[i].y + be[i].y,
                    (v[i].z - mean) * rstd * g[i].z + be[i].z, (v[i].w - mean) * rstd * g[i].w + be[i].w};
      store4<T>(orow + 4 * c, y, 4, true);
    }
  }
}

template <typename T, int VPT>
static bool launch_add_norm_vec(hipStream_t stream, dim3 grid, float* x, const float* delta, int n_delta,
                                int64_t delta_stride, const float* bias, const float* gamma, const float* beta,
                                float eps, int kind, T* out, const int* rows, int width, int write_back, int out_rows) {
#define BT_ADD_NORM_VEC(NS)                                                                                  \
  hipLaunchKernelGGL((add_norm_vec_kernel<T, VPT, NS>), grid, dim3(256), 0, stream, x, delta, delta_stride,  \
                     bias, gamma, beta, eps, kind, out, rows, width, write_back, out_rows)
  switch (n_delta) {
    case 0: BT_ADD_NORM_VEC(0); return true;
    case 1: BT_ADD_NORM_VEC(1); return true;
    case 2: BT_ADD_NORM_VEC(2); return true;
    case 3: BT_ADD_NORM_VEC(3); return true;
    case 4: BT_ADD_NORM_VEC(4); return true;
    case 5: BT_ADD_NORM_VEC(5); return true;
    case 6: BT_ADD_NORM_VEC(6); return true;
    case 7: BT_ADD_NORM_VEC(7); return true;
    case 8: BT_ADD_NORM_VEC(8); return true;
    default: return false;
  }
#undef BT_ADD_NORM_VEC
}

template <typename T>
static void launch_add_norm(hipStream_t stream, float* x, const float* delta, int n_delta, int64_t delta_stride,
                            const float* bias, const float* gamma, const float* beta, float eps, int kind,
                            T* out, const int* rows, int n_rows, int width, int write_back, int out_rows) {
  dim3 grid(n_rows);
  auto aligned = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
  bool vec = width % 4 == 0 && width <= 4096 && delta_stride % 4 == 0 && aligned(x) && aligned(delta) &&
             aligned(bias) && aligned(gamma) && aligned(beta) && aligned(out);
  bool done = false;
  if (vec && n_rows >= 512 && out_rows == 0) {        // many rows: a wave per row (row-major output only)
    dim3 row_grid((n_rows + 3) / 4);
#define BT_ADD_NORM_ROWS_NS(QPL, NS)                                                                            \
  hipLaunchKernelGGL((add_norm_rows_kernel<T, QPL, NS>), row_grid, dim3(256), 0, stream, x, delta, n_delta,      \
                     delta_stride, bias, gamma, beta, eps, kind, out, rows, n_rows, width, write_back)
#define BT_ADD_NORM_ROWS(QPL)                                                                                   \
  do {                                                                                                          \
    switch (n_delta) {                                                                                          \
      case 0: BT_ADD_NORM_ROWS_NS(QPL, 0); break;                                                               \
      case 1: BT_ADD_NORM_ROWS_NS(QPL, 1); break;                                                               \
      case 2: BT_ADD_NORM_ROWS_NS(QPL, 2); break;                                                               \
      case 3: BT_ADD_NORM_ROWS_NS(QPL, 3); break;                                                               \
      case 4: BT_ADD_NORM_ROWS_NS(QPL, 4); break;                                                               \
      default: BT_ADD_NORM_ROWS_NS(QPL, -1);                                                                    \
    }                                                                                                           \
  } while (0)
    if (width <= 1024) BT_ADD_NORM_ROWS(4);
    else if (width <= 2048) BT_ADD_NORM_ROWS(8);
    else {            // (rows so wide keep the loop: four sums of sixteen quads would not fit the registers)
      BT_ADD_NORM_ROWS_NS(16, -1);
    }
#undef BT_ADD_NORM_ROWS
#undef BT_ADD_NORM_ROWS_NS
    return;
  }
  if (vec && width <= 1024)
    done = launch_add_norm_vec<T, 1>(stream, grid, x, delta, n_delta, delta_stride, bias, gamma, beta, eps, kind, out, rows, width, write_back, out_rows);
  else if (vec && width <= 2048)
    done = launch_add_norm_vec<T, 2>(stream, grid, x, delta, n_delta, delta_stride, bias, gamma, beta, eps, kind, out, rows, width, write_back, out_rows);
  else if (vec)
    done = launch_add_norm_vec<T, 4>(stream, grid, x, delta, n_delta, delta_stride, bias, gamma, beta, eps, kind, out, rows, width, write_back, out_rows);
  if (!done)
    hipLaunchKernelGGL(add_norm_kernel<T>, grid, dim3(256), (size_t)width * sizeof(float), stream, x, delta,
                       n_delta, delta_stride, bias, gamma, beta, eps, kind, out, rows, width, write_back, out_rows);
}

BT_EXPORT int bt_add_norm(void* stream, int out_dtype, float* x, const float* delta, int n_delta,
                          int64_t delta_stride, const float* bias, const float* gamma,
                          const float* beta, float eps, int kind, void* out, const int* rows,
                          int n_rows, int width, int write_back, int out_rows) {
  if (n_rows <= 0) return BT_OK;
  if (out_rows != 0 && (out == nullptr || out_rows < n_rows))
    BT_REFUSE("add_norm: a chunk-major output of %d rows for %d rows", out_rows, n_rows);
  if (width <= 0 || width > 15360) BT_REFUSE("add_norm: width %d outside 1..15360 (the row is held in LDS)", width);
  if (kind != 0 && kind != 1) BT_REFUSE("add_norm: unknown norm kind %d", kind);
  if (out_dtype == 0)
    launch_add_norm<float>((hipStream_t)stream, x, delta, n_delta, delta_stride, bias, gamma, beta, eps, kind,
                           (float*)out, rows, n_rows, width, write_back, out_rows);
  else
    launch_add_norm<bf16_t>((hipStream_t)stream, x, delta, n_delta, delta_stride, bias, gamma, beta, eps, kind,
                            (bf16_t*)out, rows, n_rows, width, write_back, out_rows);
  return bt_check_launch("add_norm");
}

// ---------------------------------------------------------------------------------------------
// Plain matrix product C[M,N] = A[M,K] . W[N,K]^T with 32-bit FMA accumulation.
// 64 x 64 tile, K in steps of 16, 256 threads with 4 x 4 outputs each.  Any M, N, K.
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
gemm_plain_kernel(const T* __restrict__ A, int64_t lda, const T* __restrict__ W, int M, int N, int K,
                  Epilogue epi) {
  __shared__ float As[16][64 + 4];
  __shared__ float Ws[16][64 + 4];
  int tid = threadIdx.x;
  int tx = tid & 15, ty = tid >> 4;
  int m_base = blockIdx.y * 64, n_base = blockIdx.x * 64;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += 16) {
    // each thread loads 4 elements of A and of W: row = tid / 4 .. , column = (tid % 16)
    for (int e = tid; e < 64 * 16; e += 256) {
      int row = e >> 4, col = e & 15;
      int k = k0 + col;
      int m = m_base + row, n = n_base + row;
      As[col][row] = (m < M && k < K) ? to_float(A[(int64_t)m * lda + k]) : 0.f;
      Ws[col][row] = (n < N && k < K) ? to_float(W[(int64_t)n * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int m = m_base + ty * 4 + i;
    if (m < M) epilogue4<T>(epi, N, m, n_base + tx * 4, acc[i], 0);
  }
}

int bt_check_epilogue(const Epilogue& e, int N, const char* who) {
  if (e.mode < 0 || e.mode > 4) BT_REFUSE("%s: unknown epilogue mode %d", who, e.mode);
  if (e.out == nullptr) BT_REFUSE("%s: epilogue has no output", who);
  if (e.mode == EPI_QKV) {
    if (e.kv.head_dim <= 0) BT_REFUSE("%s: head size %d must be positive", who, e.kv.head_dim);
    if (e.n_q % e.kv.head_dim != 0 || e.n_kv != e.kv.kv_heads * e.kv.head_dim || e.n_q + 2 * e.n_kv != N)
      BT_REFUSE("%s: fused projection of %d columns does not split into %d query and 2 x %d key/value columns",
                who, N, e.n_q, e.n_kv);
    if (!e.tok_seq || !e.tok_pos || !e.kv.blocks || !e.kv.keys || !e.kv.values)
      BT_REFUSE("%s: the key/value scatter needs token and cache tables", who);
  }
  return BT_OK;
}

BT_EXPORT int bt_gemm_plain(void* stream, int dtype, const void* A, int64_t lda, const void* W, int M,
                            int N, int K, const Epilogue* epi) {
  if (M <= 0) return BT_OK;
  if (N <= 0 || K <= 0) BT_REFUSE("gemm_plain: N %d and K %d must be positive", N, K);
  int rc = bt_check_epilogue(*epi, N, "gemm_plain");
  if (rc) return rc;
  dim3 grid((N + 63) / 64, (M + 63) / 64), block(256);
  if (dtype == 0)
    hipLaunchKernelGGL(gemm_plain_kernel<float>, grid, block, 0, (hipStream_t)stream, (const float*)A, lda,
                       (const float*)W, M, N, K, *epi);
  else
    hipLaunchKernelGGL(gemm_plain_kernel<bf16_t>, grid, block, 0, (hipStream_t)stream, (const bf16_t*)A,
                       lda, (const bf16_t*)W, M, N, K, *epi);
  return bt_check_launch("gemm_plain");
}

// ---------------------------------------------------------------------------------------------
// Plain attention over the paged cache.  One work-group per (token, query head).
//   scores s_k = scale * (q . key_k) for keys lo <= k <= pos, lo = max(0, pos - window + 1)
//   out = sum_k softmax(s)_k value_k, softmax in 32-bit with a running maximum over chunks.
// Keys beyond the token's own position are never read.
// ---------------------------------------------------------------------------------------------
#define PLAIN_CHUNK 1024


template <typename T>
__global__ void __launch_bounds__(256)
attention_plain_kernel(AttnArgs a) {
  __shared__ float qs[256];
  __shared__ float ps[PLAIN_CHUNK];
  __shared__ float scratch[32];
  int t = blockIdx.x, head = blockIdx.y;
  int hd = a.kv.head_dim;
  int group = a.q_heads / a.kv.kv_heads;
  int kv_head = head / group;
  int seq = a.tok_seq[t], pos = a.tok_pos[t];
  const T* q = static_cast<const T*>(a.q) + (int64_t)t * a.ldq + head * hd;
  for (int c = threadIdx.x; c < hd; c += blockDim.x) qs[c] = to_float(q[c]);
  __syncthreads();
  int lo = (a.window > 0 && pos - a.window + 1 > 0) ? pos - a.window + 1 : 0;
  float run_max = -INFINITY, run_sum = 0.f, acc = 0.f;  // acc: channel threadIdx.x (< hd)
  const T* keys = static_cast<const T*>(a.kv.keys);
  const T* values = static_cast<const T*>(a.kv.values);
  for (int c0 = lo; c0 <= pos; c0 += PLAIN_CHUNK) {
    int n = pos + 1 - c0 < PLAIN_CHUNK ? pos + 1 - c0 : PLAIN_CHUNK;
    float local_max = -INFINITY;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
      int k = c0 + i;
      const T* kr = keys + kv_block_base(a.kv, seq, k, kv_head) + key_offset(hd, k, 0);
      float s = 0.f;
      for (int c = 0; c < hd; ++c) s = fmaf(qs[c], to_float(kr[c]), s);
      s *= a.scale;
      ps[i] = s;
      local_max = fmaxf(local_max, s);
    }
    float chunk_max = block_max(local_max, scratch);
    float new_max = fmaxf(run_max, chunk_max);
    float rescale = (run_max == -INFINITY) ? 0.f : expf(run_max - new_max);
    float local_sum = 0.f;
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
      float p = expf(ps[i] - new_max);
      ps[i] = p;
      local_sum += p;
    }
    float chunk_sum = block_sum(local_sum, scratch);
    run_sum = run_sum * rescale + chunk_sum;
    run_max = new_max;
    __syncthreads();
    if ((int)threadIdx.x < hd) {
      acc *= rescale;
      for (int i = 0; i < n; ++i) {
        int k = c0 + i;
        const T* vr = values + kv_block_base(a.kv, seq, k, kv_head);
        acc = fmaf(ps[i], to_float(vr[value_offset(hd, k, threadIdx.x)]), acc);
      }
    }
    __syncthreads();
  }
  if ((int)threadIdx.x < hd) {
    T* o = static_cast<T*>(a.out) + (int64_t)t * a.ldo + head * hd;
    o[threadIdx.x] = from_float<T>(run_sum > 0.f ? acc / run_sum : 0.f);
  }
}

int bt_check_attention(const AttnArgs& a, const char* who) {
  int hd = a.kv.head_dim;
  if (hd <= 0 || hd > 256) BT_REFUSE("%s: head size %d outside 1..256 (a work-group holds a query and one channel per thread)", who, hd);
  if (a.kv.kv_heads <= 0 || a.q_heads <= 0 || a.q_heads % a.kv.kv_heads != 0)
    BT_REFUSE("%s: %d query heads cannot share %d key/value heads", who, a.q_heads, a.kv.kv_heads);
  if (a.window < 0) BT_REFUSE("%s: window %d must not be negative", who, a.window);
  if (!a.q || !a.out || !a.tok_seq || !a.tok_pos || !a.seq_off || !a.seq_start || !a.kv.blocks ||
      !a.kv.keys || !a.kv.values)
    BT_REFUSE("%s: missing operand", who);
  return BT_OK;
}

BT_EXPORT int bt_attention_plain(void* stream, int dtype, const AttnArgs* args) {
  if (args->out_rows != 0) BT_REFUSE("attention_plain: a chunk-major output is written by the bfloat16 decode kernel only");
  if (args->n_tokens <= 0) return BT_OK;
  int rc = bt_check_attention(*args, "attention_plain");
  if (rc) return rc;
  dim3 grid(args->n_tokens, args->q_heads), block(256);
  if (dtype == 0)
    hipLaunchKernelGGL(attention_plain_kernel<float>, grid, block, 0, (hipStream_t)stream, *args);
  else
    hipLaunchKernelGGL(attention_plain_kernel<bf16_t>, grid, block, 0, (hipStream_t)stream, *args);
  return bt_check_launch("attention_plain");
}

// ---------------------------------------------------------------------------------------------
// Copies of keys and values between plain [tokens][kv_heads * head_dim] rows and the paged cache
// (used by mixers that do not go through the fused projection, and by tests that read the cache).
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void kv_copy_kernel(T* __restrict__ k_rows, T* __restrict__ v_rows, int64_t ld,
                               const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
                               KvView kv, int to_cache) {
  int t = blockIdx.x;
  int seq = tok_seq[t], pos = tok_pos[t];
  int hd = kv.head_dim;
  T* keys = static_cast<T*>(kv.keys);
  T* values = static_cast<T*>(kv.values);
  for (int c = threadIdx.x; c < kv.kv_heads * hd; c += blockDim.x) {
    int head = c / hd, channel = c % hd;
    int64_t base = kv_block_base(kv, seq, pos, head);
    int64_t ko = base + key_offset(hd, pos, channel), vo = base + value_offset(hd, pos, channel);
    if (to_cache) {
      keys[ko] = k_rows[(int64_t)t * ld + c];
      values[vo] = v_rows[(int64_t)t * ld + c];
    } else {
      k_rows[(int64_t)t * ld + c] = keys[ko];
      v_rows[(int64_t)t * ld + c] = values[vo];
    }
  }
}

// The same into the cache for bfloat16 rows of a prompt, with wide accesses.  A work-group takes
// four consecutive tokens of the step.  Keys: every token's row, eight channels (16 bytes) at a
// time.  Values lie with four consecutive positions interleaved per channel, so they are stored
// in runs of tokens that share such a group (same sequence, consecutive positions, same
// position / 4), each by the work-group that holds the run's first token: a full run of four is
// one 8-byte store per channel, a shorter one (the ends of a prompt that do not fall on a
// multiple of four) goes element by element.  Four consecutive tokens hold one such first token
// wherever the prompt starts, so the work-groups have equal work.
__global__ void __launch_bounds__(256)
kv_store_bf16_kernel(const bf16_t* __restrict__ k_rows, const bf16_t* __restrict__ v_rows, int64_t ld,
                     const int* __restrict__ tok_seq, const int* __restrict__ tok_pos, KvView kv, int tokens) {
  const int t0 = blockIdx.x * 4;
  // tokens t0 - 1 .. t0 + 6 (indices clamped into the step), all asked for at once
  int seqs[8], poss[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    int u = t0 - 1 + i;
    u = u < 0 ? 0 : (u < tokens ? u : tokens - 1);
    seqs[i] = tok_seq[u];
    poss[i] = tok_pos[u];
  }
  const int n = tokens - t0 < 4 ? tokens - t0 : 4;
  const int hd = kv.head_dim, width = kv.kv_heads * hd;
  bf16_t* keys = static_cast<bf16_t*>(kv.keys);
  bf16_t* values = static_cast<bf16_t*>(kv.values);
  typedef __attribute__((__vector_size__(4 * sizeof(int)))) int int4v;
  const int pieces = width >> 3;
  for (int q = threadIdx.x; q < n * pieces; q += 256) {
    int i = q / pieces, c = (q - i * pieces) * 8;
    int head = c / hd, channel = c % hd;
    int seq = seqs[1 + i], pos = poss[1 + i];
    *reinterpret_cast<int4v*>(keys + kv_block_base(kv, seq, pos, head) + key_offset(hd, pos, channel)) =
        *reinterpret_cast<const int4v*>(k_rows + (int64_t)(t0 + i) * ld + c);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (i >= n) break;
    const int t = t0 + i, seq = seqs[1 + i], pos = poss[1 + i];
    const bool continues = t > 0 && seqs[i] == seq && poss[i] == pos - 1 && (pos & 3) != 0;
    if (continues) continue;     // an earlier token stores this one's values with its own
    int run = 1;
#pragma unroll
    for (int j = 1; j < 4; ++j)
      if (run == j && t + j < tokens && seqs[1 + i + j] == seq && poss[1 + i + j] == pos + j && ((pos + j) & 3) != 0)
        run = j + 1;
    if (run == 4) {
      // pos is a multiple of four: eight channels of the four tokens are four 16-byte loads, and
      // transposed they are 64 consecutive bytes of the cache
      for (int c = threadIdx.x * 8; c < width; c += 256 * 8) {
        int head = c / hd, channel = c % hd;
        int4v row[4], quads[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) row[j] = *reinterpret_cast<const int4v*>(v_rows + (int64_t)(t + j) * ld + c);
#pragma unroll
        for (int k = 0; k < 4; ++k) {      // channels 2k and 2k + 1 lie in word k of every row
          unsigned a = row[0][k], b = row[1][k], d = row[2][k], e = row[3][k];
          quads[k] = int4v{(int)((a & 0xffffu) | (b << 16)), (int)((d & 0xffffu) | (e << 16)),
                           (int)((a >> 16) | (b & 0xffff0000u)), (int)((d >> 16) | (e & 0xffff0000u))};
        }
        int4v* to = reinterpret_cast<int4v*>(values + kv_block_base(kv, seq, pos, head) + value_offset(hd, pos, channel));
#pragma unroll
        for (int k = 0; k < 4; ++k) to[k] = quads[k];
      }
      continue;
    }
    for (int c = threadIdx.x; c < width; c += 256) {
      int head = c / hd, channel = c % hd;
      int64_t base = kv_block_base(kv, seq, pos, head);     // the run lies in one block
      for (int j = 0; j < run; ++j)
        values[base + value_offset(hd, pos + j, channel)] = v_rows[(int64_t)(t + j) * ld + c];
    }
  }
}

BT_EXPORT int bt_kv_copy(void* stream, int dtype, void* k_rows, void* v_rows, int64_t ld,
                         const int* tok_seq, const int* tok_pos, const KvView* kv, int tokens,
                         int to_cache) {
  if (tokens <= 0) return BT_OK;
  if (kv->head_dim <= 0) BT_REFUSE("kv_copy: head size %d must be positive", kv->head_dim);
  dim3 grid(tokens), block(256);
  const bool wide = dtype != 0 && to_cache && tokens > 64 && kv->head_dim % 8 == 0 && ld % 8 == 0 &&
                    ((uintptr_t)k_rows & 15) == 0 && ((uintptr_t)v_rows & 15) == 0 && ((uintptr_t)kv->keys & 15) == 0 &&
                    ((uintptr_t)kv->values & 15) == 0;
  if (wide) {
    hipLaunchKernelGGL(kv_store_bf16_kernel, dim3((tokens + 3) / 4), block, 0, (hipStream_t)stream, (const bf16_t*)k_rows,
                       (const bf16_t*)v_rows, ld, tok_seq, tok_pos, *kv, tokens);
    return bt_check_launch("kv_copy");
  }
  if (dtype == 0)
    hipLaunchKernelGGL(kv_copy_kernel<float>, grid, block, 0, (hipStream_t)stream, (float*)k_rows,
                       (float*)v_rows, ld, tok_seq, tok_pos, *kv, to_cache);
  else
    hipLaunchKernelGGL(kv_copy_kernel<bf16_t>, grid, block, 0, (hipStream_t)stream, (bf16_t*)k_rows,
                       (bf16_t*)v_rows, ld, tok_seq, tok_pos, *kv, to_cache);
  return bt_check_launch("kv_copy");
}

// ---------------------------------------------------------------------------------------------
// Sampling of each row of 32-bit logits [rows][vocab].
//   greedy: lowest index of the maximum; log-probability = log_softmax(z)[id]
//   sample: p = softmax(z / T); id = #{k : c_k < u * c_last} with c the running sum of p in
//           index order, u = ((mix(seed + gamma * (index + 1)) >> 41) + 0.5) / 2^23,
//           index = first_draw + (draw_rows ? draw_rows[row] : row); log-probability of the
//           tempered distribution.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ uint64_t splitmix64(uint64_t seed, uint64_t index) {
  uint64_t v = seed + 0x9E3779B97F4A7C15ull * (index + 1ull);
  v = (v ^ (v >> 30)) * 0xBF58476D1CE4E5B9ull;
  v = (v ^ (v >> 27)) * 0x94D049BB133111EBull;
  return v ^ (v >> 31);
}

// Two kernels, because one compute unit pulls a row of 50,257 logits (200 KB) no faster than in
// about 8 us, and the selection needs the row twice over: several work-groups per row (16, or
// more for vocabularies beyond 65,536) read their part of it ONCE into registers and leave
// (maximum, its lowest index, sum of exp(z - that maximum)); one work-group per row combines
// these and, when sampling, walks the one chunk that holds the drawn point.
#define SAMPLE_THREADS 512
#define SAMPLE_PER_THREAD 8      // a chunk holds at most SAMPLE_THREADS * SAMPLE_PER_THREAD logits
#define SAMPLE_CHUNK_MOST (SAMPLE_THREADS * SAMPLE_PER_THREAD)

static int sample_chunks(int vocab) {
  int needed = (vocab + SAMPLE_CHUNK_MOST - 1) / SAMPLE_CHUNK_MOST;
  return needed > 16 ? needed : 16;
}

struct SamplePartial {
  float top;      // maximum of z / divisor over the chunk
  float sum;      // sum of exp(z / divisor - top)
  int arg;        // lowest index of the maximum
  int pad;
};

__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_chunks_kernel(const float* __restrict__ logits, int64_t ld, int vocab, int chunk_len, float divisor,
                     SamplePartial* __restrict__ partials) {
  __shared__ float scratch[32];
  __shared__ int best_index[SAMPLE_THREADS / 64];
  __shared__ float best_value[SAMPLE_THREADS / 64];
  const int row = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
  const float* z = logits + (int64_t)row * ld;
  const int lo = chunk * chunk_len, hi = lo + chunk_len < vocab ? lo + chunk_len : vocab;
  float v[SAMPLE_PER_THREAD];
#pragma unroll
  for (int i = 0; i < SAMPLE_PER_THREAD; ++i) {
    int k = lo + tid + i * SAMPLE_THREADS;
    v[i] = k < hi ? z[k] / divisor : -INFINITY;
  }
  // maximum and its lowest index; a thread sees its indices in rising order, so `>` keeps the lowest
  float top = -INFINITY;
  int arg = 0x7fffffff;
#pragma unroll
  for (int i = 0; i < SAMPLE_PER_THREAD; ++i)
    if (v[i] > top) { top = v[i]; arg = lo + tid + i * SAMPLE_THREADS; }
  for (int o = 32; o > 0; o >>= 1) {
    float ov = __shfl_xor(top, o, 64);
    int oa = __shfl_xor(arg, o, 64);
    if (ov > top || (ov == top && oa < arg)) { top = ov; arg = oa; }
  }
  if ((tid & 63) == 0) { best_value[tid >> 6] = top; best_index[tid >> 6] = arg; }
  __syncthreads();
  top = best_value[0]; arg = best_index[0];
  for (int w = 1; w < SAMPLE_THREADS / 64; ++w)
    if (best_value[w] > top || (best_value[w] == top && best_index[w] < arg)) { top = best_value[w]; arg = best_index[w]; }
  float mine = 0.f;
  if (top != -INFINITY) {
#pragma unroll
    for (int i = 0; i < SAMPLE_PER_THREAD; ++i) mine += expf(v[i] - top);   // exp(-inf) = 0 beyond the chunk
  }
  float total = block_sum(mine, scratch);
  if (tid == 0) partials[row * gridDim.x + chunk] = SamplePartial{top, total, arg, 0};
}

__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_select_kernel(const float* __restrict__ logits, int64_t ld, int vocab, int chunk_len, int chunks, int sample,
                     float divisor, uint64_t seed, uint64_t first_draw, const int* __restrict__ draw_rows,
                     const SamplePartial* __restrict__ partials, int* __restrict__ ids, float* __restrict__ logp) {
  __shared__ float seg_sum[SAMPLE_THREADS];
  __shared__ int scratch_count[32];
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* z = logits + (int64_t)row * ld;
  const SamplePartial* part = partials + row * chunks;
  // every thread combines the few partial results itself: no exchange needed
  float top = -INFINITY;
  int arg = 0x7fffffff;
  for (int c = 0; c < chunks; ++c)
    if (part[c].top > top) { top = part[c].top; arg = part[c].arg; }   // chunks in index order: `>` keeps the lowest
  auto scaled = [&](int c) { return part[c].top == -INFINITY ? 0.f : part[c].sum * expf(part[c].top - top); };
  if (top == -INFINITY) {            // every score is -inf (all tokens excluded): nothing can be chosen
    if (tid == 0) { ids[row] = 0; logp[row] = -INFINITY; }
    return;
  }
  float total = 0.f;
  for (int c = 0; c < chunks; ++c) total += scaled(c);                  // in index order
  if (!sample) {
    if (tid == 0) {
      ids[row] = arg;
      logp[row] = z[arg] - top - logf(total);
    }
    return;
  }
  const float u = (float)(((double)(splitmix64(seed, first_draw + (uint64_t)(draw_rows ? draw_rows[row] : row)) >> 41) + 0.5) / 8388608.0);
  const float threshold = u * total;
  // the chunk in which the running sum reaches the threshold, and the sum before it
  float before = 0.f;
  int owner = chunks - 1;
  for (int c = 0; c < chunks - 1; ++c) {
    float with = before + scaled(c);
    if (with >= threshold) { owner = c; break; }
    before = with;
  }
  // within it every thread owns a contiguous segment, so that the prefix sums run in index order;
  // the answer is the number of logits whose running sum stays below the threshold
  const int lo = owner * chunk_len, hi = lo + chunk_len < vocab ? lo + chunk_len : vocab;
  const int seg = (hi - lo + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int slo = lo + tid * seg, shi = slo + seg < hi ? slo + seg : hi;
  float e[SAMPLE_PER_THREAD];
  float mine = 0.f;
#pragma unroll
  for (int i = 0; i < SAMPLE_PER_THREAD; ++i) {
    e[i] = slo + i < shi ? expf(z[slo + i] / divisor - top) : 0.f;
    mine += e[i];
  }
  seg_sum[tid] = mine;
  __syncthreads();
  float c = before;
  for (int t = 0; t < tid; ++t) c += seg_sum[t];
  int below = 0;
#pragma unroll
  for (int i = 0; i < SAMPLE_PER_THREAD; ++i) {
    c += e[i];
    if (slo + i < shi && c < threshold) ++below;
  }
  // (running sums rise with the index, so the logits below the threshold are a prefix of the chunk)
  int count = below;
  for (int o = 32; o > 0; o >>= 1) count += __shfl_xor(count, o, 64);
  if ((tid & 63) == 0) scratch_count[tid >> 6] = count;
  __syncthreads();
  if (tid == 0) {
    int all = 0;
    for (int w = 0; w < SAMPLE_THREADS / 64; ++w) all += scratch_count[w];
    int k = lo + all;
    if (k >= vocab) k = vocab - 1;
    ids[row] = k;
    logp[row] = z[k] / divisor - top - logf(total);
  }
}

// workspace: device memory for the partial results of every (row, chunk)
BT_EXPORT int64_t bt_sample_workspace_bytes(int rows, int vocab) {
  return (int64_t)rows * sample_chunks(vocab > 0 ? vocab : 1) * sizeof(SamplePartial);
}

static int launch_sample(void* stream, const float* logits, int64_t ld, int rows, int vocab, int sample,
                         float temperature, uint64_t seed, uint64_t first_draw, const int* draw_rows,
                         int* ids, float* logp, void* workspace);

BT_EXPORT int bt_sample(void* stream, const float* logits, int64_t ld, int rows, int vocab, int sample,
                        float temperature, uint64_t seed, uint64_t first_draw, const int* draw_rows,
                        int* ids, float* logp, void* workspace) {
  if (rows <= 0) return BT_OK;
  if (vocab <= 0) BT_REFUSE("sample: vocabulary %d must be positive", vocab);
  if (sample && !(temperature > 0.f)) BT_REFUSE("sample: temperature %g must be positive", (double)temperature);
  if (workspace == nullptr) BT_REFUSE("sample: no workspace");
  return launch_sample(stream, logits, ld, rows, vocab, sample, temperature, seed, first_draw, draw_rows, ids, logp,
                       workspace);
}

// The same without a workspace argument, for callers that cannot allocate (no_alloc.h): the
// partial results live in an array of the library's own on each GPU.  In host code the array's
// name is only a stand-in for the symbol; its address in a device's memory is looked up once per
// device, with that device current, and every use below goes through that address.
static __device__ __align__(256) unsigned char scratch[BT_NO_ALLOC_SCRATCH_BYTES];

#define BT_NO_ALLOC_MAX_DEVICES 64
static void* scratch_address[BT_NO_ALLOC_MAX_DEVICES];     // by device number; null = not looked up yet
static std::mutex scratch_lock;

static int scratch_on_current_device(void** address) {
  int device = -1;
  hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess) BT_REFUSE("sample_no_alloc: no current device: %s", hipGetErrorString(err));
  if (device < 0 || device >= BT_NO_ALLOC_MAX_DEVICES)
    BT_REFUSE("sample_no_alloc: device %d is beyond the %d this library keeps an address for", device, BT_NO_ALLOC_MAX_DEVICES);
  std::lock_guard<std::mutex> guard(scratch_lock);
  if (scratch_address[device] == nullptr) {
    void* found = nullptr;
    err = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
    if (err != hipSuccess || found == nullptr) {
      bt_set_error("sample_no_alloc: the scratch array has no address on device %d: %s", device, hipGetErrorString(err));
      return BT_HIP_ERROR;
    }
    scratch_address[device] = found;
  }
  *address = scratch_address[device];
  return BT_OK;
}

BT_EXPORT int64_t bt_sample_no_alloc_capacity(void) { return BT_NO_ALLOC_SCRATCH_BYTES / (int64_t)sizeof(SamplePartial); }

BT_EXPORT int bt_sample_no_alloc(void* stream, const float* logits, int64_t ld, int rows, int vocab, int sample,
                                 float temperature, uint64_t seed, uint64_t first_draw, const int* draw_rows,
                                 int* ids, float* logp) {
  if (rows <= 0) return BT_OK;
  if (vocab <= 0) BT_REFUSE("sample_no_alloc: vocabulary %d must be positive", vocab);
  if (sample && !(temperature > 0.f)) BT_REFUSE("sample_no_alloc: temperature %g must be positive", (double)temperature);
  if (logits == nullptr || ids == nullptr || logp == nullptr) BT_REFUSE("sample_no_alloc: missing operand");
  const int64_t records = (int64_t)rows * sample_chunks(vocab);
  if (records > bt_sample_no_alloc_capacity())
    BT_REFUSE("sample_no_alloc: %d rows of %d logits need %lld partial results, the fixed scratch array holds %lld "
              "(use bt_sample with a workspace of bt_sample_workspace_bytes)",
              rows, vocab, (long long)records, (long long)bt_sample_no_alloc_capacity());
  void* partials = nullptr;
  int rc = scratch_on_current_device(&partials);
  if (rc) return rc;
  return launch_sample(stream, logits, ld, rows, vocab, sample, temperature, seed, first_draw, draw_rows, ids, logp,
                       partials);
}

static int launch_sample(void* stream, const float* logits, int64_t ld, int rows, int vocab, int sample,
                         float temperature, uint64_t seed, uint64_t first_draw, const int* draw_rows,
                         int* ids, float* logp, void* workspace) {
  const int chunks = sample_chunks(vocab);
  const int chunk_len = (vocab + chunks - 1) / chunks;
  // the logits are divided by the temperature only when sampling
  const float divisor = sample ? temperature : 1.0f;
  SamplePartial* partials = static_cast<SamplePartial*>(workspace);
  hipLaunchKernelGGL(sample_chunks_kernel, dim3(chunks, rows), dim3(SAMPLE_THREADS), 0, (hipStream_t)stream,
                     logits, ld, vocab, chunk_len, divisor, partials);
  hipLaunchKernelGGL(sample_select_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, (hipStream_t)stream, logits, ld,
                     vocab, chunk_len, chunks, sample, divisor, seed, first_draw, draw_rows, partials, ids, logp);
  return bt_check_launch("sample");
}

// ---------------------------------------------------------------------------------------------
// Selection with processing of the logits (src/generation.rs:18-44), for requests that ask for more
// than plain greedy or temperature sampling.  One work-group of 1,024 threads holds a whole row in
// registers (thread t owns the indices t, t + 1024, ...), so the row is read once however many
// steps follow:
//   1. z += bias                                          (dense vector, zeros where none is set)
//   2. repetition: seen anywhere ? (z < 0 ? z r : z / r)  then  z -= clamp(f c) + p [c > 0]
//   3. sampling only: z /= T;   4. z = min(z, FLT_MAX) where 1-3 can overflow
//   5. banned tokens (n-gram followers, end-of-sequence before min_new_tokens) become -inf
//   6. sampling only: top-k (scores >= the k-th greatest; ties survive), top-p (ranked by score,
//      an item survives when the mass before it is below p; items tied with the last survivor
//      survive too), min-p (p_i >= min_p max p)
//   7. greedy: lowest index of the maximum; sampling: #{k : c_k < u c_last}, c the running sum of
//      the surviving exp(z - max) in index order; log-probability under the processed distribution
// Thresholds are found by bisection on the bits of the scores (32 counting passes over registers);
// nothing is sorted.
// ---------------------------------------------------------------------------------------------
struct ProcessArgs {
  const float* logits;
  int64_t ld;
  int vocab;
  const float* bias;          // [vocab] or null
  const int* counts_all;      // [batch rows][vocab]: occurrences in prompt and output, or null
  const int* counts_add;      // [batch rows][vocab]: what the additive penalties count, or null
  int64_t counts_ld;
  const int* batch_rows;      // [rows]: number of the row in the batch as it started; null = the row itself
  const int* ban_ids;         // banned tokens of row r: ban_ids[ban_offsets[r] .. ban_offsets[r + 1]); null = none
  const int* ban_offsets;
  float repetition, presence, frequency;
  int sample;
  float temperature;
  int clamp;
  int top_k;                  // 0 = off
  float top_p;                // >= 1 = off
  float min_p;                // <= 0 = off
  uint64_t seed, first_draw;
  int* ids;
  float* logp;
};

#define SELECT_THREADS 1024
#define SELECT_WAVES (SELECT_THREADS / 64)

__device__ __forceinline__ unsigned int ordered_key(float f) {   // larger float <=> larger key
  unsigned int b = __float_as_uint(f);
  return b ^ ((b >> 31) ? 0xFFFFFFFFu : 0x80000000u);
}

template <int PER>
__global__ void __launch_bounds__(SELECT_THREADS)
select_processed_kernel(ProcessArgs a) {
  __shared__ unsigned int ban_bits[2048];                 // one bit per token up to 65,536
  __shared__ float wave_f[SELECT_WAVES];
  __shared__ int wave_i[SELECT_WAVES];
  __shared__ float round_part[SELECT_WAVES][PER];
  __shared__ float round_sum[PER];
  __shared__ float shared_f[2];
  __shared__ int shared_i[2];
  const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int brow = a.batch_rows ? a.batch_rows[row] : row;
  const int vocab = a.vocab;

  auto block_sum_f = [&](float v) {
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) wave_f[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < SELECT_WAVES; ++w) total += wave_f[w];
    return total;
  };
  auto block_sum_i = [&](int v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    __syncthreads();
    if (lane == 0) wave_i[wave] = v;
    __syncthreads();
    int total = 0;
    for (int w = 0; w < SELECT_WAVES; ++w) total += wave_i[w];
    return total;
  };
  auto block_max_f = [&](float v) {
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) wave_f[wave] = v;
    __syncthreads();
    float top = wave_f[0];
    for (int w = 1; w < SELECT_WAVES; ++w) top = fmaxf(top, wave_f[w]);
    return top;
  };

  for (int i = tid; i < 2048; i += SELECT_THREADS) ban_bits[i] = 0u;
  __syncthreads();
  if (a.ban_ids != nullptr)
    for (int j = a.ban_offsets[row] + tid; j < a.ban_offsets[row + 1]; j += SELECT_THREADS)
      atomicOr(&ban_bits[a.ban_ids[j] >> 5], 1u << (a.ban_ids[j] & 31));
  __syncthreads();

  // steps 1 to 5; slots beyond the vocabulary hold -inf like banned tokens
  const float* zrow = a.logits + (int64_t)row * a.ld;
  float z[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int k = tid + i * SELECT_THREADS;
    float v = -INFINITY;
    if (k < vocab) {
      v = zrow[k];
      if (a.bias != nullptr) v += a.bias[k];
      if (a.counts_all != nullptr && a.repetition != 1.0f && a.counts_all[(int64_t)brow * a.counts_ld + k] > 0)
        v = v < 0.f ? v * a.repetition : v / a.repetition;
      if (a.counts_add != nullptr) {
        const int c = a.counts_add[(int64_t)brow * a.counts_ld + k];
        if (a.frequency != 0.f) v -= fminf(fmaxf(a.frequency * (float)c, -FLT_MAX), FLT_MAX);
        if (a.presence != 0.f && c > 0) v -= a.presence;
      }
      if (a.sample) v /= a.temperature;
      if (a.clamp) v = fminf(v, FLT_MAX);
      if (ban_bits[k >> 5] & (1u << (k & 31))) v = -INFINITY;
    }
    z[i] = v;
  }

  // the maximum and its lowest index
  float top = -INFINITY;
  int arg = 0x7fffffff;
#pragma unroll
  for (int i = 0; i < PER; ++i)
    if (z[i] > top) { top = z[i]; arg = tid + i * SELECT_THREADS; }   // rising indices: `>` keeps the lowest
  for (int o = 32; o > 0; o >>= 1) {
    float ov = __shfl_xor(top, o, 64);
    int oa = __shfl_xor(arg, o, 64);
    if (ov > top || (ov == top && oa < arg)) { top = ov; arg = oa; }
  }
  __syncthreads();
  if (lane == 0) { wave_f[wave] = top; wave_i[wave] = arg; }
  __syncthreads();
  top = wave_f[0]; arg = wave_i[0];
  for (int w = 1; w < SELECT_WAVES; ++w)
    if (wave_f[w] > top || (wave_f[w] == top && wave_i[w] < arg)) { top = wave_f[w]; arg = wave_i[w]; }
  if (top == -INFINITY) {            // every token is excluded: nothing can be chosen
    if (tid == 0) { a.ids[row] = 0; a.logp[row] = -INFINITY; }
    return;
  }

  // step 6a: the k-th greatest score, bit by bit: the largest T that at least k scores reach
  if (a.sample && a.top_k > 0 && a.top_k < vocab) {
    unsigned int threshold = 0u;
    for (int bit = 31; bit >= 0; --bit) {
      const unsigned int candidate = threshold | (1u << bit);
      int mine = 0;
#pragma unroll
      for (int i = 0; i < PER; ++i) mine += ordered_key(z[i]) >= candidate ? 1 : 0;
      if (block_sum_i(mine) >= a.top_k) threshold = candidate;
    }
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if (ordered_key(z[i]) < threshold) z[i] = -INFINITY;
  }

  // from here on a slot holds e = exp(z - max): 1 for the maximum, 0 for what is excluded.  The
  // order of e is the order of z (scores that round to one e count as tied and survive together),
  // and min-p is simply e >= min_p.
#pragma unroll
  for (int i = 0; i < PER; ++i) z[i] = expf(z[i] - top);
  if (a.sample && a.top_p < 1.0f) {
    float mine = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i) mine += z[i];
    const float target = a.top_p * block_sum_f(mine);
    // the smallest T whose mass strictly above it is below the target; the item at T survives
    unsigned int threshold = 0xFFFFFFFFu;
    for (int bit = 31; bit >= 0; --bit) {
      const unsigned int candidate = threshold & ~(1u << bit);
      float above = 0.f;
#pragma unroll
      for (int i = 0; i < PER; ++i) above += __float_as_uint(z[i]) > candidate ? z[i] : 0.f;   // e >= 0: its bits order it
      if (block_sum_f(above) < target) threshold = candidate;
    }
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if (__float_as_uint(z[i]) < threshold) z[i] = 0.f;
  }
  if (a.sample && a.min_p > 0.f) {
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if (z[i] < a.min_p) z[i] = 0.f;
  }

  // sums of each round of 1,024 consecutive indices, then their total in index order
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    float v = wave_sum(z[i]);
    if (lane == 0) round_part[wave][i] = v;
  }
  __syncthreads();
  if (tid < PER) {
    float v = 0.f;
    for (int w = 0; w < SELECT_WAVES; ++w) v += round_part[w][tid];
    round_sum[tid] = v;
  }
  __syncthreads();
  float total = 0.f;
  for (int i = 0; i < PER; ++i) total += round_sum[i];

  if (!a.sample) {
    if (tid == 0) {
      a.ids[row] = arg;
      a.logp[row] = -logf(total);          // the chosen token is the maximum: e = 1
    }
    return;
  }
  const float u = (float)(((double)(splitmix64(a.seed, a.first_draw + (uint64_t)brow) >> 41) + 0.5) / 8388608.0);
  const float limit = u * total;
  // the round in which the running sum reaches the limit, and the sum before it
  float before = 0.f;
  int owner = PER - 1;
  for (int i = 0; i < PER - 1; ++i) {
    float with = before + round_sum[i];
    if (with >= limit) { owner = i; break; }
    before = with;
  }
  float mine = 0.f;
#pragma unroll
  for (int i = 0; i < PER; ++i)
    if (i == owner) mine = z[i];
  // running sum over the threads of that round: inside the wave, then over the waves before
  float scan = mine;
  for (int o = 1; o < 64; o <<= 1) {
    float up = __shfl_up(scan, o, 64);
    if (lane >= o) scan += up;
  }
  __syncthreads();
  if (lane == 63) wave_f[wave] = scan;
  __syncthreads();
  float lead = before;
  for (int w = 0; w < wave; ++w) lead += wave_f[w];
  const int below = (lead + scan < limit) ? 1 : 0;
  const int count = block_sum_i(below);
  int chosen = owner * SELECT_THREADS + count;
  if (chosen >= vocab) chosen = vocab - 1;
  // the chosen token's e, from the thread that holds it
  if (tid == 0) shared_f[0] = 0.f;
  __syncthreads();
  if ((chosen & (SELECT_THREADS - 1)) == tid) {
    float e = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if (i == (chosen >> 10)) e = z[i];
    shared_f[0] = e;
  }
  __syncthreads();
  if (tid == 0) {
    a.ids[row] = chosen;
    a.logp[row] = logf(shared_f[0]) - logf(total);
  }
  (void)shared_i;
}

// Steps 1 to 5 alone, element by element, into `out`: many work-groups per row, because one
// compute unit pulls a row of logits and its two rows of counts (600 KB at a vocabulary of 50,257)
// no faster than in 25 us.  What follows then reads processed scores only: plain greedy selection
// or sampling (bt_sample, with temperature 1: it is already applied), or the truncating kernel
// above with its own processing switched off.
#define PROCESS_CHUNK 2048
__global__ void __launch_bounds__(256)
process_scores_kernel(ProcessArgs a, float* __restrict__ out, int64_t ldo) {
  const int row = blockIdx.y, lo = blockIdx.x * PROCESS_CHUNK;
  const int hi = lo + PROCESS_CHUNK < a.vocab ? lo + PROCESS_CHUNK : a.vocab;
  const int brow = a.batch_rows ? a.batch_rows[row] : row;
  const float* zrow = a.logits + (int64_t)row * a.ld;
  float* orow = out + (int64_t)row * ldo;
  for (int k = lo + threadIdx.x; k < hi; k += 256) {
    float v = zrow[k];
    if (a.bias != nullptr) v += a.bias[k];
    if (a.counts_all != nullptr && a.repetition != 1.0f && a.counts_all[(int64_t)brow * a.counts_ld + k] > 0)
      v = v < 0.f ? v * a.repetition : v / a.repetition;
    if (a.counts_add != nullptr) {
      const int c = a.counts_add[(int64_t)brow * a.counts_ld + k];
      if (a.frequency != 0.f) v -= fminf(fmaxf(a.frequency * (float)c, -FLT_MAX), FLT_MAX);
      if (a.presence != 0.f && c > 0) v -= a.presence;
    }
    if (a.sample) v /= a.temperature;
    if (a.clamp) v = fminf(v, FLT_MAX);
    orow[k] = v;
  }
  if (a.ban_ids == nullptr) return;
  __syncthreads();                         // this work-group's own scores are written: now its banned ones
  for (int j = a.ban_offsets[row] + threadIdx.x; j < a.ban_offsets[row + 1]; j += 256) {
    const int k = a.ban_ids[j];
    if (k >= lo && k < hi) orow[k] = -INFINITY;
  }
}

BT_EXPORT int bt_process_scores(void* stream, const ProcessArgs* args, int rows, float* out, int64_t ldo) {
  if (rows <= 0) return BT_OK;
  const ProcessArgs& a = *args;
  if (a.vocab <= 0 || a.logits == nullptr || out == nullptr || ldo < a.vocab) BT_REFUSE("process_scores: missing operand");
  if (a.sample && !(a.temperature > 0.f)) BT_REFUSE("process_scores: temperature %g must be positive", (double)a.temperature);
  if (!(a.repetition > 0.f)) BT_REFUSE("process_scores: repetition penalty %g must be positive", (double)a.repetition);
  if ((a.ban_ids == nullptr) != (a.ban_offsets == nullptr)) BT_REFUSE("process_scores: banned tokens need their offsets");
  dim3 grid((a.vocab + PROCESS_CHUNK - 1) / PROCESS_CHUNK, rows);
  hipLaunchKernelGGL(process_scores_kernel, grid, dim3(256), 0, (hipStream_t)stream, a, out, ldo);
  return bt_check_launch("process_scores");
}

BT_EXPORT int bt_select_processed(void* stream, const ProcessArgs* args, int rows) {
  if (rows <= 0) return BT_OK;
  const ProcessArgs& a = *args;
  if (a.vocab <= 0 || a.vocab > 65536) BT_REFUSE("select_processed: vocabulary %d outside 1..65536 (a row is held in one work-group's registers)", a.vocab);
  if (a.logits == nullptr || a.ids == nullptr || a.logp == nullptr) BT_REFUSE("select_processed: missing operand");
  if (a.sample && !(a.temperature > 0.f)) BT_REFUSE("select_processed: temperature %g must be positive", (double)a.temperature);
  if (!(a.repetition > 0.f)) BT_REFUSE("select_processed: repetition penalty %g must be positive", (double)a.repetition);
  if ((a.ban_ids == nullptr) != (a.ban_offsets == nullptr)) BT_REFUSE("select_processed: banned tokens need their offsets");
  if (a.top_k < 0 || !(a.top_p > 0.f) || a.min_p > 1.f) BT_REFUSE("select_processed: top_k %d, top_p %g or min_p %g out of range", a.top_k, (double)a.top_p, (double)a.min_p);
  hipStream_t s = (hipStream_t)stream;
  if (a.vocab <= 16 * SELECT_THREADS)
    hipLaunchKernelGGL(select_processed_kernel<16>, dim3(rows), dim3(SELECT_THREADS), 0, s, a);
  else
    hipLaunchKernelGGL(select_processed_kernel<64>, dim3(rows), dim3(SELECT_THREADS), 0, s, a);
  return bt_check_launch("select_processed");
}

// counts[rows[i]][ids[i]] += 1 for i < n: the occurrence counts the penalties read
__global__ void count_tokens_kernel(int* __restrict__ counts, int64_t ld, const int* __restrict__ rows,
                                    const int* __restrict__ ids, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) atomicAdd(&counts[(int64_t)rows[i] * ld + ids[i]], 1);
}

BT_EXPORT int bt_count_tokens(void* stream, int* counts, int64_t ld, const int* rows, const int* ids, int n) {
  if (n <= 0) return BT_OK;
  hipLaunchKernelGGL(count_tokens_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream, counts, ld, rows, ids, n);
  return bt_check_launch("count_tokens");
}

// ---------------------------------------------------------------------------------------------
// The same entry points with their arguments as one structure (calls.h), for launch lists.
// ---------------------------------------------------------------------------------------------
BT_EXPORT int bt_embed_call(void* stream, const EmbedCall* c) {
  return bt_embed(stream, c->dtype, c->ids, c->pos, c->table, c->positions, c->out, c->tokens, c->width);
}
BT_EXPORT int bt_add_norm_call(void* stream, const AddNormCall* c) {
  return bt_add_norm(stream, c->out_dtype, c->x, c->delta, c->n_delta, c->delta_stride, c->bias, c->gamma, c->beta, c->eps,
                     c->kind, c->out, c->rows, c->n_rows, c->width, c->write_back, c->out_rows);
}
BT_EXPORT int bt_gemm_plain_call(void* stream, const GemmCall* c) {
  if (c->splits != 1 || c->has_norm || c->a_rows || c->packed_columns)
    BT_REFUSE("gemm_plain: no split of K, no rows to normalise, no chunk-major rows and no packed weights");
  return bt_gemm_plain(stream, c->dtype, c->A, c->lda, c->W, c->M, c->N, c->K, &c->epi);
}
BT_EXPORT int bt_attention_plain_call(void* stream, const AttentionCall* c) {
  return bt_attention_plain(stream, c->dtype, &c->args);
}
BT_EXPORT int bt_kv_copy_call(void* stream, const KvCopyCall* c) {
  return bt_kv_copy(stream, c->dtype, c->k_rows, c->v_rows, c->ld, c->tok_seq, c->tok_pos, &c->kv, c->tokens, c->to_cache);
}
