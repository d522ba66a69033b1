// What a matrix product does with its accumulators.  Every GEMM kernel hands groups of four
// consecutive output columns of one row to `epilogue4`, which adds the bias and then either
// stores, applies the activation, writes 32-bit partial sums, or scatters a fused
// query/key/value projection into the query buffer and the paged cache.
#pragma once

#include "common.h"

enum EpilogueMode {
  EPI_STORE = 0,  // out[m][n] = acc + bias                      (element type T)
  EPI_ACT = 1,    // out[m][n] = act(acc + bias)                 (element type T)
  EPI_F32 = 2,    // out[split][m][n] = acc (+ bias in split 0)  (float; the consumer sums the splits)
  EPI_QKV = 3,    // columns [0,n_q) -> out, [n_q,n_q+n_kv) -> keys, the next n_kv -> values
  EPI_RESIDUAL = 4,  // out[m][n] += acc + bias                  (float: the residual stream itself)
};

enum Activation {
  ACT_GELU_TANH = 0,
  ACT_GELU_ERF = 1,
};

// Mirrored field by field by a ctypes.Structure on the Python side.
struct Epilogue {
  int mode;
  int act;
  const float* bias;     // [N] or null
  void* out;
  int64_t ldo;           // row pitch of out, in elements
  int64_t split_stride;  // elements between the partial sums of two splits (EPI_F32)
  int n_q;
  int n_kv;
  const int* tok_seq;    // [M] index of the token's sequence in the step
  const int* tok_pos;    // [M] position of the token in its sequence
  KvView kv;
  int out_rows;          // EPI_STORE, EPI_ACT: 0, or `out` is chunk-major with that many rows (activation_offset)
};

// 32-bit activations.  The float32 path (T = float) uses the library's tanhf / erff; the
// bfloat16 path writes the tanh form as x / (1 + exp(-2u)), which is the same function
// (0.5 (1 + tanh u) = 1 / (1 + exp(-2u))) evaluated with the hardware exponential: its error
// (a few ulp of float32) is far below the rounding of the bfloat16 result, and it is a handful of
// instructions instead of some forty for each of the millions of elements a prefill produces.
template <typename T>
__device__ __forceinline__ float activate(float x, int act) {
  if (act == ACT_GELU_TANH) {
    // 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))
    float inner = 0.7978845608028654f * (x + 0.044715f * x * x * x);
    if (sizeof(T) == 2) return x / (1.0f + __expf(-2.0f * inner));
    return 0.5f * x * (1.0f + tanhf(inner));
  }
  // x (1 + erf(x / sqrt 2)) / 2
  return 0.5f * x * (1.0f + erff(x * 0.7071067811865476f));
}

template <typename T>
__device__ __forceinline__ void store4(T* dst, const float* v, int count, bool aligned);

template <>
__device__ __forceinline__ void store4<float>(float* dst, const float* v, int count, bool aligned) {
  if (count == 4 && aligned) {
    *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i < count) dst[i] = v[i];
  }
}
template <>
__device__ __forceinline__ void store4<bf16_t>(bf16_t* dst, const float* v, int count, bool aligned) {
  if (count == 4 && aligned) {
    bf16x4 packed = {(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
    *reinterpret_cast<bf16x4*>(dst) = packed;
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i < count) dst[i] = (bf16_t)v[i];
  }
}

// What an epilogue needs from memory besides the accumulators, fetched at the START of a kernel
// so that no load is left on the critical path after the last multiply: the bias (plus the old
// value of the residual stream in EPI_RESIDUAL) and, for the key/value scatter, where the row's
// token lives in the paged cache.
struct EpiloguePrefetch {
  float add[4];
  int64_t kv_base;   // start of the (block, head) plane of the token; valid for key/value columns
  int pos;
};

// A valid address for the loads of an epilogue mode that is not in use: the prefetch below has
// no branches, so every load in it is always issued (and its result discarded where unused).
__device__ int bt_dummy_words[4] = {0, 0, 0, 0};

__device__ __forceinline__ EpiloguePrefetch epilogue_prefetch(const Epilogue& e, int M, int N, int m, int n0,
                                                              int split) {
  // Branch-free on purpose: with no control flow the compiler issues these loads among the
  // caller's own and waits for none of them before it has to.
  EpiloguePrefetch p;
  const int mm = m < M ? m : M - 1;
  const bool with_bias = e.bias != nullptr && split == 0;
  const bool residual = e.mode == EPI_RESIDUAL;
  const bool scatter = e.mode == EPI_QKV;
  const float* dummy = reinterpret_cast<const float*>(bt_dummy_words);
  const float* bias = with_bias ? e.bias : dummy;
  const float* x = residual ? static_cast<const float*>(e.out) + (int64_t)mm * e.ldo : dummy;
  const int* tok_seq = scatter ? e.tok_seq : bt_dummy_words;
  const int* tok_pos = scatter ? e.tok_pos : bt_dummy_words;
  int seq = tok_seq[scatter ? mm : 0];
  int pos = tok_pos[scatter ? mm : 0];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int nn = n0 + i < N ? n0 + i : N - 1;
    float b = bias[with_bias ? nn : 0];
    float xv = x[residual ? nn : 0];
    p.add[i] = (with_bias ? b : 0.f) + (residual ? xv : 0.f);
  }
  // key/value columns: where the token's position lives in the paged cache
  int c = n0 - e.n_q;
  if (c >= e.n_kv) c -= e.n_kv;
  const bool kv_column = scatter && n0 >= e.n_q && n0 < N;
  const int head = kv_column ? c / e.kv.head_dim : 0;
  const int* blocks = kv_column ? e.kv.blocks : bt_dummy_words;
  int block = blocks[kv_column ? (int64_t)seq * e.kv.max_blocks + pos / BT_KV_BLOCK : 0];
  p.kv_base = kv_plane(e.kv, block, head);
  p.pos = pos;
  return p;
}

// The epilogue with everything but the accumulators already in registers.
template <typename T>
__device__ __forceinline__ void epilogue4_prefetched(const Epilogue& e, int N, int m, int n0, const float* acc,
                                                     int split, const EpiloguePrefetch& p) {
  int count = N - n0 < 4 ? N - n0 : 4;
  if (count <= 0) return;
  float v[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = acc[i] + p.add[i];
  bool aligned = (e.ldo & 3) == 0;
  if (e.mode == EPI_STORE) {
    if (e.out_rows == 0) store4<T>(static_cast<T*>(e.out) + (int64_t)m * e.ldo + n0, v, count, aligned);     // (one branch for all threads)
    else store4<T>(static_cast<T*>(e.out) + activation_offset<T>(e.out_rows, e.ldo, m, n0), v, count, true);
  } else if (e.mode == EPI_ACT) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = activate<T>(v[i], e.act);
    if (e.out_rows == 0) store4<T>(static_cast<T*>(e.out) + (int64_t)m * e.ldo + n0, v, count, aligned);     // (one branch for all threads)
    else store4<T>(static_cast<T*>(e.out) + activation_offset<T>(e.out_rows, e.ldo, m, n0), v, count, true);
  } else if (e.mode == EPI_F32) {
    store4<float>(static_cast<float*>(e.out) + (int64_t)split * e.split_stride + (int64_t)m * e.ldo + n0,
                  v, count, aligned);
  } else if (e.mode == EPI_RESIDUAL) {
    store4<float>(static_cast<float*>(e.out) + (int64_t)m * e.ldo + n0, v, count, aligned);
  } else {
    if (n0 < e.n_q) {
      store4<T>(static_cast<T*>(e.out) + (int64_t)m * e.ldo + n0, v, count, aligned);
    } else {
      int c = n0 - e.n_q;
      bool is_value = c >= e.n_kv;
      if (is_value) c -= e.n_kv;
      int channel = c % e.kv.head_dim;
      if (!is_value) {
        store4<T>(static_cast<T*>(e.kv.keys) + p.kv_base + key_offset(e.kv.head_dim, p.pos, channel), v, count, true);
      } else {
        T* dst = static_cast<T*>(e.kv.values) + p.kv_base + value_offset(e.kv.head_dim, p.pos, channel);
#pragma unroll
        for (int i = 0; i < 4; ++i)     // consecutive channels of one position lie four elements apart
          if (i < count) dst[4 * i] = from_float<T>(v[i]);
      }
    }
  }
}

// Row m, columns n0 .. n0+3 (n0 a multiple of four), of an [M, N] product; `split` is the
// index of the K slice that produced `acc`.
template <typename T>
__device__ __forceinline__ void epilogue4(const Epilogue& e, int N, int m, int n0, const float* acc,
                                          int split) {
  int count = N - n0 < 4 ? N - n0 : 4;
  if (count <= 0) return;
  float v[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float b = (e.bias != nullptr && split == 0 && i < count) ? e.bias[n0 + i] : 0.f;
    v[i] = acc[i] + b;
  }
  bool aligned = (e.ldo & 3) == 0;
  if (e.mode == EPI_STORE) {
    if (e.out_rows == 0) store4<T>(static_cast<T*>(e.out) + (int64_t)m * e.ldo + n0, v, count, aligned);     // (one branch for all threads)
    else store4<T>(static_cast<T*>(e.out) + activation_offset<T>(e.out_rows, e.ldo, m, n0), v, count, true);
  } else if (e.mode == EPI_ACT) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = activate<T>(v[i], e.act);
    if (e.out_rows == 0) store4<T>(static_cast<T*>(e.out) + (int64_t)m * e.ldo + n0, v, count, aligned);     // (one branch for all threads)
    else store4<T>(static_cast<T*>(e.out) + activation_offset<T>(e.out_rows, e.ldo, m, n0), v, count, true);
  } else if (e.mode == EPI_F32) {
    store4<float>(static_cast<float*>(e.out) + (int64_t)split * e.split_stride + (int64_t)m * e.ldo + n0,
                  v, count, aligned);
  } else if (e.mode == EPI_RESIDUAL) {
    float* x = static_cast<float*>(e.out) + (int64_t)m * e.ldo + n0;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i < count) v[i] += x[i];
    store4<float>(x, v, count, aligned);
#ifdef BT_EPILOGUE_ANY_HEAD_SIZE
  } else if ((e.kv.head_dim & 3) != 0) {
    // EPI_QKV with a head size that four columns do not divide: every column finds its own place
    // among the queries, keys and values.  Compiled into the plain product only (it defines
    // BT_EPILOGUE_ANY_HEAD_SIZE): the MFMA kernels refuse such head sizes, and in them this path
    // would only cost registers (their tiles of 128 x 128 spilled with it, at a third of the speed).
    int seq = e.tok_seq[m], pos = e.tok_pos[m];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (i >= count) break;
      int n = n0 + i;
      if (n < e.n_q) {
        static_cast<T*>(e.out)[(int64_t)m * e.ldo + n] = from_float<T>(v[i]);
        continue;
      }
      int c = n - e.n_q;
      bool is_value = c >= e.n_kv;
      if (is_value) c -= e.n_kv;
      int head = c / e.kv.head_dim, channel = c % e.kv.head_dim;
      int64_t base = kv_block_base(e.kv, seq, pos, head);
      if (!is_value) static_cast<T*>(e.kv.keys)[base + key_offset(e.kv.head_dim, pos, channel)] = from_float<T>(v[i]);
      else static_cast<T*>(e.kv.values)[base + value_offset(e.kv.head_dim, pos, channel)] = from_float<T>(v[i]);
    }
#endif
  } else {  // EPI_QKV: head_dim (and with it n_q and n_kv) is a multiple of four, so the four columns share a head
    if (n0 < e.n_q) {
      store4<T>(static_cast<T*>(e.out) + (int64_t)m * e.ldo + n0, v, count, aligned);
    } else {
      int c = n0 - e.n_q;
      bool is_value = c >= e.n_kv;
      if (is_value) c -= e.n_kv;
      int head = c / e.kv.head_dim, channel = c % e.kv.head_dim;
      int seq = e.tok_seq[m], pos = e.tok_pos[m];
      int64_t base = kv_block_base(e.kv, seq, pos, head);
      if (!is_value) {
        store4<T>(static_cast<T*>(e.kv.keys) + base + key_offset(e.kv.head_dim, pos, channel), v, count,
                  true);
      } else {
        T* dst = static_cast<T*>(e.kv.values) + base + value_offset(e.kv.head_dim, pos, channel);
#pragma unroll
        for (int i = 0; i < 4; ++i)     // consecutive channels of one position lie four elements apart
          if (i < count) dst[4 * i] = from_float<T>(v[i]);
      }
    }
  }
}
