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
};

__device__ __forceinline__ float activate(float x, int act) {
  if (act == ACT_GELU_TANH) {
    // 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))
    float inner = 0.7978845608028654f * (x + 0.044715f * x * x * x);
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
    for (int i = 0; i < count; ++i) dst[i] = v[i];
  }
}
template <>
__device__ __forceinline__ void store4<bf16_t>(bf16_t* dst, const float* v, int count, bool aligned) {
  if (count == 4 && aligned) {
    bf16x4 packed = {(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
    *reinterpret_cast<bf16x4*>(dst) = packed;
  } else {
    for (int i = 0; i < count; ++i) dst[i] = (bf16_t)v[i];
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
    store4<T>(static_cast<T*>(e.out) + (int64_t)m * e.ldo + n0, v, count, aligned);
  } else if (e.mode == EPI_ACT) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = activate(v[i], e.act);
    store4<T>(static_cast<T*>(e.out) + (int64_t)m * e.ldo + n0, v, count, aligned);
  } else if (e.mode == EPI_F32) {
    store4<float>(static_cast<float*>(e.out) + (int64_t)split * e.split_stride + (int64_t)m * e.ldo + n0,
                  v, count, aligned);
  } else {  // EPI_QKV: n_q, n_kv and head_dim are multiples of 16, so the four columns share a head
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
        T* dst = static_cast<T*>(e.kv.values) + base;
        for (int i = 0; i < count; ++i) dst[value_offset(e.kv.head_dim, pos, channel + i)] = from_float<T>(v[i]);
      }
    }
  }
}
