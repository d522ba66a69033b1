// A kernel that a toy part of the tests brings along: it turns the channel pairs (i, i + h/2) of
// every head of the first `parts` sections of each row by the angle position * freq[i], in float32,
// in place.  Compiled through the package's build (kernels.build.register_module) and called
// through its launch-list form, like the package's own kernels.
#include <hip/hip_bf16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "host.h"      // the package's error reporting: bt_set_error, bt_check_launch, bt_last_error

struct RotaryTurnCall {
  int dtype;             // 0: float32, 1: bfloat16
  int tokens, parts, heads, head_dim;
  int64_t ld;            // elements from one row to the next
  void* rows;            // [tokens][ld]; section p of a row is columns p * heads * head_dim ...
  const int* positions;  // [tokens]
  const float* freq;     // [head_dim / 2]
};

template <typename T>
__global__ void rotary_turn_kernel(RotaryTurnCall c) {
  const int half = c.head_dim / 2;
  const int64_t index = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = (int64_t)c.tokens * c.parts * c.heads * half;
  if (index >= total) return;
  const int i = (int)(index % half);
  const int head = (int)(index / half % c.heads);
  const int part = (int)(index / half / c.heads % c.parts);
  const int token = (int)(index / half / c.heads / c.parts);
  T* row = (T*)c.rows + token * c.ld + ((int64_t)part * c.heads + head) * c.head_dim;
  const float angle = (float)c.positions[token] * c.freq[i];
  const float cs = cosf(angle), sn = sinf(angle);
  const float first = (float)row[i], second = (float)row[i + half];
  row[i] = (T)(first * cs - second * sn);
  row[i + half] = (T)(second * cs + first * sn);
}

BT_EXPORT int bt_toy_rotary_turn_call(void* stream, const RotaryTurnCall* c) {
  if (c->head_dim <= 0 || c->head_dim % 2 != 0) {
    bt_set_error("toy_rotary_turn: head size %d must be even", c->head_dim);
    return BT_REFUSED;
  }
  if (c->ld < (int64_t)c->parts * c->heads * c->head_dim) {
    bt_set_error("toy_rotary_turn: rows of %lld elements do not hold %d sections of %d heads of %d",
                 (long long)c->ld, c->parts, c->heads, c->head_dim);
    return BT_REFUSED;
  }
  const int64_t total = (int64_t)c->tokens * c->parts * c->heads * (c->head_dim / 2);
  if (total == 0) return BT_OK;
  const int threads = 256;
  const unsigned blocks = (unsigned)((total + threads - 1) / threads);
  if (c->dtype == 0)
    hipLaunchKernelGGL(rotary_turn_kernel<float>, dim3(blocks), dim3(threads), 0, (hipStream_t)stream, *c);
  else
    hipLaunchKernelGGL(rotary_turn_kernel<__hip_bfloat16>, dim3(blocks), dim3(threads), 0, (hipStream_t)stream, *c);
  return bt_check_launch("toy_rotary_turn");
}
