// Shared device helpers for the gfx950 kernels: element types, vector types,
// the paged key/value addressing and wave/block reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define BT_EXPORT extern "C" __attribute__((visibility("default")))

// Error codes returned by every entry point (0 = launched).
#define BT_OK 0
#define BT_REFUSED 1  // the sizes are outside what the kernel takes; see bt_last_error()
#define BT_HIP_ERROR 2

// Tokens per block of the paged key/value storage.  A key tile of 32 never straddles a block.
#define BT_KV_BLOCK 64

typedef __bf16 bf16_t;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

void bt_set_error(const char* fmt, ...);
int bt_check_launch(const char* what);

#define BT_REFUSE(...)            \
  do {                            \
    bt_set_error(__VA_ARGS__);    \
    return BT_REFUSED;            \
  } while (0)

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) { return (float)v; }

template <typename T>
__device__ __forceinline__ T from_float(float v);
template <>
__device__ __forceinline__ float from_float<float>(float v) { return v; }
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float v) { return (bf16_t)v; }  // round to nearest even

// Geometry of one group of layers in the paged key/value storage.  A (block, head) *plane* holds
// the keys (or values) of one head for the 64 positions of one block:
//   keys:   plane = [BT_KV_BLOCK][head_dim]
//   values: plane = [BT_KV_BLOCK / 4][head_dim][4]   (four positions interleaved per channel, so
//           that a lane reads four consecutive positions of one channel at once)
// The plane of (block, head) starts block * block_stride + head * head_stride elements into the
// layer: the storage decides which of the two lies closer together (with the heads outermost, the
// blocks a sequence took one after the other are one contiguous run for each head).
// `blocks` is the table of the step's sequences: blocks[seq * max_blocks + position / BT_KV_BLOCK].
struct KvView {
  void* keys;            // base of the layer
  void* values;          // base of the layer
  const int* blocks;     // [n_seqs][max_blocks]
  int max_blocks;
  int kv_heads;
  int head_dim;
  int64_t block_stride;  // elements from a block's plane to the next block's, same head
  int64_t head_stride;   // elements from a head's plane to the next head's, same block
};

__device__ __forceinline__ int64_t kv_plane(const KvView& kv, int block, int kv_head) {
  return (int64_t)block * kv.block_stride + (int64_t)kv_head * kv.head_stride;
}
__device__ __forceinline__ int64_t kv_block_base(const KvView& kv, int seq, int pos, int kv_head) {
  return kv_plane(kv, kv.blocks[(int64_t)seq * kv.max_blocks + pos / BT_KV_BLOCK], kv_head);
}
// Element offset of key (pos, channel) inside its (block, head) plane.
__device__ __forceinline__ int key_offset(int head_dim, int pos, int channel) {
  return (pos % BT_KV_BLOCK) * head_dim + channel;
}
// Element offset of value (pos, channel) inside its (block, head) plane.
__device__ __forceinline__ int value_offset(int head_dim, int pos, int channel) {
  int p = pos % BT_KV_BLOCK;
  return ((p >> 2) * head_dim + channel) * 4 + (p & 3);
}

// Activations of a step of few rows may be kept "chunk-major": the chunks of 64 bytes of K (32
// bfloat16, 16 float32 columns) one after the other, each holding that chunk of every row,
// [columns / chunk][rows][chunk].  The lanes of an MFMA operand load (16 rows by 64 bytes) then read
// one contiguous KiB, where row-major rows lie a whole row apart: reading 64 rows of 1,600
// columns that way takes a work-group 1 us instead of 5.8.  Element offset of (row, column);
// `rows` = 0 means row-major with the given pitch.
template <typename T>
__host__ __device__ __forceinline__ int64_t activation_offset(int rows, int64_t pitch, int row, int column) {
  constexpr int CHUNK = 64 / (int)sizeof(T);
  return rows > 0 ? ((int64_t)(column / CHUNK) * rows + row) * CHUNK + column % CHUNK : (int64_t)row * pitch + column;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// Block-wide reductions for blocks of up to 1024 threads; `scratch` holds 32 floats of LDS.
// Every thread gets the result.  Safe to call repeatedly with the same scratch.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, waves = (blockDim.x + 63) >> 6;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < waves; ++w) total += scratch[w];
  return total;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
  v = wave_max(v);
  int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, waves = (blockDim.x + 63) >> 6;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float top = scratch[0];
  for (int w = 1; w < waves; ++w) top = fmaxf(top, scratch[w]);
  return top;
}
