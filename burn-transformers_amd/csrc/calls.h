// One calling convention for every kernel entry point, so that a step can be a LIST of calls.
//
// Each kernel module exports, beside its entry points with spelled-out arguments, a second form
//     int bt_<kernel>_call(void* stream, const <Kernel>Call* call)
// that takes the same arguments as one plain structure.  A launch list (program.cpp) is then an
// array of (function, structure) pairs that one C++ loop walks: the host cost of a step is one
// call from Python plus the launches themselves, instead of an interpreter round trip per kernel.
// The structures are mirrored field by field by ctypes.Structure classes on the Python side.
#pragma once

#include "attention.h"
#include "epilogue.h"

// Rows of the float32 residual stream that the skinny product normalises itself.
struct NormOperand {
  const float* x;        // [M][ldx] float32 rows
  int64_t ldx;
  const float* gamma;    // [K]
  const float* beta;     // [K] or null
  float eps;
  int kind;              // 0: layer norm, 1: RMS norm
};

struct EmbedCall {
  int dtype;
  int tokens;
  int width;
  const int* ids;
  const int* pos;          // or null
  const void* table;
  const void* positions;   // or null
  float* out;
};

struct AddNormCall {
  int out_dtype;
  int n_delta;
  int kind;
  int n_rows;
  int width;
  int write_back;
  int out_rows;
  float eps;
  float* x;
  const float* delta;
  int64_t delta_stride;
  const float* bias;
  const float* gamma;
  const float* beta;
  void* out;
  const int* rows;
};

// A matrix product on any of the product kernels; fields a kernel does not have are ignored by it.
struct GemmCall {
  int dtype;
  int M, N, K;
  int splits;
  int variant;
  int packed_columns;    // skinny: the weights are a packed copy for that many columns per work-group
  int a_rows;            // skinny: A is chunk-major with that many rows
  int has_norm;          // skinny: A is absent and `norm` describes the rows to normalise
  const void* A;
  int64_t lda;
  const void* W;
  Epilogue epi;
  NormOperand norm;
};

struct AttentionCall {
  int dtype;             // plain kernel only; the others are built for one element type
  AttnArgs args;
};

struct KvCopyCall {
  int dtype;
  int tokens;
  int to_cache;
  void* k_rows;
  void* v_rows;
  int64_t ld;
  const int* tok_seq;
  const int* tok_pos;
  KvView kv;
};
