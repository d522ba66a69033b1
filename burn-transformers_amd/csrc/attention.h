// Arguments of the attention kernels (plain and MFMA); mirrored by a ctypes.Structure.
#pragma once

#include "common.h"

struct AttnArgs {
  const void* q;        // [tokens][ldq]; head j at columns j * head_dim
  int64_t ldq;
  void* out;            // [tokens][ldo]
  int64_t ldo;
  const int* tok_seq;   // [tokens]
  const int* tok_pos;   // [tokens]
  const int* seq_off;   // [n_seqs + 1] first token of each sequence in the step
  const int* seq_start; // [n_seqs] position of that first token
  KvView kv;
  int q_heads;
  int n_tokens;
  int n_seqs;
  int max_count;        // most tokens any sequence brings in this step
  int window;           // 0 = all earlier keys
  float scale;
  // With splits > 1 the keys are cut into that many runs, each run is a work-group of its own that
  // leaves (output row, maximum, sum) in `partial` [rows][q_heads][splits][head_dim + 2], and a
  // second kernel joins them into `out`.  Decode: the runs of every sequence's keys, a row is a
  // sequence.  Prompts (bfloat16, heads of 64, no window): the runs of every query tile's keys, a
  // row is a token of the step.
  int splits;
  float* partial;
  // Decode (bfloat16 MFMA kernels) only: 0, or `out` is chunk-major with that many rows
  // (activation_offset in common.h); ldo is then not used.
  int out_rows;
};
