// An entry point for callers that cannot allocate.
//
// bt_sample_no_alloc has no counterpart in the reference.  It is for callers that must not call
// hipMalloc or any routine that might: code under HIP graph capture, tight serving loops,
// harnesses that forbid allocation.  It is bt_sample (greedy or temperature selection of one token
// per row of float32 logits, same kernels, same results bit for bit) without the workspace
// argument: the partial results that the first kernel leaves for the second (one 16-byte record per
// row and chunk of the vocabulary) live in a fixed array in device memory that belongs to the
// library, BT_NO_ALLOC_SCRATCH_BYTES on every GPU the library runs on, held until the process ends.
//
// Limits: rows * chunks(vocab) records must fit the array, chunks(vocab) being
// max(16, ceil(vocab / 4096)): with 64 KiB that is 4,096 records, for instance 256 rows of a
// vocabulary of up to 65,536 tokens, or 64 rows of up to 262,144.  Larger calls are refused with a
// message (BT_REFUSED, bt_last_error()); nothing is launched then.
//
// Every call on a GPU uses that GPU's one array and nothing waits for the call before: two calls
// whose kernels can overlap on one GPU (different streams, different threads) race, and the
// caller must order them.  Calls on one stream are ordered by the stream.  The array keeps the last
// call's records; nothing in it has to start at zero, because the first kernel writes every
// record that the second reads.
//
// The call allocates nothing, frees nothing and synchronises nothing.  The first call on each
// device looks the array's address on that device up once (hipGetSymbolAddress) and keeps it.
#pragma once

#include <stdint.h>

#define BT_NO_ALLOC_SCRATCH_BYTES (64 * 1024)

extern "C" __attribute__((visibility("default")))
int bt_sample_no_alloc(void* stream, const float* logits, int64_t ld, int rows, int vocab, int sample,
                       float temperature, uint64_t seed, uint64_t first_draw, const int* draw_rows,
                       int* ids, float* logp);

// The most records (rows * chunks) a call may need; what bt_sample_no_alloc compares with.
extern "C" __attribute__((visibility("default")))
int64_t bt_sample_no_alloc_capacity(void);
