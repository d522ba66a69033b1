// The host loop of a step: a launch list, walked in C++.
//
// A step of the model is a few hundred kernel launches whose arguments depend only on the step's
// shape (tokens, sequences, wanted rows) and on addresses that do not move (weights, workspaces,
// the step's integer tables): the parts of the model emit them ONCE per shape as a list of
// (entry point, argument structure) pairs, and every step of that shape is then one call of
// bt_program_run, which walks the list and calls each kernel module's entry point.  Python is left
// out of the loop: a launch costs what hipLaunchKernel costs.
//
// Every entry point has the signature `int (void* stream, const void* call)` (calls.h) and returns
// 0 when its kernels were launched.  The walk stops at the first entry that returns something
// else; its index and code go back to the caller, who asks that entry's module for the message.
#include <stdint.h>

extern "C" {

typedef int (*bt_call_fn)(void* stream, const void* call);

struct LaunchEntry {
  bt_call_fn call;
  const void* args;
};

// Runs entries[0 .. count) on `stream`.  Returns 0, or the code of the entry that refused, whose
// index is written to *failed (entries before it have been launched, entries after it not).
__attribute__((visibility("default")))
int bt_program_run(void* stream, const LaunchEntry* entries, int count, int* failed) {
  for (int i = 0; i < count; ++i) {
    int rc = entries[i].call(stream, entries[i].args);
    if (rc != 0) {
      if (failed) *failed = i;
      return rc;
    }
  }
  if (failed) *failed = -1;
  return 0;
}

}  // extern "C"
