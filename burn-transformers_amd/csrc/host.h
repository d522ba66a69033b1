// Host-side error reporting shared by every kernel module (one copy per shared library).
#pragma once

#include <stdarg.h>
#include <stdio.h>

#include "common.h"

static thread_local char bt_error_text[512] = "";

void bt_set_error(const char* fmt, ...) {
  va_list args;
  va_start(args, fmt);
  vsnprintf(bt_error_text, sizeof(bt_error_text), fmt, args);
  va_end(args);
}

int bt_check_launch(const char* what) {
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    bt_set_error("%s: %s", what, hipGetErrorString(err));
    return BT_HIP_ERROR;
  }
  return BT_OK;
}

BT_EXPORT const char* bt_last_error() { return bt_error_text; }
