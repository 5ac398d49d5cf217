// Host-side helpers shared by the translation units of libhdmoe.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>

#include "../../include/hdmoe.h"

// thread-local message behind hdmoe_last_error()
char* hdmoe_error_buffer();
constexpr int HDMOE_ERRBUF = 512;

static inline int hdmoe_fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(hdmoe_error_buffer(), HDMOE_ERRBUF, fmt, ap);
  va_end(ap);
  return code;
}

// Launch errors are read with hipGetLastError only: it does not synchronise.
static inline int hdmoe_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return hdmoe_fail(HDMOE_E_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return HDMOE_OK;
}

#define HDMOE_REQUIRE_PTR(p)                                                   \
  do {                                                                         \
    if ((p) == nullptr) return hdmoe_fail(HDMOE_E_NULL, "%s: %s is NULL", __func__, #p); \
  } while (0)

static inline size_t hdmoe_align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

constexpr int HDMOE_NUM_CU = 256;   // MI355X
constexpr int HDMOE_NUM_XCD = 8;
