// Shared between the translation units of libfrnn_rt.so; not part of the C ABI.
#ifndef FRNN_INTERNAL_H
#define FRNN_INTERNAL_H

#include <stddef.h>

struct frnn_kernel_s {
  void* fn;            // hipFunction_t
  size_t kernarg;      // bytes of the kernel's explicit arguments as its code object declares them (0 = unknown)
};

// records the calling thread's error message (what frnn_last_error() returns) and returns `code`
__attribute__((visibility("hidden"))) int frnn_detail_fail(int code, const char* fmt, ...)
    __attribute__((format(printf, 2, 3)));

#endif
