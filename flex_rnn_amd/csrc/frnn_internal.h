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


// hipModuleLaunchKernel as resolved at run time by frnn_rt.cpp (the HIP runtime the process already holds), or null
// before any HIP call was made there.  frnn_static.hip, which is linked against the HIP runtime, checks that it is
// bound to the same one.
extern "C" __attribute__((visibility("hidden"))) void* frnn_detail_runtime_launch_symbol();

#endif
